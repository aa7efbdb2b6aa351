// The backward pass around one LayerNorm in a single launch.
//
// The reference runs it as two or three kernels that hand a [B,J,I] tensor to
// each other through memory (pytorch_module/encoder.cu:160-166 and 196-212):
//   BackwardScaleBias            (block_bsb_ebsb.cuh:178-216)   G = DOUT * gamma, d gamma, d beta
//     or ExtendedBackwardScaleBias (block_bsb_ebsb.cuh:376-420) G = (D1 + D2) * gamma, ..., d linear-bias
//   BackwardLayerNormResidualDropout (block_blnrd.cuh:203-259)  from G: d(LN input), d(dropout input)
//   BackwardAttnOutBias          (block_baob.cuh:79-97)         column sum of d(dropout input)
// Every one of them works on whole rows of I features, so one wave can take a
// row through all the steps while it is in registers: G is rounded to fp16 and
// stored exactly as the separate kernels would, the later steps start from the
// rounded value as they do there, and the column sums accumulate per lane over
// the rows the wave visits.  Waves of a block combine their sums
// through LDS into one fp32 partial row per block; the shared finishing launch
// adds the partial rows.
#include "sub_ops.hpp"

namespace sub {

namespace {

constexpr int LN_BLOCK = 512;
constexpr int LN_WPB = LN_BLOCK / WAVE;

// The inputs of one row, as loaded (one 128-bit pack per lane and chunk).
template <int VPL>
struct LnRow {
    h8 in[VPL], d1[VPL], d2[VPL], dl[VPL], df[VPL], mk[VPL];
    uint32_t mkb[VPL];          // PACKED: the mask of the pack as 8 bits, in place of mk
    float is;
    RowIdx ix;
};

template <int VPL, bool EXT, bool PACKED, bool MOVE>
__device__ __forceinline__ void ln_load_row(const RowSpace& rs, const LnBwdArgs& a, unsigned row, int lane,
                                            const int (&nv)[VPL], LnRow<VPL>& r) {
    r.ix = row_index(rs, row);
    const long oin = view_offset(a.in, r.ix), o1 = view_offset(a.d1, r.ix), odf = view_offset(a.diff, r.ix),
               omk = view_offset(a.mask, r.ix);
    const long o2 = EXT ? view_offset(a.d2, r.ix) : 0, odl = EXT ? view_offset(a.dlinear, r.ix) : 0;
    r.is = (float)a.istd.p[view_offset(a.istd, r.ix)];
#pragma unroll
    for (int c = 0; c < VPL; ++c) {
        const int e0 = (c * WAVE + lane) * 8;
        r.in[c] = r.d1[c] = r.d2[c] = r.dl[c] = r.df[c] = r.mk[c] = (h8)(half_t)0.0f;
        r.mkb[c] = 0;
        if (nv[c]) {
            r.in[c] = ldg8<true>(a.in.p + oin + e0);          // saved by the forward pass
            // the incoming gradient of the plain form is the caller's tensor;
            // those of the extended form are intermediates on their last use
            r.d1[c] = ldg8<EXT>(a.d1.p + o1 + e0);
            if (EXT) {
                r.d2[c] = ldg8<true>(a.d2.p + o2 + e0);
                if (!MOVE) r.dl[c] = ldg8<true>(a.dlinear.p + odl + e0);
            }
            r.df[c] = ldg8<true>(a.diff.p + odf + e0);
            if (PACKED) r.mkb[c] = a.mask_bits[(size_t)row * (rs.R >> 3) + (c * WAVE + lane)];
            else r.mk[c] = ldg8<true>(a.mask.p + omk + e0);
        }
    }
}

// VPL: 128-bit packs per lane and row (row length <= VPL * 512).  EXT: the
// extended form (two incoming gradients, linear-bias and output-bias sums).
// MOVE: see LnBwdArgs::move_sum (sums of the plain form: d scale, d bias, column sum of d_drop_in; of
// the extended form: d scale, d bias, column sum of d_drop_in = d output-bias).
template <int VPL, bool EXT, bool PACKED, bool MOVE>
__global__ __launch_bounds__(LN_BLOCK) void k_lnbwd(RowSpace rs, LnBwdArgs a, float* ws, unsigned nrows) {
    constexpr int NS = MOVE ? 3 : (EXT ? 4 : 2);
    constexpr int S_DROP = MOVE ? 2 : 3;          // which sum takes d_drop_in
    __shared__ float red[LN_WPB][VPL * WAVE * 8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float invn = 1.0f / (float)rs.R;
    float acc[NS][VPL][8];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int c = 0; c < VPL; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[s][c][i] = 0.f;
    int nv[VPL];
    F8 fsc[VPL];
#pragma unroll
    for (int c = 0; c < VPL; ++c) {
        const int e0 = (c * WAVE + lane) * 8;
        nv[c] = e0 < rs.R ? 8 : 0;                 // rows are whole 8-packs here
        fsc[c] = ld8<true>(a.scale, 0, e0, nv[c]);
    }
    const unsigned stride = gridDim.x * LN_WPB;
    unsigned row = blockIdx.x * LN_WPB + wave;
    LnRow<VPL> cur, nxt;
    if (row < nrows) ln_load_row<VPL, EXT, PACKED, MOVE>(rs, a, row, lane, nv, cur);
    for (; row < nrows; row += stride) {
        // the next row's loads are in flight while this one is worked on
        const bool more = row + stride < nrows;
        if (more) ln_load_row<VPL, EXT, PACKED, MOVE>(rs, a, row + stride, lane, nv, nxt);
        float g[VPL][8], df[VPL][8];
        float s1 = 0.f, s2 = 0.f;
        const long og = view_offset(a.g, cur.ix);
        const float is = cur.is;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            const int e0 = (c * WAVE + lane) * 8;
            h8 o;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float d = EXT ? (float)cur.d1[c][i] + (float)cur.d2[c][i] : (float)cur.d1[c][i];
                o[i] = (half_t)(d * fsc[c].v[i]);
                acc[0][c][i] += d * (float)cur.in[c][i];
                acc[1][c][i] += d;
                if (EXT && !MOVE) acc[2][c][i] += (float)cur.dl[c][i];
            }
            o = pin(o);
            if (nv[c] && a.write_g) stg8<true>(a.g.p + og + e0, o);     // nothing reads G again
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                g[c][i] = (float)o[i];
                df[c][i] = (float)cur.df[c][i];
                s1 += g[c][i];
                s2 = __fmaf_rn(g[c][i], df[c][i], s2);
            }
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        const float c1 = s1 * is * invn;
        const float c2 = s2 * is * is * is * invn;
        const long oa = view_offset(a.d_ln_in, cur.ix), ob = view_offset(a.d_drop_in, cur.ix);
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            const int e0 = (c * WAVE + lane) * 8;
            if (!nv[c]) continue;
            h8 x, y;
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (half_t)ln_bwd_value(g[c][i], df[c][i], is, c1, c2);
            x = pin(x);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool kept = PACKED ? ((cur.mkb[c] >> i) & 1u) != 0 : cur.mk[c][i] != (half_t)0.0f;
                y[i] = kept ? x[i] : (half_t)0.0f;
                if (EXT || MOVE) acc[S_DROP][c][i] += (float)y[i];
            }
            stg8<false>(a.d_ln_in.p + oa + e0, x);
            stg8<false>(a.d_drop_in.p + ob + e0, y);
        }
        if (more) cur = nxt;
    }
    // One partial row per block and sum: ws[(s * gridDim.x + block) * R + feature].
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        __syncthreads();
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            float* dst = &red[wave][(c * WAVE + lane) * 8];
            *reinterpret_cast<float4*>(dst) = make_float4(acc[s][c][0], acc[s][c][1], acc[s][c][2], acc[s][c][3]);
            *reinterpret_cast<float4*>(dst + 4) = make_float4(acc[s][c][4], acc[s][c][5], acc[s][c][6], acc[s][c][7]);
        }
        __syncthreads();
        for (int f = threadIdx.x; f < rs.R; f += LN_BLOCK) {
            float t = 0.f;
#pragma unroll
            for (int w = 0; w < LN_WPB; ++w) t += red[w][f];
            ws[((long)s * gridDim.x + blockIdx.x) * rs.R + f] = t;
        }
    }
}

// The same launch for a flat row space with sixteen waves per workgroup and one row per wave and pass:
// four waves per SIMD take turns on the 500 vector instructions a row needs, where the kernel above
// has two (its registers: this row, the next row's loads, 48 column-sum accumulators).  To fit the 128
// registers that leaves a lane, the row's loads are not held beyond their use, the LayerNorm scale is
// fetched with the row, and the column sum of d_drop_in does not live in registers: a wave adds its
// rows' values into its own slab of LDS, which the reduction of the other sums reuses afterwards.
// Same arithmetic per row; a column sum adds a lane's rows in order, then the waves in order.
// SEG > 1: rows of up to SEG * 1024 features, a row shared by SEG waves that take 1024 features each
// (a lane still owns 16 columns, so the column sums stay in registers); the two sums over the row that
// the LayerNorm backward needs meet in LDS, in wave order, behind one barrier per pass -- which is why
// every wave then makes the same number of passes, a wave without a row walking row 0 and keeping nothing.
constexpr int LNF_BLOCK = 1024;
constexpr int LNF_WPB = LNF_BLOCK / WAVE;

template <int VPL, bool EXT, bool PACKED, bool MOVE, int SEG = 1>
__global__ __launch_bounds__(LNF_BLOCK) void k_lnbwd_flat(int R, LnBwdArgs a, float* ws, unsigned nrows) {
    static_assert(SEG == 1 || VPL == 2, "a segment is 1024 features: two packs per lane");
    constexpr int ROWS = LNF_WPB / SEG;           // rows per workgroup and pass
    __shared__ float stat[2][LNF_WPB][2];         // SEG > 1: the waves' shares of the two row sums, by pass parity
    constexpr int NS = MOVE ? 3 : (EXT ? 4 : 2);
    constexpr int S_DROP = MOVE ? 2 : 3;          // which sum takes d_drop_in
    constexpr bool DROP_SUM = EXT || MOVE;
    constexpr int NR = DROP_SUM ? NS - 1 : NS;    // sums kept in registers
    __shared__ float red[LNF_WPB][VPL * WAVE * 8];
    __shared__ float red2[LNF_WPB][VPL * WAVE * 8];     // a second set of slabs: two sums per reduction pass
    typedef int i4v __attribute__((ext_vector_type(4)));
    fetch_args_now(R, nrows, a.in.p, a.in.s3, a.d1.p, a.d1.s3, a.diff.p, a.diff.s3, a.istd.p, a.istd.s3, a.scale.p, a.g.p,
                   a.g.s3, a.d_ln_in.p, a.d_ln_in.s3, a.d_drop_in.p, a.d_drop_in.s3, a.write_g, ws);
    if (EXT) fetch_args_now(a.d2.p, a.d2.s3);
    if (EXT && !MOVE) fetch_args_now(a.dlinear.p, a.dlinear.s3);
    if (PACKED) fetch_args_now(a.mask_bits);
    else fetch_args_now(a.mask.p, a.mask.s3);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rslot = SEG > 1 ? wave / SEG : wave, seg = SEG > 1 ? wave % SEG : 0;
    const float invn = 1.0f / (float)R;
    float acc[NR][VPL][8];
#pragma unroll
    for (int s = 0; s < NR; ++s)
#pragma unroll
        for (int c = 0; c < VPL; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[s][c][i] = 0.f;
    // A chunk outside the row reads the row's first pack and has it and-ed away: no branch around a load.
    bool inside[VPL];
    int e0[VPL], keep_all[VPL];
#pragma unroll
    for (int c = 0; c < VPL; ++c) {
        e0[c] = seg * (VPL * WAVE * 8) + (c * WAVE + lane) * 8;
        inside[c] = e0[c] < R;
        keep_all[c] = inside[c] ? -1 : 0;
        if (!inside[c]) e0[c] = 0;
    }
    auto masked = [&](h8 v, int c) { return __builtin_bit_cast(h8, __builtin_bit_cast(i4v, v) & keep_all[c]); };
    float* const slab = &red[wave][lane * 8];     // + c * 512: this lane's 8 columns of pack c
    bool first_row = true;
    const unsigned row_stride = gridDim.x * ROWS;
    const unsigned npass = SEG > 1 ? (nrows + row_stride - 1) / row_stride : 0;
    unsigned row_at = blockIdx.x * ROWS + rslot;
    for (unsigned pass = 0; SEG > 1 ? pass < npass : row_at < nrows; ++pass, row_at += row_stride) {
        const bool active = SEG == 1 || row_at < nrows;
        const unsigned row = active ? row_at : 0;
        h8 in[VPL], d1[VPL], d2[VPL], dl[VPL], df[VPL], mk[VPL], sc[VPL];
        uint32_t mkb[VPL];
        const half_t isth = a.istd.p[(long)row * a.istd.s3];
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            in[c] = ldg8<true>(a.in.p + (long)row * a.in.s3 + e0[c]);          // saved by the forward pass
            // the incoming gradient of the plain form is the caller's tensor;
            // those of the extended form are intermediates on their last use
            d1[c] = ldg8<EXT>(a.d1.p + (long)row * a.d1.s3 + e0[c]);
            if (EXT) {
                d2[c] = ldg8<true>(a.d2.p + (long)row * a.d2.s3 + e0[c]);
                if (!MOVE) dl[c] = ldg8<true>(a.dlinear.p + (long)row * a.dlinear.s3 + e0[c]);
            }
            sc[c] = ldg8<false>(a.scale.p + e0[c]);
            df[c] = ldg8<true>(a.diff.p + (long)row * a.diff.s3 + e0[c]);
            if (PACKED) mkb[c] = a.mask_bits[(size_t)row * (R >> 3) + (e0[c] >> 3)];
            else mk[c] = ldg8<true>(a.mask.p + (long)row * a.mask.s3 + e0[c]);
        }
        const float is = (float)isth;
        float s1 = 0.f, s2 = 0.f;
        h8 gh[VPL];
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            const h8 in8 = masked(in[c], c), d18 = masked(d1[c], c), sc8 = masked(sc[c], c);
            h8 d28, dl8;
            if (EXT) d28 = masked(d2[c], c);
            if (EXT && !MOVE) dl8 = masked(dl[c], c);
            df[c] = masked(df[c], c);
            h8 o;
            if (active) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float d = EXT ? (float)d18[i] + (float)d28[i] : (float)d18[i];
                    o[i] = (half_t)(d * (float)sc8[i]);
                    acc[0][c][i] += d * (float)in8[i];
                    acc[1][c][i] += d;
                    if (EXT && !MOVE) acc[2][c][i] += (float)dl8[i];
                }
            } else {
                o = (h8)(half_t)0.0f;
            }
            o = pin(o);
            if (active && inside[c] && a.write_g) stg8<true>(a.g.p + (long)row * a.g.s3 + e0[c], o);     // nothing reads G again
            gh[c] = o;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                s1 += (float)o[i];
                s2 = __fmaf_rn((float)o[i], (float)df[c][i], s2);
            }
            // one pack after the other: interleaved, their converted values do not fit the registers
            __builtin_amdgcn_sched_barrier(0);
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        if constexpr (SEG > 1) {
            float (*st)[2] = stat[pass & 1];
            if (lane == 0) { st[wave][0] = s1; st[wave][1] = s2; }
            __syncthreads();          // every wave, every pass (a wave two passes on writes the other half of `stat`)
            s1 = 0.f; s2 = 0.f;
#pragma unroll
            for (int k = 0; k < SEG; ++k) { s1 += st[rslot * SEG + k][0]; s2 += st[rslot * SEG + k][1]; }
        }
        const float c1 = s1 * is * invn;
        const float c2 = s2 * is * is * is * invn;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            h8 x, y;
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = (half_t)ln_bwd_value((float)gh[c][i], (float)df[c][i], is, c1, c2);
            x = pin(x);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool kept = PACKED ? ((mkb[c] >> i) & 1u) != 0 : mk[c][i] != (half_t)0.0f;
                y[i] = kept ? x[i] : (half_t)0.0f;
            }
            if (DROP_SUM && active) {
                // (a chunk outside the row: x comes out as -c1, which must not be summed)
                const h8 ys = masked(y, c);
                float4 lo = make_float4((float)ys[0], (float)ys[1], (float)ys[2], (float)ys[3]);
                float4 hi = make_float4((float)ys[4], (float)ys[5], (float)ys[6], (float)ys[7]);
                if (!first_row) {
                    const float4 plo = *reinterpret_cast<const float4*>(slab + c * 512);
                    const float4 phi = *reinterpret_cast<const float4*>(slab + c * 512 + 4);
                    lo.x += plo.x; lo.y += plo.y; lo.z += plo.z; lo.w += plo.w;
                    hi.x += phi.x; hi.y += phi.y; hi.z += phi.z; hi.w += phi.w;
                }
                *reinterpret_cast<float4*>(slab + c * 512) = lo;
                *reinterpret_cast<float4*>(slab + c * 512 + 4) = hi;
            }
            if (active && inside[c]) {
                stg8<false>(a.d_ln_in.p + (long)row * a.d_ln_in.s3 + e0[c], x);
                stg8<false>(a.d_drop_in.p + (long)row * a.d_drop_in.s3 + e0[c], y);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (active) first_row = false;
    }
    if (DROP_SUM && first_row) {                   // a wave without a row
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            *reinterpret_cast<float4*>(slab + c * 512) = make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4*>(slab + c * 512 + 4) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    // One partial row per block and sum: ws[(s * gridDim.x + block) * R + feature].  The sum of
    // d_drop_in lies in the slabs already; the others follow from the registers, through the second
    // set of slabs and then the first again, two sums per pass.
    float* const slab2 = &red2[wave][lane * 8];
    auto put = [&](float* dst, int s) {
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            *reinterpret_cast<float4*>(dst + c * 512) = make_float4(acc[s][c][0], acc[s][c][1], acc[s][c][2], acc[s][c][3]);
            *reinterpret_cast<float4*>(dst + c * 512 + 4) = make_float4(acc[s][c][4], acc[s][c][5], acc[s][c][6], acc[s][c][7]);
        }
    };
    // (feature f lies in the slabs of the waves of its segment)
    auto reduce = [&](const float (*from)[VPL * WAVE * 8], int s) {
        for (int f = threadIdx.x; f < R; f += LNF_BLOCK) {
            const int sg = SEG > 1 ? f / (VPL * WAVE * 8) : 0, fl = SEG > 1 ? f % (VPL * WAVE * 8) : f;
            float t = 0.f;
#pragma unroll
            for (int w = 0; w < ROWS; ++w) t += from[w * SEG + sg][fl];
            ws[((long)s * gridDim.x + blockIdx.x) * R + f] = t;
        }
    };
    constexpr int START = DROP_SUM ? 1 : 0;        // register sums that the first pass leaves
    static_assert(START + 2 >= NR, "one more pass takes the rest");
    if (DROP_SUM) {
        put(slab2, 0);
        __syncthreads();
        reduce(red, S_DROP);
        reduce(red2, 0);
    }
    // (with MOVE the register sums are 0, 1; without it 0, 1 and for the extended form 2)
    if constexpr (START < NR) {
        __syncthreads();                           // every wave is done reading both sets
        put(slab, START);
        if constexpr (START + 1 < NR) put(slab2, START + 1);
        __syncthreads();
        reduce(red, START);
        if constexpr (START + 1 < NR) reduce(red2, START + 1);
    }
}

inline int lnbwd_blocks(long nrows) {
    // two rows per wave where there are enough rows; at most 2048 waves
    long blocks = (nrows + 2L * LN_WPB - 1) / (2L * LN_WPB);
    if (blocks < 1) blocks = 1;
    if (blocks > 256) blocks = 256;
    return (int)blocks;
}

}  // namespace

bool lnbwd_supported(const RowSpace& rs, const LnBwdArgs& a, bool ext) {
    if (rs.R <= 0 || rs.R > 4096 || rs.R % 8 != 0) return false;
    // rows beyond 1024 features: only the sixteen-wave kernel, whose waves share a row
    if (rs.R > 1024 && !(rs.flat && !(ext && !a.move_sum))) return false;
    if (rs.rows() <= 0 || rs.rows() >= (1L << 31)) return false;
    bool ok = a.in.vec && a.d1.vec && a.diff.vec && (a.mask.vec || a.mask_bits) && a.g.vec && a.d_ln_in.vec && a.d_drop_in.vec &&
              a.scale.vec;
    if (ext) ok = ok && a.d2.vec && a.dlinear.vec;
    return ok;
}

size_t lnbwd_ws_floats(const RowSpace& rs, bool ext) {
    return (size_t)(ext ? 4 : 3) * lnbwd_blocks(rs.rows()) * rs.R;      // (3: the plain form with move_sum)
}

void launch_lnbwd(const RowSpace& rs, const LnBwdArgs& a, bool ext, half_t* const sums[4], float* ws,
                  hipStream_t st, FinishJobs* defer) {
    if (!lnbwd_supported(rs, a, ext)) fail("fused LayerNorm backward: unsupported shape or layout");
    if (!ws) fail("fused LayerNorm backward: no reduction workspace");
    const unsigned nrows = (unsigned)rs.rows();
    const int blocks = lnbwd_blocks(nrows);
    const int vpl = rs.R <= 512 ? 1 : 2;
    if (rs.R > 1024) {
        // (lnbwd_supported has ruled out the extended form without move_sum: MOVE_ is EXT_ || move_sum)
#define SUB_LNBWD_WIDE(EXT_, MOVE_, SEG_)                                                                         \
    do {                                                                                                          \
        if (a.mask_bits)                                                                                          \
            hipLaunchKernelGGL((k_lnbwd_flat<2, EXT_, true, MOVE_, SEG_>), dim3(blocks), dim3(LNF_BLOCK), 0, st, rs.R, a, ws, nrows); \
        else                                                                                                      \
            hipLaunchKernelGGL((k_lnbwd_flat<2, EXT_, false, MOVE_, SEG_>), dim3(blocks), dim3(LNF_BLOCK), 0, st, rs.R, a, ws, nrows); \
    } while (0)
#define SUB_LNBWD_WIDE_SEG(SEG_)                                                                                  \
    do {                                                                                                          \
        if (ext) SUB_LNBWD_WIDE(true, true, SEG_);                                                                \
        else if (a.move_sum) SUB_LNBWD_WIDE(false, true, SEG_);                                                   \
        else SUB_LNBWD_WIDE(false, false, SEG_);                                                                  \
    } while (0)
        if (rs.R <= 2048) SUB_LNBWD_WIDE_SEG(2);
        else SUB_LNBWD_WIDE_SEG(4);
#undef SUB_LNBWD_WIDE_SEG
#undef SUB_LNBWD_WIDE
    } else {
#define SUB_LNBWD_K(KERNEL_, BLOCK_, FIRST_, VPL_, EXT_)                                                          \
    do {                                                                                                          \
        if (a.mask_bits && a.move_sum)                                                                            \
            hipLaunchKernelGGL((KERNEL_<VPL_, EXT_, true, true>), dim3(blocks), dim3(BLOCK_), 0, st, FIRST_, a, ws, nrows);  \
        else if (a.mask_bits)                                                                                     \
            hipLaunchKernelGGL((KERNEL_<VPL_, EXT_, true, false>), dim3(blocks), dim3(BLOCK_), 0, st, FIRST_, a, ws, nrows); \
        else if (a.move_sum)                                                                                      \
            hipLaunchKernelGGL((KERNEL_<VPL_, EXT_, false, true>), dim3(blocks), dim3(BLOCK_), 0, st, FIRST_, a, ws, nrows); \
        else                                                                                                      \
            hipLaunchKernelGGL((KERNEL_<VPL_, EXT_, false, false>), dim3(blocks), dim3(BLOCK_), 0, st, FIRST_, a, ws, nrows); \
    } while (0)
    // (the extended form with its four sums does not fit the sixteen-wave kernel's registers)
#define SUB_LNBWD(VPL_, EXT_)                                                                                     \
    do {                                                                                                          \
        if (rs.flat && !(EXT_ && !a.move_sum)) SUB_LNBWD_K(k_lnbwd_flat, LNF_BLOCK, rs.R, VPL_, EXT_);            \
        else SUB_LNBWD_K(k_lnbwd, LN_BLOCK, rs, VPL_, EXT_);                                                      \
    } while (0)
    if (ext) {
        if (vpl == 1) SUB_LNBWD(1, true);
        else SUB_LNBWD(2, true);
    } else {
        if (vpl == 1) SUB_LNBWD(1, false);
        else SUB_LNBWD(2, false);
    }
#undef SUB_LNBWD_K
#undef SUB_LNBWD
    }
    check_launch("fused LayerNorm backward");
    // with move_sum both forms have three sums; the extended form's third is the output-bias gradient
    FinishArgs fo{{sums[0], sums[1], a.move_sum && ext ? sums[3] : sums[2], sums[3]}, 0, 0, 1, 1};
    FinishJob job{ws, fo, a.move_sum ? 3 : (ext ? 4 : 2), 1, blocks, rs.R};
    finish_or_defer(defer, job, st);
}

}  // namespace sub
