// Attention scores without their round trip through memory.
//
// The reference forms the scaled scores with a batched GEMM, writes them out
// and reads them back in the softmax kernel (pytorch_module/encoder.cu:104-121:
// Einsum -> BETA, then Softmax), and likewise in the backward pass writes
// d(dropped softmax) and reads it back in BackwardSoftmax (encoder.cu:228-247).
// A row of scores is only head_size long in its contraction, so a workgroup can
// form a block of 32 complete rows with MFMA straight from the projections
// (operand fragments are loaded from global memory in MFMA layout, no LDS),
// park it in LDS as fp16 -- the same rounding the stored tensor would get -- and
// run the row operator on it.  Everything the row operator writes is written as
// before; only the score tensor itself (BETA, resp. DATTN_DROP) is not.
//
//   forward : S = alpha * Q.K^T        -> softmax + dropout -> ALPHA, mask, ATTN_DROP
//   backward: G = dO.V^T               -> softmax backward  -> DBETA
#include "sub_ops.hpp"

namespace sub {

namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
constexpr int ROWS = 32;                  // score rows per workgroup (one MFMA tile high)
constexpr float LOG2E = 1.4426950408889634f;

// The key-side MFMA operand of one wave: its quarter of the keys (NT tiles of 32),
// all P features, kept in registers and reused for every block of query rows the
// workgroup goes through (lane = key row, 8 consecutive features per k-step).
template <int P, int NT>
__device__ __forceinline__ void load_keys(const ScoreArgs& a, unsigned h, unsigned b, int wave, int lane,
                                          h8 (&fk)[NT][P / 16]) {
    const int l32 = lane & 31, hi = lane >> 5;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const half_t* krow = a.rows_m + (long)h * a.m_sh + (long)b * a.m_sb +
                             (long)((wave * NT + t) * 32 + l32) * a.m_sr + hi * 8;
#pragma unroll
        for (int ks = 0; ks < P / 16; ++ks) fk[t][ks] = *reinterpret_cast<const h8*>(krow + ks * 16);
    }
}

template <int P>
__device__ __forceinline__ void load_queries(const ScoreArgs& a, unsigned h, unsigned b, unsigned j0, int lane,
                                             h8 (&fq)[P / 16]) {
    const int l32 = lane & 31, hi = lane >> 5;
    const half_t* qrow = a.rows_n + (long)h * a.n_sh + (long)b * a.n_sb + (long)(j0 + l32) * a.n_sr + hi * 8;
#pragma unroll
    for (int ks = 0; ks < P / 16; ++ks) fq[ks] = *reinterpret_cast<const h8*>(qrow + ks * 16);
}

// 32 query rows x R keys of scores into `stage` ([32][R + 8] fp16): each wave
// forms the columns of its quarter of the keys, contraction over the P features.
template <int P, int NT>
__device__ __forceinline__ void score_tile(const h8 (&fk)[NT][P / 16], const h8 (&fq)[P / 16], float alpha,
                                           int wave, int lane, half_t* stage, int pitch) {
    const int l32 = lane & 31, hi = lane >> 5;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        f16v acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < P / 16; ++ks)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk[t][ks], fq[ks], acc, 0, 0, 0);
        // D[key, query]: lane = query row l32, registers = keys q*8 + hi*4 + 0..3 of the tile
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            h4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (half_t)(acc[q * 4 + e] * alpha);
            *reinterpret_cast<h4*>(stage + l32 * pitch + (wave * NT + t) * 32 + q * 8 + hi * 4) = w;
        }
    }
}

// Rows per workgroup: TILES blocks of 32 query rows of one head and sample, gone
// through one after the other with the key fragments held in registers.
constexpr int TILES = 4;

// grid.x = (heads * samples * queries) / (32 * TILES).  Row numbering is the canonical one
// of the [H,B,J,K] tensors (rs = {1, H, B, J} x K, not merged).
// How the rows of a block are gone through by a wave: rows of up to 128 (256)
// elements take a quarter (half) of a wave, so four (two) sit side by side.
template <int R>
struct RowPlan {
    static constexpr int GRP = R >= 512 ? WAVE : R / 8;        // lanes per row
    static constexpr int SPW = WAVE / GRP;                     // rows side by side
    static constexpr int VPL = R > 512 ? R / 512 : 1;          // 8-packs per lane
    static constexpr int RP = SPW == 1 ? 4 : (SPW == 2 ? 4 : 2);   // rows per lane group and pass
    static constexpr int PER_PASS = RP * SPW;
};

// NW waves per workgroup, each forming NT tiles of 32 keys: R = 32 * NT * NW.
template <int P, int NT, int NW>
__global__ __launch_bounds__(NW * WAVE) void k_scores_softmax(RowSpace rs, ScoreArgs a, View alpha, View mask,
                                                              View drop, PhiloxKey key_) {
    constexpr int R = 32 * NT * NW;
    using RPn = RowPlan<R>;
    constexpr int GRP = RPn::GRP, SPW = RPn::SPW, VPL = RPn::VPL, RP = RPn::RP;
    constexpr int PITCH = R + 8;
    constexpr int RPW = ROWS / NW;           // rows per wave
    static_assert(RPW % RPn::PER_PASS == 0, "rows per wave must be whole passes");
    __shared__ __attribute__((aligned(16))) half_t stage[ROWS * PITCH];
    const PhiloxKey key = resolved(key_);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int gl = lane % GRP, sub = lane / GRP;
    const RowIdx ixb = row_index(rs, blockIdx.x * (ROWS * TILES));
    h8 fk[NT][P / 16], fq[P / 16];
    load_keys<P, NT>(a, ixb.i1, ixb.i2, wave, lane, fk);
    load_queries<P>(a, ixb.i1, ixb.i2, ixb.i3, lane, fq);
    for (int tile = 0; tile < TILES; ++tile) {
        const unsigned row_base = (blockIdx.x * TILES + tile) * ROWS;
        if (tile) __syncthreads();                 // the previous tile's rows have been read
        score_tile<P, NT>(fk, fq, a.alpha, wave, lane, stage, PITCH);
        if (tile + 1 < TILES) load_queries<P>(a, ixb.i1, ixb.i2, ixb.i3 + (tile + 1) * ROWS, lane, fq);
        __syncthreads();
#pragma unroll
        for (int pass = 0; pass < RPW / RPn::PER_PASS; ++pass) {
            float x[RP][VPL][8];
            float m[RP], s[RP];
            RowIdx ix[RP];
#pragma unroll
            for (int r = 0; r < RP; ++r) {
                const int rl = wave * RPW + pass * RPn::PER_PASS + r * SPW + sub;
                ix[r] = row_index(rs, row_base + rl);
                m[r] = -INFINITY;
#pragma unroll
                for (int c = 0; c < VPL; ++c) {
                    const int e0 = (c * GRP + gl) * 8;
                    h8 v = *reinterpret_cast<const h8*>(stage + rl * PITCH + e0);
#pragma unroll
                    for (int i = 0; i < 8; ++i) { x[r][c][i] = (float)v[i]; m[r] = fmaxf(m[r], x[r][c][i]); }
                }
            }
#pragma unroll
            for (int r = 0; r < RP; ++r) m[r] = group_max<GRP>(m[r]);
#pragma unroll
            for (int r = 0; r < RP; ++r) {
                s[r] = 0.f;
#pragma unroll
                for (int c = 0; c < VPL; ++c)
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        x[r][c][i] = __builtin_amdgcn_exp2f((x[r][c][i] - m[r]) * LOG2E);
                        s[r] += x[r][c][i];
                    }
            }
#pragma unroll
            for (int r = 0; r < RP; ++r) s[r] = group_sum<GRP>(s[r]);
#pragma unroll
            for (int r = 0; r < RP; ++r) {
                const unsigned row = row_base + wave * RPW + pass * RPn::PER_PASS + r * SPW + sub;
                const float inv = 1.0f / s[r];
                const long oa = view_offset(alpha, ix[r]), om = view_offset(mask, ix[r]), od = view_offset(drop, ix[r]);
#pragma unroll
                for (int c = 0; c < VPL; ++c) {
                    const int e0 = (c * GRP + gl) * 8;
                    h8 al, d;
                    const uint32_t bits = keep_bits8(key, (uint64_t)row * (uint64_t)R + (uint64_t)e0);
#pragma unroll
                    for (int i = 0; i < 8; ++i) al[i] = (half_t)(x[r][c][i] * inv);
                    al = pin(al);
#pragma unroll
                    for (int i = 0; i < 8; ++i) d[i] = ((bits >> i) & 1u) ? al[i] : (half_t)0.0f;
                    stg8<true>(alpha.p + oa + e0, al);
                    stg8<true>(mask.p + om + e0, mask_h8(bits));
                    stg8<false>(drop.p + od + e0, d);
                }
            }
        }
    }
}

template <int P, int NT, int NW>
__global__ __launch_bounds__(NW * WAVE) void k_dscores_bs(RowSpace rs, ScoreArgs a, View alpha, View mask, View dbeta) {
    constexpr int R = 32 * NT * NW;
    using RPn = RowPlan<R>;
    constexpr int GRP = RPn::GRP, SPW = RPn::SPW, VPL = RPn::VPL, RP = RPn::RP;
    constexpr int PITCH = R + 8;
    constexpr int RPW = ROWS / NW;
    static_assert(RPW % RPn::PER_PASS == 0, "rows per wave must be whole passes");
    __shared__ __attribute__((aligned(16))) half_t stage[ROWS * PITCH];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int gl = lane % GRP, sub = lane / GRP;
    const RowIdx ixb = row_index(rs, blockIdx.x * (ROWS * TILES));
    h8 fk[NT][P / 16], fq[P / 16];
    load_keys<P, NT>(a, ixb.i1, ixb.i2, wave, lane, fk);
    load_queries<P>(a, ixb.i1, ixb.i2, ixb.i3, lane, fq);
    for (int tile = 0; tile < TILES; ++tile) {
        const unsigned row_base = (blockIdx.x * TILES + tile) * ROWS;
        if (tile) __syncthreads();
        score_tile<P, NT>(fk, fq, a.alpha, wave, lane, stage, PITCH);
        if (tile + 1 < TILES) load_queries<P>(a, ixb.i1, ixb.i2, ixb.i3 + (tile + 1) * ROWS, lane, fq);
        __syncthreads();
#pragma unroll
        for (int pass = 0; pass < RPW / RPn::PER_PASS; ++pass) {
            float al[RP][VPL][8], g[RP][VPL][8];
            float s[RP];
            RowIdx ix[RP];
#pragma unroll
            for (int r = 0; r < RP; ++r) {
                const int rl = wave * RPW + pass * RPn::PER_PASS + r * SPW + sub;
                ix[r] = row_index(rs, row_base + rl);
                const long oa = view_offset(alpha, ix[r]), om = view_offset(mask, ix[r]);
                s[r] = 0.f;
#pragma unroll
                for (int c = 0; c < VPL; ++c) {
                    const int e0 = (c * GRP + gl) * 8;
                    const h8 va = ldg8<true>(alpha.p + oa + e0);
                    const h8 vm = ldg8<true>(mask.p + om + e0);
                    const h8 vd = *reinterpret_cast<const h8*>(stage + rl * PITCH + e0);
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        al[r][c][i] = (float)va[i];
                        g[r][c][i] = (float)vm[i] * (float)vd[i];
                        s[r] += al[r][c][i] * g[r][c][i];
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < RP; ++r) s[r] = group_sum<GRP>(s[r]);
#pragma unroll
            for (int r = 0; r < RP; ++r) {
                const long oo = view_offset(dbeta, ix[r]);
#pragma unroll
                for (int c = 0; c < VPL; ++c) {
                    const int e0 = (c * GRP + gl) * 8;
                    h8 o;
#pragma unroll
                    for (int i = 0; i < 8; ++i) o[i] = (half_t)(1.0f * al[r][c][i] * (g[r][c][i] - s[r]));
                    stg8<false>(dbeta.p + oo + e0, o);
                }
            }
        }
    }
}

template <int P>
bool dispatch_fwd(int R, dim3 grid, hipStream_t st, const RowSpace& rs, const ScoreArgs& a, View alpha, View mask,
                  View drop, PhiloxKey key) {
    switch (R) {
        case 128: hipLaunchKernelGGL((k_scores_softmax<P, 1, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, drop, key); return true;
        case 256: hipLaunchKernelGGL((k_scores_softmax<P, 2, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, drop, key); return true;
        case 512: hipLaunchKernelGGL((k_scores_softmax<P, 4, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, drop, key); return true;
        case 1024: hipLaunchKernelGGL((k_scores_softmax<P, 8, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, drop, key); return true;
        default: return false;
    }
}
template <int P>
bool dispatch_bwd(int R, dim3 grid, hipStream_t st, const RowSpace& rs, const ScoreArgs& a, View alpha, View mask,
                  View dbeta) {
    switch (R) {
        case 128: hipLaunchKernelGGL((k_dscores_bs<P, 1, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, dbeta); return true;
        case 256: hipLaunchKernelGGL((k_dscores_bs<P, 2, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, dbeta); return true;
        case 512: hipLaunchKernelGGL((k_dscores_bs<P, 4, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, dbeta); return true;
        case 1024: hipLaunchKernelGGL((k_dscores_bs<P, 8, 4>), grid, dim3(256), 0, st, rs, a, alpha, mask, dbeta); return true;
        default: return false;
    }
}

}  // namespace

bool scores_fusable(const RowSpace& rs, const ScoreArgs& a, int P, std::initializer_list<const View*> views) {
    if (rs.n0 != 1 || rs.flat) return false;                       // rows numbered over (H, B, J)
    if (rs.R != 128 && rs.R != 256 && rs.R != 512 && rs.R != 1024) return false;
    if (P != 64 && P != 128) return false;
    if (rs.n3 % (ROWS * TILES) != 0) return false;                 // a workgroup's rows share head and sample
    if (rs.rows() <= 0 || rs.rows() / (ROWS * TILES) > 0x7fffffffL) return false;
    for (const View* v : views) if (!v->vec) return false;
    auto al = [](const void* p, long s1, long s2, long s3) {
        return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && s1 % 8 == 0 && s2 % 8 == 0 && s3 % 8 == 0;
    };
    return al(a.rows_n, a.n_sh, a.n_sb, a.n_sr) && al(a.rows_m, a.m_sh, a.m_sb, a.m_sr);
}

bool launch_scores_softmax(const RowSpace& rs, const ScoreArgs& a, int P, View alpha, View mask, View drop,
                           PhiloxKey key, hipStream_t st) {
    if (!scores_fusable(rs, a, P, {&alpha, &mask, &drop})) return false;
    dim3 grid((unsigned)(rs.rows() / (ROWS * TILES)));
    bool ok = P == 64 ? dispatch_fwd<64>(rs.R, grid, st, rs, a, alpha, mask, drop, key)
                      : dispatch_fwd<128>(rs.R, grid, st, rs, a, alpha, mask, drop, key);
    if (ok) check_launch("scores + softmax");
    return ok;
}

bool launch_dscores_bs(const RowSpace& rs, const ScoreArgs& a, int P, View alpha, View mask, View dbeta,
                       hipStream_t st) {
    if (!scores_fusable(rs, a, P, {&alpha, &mask, &dbeta})) return false;
    dim3 grid((unsigned)(rs.rows() / (ROWS * TILES)));
    bool ok = P == 64 ? dispatch_bwd<64>(rs.R, grid, st, rs, a, alpha, mask, dbeta)
                      : dispatch_bwd<128>(rs.R, grid, st, rs, a, alpha, mask, dbeta);
    if (ok) check_launch("d(scores) + softmax backward");
    return ok;
}

}  // namespace sub
