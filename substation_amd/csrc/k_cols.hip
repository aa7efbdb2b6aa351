// Column reductions: gradients of per-feature vectors (LayerNorm scale/bias,
// linear biases) fused with the elementwise work that shares their inputs.
// Counterparts: pytorch_module/block_bsb_ebsb.cuh:12-420, block_bdrlb.cuh:13-146,
// block_baob.cuh:10-97, block_baib.cuh:15-211.
//
// The reference gives each feature one 32-thread warp that walks every token.
// Here tokens are split into chunks so that the grid fills 256 CUs: each block
// reduces its token chunk for a strip of features into fp32 partials
// (deterministically, no atomics), and a small second kernel adds the partials.
#include "sub_ops.hpp"
#include "sub_finish.hpp"

namespace sub {

namespace {

constexpr int BLOCK = 256;
constexpr int WPB = BLOCK / WAVE;

enum ColKind { COL_BSB, COL_EBSB, COL_BDRLB, COL_BAOB, COL_BDRLB_OUT };

struct ColArgs {
    View v[7];
    int act;
};

template <int KIND> struct ColTraits;
template <> struct ColTraits<COL_BSB> { static constexpr int NS = 2; };
template <> struct ColTraits<COL_EBSB> { static constexpr int NS = 3; };
template <> struct ColTraits<COL_BDRLB> { static constexpr int NS = 1; };
template <> struct ColTraits<COL_BAOB> { static constexpr int NS = 1; };
template <> struct ColTraits<COL_BDRLB_OUT> { static constexpr int NS = 1; };

template <int KIND> struct ColIn;      // which views are read: count and indices into ColArgs::v
// `nt`: inputs read here for the last time (saved by the forward pass, or the
// previous launch's output that nothing else consumes): streamed
template <> struct ColIn<COL_BSB> { static constexpr int N = 2; static constexpr int idx[4] = {0, 1, 0, 0}; static constexpr bool nt[4] = {true, false, false, false}; };
template <> struct ColIn<COL_EBSB> { static constexpr int N = 4; static constexpr int idx[4] = {0, 1, 2, 4}; static constexpr bool nt[4] = {true, true, false, true}; };
template <> struct ColIn<COL_BDRLB> { static constexpr int N = 3; static constexpr int idx[4] = {0, 1, 2, 0}; static constexpr bool nt[4] = {true, true, true, false}; };
// the ReLU gate read off the forward pass's output: DROP2 > 0 exactly where the mask kept a positive LIN1
template <> struct ColIn<COL_BDRLB_OUT> { static constexpr int N = 2; static constexpr int idx[4] = {0, 1, 0, 0}; static constexpr bool nt[4] = {true, false, false, false}; };
template <> struct ColIn<COL_BAOB> { static constexpr int N = 1; static constexpr int idx[4] = {0, 0, 0, 0}; static constexpr bool nt[4] = {false, false, false, false}; };

// Raw 128-bit loads of the inputs of one row chunk (inputs T, T+1, ...).
template <int KIND, int T>
__device__ __forceinline__ void col_load_raw(const ColArgs& a, const RowIdx& ix, int e0, int nv,
                                             h8 (&raw)[ColIn<KIND>::N]) {
    if constexpr (T < ColIn<KIND>::N) {
        const View& v = a.v[ColIn<KIND>::idx[T]];
        raw[T] = (h8)(half_t)0.0f;
        if (nv) raw[T] = ldg8<ColIn<KIND>::nt[T]>(v.p + view_offset(v, ix) + e0);
        col_load_raw<KIND, T + 1>(a, ix, e0, nv, raw);
    }
}

// One 8-pack of one row: elementwise output (stored to v[3]) and the running sums.
template <int KIND>
__device__ __forceinline__ void col_compute(const ColArgs& a, const RowIdx& ix, int e0, int nv,
                                            const F8 (&in)[4], const F8& fscale,
                                            float (&acc)[ColTraits<KIND>::NS][8]) {
    if (KIND == COL_BSB) {
        // in0 IN (normed), in1 DOUT -> DIN
        h8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            o[i] = (half_t)(in[1].v[i] * fscale.v[i]);
            acc[0][i] += in[1].v[i] * in[0].v[i];
            acc[1][i] += in[1].v[i];
        }
        store8h(a.v[3], view_offset(a.v[3], ix), e0, nv, o);
    } else if (KIND == COL_EBSB) {
        // in0 IN, in1 DOUT1, in2 DOUT2, in3 DLINEAR -> DIN
        h8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float d = in[1].v[i] + in[2].v[i];
            o[i] = (half_t)(d * fscale.v[i]);
            acc[0][i] += d * in[0].v[i];
            acc[1][i] += d;
            acc[2][i] += in[3].v[i];
        }
        store8h(a.v[3], view_offset(a.v[3], ix), e0, nv, o);
    } else if (KIND == COL_BDRLB) {
        // in0 DDROP, in1 MASK, in2 LIN -> DLINEAR
        h8 oh;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float d = in[0].v[i] * in[1].v[i];
            float g = a.act == ACT_GELU ? gelu_bwd(in[2].v[i], d) : (in[2].v[i] > 0.f ? d : 0.f);
            oh[i] = (half_t)g;
        }
        oh = pin(oh);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[0][i] += i < nv ? (float)oh[i] : 0.f;
        store8h(a.v[3], view_offset(a.v[3], ix), e0, nv, oh);
    } else if (KIND == COL_BDRLB_OUT) {
        // in0 DDROP, in1 DROP2 (= relu(LIN1) * mask) -> DLINEAR
        h8 oh;
#pragma unroll
        for (int i = 0; i < 8; ++i) oh[i] = (half_t)(in[1].v[i] > 0.f ? in[0].v[i] : 0.f);
        oh = pin(oh);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[0][i] += i < nv ? (float)oh[i] : 0.f;
        store8h(a.v[3], view_offset(a.v[3], ix), e0, nv, oh);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[0][i] += in[0].v[i];
    }
}

// grid.x = feature strips of lpr*8 features, grid.y = token chunks, grid.z = kept
// outer index (i0,i1).  The sums run over the two inner outer dims (i2,i3).
// FAST: every big tensor is vectorisable (128-bit packs kept raw until used).
template <int KIND, bool FAST>
__global__ __launch_bounds__(BLOCK) void k_colreduce(RowSpace rs, ColArgs a, float* ws, int lpr_log2,
                                                     long rows_per_block, long nrows) {
    constexpr int NS = ColTraits<KIND>::NS;
    constexpr int NIN = ColIn<KIND>::N;
    constexpr int U = FAST ? 2 : 1;                    // rows in flight per lane
    __shared__ float red[BLOCK][9];          // +1 pad: conflict-free column reads
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lpr = 1 << lpr_log2, rpw = WAVE >> lpr_log2;
    const int fl = lane & (lpr - 1), sub = lane >> lpr_log2;
    const int e0 = (blockIdx.x * lpr + fl) * 8;
    int nv = rs.R - e0; nv = nv < 0 ? 0 : (nv > 8 ? 8 : nv);
    long row_begin = (long)blockIdx.y * rows_per_block;
    long row_end = row_begin + rows_per_block; row_end = row_end < nrows ? row_end : nrows;
    float acc[NS][8];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[s][i] = 0.f;
    F8 fscale;
    if (KIND == COL_BSB || KIND == COL_EBSB) fscale = load8(a.v[5], 0, e0, nv);
    if (nv > 0) {
        const unsigned n3 = (unsigned)rs.n3, stride = WPB * rpw;
        const unsigned i1 = blockIdx.z % (unsigned)rs.n1, i0 = blockIdx.z / (unsigned)rs.n1;
        for (unsigned row = (unsigned)row_begin + wave * rpw + sub; row < (unsigned)row_end; row += stride * U) {
            RowIdx ix[U];
            h8 raw[U][NIN];
            F8 gen[4];
            int nvu[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                unsigned r = row + u * stride;
                nvu[u] = r < (unsigned)row_end ? nv : 0;
                r = nvu[u] ? r : row;
                ix[u].i0 = i0; ix[u].i1 = i1;
                ix[u].i2 = r / n3; ix[u].i3 = r - ix[u].i2 * n3;
                if (FAST) {
                    col_load_raw<KIND, 0>(a, ix[u], e0, nvu[u], raw[u]);
                } else {
#pragma unroll
                    for (int t = 0; t < NIN; ++t) {
                        const View& v = a.v[ColIn<KIND>::idx[t]];
                        gen[t] = load8(v, view_offset(v, ix[u]), e0, nvu[u]);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (!nvu[u]) continue;
                if (FAST) {
#pragma unroll
                    for (int t = 0; t < NIN; ++t)
#pragma unroll
                        for (int i = 0; i < 8; ++i) gen[t].v[i] = (float)raw[u][t][i];
                }
                col_compute<KIND>(a, ix[u], e0, nvu[u], gen, fscale, acc);
            }
        }
    }
    const int ntc = gridDim.y;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 8; ++i) red[tid][i] = acc[s][i];
        __syncthreads();
        if (tid < lpr && nv > 0) {
            float tot[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) tot[i] = 0.f;
            for (int t = tid; t < BLOCK; t += lpr)
#pragma unroll
                for (int i = 0; i < 8; ++i) tot[i] += red[t][i];
            float* dst = ws + (((long)s * gridDim.z + blockIdx.z) * ntc + blockIdx.y) * rs.R + e0;
            for (int i = 0; i < nv; ++i) dst[i] = tot[i];
        }
    }
}

// Adds the ntc partials of every (sum, kept index, feature) of up to
// kMaxFinishJobs operators in one launch: blockIdx.y selects the operator, 32
// features x 8 slices per block, the slices combined through LDS.
__global__ __launch_bounds__(kFinishThreads) void k_colfinish(FinishJobs jobs) {
    __shared__ float red[8][33];
    finish_block(jobs.j[blockIdx.y], blockIdx.x, red);
}

struct ColPlan {
    int lpr_log2, nstrips, ntc;
    long rows_per_block;
};

inline ColPlan col_plan(const RowSpace& rs) {
    const long nbatch = (long)rs.n0 * rs.n1;
    ColPlan p;
    int chunks = (rs.R + 7) / 8;
    p.lpr_log2 = 0;
    // at most 16 lanes (128 features, 256 contiguous bytes) per row: more strips,
    // fewer token chunks for the finishing kernel to add up
    while ((1 << p.lpr_log2) < chunks && p.lpr_log2 < 4) ++p.lpr_log2;
    int lpr = 1 << p.lpr_log2;
    p.nstrips = (chunks + lpr - 1) / lpr;
    long nrows = (long)rs.n2 * rs.n3;
    int rows_per_iter = WPB * (WAVE / lpr);
    // aim for ~2048 blocks in total (8 per CU), at least one 2-row-deep iteration per wave
    long want_tc = 2048 / (p.nstrips * nbatch); if (want_tc < 1) want_tc = 1;
    long rpb = (nrows + want_tc - 1) / want_tc;
    if (rpb < 2L * rows_per_iter) rpb = 2L * rows_per_iter;
    rpb = (rpb + rows_per_iter - 1) / rows_per_iter * rows_per_iter;
    p.rows_per_block = rpb;
    p.ntc = (int)((nrows + rpb - 1) / rpb);
    if (p.ntc < 1) p.ntc = 1;
    return p;
}

template <int KIND>
void run_col(const RowSpace& rs, const ColArgs& a, FinishArgs fo, float* ws, hipStream_t st,
             const char* what, FinishJobs* defer) {
    constexpr int NS = ColTraits<KIND>::NS;
    if (rs.R <= 0) return;
    if (!ws) fail(std::string(what) + ": no reduction workspace");
    ColPlan p = col_plan(rs);
    long nrows = (long)rs.n2 * rs.n3;
    int nbatch = rs.n0 * rs.n1;
    if (nrows == 0 || nbatch == 0) return;
    if (nbatch > 65535) fail(std::string(what) + ": too many kept rows");
    fo.n1 = rs.n1;
    bool fast = true;       // inputs and the elementwise output are all 128-bit addressable
    for (int t = 0; t < ColIn<KIND>::N; ++t) fast = fast && a.v[ColIn<KIND>::idx[t]].vec;
    if (KIND != COL_BAOB) fast = fast && a.v[3].vec;
    if (fast)
        hipLaunchKernelGGL((k_colreduce<KIND, true>), dim3(p.nstrips, p.ntc, nbatch), dim3(BLOCK), 0, st, rs,
                           a, ws, p.lpr_log2, p.rows_per_block, nrows);
    else
        hipLaunchKernelGGL((k_colreduce<KIND, false>), dim3(p.nstrips, p.ntc, nbatch), dim3(BLOCK), 0, st, rs,
                           a, ws, p.lpr_log2, p.rows_per_block, nrows);
    check_launch(what);
    FinishJob job{ws, fo, NS, nbatch, p.ntc, rs.R};
    finish_or_defer(defer, job, st);
}

// One wave per (i0,i1,i2): sum over i3 and the row.
__global__ __launch_bounds__(BLOCK) void k_rowgroup_sum(RowSpace rs, View d, View out, long ngroups) {
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * WPB;
    for (long g = (long)blockIdx.x * WPB + (threadIdx.x >> 6); g < ngroups; g += nwaves) {
        unsigned gg = (unsigned)g;
        unsigned r = gg / (unsigned)rs.n2; unsigned i2 = gg - r * (unsigned)rs.n2;
        unsigned i0 = r / (unsigned)rs.n1; unsigned i1 = r - i0 * (unsigned)rs.n1;
        long base = (long)i0 * d.s0 + (long)i1 * d.s1 + (long)i2 * d.s2;
        float s = 0.f;
        for (int i3 = 0; i3 < rs.n3; ++i3) {
            long ob = base + (long)i3 * d.s3;
            for (int e0 = lane * 8; e0 < rs.R; e0 += WAVE * 8) {
                int nv = rs.R - e0; nv = nv > 8 ? 8 : nv;
                F8 f = load8(d, ob, e0, nv);
#pragma unroll
                for (int i = 0; i < 8; ++i) s += f.v[i];
            }
        }
        s = wave_sum(s);
        if (lane == 0) out.p[(long)i0 * out.s0 + (long)i1 * out.s1 + (long)i2 * out.s2] = (half_t)s;
    }
}

}  // namespace

void launch_colfinish(const FinishJobs& jobs, hipStream_t st) {
    if (jobs.n == 0) return;
    hipLaunchKernelGGL(k_colfinish, dim3((unsigned)finish_groups(jobs), jobs.n), dim3(kFinishThreads), 0, st, jobs);
    check_launch("column-sum finish");
}

size_t colreduce_ws_floats(const RowSpace& rs, int nsums) {
    ColPlan p = col_plan(rs);
    return (size_t)nsums * rs.n0 * rs.n1 * p.ntc * rs.R;
}

void launch_bsb(const RowSpace& rs, View in, View dout, View scale, View din, ColOut dscale,
                ColOut dbias, float* ws, hipStream_t st, FinishJobs* defer) {
    ColArgs a{}; a.v[0] = in; a.v[1] = dout; a.v[3] = din; a.v[5] = scale; a.act = 0;
    FinishArgs fo{{dscale.p, dbias.p, nullptr}, 0, 0, 1, 1};
    run_col<COL_BSB>(rs, a, fo, ws, st, "backward scale-bias", defer);
}

void launch_ebsb(const RowSpace& rs, View in, View dout1, View dout2, View dlinear, View scale,
                 View din, ColOut dscale, ColOut dbias, ColOut dlinear_bias, float* ws,
                 hipStream_t st, FinishJobs* defer) {
    ColArgs a{}; a.v[0] = in; a.v[1] = dout1; a.v[2] = dout2; a.v[3] = din; a.v[4] = dlinear;
    a.v[5] = scale; a.act = 0;
    FinishArgs fo{{dscale.p, dbias.p, dlinear_bias.p}, 0, 0, 1, 1};
    run_col<COL_EBSB>(rs, a, fo, ws, st, "extended backward scale-bias", defer);
}

void launch_bdrlb(const RowSpace& rs, View ddrop, View mask, View lin, View dlinear, ColOut dbias,
                  int act, float* ws, hipStream_t st, FinishJobs* defer) {
    ColArgs a{}; a.v[0] = ddrop; a.v[1] = mask; a.v[2] = lin; a.v[3] = dlinear; a.act = act;
    FinishArgs fo{{dbias.p, nullptr, nullptr}, 0, 0, 1, 1};
    run_col<COL_BDRLB>(rs, a, fo, ws, st, "backward dropout-activation-bias", defer);
}

void launch_bdrlb_from_output(const RowSpace& rs, View ddrop, View out, View dlinear, ColOut dbias, float* ws,
                              hipStream_t st, FinishJobs* defer) {
    ColArgs a{}; a.v[0] = ddrop; a.v[1] = out; a.v[3] = dlinear; a.act = 0;
    FinishArgs fo{{dbias.p, nullptr, nullptr}, 0, 0, 1, 1};
    run_col<COL_BDRLB_OUT>(rs, a, fo, ws, st, "backward dropout-relu-bias", defer);
}

void launch_baob(const RowSpace& rs, View datt, ColOut dbo, float* ws, hipStream_t st, FinishJobs* defer) {
    ColArgs a{}; a.v[0] = datt; a.act = 0;
    FinishArgs fo{{dbo.p, nullptr, nullptr}, 0, 0, 1, 1};
    run_col<COL_BAOB>(rs, a, fo, ws, st, "backward attention-output bias", defer);
}

void launch_colsum(const RowSpace& rs, View d, half_t* out, long ob0, long ob1, long of, float* ws,
                   hipStream_t st, FinishJobs* defer) {
    ColArgs a{}; a.v[0] = d; a.act = 0;
    FinishArgs fo{{out, nullptr, nullptr}, ob0, ob1, of, 1};
    run_col<COL_BAOB>(rs, a, fo, ws, st, "column sum", defer);
}

void launch_baib(const RowSpace& rs, View d, View out, hipStream_t st) {
    long ngroups = (long)rs.n0 * rs.n1 * rs.n2;
    if (ngroups == 0) return;
    long blocks = (ngroups + WPB - 1) / WPB;
    if (blocks > 256L * 64) blocks = 256L * 64;
    hipLaunchKernelGGL(k_rowgroup_sum, dim3((unsigned)blocks), dim3(BLOCK), 0, st, rs, d, out, ngroups);
    check_launch("backward attention-input biases");
}

}  // namespace sub
