// Elementwise operators: bias + activation + dropout (forward), and the plain
// add used for the attention input biases and the encoder-input gradient.
// Counterparts: pytorch_module/block_bad.cuh:28-145, block_aib.cuh:17-155,
// block_bei.cuh:12-106.  Each lane moves one 128-bit pack per tensor per step.
#include "sub_ops.hpp"

namespace sub {

namespace {

constexpr int BLOCK = 256;

__device__ __forceinline__ float gelu_fwd(float x) {
    const float c = 0.7978845608028654f;
    float u = c * (x + 0.044715f * x * x * x);
    float t = 1.0f - 2.0f / (1.0f + __expf(2.0f * u));   // tanh(u)
    return 0.5f * x * (1.0f + t);
}

__global__ __launch_bounds__(BLOCK) void k_bad(RowSpace rs, View in, View bias, View lin, View mask,
                                               View out, int act, PhiloxKey key, long nchunks, int cpr) {
    const long stride = (long)gridDim.x * BLOCK;
    for (long idx = (long)blockIdx.x * BLOCK + threadIdx.x; idx < nchunks; idx += stride) {
        long row = idx / cpr;
        int e0 = (int)(idx - row * cpr) * 8;
        int nv = rs.R - e0; nv = nv > 8 ? 8 : nv;
        RowIdx ix = row_index(rs, row);
        F8 fi = load8(in, view_offset(in, ix), e0, nv);
        F8 fb = load8(bias, 0, e0, nv);
        uint32_t bits = keep_bits8(key, (uint64_t)row * (uint64_t)rs.R + (uint64_t)e0);
        h8 lh, oh;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            lh[i] = (half_t)(fi.v[i] + fb.v[i]);
            float l = (float)lh[i];
            float a = act == ACT_GELU ? gelu_fwd(l) : fmaxf(l, 0.f);
            oh[i] = ((bits >> i) & 1u) ? (half_t)a : (half_t)0.0f;
        }
        store8h(lin, view_offset(lin, ix), e0, nv, lh);
        store8h(mask, view_offset(mask, ix), e0, nv, mask_h8(bits));
        store8h(out, view_offset(out, ix), e0, nv, oh);
    }
}

__global__ __launch_bounds__(BLOCK) void k_add(RowSpace rs, View a, View b, View out, long nchunks,
                                               int cpr) {
    const long stride = (long)gridDim.x * BLOCK;
    for (long idx = (long)blockIdx.x * BLOCK + threadIdx.x; idx < nchunks; idx += stride) {
        long row = idx / cpr;
        int e0 = (int)(idx - row * cpr) * 8;
        int nv = rs.R - e0; nv = nv > 8 ? 8 : nv;
        RowIdx ix = row_index(rs, row);
        F8 fa = load8(a, view_offset(a, ix), e0, nv);
        F8 fb = load8(b, view_offset(b, ix), e0, nv);
        F8 o;
#pragma unroll
        for (int i = 0; i < 8; ++i) o.v[i] = fa.v[i] + fb.v[i];
        store8(out, view_offset(out, ix), e0, nv, o);
    }
}

inline int elem_grid(long nchunks) {
    long blocks = (nchunks + BLOCK - 1) / BLOCK;
    const long cap = 256L * 32;
    return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

}  // namespace

void launch_bad(const RowSpace& rs, View in, View bias, View lin, View mask, View out, int act,
                PhiloxKey key, hipStream_t st) {
    int cpr = (rs.R + 7) / 8;
    long nchunks = rs.rows() * cpr;
    if (nchunks == 0) return;
    hipLaunchKernelGGL(k_bad, dim3(elem_grid(nchunks)), dim3(BLOCK), 0, st, rs, in, bias, lin, mask,
                       out, act, key, nchunks, cpr);
    check_launch("bias-activation-dropout");
}

void launch_add(const RowSpace& rs, View a, View b, View out, hipStream_t st) {
    int cpr = (rs.R + 7) / 8;
    long nchunks = rs.rows() * cpr;
    if (nchunks == 0) return;
    hipLaunchKernelGGL(k_add, dim3(elem_grid(nchunks)), dim3(BLOCK), 0, st, rs, a, b, out, nchunks, cpr);
    check_launch("add");
}

}  // namespace sub
