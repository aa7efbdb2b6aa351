// Row operators: softmax(+scale+dropout), softmax backward, bias+dropout+
// residual+LayerNorm, LayerNorm backward(+dropout backward).
// One wave64 per row, the whole row in registers (single global read), fp32 math,
// 128-bit accesses where the row dimension is contiguous.
// Counterparts: pytorch_module/block_softmax.cuh:12-188, block_bs.cuh:13-156,
// block_bdrln.cuh:17-352, block_blnrd.cuh:14-259.
#include "sub_ops.hpp"

namespace sub {

namespace {

constexpr int BLOCK = 256;
constexpr int WPB = BLOCK / WAVE;
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ int nvalid_at(int R, int e0) {
    int n = R - e0;
    return n < 0 ? 0 : (n > 8 ? 8 : n);
}

template <int VPL>
__global__ __launch_bounds__(BLOCK) void k_softmax(RowSpace rs, View beta, View alpha, View mask,
                                                   View drop, float scale, PhiloxKey key, long nrows) {
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * WPB;
    for (long row = (long)blockIdx.x * WPB + (threadIdx.x >> 6); row < nrows; row += nwaves) {
        RowIdx ix = row_index(rs, row);
        const long ob = view_offset(beta, ix);
        float x[VPL][8];
        float m = -INFINITY;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            F8 f = load8(beta, ob, e0, nv, -INFINITY);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                x[c][i] = f.v[i] * scale;
                m = fmaxf(m, x[c][i]);
            }
        }
        m = wave_max(m);
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                x[c][i] = __builtin_amdgcn_exp2f((x[c][i] - m) * LOG2E);
                s += x[c][i];
            }
        s = wave_sum(s);
        const float inv = 1.0f / s;
        const long oa = view_offset(alpha, ix), om = view_offset(mask, ix), od = view_offset(drop, ix);
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            if (nv > 0) {
                h8 a, d;
                uint32_t bits = keep_bits8(key, (uint64_t)row * (uint64_t)rs.R + (uint64_t)e0);
                h8 mk = mask_h8(bits);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    a[i] = (half_t)(x[c][i] * inv);
                    d[i] = ((bits >> i) & 1u) ? a[i] : (half_t)0.0f;
                }
                store8h(alpha, oa, e0, nv, a);
                store8h(mask, om, e0, nv, mk);
                store8h(drop, od, e0, nv, d);
            }
        }
    }
}

template <int VPL>
__global__ __launch_bounds__(BLOCK) void k_bs(RowSpace rs, View alpha, View mask, View ddrop,
                                              View dbeta, float scale, long nrows) {
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * WPB;
    for (long row = (long)blockIdx.x * WPB + (threadIdx.x >> 6); row < nrows; row += nwaves) {
        RowIdx ix = row_index(rs, row);
        const long oa = view_offset(alpha, ix), om = view_offset(mask, ix), od = view_offset(ddrop, ix);
        float a[VPL][8], g[VPL][8];
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            F8 fa = load8(alpha, oa, e0, nv), fm = load8(mask, om, e0, nv), fd = load8(ddrop, od, e0, nv);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[c][i] = fa.v[i];
                g[c][i] = fm.v[i] * fd.v[i];
                s += a[c][i] * g[c][i];
            }
        }
        s = wave_sum(s);
        const long oo = view_offset(dbeta, ix);
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            if (nv > 0) {
                F8 o;
#pragma unroll
                for (int i = 0; i < 8; ++i) o.v[i] = scale * a[c][i] * (g[c][i] - s);
                store8(dbeta, oo, e0, nv, o);
            }
        }
    }
}

template <int VPL>
__global__ __launch_bounds__(BLOCK) void k_bdrln(RowSpace rs, View in, View resid, View lin_bias,
                                                 View scale, View bias, View lin, View mask,
                                                 View diff, View normed, View out, View istd,
                                                 PhiloxKey key, float eps, long nrows) {
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * WPB;
    const float invn = 1.0f / (float)rs.R;
    for (long row = (long)blockIdx.x * WPB + (threadIdx.x >> 6); row < nrows; row += nwaves) {
        RowIdx ix = row_index(rs, row);
        const long oi = view_offset(in, ix), orr = view_offset(resid, ix);
        const long ol = view_offset(lin, ix), om = view_offset(mask, ix);
        float r[VPL][8];
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            F8 fi = load8(in, oi, e0, nv), fr = load8(resid, orr, e0, nv);
            F8 fb = load8(lin_bias, 0, e0, nv);
            uint32_t bits = nv > 0 ? keep_bits8(key, (uint64_t)row * (uint64_t)rs.R + (uint64_t)e0) : 0u;
            h8 lh;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                lh[i] = (half_t)(fi.v[i] + fb.v[i]);           // LIN is stored; use its rounded value
                float kept = ((bits >> i) & 1u) ? (float)lh[i] : 0.f;
                r[c][i] = i < nv ? kept + fr.v[i] : 0.f;
                s += r[c][i];
            }
            if (nv > 0) {
                store8h(lin, ol, e0, nv, lh);
                store8h(mask, om, e0, nv, mask_h8(bits));
            }
        }
        const float mean = wave_sum(s) * invn;
        float q = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                r[c][i] = i < nv ? r[c][i] - mean : 0.f;
                q += r[c][i] * r[c][i];
            }
        }
        const float var = wave_sum(q) * invn;
        const float is = rsqrtf(var + eps);
        if (lane == 0) istd.p[view_offset(istd, ix)] = (half_t)is;
        const long od = view_offset(diff, ix), on = view_offset(normed, ix), oo = view_offset(out, ix);
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            if (nv > 0) {
                F8 fs = load8(scale, 0, e0, nv), fb = load8(bias, 0, e0, nv);
                F8 d, n, o;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    d.v[i] = r[c][i];
                    n.v[i] = r[c][i] * is;
                    o.v[i] = n.v[i] * fs.v[i] + fb.v[i];
                }
                store8(diff, od, e0, nv, d);
                store8(normed, on, e0, nv, n);
                store8(out, oo, e0, nv, o);
            }
        }
    }
}

template <int VPL>
__global__ __launch_bounds__(BLOCK) void k_blnrd(RowSpace rs, View dout, View istd, View diff,
                                                 View mask, View d_ln_in, View d_drop_in, long nrows) {
    const int lane = threadIdx.x & 63;
    const long nwaves = (long)gridDim.x * WPB;
    const float invn = 1.0f / (float)rs.R;
    for (long row = (long)blockIdx.x * WPB + (threadIdx.x >> 6); row < nrows; row += nwaves) {
        RowIdx ix = row_index(rs, row);
        const long oo = view_offset(dout, ix), od = view_offset(diff, ix);
        float g[VPL][8], df[VPL][8];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            F8 fg = load8(dout, oo, e0, nv), fd = load8(diff, od, e0, nv);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                g[c][i] = fg.v[i];
                df[c][i] = fd.v[i];
                s1 += g[c][i];
                s2 += g[c][i] * df[c][i];
            }
        }
        s1 = wave_sum(s1);
        s2 = wave_sum(s2);
        const float is = (float)istd.p[view_offset(istd, ix)];
        const float c1 = s1 * is * invn;
        const float c2 = s2 * is * is * is * invn;
        const long om = view_offset(mask, ix), o1 = view_offset(d_ln_in, ix), o2 = view_offset(d_drop_in, ix);
#pragma unroll
        for (int c = 0; c < VPL; ++c) {
            int e0 = (c * WAVE + lane) * 8;
            int nv = nvalid_at(rs.R, e0);
            if (nv > 0) {
                F8 fm = load8(mask, om, e0, nv);
                h8 a, b;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    a[i] = (half_t)(g[c][i] * is - c1 - df[c][i] * c2);
                    b[i] = fm.v[i] != 0.f ? a[i] : (half_t)0.0f;
                }
                store8h(d_ln_in, o1, e0, nv, a);
                store8h(d_drop_in, o2, e0, nv, b);
            }
        }
    }
}

inline int pick_vpl(int R, const char* what) {
    if (R <= 0) fail(std::string(what) + ": empty row");
    if (R <= 512) return 1;
    if (R <= 1024) return 2;
    if (R <= 2048) return 4;
    if (R <= 4096) return 8;
    fail(std::string(what) + ": rows longer than 4096 elements are not supported");
}

inline int row_grid(long nrows) {
    long blocks = (nrows + WPB - 1) / WPB;
    const long cap = 256L * 64;          // 256 CUs, waves beyond this loop
    return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

}  // namespace

#define SUB_DISPATCH_VPL(vpl, KERNEL, ...)                                                   \
    switch (vpl) {                                                                           \
        case 1: hipLaunchKernelGGL(KERNEL<1>, dim3(grid), dim3(BLOCK), 0, st, __VA_ARGS__); break; \
        case 2: hipLaunchKernelGGL(KERNEL<2>, dim3(grid), dim3(BLOCK), 0, st, __VA_ARGS__); break; \
        case 4: hipLaunchKernelGGL(KERNEL<4>, dim3(grid), dim3(BLOCK), 0, st, __VA_ARGS__); break; \
        default: hipLaunchKernelGGL(KERNEL<8>, dim3(grid), dim3(BLOCK), 0, st, __VA_ARGS__); break; \
    }

void launch_softmax(const RowSpace& rs, View beta, View alpha, View mask, View drop, float scale,
                    PhiloxKey key, hipStream_t st) {
    long nrows = rs.rows();
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "softmax");
    int grid = row_grid(nrows);
    SUB_DISPATCH_VPL(vpl, k_softmax, rs, beta, alpha, mask, drop, scale, key, nrows);
    check_launch("softmax");
}

void launch_bs(const RowSpace& rs, View alpha, View mask, View ddrop, View dbeta, float scale,
               hipStream_t st) {
    long nrows = rs.rows();
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "softmax backward");
    int grid = row_grid(nrows);
    SUB_DISPATCH_VPL(vpl, k_bs, rs, alpha, mask, ddrop, dbeta, scale, nrows);
    check_launch("softmax backward");
}

void launch_bdrln(const RowSpace& rs, View in, View resid, View lin_bias, View scale, View bias,
                  View lin, View mask, View diff, View normed, View out, View istd, PhiloxKey key,
                  float eps, hipStream_t st) {
    long nrows = rs.rows();
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "bias-dropout-residual-layernorm");
    int grid = row_grid(nrows);
    SUB_DISPATCH_VPL(vpl, k_bdrln, rs, in, resid, lin_bias, scale, bias, lin, mask, diff, normed,
                     out, istd, key, eps, nrows);
    check_launch("bias-dropout-residual-layernorm");
}

void launch_blnrd(const RowSpace& rs, View dout, View istd, View diff, View mask, View d_ln_in,
                  View d_drop_in, hipStream_t st) {
    long nrows = rs.rows();
    if (nrows == 0) return;
    int vpl = pick_vpl(rs.R, "layernorm backward");
    int grid = row_grid(nrows);
    SUB_DISPATCH_VPL(vpl, k_blnrd, rs, dout, istd, diff, mask, d_ln_in, d_drop_in, nrows);
    check_launch("layernorm backward");
}

}  // namespace sub
