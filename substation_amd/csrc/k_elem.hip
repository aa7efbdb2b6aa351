// Elementwise operators: bias + activation + dropout (forward), and the plain
// add used for the attention input biases and the encoder-input gradient.
// Counterparts: pytorch_module/block_bad.cuh:28-145, block_aib.cuh:17-155,
// block_bei.cuh:12-106.  Each lane moves 128-bit packs, two per tensor per step.
#include "sub_ops.hpp"

namespace sub {

namespace {

constexpr int BLOCK = 256;
constexpr int UNROLL = 2;

struct Chunk {
    unsigned row;
    int e0, nv;
    RowIdx ix;
};

template <bool FLAT = false>
__device__ __forceinline__ Chunk chunk_of(const RowSpace& rs, unsigned idx, unsigned nchunks, unsigned cpr) {
    Chunk c;
    const bool live = idx < nchunks;
    unsigned id = live ? idx : 0;
    c.row = id / cpr;
    c.e0 = (int)(id - c.row * cpr) * 8;
    int nv = rs.R - c.e0;
    c.nv = live ? (nv > 8 ? 8 : nv) : 0;
    c.ix = row_index_of<FLAT>(rs, c.row);
    return c;
}

// ACT, FLAT: the activation and a flat row space as compile-time facts (a choice of activation per element
// is a branch per element; a strided row space three divisions per pack of 8).
template <bool FAST, int ACT = -1, bool FLAT = false>
__global__ __launch_bounds__(BLOCK) void k_bad(RowSpace rs, View in, View bias, View lin, View mask,
                                               View out, int act, PhiloxKey key_, unsigned nchunks,
                                               unsigned cpr, int out_only) {
    const PhiloxKey key = resolved(key_);
    const unsigned stride = gridDim.x * BLOCK;
    for (unsigned base = blockIdx.x * BLOCK + threadIdx.x; base < nchunks; base += stride * UNROLL) {
        Chunk c[UNROLL];
        F8 fi[UNROLL], fb[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            c[u] = chunk_of<FLAT>(rs, base + u * stride, nchunks, cpr);
            fi[u] = ld8<FAST, true>(in, view_offset_of<FLAT>(in, c[u].ix), c[u].e0, c[u].nv);
            fb[u] = ld8<FAST>(bias, 0, c[u].e0, c[u].nv);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (c[u].nv == 0) continue;
            uint32_t bits = keep_pack<FAST>(key, (uint64_t)c[u].row * (uint64_t)rs.R + (uint64_t)c[u].e0);
            h8 lh, oh;
#pragma unroll
            for (int i = 0; i < 8; ++i) lh[i] = (half_t)(fi[u].v[i] + fb[u].v[i]);
            lh = pin(lh);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float l = (float)lh[i];
                float a = (ACT < 0 ? act : ACT) == ACT_GELU ? gelu_fwd(l) : fmaxf(l, 0.f);
                oh[i] = ((bits >> i) & 1u) ? (half_t)a : (half_t)0.0f;
            }
            if (!out_only) {
                st8h<FAST, true>(lin, view_offset_of<FLAT>(lin, c[u].ix), c[u].e0, c[u].nv, lh);
                st8h<FAST, true>(mask, view_offset_of<FLAT>(mask, c[u].ix), c[u].e0, c[u].nv, mask_h8(bits));
            }
            st8h<FAST>(out, view_offset_of<FLAT>(out, c[u].ix), c[u].e0, c[u].nv, oh);
        }
    }
}

template <bool FAST>
__global__ __launch_bounds__(BLOCK) void k_add(RowSpace rs, View a, View b, View out, unsigned nchunks,
                                               unsigned cpr) {
    const unsigned stride = gridDim.x * BLOCK;
    for (unsigned base = blockIdx.x * BLOCK + threadIdx.x; base < nchunks; base += stride * UNROLL) {
        Chunk c[UNROLL];
        F8 fa[UNROLL], fb[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            c[u] = chunk_of(rs, base + u * stride, nchunks, cpr);
            fa[u] = ld8<FAST>(a, view_offset(a, c[u].ix), c[u].e0, c[u].nv);
            // b may be a broadcast along the row (stride 0): generic load
            fb[u] = b.vec ? ld8<FAST>(b, view_offset(b, c[u].ix), c[u].e0, c[u].nv)
                          : load8(b, view_offset(b, c[u].ix), c[u].e0, c[u].nv);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (c[u].nv == 0) continue;
            h8 o;
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = (half_t)(fa[u].v[i] + fb[u].v[i]);
            st8h<FAST>(out, view_offset(out, c[u].ix), c[u].e0, c[u].nv, o);
        }
    }
}

inline int elem_grid(long nchunks) {
    long blocks = (nchunks + (long)BLOCK * UNROLL - 1) / ((long)BLOCK * UNROLL);
    const long cap = 256L * 32;
    return (int)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

inline unsigned check_chunks(long nchunks, const char* what) {
    if (nchunks >= (1L << 31)) fail(std::string(what) + ": tensor too large");
    return (unsigned)nchunks;
}

}  // namespace

void launch_bad(const RowSpace& rs, View in, View bias, View lin, View mask, View out, int act,
                PhiloxKey key, hipStream_t st, bool out_only) {
    unsigned cpr = (unsigned)((rs.R + 7) / 8);
    unsigned nchunks = check_chunks(rs.rows() * cpr, "bias-activation-dropout");
    if (nchunks == 0) return;
    const bool fast = in.vec && bias.vec && lin.vec && mask.vec && out.vec;
#define SUB_BAD(...) hipLaunchKernelGGL((k_bad<__VA_ARGS__>), dim3(elem_grid(nchunks)), dim3(BLOCK), 0, st, rs, in, bias, lin, \
                                        mask, out, act, key, nchunks, cpr, out_only ? 1 : 0)
    if (fast && rs.flat && act == ACT_GELU) SUB_BAD(true, ACT_GELU, true);
    else if (fast && rs.flat) SUB_BAD(true, ACT_RELU, true);
    else if (fast && act == ACT_GELU) SUB_BAD(true, ACT_GELU, false);
    else if (fast) SUB_BAD(true, ACT_RELU, false);
#undef SUB_BAD
    else
        hipLaunchKernelGGL(k_bad<false>, dim3(elem_grid(nchunks)), dim3(BLOCK), 0, st, rs, in, bias, lin,
                           mask, out, act, key, nchunks, cpr, out_only ? 1 : 0);
    check_launch("bias-activation-dropout");
}

void launch_add(const RowSpace& rs, View a, View b, View out, hipStream_t st) {
    unsigned cpr = (unsigned)((rs.R + 7) / 8);
    unsigned nchunks = check_chunks(rs.rows() * cpr, "add");
    if (nchunks == 0) return;
    const bool fast = a.vec && out.vec;
    if (fast)
        hipLaunchKernelGGL(k_add<true>, dim3(elem_grid(nchunks)), dim3(BLOCK), 0, st, rs, a, b, out, nchunks, cpr);
    else
        hipLaunchKernelGGL(k_add<false>, dim3(elem_grid(nchunks)), dim3(BLOCK), 0, st, rs, a, b, out, nchunks, cpr);
    check_launch("add");
}

}  // namespace sub
