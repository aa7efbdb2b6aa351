// Device-side building blocks for the fused (memory-bound) operators:
// 128-bit fp16 packs with fp32 math, wave64 reductions on DPP, strided views.
// Takes the place of pytorch_module/{half8,vector_types,warpreduce}.cuh.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

#include "sub_philox.hpp"

namespace sub {

typedef _Float16 half_t;
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

constexpr int WAVE = 64;

// Row space: up to four outer dimensions (canonical order) times a row of R
// elements.  The canonical element index of (row r, column e) is r*R + e.
// flat != 0: the three leading outer dims have extent 1 (after the host merged
// dims that every view strides through uniformly), so row == i3.
struct RowSpace {
    int n0, n1, n2, n3;
    int R;
    int flat;
    long rows() const { return (long)n0 * n1 * n2 * n3; }
};

// A tensor seen through the row space: strides of the four outer dims and of
// the row dim, in elements.  vec != 0 promises that 8 consecutive row elements
// starting at a multiple of 8 are one aligned 16-byte word.
struct View {
    half_t* p;
    long s0, s1, s2, s3;
    long sr;
    int vec;
};

struct F8 {
    float v[8];
};

// Outer indices of a row, computed once and reused for every view.
struct RowIdx {
    unsigned i0, i1, i2, i3;
};
__device__ __forceinline__ RowIdx row_index(const RowSpace& rs, unsigned row) {
    RowIdx x;
    if (rs.flat) {
        x.i0 = x.i1 = x.i2 = 0; x.i3 = row;
    } else {
        unsigned r = row / (unsigned)rs.n3; x.i3 = row - r * (unsigned)rs.n3;
        unsigned q = r / (unsigned)rs.n2; x.i2 = r - q * (unsigned)rs.n2;
        x.i0 = q / (unsigned)rs.n1; x.i1 = q - x.i0 * (unsigned)rs.n1;
    }
    return x;
}
__device__ __forceinline__ long view_offset(const View& t, const RowIdx& x) {
    return (long)x.i0 * t.s0 + (long)x.i1 * t.s1 + (long)x.i2 * t.s2 + (long)x.i3 * t.s3;
}

// The same for a kernel instantiated for a flat row space (FLAT: RowSpace::flat, the row is its only
// index): one multiplication per view in place of three divisions per row and four products per view.
template <bool FLAT>
__device__ __forceinline__ RowIdx row_index_of(const RowSpace& rs, unsigned row) {
    if (FLAT) { RowIdx x; x.i0 = x.i1 = x.i2 = 0; x.i3 = row; return x; }
    return row_index(rs, row);
}
template <bool FLAT>
__device__ __forceinline__ long view_offset_of(const View& t, const RowIdx& x) {
    return FLAT ? (long)x.i3 * t.s3 : view_offset(t, x);
}

// Load 8 row elements e0 .. e0+7 (nvalid of them inside the row) as fp32.
__device__ __forceinline__ F8 load8(const View& t, long base, int e0, int nvalid, float fill = 0.f) {
    F8 r;
    const half_t* p = t.p + base;
    if (t.vec && nvalid == 8) {
        h8 v = *reinterpret_cast<const h8*>(p + e0);
#pragma unroll
        for (int i = 0; i < 8; ++i) r.v[i] = (float)v[i];
    } else if (t.sr == 0) {
        float x = nvalid > 0 ? (float)p[0] : fill;
#pragma unroll
        for (int i = 0; i < 8; ++i) r.v[i] = i < nvalid ? x : fill;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) r.v[i] = i < nvalid ? (float)p[(long)(e0 + i) * t.sr] : fill;
    }
    return r;
}

__device__ __forceinline__ h8 to_h8(const F8& x) {
    h8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (half_t)x.v[i];
    return v;
}

__device__ __forceinline__ void store8h(const View& t, long base, int e0, int nvalid, h8 v) {
    half_t* p = t.p + base;
    if (t.vec && nvalid == 8) {
        *reinterpret_cast<h8*>(p + e0) = v;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i < nvalid) p[(long)(e0 + i) * t.sr] = v[i];
    }
}

__device__ __forceinline__ void store8(const View& t, long base, int e0, int nvalid, const F8& x) {
    store8h(t, base, e0, nvalid, to_h8(x));
}

// FAST variants: every view is vectorisable and rows are whole 8-packs, so a
// chunk is either entirely inside the row (nvalid == 8) or entirely outside.
// NT marks a streamed tensor: one saved for the backward pass (written now,
// read again only much later) or read for the last time.  The nontemporal hint
// keeps it from displacing lines that the next launch is about to read; tensors
// handed to the next launch and the per-feature vectors every wave re-reads are
// accessed normally.  (A compile-time choice: a run-time select between the two
// access forms is folded into one plain access by the optimiser.)
template <bool NT>
__device__ __forceinline__ h8 ldg8(const half_t* p) {
    return NT ? __builtin_nontemporal_load(reinterpret_cast<const h8*>(p))
              : *reinterpret_cast<const h8*>(p);
}
template <bool NT>
__device__ __forceinline__ void stg8(half_t* p, h8 v) {
    if (NT) __builtin_nontemporal_store(v, reinterpret_cast<h8*>(p));
    else *reinterpret_cast<h8*>(p) = v;
}

template <bool FAST, bool NT = false>
__device__ __forceinline__ F8 ld8(const View& t, long base, int e0, int nvalid, float fill = 0.f) {
    if (FAST) {
        // A chunk outside the row reads the row's first pack instead (`base` is a valid row
        // also for a lane without one) and is replaced afterwards.  No branch around the load:
        // the wait for it would sit inside the branch, and a kernel that reads three tensors
        // would make three round trips to memory one after the other instead of one.
        const bool inside = nvalid != 0;
        const h8 v = ldg8<NT>(t.p + base + (inside ? e0 : 0));
        F8 r;
#pragma unroll
        for (int i = 0; i < 8; ++i) r.v[i] = inside ? (float)v[i] : fill;
        return r;
    }
    return load8(t, base, e0, nvalid, fill);
}

template <bool FAST, bool NT = false>
__device__ __forceinline__ void st8h(const View& t, long base, int e0, int nvalid, h8 v) {
    if (FAST) {
        if (nvalid) stg8<NT>(t.p + base + e0, v);
    } else {
        store8h(t, base, e0, nvalid, v);
    }
}

// Kernel arguments wanted in registers now.  Left alone, the compiler fetches each argument where it is
// first used, with a wait of its own: a kernel with many of them then starts with four or five scalar
// round trips to memory one after the other (about half a microsecond each) before its first vector
// load is issued.  Named here, they are fetched in one go.
template <typename T>
__device__ __forceinline__ void fetch_arg_now(const T& v) {
    if constexpr (sizeof(T) < 4) { const int w = (int)v; asm volatile("" ::"s"(w)); }
    else asm volatile("" ::"s"(v));
}
template <typename... T>
__device__ __forceinline__ void fetch_args_now(const T&... v) { (fetch_arg_now(v), ...); }

// The key a kernel works with: the device-side step counter, if any, folded in.
__device__ __forceinline__ PhiloxKey resolved(PhiloxKey k) {
    if (k.step_dev) k.step += *k.step_dev;
    k.step_dev = nullptr;
    return k;
}

// x ^ y ^ k in one instruction (k uniform).
__device__ __forceinline__ uint32_t xor3(uint32_t x, uint32_t y, uint32_t k) {
    uint32_t r;
    asm("v_bitop3_b32 %0, %1, %2, %3 bitop3:0x96" : "=v"(r) : "v"(x), "v"(y), "s"(k));
    return r;
}

// philox_group() of sub_philox.hpp, bit for bit, with the two xors of each
// half-round folded into one instruction.
__device__ __forceinline__ U4 philox_group_dev(const PhiloxKey& k, uint64_t g) {
    U4 c;
    c.x = (uint32_t)g; c.y = (uint32_t)(g >> 32); c.z = k.site; c.w = k.step;
    uint32_t k0 = k.k0, k1 = k.k1;
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        uint32_t hi0, lo0, hi1, lo1;
        mulhilo(0xD2511F53u, c.x, hi0, lo0);
        mulhilo(0xCD9E8D57u, c.z, hi1, lo1);
        U4 n;
        n.x = xor3(hi1, c.y, k0);
        n.y = lo1;
        n.z = xor3(hi0, c.w, k1);
        n.w = lo0;
        c = n;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c;
}

// Keep bits of the 8-pack that starts at canonical element e.  FAST: rows are whole 8-packs, so
// e is a multiple of 8 and the pack is one Philox group (no second call, no branch on e & 7).
template <bool FAST>
__device__ __forceinline__ uint32_t keep_pack(const PhiloxKey& key, uint64_t e) {
    return FAST ? keep8(philox_group_dev(key, e >> 3), key.thr) : keep_bits8(key, e);
}

// The 32 keep bits of key tile t of score row `row` in the attention kernels' format (bit k =
// key 32 t + k of a row of nk keys): four Philox groups.
__device__ __forceinline__ uint32_t attention_keep_word(const PhiloxKey& key, uint64_t row, uint32_t nk, uint32_t t) {
    const uint64_t g0 = row * (nk / 8) + 4 * t;
    return keep8(philox_group_dev(key, g0), key.thr) | (keep8(philox_group_dev(key, g0 + 1), key.thr) << 8) |
           (keep8(philox_group_dev(key, g0 + 2), key.thr) << 16) | (keep8(philox_group_dev(key, g0 + 3), key.thr) << 24);
}

// The ReLU-dropout epilogue of the eight-wave 256x256 contraction kernel walks its tile so that lane
// `lane` of wave `wave` (of 8: 2 rows x 4 columns of waves) stores 16 packs of 8 outputs, pack c at
//   row = 256 tile_m + 128 (wave / 4) + 8 c + lane / 8,   column = 256 tile_n + 64 (wave % 4) + 8 (lane % 8)
// of the dense [M][N] output.  Its keep bits are 128 bits per lane, pack c in byte 15 - c: four words,
// word j = bytes of packs 15 - 4 j (lowest byte) .. 12 - 4 j.  This draws them for one lane.
struct KeepWords { uint32_t w[4]; };
__device__ __forceinline__ KeepWords relu_dropout_keep_words(const PhiloxKey& key, uint32_t N, uint32_t tile_m,
                                                             uint32_t tile_n, uint32_t wave, uint32_t lane) {
    const uint64_t row0 = (uint64_t)tile_m * 256 + (wave >> 2) * 128 + (lane >> 3);
    const uint64_t g0 = (row0 * N + (uint64_t)tile_n * 256 + (wave & 3) * 64 + (lane & 7) * 8) >> 3;
    KeepWords k;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t w = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int c = 15 - 4 * j - b;
            w |= keep8(philox_group_dev(key, g0 + (uint64_t)c * N), key.thr) << (8 * b);
        }
        k.w[j] = w;
    }
    return k;
}

// d(LN input) of one element: g * istd - c1 - diff * c2, with the contraction
// into FMAs spelled out so that every kernel that evaluates it rounds alike.
__device__ __forceinline__ float ln_bwd_value(float g, float diff, float istd, float c1, float c2) {
    return __fmaf_rn(-diff, c2, __fmaf_rn(g, istd, -c1));
}

// ---- wave64 reductions ------------------------------------------------------
// Two quad permutes, two row mirrors (DPP), then the four row totals are read
// with v_readlane and combined; the result is uniform across the wave.
template <int CTRL>
__device__ __forceinline__ float dpp(float x) {
    int i = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true);
    return __int_as_float(i);
}

__device__ __forceinline__ float wave_sum(float x) {
    x += dpp<0xB1>(x);    // quad_perm [1,0,3,2]
    x += dpp<0x4E>(x);    // quad_perm [2,3,0,1]
    x += dpp<0x141>(x);   // row_half_mirror
    x += dpp<0x140>(x);   // row_mirror
    int xi = __float_as_int(x);
    float a = __int_as_float(__builtin_amdgcn_readlane(xi, 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(xi, 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(xi, 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(xi, 48));
    return (a + b) + (c + d);
}

__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp<0xB1>(x));
    x = fmaxf(x, dpp<0x4E>(x));
    x = fmaxf(x, dpp<0x141>(x));
    x = fmaxf(x, dpp<0x140>(x));
    int xi = __float_as_int(x);
    float a = __int_as_float(__builtin_amdgcn_readlane(xi, 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(xi, 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(xi, 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(xi, 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Reductions over aligned groups of GRP lanes (64, 32 or 16): short rows sit
// side by side in one wave.  Every lane of a group ends up with the group's
// value (the four DPP steps above already total each 16-lane row).
template <int GRP>
__device__ __forceinline__ float group_sum(float x) {
    if (GRP == 64) return wave_sum(x);
    x += dpp<0xB1>(x);
    x += dpp<0x4E>(x);
    x += dpp<0x141>(x);
    x += dpp<0x140>(x);
    if (GRP == 32) x += __shfl_xor(x, 16);
    return x;
}
template <int GRP>
__device__ __forceinline__ float group_max(float x) {
    if (GRP == 64) return wave_max(x);
    x = fmaxf(x, dpp<0xB1>(x));
    x = fmaxf(x, dpp<0x4E>(x));
    x = fmaxf(x, dpp<0x141>(x));
    x = fmaxf(x, dpp<0x140>(x));
    if (GRP == 32) x = fmaxf(x, __shfl_xor(x, 16));
    return x;
}

// Makes a rounded fp16 pack opaque to the optimiser, so that a second output
// derived from it (value * {0,1} mask) is bit-identical to it rather than
// recomputed through a differently rounded (fused) conversion.
__device__ __forceinline__ h8 pin(h8 v) {
    typedef int i4 __attribute__((ext_vector_type(4)));
    i4 t = __builtin_bit_cast(i4, v);
    asm volatile("" : "+v"(t));
    return __builtin_bit_cast(h8, t);
}

// {0,1} mask pack from keep bits
__device__ __forceinline__ h8 mask_h8(uint32_t bits) {
    h8 m;
#pragma unroll
    for (int i = 0; i < 8; ++i) m[i] = ((bits >> i) & 1u) ? (half_t)1.0f : (half_t)0.0f;
    return m;
}

// tanh-form GELU (substation/transformer.py:11-28) written through the logistic function:
// 0.5 x (1 + tanh(u)) = x s(2u) with u = sqrt(2/pi) (x + 0.044715 x^3), s(z) = e^z / (1 + e^z), and
// its derivative s + x s (1 - s) d(2u)/dx.  One v_exp_f32 and one v_rcp_f32 per value.  The order
// of the operations is fixed (no contraction left to the compiler), so that the operator kernels
// and the epilogues of the contractions give the same bits.
struct GeluTerms {
    float s, r;                   // s(2u) and 1 - s(2u)
};

__device__ __forceinline__ GeluTerms gelu_terms(float x, float x2) {
#pragma clang fp contract(off)
    const float k0 = 2.302208198144325f;             // 2 sqrt(2/pi) log2(e)
    const float k1 = 0.1029432395800235f;           // k0 * 0.044715
    float w = x * __builtin_fmaf(x2, k1, k0);        // 2u log2(e)
    w = fminf(w, 64.0f);                             // e^z stays finite: s = 1 from there on anyway
    const float e = __builtin_amdgcn_exp2f(w);
    GeluTerms t;
    t.r = __builtin_amdgcn_rcpf(1.0f + e);
    t.s = e * t.r;
    return t;
}

// (The results pass through a register as fp32: a conversion to fp16 that follows rounds that value,
// whereas fused with the last multiplication into one instruction it would round the exact product.)
__device__ __forceinline__ float gelu_fwd(float x) {
#pragma clang fp contract(off)
    float g = x * gelu_terms(x, x * x).s;
    asm volatile("" : "+v"(g));
    return g;
}

// gelu'(x) * d
__device__ __forceinline__ float gelu_bwd(float x, float d) {
#pragma clang fp contract(off)
    const float x2 = x * x;
    const GeluTerms t = gelu_terms(x, x2);
    const float zp = __builtin_fmaf(x2, 0.21406444881780073f, 1.5957691216057308f);   // d(2u)/dx
    const float q = (x * zp) * t.r;
    float g = __builtin_fmaf(t.s, q, t.s) * d;
    asm volatile("" : "+v"(g));
    return g;
}

}  // namespace sub
