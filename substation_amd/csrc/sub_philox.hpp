// Counter-based dropout masks: Philox4x32-10 (Salmon et al., SC'11), usable from
// host and device code.  Replaces the per-thread cuRAND state of
// pytorch_module/blocks.cuh:24-51 with a stateless map from the canonical
// element index to 16 random bits, so masks do not depend on layout or launch
// geometry:
//   counter = (lo32(e >> 3), hi32(e >> 3), site, step), key = (lo32(seed), hi32(seed))
//   field   = 16-bit field (e & 7) of the 128-bit output (little-endian per word)
//   keep    = field >= round(p * 65536)
#pragma once

#include <cstdint>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define SUB_HD __host__ __device__ __forceinline__
#else
#define SUB_HD inline
#endif

namespace sub {

struct PhiloxKey {
    uint32_t k0, k1;     // seed
    uint32_t site, step; // counter words 2 and 3
    uint32_t thr;        // drop threshold on a 16-bit field, 0..65536
    // Optional step counter in device memory, added to `step` when a kernel
    // starts: launches recorded in a HIP graph then draw new masks on every
    // replay (their arguments, `step` included, are frozen at capture).
    const uint32_t* step_dev = nullptr;
};

struct U4 { uint32_t x, y, z, w; };

SUB_HD void mulhilo(uint32_t a, uint32_t b, uint32_t& hi, uint32_t& lo) {
    uint64_t p = (uint64_t)a * (uint64_t)b;
    hi = (uint32_t)(p >> 32);
    lo = (uint32_t)p;
}

SUB_HD U4 philox4x32_10(U4 c, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        uint32_t hi0, lo0, hi1, lo1;
        mulhilo(0xD2511F53u, c.x, hi0, lo0);
        mulhilo(0xCD9E8D57u, c.z, hi1, lo1);
        U4 n;
        n.x = hi1 ^ c.y ^ k0;
        n.y = lo1;
        n.z = hi0 ^ c.w ^ k1;
        n.w = lo0;
        c = n;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c;
}

// 128 random bits for the group of 8 canonical elements 8g .. 8g+7.
SUB_HD U4 philox_group(const PhiloxKey& k, uint64_t g) {
    U4 c;
    c.x = (uint32_t)g; c.y = (uint32_t)(g >> 32); c.z = k.site; c.w = k.step;
    return philox4x32_10(c, k.k0, k.k1);
}

SUB_HD uint32_t field16(const U4& r, int i) {
    uint32_t w = (i >> 1) == 0 ? r.x : (i >> 1) == 1 ? r.y : (i >> 1) == 2 ? r.z : r.w;
    return (i & 1) ? (w >> 16) : (w & 0xFFFFu);
}

// Keep bits of the 8 elements of one Philox group: bit i set = 16-bit field i >= thr.
// On the device both fields of a word are compared at once: thr - field, saturating at 0,
// is non-zero exactly where the element is dropped (v_pk_sub_u16 clamp, v_pk_min_u16
// against 1: the word's two drop bits at positions 0 and 16); the four words are shifted
// together and the upper fields' bits folded down beside the lower ones'.  About 15
// instructions where a compare and a select per field take 30.
SUB_HD uint32_t keep8(const U4& r, uint32_t thr) {
#if defined(__HIP_DEVICE_COMPILE__)
    // (spelled as instructions: written as min(sub_sat(thr, field), 1) the compiler turns the
    // pair back into a compare and a select per field)
    const uint32_t thr2 = (thr & 0xffffu) * 0x10001u, one2 = 0x10001u;
    auto drop2 = [&](uint32_t w) {
        uint32_t d;
        asm("v_pk_sub_u16 %0, %1, %2 clamp\n\tv_pk_min_u16 %0, %0, %3" : "=&v"(d) : "v"(thr2), "v"(w), "v"(one2));
        return d;
    };
    const uint32_t d = drop2(r.x) | (drop2(r.y) << 2) | (drop2(r.z) << 4) | (drop2(r.w) << 6);
    const uint32_t all = 0u - (thr >> 16);                         // thr = 2^16: every element dropped
    return ~(d | (d >> 15) | all) & 0xffu;
#else
    uint32_t b = 0;
    for (int i = 0; i < 8; ++i) b |= (field16(r, i) >= thr ? 1u : 0u) << i;
    return b;
#endif
}

// Keep-bits (bit i set = element e0+i kept) for 8 consecutive canonical elements
// starting at e0.  One Philox call when e0 is a multiple of 8, two otherwise.
SUB_HD uint32_t keep_bits8(const PhiloxKey& k, uint64_t e0) {
    uint64_t g = e0 >> 3;
    int off = (int)(e0 & 7);
    U4 r0 = philox_group(k, g);
    uint32_t bits = 0;
    if (off == 0) {
        bits = keep8(r0, k.thr);
    } else {
        U4 r1 = philox_group(k, g + 1);
        for (int i = 0; i < 8; ++i) {
            int f = off + i;
            uint32_t v = f < 8 ? field16(r0, f) : field16(r1, f - 8);
            bits |= (v >= k.thr ? 1u : 0u) << i;
        }
    }
    return bits;
}

inline uint32_t threshold16(float p) {
    double t = (double)p * 65536.0 + 0.5;
    if (t < 0) t = 0;
    if (t > 65536.0) t = 65536.0;
    return (uint32_t)t;
}

}  // namespace sub
