// Self-attention without score-sized tensors in memory.
//
// The reference keeps five tensors of the size of the score matrix per layer
// (pytorch_module/encoder.cu:104-131 forward: BETA, ALPHA, ATTN_DROP_MASK,
// ATTN_DROP; :222-262 backward: DATTN_DROP, DBETA) and moves each of them
// through memory two or three times.  Here a tile of 32 x 32 scores lives only in
// the accumulator registers of one wave:
//
//   forward     per 32 queries, over all keys: S = a.Q.K^T, running softmax
//               (max and sum per query), dropout, O += P_drop.V; writes O, the
//               log-sum-exp of each score row and one keep bit per score
//   backward dQ per 32 queries, over all keys: recomputes P from the log-sum-exp,
//               dP = dO.V^T, dS = P (keep.dP - D), dQ += dS.K with D = rowsum(dO o O)
//   backward dK, dV  per 32 keys, over all queries: the same dS and P_drop,
//               dK += dS^T.Q, dV += P_drop^T.dO
//
// Scores are formed as D[key, query] (dQ, forward) so that everything that is
// per query -- running max, sum, log-sum-exp, D, the keep word -- is per lane,
// and as D[query, key] in the dK/dV kernel.  Either way the score tile is, as it
// lies in the accumulator registers, the B operand of the next product with the
// contraction index running over the registers in the order
//   element i of step s  <->  index (2s + i/4)*8 + 4*(lane/32) + i%4 ;
// the A operand is gathered in the same order from an LDS tile with the
// transposing read, so no score ever moves between lanes.
#include "sub_ops.hpp"

namespace sub {

namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef short s4v __attribute__((ext_vector_type(4)));
typedef short s8v __attribute__((ext_vector_type(8)));
constexpr float LOG2E = 1.4426950408889634f;
constexpr int QB = 128;           // positions per workgroup: 4 waves x 32

template <int P>
struct Geo {
    static constexpr int NKS = P / 16;             // k-steps of a contraction over the features
    static constexpr int NPT = P / 32;             // 32-wide tiles of the feature dim
    static constexpr int PITCH = P + 8;            // halves per row of an LDS tile
    static constexpr int TILE = 32 * PITCH;        // 32 positions
    static constexpr int VL = (32 * (P / 8)) / 256; // 16-byte words per thread and tile
};

// Fragment of 32 rows (one per lane%32) with the features as contraction index:
// A or B operand of v_mfma_f32_32x32x16_f16, straight from global memory.
template <int P>
__device__ __forceinline__ void row_frags(const AttnSide& t, unsigned h, unsigned b, unsigned pos, int hi,
                                          h8 (&f)[P / 16]) {
    const half_t* p = t.p + (long)h * t.sh + (long)b * t.sb + (long)pos * t.sr + hi * 8;
#pragma unroll
    for (int ks = 0; ks < P / 16; ++ks) f[ks] = *reinterpret_cast<const h8*>(p + ks * 16);
}

// The same fragment from an LDS tile [32 positions][P].
template <int P>
__device__ __forceinline__ void row_frags_lds(const half_t* tile, int l32, int hi, h8 (&f)[P / 16]) {
#pragma unroll
    for (int ks = 0; ks < P / 16; ++ks)
        f[ks] = *reinterpret_cast<const h8*>(tile + l32 * Geo<P>::PITCH + hi * 8 + ks * 16);
}

// A tile of 32 positions x P features: global -> registers -> LDS, all threads.
template <int P>
__device__ __forceinline__ void tile_fetch(const AttnSide& t, unsigned h, unsigned b, unsigned pos0, int tid,
                                           h8 (&r)[Geo<P>::VL]) {
#pragma unroll
    for (int i = 0; i < Geo<P>::VL; ++i) {
        const int id = tid + i * 256, row = id / (P / 8), c = id % (P / 8);
        r[i] = *reinterpret_cast<const h8*>(t.p + (long)h * t.sh + (long)b * t.sb + (long)(pos0 + row) * t.sr +
                                            c * 8);
    }
}
template <int P>
__device__ __forceinline__ void tile_put(half_t* tile, int tid, const h8 (&r)[Geo<P>::VL]) {
#pragma unroll
    for (int i = 0; i < Geo<P>::VL; ++i) {
        const int id = tid + i * 256, row = id / (P / 8), c = id % (P / 8);
        *reinterpret_cast<h8*>(tile + row * Geo<P>::PITCH + c * 8) = r[i];
    }
}

// A operand with the tile's positions as contraction index: lane%32 = feature
// m0 + lane%32, elements = positions in the register order of a score tile.
// ds_read_b64_tr_b16: within 16 lanes, lane i receives T[k0 + 0..3][m0 + i] when
// lane l addresses T[k0 + l/4][m0 + 4*(l%4)].
__device__ __forceinline__ h8 tr_frag(const half_t* tile, int pitch, int m0, int s, int lane) {
    const int g = lane >> 4, l = lane & 15;
    const int k = 16 * s + 4 * (g >> 1) + (l >> 2);
    const int m = m0 + 16 * (g & 1) + 4 * (l & 3);
    const half_t* p = tile + k * pitch + m;
    typedef s4v __attribute__((address_space(3))) * lds_s4;
    s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(p));
    s4v up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(p + 8 * pitch));
    s8v r = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(h8, r);
}

// Position (within a tile of 32) that accumulator register v of a lane holds.
__device__ __forceinline__ constexpr int reg_pos(int v, int hi) { return (v >> 2) * 8 + hi * 4 + (v & 3); }

// Output rows: D[feature, position] accumulators -> t[position][feature], 8-byte pieces.
template <int P>
__device__ __forceinline__ void store_rows(const AttnSide& t, unsigned h, unsigned b, unsigned pos, int hi,
                                           const f16v (&acc)[P / 32], float scale) {
    half_t* p = const_cast<half_t*>(t.p) + (long)h * t.sh + (long)b * t.sb + (long)pos * t.sr + hi * 4;
#pragma unroll
    for (int pt = 0; pt < P / 32; ++pt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            h4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (half_t)(acc[pt][q * 4 + e] * scale);
            *reinterpret_cast<h4*>(p + pt * 32 + q * 8) = w;
        }
}

__device__ __forceinline__ uint32_t keep8(const U4& r, uint32_t thr) {
    uint32_t b = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) b |= (field16(r, i) >= thr ? 1u : 0u) << i;
    return b;
}

// ---------------------------------------------------------------------------
// forward.  grid = H * B * (J / 128); wave = 32 queries.
// ---------------------------------------------------------------------------
template <int P>
__global__ __launch_bounds__(256) void k_mha_fwd(AttnArgs a, PhiloxKey key_) {
    using G = Geo<P>;
    __shared__ __attribute__((aligned(16))) half_t vt[2][G::TILE];
    const PhiloxKey key = resolved(key_);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    const unsigned qblocks = a.J / QB;
    const unsigned qb = blockIdx.x % qblocks, hb = blockIdx.x / qblocks;
    const unsigned b = hb % a.B, h = hb / a.B;
    const unsigned j = qb * QB + wave * 32 + l32;                    // this lane's query
    const unsigned row = (h * a.B + b) * a.J + j;                    // its score row
    const unsigned nt = a.K / 32;
    const float c = a.alpha * LOG2E;

    h8 fq[G::NKS], fk[G::NKS], vr[G::VL];
    row_frags<P>(a.q, h, b, j, hi, fq);
    row_frags<P>(a.k, h, b, l32, hi, fk);
    tile_fetch<P>(a.v, h, b, 0, tid, vr);
    tile_put<P>(vt[0], tid, vr);
    __syncthreads();

    f16v o[G::NPT];
#pragma unroll
    for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[pt][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;                            // l_run: this lane's keys only

    for (unsigned t = 0; t < nt; ++t) {
        h8 fkn[G::NKS];
        const bool more = t + 1 < nt;
        if (more) {
            row_frags<P>(a.k, h, b, (t + 1) * 32 + l32, hi, fkn);
            tile_fetch<P>(a.v, h, b, (t + 1) * 32, tid, vr);
        }
        f16v s;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk[ks], fq[ks], s, 0, 0, 0);

        // keep bits of the 32 scores (this query, keys of tile t): each half of the
        // wave draws two of the four groups of 8 and the halves trade them
        uint32_t word = 0xffffffffu;
        if (key.thr) {
            const uint64_t g0 = (uint64_t)row * (a.K / 8) + 4 * t + 2 * hi;
            const uint32_t mine = keep8(philox_group(key, g0), key.thr) |
                                  (keep8(philox_group(key, g0 + 1), key.thr) << 8);
            const uint32_t other = (uint32_t)__shfl_xor((int)mine, 32);
            word = hi ? (other | (mine << 16)) : (mine | (other << 16));
        }
        if (hi == 0) a.keep[(size_t)row * nt + t] = word;
        const uint32_t nib = word >> (hi * 4);                       // bit reg_pos(v, 0) of nib = keep of register v

        float mt = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] *= c; mt = fmaxf(mt, s[v]); }
        mt = fmaxf(mt, __shfl_xor(mt, 32));
        const float m_new = fmaxf(m_run, mt);
        const float corr = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        l_run *= corr;
#pragma unroll
        for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
            for (int v = 0; v < 16; ++v) o[pt][v] *= corr;
        h8 pb[2];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float p = __builtin_amdgcn_exp2f(s[v] - m_new);
            l_run += p;
            pb[v >> 3][v & 7] = ((nib >> reg_pos(v, 0)) & 1u) ? (half_t)p : (half_t)0.0f;
        }
        const half_t* vtile = vt[t & 1];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt)
                o[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(tr_frag(vtile, G::PITCH, pt * 32, st, lane), pb[st],
                                                               o[pt], 0, 0, 0);
        if (more) {
            tile_put<P>(vt[(t + 1) & 1], tid, vr);
#pragma unroll
            for (int ks = 0; ks < G::NKS; ++ks) fk[ks] = fkn[ks];
        }
        __syncthreads();
    }
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    store_rows<P>(a.o, h, b, j, hi, o, 1.0f / l_tot);
    if (hi == 0) a.lse[row] = m_run + __builtin_amdgcn_logf(l_tot);
}

// ---------------------------------------------------------------------------
// backward, dQ.  grid = H * B * (J / 128); wave = 32 queries.
// ---------------------------------------------------------------------------
template <int P>
__global__ __launch_bounds__(256) void k_mha_bwd_dq(AttnArgs a) {
    using G = Geo<P>;
    __shared__ __attribute__((aligned(16))) half_t kt[2][G::TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    const unsigned qblocks = a.J / QB;
    const unsigned qb = blockIdx.x % qblocks, hb = blockIdx.x / qblocks;
    const unsigned b = hb % a.B, h = hb / a.B;
    const unsigned j = qb * QB + wave * 32 + l32;
    const unsigned row = (h * a.B + b) * a.J + j;
    const unsigned nt = a.K / 32;
    const float c = a.alpha * LOG2E;

    h8 fq[G::NKS], fdo[G::NKS], fv[G::NKS], kr[G::VL];
    row_frags<P>(a.q, h, b, j, hi, fq);
    row_frags<P>(a.d_o, h, b, j, hi, fdo);
    float dsum;
    {
        h8 fo[G::NKS];
        row_frags<P>(a.o, h, b, j, hi, fo);
        float part = 0.f;
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks)
#pragma unroll
            for (int i = 0; i < 8; ++i) part += (float)fdo[ks][i] * (float)fo[ks][i];
        dsum = part + __shfl_xor(part, 32);
        if (hi == 0) a.dsum[row] = dsum;
    }
    const float lse = a.lse[row];
    row_frags<P>(a.v, h, b, l32, hi, fv);
    tile_fetch<P>(a.k, h, b, 0, tid, kr);
    tile_put<P>(kt[0], tid, kr);
    uint32_t word = a.keep[(size_t)row * nt];
    __syncthreads();

    f16v dq[G::NPT];
#pragma unroll
    for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) dq[pt][v] = 0.f;

    for (unsigned t = 0; t < nt; ++t) {
        h8 fvn[G::NKS];
        uint32_t wordn = 0;
        const bool more = t + 1 < nt;
        if (more) {
            row_frags<P>(a.v, h, b, (t + 1) * 32 + l32, hi, fvn);
            tile_fetch<P>(a.k, h, b, (t + 1) * 32, tid, kr);
            wordn = a.keep[(size_t)row * nt + t + 1];
        }
        const half_t* ktile = kt[t & 1];
        h8 fk[G::NKS];
        row_frags_lds<P>(ktile, l32, hi, fk);
        f16v s, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk[ks], fq[ks], s, 0, 0, 0);
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) dp = __builtin_amdgcn_mfma_f32_32x32x16_f16(fv[ks], fdo[ks], dp, 0, 0, 0);
        const uint32_t nib = word >> (hi * 4);
        h8 ds[2];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float p = __builtin_amdgcn_exp2f(fmaf(s[v], c, -lse));
            const float g = ((nib >> reg_pos(v, 0)) & 1u) ? dp[v] : 0.f;
            ds[v >> 3][v & 7] = (half_t)(p * (g - dsum));
        }
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt)
                dq[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(tr_frag(ktile, G::PITCH, pt * 32, st, lane), ds[st],
                                                                dq[pt], 0, 0, 0);
        if (more) {
            tile_put<P>(kt[(t + 1) & 1], tid, kr);
#pragma unroll
            for (int ks = 0; ks < G::NKS; ++ks) fv[ks] = fvn[ks];
            word = wordn;
        }
        __syncthreads();
    }
    store_rows<P>(a.dq, h, b, j, hi, dq, a.alpha);
}

// ---------------------------------------------------------------------------
// backward, dK and dV.  grid = H * B * (K / 128); wave = 32 keys.
// Per tile of 32 queries the workgroup stages Q, dO, the two row statistics and
// the keep words of its four key tiles in LDS.
// ---------------------------------------------------------------------------
template <int P>
struct KvStage {
    half_t q[Geo<P>::TILE];
    half_t d_o[Geo<P>::TILE];
    float lse[32];
    float dsum[32];
    uint32_t keep[4][32];         // [wave's key tile][query]
};

template <int P>
__global__ __launch_bounds__(256) void k_mha_bwd_dkv(AttnArgs a) {
    using G = Geo<P>;
    __shared__ __attribute__((aligned(16))) KvStage<P> stage[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    const unsigned kblocks = a.K / QB;
    const unsigned kb = blockIdx.x % kblocks, hb = blockIdx.x / kblocks;
    const unsigned b = hb % a.B, h = hb / a.B;
    const unsigned kpos = kb * QB + wave * 32 + l32;                 // this lane's key
    const unsigned row0 = (h * a.B + b) * a.J;                       // score row of query 0
    const unsigned nq = a.J / 32, nkt = a.K / 32;
    const float c = a.alpha * LOG2E;

    h8 fk[G::NKS], fv[G::NKS], qr[G::VL], dr[G::VL];
    float stat = 0.f;
    uint4 kw = make_uint4(0, 0, 0, 0);
    row_frags<P>(a.k, h, b, kpos, hi, fk);
    row_frags<P>(a.v, h, b, kpos, hi, fv);

    auto fetch = [&](unsigned qt) {
        tile_fetch<P>(a.q, h, b, qt * 32, tid, qr);
        tile_fetch<P>(a.d_o, h, b, qt * 32, tid, dr);
        const unsigned r = row0 + qt * 32 + (tid & 31);
        if (tid < 32) stat = a.lse[r];
        else if (tid < 64) stat = a.dsum[r];
        else if (tid < 96) kw = *reinterpret_cast<const uint4*>(a.keep + (size_t)r * nkt + kb * 4);
    };
    auto put = [&](KvStage<P>& s) {
        tile_put<P>(s.q, tid, qr);
        tile_put<P>(s.d_o, tid, dr);
        if (tid < 32) s.lse[tid] = stat;
        else if (tid < 64) s.dsum[tid - 32] = stat;
        else if (tid < 96) {
            s.keep[0][tid - 64] = kw.x; s.keep[1][tid - 64] = kw.y;
            s.keep[2][tid - 64] = kw.z; s.keep[3][tid - 64] = kw.w;
        }
    };
    fetch(0);
    put(stage[0]);
    __syncthreads();

    f16v dk[G::NPT], dv[G::NPT];
#pragma unroll
    for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) { dk[pt][v] = 0.f; dv[pt][v] = 0.f; }

    for (unsigned qt = 0; qt < nq; ++qt) {
        const bool more = qt + 1 < nq;
        if (more) fetch(qt + 1);
        const KvStage<P>& sg = stage[qt & 1];
        h8 fq[G::NKS], fdo[G::NKS];
        row_frags_lds<P>(sg.q, l32, hi, fq);
        row_frags_lds<P>(sg.d_o, l32, hi, fdo);
        f16v s, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(fq[ks], fk[ks], s, 0, 0, 0);
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) dp = __builtin_amdgcn_mfma_f32_32x32x16_f16(fdo[ks], fv[ks], dp, 0, 0, 0);
        // D[query, key]: lane = key, register v = query reg_pos(v, hi)
        h8 pd[2], ds[2];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 ls = *reinterpret_cast<const float4*>(sg.lse + q * 8 + hi * 4);
            const float4 dd = *reinterpret_cast<const float4*>(sg.dsum + q * 8 + hi * 4);
            const uint4 w = *reinterpret_cast<const uint4*>(sg.keep[wave] + q * 8 + hi * 4);
            const float lsv[4] = {ls.x, ls.y, ls.z, ls.w}, ddv[4] = {dd.x, dd.y, dd.z, dd.w};
            const uint32_t wv[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int v = q * 4 + e;
                const float p = __builtin_amdgcn_exp2f(fmaf(s[v], c, -lsv[e]));
                const bool keep = (wv[e] >> l32) & 1u;
                pd[v >> 3][v & 7] = keep ? (half_t)p : (half_t)0.0f;
                ds[v >> 3][v & 7] = (half_t)(p * ((keep ? dp[v] : 0.f) - ddv[e]));
            }
        }
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt) {
                dv[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(tr_frag(sg.d_o, G::PITCH, pt * 32, st, lane), pd[st],
                                                                dv[pt], 0, 0, 0);
                dk[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(tr_frag(sg.q, G::PITCH, pt * 32, st, lane), ds[st],
                                                                dk[pt], 0, 0, 0);
            }
        if (more) put(stage[(qt + 1) & 1]);
        __syncthreads();
    }
    store_rows<P>(a.dk, h, b, kpos, hi, dk, a.alpha);
    store_rows<P>(a.dv, h, b, kpos, hi, dv, 1.0f);
}

bool side_ok(const AttnSide& s) {
    return s.p && (reinterpret_cast<uintptr_t>(s.p) & 15) == 0 && s.sh % 8 == 0 && s.sb % 8 == 0 && s.sr % 8 == 0;
}

}  // namespace

bool mha_shape_ok(long H, long B, long J, long K, long P) {
    if (P != 64 && P != 128) return false;
    if (J <= 0 || K <= 0 || J % QB != 0 || K % QB != 0) return false;
    if (H * B * J > 0x7fffffffL || H * B * (J / QB) > 0x7fffffffL || H * B * (K / QB) > 0x7fffffffL) return false;
    return true;
}

size_t mha_stat_bytes(long H, long B, long J) { return (size_t)(H * B * J) * 2 * sizeof(float); }
size_t mha_keep_bytes(long H, long B, long J, long K) { return (size_t)(H * B * J) * (size_t)(K / 32) * 4; }

bool mha_forward_ok(const AttnArgs& a, int P) {
    return mha_shape_ok(a.H, a.B, a.J, a.K, P) && side_ok(a.q) && side_ok(a.k) && side_ok(a.v) && side_ok(a.o) &&
           a.lse && a.keep && (reinterpret_cast<uintptr_t>(a.lse) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(a.keep) & 15) == 0;
}

void launch_mha_forward(const AttnArgs& a, int P, PhiloxKey key, hipStream_t st) {
    if (!mha_forward_ok(a, P)) fail("attention forward: shape, strides or alignment not supported");
    dim3 grid((unsigned)(a.H * a.B * (a.J / QB)));
    if (P == 64) hipLaunchKernelGGL(k_mha_fwd<64>, grid, dim3(256), 0, st, a, key);
    else hipLaunchKernelGGL(k_mha_fwd<128>, grid, dim3(256), 0, st, a, key);
    check_launch("attention forward");
}

bool mha_backward_ok(const AttnArgs& a, int P) {
    return mha_forward_ok(a, P) && a.dsum && side_ok(a.d_o) && side_ok(a.dq) && side_ok(a.dk) && side_ok(a.dv);
}

void launch_mha_backward_dq(const AttnArgs& a, int P, hipStream_t st) {
    if (!mha_backward_ok(a, P)) fail("attention backward: shape, strides or alignment not supported");
    dim3 grid((unsigned)(a.H * a.B * (a.J / QB)));
    if (P == 64) hipLaunchKernelGGL(k_mha_bwd_dq<64>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(k_mha_bwd_dq<128>, grid, dim3(256), 0, st, a);
    check_launch("attention backward (dQ)");
}

void launch_mha_backward_dkv(const AttnArgs& a, int P, hipStream_t st) {
    if (!mha_backward_ok(a, P)) fail("attention backward: shape, strides or alignment not supported");
    dim3 grid((unsigned)(a.H * a.B * (a.K / QB)));
    if (P == 64) hipLaunchKernelGGL(k_mha_bwd_dkv<64>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(k_mha_bwd_dkv<128>, grid, dim3(256), 0, st, a);
    check_launch("attention backward (dK, dV)");
}

}  // namespace sub
