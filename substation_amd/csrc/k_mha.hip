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
constexpr float RESCALE_SLACK = 8.f;   // unnormalised probabilities stay below 2^8

template <int P>
struct Geo {
    static constexpr int NKS = P / 16;             // k-steps of a contraction over the features
    static constexpr int NPT = P / 32;             // 32-wide tiles of the feature dim
    static constexpr int TILE = 32 * P;            // halves of an LDS tile of 32 positions
    static constexpr int VL = (32 * (P / 8)) / 256; // 16-byte words per thread and tile

    // LDS tiles are [position][feature] without padding; the index of a 16-byte
    // chunk within its row is xor-ed with a function of the row chosen so that both
    // ways of reading a tile are free of bank conflicts: 16 consecutive rows at one
    // chunk (the features as contraction index, ds_read_b128) and 4 consecutive
    // rows x 4 adjacent chunks (the positions as contraction index, transposing read).
    static __device__ __forceinline__ int swz(int row) {
        return P == 64 ? ((((row >> 1) & 1) << 2) | ((row >> 2) & 3)) : (((row & 3) << 2) | ((row >> 2) & 3));
    }
    // offset in halves of chunk c of a row
    static __device__ __forceinline__ int at(int row, int c) { return row * P + ((c ^ swz(row)) << 3); }
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

// The same fragment from an LDS tile.
template <int P>
__device__ __forceinline__ void row_frags_lds(const half_t* tile, int l32, int hi, h8 (&f)[P / 16]) {
#pragma unroll
    for (int ks = 0; ks < P / 16; ++ks)
        f[ks] = *reinterpret_cast<const h8*>(tile + Geo<P>::at(l32, 2 * ks + hi));
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
        *reinterpret_cast<h8*>(tile + Geo<P>::at(row, c)) = r[i];
    }
}

// A operand with the tile's positions as contraction index: lane%32 = feature
// m0 + lane%32, elements = positions in the register order of a score tile.
// ds_read_b64_tr_b16: within 16 lanes, lane i receives T[k0 + 0..3][m0 + i] when
// lane l addresses T[k0 + l/4][m0 + 4*(l%4)].
template <int P>
__device__ __forceinline__ h8 tr_frag(const half_t* tile, int m0, int s, int lane) {
    const int g = lane >> 4, l = lane & 15;
    const int k = 16 * s + 4 * (g >> 1) + (l >> 2);
    const int m = m0 + 16 * (g & 1) + 4 * (l & 3);
    typedef s4v __attribute__((address_space(3))) * lds_s4;
    s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(tile + Geo<P>::at(k, m >> 3) + (m & 7)));
    s4v up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(tile + Geo<P>::at(k + 8, m >> 3) + (m & 7)));
    s8v r = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(h8, r);
}

// Workgroups are dealt to the 8 XCDs (each with its own L2) in turn.  Renumbered
// so that consecutive logical blocks -- the blocks of one head and sample, which
// read the same K, V (or Q, dO) -- run on one XCD and share its L2.
__device__ __forceinline__ unsigned logical_block() {
    const unsigned n = gridDim.x, bid = blockIdx.x;
    return (n % 8u) ? bid : (bid % 8u) * (n / 8u) + bid / 8u;
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

// x where bit `pos` of `bits` is set, else +0.0
__device__ __forceinline__ float keep_if(float x, uint32_t bits, int pos) {
    return __int_as_float(__float_as_int(x) & __builtin_amdgcn_sbfe((int)bits, pos, 1));
}

// Sums over the 128 positions of a workgroup of the rows store_rows() writes
// (same rounding), one value per feature: 32 lanes hold the positions of a
// wave, the four waves meet in LDS (`red`: 4 * P floats, free to use).
template <int P>
__device__ __forceinline__ void column_sums(const f16v (&acc)[P / 32], float scale, float* red, float* out,
                                            int tid) {
    const int lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    // Five DPP steps per value and no trip through LDS: four total each row of 16 lanes, the fifth
    // (row_bcast15 into rows 1 and 3) adds the row below, so that lanes 16..31 (48..63) hold the total
    // of lanes 0..31 (32..63).  All values first and then the store: the chains are independent and
    // fill each other's wait states.  (With a ds_bpermute as the last step the 32 values of a lane went
    // through LDS one after the other, 2 to 3 us at the end of every workgroup.)
    float x[P / 32][16];
#pragma unroll
    for (int pt = 0; pt < P / 32; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float t = (float)(half_t)(acc[pt][v] * scale);
            t += dpp<0xB1>(t);
            t += dpp<0x4E>(t);
            t += dpp<0x141>(t);
            t += dpp<0x140>(t);
            t += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(t), 0x142, 0xA, 0xF, false));
            x[pt][v] = t;
        }
    if (l32 == 16) {
#pragma unroll
        for (int pt = 0; pt < P / 32; ++pt)
#pragma unroll
            for (int v = 0; v < 16; ++v) red[wave * P + pt * 32 + reg_pos(v, hi)] = x[pt][v];
    }
    __syncthreads();
    if (tid < P) out[tid] = (red[tid] + red[P + tid]) + (red[2 * P + tid] + red[3 * P + tid]);
}

// Additive attention mask (substation/attention.py:65-68: added to the raw scores,
// before the scaling) for the 16 scores of a lane.  QUERY_LANES: the lane holds
// one query and registers run over keys (forward, dQ); otherwise the lane holds
// one key and registers run over queries (dK/dV).  The values of a tile are loaded
// while the tile before it is worked on, ahead of that pass's K/V (Q/dO) loads:
// loads complete in order, so a wait for mask values issued after those would
// also wait for them.
struct MaskRegs { h4 q[4]; };

template <bool QUERY_LANES>
__device__ __forceinline__ void load_mask(const AttnArgs& a, unsigned lane_pos, unsigned tile0, int hi, MaskRegs& mk) {
    const long lane_stride = QUERY_LANES ? a.am_sj : a.am_sk, reg_stride = QUERY_LANES ? a.am_sk : a.am_sj;
    const half_t* m = a.amask + (long)lane_pos * lane_stride + (long)tile0 * reg_stride;
    if (reg_stride == 1) {
#pragma unroll
        for (int q = 0; q < 4; ++q) mk.q[q] = *reinterpret_cast<const h4*>(m + q * 8 + hi * 4);
    } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) mk.q[v >> 2][v & 3] = m[(long)reg_pos(v, hi) * reg_stride];
    }
}

// The scores of a tile start from the mask's values instead of zero: the product
// accumulates on top of them.
__device__ __forceinline__ void start_from_mask(const MaskRegs& mk, f16v& s) {
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = (float)mk.q[v >> 2][v & 3];
}

// ---------------------------------------------------------------------------
// What a mask leaves to do.  Each 32x32 block of the mask is classed as mixed,
// dead (all -inf: the scores vanish) or clear (all zero: nothing to add).  Per
// workgroup of the attention kernels (128 queries, or 128 keys in the dK/dV
// kernel) a list names the tiles of the other side that are not dead for all
// four waves; the kernels walk that list instead of all tiles.
//   row of a list: [0] = number of entries, then the entries, then padding that
//   reads as "tile 0, dead for all waves" (the kernels read up to 3 past the end).
//   entry: bits 0..15 tile index, bits 16+2w.. the class of the block for wave w.
// ---------------------------------------------------------------------------
enum : uint32_t { BLOCK_MIXED = 0, BLOCK_DEAD = 1, BLOCK_CLEAR = 2 };
constexpr uint32_t kAllDead = BLOCK_DEAD * 0x55u << 16;
constexpr int kListPad = 4;       // the count and three entries of padding

// One wave per 32x32 block of the mask.
__global__ __launch_bounds__(64) void k_mha_mask_classes(const half_t* mask, long sj, long sk, int K, uint8_t* cls) {
    const int lane = threadIdx.x, nkb = K / 32;
    const int qb = blockIdx.x / nkb, kb = blockIdx.x % nkb;
    const half_t* p = mask + (long)(qb * 32 + (lane & 31)) * sj + (long)(kb * 32 + (lane >> 5) * 16) * sk;
    bool dead = true, clear = true;
    for (int i = 0; i < 16; ++i) {
        const float x = (float)p[(long)i * sk];
        dead = dead && (x == -INFINITY);
        clear = clear && (x == 0.f);
    }
    const bool all_dead = __builtin_amdgcn_ballot_w64(dead) == ~0ull;
    const bool all_clear = __builtin_amdgcn_ballot_w64(clear) == ~0ull;
    if (lane == 0) cls[blockIdx.x] = all_dead ? BLOCK_DEAD : all_clear ? BLOCK_CLEAR : BLOCK_MIXED;
}

// One wave per list row: blocks 0 .. J/128-1 build the key-tile lists of the query
// blocks, the others the query-tile lists of the key blocks.
__global__ __launch_bounds__(64) void k_mha_mask_lists(const uint8_t* cls, int J, int K, uint32_t* qlist, uint32_t* klist) {
    const int lane = threadIdx.x, nqb = J / 32, nkb = K / 32;
    const bool by_query = (int)blockIdx.x < J / QB;
    const int blk = by_query ? blockIdx.x : blockIdx.x - J / QB;
    const int ntiles = by_query ? nkb : nqb;
    uint32_t* row = (by_query ? qlist : klist) + (size_t)blk * (ntiles + kListPad);
    unsigned count = 0;
    for (int t0 = 0; t0 < ntiles; t0 += 64) {
        const int t = t0 + lane;
        uint32_t e = kAllDead;
        if (t < ntiles) {
            e = (uint32_t)t;
            for (int w = 0; w < 4; ++w) {
                const uint32_t c = by_query ? cls[(size_t)(blk * 4 + w) * nkb + t] : cls[(size_t)t * nkb + blk * 4 + w];
                e |= c << (16 + 2 * w);
            }
        }
        const bool live = (e & (0xffu << 16)) != kAllDead;
        const unsigned long long m = __builtin_amdgcn_ballot_w64(live);
        if (live) row[1 + count + __builtin_popcountll(m & ((1ull << lane) - 1))] = e;
        count += (unsigned)__builtin_popcountll(m);
    }
    if (lane == 0) row[0] = count;
    for (int i = count + lane; i < ntiles + kListPad - 1; i += 64) row[1 + i] = kAllDead;
}

// Which block of 128 (and which head and sample) a workgroup takes when a mask has
// left the blocks unequal amounts to do.  Workgroups start in the order of their
// index.  The blocks of a head and sample are ranked long to short (the reverse of
// their positions when the last has more to do than the first: a causal mask seen
// from the queries) and dealt in four passes over the heads and samples of an XCD,
// a quarter of the ranks per pass, so that the launch does not end on a few long
// blocks running alone.
__device__ __forceinline__ void masked_order(const uint32_t* list, unsigned nblocks, unsigned ntiles, unsigned ngroups,
                                             unsigned lb, unsigned& blk, unsigned& hb) {
    blk = lb % nblocks; hb = lb / nblocks;
    if (!list) return;
    const bool rev = list[(size_t)(nblocks - 1) * (ntiles + kListPad)] > list[0];
    unsigned rank = blk;
    if (nblocks % 4 == 0 && ngroups % 8 == 0) {
        const unsigned gx = ngroups / 8, per = nblocks / 4;          // groups per XCD; blocks per pass and group
        const unsigned x = lb / (gx * nblocks), i = lb % (gx * nblocks);
        const unsigned pass = i / (gx * per), rem = i % (gx * per);
        hb = x * gx + rem / per;
        rank = pass * per + rem % per;
    }
    blk = rev ? nblocks - 1 - rank : rank;
}

// Entry i of a list row; without a list every tile is walked and treated as mixed.
template <bool MASKED>
__device__ __forceinline__ uint32_t live_entry(const uint32_t* row, unsigned i) {
    return (MASKED && row) ? row[1 + i] : i;
}
__device__ __forceinline__ unsigned entry_tile(uint32_t e) { return e & 0xffffu; }
__device__ __forceinline__ uint32_t entry_class(uint32_t e, int wave) {
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)((e >> (16 + 2 * wave)) & 3u));
}

// ---------------------------------------------------------------------------
// All three kernels stream tiles of 32 positions through a ring of three LDS
// buffers: while tile t is worked on, tile t+1 already lies in LDS (its row
// fragments are read ahead, during the vector work on tile t) and tile t+2 is on
// its way from memory in registers.  One barrier per tile.
// ---------------------------------------------------------------------------
constexpr int RING = 3;

// Every load issued so far has arrived.  Placed before a main loop: a load of the
// prologue whose first use is inside the loop would otherwise put its wait there,
// where on every later pass it waits for the loads that pass has just issued.
__device__ __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0)

// ---------------------------------------------------------------------------
// forward.  grid = H * B * (J / 128); wave = 32 queries.
// ---------------------------------------------------------------------------
template <int P, bool MASKED>
__global__ __launch_bounds__(256) void k_mha_fwd(AttnArgs a, PhiloxKey key_) {
    using G = Geo<P>;
    __shared__ __attribute__((aligned(16))) half_t kt[RING][G::TILE];
    __shared__ __attribute__((aligned(16))) half_t vt[RING][G::TILE];
    const PhiloxKey key = resolved(key_);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    const unsigned qblocks = a.J / QB;
    const unsigned lb = logical_block();
    const unsigned nt = a.K / 32;
    unsigned qb = lb % qblocks, hb = lb / qblocks;
    if (MASKED) masked_order(a.qlist, qblocks, nt, a.H * a.B, lb, qb, hb);
    const unsigned b = hb % a.B, h = hb / a.B;
    const unsigned j = qb * QB + wave * 32 + l32;                    // this lane's query
    const unsigned row = (h * a.B + b) * a.J + j;                    // its score row
    const float c = a.alpha * LOG2E;
    // the key tiles to walk: all of them, or those a mask leaves for these 128 queries
    const uint32_t* live = (MASKED && a.qlist) ? a.qlist + (size_t)qb * (nt + kListPad) : nullptr;
    const unsigned n = live ? live[0] : nt;
    uint32_t e0 = live_entry<MASKED>(live, 0), e1 = live_entry<MASKED>(live, 1), e2 = live_entry<MASKED>(live, 2);

    h8 fq[G::NKS], fk[G::NKS], kr[G::VL], vr[G::VL];
    {   // the first two tiles and the query rows: all loads in flight together
        h8 kr1[G::VL], vr1[G::VL];
        tile_fetch<P>(a.k, h, b, entry_tile(e0) * 32, tid, kr);
        tile_fetch<P>(a.v, h, b, entry_tile(e0) * 32, tid, vr);
        tile_fetch<P>(a.k, h, b, entry_tile(e1) * 32, tid, kr1);
        tile_fetch<P>(a.v, h, b, entry_tile(e1) * 32, tid, vr1);
        row_frags<P>(a.q, h, b, j, hi, fq);
        tile_put<P>(kt[0], tid, kr);
        tile_put<P>(vt[0], tid, vr);
        tile_put<P>(kt[1], tid, kr1);
        tile_put<P>(vt[1], tid, vr1);
    }
    __syncthreads();
    row_frags_lds<P>(kt[0], l32, hi, fk);

    f16v o[G::NPT];
#pragma unroll
    for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[pt][v] = 0.f;
    float m_ref = -INFINITY, l_run = 0.f;                            // l_run: this lane's keys only
    const float slack = RESCALE_SLACK / c;
    int cur = 0, nxt = 1, nn = 2;
    MaskRegs mk = {};
    if (MASKED && n > 0 && entry_class(e0, wave) != BLOCK_CLEAR) load_mask<true>(a, j, entry_tile(e0) * 32, hi, mk);
    // keep words drawn ahead of this launch are fetched a tile early: at the place of their
    // use the load would stand between the scores and their exponentials
    uint32_t word_ahead = 0;
    if (key.thr && n > 0 && entry_tile(e0) < a.keep_tiles_ready) word_ahead = a.keep[(size_t)row * nt + entry_tile(e0)];
    wait_loads();

    for (unsigned i = 0; i < n; ++i) {
        const uint32_t e3 = live_entry<MASKED>(live, i + 3);
        const unsigned t = entry_tile(e0);
        const bool from_mask = MASKED && entry_class(e0, wave) != BLOCK_CLEAR;
        const bool fetch = i + 2 < n;
        const uint32_t word_ready = word_ahead;
        if (key.thr && i + 1 < n && entry_tile(e1) < a.keep_tiles_ready)
            word_ahead = a.keep[(size_t)row * nt + entry_tile(e1)];
        if (fetch) {
            tile_fetch<P>(a.k, h, b, entry_tile(e2) * 32, tid, kr);
            tile_fetch<P>(a.v, h, b, entry_tile(e2) * 32, tid, vr);
        }
        f16v s;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = 0.f;
        if (from_mask) start_from_mask(mk, s);
        if (MASKED && i + 1 < n && entry_class(e1, wave) != BLOCK_CLEAR) load_mask<true>(a, j, entry_tile(e1) * 32, hi, mk);
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk[ks], fq[ks], s, 0, 0, 0);
        // fragments for the second product of this tile and the first of the next
        h8 va[2][G::NPT];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt) va[st][pt] = tr_frag<P>(vt[cur], pt * 32, st, lane);
        row_frags_lds<P>(kt[nxt], l32, hi, fk);

        // keep bits of the 32 scores (this query, keys of tile t): each half of the
        // wave draws two of the four groups of 8 and the halves trade them
        uint32_t word = 0xffffffffu;
        if (key.thr && t < a.keep_tiles_ready) {
            word = word_ready;                                       // drawn ahead of this launch
        } else if (key.thr) {
            const uint64_t g0 = (uint64_t)row * (a.K / 8) + 4 * t + 2 * hi;
            const uint32_t mine = keep8(philox_group_dev(key, g0), key.thr) |
                                  (keep8(philox_group_dev(key, g0 + 1), key.thr) << 8);
            // v_permlane32_swap on two copies: [0] holds the lower half's value in both halves
            // of the wave, [1] the upper half's
            const auto both = __builtin_amdgcn_permlane32_swap(mine, mine, false, false);
            word = both[0] | (both[1] << 16);
        }
        if (hi == 0 && t >= a.keep_tiles_ready) a.keep[(size_t)row * nt + t] = word;
        const uint32_t nib = word >> (hi * 4);                       // bit reg_pos(v, 0) of nib = keep of register v

        // Running softmax with a reference value per query that trails the running
        // maximum by up to RESCALE_SLACK (in log2 units): the accumulators are only
        // rescaled when some query of the wave outgrows its reference by more, which
        // after the first tiles is rare.  Scores and reference are in raw units.
        // The exponentials are taken against the reference as it stands, beside the search
        // for the tile's maximum rather than behind it (the chain maximum -> exchange between
        // the wave's halves -> vote -> exponentials left the wave with nothing to issue), and
        // again in the rare case that the reference moves.
        float ex[16];
        {
            const float mc0 = m_ref == -INFINITY ? 0.f : -m_ref * c;
#pragma unroll
            for (int v = 0; v < 16; ++v) ex[v] = __builtin_amdgcn_exp2f(fmaf(s[v], c, mc0));
        }
        float mt = s[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) mt = fmaxf(mt, s[v]);
        {
            const auto both = __builtin_amdgcn_permlane32_swap(__float_as_uint(mt), __float_as_uint(mt), false, false);
            mt = fmaxf(__uint_as_float(both[0]), __uint_as_float(both[1]));
        }
        if (__builtin_amdgcn_ballot_w64(mt > m_ref + slack) != 0) {
            const float m_new = fmaxf(m_ref, mt);
            // (masked: a query that has seen no key yet has nothing to rescale; the
            // difference of its two infinities is not a number)
            const float corr = (MASKED && m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f((m_ref - m_new) * c);
            m_ref = m_new;
            l_run *= corr;
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[pt][v] *= corr;
            // (masked: a query whose keys so far are all masked out has no reference yet)
            const float mc = m_ref == -INFINITY ? 0.f : -m_ref * c;
#pragma unroll
            for (int v = 0; v < 16; ++v) ex[v] = __builtin_amdgcn_exp2f(fmaf(s[v], c, mc));
        }
        h8 pb[2];
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = ex[v];
        {   // four partial sums: a single one would be a chain of 16 dependent additions
            float l4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int v = 0; v < 16; ++v) l4[v & 3] += s[v];
            l_run += (l4[0] + l4[1]) + (l4[2] + l4[3]);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = keep_if(s[v], nib, reg_pos(v, 0));
#pragma unroll
        for (int v = 0; v < 16; ++v) pb[v >> 3][v & 7] = (half_t)s[v];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt)
                o[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[st][pt], pb[st], o[pt], 0, 0, 0);
        if (fetch) {
            tile_put<P>(kt[nn], tid, kr);
            tile_put<P>(vt[nn], tid, vr);
        }
        __syncthreads();
        const int x = cur; cur = nxt; nxt = nn; nn = x;
        e0 = e1; e1 = e2; e2 = e3;
    }
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    store_rows<P>(a.o, h, b, j, hi, o, 1.0f / l_tot);
    if (hi == 0) a.lse[row] = m_ref * c + __builtin_amdgcn_logf(l_tot);
}

// ---------------------------------------------------------------------------
// backward, dQ.  grid = H * B * (J / 128); wave = 32 queries.
// ---------------------------------------------------------------------------
template <int P, bool MASKED>
__global__ __launch_bounds__(256, !MASKED ? (P == 128 ? 2 : 3) : 1) void k_mha_bwd_dq(AttnArgs a) {
    using G = Geo<P>;
    // Head size 128: with the key and value fragments of a whole tile in registers a tile ahead the kernel
    // needs 300 registers per lane and runs one wave per SIMD; read two k-slices ahead of their use instead,
    // it fits 256 and two waves share a SIMD.
    constexpr bool JIT = !MASKED;
    __shared__ __attribute__((aligned(16))) half_t kt[RING][G::TILE];
    __shared__ __attribute__((aligned(16))) half_t vt[RING][G::TILE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    const unsigned qblocks = a.J / QB;
    const unsigned lb = logical_block();
    const unsigned nt = a.K / 32;
    unsigned qb = lb % qblocks, hb = lb / qblocks;
    if (MASKED) masked_order(a.qlist, qblocks, nt, a.H * a.B, lb, qb, hb);
    const unsigned b = hb % a.B, h = hb / a.B;
    const unsigned j = qb * QB + wave * 32 + l32;
    const unsigned row = (h * a.B + b) * a.J + j;
    const float c = a.alpha * LOG2E;
    const uint32_t* live = (MASKED && a.qlist) ? a.qlist + (size_t)qb * (nt + kListPad) : nullptr;
    const unsigned n = live ? live[0] : nt;
    uint32_t e0 = live_entry<MASKED>(live, 0), e1 = live_entry<MASKED>(live, 1), e2 = live_entry<MASKED>(live, 2);

    h8 fq[G::NKS], fdo[G::NKS], fk[G::NKS], fv[G::NKS], kr[G::VL], vr[G::VL];
    float dsum, lse;
    uint32_t word;
    {   // the first two tiles, the rows of this lane's query and its statistics: all
        // loads in flight together
        h8 kr1[G::VL], vr1[G::VL], fo[G::NKS];
        tile_fetch<P>(a.k, h, b, entry_tile(e0) * 32, tid, kr);
        tile_fetch<P>(a.v, h, b, entry_tile(e0) * 32, tid, vr);
        tile_fetch<P>(a.k, h, b, entry_tile(e1) * 32, tid, kr1);
        tile_fetch<P>(a.v, h, b, entry_tile(e1) * 32, tid, vr1);
        row_frags<P>(a.q, h, b, j, hi, fq);
        row_frags<P>(a.d_o, h, b, j, hi, fdo);
        row_frags<P>(a.o, h, b, j, hi, fo);
        lse = a.lse[row];
        word = a.keep[(size_t)row * nt + entry_tile(e0)];
        tile_put<P>(kt[0], tid, kr);
        tile_put<P>(vt[0], tid, vr);
        tile_put<P>(kt[1], tid, kr1);
        tile_put<P>(vt[1], tid, vr1);
        float part = 0.f;
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks)
#pragma unroll
            for (int i = 0; i < 8; ++i) part += (float)fdo[ks][i] * (float)fo[ks][i];
        dsum = part + __shfl_xor(part, 32);
        if (hi == 0) a.dsum[row] = dsum;
    }
    __syncthreads();
    if constexpr (!JIT) {
        row_frags_lds<P>(kt[0], l32, hi, fk);
        row_frags_lds<P>(vt[0], l32, hi, fv);
    }

    f16v dq[G::NPT];
#pragma unroll
    for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) dq[pt][v] = 0.f;
    int cur = 0, nxt = 1, nn = 2;
    MaskRegs mk = {};
    if (MASKED && n > 0 && entry_class(e0, wave) != BLOCK_CLEAR) load_mask<true>(a, j, entry_tile(e0) * 32, hi, mk);
    wait_loads();

    for (unsigned i = 0; i < n; ++i) {
        const uint32_t e3 = live_entry<MASKED>(live, i + 3);
        const bool from_mask = MASKED && entry_class(e0, wave) != BLOCK_CLEAR;
        const bool fetch = i + 2 < n;
        if (fetch) {
            tile_fetch<P>(a.k, h, b, entry_tile(e2) * 32, tid, kr);
            tile_fetch<P>(a.v, h, b, entry_tile(e2) * 32, tid, vr);
        }
        const uint32_t wordn = i + 1 < n ? a.keep[(size_t)row * nt + entry_tile(e1)] : 0u;
        f16v s, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = 0.f; }
        if (from_mask) start_from_mask(mk, s);
        if (MASKED && i + 1 < n && entry_class(e1, wave) != BLOCK_CLEAR) load_mask<true>(a, j, entry_tile(e1) * 32, hi, mk);
        if constexpr (JIT) {
            h8 ck[2], cv[2];
            ck[0] = *reinterpret_cast<const h8*>(kt[cur] + G::at(l32, hi));
            cv[0] = *reinterpret_cast<const h8*>(vt[cur] + G::at(l32, hi));
#pragma unroll
            for (int ks = 0; ks < G::NKS; ++ks) {
                if (ks + 1 < G::NKS) {
                    ck[(ks + 1) & 1] = *reinterpret_cast<const h8*>(kt[cur] + G::at(l32, 2 * (ks + 1) + hi));
                    cv[(ks + 1) & 1] = *reinterpret_cast<const h8*>(vt[cur] + G::at(l32, 2 * (ks + 1) + hi));
                }
                s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ck[ks & 1], fq[ks], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_f16(cv[ks & 1], fdo[ks], dp, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < G::NKS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(fk[ks], fq[ks], s, 0, 0, 0);
#pragma unroll
            for (int ks = 0; ks < G::NKS; ++ks) dp = __builtin_amdgcn_mfma_f32_32x32x16_f16(fv[ks], fdo[ks], dp, 0, 0, 0);
        }
        h8 ka[2][G::NPT];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt) ka[st][pt] = tr_frag<P>(kt[cur], pt * 32, st, lane);
        if constexpr (!JIT) {
            row_frags_lds<P>(kt[nxt], l32, hi, fk);
            row_frags_lds<P>(vt[nxt], l32, hi, fv);
        }
        const uint32_t nib = word >> (hi * 4);
        // stage by stage over the 16 scores of the lane, so that consecutive
        // instructions do not depend on one another
        h8 ds[2];
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = fmaf(s[v], c, -lse);
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] = __builtin_amdgcn_exp2f(s[v]);
#pragma unroll
        for (int v = 0; v < 16; ++v) dp[v] = keep_if(dp[v], nib, reg_pos(v, 0));
#pragma unroll
        for (int v = 0; v < 16; ++v) dp[v] -= dsum;
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] *= dp[v];
#pragma unroll
        for (int v = 0; v < 16; ++v) ds[v >> 3][v & 7] = (half_t)s[v];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt)
                dq[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[st][pt], ds[st], dq[pt], 0, 0, 0);
        if (fetch) {
            tile_put<P>(kt[nn], tid, kr);
            tile_put<P>(vt[nn], tid, vr);
        }
        word = wordn;
        __syncthreads();
        const int x = cur; cur = nxt; nxt = nn; nn = x;
        e0 = e1; e1 = e2; e2 = e3;
    }
    store_rows<P>(a.dq, h, b, j, hi, dq, a.alpha);
    if (a.bias_q)
        column_sums<P>(dq, a.alpha, reinterpret_cast<float*>(&kt[0][0]),
                       a.bias_q + ((size_t)h * (a.B * qblocks) + b * qblocks + qb) * P, tid);
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

template <int P, bool MASKED>
__global__ __launch_bounds__(256, (P == 64 && MASKED) ? 2 : 1) void k_mha_bwd_dkv(AttnArgs a) {
    using G = Geo<P>;
    __shared__ __attribute__((aligned(16))) KvStage<P> stage[RING];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, hi = lane >> 5;
    const unsigned kblocks = a.K / QB;
    const unsigned lb = logical_block();
    const unsigned nq = a.J / 32, nkt = a.K / 32;
    unsigned kb = lb % kblocks, hb = lb / kblocks;
    if (MASKED) masked_order(a.klist, kblocks, nq, a.H * a.B, lb, kb, hb);
    const unsigned b = hb % a.B, h = hb / a.B;
    const unsigned kpos = kb * QB + wave * 32 + l32;                 // this lane's key
    const unsigned row0 = (h * a.B + b) * a.J;                       // score row of query 0
    const float c = a.alpha * LOG2E;
    // the query tiles to walk: all of them, or those a mask leaves for these 128 keys
    const uint32_t* live = (MASKED && a.klist) ? a.klist + (size_t)kb * (nq + kListPad) : nullptr;
    const unsigned n = live ? live[0] : nq;
    uint32_t e0 = live_entry<MASKED>(live, 0), e1 = live_entry<MASKED>(live, 1), e2 = live_entry<MASKED>(live, 2);

    h8 fk[G::NKS], fv[G::NKS], fq[G::NKS], fdo[G::NKS];
    struct InFlight {             // one tile of queries on its way from memory
        h8 q[G::VL], d_o[G::VL];
        float stat;
        uint4 kw;
    };
    auto fetch = [&](unsigned qt, InFlight& f) {
        tile_fetch<P>(a.q, h, b, qt * 32, tid, f.q);
        tile_fetch<P>(a.d_o, h, b, qt * 32, tid, f.d_o);
        const unsigned r = row0 + qt * 32 + (tid & 31);
        if (tid < 32) f.stat = a.lse[r];
        else if (tid < 64) f.stat = a.dsum[r];
        else if (tid < 96) f.kw = *reinterpret_cast<const uint4*>(a.keep + (size_t)r * nkt + kb * 4);
    };
    auto put = [&](KvStage<P>& sg, const InFlight& f) {
        tile_put<P>(sg.q, tid, f.q);
        tile_put<P>(sg.d_o, tid, f.d_o);
        if (tid < 32) sg.lse[tid] = f.stat;
        else if (tid < 64) sg.dsum[tid - 32] = f.stat;
        else if (tid < 96) {
            sg.keep[0][tid - 64] = f.kw.x; sg.keep[1][tid - 64] = f.kw.y;
            sg.keep[2][tid - 64] = f.kw.z; sg.keep[3][tid - 64] = f.kw.w;
        }
    };
    InFlight fl;
    fl.stat = 0.f; fl.kw = make_uint4(0, 0, 0, 0);
    {
        InFlight f1;
        f1.stat = 0.f; f1.kw = make_uint4(0, 0, 0, 0);
        fetch(entry_tile(e0), fl);
        fetch(entry_tile(e1), f1);
        row_frags<P>(a.k, h, b, kpos, hi, fk);
        row_frags<P>(a.v, h, b, kpos, hi, fv);
        put(stage[0], fl);
        put(stage[1], f1);
    }
    __syncthreads();
    row_frags_lds<P>(stage[0].q, l32, hi, fq);
    row_frags_lds<P>(stage[0].d_o, l32, hi, fdo);

    f16v dk[G::NPT], dv[G::NPT];
#pragma unroll
    for (int pt = 0; pt < G::NPT; ++pt)
#pragma unroll
        for (int v = 0; v < 16; ++v) { dk[pt][v] = 0.f; dv[pt][v] = 0.f; }
    int cur = 0, nxt = 1, nn = 2;
    MaskRegs mk = {};
    if (MASKED && n > 0 && entry_class(e0, wave) != BLOCK_CLEAR) load_mask<false>(a, kpos, entry_tile(e0) * 32, hi, mk);
    wait_loads();

    for (unsigned i = 0; i < n; ++i) {
        const uint32_t e3 = live_entry<MASKED>(live, i + 3);
        const bool from_mask = MASKED && entry_class(e0, wave) != BLOCK_CLEAR;
        const bool more = i + 2 < n;
        if (more) fetch(entry_tile(e2), fl);
        const KvStage<P>& sg = stage[cur];
        f16v s, dp;
#pragma unroll
        for (int v = 0; v < 16; ++v) { s[v] = 0.f; dp[v] = 0.f; }
        if (from_mask) start_from_mask(mk, s);
        if (MASKED && i + 1 < n && entry_class(e1, wave) != BLOCK_CLEAR) load_mask<false>(a, kpos, entry_tile(e1) * 32, hi, mk);
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(fq[ks], fk[ks], s, 0, 0, 0);
#pragma unroll
        for (int ks = 0; ks < G::NKS; ++ks) dp = __builtin_amdgcn_mfma_f32_32x32x16_f16(fdo[ks], fv[ks], dp, 0, 0, 0);
        h8 qa[2][G::NPT], da[2][G::NPT];
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt) {
                da[st][pt] = tr_frag<P>(sg.d_o, pt * 32, st, lane);
                qa[st][pt] = tr_frag<P>(sg.q, pt * 32, st, lane);
            }
        row_frags_lds<P>(stage[nxt].q, l32, hi, fq);
        row_frags_lds<P>(stage[nxt].d_o, l32, hi, fdo);
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
                const int keep = __builtin_amdgcn_sbfe((int)wv[e], l32, 1);
                pd[v >> 3][v & 7] = (half_t)__int_as_float(__float_as_int(p) & keep);
                ds[v >> 3][v & 7] = (half_t)(p * (__int_as_float(__float_as_int(dp[v]) & keep) - ddv[e]));
            }
        }
#pragma unroll
        for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int pt = 0; pt < G::NPT; ++pt) {
                dv[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(da[st][pt], pd[st], dv[pt], 0, 0, 0);
                dk[pt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa[st][pt], ds[st], dk[pt], 0, 0, 0);
            }
        if (more) put(stage[nn], fl);
        __syncthreads();
        const int x = cur; cur = nxt; nxt = nn; nn = x;
        e0 = e1; e1 = e2; e2 = e3;
    }
    store_rows<P>(a.dk, h, b, kpos, hi, dk, a.alpha);
    store_rows<P>(a.dv, h, b, kpos, hi, dv, 1.0f);
    if (a.bias_kv) {
        const size_t ntc = (size_t)a.B * kblocks, part = (size_t)h * ntc + b * kblocks + kb;
        float* red = reinterpret_cast<float*>(&stage[0]);
        column_sums<P>(dk, a.alpha, red, a.bias_kv + part * P, tid);
        column_sums<P>(dv, 1.0f, red + 4 * P, a.bias_kv + ((size_t)a.H * ntc + part) * P, tid);
    }
}

// 8-byte loads of four mask values along whichever dim is contiguous
bool mask_ok(const AttnArgs& a) {
    if (!a.amask) return true;
    if ((reinterpret_cast<uintptr_t>(a.amask) & 7) != 0) return false;
    if (a.am_sk == 1) return a.am_sj % 4 == 0;
    if (a.am_sj == 1) return a.am_sk % 4 == 0;
    return true;
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
    return mha_shape_ok(a.H, a.B, a.J, a.K, P) && a.alpha > 0.f && side_ok(a.q) && side_ok(a.k) && side_ok(a.v) && side_ok(a.o) &&
           a.lse && a.keep && (reinterpret_cast<uintptr_t>(a.lse) & 15) == 0 &&
           (reinterpret_cast<uintptr_t>(a.keep) & 15) == 0 && mask_ok(a);
}

namespace {
size_t up16(size_t x) { return (x + 15) & ~(size_t)15; }
size_t qlist_bytes(long J, long K) { return up16((size_t)(J / QB) * (size_t)(K / 32 + kListPad) * 4); }
size_t klist_bytes(long J, long K) { return up16((size_t)(K / QB) * (size_t)(J / 32 + kListPad) * 4); }
}  // namespace

size_t mha_mask_plan_bytes(long J, long K) {
    return qlist_bytes(J, K) + klist_bytes(J, K) + up16((size_t)(J / 32) * (size_t)(K / 32));
}

void launch_mha_mask_plan(AttnArgs& a, void* plan, bool rebuild, hipStream_t st) {
    uint32_t* qlist = (uint32_t*)plan;
    uint32_t* klist = (uint32_t*)((char*)plan + qlist_bytes(a.J, a.K));
    uint8_t* cls = (uint8_t*)plan + qlist_bytes(a.J, a.K) + klist_bytes(a.J, a.K);
    if (rebuild) {
        hipLaunchKernelGGL(k_mha_mask_classes, dim3((unsigned)((a.J / 32) * (a.K / 32))), dim3(64), 0, st, a.amask,
                           a.am_sj, a.am_sk, a.K, cls);
        hipLaunchKernelGGL(k_mha_mask_lists, dim3((unsigned)(a.J / QB + a.K / QB)), dim3(64), 0, st, cls, a.J, a.K, qlist,
                           klist);
    }
    a.qlist = qlist; a.klist = klist;
}

void launch_mha_forward(const AttnArgs& a, int P, PhiloxKey key, hipStream_t st) {
    if (!mha_forward_ok(a, P)) fail("attention forward: shape, strides or alignment not supported");
    dim3 grid((unsigned)(a.H * a.B * (a.J / QB)));
    if (a.amask) {
        if (P == 64) hipLaunchKernelGGL((k_mha_fwd<64, true>), grid, dim3(256), 0, st, a, key);
        else hipLaunchKernelGGL((k_mha_fwd<128, true>), grid, dim3(256), 0, st, a, key);
    } else {
        if (P == 64) hipLaunchKernelGGL((k_mha_fwd<64, false>), grid, dim3(256), 0, st, a, key);
        else hipLaunchKernelGGL((k_mha_fwd<128, false>), grid, dim3(256), 0, st, a, key);
    }
    check_launch("attention forward");
}

bool mha_backward_ok(const AttnArgs& a, int P) {
    return mha_forward_ok(a, P) && a.dsum && side_ok(a.d_o) && side_ok(a.dq) && side_ok(a.dk) && side_ok(a.dv);
}

void launch_mha_backward_dq(const AttnArgs& a, int P, hipStream_t st) {
    if (!mha_backward_ok(a, P)) fail("attention backward: shape, strides or alignment not supported");
    dim3 grid((unsigned)(a.H * a.B * (a.J / QB)));
    if (a.amask) {
        if (P == 64) hipLaunchKernelGGL((k_mha_bwd_dq<64, true>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((k_mha_bwd_dq<128, true>), grid, dim3(256), 0, st, a);
    } else {
        if (P == 64) hipLaunchKernelGGL((k_mha_bwd_dq<64, false>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((k_mha_bwd_dq<128, false>), grid, dim3(256), 0, st, a);
    }
    check_launch("attention backward (dQ)");
}

void launch_mha_backward_dkv(const AttnArgs& a, int P, hipStream_t st) {
    if (!mha_backward_ok(a, P)) fail("attention backward: shape, strides or alignment not supported");
    dim3 grid((unsigned)(a.H * a.B * (a.K / QB)));
    if (a.amask) {
        if (P == 64) hipLaunchKernelGGL((k_mha_bwd_dkv<64, true>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((k_mha_bwd_dkv<128, true>), grid, dim3(256), 0, st, a);
    } else {
        if (P == 64) hipLaunchKernelGGL((k_mha_bwd_dkv<64, false>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((k_mha_bwd_dkv<128, false>), grid, dim3(256), 0, st, a);
    }
    check_launch("attention backward (dK, dV)");
}

}  // namespace sub
