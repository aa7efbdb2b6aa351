// Tensor contractions: strided, batched fp16 GEMM with fp32 accumulation on the
// gfx950 matrix cores (v_mfma_f32_32x32x16_f16), honouring each operand's
// stride layout.  Takes the place of the cuBLAS calls behind
// pytorch_module/gemm.cuh:52-147.
//
//   C[b, m, n] = alpha * sum_k A[b, m, k] * B[b, k, n]  (+ bias)
//
// Operands may be contiguous along the contraction (K) or along their free
// dimension (M resp. N); an operand that is contiguous along its free dimension
// lies in LDS as in memory and is gathered with the transposing LDS read, so the
// matrix-core fragments are always 8 consecutive k per lane.  (Turning such tiles
// around in registers on the way into LDS instead, to read them at the full rate of
// ds_read_b128, was measured: 1 to 3 us slower per product of 34 GFLOP.)
// The output is produced transposed in the
// accumulators (4 consecutive n per lane), staged through LDS and written as
// full 128-bit rows.
#include <type_traits>
#include <cstring>

#include "sub_ops.hpp"
#include "sub_finish.hpp"

namespace sub {

namespace {

typedef float f16v __attribute__((ext_vector_type(16)));

struct GemmArgs {
    const half_t* A; const half_t* B; half_t* C;
    int M, N, K1, K0;
    long sAM, sAK1, sAK0;
    long sBN, sBK1, sBK0;
    long sCM, sCN;
    int nb1, nb2;                 // sizes of batch dims 1 and 2 (dim 0 is the quotient)
    long sAb[3], sBb[3], sCb[3];
    float alpha;
    const half_t* bias; long sbM, sbN, sbb[3];
    int splits;                   // > 1: the k range is split, fp32 partial tiles go to `partial`
    float* partial;               // [split][batch][M][N]
    int relu_dropout = 0;         // epilogue of the asynchronous kernel: ReLU and dropout after the addend
    PhiloxKey key;
    const half_t* gate = nullptr; // or: zero where gate <= 0 (strides of `bias`), column sums per 128-row slab
    float* colsum = nullptr;
    const uint32_t* keep_words = nullptr;  // relu_dropout: the keep bits, drawn ahead (relu_dropout_keep_words)
    uint32_t* gate_bits_out = nullptr;     // relu_dropout: one bit per output, set where it is positive
    const uint32_t* gate_bits = nullptr;   // gate: those bits instead of the values of `gate`
    int act = ACT_RELU;                    // the activation of relu_dropout / gate (GemmEpilogue::act)
    half_t* pre_out = nullptr;             // GELU with dropout: where the rounded sum before the activation goes
    // GemmSideJob of the eight-wave asynchronous kernel: workgroups side_first .. gridDim.x - 1 draw
    // the attention keep words of key tiles 0 .. side_tiles_done - 1 of side_rows score rows
    unsigned side_first = 0, side_blocks = 0;
    PhiloxKey side_key;
    uint32_t* side_keep = nullptr;
    uint32_t side_rows = 0, side_nk = 0, side_tiles_done = 0;
};

// The arguments every tile of a product needs, fetched in one go at the start of the workgroup
// (fetch_args_now): the index arithmetic between them would otherwise be interleaved with four or
// five scalar round trips.
__device__ __forceinline__ void fetch_gemm_args(const GemmArgs& g) {
    fetch_args_now(g.A, g.B, g.C, g.M, g.N, g.K1, g.K0, g.sAM, g.sAK1, g.sAK0, g.sBN, g.sBK1, g.sBK0, g.sCM, g.nb1, g.nb2,
                   g.sAb[0], g.sAb[1], g.sAb[2], g.sBb[0], g.sBb[1], g.sBb[2], g.sCb[0], g.sCb[1], g.sCb[2], g.alpha,
                   g.bias, g.sbM, g.splits);
}

// A workgroup that multiplies nothing (see GemmSideJob): workgroup sb of nsb.
__device__ __forceinline__ void side_block(const GemmArgs& g, unsigned sb, unsigned nsb) {
    const PhiloxKey key = resolved(g.side_key);
    const uint32_t nt = g.side_nk / 32, td = g.side_tiles_done;
    // word w of rows * td is (row w / td, tile w % td); a thread walks w in steps of `stride`, carrying row
    // and tile along instead of dividing (a 64-bit division is as long as one of the word's four draws)
    const uint32_t stride = nsb * blockDim.x, first = sb * blockDim.x + threadIdx.x;
    const uint32_t srow = stride / td, st = stride - srow * td;
    uint32_t row = first / td, t = first - row * td;
    for (; row < g.side_rows; row += srow) {
        g.side_keep[(size_t)row * nt + t] = attention_keep_word(key, row, g.side_nk, t);
        t += st;
        if (t >= td) { t -= td; ++row; }
    }
}

// ---------------------------------------------------------------------------
// Scalar fallback: any strides, any sizes.  One thread per output element.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_gemm_scalar(GemmArgs g, long total) {
    long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int n = (int)(idx % g.N); long r = idx / g.N;
    int m = (int)(r % g.M); long b = r / g.M;
    long b2 = b % g.nb2; long t = b / g.nb2;
    long b1 = t % g.nb1; long b0 = t / g.nb1;
    const half_t* a = g.A + b0 * g.sAb[0] + b1 * g.sAb[1] + b2 * g.sAb[2] + (long)m * g.sAM;
    const half_t* bp = g.B + b0 * g.sBb[0] + b1 * g.sBb[1] + b2 * g.sBb[2] + (long)n * g.sBN;
    float acc = 0.f;
    for (int k0 = 0; k0 < g.K0; ++k0) {
        const half_t* a0 = a + (long)k0 * g.sAK0;
        const half_t* b0p = bp + (long)k0 * g.sBK0;
        for (int k = 0; k < g.K1; ++k) acc += (float)a0[(long)k * g.sAK1] * (float)b0p[(long)k * g.sBK1];
    }
    half_t out = (half_t)(acc * g.alpha);
    if (g.bias)     // same two roundings as the product followed by a separate add
        out = (half_t)((float)out + (float)g.bias[b0 * g.sbb[0] + b1 * g.sbb[1] + b2 * g.sbb[2] +
                                                  (long)m * g.sbM + (long)n * g.sbN]);
    g.C[b0 * g.sCb[0] + b1 * g.sCb[1] + b2 * g.sCb[2] + (long)m * g.sCM + (long)n * g.sCN] = out;
}

// ---------------------------------------------------------------------------
// MFMA kernel.  256 threads = 2x2 waves; each wave owns TM x TN tiles of 32x32.
// ---------------------------------------------------------------------------
constexpr int BK = 64;            // k per LDS tile

constexpr int MC_PAD = 32;        // halves of padding per k-row of a free-dim-contiguous tile

typedef short s4v __attribute__((ext_vector_type(4)));

// One operand tile in LDS: ROWS (free dim) x BK (k).
//
// KC (k contiguous in memory): rows of 64 halves = eight 16-byte slots, the slot
// index xor-ed with a function of the row so that the fragment reads (32
// consecutive rows, one slot) spread over the banks.  A fragment is one
// ds_read_b128: 8 consecutive k of one row.
//
// !KC (free dim contiguous in memory): the tile is stored as it lies in memory,
// [k][free] with a padded pitch, and fragments are gathered with the LDS
// transpose read ds_read_b64_tr_b16.  Within each group of 16 lanes, lane i of
// that instruction receives, as element e, the (i%4)-th half of the 8
// bytes addressed by lane 4e + i/4.  With lane l addressing
// T[k0 + l/4][m0 + 4*(l%4) ..+3], lane i ends up with T[k0 + 0..3][m0 + i]:
// four consecutive k of its own row, which is what the matrix core wants.
template <int ROWS, bool KC, int NT = 256>
struct Tile {
    static constexpr int PITCH = KC ? BK : ROWS + MC_PAD;            // halves
    static constexpr int HALVES = KC ? ROWS * BK : BK * (ROWS + MC_PAD);
    static constexpr int NV = ROWS * 8 / NT;                          // 16-byte loads per thread (NT threads)
    static constexpr int VPR = ROWS / 8;                              // vectors per k-row (!KC)

    static __device__ __forceinline__ int kc_off(int row, int slot) {
        return row * BK + ((slot ^ (row ^ (row >> 3))) & 7) * 8;
    }

    // base points at (free0, k-tile start) of the current batch; sF / sK are the
    // strides of the free dim and of k; nfree / nk the extents left.
    // Per-thread element offsets of its NV vectors within a tile (constant over
    // the k loop) and, for edge tiles, which of them lie inside the free extent.
    static __device__ __forceinline__ void offsets(unsigned (&off)[NV], unsigned& okmask, long sF, long sK,
                                                   int nfree, int tid) {
        okmask = 0;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            int id = tid + i * NT;
            if (KC) {
                int row = id >> 3, slot = id & 7;
                off[i] = (unsigned)((long)row * sF + slot * 8);
                okmask |= (row < nfree ? 1u : 0u) << i;
            } else {
                int k = id / VPR, mv = id % VPR;
                off[i] = (unsigned)((long)k * sK + mv * 8);
                okmask |= (mv * 8 + 8 <= nfree ? 1u : 0u) << i;
            }
        }
    }

    // CHECK = false: the whole tile is inside the matrix, no predication.
    // `tile` is wave-uniform; nk = k extent left at the start of this tile.
    template <bool CHECK>
    static __device__ __forceinline__ void load(h8 (&v)[NV], const half_t* tile, const unsigned (&off)[NV],
                                                unsigned okmask, int nk, int tid) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const h8* p = reinterpret_cast<const h8*>(tile + off[i]);
            if (!CHECK) {
                v[i] = *p;
            } else {
                int id = tid + i * NT;
                bool kok = KC ? ((id & 7) * 8 + 8 <= nk) : (id / VPR < nk);
                v[i] = (h8)(half_t)0.0f;
                if (kok && ((okmask >> i) & 1u)) v[i] = *p;
            }
        }
    }

    static __device__ __forceinline__ void store(const h8 (&v)[NV], half_t* lds, int tid) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            int id = tid + i * NT;
            if (KC) {
                *reinterpret_cast<h8*>(lds + kc_off(id >> 3, id & 7)) = v[i];
            } else {
                *reinterpret_cast<h8*>(lds + (id / VPR) * PITCH + (id % VPR) * 8) = v[i];
            }
        }
    }

    // Fragment of the 32-row block starting at row0 for k-step ks (16 k): lane
    // (l32 = lane%32, hi = lane/32) gets k = ks*16 + 8*hi + 0..7 of row row0+l32.
    static __device__ __forceinline__ h8 frag(const half_t* lds, int row0, int ks, int lane) {
        if (KC) {
            return *reinterpret_cast<const h8*>(lds + kc_off(row0 + (lane & 31), ks * 2 + (lane >> 5)));
        } else {
            const int g = lane >> 4, l = lane & 15;
            const int k = ks * 16 + 8 * (g >> 1) + (l >> 2);
            const int m = row0 + 16 * (g & 1) + 4 * (l & 3);
            const half_t* p = lds + k * PITCH + m;
            typedef s4v __attribute__((address_space(3))) * lds_s4;
            s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(p));
            s4v hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(p + 4 * PITCH));
            typedef short s8 __attribute__((ext_vector_type(8)));
            s8 r = __builtin_shufflevector(lo, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(h8, r);
        }
    }
};

// LDS (in halves) of one workgroup of the register-staged kernel: two pipeline
// stages, reused by the epilogue's per-wave staging slabs.
template <int TM, int TN, bool AKC, bool BKC, int WM = 2>
constexpr int mfma_lds_halves() {
    constexpr int stage = Tile<32 * WM * TM, AKC, 128 * WM>::HALVES + Tile<64 * TN, BKC, 128 * WM>::HALVES;
    constexpr int slabs = 2 * WM * 32 * (32 * TN + 8);
    return 2 * stage > slabs ? 2 * stage : slabs;
}

// Issue order of one k-tile of the register-staged loop (16 matrix instructions for a
// 2 x 2 wave tile): with a single wave on a SIMD nothing else fills the matrix pipe while
// that wave issues LDS reads, so the fragment reads of the next k-slice and the global
// loads of the tile after next are dealt out between the matrix instructions instead of in
// clumps (left to itself the compiler issues up to 15 reads in a row).  The LDS writes of
// the next tile come after the last fragment read (the compiler cannot tell the two
// stages apart and keeps them in program order), two per matrix instruction of the last
// k-slice.  RA / RB: LDS reads per fragment of A / B (1 ds_read_b128, or 2 transposing
// reads).  Measured at M = 4096, N = 1024, K = 4096: 53 -> 47 us (both operands
// transposed), 59 -> 53 us, a pair of such products 82 -> 77 us.
template <int RA, int RB, int NLOAD>
__device__ __forceinline__ void sched_k_tile() {
    constexpr int R1 = 2 * RA + 2 * RB;              // the reads of one k-slice
    __builtin_amdgcn_sched_group_barrier(0x100, R1, 0);
#define SUB_SCHED_ONE(m)                                                                          \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                            \
    if constexpr ((m) < 12) __builtin_amdgcn_sched_group_barrier(0x100, (R1 * ((m) + 1)) / 4 - (R1 * (m)) / 4, 0); \
    if constexpr ((m) < NLOAD) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                 \
    if constexpr ((m) >= 12) __builtin_amdgcn_sched_group_barrier(0x200, (NLOAD * ((m) - 11)) / 4 - (NLOAD * ((m) - 12)) / 4, 0);
    SUB_SCHED_ONE(0) SUB_SCHED_ONE(1) SUB_SCHED_ONE(2) SUB_SCHED_ONE(3) SUB_SCHED_ONE(4) SUB_SCHED_ONE(5)
    SUB_SCHED_ONE(6) SUB_SCHED_ONE(7) SUB_SCHED_ONE(8) SUB_SCHED_ONE(9) SUB_SCHED_ONE(10) SUB_SCHED_ONE(11)
    SUB_SCHED_ONE(12) SUB_SCHED_ONE(13) SUB_SCHED_ONE(14) SUB_SCHED_ONE(15)
#undef SUB_SCHED_ONE
}

// One workgroup's share of a product: block `block_id` of `nblocks`.  WM x 2 waves
// (WM = 2: 256 threads; WM = 4: 512 threads and a tile twice as tall, whose workgroup
// draws a quarter less from L2 per flop than two workgroups with square tiles).
template <int TM, int TN, bool AKC, bool BKC, bool FULL, int WM = 2>
__device__ __forceinline__ void gemm_mfma_body(const GemmArgs& g, long block_id, long nblocks, half_t* lds) {
    constexpr int BM = 32 * WM * TM, BN = 64 * TN, NT = 128 * WM;
    using TA = Tile<BM, AKC, NT>;
    using TB = Tile<BN, BKC, NT>;
    constexpr int STAGE = TA::HALVES + TB::HALVES;                   // one pipeline stage
    constexpr int STAGE_PITCH = 32 * TN + 8;                          // halves
    constexpr int STAGE_WAVE = 32 * STAGE_PITCH;                      // one 32-row slab per wave

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, hi = lane >> 5;

    // Workgroup -> tile.  Workgroups are dealt round-robin to the 8 XCDs (each
    // with its own L2), so consecutive logical tiles are given to one XCD, and
    // within a batch tiles are walked in groups of 8 tile-rows so that the
    // workgroups resident together share A and B tiles in that L2.
    // (32-bit arithmetic: a launch has fewer than 2^31 workgroups, and each 64-bit division here is 130
    // instructions that stand between the start of the workgroup and its first load)
    fetch_gemm_args(g);
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    unsigned lid = (unsigned)block_id;
    if ((nblocks & 7) == 0) lid = (lid & 7u) * (unsigned)(nblocks >> 3) + (lid >> 3);
    const unsigned per_batch = (unsigned)(tiles_m * tiles_n);
    const int split = (int)(lid % (unsigned)g.splits);        // k-splits of one tile sit next to each other
    lid /= (unsigned)g.splits;
    const unsigned bz = lid / per_batch;
    int r = (int)(lid - bz * per_batch);
    // (a tall tile's rows are the dearer operand: the 16 tiles an XCD holds of one product as 2 rows x 8
    // columns draw 192 KiB per k-step into its L2, as 8 x 2 288 KiB; measured 0.7 us per pair launch)
    constexpr int GM = WM == 4 ? 2 : 8;
    const int grp = r / (GM * tiles_n), first_m = grp * GM;
    const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int rr = r - grp * GM * tiles_n;
    const int tile_m = first_m + rr % gsz, tile_n = rr / gsz;
    const unsigned tq = bz / (unsigned)g.nb2;
    const long b2 = bz - tq * (unsigned)g.nb2, b0 = tq / (unsigned)g.nb1, b1 = tq - (unsigned)b0 * (unsigned)g.nb1;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const half_t* Ab = g.A + b0 * g.sAb[0] + b1 * g.sAb[1] + b2 * g.sAb[2] + (long)m0 * g.sAM;
    const half_t* Bb = g.B + b0 * g.sBb[0] + b1 * g.sBb[1] + b2 * g.sBb[2] + (long)n0 * g.sBN;
    const int mleft = g.M - m0, nleft = g.N - n0;

    const int tiles_per_k1 = (g.K1 + BK - 1) / BK;
    const int nkt_all = g.K0 * tiles_per_k1;
    // this workgroup's share of the k-tiles
    const int kt_begin = (int)((long)nkt_all * split / g.splits);
    const int nkt = (int)((long)nkt_all * (split + 1) / g.splits) - kt_begin;

    f16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // Software pipeline: two register sets hold the global loads of the next two
    // k-tiles (issued one and two iterations ahead), two LDS stages hold the
    // current tile and the one being written.
    h8 ra0[TA::NV], rb0[TB::NV], ra1[TA::NV], rb1[TB::NV];
    unsigned offa[TA::NV], offb[TB::NV], oka, okb;
    TA::offsets(offa, oka, g.sAM, g.sAK1, mleft, tid);
    TB::offsets(offb, okb, g.sBN, g.sBK1, nleft, tid);

    // Running (wave-uniform) pointers to the next k-tile to fetch.  Past the last
    // tile they stay on it: the surplus prefetches re-read valid memory and are
    // never consumed, which keeps the loop body free of branches.
    int kin = kt_begin % tiles_per_k1, fetched = 0;
    const half_t* pa = Ab + (long)(kt_begin / tiles_per_k1) * g.sAK0 + (long)kin * BK * g.sAK1;
    const half_t* pb = Bb + (long)(kt_begin / tiles_per_k1) * g.sBK0 + (long)kin * BK * g.sBK1;
    const long stepA = (long)BK * g.sAK1, stepB = (long)BK * g.sBK1;
    const long wrapA = g.sAK0 - (long)(tiles_per_k1 - 1) * stepA;
    const long wrapB = g.sBK0 - (long)(tiles_per_k1 - 1) * stepB;

#define SUB_GEMM_ISSUE(RA, RB)                                                                    \
    do {                                                                                          \
        TA::template load<!FULL>(RA, pa, offa, oka, g.K1 - kin * BK, tid);                        \
        TB::template load<!FULL>(RB, pb, offb, okb, g.K1 - kin * BK, tid);                        \
        const bool more_ = fetched + 1 < nkt;                                                     \
        const bool wrap_ = kin + 1 == tiles_per_k1;                                               \
        pa += more_ ? (wrap_ ? wrapA : stepA) : 0;                                                \
        pb += more_ ? (wrap_ ? wrapB : stepB) : 0;                                                \
        kin = more_ ? (wrap_ ? 0 : kin + 1) : kin;                                                \
        fetched += more_ ? 1 : 0;                                                                 \
    } while (0)

#define SUB_GEMM_COMPUTE(stage_)                                                                  \
    do {                                                                                          \
        const half_t* sA = lds + (stage_) * STAGE;                                                \
        const half_t* sB = sA + TA::HALVES;                                                       \
        h8 fa[2][TM], fb[2][TN];                                                                  \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                                            \
            fa[0][i] = TA::frag(sA, (wm * TM + i) * 32, 0, lane);                                 \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                            \
            fb[0][j] = TB::frag(sB, (wn * TN + j) * 32, 0, lane);                                 \
        _Pragma("unroll") for (int ks = 0; ks < BK / 16; ++ks) {                                  \
            if (ks + 1 < BK / 16) {                                                               \
                _Pragma("unroll") for (int i = 0; i < TM; ++i)                                    \
                    fa[(ks + 1) & 1][i] = TA::frag(sA, (wm * TM + i) * 32, ks + 1, lane);         \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                    \
                    fb[(ks + 1) & 1][j] = TB::frag(sB, (wn * TN + j) * 32, ks + 1, lane);         \
            }                                                                                     \
            /* D^T tiles: rows of the MFMA result run along n, columns along m. */                \
            _Pragma("unroll") for (int i = 0; i < TM; ++i)                                        \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                    \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ks & 1][j], fa[ks & 1][i], \
                                                                       acc[i][j], 0, 0, 0);       \
        }                                                                                         \
    } while (0)

#define SUB_GEMM_STORE(stage_, RA, RB)                                                            \
    do {                                                                                          \
        half_t* dA = lds + (stage_) * STAGE;                                                      \
        TA::store(RA, dA, tid);                                                                   \
        TB::store(RB, dA + TA::HALVES, tid);                                                      \
    } while (0)

    SUB_GEMM_ISSUE(ra0, rb0);          // tile 0
    SUB_GEMM_ISSUE(ra1, rb1);          // tile 1 (or tile 0 again)
    SUB_GEMM_STORE(0, ra0, rb0);
    __syncthreads();

    // Step 2p: stage 0 holds tile 2p, set 1 holds tile 2p+1 in flight, set 0 is free.
    const int npairs = nkt >> 1;
    constexpr bool kSched = TM == 2 && TN == 2 && FULL;
    for (int p = 0; p < npairs; ++p) {
        SUB_GEMM_ISSUE(ra0, rb0);                 // tile 2p+2
        SUB_GEMM_COMPUTE(0);
        SUB_GEMM_STORE(1, ra1, rb1);              // tile 2p+1
        if constexpr (kSched) sched_k_tile<AKC ? 1 : 2, BKC ? 1 : 2, TA::NV + TB::NV>();
        __syncthreads();
        if constexpr (kSched) __builtin_amdgcn_sched_barrier(0);
        SUB_GEMM_ISSUE(ra1, rb1);                 // tile 2p+3
        SUB_GEMM_COMPUTE(1);
        SUB_GEMM_STORE(0, ra0, rb0);              // tile 2p+2 (a surplus copy when 2p+2 == nkt)
        if constexpr (kSched) sched_k_tile<AKC ? 1 : 2, BKC ? 1 : 2, TA::NV + TB::NV>();
        __syncthreads();
        if constexpr (kSched) __builtin_amdgcn_sched_barrier(0);
    }
    if (nkt & 1) {
        SUB_GEMM_COMPUTE(0);
        __syncthreads();                          // the epilogue reuses the tile memory
    }
#undef SUB_GEMM_COMPUTE
#undef SUB_GEMM_STORE
#undef SUB_GEMM_ISSUE

    if (g.splits > 1) {
        // split k: raw fp32 partial tile, [split][batch][M][N]; a second kernel adds them up
        const long nb_total = nblocks / g.splits / per_batch;
        float* P = g.partial + ((long)split * nb_total + bz) * (long)g.M * g.N;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    int mm = m0 + wm * 32 * TM + i * 32 + l32;
                    int nn = n0 + wn * 32 * TN + j * 32 + q * 8 + hi * 4;
                    if (mm < g.M && nn + 4 <= g.N) {
                        float4 v4 = make_float4(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1],
                                                acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]);
                        *reinterpret_cast<float4*>(P + (long)mm * g.N + nn) = v4;
                    }
                }
        return;
    }
    // Epilogue: per 32-row slab, accumulators -> LDS (8-byte packs of 4
    // consecutive n) -> 16-byte row segments -> global.
    half_t* stage = lds + wave * STAGE_WAVE;
    half_t* Cb = g.C + b0 * g.sCb[0] + b1 * g.sCb[1] + b2 * g.sCb[2];
    const half_t* biasb = g.bias ? g.bias + b0 * g.sbb[0] + b1 * g.sbb[1] + b2 * g.sbb[2] : nullptr;
    constexpr int LPR = 4 * TN;                // lanes per output row (16 bytes each)
    constexpr int RPI = 64 / LPR;              // rows per store instruction
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int mrow = m0 + wm * 32 * TM + i * 32;      // first row of this slab
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                h4 w;
                int ncol = j * 32 + q * 8 + hi * 4;        // within the wave's columns
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (half_t)(acc[i][j][q * 4 + e] * g.alpha);
                *reinterpret_cast<h4*>(stage + l32 * STAGE_PITCH + ncol) = w;
            }
        // LDS operations of one wave execute in order: the reads below see the writes above.
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
            int r = it * RPI + lane / LPR, c8 = (lane % LPR) * 8;
            h8 val = *reinterpret_cast<const h8*>(stage + r * STAGE_PITCH + c8);
            int mm = mrow + r, nn = n0 + wn * 32 * TN + c8;
            if (mm < g.M && nn + 8 <= g.N) {
                if (biasb) {
                    // the addend (a bias row or a whole tensor) is N-contiguous like C
                    h8 ad = *reinterpret_cast<const h8*>(biasb + (long)mm * g.sbM + nn);
                    // the sum of two halves is exact in fp32: the packed half add rounds as the
                    // conversion of that sum would
                    val = val + ad;
                }
                *reinterpret_cast<h8*>(Cb + (long)mm * g.sCM + nn) = val;
            }
        }
    }
}

template <int TM, int TN, bool AKC, bool BKC, bool FULL>
__global__ __launch_bounds__(256) void k_gemm_mfma(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) half_t lds[mfma_lds_halves<TM, TN, AKC, BKC>()];
    gemm_mfma_body<TM, TN, AKC, BKC, FULL>(g, blockIdx.x, gridDim.x, lds);
}

// Two independent products with the same number of 128x128 tiles in one launch,
// eight workgroups of the one, then eight of the other: every XCD and (with about
// one tile per CU each) every CU gets workgroups of both, two per CU, and while
// one of them waits -- for its operands, at its barrier, in its first fetch or
// its output write -- the other one runs.  Alone, each product would leave a
// single wave on every SIMD.
template <bool A1, bool B1, bool A2, bool B2>
__global__ __launch_bounds__(256) void k_gemm_pair(GemmArgs g1, GemmArgs g2, unsigned n1, unsigned n2, GemmArgs g3,
                                                   unsigned n3, FinishJobs tail, unsigned tail_groups) {
    constexpr int L1 = mfma_lds_halves<2, 2, A1, B1>(), L2 = mfma_lds_halves<2, 2, A2, B2>();
    __shared__ __attribute__((aligned(16))) half_t lds[L1 > L2 ? L1 : L2];
    static_assert(sizeof(lds) >= 8 * 33 * sizeof(float) && kFinishThreads == 256, "finish_block needs this much");
    // n1, n2: workgroups of the two products (multiples of 8).  While both have
    // some left they alternate in groups of 8; the rest belongs to the larger one.
    const unsigned b = blockIdx.x, both = 2 * (n1 < n2 ? n1 : n2);
    if (b >= n1 + n2) {
        const unsigned t = b - (n1 + n2);
        if (t < n3) {
            // a third product (n3 workgroups, a multiple of 8, read like the second one)
            // in the places that the pair leaves free with two workgroups per CU
            gemm_mfma_body<2, 2, A2, B2, true>(g3, t, n3, lds);
        } else {
            // Workgroups past the tiles finish column sums of earlier launches: they are
            // dispatched last, into places that tiles leave free or vacate first, and
            // spare the pass a launch of their own.
            finish_block(tail.j[(t - n3) / tail_groups], (t - n3) % tail_groups, reinterpret_cast<float (*)[33]>(lds));
        }
        return;
    }
    if (b < both) {
        const unsigned id = ((b >> 4) << 3) | (b & 7);
        if ((b >> 3) & 1) gemm_mfma_body<2, 2, A2, B2, true>(g2, id, n2, lds);
        else gemm_mfma_body<2, 2, A1, B1, true>(g1, id, n1, lds);
    } else {
        const unsigned id = b - both / 2;
        if (n2 > n1) gemm_mfma_body<2, 2, A2, B2, true>(g2, id, n2, lds);
        else gemm_mfma_body<2, 2, A1, B1, true>(g1, id, n1, lds);
    }
}

// The same with 256 x 128 tiles and one workgroup of eight waves (4 x 2, each 64 x 64 as
// above) per CU, for pairs whose tiles are then about one per CU.  What bounds these
// products is what the L2s deliver to the CUs; the two workgroups that shared a CU each
// fetched their own 128 rows of the second operand, the tall tile fetches them once: a
// quarter less from L2 per flop (dXlin1 + dWlin1 at 4096 x 1024 x 4096 each: 86.5 -> 79.8 us,
// A/B on one device).
template <bool A1, bool B1, bool A2, bool B2>
__global__ __launch_bounds__(512) void k_gemm_pair8(GemmArgs g1, GemmArgs g2, unsigned n1, unsigned n2, GemmArgs g3,
                                                    unsigned n3, FinishJobs tail, unsigned tail_groups) {
    constexpr int L1 = mfma_lds_halves<2, 2, A1, B1, 4>(), L2 = mfma_lds_halves<2, 2, A2, B2, 4>();
    __shared__ __attribute__((aligned(16))) half_t lds[L1 > L2 ? L1 : L2];
    const unsigned b = blockIdx.x, both = 2 * (n1 < n2 ? n1 : n2);
    if (b >= n1 + n2) {
        const unsigned t = b - (n1 + n2);
        if (t < n3) {
            gemm_mfma_body<2, 2, A2, B2, true, 4>(g3, t, n3, lds);
        } else {
            if (threadIdx.x >= kFinishThreads) return;        // a finishing workgroup is four waves
            finish_block(tail.j[(t - n3) / tail_groups], (t - n3) % tail_groups, reinterpret_cast<float (*)[33]>(lds));
        }
        return;
    }
    if (b < both) {
        const unsigned id = ((b >> 4) << 3) | (b & 7);
        if ((b >> 3) & 1) gemm_mfma_body<2, 2, A2, B2, true, 4>(g2, id, n2, lds);
        else gemm_mfma_body<2, 2, A1, B1, true, 4>(g1, id, n1, lds);
    } else {
        const unsigned id = b - both / 2;
        if (n2 > n1) gemm_mfma_body<2, 2, A2, B2, true, 4>(g2, id, n2, lds);
        else gemm_mfma_body<2, 2, A1, B1, true, 4>(g1, id, n1, lds);
    }
}

// ---------------------------------------------------------------------------
// Asynchronous variant for full tiles: global memory -> LDS directly
// (global_load_lds_dwordx4), a ring of S stages, no staging registers and no
// ds_write.  Each wave instruction deposits 64 x 16 bytes at consecutive LDS
// addresses, so the lane -> global-chunk map is chosen such that the bytes land
// in the (bank-swizzled) tile layout the fragment reads expect.  The stages are
// separate __shared__ arrays and the k loop is unrolled over them, which lets
// the compiler see that the fragment reads of one stage do not depend on the
// loads in flight to another; completion is tracked by hand with s_waitcnt
// vmcnt(n) followed by a plain s_barrier.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef __attribute__((address_space(1))) const void* global_void_ptr;

constexpr int waitcnt_vm(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | 0x0F70; }

template <int ROWS, bool KC, int NW>
struct DTile {
    static constexpr int HALVES = ROWS * BK;
    static constexpr int NV = ROWS / (8 * NW);      // loads per thread: the tile is ROWS / 8 slabs of 1024 bytes
    static constexpr int VPR = ROWS / 8;            // 16-byte units per k-row (!KC)

    static __device__ __forceinline__ int kc_off(int row, int slot) {
        return row * BK + ((slot ^ (row ^ (row >> 3))) & 7) * 8;
    }
    // !KC: [k][free] with the 16-byte unit index xor-ed so that the four k-rows a
    // 16-lane group of the transpose read touches fall into different banks.
    static __device__ __forceinline__ int mc_swz(int k) {
        return VPR >= 16 ? ((k & 3) << 2) : (((k >> 1) & 1) << 2);
    }

    // Element offset (from the tile's first element in global memory) of the
    // chunk lane `lane` of wave `wave` fetches with its i-th load.
    static __device__ __forceinline__ void offsets(unsigned (&off)[NV], long sF, long sK, int wave, int lane) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int inst = wave * NV + i;          // which 1024-byte slab of the tile
            if (KC) {
                int row = inst * 8 + (lane >> 3), pslot = lane & 7;
                int lslot = (pslot ^ (row ^ (row >> 3))) & 7;
                off[i] = (unsigned)((long)row * sF + lslot * 8);
            } else {
                constexpr int KPI = 64 / VPR;        // k-rows per instruction
                int k = inst * KPI + lane / VPR, punit = lane % VPR;
                int lunit = punit ^ mc_swz(k);
                off[i] = (unsigned)((long)k * sK + lunit * 8);
            }
        }
    }

    static __device__ __forceinline__ void issue(half_t* stage, const half_t* tile, const unsigned (&off)[NV],
                                                 int wave) {
#pragma unroll
        for (int i = 0; i < NV; ++i)
            __builtin_amdgcn_global_load_lds((global_void_ptr)(tile + off[i]),
                                             (lds_void_ptr)(stage + (wave * NV + i) * 512), 16, 0, 0);
    }

    // KC fragments from one address register per wave and operand: with
    // base = kc_off(row0 + lane % 32, lane / 32) (row0 a multiple of 32), the fragment of the
    // idx-th 32-row block below row0 at k-step ks lies at
    //   (base ^ ((2 ks ^ 4 (idx & 1)) * 8)) + idx * 32 * BK
    // (32 rows further the swizzle flips bit 2 of the slot, a k-step further the slot moves
    // by 2, and neither carries).  The eight-wave kernel computes that inside its loop from a
    // value the compiler cannot see through: left to itself it keeps all 24 addresses of a
    // wave in registers across the loop and spills other things.  (The four-wave kernel has
    // the registers and got slower with it: 40 -> 43 us at M = 4096, N = 1024, K = 4096.)
    static __device__ __forceinline__ int frag_base(int row0, int lane) {
        return kc_off(row0 + (lane & 31), lane >> 5);
    }
    static __device__ __forceinline__ h8 frag_at(const half_t* lds, int base, int idx, int ks) {
        return *reinterpret_cast<const h8*>(lds + ((base ^ (((2 * ks) ^ (4 * (idx & 1))) * 8)) + idx * 32 * BK));
    }

    static __device__ __forceinline__ h8 frag(const half_t* lds, int row0, int ks, int lane) {
        if (KC) {
            return *reinterpret_cast<const h8*>(lds + kc_off(row0 + (lane & 31), ks * 2 + (lane >> 5)));
        } else {
            const int g = lane >> 4, l = lane & 15;
            const int k = ks * 16 + 8 * (g >> 1) + (l >> 2);       // and k + 4 for the second half
            const int m = row0 + 16 * (g & 1) + 4 * (l & 3);
            // k & 3 == (k + 4) & 3 and ((k+4) >> 1) & 1 differs: recompute the swizzle per row
            const half_t* p0 = lds + k * ROWS + (((m >> 3) ^ mc_swz(k)) << 3) + (m & 7);
            const half_t* p1 = lds + (k + 4) * ROWS + (((m >> 3) ^ mc_swz(k + 4)) << 3) + (m & 7);
            typedef s4v __attribute__((address_space(3))) * lds_s4;
            s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(p0));
            s4v hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4)(p1));
            typedef short s8 __attribute__((ext_vector_type(8)));
            s8 r = __builtin_shufflevector(lo, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(h8, r);
        }
    }
};

// Issue order of half a step of the eight-wave kernel: NM matrix instructions with NR
// fragment reads dealt out evenly between them (after FIRST reads in front).
template <int m, int NM, int NR>
__device__ __forceinline__ void sched_mfma_reads_from() {
    if constexpr (m < NM) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int r = (NR * (m + 1)) / NM - (NR * m) / NM;
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
        sched_mfma_reads_from<m + 1, NM, NR>();
    }
}
// NM matrix instructions, each followed by NV vector instructions.
template <int NM, int NV, int m = 0>
__device__ __forceinline__ void sched_mfma_valu() {
    if constexpr (m < NM) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, NV, 0);
        sched_mfma_valu<NM, NV, m + 1>();
    }
}
template <int FIRST, int NM, int NR>
__device__ __forceinline__ void sched_half_step() {
    if constexpr (FIRST > 0) __builtin_amdgcn_sched_group_barrier(0x100, FIRST, 0);
    sched_mfma_reads_from<0, NM, NR>();
}

// NW waves as 2 x (NW / 2); each wave owns TM x TN accumulator tiles of 32 x 32.
// Eight waves (two per SIMD) on a 256 x 256 tile: a wave cannot issue past an
// asynchronous load that the memory path has not accepted yet, and with all 256 CUs
// drawing on L2 that takes long (measured: the loads of a step alone cost about as
// much time as its multiplications, and with one wave per SIMD the two add up);
// while one wave of a SIMD sits in the issue of its loads the other multiplies.
// EPI: what the epilogue does after the scaling and the optional addend.  A template
// parameter so that the plain kernel does not carry the registers of the others.
// EPI_RELU_DROPOUT_PRE: EPI_RELU_DROPOUT with the keep bits drawn ahead of the launch (GemmEpilogue::keep_words)
// EPI_GELU_DROPOUT: as EPI_RELU_DROPOUT with GELU; also stores the rounded sum before the activation
// (GemmArgs::pre_out, which the backward pass needs) and leaves the keep bits where the ReLU form leaves its gate bits.
// EPI_GELU_GATE_COLSUM: the backward counterpart: out = keep bit ? gelu'(pre-activation) * product : 0, and column sums.
enum { EPI_PLAIN = 0, EPI_RELU_DROPOUT = 1, EPI_GATE_COLSUM = 2, EPI_RELU_DROPOUT_PRE = 3, EPI_GELU_DROPOUT = 4,
       EPI_GELU_GATE_COLSUM = 5 };

template <int TM, int TN, bool AKC, bool BKC, int S, int NW, int EPI = EPI_PLAIN>
__global__ __launch_bounds__(NW * 64) void k_gemm_dma(GemmArgs g) {
    static_assert(S == 2 || S == 3, "two or three LDS stages");
    static_assert(NW == 4 || NW == 8, "four or eight waves");
    constexpr int WN = NW / 2;
    constexpr int BM = 64 * TM, BN = 32 * TN * WN;
    using TA = DTile<BM, AKC, NW>;
    using TB = DTile<BN, BKC, NW>;
    constexpr int STAGE = TA::HALVES + TB::HALVES;
    constexpr int STAGE_PITCH = 32 * TN + 8;
    constexpr int STAGE_WAVE = 32 * STAGE_PITCH;
    static_assert(NW * STAGE_WAVE <= STAGE, "epilogue staging must fit one stage");
    // one array per stage: the compiler then sees that an asynchronous load into one
    // stage does not alias the fragment reads from another, and adds no waits of its own
    __shared__ __attribute__((aligned(16))) half_t st0[STAGE];
    __shared__ __attribute__((aligned(16))) half_t st1[STAGE];
    __shared__ __attribute__((aligned(16))) half_t st2[S > 2 ? STAGE : 8];
    constexpr int L = TA::NV + TB::NV;               // loads per thread per tile

    // (the wave index as a scalar: LDS destinations of the asynchronous loads are then scalar arithmetic)
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, hi = lane >> 5;

    fetch_gemm_args(g);
    const int tiles_m = g.M / BM, tiles_n = g.N / BN;
    unsigned lid = blockIdx.x;
    {
        unsigned nblocks = gridDim.x;
        if constexpr (NW == 8 && EPI == EPI_PLAIN) {
            if (g.side_blocks) {
                if (blockIdx.x >= g.side_first) { side_block(g, blockIdx.x - g.side_first, g.side_blocks); return; }
                nblocks = g.side_first;
            }
        }
        if ((nblocks & 7) == 0) lid = (lid & 7u) * (nblocks >> 3) + (lid >> 3);
    }
    // (32-bit arithmetic, as in the register-staged kernel)
    const unsigned per_batch = (unsigned)(tiles_m * tiles_n);
    const unsigned bz = lid / per_batch;
    int r = (int)(lid - bz * per_batch);
    constexpr int GM = 8;
    const int grp = r / (GM * tiles_n), first_m = grp * GM;
    const int gsz = tiles_m - first_m < GM ? tiles_m - first_m : GM;
    const int rr = r - grp * GM * tiles_n;
    const int tile_m = first_m + rr % gsz, tile_n = rr / gsz;
    const unsigned tq = bz / (unsigned)g.nb2;
    const long b2 = bz - tq * (unsigned)g.nb2, b0 = tq / (unsigned)g.nb1, b1 = tq - (unsigned)b0 * (unsigned)g.nb1;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    // (the tile pointers are the same for every lane: kept in scalar registers, a load's address is
    // scalar base + 32-bit lane offset instead of a 64-bit vector addition per load)
    auto uniform = [](const half_t* p) {
        const uint64_t v = reinterpret_cast<uint64_t>(p);
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        const uint32_t hi2 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
        return reinterpret_cast<const half_t*>(((uint64_t)hi2 << 32) | lo);
    };
    const half_t* pa = uniform(g.A + b0 * g.sAb[0] + b1 * g.sAb[1] + b2 * g.sAb[2] + (long)m0 * g.sAM);
    const half_t* pb = uniform(g.B + b0 * g.sBb[0] + b1 * g.sBb[1] + b2 * g.sBb[2] + (long)n0 * g.sBN);

    const int tiles_per_k1 = g.K1 / BK;
    const int nkt = g.K0 * tiles_per_k1;

    f16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    unsigned offa[TA::NV], offb[TB::NV];
    TA::offsets(offa, g.sAM, g.sAK1, wave, lane);
    TB::offsets(offb, g.sBN, g.sBK1, wave, lane);

    int kin = 0, fetched = 0;
    const long stepA = (long)BK * g.sAK1, stepB = (long)BK * g.sBK1;
    const long wrapA = g.sAK0 - (long)(tiles_per_k1 - 1) * stepA;
    const long wrapB = g.sBK0 - (long)(tiles_per_k1 - 1) * stepB;

    // Fetch the next k-tile into `stage`; past the last tile the pointers stay put
    // (surplus fetches re-read valid memory and keep the vmcnt bookkeeping uniform).
#define SUB_DMA_ISSUE(stage_)                                                                     \
    do {                                                                                          \
        TA::issue(stage_, pa, offa, wave);                                                        \
        TB::issue(stage_ + TA::HALVES, pb, offb, wave);                                           \
        const bool more_ = fetched + 1 < nkt;                                                     \
        const bool wrap_ = kin + 1 == tiles_per_k1;                                               \
        pa += more_ ? (wrap_ ? wrapA : stepA) : 0;                                                \
        pb += more_ ? (wrap_ ? wrapB : stepB) : 0;                                                \
        kin = more_ ? (wrap_ ? 0 : kin + 1) : kin;                                                \
        fetched += more_ ? 1 : 0;                                                                 \
    } while (0)

    // ReLU-dropout epilogue: the keep bits of the 16 packs of 8 outputs this lane stores are
    // drawn during the multiplication, one Philox call per step, where the vector unit is
    // otherwise idle; the epilogue only picks its byte.  Pack c (0..15) covers output row
    // (first row of the wave) + 8 c + lane / 8, so its group of 8 canonical elements is
    // kb_group0 + c * sCM.  Every step shifts the 128 bits up by a byte and draws pack
    // (kb_next & 15); the start is chosen so that the last 16 steps draw packs 0..15 in order.
    constexpr int LPR = 4 * TN;                      // lanes per output row of the wave's slab
    constexpr int RPI = 64 / LPR;                    // rows per store instruction
    constexpr bool DRAWS = EPI == EPI_RELU_DROPOUT || EPI == EPI_GELU_DROPOUT;    // keep bits drawn in the main loop
    static_assert(!DRAWS || TM * (32 / RPI) == 16, "16 packs of keep bits per lane");
    PhiloxKey rd_key = g.key;
    uint32_t kb[4] = {0u, 0u, 0u, 0u};
    uint64_t kb_group0 = 0;
    int kb_next = 0;
    if (DRAWS) {
        rd_key = resolved(g.key);
        const uint64_t row = (uint64_t)(m0 + wm * 32 * TM + lane / LPR);
        kb_group0 = (row * (uint64_t)g.sCM + (uint64_t)(n0 + wn * 32 * TN + (lane % LPR) * 8)) >> 3;
        kb_next = nkt >= 16 ? (16 - (nkt & 15)) & 15 : 0;
    }
#define SUB_DMA_KEEP()                                                                            \
    do {                                                                                          \
        const U4 r_ = philox_group(rd_key, kb_group0 + (uint64_t)(kb_next & 15) * (uint64_t)g.sCM); \
        const uint32_t b_ = keep8(r_, rd_key.thr);                                                \
        kb[3] = (kb[3] << 8) | (kb[2] >> 24);                                                     \
        kb[2] = (kb[2] << 8) | (kb[1] >> 24);                                                     \
        kb[1] = (kb[1] << 8) | (kb[0] >> 24);                                                     \
        kb[0] = (kb[0] << 8) | b_;                                                                \
        ++kb_next;                                                                                \
    } while (0)

    // What the epilogue reads besides the accumulators is requested here, ahead of the contraction: behind it the
    // round trip to memory would stand in the open (the loads complete in order, ahead of the tiles').
    half_t* Cb = g.C + b0 * g.sCb[0] + b1 * g.sCb[1] + b2 * g.sCb[2];
    const half_t* biasb = g.bias ? g.bias + b0 * g.sbb[0] + b1 * g.sbb[1] + b2 * g.sbb[2] : nullptr;
    // a bias row (the same for every row of the output): a lane's 8 columns are the same in all of its
    // packs, so it loads them once instead of before every store
    const bool bias_row = biasb && g.sbM == 0;
    h8 bias8 = (h8)(half_t)0.0f;
    if (bias_row) bias8 = *reinterpret_cast<const h8*>(biasb + n0 + wn * 32 * TN + (lane % LPR) * 8);
    // One bit per output of the ReLU-dropout epilogue (set = positive), a dword per lane and 32-row
    // slab in the order this epilogue walks the tile: the gate epilogue of a product with the same
    // output shape reads 1/16 of what the outputs themselves would cost it.
    constexpr bool RELU_DROP = EPI == EPI_RELU_DROPOUT || EPI == EPI_RELU_DROPOUT_PRE;
    constexpr bool GELU_DROP = EPI == EPI_GELU_DROPOUT;
    constexpr bool GATED = EPI == EPI_GATE_COLSUM || EPI == EPI_GELU_GATE_COLSUM;
    static_assert(EPI == EPI_PLAIN || 32 / RPI == 4, "four packs of 8 outputs per lane and slab");
    const long bits_at = (((long)tile_m * tiles_n + tile_n) * NW + wave) * (TM * 64) + lane;
    uint32_t gbits[TM];
    if (GATED && g.gate_bits) {
#pragma unroll
        for (int i = 0; i < TM; ++i) gbits[i] = g.gate_bits[bits_at + i * 64];
    }

    constexpr int RA_ = AKC ? 1 : 2, RB_ = BKC ? 1 : 2;      // LDS reads per fragment
    const int fbase_a = TA::frag_base(wm * TM * 32, lane), fbase_b = TB::frag_base(wn * TN * 32, lane);
#define SUB_DMA_FRAG_A(i_, ks_) (AKC && NW == 8 ? TA::frag_at(sA, ba_, i_, ks_) : TA::frag(sA, (wm * TM + (i_)) * 32, ks_, lane))
#define SUB_DMA_FRAG_B(j_, ks_) (BKC && NW == 8 ? TB::frag_at(sB, bb_, j_, ks_) : TB::frag(sB, (wn * TN + (j_)) * 32, ks_, lane))
#define SUB_DMA_COMPUTE(stage_, nx_)                                                              \
    do {                                                                                          \
        const half_t* sA = stage_;                                                                \
        const half_t* sB = stage_ + TA::HALVES;                                                   \
        h8 fa[2][TM], fb[2][TN];                                                                  \
        int ba_ = fbase_a, bb_ = fbase_b;                                                         \
        if constexpr (NW == 8) asm volatile("" : "+v"(ba_), "+v"(bb_));                           \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                                            \
            fa[0][i] = SUB_DMA_FRAG_A(i, 0);                                                      \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                            \
            fb[0][j] = SUB_DMA_FRAG_B(j, 0);                                                      \
        _Pragma("unroll") for (int ks = 0; ks < BK / 16; ++ks) {                                  \
            if (NW == 8 && ks == BK / 32) {                                                       \
                /* first half: the reads of k-slices 1 and 2 between the products of 0 and 1 */   \
                sched_half_step<TM * RA_ + TN * RB_, 2 * TM * TN, 2 * (TM * RA_ + TN * RB_)>();   \
                if (late) SUB_DMA_ISSUE(nx_);                                                     \
                __builtin_amdgcn_sched_barrier(0);                                                \
            }                                                                                     \
            if (NW == 8 && DRAWS && ks == BK / 16 - 1) {                                          \
                /* the last k-slice shares its issue slots with the keep bits: the fragments of  \
                   the slice before are dead by now, so the draw costs no registers */           \
                sched_half_step<0, TM * TN, TM * RA_ + TN * RB_>();                               \
                __builtin_amdgcn_sched_barrier(0);                                                \
                SUB_DMA_KEEP();                                                                   \
            }                                                                                     \
            if (ks + 1 < BK / 16) {                                                               \
                _Pragma("unroll") for (int i = 0; i < TM; ++i)                                    \
                    fa[(ks + 1) & 1][i] = SUB_DMA_FRAG_A(i, ks + 1);                              \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                    \
                    fb[(ks + 1) & 1][j] = SUB_DMA_FRAG_B(j, ks + 1);                              \
            }                                                                                     \
            _Pragma("unroll") for (int i = 0; i < TM; ++i)                                        \
                _Pragma("unroll") for (int j = 0; j < TN; ++j)                                    \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ks & 1][j], fa[ks & 1][i], \
                                                                       acc[i][j], 0, 0, 0);       \
        }                                                                                         \
        /* second half: the reads of k-slice 3 between the products of k-slice 2 */               \
        if constexpr (NW == 8 && !DRAWS)                                                          \
            sched_half_step<0, 2 * TM * TN, TM * RA_ + TN * RB_>();                               \
        if constexpr (NW == 8 && DRAWS) sched_mfma_valu<TM * TN, 12>();                           \
    } while (0)

    // One step: tile kt is complete once at most the L loads of tile kt+1 are
    // outstanding; the barrier also says every wave is done reading the stage
    // that the fetch below overwrites (it was computed on one step earlier).
#define SUB_DMA_STEP(cur_, nxt2_)                                                                 \
    do {                                                                                          \
        __builtin_amdgcn_s_waitcnt(waitcnt_vm((S - 2) * L));                                      \
        __builtin_amdgcn_s_barrier();                                                             \
        if (!late) SUB_DMA_ISSUE(nxt2_);                                                          \
        /* keep the fetches ahead of the multiply phase: the scheduler must not sink them */      \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SUB_DMA_COMPUTE(cur_, nxt2_);                                                            \
    } while (0)

    // Eight waves: the second wave of each SIMD issues its loads half a step after
    // the first, so that the two are not held up in the issue at the same time.
    const bool late = NW == 8 && __builtin_amdgcn_readfirstlane(wave) >= 4;
    // S stages: while tile kt is multiplied, tiles kt+1 .. kt+S-2 are landed or on
    // their way and the fetch of tile kt+S-1 goes into the stage of tile kt-1.
    // (One array per stage and each round of S steps as straight-line code: with one
    // array for the ring, or the steps behind conditions of their own, the compiler
    // no longer sees which stage a fragment read touches and waits for every load
    // in flight before it.  More than three stages of 128 x 128 tiles gained nothing.)
    if (S == 2) {
        SUB_DMA_ISSUE(st0);
        const int nr = nkt / 2;
        for (int p = 0; p < nr; ++p) {
            SUB_DMA_STEP(st0, st1);
            SUB_DMA_STEP(st1, st0);
        }
        if (nkt & 1) SUB_DMA_STEP(st0, st1);
    } else if (S == 3) {
        SUB_DMA_ISSUE(st0);
        SUB_DMA_ISSUE(st1);
        const int nr = nkt / 3, rem = nkt - 3 * nr;
        for (int p = 0; p < nr; ++p) {
            SUB_DMA_STEP(st0, st2);
            SUB_DMA_STEP(st1, st0);
            SUB_DMA_STEP(st2, st1);
        }
        if (rem >= 1) SUB_DMA_STEP(st0, st2);
        if (rem >= 2) SUB_DMA_STEP(st1, st0);
    }
    if (DRAWS)
        for (int c = nkt; c < 16; ++c) SUB_DMA_KEEP();        // a contraction shorter than 16 steps
#undef SUB_DMA_STEP
#undef SUB_DMA_COMPUTE
#undef SUB_DMA_FRAG_A
#undef SUB_DMA_FRAG_B
#undef SUB_DMA_KEEP
#undef SUB_DMA_ISSUE
    // surplus fetches may still be landing: drain them before LDS is reused
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();

    half_t* stage = st0 + wave * STAGE_WAVE;
    float colsum[8];              // gate mode: this lane's 8 columns summed over its rows of the wave's slab
#pragma unroll
    for (int e = 0; e < 8; ++e) colsum[e] = 0.f;
    if (EPI == EPI_RELU_DROPOUT_PRE) {
        const uint4 w = reinterpret_cast<const uint4*>(g.keep_words)[(((long)tile_m * tiles_n + tile_n) * NW + wave) * 64 + lane];
        kb[0] = w.x; kb[1] = w.y; kb[2] = w.z; kb[3] = w.w;
    }
    // The lane's stores walk down the tile RPI rows at a time: running pointers (a 64-bit product
    // per store otherwise), and one copy of the loop per kind of addend (none, a bias row, a tensor:
    // chosen per store, the branches joined in a wait for every store issued so far).  Most products
    // have alpha = 1: no multiplication then.
    const bool alpha_one = g.alpha == 1.0f;
    const long c_step = (long)RPI * g.sCM, b_step = (long)RPI * g.sbM;
    const int row_first = m0 + wm * 32 * TM + lane / LPR, col_first = n0 + wn * 32 * TN + (lane % LPR) * 8;
    half_t* const c_first = Cb + (long)row_first * g.sCM + col_first;
    const long b_first = (long)row_first * g.sbM + col_first;        // addend and gate share their strides
    auto store_tile = [&](auto addend_kind) {
        constexpr int ADD = decltype(addend_kind)::value;           // 0 none, 1 a bias row, 2 a tensor
        half_t* cp = c_first;
        const half_t* bp = ADD == 2 ? biasb + b_first : nullptr;
        // (the GELU form reads the pre-activation values there, and the keep bits besides)
        const half_t* gp = (EPI == EPI_GELU_GATE_COLSUM || (EPI == EPI_GATE_COLSUM && !g.gate_bits)) ? g.gate + b_first : nullptr;
        half_t* lp = GELU_DROP ? g.pre_out + (c_first - Cb) : nullptr;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            uint32_t positive = 0;
            if (alpha_one) {
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        h4 w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = (half_t)acc[i][j][q * 4 + e];
                        *reinterpret_cast<h4*>(stage + l32 * STAGE_PITCH + j * 32 + q * 8 + hi * 4) = w;
                    }
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        h4 w;
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = (half_t)(acc[i][j][q * 4 + e] * g.alpha);
                        *reinterpret_cast<h4*>(stage + l32 * STAGE_PITCH + j * 32 + q * 8 + hi * 4) = w;
                    }
            }
#pragma unroll
            for (int it = 0; it < 32 / RPI; ++it) {
                const int rr2 = it * RPI + lane / LPR, c8 = (lane % LPR) * 8;
                h8 val = *reinterpret_cast<const h8*>(stage + rr2 * STAGE_PITCH + c8);
                // packed half add: the same single rounding as through fp32
                if (ADD == 1) val = val + bias8;
                if (ADD == 2) val = val + *reinterpret_cast<const h8*>(bp);
                if (EPI == EPI_GATE_COLSUM) {
                    // the ReLU layer's backward-dropout-activation: zero where the forward output was not positive
                    if (g.gate_bits) {
                        const uint32_t bits = gbits[i] >> (8 * it);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            val[e] = ((bits >> e) & 1u) ? val[e] : (half_t)0.0f;
                            colsum[e] += (float)val[e];
                        }
                    } else {
                        const h8 gt = *reinterpret_cast<const h8*>(gp);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            val[e] = (float)gt[e] > 0.f ? val[e] : (half_t)0.0f;
                            colsum[e] += (float)val[e];
                        }
                    }
                }
                if (EPI == EPI_GELU_GATE_COLSUM) {
                    // the GELU layer's backward-dropout-activation, as the operator computes it
                    const uint32_t bits = gbits[i] >> (8 * it);
                    const h8 lin = *reinterpret_cast<const h8*>(gp);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        // (computed for every element and then selected: no branch per element)
                        const float gv = gelu_bwd((float)lin[e], (float)val[e]);
                        val[e] = ((bits >> e) & 1u) ? (half_t)gv : (half_t)0.0f;
                        colsum[e] += (float)val[e];
                    }
                }
                if (GELU_DROP) {
                    *reinterpret_cast<h8*>(lp) = val;              // the pre-activation, for the backward pass
                    lp += c_step;
                    const int c = i * (32 / RPI) + it, byte = 15 - c;
                    const uint32_t bits = kb[byte >> 2] >> ((byte & 3) * 8);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float gv = gelu_fwd((float)val[e]);       // for every element, then selected: no branches
                        val[e] = ((bits >> e) & 1u) ? (half_t)gv : (half_t)0.0f;
                    }
                    positive |= (bits & 0xffu) << (8 * it);        // here: the keep bits
                }
                if (RELU_DROP) {
                    // what the bias-activation-dropout operator does to the rounded sum, with the
                    // same keep bits (the element index is the offset into the dense output):
                    // pack c sits in byte 15 - c of the bits drawn in the main loop
                    const int c = i * (32 / RPI) + it, byte = 15 - c;
                    const uint32_t bits = kb[byte >> 2] >> ((byte & 3) * 8);
                    val = __builtin_elementwise_max(val, (h8)(half_t)0.0f);       // ReLU, packed
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        val[e] = ((bits >> e) & 1u) ? val[e] : (half_t)0.0f;
                        positive |= (val[e] > (half_t)0.0f ? 1u : 0u) << (8 * it + e);
                    }
                }
                *reinterpret_cast<h8*>(cp) = val;
                cp += c_step;
                if (ADD == 2) bp += b_step;
                if (GATED) gp += b_step;
            }
            if ((RELU_DROP || GELU_DROP) && g.gate_bits_out) g.gate_bits_out[bits_at + i * 64] = positive;
        }
    };
    if (GATED || !biasb) store_tile(std::integral_constant<int, 0>{});     // (a gated product has no addend)
    else if (bias_row) store_tile(std::integral_constant<int, 1>{});
    else store_tile(std::integral_constant<int, 2>{});
    if (GATED) {
        // lanes LPR apart hold the same 8 columns for other rows: add them up, then one fp32
        // row of partial sums per 128-row slab of the output (a finishing launch adds the slabs)
#pragma unroll
        for (int o = LPR; o < 64; o <<= 1)
#pragma unroll
            for (int e = 0; e < 8; ++e) colsum[e] += __shfl_xor(colsum[e], o);
        if (lane < LPR) {
            float* dst = g.colsum + ((long)tile_m * 2 + wm) * g.N + n0 + wn * 32 * TN + lane * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) dst[e] = colsum[e];
        }
    }
}

// Adds the k-split partials: C[b,m,n] = fp16(alpha * sum_s P[s][b][m][n]) (+ addend).
__device__ __forceinline__ void splitk_sum_block(const GemmArgs& g, long nb_total, long block) {
    const long quads = (long)g.N / 4;
    long idx = block * 256 + threadIdx.x;
    if (idx >= nb_total * g.M * quads) return;
    int nq = (int)(idx % quads); long rr = idx / quads;
    int m = (int)(rr % g.M); long bz = rr / g.M;
    const long slab = nb_total * (long)g.M * g.N;
    const float* p = g.partial + (bz * g.M + m) * (long)g.N + nq * 4;
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 v[8];                  // at most 8 splits: all loads in flight at once
#pragma unroll
    for (int s = 0; s < 8; ++s)
        v[s] = s < g.splits ? *reinterpret_cast<const float4*>(p + (long)s * slab) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int s = 0; s < 8; ++s) { t.x += v[s].x; t.y += v[s].y; t.z += v[s].z; t.w += v[s].w; }
    long b2 = bz % g.nb2; long tt = bz / g.nb2;
    long b1 = tt % g.nb1; long b0 = tt / g.nb1;
    half_t* c = g.C + b0 * g.sCb[0] + b1 * g.sCb[1] + b2 * g.sCb[2] + (long)m * g.sCM + nq * 4;
    h4 o;
    o[0] = (half_t)(t.x * g.alpha); o[1] = (half_t)(t.y * g.alpha);
    o[2] = (half_t)(t.z * g.alpha); o[3] = (half_t)(t.w * g.alpha);
    if (g.bias) {
        const half_t* ad = g.bias + b0 * g.sbb[0] + b1 * g.sbb[1] + b2 * g.sbb[2] + (long)m * g.sbM + nq * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (half_t)((float)o[e] + (float)ad[e]);
    }
    *reinterpret_cast<h4*>(c) = o;
}

__global__ __launch_bounds__(256) void k_gemm_splitk_reduce(GemmArgs g, long nb_total) {
    splitk_sum_block(g, nb_total, blockIdx.x);
}

inline bool mult8(long x) { return (x & 7) == 0; }
inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Canonical form: C contiguous along N (swap the operands otherwise).
struct Canon {
    GemmArgs a;
    bool ok_c;       // C has a unit stride along N after canonicalisation
};

Canon canonicalise(const GemmShape& s, const half_t* A, const half_t* B, half_t* C, float alpha,
                   const GemmEpilogue& ep) {
    Canon c;
    GemmArgs& a = c.a;
    const bool swap = s.sCN != 1 && s.sCM == 1;
    if (!swap) {
        a.A = A; a.B = B; a.M = (int)s.M; a.N = (int)s.N;
        a.sAM = s.sAM; a.sAK1 = s.sAK1; a.sAK0 = s.sAK0;
        a.sBN = s.sBN; a.sBK1 = s.sBK1; a.sBK0 = s.sBK0;
        a.sCM = s.sCM; a.sCN = s.sCN;
        for (int i = 0; i < 3; ++i) { a.sAb[i] = s.sAb[i]; a.sBb[i] = s.sBb[i]; }
        a.sbM = ep.sbM; a.sbN = ep.sbN;
    } else {
        a.A = B; a.B = A; a.M = (int)s.N; a.N = (int)s.M;
        a.sAM = s.sBN; a.sAK1 = s.sBK1; a.sAK0 = s.sBK0;
        a.sBN = s.sAM; a.sBK1 = s.sAK1; a.sBK0 = s.sAK0;
        a.sCM = s.sCN; a.sCN = s.sCM;
        for (int i = 0; i < 3; ++i) { a.sAb[i] = s.sBb[i]; a.sBb[i] = s.sAb[i]; }
        a.sbM = ep.sbN; a.sbN = ep.sbM;
    }
    a.C = C; a.K1 = (int)s.K1; a.K0 = (int)s.K0;
    a.nb1 = (int)s.nb[1]; a.nb2 = (int)s.nb[2];
    for (int i = 0; i < 3; ++i) { a.sCb[i] = s.sCb[i]; a.sbb[i] = ep.sbb[i]; }
    a.alpha = alpha; a.bias = ep.bias;
    a.relu_dropout = ep.relu_dropout ? 1 : 0; a.key = ep.key;
    a.gate = ep.gate; a.colsum = ep.colsum; a.gate_bits_out = ep.gate_bits_out; a.gate_bits = ep.gate_bits;
    a.keep_words = ep.keep_words; a.act = ep.act; a.pre_out = ep.pre_out;
    a.splits = 1; a.partial = nullptr;
    c.ok_c = a.sCN == 1;
    return c;
}

// 0 = scalar, 1 = MFMA
int pick_kind(const Canon& c, bool& akc, bool& bkc) {
    const GemmArgs& a = c.a;
    if (!c.ok_c) return 0;
    if (a.M <= 0 || a.N <= 0 || a.K1 <= 0) return 0;
    akc = a.sAK1 == 1; bkc = a.sBK1 == 1;
    if (!akc && a.sAM != 1) return 0;
    if (!bkc && a.sBN != 1) return 0;
    if (!al16(a.A) || !al16(a.B) || !al16(a.C)) return 0;
    if (a.K0 > 1 && a.K1 % BK != 0) return 0;
    if (a.bias && !(a.sbN == 1 && mult8(a.sbM) && mult8(a.sbb[0]) && mult8(a.sbb[1]) && mult8(a.sbb[2]) &&
                    al16(a.bias)))
        return 0;
    if (a.gate && !(a.sbN == 1 && mult8(a.sbM) && al16(a.gate) && !a.bias && a.colsum)) return 0;
    // GELU: the backward form needs the keep bits, the forward form a place for the pre-activation and for those bits
    if (a.act == ACT_GELU && a.gate && !a.gate_bits) return 0;
    if (a.act == ACT_GELU && a.relu_dropout && !(a.pre_out && al16(a.pre_out) && a.gate_bits_out && !a.keep_words)) return 0;
    // every 16-byte access must be aligned and whole
    bool ok = mult8(a.N) && mult8(a.sCM) && mult8(a.sCb[0]) && mult8(a.sCb[1]) && mult8(a.sCb[2]);
    ok = ok && mult8(a.sAK0) && mult8(a.sAb[0]) && mult8(a.sAb[1]) && mult8(a.sAb[2]);
    ok = ok && mult8(a.sBK0) && mult8(a.sBb[0]) && mult8(a.sBb[1]) && mult8(a.sBb[2]);
    if (akc) ok = ok && mult8(a.K1) && mult8(a.sAM); else ok = ok && mult8(a.M) && mult8(a.sAK1);
    if (bkc) ok = ok && mult8(a.K1) && mult8(a.sBN); else ok = ok && mult8(a.N) && mult8(a.sBK1);
    return ok ? 1 : 0;
}

// Block tile for a problem: 22 = 128x128, 44 = 256x256, 21 = 128x64.
int pick_tile(const GemmArgs& a, long batch, bool akc, bool bkc) {
    if (a.N <= 64) return 21;      // head-size wide outputs of the attention products
    // 256x256 tiles halve the L2->LDS traffic per flop; they pay once the output
    // alone has enough of them to keep most of the 256 CUs busy in every round of
    // tiles (asynchronous kernel only: whole tiles, no split contraction).  With
    // an operand that is read through the slower LDS transpose path the bar is
    // higher: three quarters of a round is not enough then (measured).
    if (a.M % 256 == 0 && a.N % 256 == 0 && a.K1 % BK == 0 && a.splits == 1) {
        const long tiles = (long)(a.M / 256) * (a.N / 256) * batch;
        const long rounds = (tiles + 255) / 256;
        const double fill = (double)tiles / (double)(rounds * 256);
        if (fill >= ((akc && bkc) ? 0.7 : 0.9)) return 44;
    }
    return 22;
}

template <int TM, int TN, bool FULL>
void launch_mfma2(const GemmArgs& a, bool akc, bool bkc, dim3 grid, hipStream_t st) {
    if (akc && bkc) hipLaunchKernelGGL((k_gemm_mfma<TM, TN, true, true, FULL>), grid, dim3(256), 0, st, a);
    else if (akc) hipLaunchKernelGGL((k_gemm_mfma<TM, TN, true, false, FULL>), grid, dim3(256), 0, st, a);
    else if (bkc) hipLaunchKernelGGL((k_gemm_mfma<TM, TN, false, true, FULL>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((k_gemm_mfma<TM, TN, false, false, FULL>), grid, dim3(256), 0, st, a);
}

template <int TM, int TN, int S, int NW, int EPI>
void launch_dma3(const GemmArgs& a, bool akc, bool bkc, dim3 grid, hipStream_t st) {
    if (akc && bkc) hipLaunchKernelGGL((k_gemm_dma<TM, TN, true, true, S, NW, EPI>), grid, dim3(NW * 64), 0, st, a);
    else if (akc) hipLaunchKernelGGL((k_gemm_dma<TM, TN, true, false, S, NW, EPI>), grid, dim3(NW * 64), 0, st, a);
    else if (bkc) hipLaunchKernelGGL((k_gemm_dma<TM, TN, false, true, S, NW, EPI>), grid, dim3(NW * 64), 0, st, a);
    else hipLaunchKernelGGL((k_gemm_dma<TM, TN, false, false, S, NW, EPI>), grid, dim3(NW * 64), 0, st, a);
}

template <int TM, int TN, int S, int NW>
void launch_dma2(const GemmArgs& a, bool akc, bool bkc, dim3 grid, hipStream_t st) {
    if (a.relu_dropout || a.gate) {
        // only the eight-wave 256x256 kernel carries these epilogues
        if constexpr (NW == 8) {
            if (a.gate && a.act == ACT_GELU) launch_dma3<TM, TN, S, NW, EPI_GELU_GATE_COLSUM>(a, akc, bkc, grid, st);
            else if (a.gate) launch_dma3<TM, TN, S, NW, EPI_GATE_COLSUM>(a, akc, bkc, grid, st);
            else if (a.act == ACT_GELU) launch_dma3<TM, TN, S, NW, EPI_GELU_DROPOUT>(a, akc, bkc, grid, st);
            else if (a.keep_words) launch_dma3<TM, TN, S, NW, EPI_RELU_DROPOUT_PRE>(a, akc, bkc, grid, st);
            else launch_dma3<TM, TN, S, NW, EPI_RELU_DROPOUT>(a, akc, bkc, grid, st);
            return;
        } else {
            fail("gemm: this kernel variant has no ReLU-dropout or gate epilogue");
        }
    }
    launch_dma3<TM, TN, S, NW, EPI_PLAIN>(a, akc, bkc, grid, st);
}

template <int TM, int TN>
void launch_dma(const GemmArgs& a, bool akc, bool bkc, dim3 grid, hipStream_t st) {
    if constexpr (TM * TN >= 16) {                    // 256x256 tiles: two 64 KiB stages, eight waves
        launch_dma2<TM, TN / 2, 2, 8>(a, akc, bkc, grid, st);
    } else {
        launch_dma2<TM, TN, 3, 4>(a, akc, bkc, grid, st);
    }
}

template <int TM, int TN, bool DMA_OK>
void launch_mfma(const GemmArgs& a, bool akc, bool bkc, long batch, bool dma, hipStream_t st) {
    long nblocks = (long)((a.N + 64 * TN - 1) / (64 * TN)) * ((a.M + 64 * TM - 1) / (64 * TM)) * batch *
                   a.splits;
    if (nblocks > 0x7fffffffL) fail("gemm: too many tiles");
    dim3 grid((unsigned)nblocks + a.side_blocks);
    const bool full = a.M % (64 * TM) == 0 && a.N % (64 * TN) == 0 && a.K1 % BK == 0;
    if (DMA_OK && full && dma && a.splits == 1) { launch_dma<TM, TN>(a, akc, bkc, grid, st); return; }
    if constexpr (TM * TN >= 16) {
        // 256 x 256 tiles exist in the asynchronous kernel only; pick_tile chooses them for whole tiles alone
        fail("gemm: 256x256 tiles need whole tiles and an unsplit contraction");
    } else {
        if (full) launch_mfma2<TM, TN, true>(a, akc, bkc, grid, st);
        else launch_mfma2<TM, TN, false>(a, akc, bkc, grid, st);
    }
    if (a.splits > 1) {
        long n = batch * (long)a.M * (a.N / 4);
        hipLaunchKernelGGL(k_gemm_splitk_reduce, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, batch);
    }
}

constexpr size_t kSplitMaxOut = 2u << 20;     // largest output (elements) whose contraction is split
constexpr long kSplitTarget = 256;            // workgroups a split product aims for (the CUs of the device)

// How many ways to split k so that a small output still fills the chip: the
// weight-gradient products have few output tiles and a long contraction.
int pick_splits(const GemmArgs& a, long batch, size_t ws_floats) {
    const long tiles = (long)((a.M + 127) / 128) * ((a.N + 127) / 128) * batch;
    const int nkt = a.K0 * ((a.K1 + BK - 1) / BK);
    // one workgroup per CU: a second, partly filled round costs more than it gains
    int splits = (int)(kSplitTarget / tiles);
    if (splits > 8) splits = 8;
    while (splits > 1 && nkt / splits < 8) --splits;
    const size_t need = (size_t)batch * a.M * a.N;          // floats per split
    while (splits > 1 && need * splits > ws_floats) --splits;
    if (a.N % 4 != 0) splits = 1;
    return splits < 1 ? 1 : splits;
}

}  // namespace

int gemm_kernel_kind(const GemmShape& s, const void* A, const void* B, const void* C,
                     const GemmEpilogue& ep) {
    Canon c = canonicalise(s, (const half_t*)A, (const half_t*)B, (half_t*)C, 1.f, ep);
    bool akc, bkc;
    return pick_kind(c, akc, bkc);
}

bool gemm_relu_dropout_ok(const GemmShape& s, const void* A, const void* B, const void* C,
                          const GemmEpilogue& ep) {
    if (s.batch() != 1 || s.sCN != 1 || s.sCM != s.N) return false;       // one dense row-major output
    Canon c = canonicalise(s, (const half_t*)A, (const half_t*)B, (half_t*)C, 1.f, ep);
    bool akc, bkc;
    return pick_kind(c, akc, bkc) == 1 && pick_tile(c.a, 1, akc, bkc) == 44;
}

size_t gemm_splitk_ws_floats(const GemmShape& s) {
    // only small outputs are split (measured: beyond ~2M elements the fp32 partial
    // traffic costs more than the extra workgroups gain)
    size_t per = (size_t)s.batch() * s.M * s.N;
    long tiles = ((s.M + 127) / 128) * ((s.N + 127) / 128) * s.batch();
    if (tiles > kSplitTarget / 2 || per > kSplitMaxOut) return 0;
    size_t splits = kSplitTarget / tiles;
    if (splits > 8) splits = 8;
    return per * splits;
}

namespace {

// What launch_gemm_pair would launch: the two products as the kernel takes them and,
// when one is offered and fits, a third one behind them.
struct PairSel {
    Canon c[2], c3;
    long n[2] = {0, 0}, n3 = 0;
    int variant = -1;          // instantiated orientation of the pair
};

bool pair_select(const GemmShape* const sh[2], const Canon cin[2], float* ws, size_t ws_floats,
                 const PairThird* third, PairSel& out) {
    bool akc[2], bkc[2], split_used = false;
    int nkt[2];
    for (int i = 0; i < 2; ++i) {
        out.c[i] = cin[i];
        const long batch = sh[i]->batch();
        if (batch == 0 || pick_kind(out.c[i], akc[i], bkc[i]) != 1) return false;
        GemmArgs& a = out.c[i].a;
        if (a.M % 128 || a.N % 128 || a.K1 % BK) return false;
        out.n[i] = (long)(a.M / 128) * (a.N / 128) * batch;
        // a small output has its contraction split, as on its own (the scratch serves one product)
        if (ws && !split_used && out.n[i] < 128 && (size_t)batch * a.M * a.N <= kSplitMaxOut) {
            a.splits = pick_splits(a, batch, ws_floats);
            if (a.splits > 1) { a.partial = ws; split_used = true; out.n[i] *= a.splits; }
        }
        if (out.n[i] % 8 || out.n[i] < 128 || out.n[i] > 384) return false;
        if (pick_tile(a, batch, akc[i], bkc[i]) != 22) return false;
        if (akc[i] && bkc[i]) return false;                  // the asynchronous kernel's products stay on their own
        nkt[i] = a.K0 * (a.K1 / BK) / a.splits;
    }
    if (akc[0] && !bkc[0] && !akc[1] && !bkc[1]) out.variant = 0;
    else if (!akc[0] && !bkc[0] && !akc[1] && !bkc[1]) out.variant = 1;
    else if (akc[0] && !bkc[0] && akc[1] && !bkc[1]) out.variant = 2;
    else return false;
    // A third product rides along when its whole tiles fit into the places the pair
    // leaves free (two workgroups per CU), it is read the way the second one is, and
    // its contraction is not longer than theirs: the launch then takes no longer.
    out.n3 = 0;
    if (third && third->shape) {
        const long batch = third->shape->batch();
        out.c3 = canonicalise(*third->shape, third->A, third->B, third->C, third->alpha, GemmEpilogue{});
        bool a3 = false, b3 = false;
        const GemmArgs& a = out.c3.a;
        if (batch > 0 && pick_kind(out.c3, a3, b3) == 1 && a.M % 128 == 0 && a.N % 128 == 0 && a.K1 % BK == 0 &&
            a3 == akc[1] && b3 == bkc[1]) {
            const long n3 = (long)(a.M / 128) * (a.N / 128) * batch;
            const int nkt3 = a.K0 * (a.K1 / BK);
            if (n3 % 8 == 0 && out.n[0] + out.n[1] + n3 <= 512 && nkt3 <= (nkt[0] > nkt[1] ? nkt[0] : nkt[1]))
                out.n3 = n3;
        }
    }
    return true;
}

}  // namespace

bool gemm_pair_takes_third(const GemmShape& s1, const half_t* A1, const half_t* B1, half_t* C1,
                           const GemmEpilogue& ep1, const GemmShape& s2, const half_t* A2, const half_t* B2,
                           half_t* C2, const GemmEpilogue& ep2, float* ws, size_t ws_floats,
                           const PairThird& third) {
    const GemmShape* sh[2] = {&s1, &s2};
    const Canon c[2] = {canonicalise(s1, A1, B1, C1, 1.f, ep1), canonicalise(s2, A2, B2, C2, 1.f, ep2)};
    PairSel sel;
    return pair_select(sh, c, ws, ws_floats, &third, sel) && sel.n3 > 0;
}

bool gemm_pair_ok(const GemmShape& s1, const half_t* A1, const half_t* B1, half_t* C1, const GemmEpilogue& ep1,
                  const GemmShape& s2, const half_t* A2, const half_t* B2, half_t* C2, const GemmEpilogue& ep2,
                  float* ws, size_t ws_floats) {
    const GemmShape* sh[2] = {&s1, &s2};
    const Canon c[2] = {canonicalise(s1, A1, B1, C1, 1.f, ep1), canonicalise(s2, A2, B2, C2, 1.f, ep2)};
    PairSel sel;
    return pair_select(sh, c, ws, ws_floats, nullptr, sel);
}

// Two independent products in one launch (see k_gemm_pair).  Returns false, having
// launched nothing, unless both are products the register-staged kernel would take
// as whole 128x128 tiles with about one tile per CU, in an operand orientation
// that is instantiated; the caller then launches them one after the other.
bool launch_gemm_pair(const GemmShape& s1, const half_t* A1, const half_t* B1, half_t* C1, float alpha1,
                      const GemmEpilogue& ep1, const GemmShape& s2, const half_t* A2, const half_t* B2,
                      half_t* C2, float alpha2, const GemmEpilogue& ep2, hipStream_t st, float* ws,
                      size_t ws_floats, FinishJobs* tail, PairThird* third) {
    const GemmShape* sh[2] = {&s1, &s2};
    const Canon cin[2] = {canonicalise(s1, A1, B1, C1, alpha1, ep1), canonicalise(s2, A2, B2, C2, alpha2, ep2)};
    PairSel sel;
    if (!pair_select(sh, cin, ws, ws_floats, third, sel)) return false;
    {
        // 256 x 128 tiles when they are whole, unsplit and about one per CU
        bool ok = true;
        long n8[3] = {0, 0, 0};
        for (int i = 0; i < 2; ++i) {
            const GemmArgs& a = sel.c[i].a;
            ok = ok && a.splits == 1 && a.M % 256 == 0;
            n8[i] = sel.n[i] / 2;
            ok = ok && n8[i] % 8 == 0;
        }
        if (sel.n3) { ok = ok && sel.c3.a.M % 256 == 0; n8[2] = sel.n3 / 2; ok = ok && n8[2] % 8 == 0; }
        else if (third && third->shape) ok = false;            // a third product was offered and did not fit
        ok = ok && n8[0] + n8[1] + n8[2] <= 256 && n8[0] + n8[1] + n8[2] >= 192;
        if (ok) {
            FinishJobs tj;
            unsigned tg = 1;
            if (tail && tail->n > 0) {
                const long groups = finish_groups(*tail);
                if (groups * tail->n <= 4096) { tj = *tail; tg = (unsigned)groups; }
            }
            GemmArgs g3{};
            if (sel.n3) g3 = sel.c3.a;
            dim3 grid((unsigned)(n8[0] + n8[1] + n8[2]) + (unsigned)tj.n * tg);
            const GemmArgs& g1 = sel.c[0].a;
            const GemmArgs& g2 = sel.c[1].a;
            const unsigned m1 = (unsigned)n8[0], m2 = (unsigned)n8[1], m3 = (unsigned)n8[2];
            if (sel.variant == 0)
                hipLaunchKernelGGL((k_gemm_pair8<true, false, false, false>), grid, dim3(512), 0, st, g1, g2, m1, m2, g3, m3, tj, tg);
            else if (sel.variant == 1)
                hipLaunchKernelGGL((k_gemm_pair8<false, false, false, false>), grid, dim3(512), 0, st, g1, g2, m1, m2, g3, m3, tj, tg);
            else
                hipLaunchKernelGGL((k_gemm_pair8<true, false, true, false>), grid, dim3(512), 0, st, g1, g2, m1, m2, g3, m3, tj, tg);
            if (tj.n > 0) tail->n = 0;
            if (sel.n3) third->taken = true;
            check_launch("gemm pair (256 x 128 tiles)");
            return true;
        }
    }
    // column sums of earlier launches, finished by workgroups after the tiles (none of them
    // may be a sum that this launch itself contributes to)
    FinishJobs tj;
    unsigned tg = 1;
    if (tail && tail->n > 0) {
        const long groups = finish_groups(*tail);
        if (groups * tail->n <= 4096) { tj = *tail; tg = (unsigned)groups; }
    }
    const unsigned n1 = (unsigned)sel.n[0], n2 = (unsigned)sel.n[1], n3 = (unsigned)sel.n3;
    GemmArgs g3{};
    if (n3) g3 = sel.c3.a;
    dim3 grid(n1 + n2 + n3 + (unsigned)tj.n * tg);
    const GemmArgs& g1 = sel.c[0].a;
    const GemmArgs& g2 = sel.c[1].a;
    if (sel.variant == 0)
        hipLaunchKernelGGL((k_gemm_pair<true, false, false, false>), grid, dim3(256), 0, st, g1, g2, n1, n2, g3, n3, tj, tg);
    else if (sel.variant == 1)
        hipLaunchKernelGGL((k_gemm_pair<false, false, false, false>), grid, dim3(256), 0, st, g1, g2, n1, n2, g3, n3, tj, tg);
    else
        hipLaunchKernelGGL((k_gemm_pair<true, false, true, false>), grid, dim3(256), 0, st, g1, g2, n1, n2, g3, n3, tj, tg);
    if (tj.n > 0) tail->n = 0;         // taken: nothing left for the caller to finish
    if (n3) third->taken = true;
    for (int i = 0; i < 2; ++i)
        if (sel.c[i].a.splits > 1) {
            const long batch = sh[i]->batch(), nq = batch * (long)sel.c[i].a.M * (sel.c[i].a.N / 4);
            hipLaunchKernelGGL(k_gemm_splitk_reduce, dim3((unsigned)((nq + 255) / 256)), dim3(256), 0, st, sel.c[i].a, batch);
        }
    check_launch("gemm pair");
    return true;
}

void launch_gemm(const GemmShape& s, const half_t* A, const half_t* B, half_t* C, float alpha,
                 const GemmEpilogue& ep, hipStream_t st, float* ws, size_t ws_floats, GemmSideJob* side) {
    long batch = s.batch();
    if (batch == 0 || s.M == 0 || s.N == 0) return;
    Canon c = canonicalise(s, A, B, C, alpha, ep);
    bool akc = false, bkc = false;
    int kind = pick_kind(c, akc, bkc);
    if (kind == 1) {
        // The asynchronous 128x128 kernel is taken when both operands are k-contiguous and there
        // is at most about one tile per CU, where the register-staged kernel has no second
        // workgroup to hide its waits behind.
        const long tiles128 = (long)((c.a.M + 127) / 128) * ((c.a.N + 127) / 128) * batch;
        if (ws && (size_t)batch * c.a.M * c.a.N <= kSplitMaxOut) {
            c.a.splits = pick_splits(c.a, batch, ws_floats);
            c.a.partial = ws;
        }
        const int tile = pick_tile(c.a, batch, akc, bkc);
        if (side) side->tiles_done = 0;
        if (side && side->keep && side->key.thr && tile == 44 && !ep.relu_dropout && !ep.gate && c.a.splits == 1) {
            // CUs the tiles leave idle draw attention keep bits meanwhile: what fits into the time the
            // product takes (about 9 us + 1.5 us per k-tile; the rate per CU and us is the measured break-even:
            // 12 of the 16 key tiles of the bench workload cost the launch 0.3 us, 14 cost it 2.5, all 16 6 us)
            const long tiles = (long)(c.a.M / 256) * (c.a.N / 256) * batch;
            const long idle = 256 - tiles, nkt = (long)c.a.K0 * (c.a.K1 / BK);
            if (tiles >= 128 && idle >= 32 && side->nk % 32 == 0) {
                const double groups = (double)idle * (9.0 + 1.5 * (double)nkt) * 1600.0;
                long td = (long)(groups / (4.0 * (double)side->rows));
                if (td > side->nk / 32) td = side->nk / 32;
                if (td > 0) {
                    c.a.side_first = (unsigned)tiles; c.a.side_blocks = (unsigned)idle;
                    c.a.side_key = side->key; c.a.side_keep = side->keep;
                    c.a.side_rows = side->rows; c.a.side_nk = side->nk; c.a.side_tiles_done = (uint32_t)td;
                    side->tiles_done = (uint32_t)td;
                }
            }
        }
        if ((ep.relu_dropout || ep.gate) && (tile != 44 || batch != 1 || s.sCN != 1 || s.sCM != s.N))
            fail("gemm: the ReLU-dropout epilogue needs the 256x256 asynchronous kernel (see gemm_relu_dropout_ok)");
        const bool dma = akc && bkc && tiles128 <= 384;
        if (tile == 44) launch_mfma<4, 4, true>(c.a, akc, bkc, batch, true, st);
        else if (tile == 21) launch_mfma<2, 1, false>(c.a, akc, bkc, batch, false, st);
        else launch_mfma<2, 2, true>(c.a, akc, bkc, batch, dma, st);
    } else {
        if (ep.relu_dropout || ep.gate) fail("gemm: the ReLU-dropout epilogue needs the MFMA kernel");
        long total = batch * (long)c.a.M * c.a.N;
        long blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffL) fail("gemm: problem too large for the scalar kernel");
        hipLaunchKernelGGL(k_gemm_scalar, dim3((unsigned)blocks), dim3(256), 0, st, c.a, total);
    }
    check_launch("gemm");
}

}  // namespace sub
