// Tensor contractions: strided, batched fp16 GEMM with fp32 accumulation on the
// gfx950 matrix cores (v_mfma_f32_32x32x16_f16), honouring each operand's
// stride layout.  Takes the place of the cuBLAS calls behind
// pytorch_module/gemm.cuh:52-147.
//
//   C[b, m, n] = alpha * sum_k A[b, m, k] * B[b, k, n]  (+ bias)
//
// Operands may be contiguous along the contraction (K) or along their free
// dimension (M resp. N); an operand that is contiguous along its free dimension
// is transposed in registers on the way into LDS, so the matrix-core fragments
// are always 8 consecutive k per lane.  The output is produced transposed in the
// accumulators (4 consecutive n per lane), staged through LDS and written as
// full 128-bit rows.
#include "sub_ops.hpp"

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
};

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
    acc *= g.alpha;
    if (g.bias)
        acc += (float)g.bias[b0 * g.sbb[0] + b1 * g.sbb[1] + b2 * g.sbb[2] + (long)m * g.sbM + (long)n * g.sbN];
    g.C[b0 * g.sCb[0] + b1 * g.sCb[1] + b2 * g.sCb[2] + (long)m * g.sCM + (long)n * g.sCN] = (half_t)acc;
}

// ---------------------------------------------------------------------------
// MFMA kernel.  256 threads = 2x2 waves; each wave owns TM x TN tiles of 32x32.
// ---------------------------------------------------------------------------
constexpr int BK = 64;            // k per LDS tile: one 128-byte line per row

// LDS tile: rows of 64 halves (eight 16-byte slots); the slot index is xor-ed
// with a function of the row so that both the fragment reads (32 consecutive
// rows, one slot) and the transposing writes (rows 8 apart) spread over banks.
__device__ __forceinline__ int lds_off(int row, int slot) {
    return row * BK + ((slot ^ (row ^ (row >> 3))) & 7) * 8;
}

template <int ROWS, bool KC>
struct TileLoader {
    // ROWS rows (free dim) x BK k.  KC: k contiguous in memory, else the free dim.
    static constexpr int NV = ROWS / 32;          // 16-byte loads per thread
    static_assert(KC || NV % 4 == 0, "transposing loader needs at least 128 rows");

    // base points at (free0, k-tile start) of the current batch; sF / sK are the
    // strides of the free dim and of k; nfree / nk are the extents left.
    static __device__ __forceinline__ void load(h8 (&v)[NV], const half_t* base, long sF, long sK,
                                                int nfree, int nk, int tid) {
        if (KC) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                int id = tid + i * 256;
                int row = id >> 3, slot = id & 7;
                bool ok = row < nfree && slot * 8 + 8 <= nk;
                if (ok) v[i] = *reinterpret_cast<const h8*>(base + (long)row * sF + slot * 8);
                else v[i] = (h8)(half_t)0.0f;
            }
        } else {
            constexpr int FB = ROWS / 8;          // 8-wide blocks along the free dim
            constexpr int KQ = 256 / FB;          // k-quads covered per pass
            int fb = tid % FB, kq = tid / FB;
#pragma unroll
            for (int p = 0; p < NV / 4; ++p)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int k = (p * KQ + kq) * 4 + i;
                    bool ok = fb * 8 + 8 <= nfree && k < nk;
                    if (ok) v[p * 4 + i] = *reinterpret_cast<const h8*>(base + (long)k * sK + fb * 8);
                    else v[p * 4 + i] = (h8)(half_t)0.0f;
                }
        }
    }

    static __device__ __forceinline__ void store(const h8 (&v)[NV], half_t* lds, int tid) {
        if (KC) {
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                int id = tid + i * 256;
                int row = id >> 3, slot = id & 7;
                *reinterpret_cast<h8*>(lds + lds_off(row, slot)) = v[i];
            }
        } else {
            constexpr int FB = ROWS / 8;
            constexpr int KQ = 256 / FB;
            int fb = tid % FB, kq = tid / FB;
#pragma unroll
            for (int p = 0; p < NV / 4; ++p) {
                int kcol = (p * KQ + kq) * 4;     // first of 4 consecutive k
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    h4 w;
                    w[0] = v[p * 4 + 0][r]; w[1] = v[p * 4 + 1][r];
                    w[2] = v[p * 4 + 2][r]; w[3] = v[p * 4 + 3][r];
                    int row = fb * 8 + r;
                    *reinterpret_cast<h4*>(lds + lds_off(row, kcol >> 3) + (kcol & 7)) = w;
                }
            }
        }
    }
};

template <int TM, int TN, bool AKC, bool BKC>
__global__ __launch_bounds__(256) void k_gemm_mfma(GemmArgs g) {
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int TILE_A = BM * BK, TILE_B = BN * BK;             // halves
    constexpr int STAGE_PITCH = 32 * TN + 8;                       // halves
    constexpr int STAGE_WAVE = 32 * STAGE_PITCH;                   // one 32-row slab per wave
    constexpr int LDS_TILES = 2 * (TILE_A + TILE_B);
    constexpr int LDS_STAGE = 4 * STAGE_WAVE;
    constexpr int LDS_HALVES = LDS_TILES > LDS_STAGE ? LDS_TILES : LDS_STAGE;
    __shared__ __attribute__((aligned(16))) half_t lds[LDS_HALVES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, hi = lane >> 5;

    // batch offsets
    long bz = blockIdx.z;
    long b2 = bz % g.nb2; long t = bz / g.nb2;
    long b1 = t % g.nb1; long b0 = t / g.nb1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const half_t* Ab = g.A + b0 * g.sAb[0] + b1 * g.sAb[1] + b2 * g.sAb[2] + (long)m0 * g.sAM;
    const half_t* Bb = g.B + b0 * g.sBb[0] + b1 * g.sBb[1] + b2 * g.sBb[2] + (long)n0 * g.sBN;
    const int mleft = g.M - m0, nleft = g.N - n0;

    const int tiles_per_k1 = (g.K1 + BK - 1) / BK;
    const int nkt = g.K0 * tiles_per_k1;

    f16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    using LA = TileLoader<BM, AKC>;
    using LB = TileLoader<BN, BKC>;
    h8 ra[LA::NV], rb[LB::NV];

#define SUB_GEMM_ISSUE(kt_)                                                                       \
    do {                                                                                          \
        int k0_ = (kt_) / tiles_per_k1, kk_ = ((kt_) - k0_ * tiles_per_k1) * BK;                  \
        LA::load(ra, Ab + (long)k0_ * g.sAK0 + (long)kk_ * g.sAK1, g.sAM, g.sAK1, mleft,          \
                 g.K1 - kk_, tid);                                                                \
        LB::load(rb, Bb + (long)k0_ * g.sBK0 + (long)kk_ * g.sBK1, g.sBN, g.sBK1, nleft,          \
                 g.K1 - kk_, tid);                                                                \
    } while (0)

    SUB_GEMM_ISSUE(0);
    LA::store(ra, lds, tid);
    LB::store(rb, lds + TILE_A, tid);
    __syncthreads();

    for (int kt = 0; kt < nkt; ++kt) {
        const int cur = kt & 1;
        const half_t* sA = lds + cur * (TILE_A + TILE_B);
        const half_t* sB = sA + TILE_A;
        if (kt + 1 < nkt) SUB_GEMM_ISSUE(kt + 1);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            h8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i] = *reinterpret_cast<const h8*>(sA + lds_off(wm * 32 * TM + i * 32 + l32, ks * 2 + hi));
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = *reinterpret_cast<const h8*>(sB + lds_off(wn * 32 * TN + j * 32 + l32, ks * 2 + hi));
            // D^T tiles: rows of the MFMA result run along n, columns along m.
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nkt) {
            half_t* dA = lds + (cur ^ 1) * (TILE_A + TILE_B);
            LA::store(ra, dA, tid);
            LB::store(rb, dA + TILE_A, tid);
        }
        __syncthreads();
    }

#undef SUB_GEMM_ISSUE
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
                for (int e = 0; e < 4; ++e) {
                    float x = acc[i][j][q * 4 + e] * g.alpha;
                    if (biasb) {
                        int mm = mrow + l32, nn = n0 + wn * 32 * TN + ncol + e;
                        if (mm < g.M && nn < g.N) x += (float)biasb[(long)mm * g.sbM + (long)nn * g.sbN];
                    }
                    w[e] = (half_t)x;
                }
                *reinterpret_cast<h4*>(stage + l32 * STAGE_PITCH + ncol) = w;
            }
        // LDS operations of one wave execute in order: the reads below see the writes above.
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
            int r = it * RPI + lane / LPR, c8 = (lane % LPR) * 8;
            h8 val = *reinterpret_cast<const h8*>(stage + r * STAGE_PITCH + c8);
            int mm = mrow + r, nn = n0 + wn * 32 * TN + c8;
            if (mm < g.M && nn + 8 <= g.N)
                *reinterpret_cast<h8*>(Cb + (long)mm * g.sCM + nn) = val;
        }
    }
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
    // every 16-byte access must be aligned and whole
    bool ok = mult8(a.N) && mult8(a.sCM) && mult8(a.sCb[0]) && mult8(a.sCb[1]) && mult8(a.sCb[2]);
    ok = ok && mult8(a.sAK0) && mult8(a.sAb[0]) && mult8(a.sAb[1]) && mult8(a.sAb[2]);
    ok = ok && mult8(a.sBK0) && mult8(a.sBb[0]) && mult8(a.sBb[1]) && mult8(a.sBb[2]);
    if (akc) ok = ok && mult8(a.K1) && mult8(a.sAM); else ok = ok && mult8(a.M) && mult8(a.sAK1);
    if (bkc) ok = ok && mult8(a.K1) && mult8(a.sBN); else ok = ok && mult8(a.N) && mult8(a.sBK1);
    return ok ? 1 : 0;
}

template <int TM, int TN>
void launch_mfma(const GemmArgs& a, bool akc, bool bkc, long batch, hipStream_t st) {
    dim3 grid((a.N + 64 * TN - 1) / (64 * TN), (a.M + 64 * TM - 1) / (64 * TM), (unsigned)batch);
    if (akc && bkc) hipLaunchKernelGGL((k_gemm_mfma<TM, TN, true, true>), grid, dim3(256), 0, st, a);
    else if (akc) hipLaunchKernelGGL((k_gemm_mfma<TM, TN, true, false>), grid, dim3(256), 0, st, a);
    else if (bkc) hipLaunchKernelGGL((k_gemm_mfma<TM, TN, false, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((k_gemm_mfma<TM, TN, false, false>), grid, dim3(256), 0, st, a);
}

}  // namespace

int gemm_kernel_kind(const GemmShape& s, const void* A, const void* B, const void* C) {
    GemmEpilogue ep;
    Canon c = canonicalise(s, (const half_t*)A, (const half_t*)B, (half_t*)C, 1.f, ep);
    bool akc, bkc;
    return pick_kind(c, akc, bkc);
}

void launch_gemm(const GemmShape& s, const half_t* A, const half_t* B, half_t* C, float alpha,
                 const GemmEpilogue& ep, hipStream_t st) {
    long batch = s.batch();
    if (batch == 0 || s.M == 0 || s.N == 0) return;
    if (batch > 65535) fail("gemm: more than 65535 batches");
    Canon c = canonicalise(s, A, B, C, alpha, ep);
    bool akc = false, bkc = false;
    int kind = pick_kind(c, akc, bkc);
    if (kind == 1) {
        launch_mfma<2, 2>(c.a, akc, bkc, batch, st);
    } else {
        long total = batch * (long)c.a.M * c.a.N;
        long blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffL) fail("gemm: problem too large for the scalar kernel");
        hipLaunchKernelGGL(k_gemm_scalar, dim3((unsigned)blocks), dim3(256), 0, st, c.a, total);
    }
    check_launch("gemm");
}

}  // namespace sub
