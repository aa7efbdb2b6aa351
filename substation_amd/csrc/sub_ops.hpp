// Launchers of the device kernels (one per fused operator + the GEMM).
#pragma once

#include <hip/hip_runtime.h>

#include "sub_common.hpp"
#include "sub_device.hpp"

namespace sub {

enum Activation { ACT_RELU = 0, ACT_GELU = 1 };

inline void check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) fail(std::string(what) + ": " + hipGetErrorString(e));
}

// --- row operators (one wave per row, row held in registers) -----------------
// amask: optional additive attention mask over (query, key) positions (p == nullptr: none)
void launch_softmax(const RowSpace& rs, View beta, View alpha, View mask, View drop, View amask,
                    float scale, float mscale, PhiloxKey key, hipStream_t st);
void launch_bs(const RowSpace& rs, View alpha, View mask, View ddrop, View dbeta, float scale,
               hipStream_t st);
// Side job of launch_bdrln (a launch that waits for memory with its vector units idle): `blocks`
// workgroups behind those of the rows draw the keep words of the ReLU-dropout epilogue
// (relu_dropout_keep_words) of a later product with a dense [M][N] output in 256x256 tiles, word
// quadruple ((tile_m * N/256 + tile_n) * 8 + wave) * 64 + lane of `out` (M * N / 8 bytes).
struct KeepWordsJob {
    PhiloxKey key;
    uint32_t* out = nullptr;
    uint32_t M = 0, N = 0;
    uint32_t blocks = 0;         // set by launch_bdrln; 0 = not taken
};
// write_lin = false: `lin` (input + bias, which the backward pass does not read) is not stored.
// mask_bits (optional; rows of whole 8-packs): the dropout mask as one bit per element in canonical
// order -- byte row * R / 8 + e / 8, bit e % 8 -- instead of the 0/1 tensor `mask`, which is then
// neither written (bdrln) nor read (blnrd, the fused LayerNorm backward): 1/16 of the bytes.
void launch_bdrln(const RowSpace& rs, View in, View resid, View lin_bias, View scale, View bias,
                  View lin, View mask, View diff, View normed, View out, View istd, PhiloxKey key,
                  float eps, hipStream_t st, uint8_t* mask_bits = nullptr, bool write_lin = true,
                  KeepWordsJob* side = nullptr);
void launch_blnrd(const RowSpace& rs, View dout, View istd, View diff, View mask, View d_ln_in,
                  View d_drop_in, hipStream_t st, const uint8_t* mask_bits = nullptr);

// --- elementwise operators ---------------------------------------------------
// out_only: neither LIN (input + bias) nor the mask is written, only the output
void launch_bad(const RowSpace& rs, View in, View bias, View lin, View mask, View out, int act,
                PhiloxKey key, hipStream_t st, bool out_only = false);
// out = a + b (b may be a broadcast view): bei, aib
void launch_add(const RowSpace& rs, View a, View b, View out, hipStream_t st);

// --- column reductions -------------------------------------------------------
// Sums over the two inner outer dims (n2, n3) of the row space, one result per
// (n0, n1, row element).  `ws` is fp32 scratch of at least colreduce_ws_floats()
// elements.
struct ColOut {
    half_t* p;   // dense [R]
};
// The second stage of a column reduction (adding the per-chunk partials).  It
// can be deferred: several operators then share one finishing launch, each with
// its own scratch region.
struct FinishArgs {
    half_t* out[4];
    long ob0, ob1, of;      // output strides of the kept dims (i0, i1) and of the feature
    int n1;
};
struct FinishJob {
    const float* ws;
    FinishArgs fo;
    int ns, nbatch, ntc, R;
};
constexpr int kMaxFinishJobs = 6;
struct FinishJobs {
    FinishJob j[kMaxFinishJobs];
    int n = 0;
};
void launch_colfinish(const FinishJobs& jobs, hipStream_t st);
// Hands a reduction's second stage to the list, or launches it at once when there is none.  A full list is
// finished first (its partials are complete by the time that launch runs: the stream orders them).
inline void finish_or_defer(FinishJobs* defer, const FinishJob& job, hipStream_t st) {
    if (!defer) {
        FinishJobs one; one.n = 1; one.j[0] = job;
        launch_colfinish(one, st);
        return;
    }
    if (defer->n >= kMaxFinishJobs) {
        launch_colfinish(*defer, st);
        defer->n = 0;
    }
    defer->j[defer->n++] = job;
}
size_t colreduce_ws_floats(const RowSpace& rs, int nsums);
void launch_bsb(const RowSpace& rs, View in, View dout, View scale, View din, ColOut dscale,
                ColOut dbias, float* ws, hipStream_t st, FinishJobs* defer = nullptr);
void launch_ebsb(const RowSpace& rs, View in, View dout1, View dout2, View dlinear, View scale,
                 View din, ColOut dscale, ColOut dbias, ColOut dlinear_bias, float* ws,
                 hipStream_t st, FinishJobs* defer = nullptr);
void launch_bdrlb(const RowSpace& rs, View ddrop, View mask, View lin, View dlinear, ColOut dbias,
                  int act, float* ws, hipStream_t st, FinishJobs* defer = nullptr);
// bdrlb for ReLU with the gate read off the forward pass's output (out > 0 exactly where the
// mask kept a positive pre-activation): neither the mask nor LIN is read
void launch_bdrlb_from_output(const RowSpace& rs, View ddrop, View out, View dlinear, ColOut dbias, float* ws,
                              hipStream_t st, FinishJobs* defer = nullptr);
void launch_baob(const RowSpace& rs, View datt, ColOut dbo, float* ws, hipStream_t st,
                 FinishJobs* defer = nullptr);
// out[i0,i1,e] = sum over (i2,i3) of d; out strides ob0, ob1 (kept dims) and of.
void launch_colsum(const RowSpace& rs, View d, half_t* out, long ob0, long ob1, long of, float* ws,
                   hipStream_t st, FinishJobs* defer = nullptr);
// The backward pass around one LayerNorm in one launch: the scale/bias gradients
// (and, extended, the linear-bias and output-bias gradients) with G = (d1 [+ d2])
// * scale, then the LayerNorm and dropout backward from G.  sums = {dscale, dbias,
// dlinear_bias, d_output_bias}; the last two only in the extended form.
struct LnBwdArgs {
    View in, d1, d2, dlinear, diff, mask, istd, scale;     // inputs (d2, dlinear: extended form)
    View g, d_ln_in, d_drop_in;                            // outputs
    const uint8_t* mask_bits = nullptr;                    // see launch_bdrln; replaces `mask`
    bool write_g = true;                                   // false: g (which nothing reads afterwards) is not stored
    // The column sum of `dlinear` that the extended form owes (the gradient of the second linear
    // bias) is the column sum of what the plain form writes as d_drop_in one LayerNorm earlier in
    // the backward pass: with move_sum the plain form adds that third sum (sums[2]) and the extended
    // form neither reads `dlinear` nor sums it (its sums are then d scale, d bias, d output-bias).
    bool move_sum = false;
};
bool lnbwd_supported(const RowSpace& rs, const LnBwdArgs& a, bool ext);
size_t lnbwd_ws_floats(const RowSpace& rs, bool ext);
void launch_lnbwd(const RowSpace& rs, const LnBwdArgs& a, bool ext, half_t* const sums[4], float* ws,
                  hipStream_t st, FinishJobs* defer = nullptr);
// Row sums: out[row-group] = sum over (n3, R) for each (n0,n1,n2): baib.
void launch_baib(const RowSpace& rs, View d, View out, hipStream_t st);

// --- attention scores formed in place (no round trip of the score tensor) -----
// rows_n: one row of head_size features per query position, rows_m: per key
// position; strides over (head, sample, position); the feature dim is contiguous.
struct ScoreArgs {
    const half_t* rows_n; const half_t* rows_m;
    long n_sh, n_sb, n_sr;
    long m_sh, m_sb, m_sr;
    float alpha;                 // scores = alpha * rows_n . rows_m^T, rounded to fp16
};
// Both return false, having launched nothing, when the shape or the layouts rule
// the fused kernel out.  rs: rows over (H, B, J), row length K, not merged.
// scores -> softmax -> dropout: writes alpha, mask, drop.
bool launch_scores_softmax(const RowSpace& rs, const ScoreArgs& a, int head_size, View alpha, View mask,
                           View drop, PhiloxKey key, hipStream_t st);
// d(dropped softmax) = rows_n . rows_m^T -> softmax backward: writes dbeta.
bool launch_dscores_bs(const RowSpace& rs, const ScoreArgs& a, int head_size, View alpha, View mask,
                       View dbeta, hipStream_t st);

// --- self-attention with the scores kept in registers -------------------------
// One of Q, K, V, the output or a gradient of these: rows of head_size contiguous
// features, strided over (head, sample, position).
struct AttnSide {
    const half_t* p = nullptr;
    long sh = 0, sb = 0, sr = 0;
};
struct AttnArgs {
    AttnSide q, k, v;          // projections (read)
    AttnSide o;                // forward: the output (written); backward: read
    AttnSide d_o;              // backward: gradient of the output (read)
    AttnSide dq, dk, dv;       // backward: gradients of the projections (written)
    float* lse = nullptr;      // [H*B*J]  log2-domain log-sum-exp of each score row
    float* dsum = nullptr;     // [H*B*J]  row sums of dO o O (written by the dQ launch, read by the dK/dV one)
    uint32_t* keep = nullptr;  // [H*B*J][K/32]  keep bits of the softmax dropout, bit k%32 of word k/32
    // forward: the words of key tiles 0 .. keep_tiles_ready-1 of every row are in `keep` already
    // (GemmSideJob); the kernel draws and stores the others
    uint32_t keep_tiles_ready = 0;
    int H = 0, B = 0, J = 0, K = 0;
    float alpha = 1.f;         // score scale
    // optional (backward): per-workgroup sums over positions of the rounded dq resp.
    // dk, dv rows, for the gradient of the projection biases.  bias_q: [H][B*J/128][P]
    // floats, bias_kv: [2][H][B*K/128][P] (dk, then dv).
    float* bias_q = nullptr;
    float* bias_kv = nullptr;
    const half_t* amask = nullptr;   // optional additive mask over (query, key), added before the scaling
    long am_sj = 0, am_sk = 0;
    // optional, with amask: [J/32][K/32] bytes, non-zero where the mask is -inf over the
    // whole 32x32 block (mha_mask_blocks); such tiles are not computed at all
    // optional, built from the mask by launch_mha_mask_plan: per block of 128 queries the
    // key tiles the mask leaves to do, per block of 128 keys the query tiles
    const uint32_t* qlist = nullptr;
    const uint32_t* klist = nullptr;
};
// head_size 64 or 128, J and K multiples of 128
bool mha_shape_ok(long H, long B, long J, long K, long head_size);
size_t mha_stat_bytes(long H, long B, long J);          // lse followed by dsum
size_t mha_keep_bytes(long H, long B, long J, long K);
bool mha_forward_ok(const AttnArgs& a, int head_size);
bool mha_backward_ok(const AttnArgs& a, int head_size);
void launch_mha_forward(const AttnArgs& a, int head_size, PhiloxKey key, hipStream_t st);
// skip[J/32][K/32] = 1 where mask[j][k] is -inf for every (j, k) of the block
// Device bytes of the plan of a [J, K] mask, and the launches that fill it (rebuild)
// and point the arguments at it.  J and K multiples of 128.
size_t mha_mask_plan_bytes(long J, long K);
void launch_mha_mask_plan(AttnArgs& a, void* plan, bool rebuild, hipStream_t st);
void launch_mha_backward_dq(const AttnArgs& a, int head_size, hipStream_t st);
void launch_mha_backward_dkv(const AttnArgs& a, int head_size, hipStream_t st);

// --- dimension order --------------------------------------------------------
// dst (dense, order ld) = src (dense, order ls): the same logical tensor in another dimension order.
void launch_relayout(const Layout& ls, const Layout& ld, const half_t* src, half_t* dst, hipStream_t st);
// Several tensors in one launch (eight to a launch).
struct RelayoutJob { Layout ls, ld; const half_t* src; half_t* dst; };
void launch_relayout_batch(const RelayoutJob* jobs, int n, hipStream_t st);

// --- measurement --------------------------------------------------------------
// `workgroups` workgroups of eight waves each read `iters` chunks of 64 KiB from a working set of
// `working_set` bytes at buf (form 0: into registers, 1: into LDS with asynchronous loads), copy them into the
// `working_set` bytes behind (form 2) or only write those (form 3); every workgroup leaves
// (cycle counter, wall counter) at its start and end in stamps[4 * workgroup ..].
void launch_fetch_probe(const void* buf, size_t working_set, int form, int iters, int workgroups,
                        unsigned long long* stamps, int* sink, hipStream_t st);

// --- tensor contraction ------------------------------------------------------
// Optional addend of the output: C = fp16(fp16(alpha * A.B) + addend), a bias
// that broadcasts along M or N, or a whole tensor (a residual).
struct GemmEpilogue {
    const half_t* bias = nullptr;
    int64_t sbM = 0, sbN = 0;       // addend strides along M and N
    int64_t sbb[3] = {0, 0, 0};     // and along the batch dims
    // after the addend: out = keep ? max(x, 0) : 0 with the keep bits of `key`, the element
    // index being the offset into C (C dense in canonical order).  See gemm_relu_dropout_ok.
    bool relu_dropout = false;
    PhiloxKey key;
    // or: out = gate > 0 ? x : 0 with `gate` laid out like an addend (strides sbM, sbN, sbb), and the
    // column sums of out over the rows of every 128-row slab as fp32 rows of `colsum` ([M / 128][N]);
    // same conditions as relu_dropout (gemm_relu_dropout_ok)
    const half_t* gate = nullptr;
    float* colsum = nullptr;
    // relu_dropout: also writes one bit per output (set = positive), M * N / 8 bytes in the kernel's
    // own order; gate: reads those bits, written by a product of the same output shape, instead of
    // the values of `gate` (which must still be given)
    uint32_t* gate_bits_out = nullptr;
    const uint32_t* gate_bits = nullptr;
    // relu_dropout: the keep bits drawn ahead by a KeepWordsJob with the same key, M and N; without
    // them the kernel draws them itself during the contraction
    const uint32_t* keep_words = nullptr;
    // The activation of relu_dropout and gate.  ACT_GELU: relu_dropout computes keep ? gelu(x) : 0, also
    // stores x (the rounded sum with its addend, which the backward pass needs) to `pre_out`, laid out
    // like C, and writes the keep bits to gate_bits_out (both required; no keep_words); gate computes
    // keep ? gelu'(gate) * x : 0 with `gate` the pre-activation values and gate_bits those keep bits (required).
    int act = ACT_RELU;
    half_t* pre_out = nullptr;
};
// Work that needs no memory path, offered to a product whose 256x256 tiles leave CUs idle: the
// keep bits of the attention dropout (attention_keep_word) for the first `tiles_done` key tiles of
// every score row, drawn by workgroups behind the product's tiles on the CUs these leave free.
// launch_gemm sets tiles_done (0: not taken) from the number of idle CUs and the length of the
// product; the attention kernel then draws only the other tiles' bits itself.
struct GemmSideJob {
    PhiloxKey key;
    uint32_t* keep = nullptr;       // [rows][nk / 32]
    uint32_t rows = 0, nk = 0;
    uint32_t tiles_done = 0;        // out
};
// `ws` (optional): fp32 scratch of ws_floats elements for splitting the
// contraction of small-output products across workgroups.
void launch_gemm(const GemmShape& g, const half_t* A, const half_t* B, half_t* C, float alpha,
                 const GemmEpilogue& ep, hipStream_t st, float* ws = nullptr, size_t ws_floats = 0,
                 GemmSideJob* side = nullptr);
// Can launch_gemm apply ep.relu_dropout to this product?  Only the asynchronous kernel with
// 256x256 tiles does, on a single dense row-major output.
bool gemm_relu_dropout_ok(const GemmShape& g, const void* A, const void* B, const void* C, const GemmEpilogue& ep);
// A third product offered to launch_gemm_pair: taken (and `taken` set) when its
// whole 128x128 tiles fit into the places the pair leaves free on the CUs, it is
// read the way the pair's second product is and its contraction is no longer
// than theirs; the launch then takes about as long as without it.  Its
// contraction is never split.
struct PairThird {
    const GemmShape* shape = nullptr;
    const half_t* A = nullptr;
    const half_t* B = nullptr;
    half_t* C = nullptr;
    float alpha = 1.f;
    bool taken = false;
};
// Two independent contractions in one launch, their workgroups interleaved so that
// every CU works on both at once.  Returns false, having launched nothing, when
// the pair does not qualify (then call launch_gemm for each).  `tail` (optional):
// deferred column sums of EARLIER launches, finished by extra workgroups of this
// launch; tail->n is set to 0 when they were taken, else it is left as it was.
bool launch_gemm_pair(const GemmShape& g1, const half_t* A1, const half_t* B1, half_t* C1, float alpha1,
                      const GemmEpilogue& ep1, const GemmShape& g2, const half_t* A2, const half_t* B2,
                      half_t* C2, float alpha2, const GemmEpilogue& ep2, hipStream_t st, float* ws = nullptr,
                      size_t ws_floats = 0, FinishJobs* tail = nullptr, PairThird* third = nullptr);
// Would launch_gemm_pair take these two products as one launch?
bool gemm_pair_ok(const GemmShape& g1, const half_t* A1, const half_t* B1, half_t* C1, const GemmEpilogue& ep1,
                  const GemmShape& g2, const half_t* A2, const half_t* B2, half_t* C2, const GemmEpilogue& ep2,
                  float* ws, size_t ws_floats);
// Would launch_gemm_pair with these two products take `third` along?
bool gemm_pair_takes_third(const GemmShape& g1, const half_t* A1, const half_t* B1, half_t* C1,
                           const GemmEpilogue& ep1, const GemmShape& g2, const half_t* A2, const half_t* B2,
                           half_t* C2, const GemmEpilogue& ep2, float* ws, size_t ws_floats,
                           const PairThird& third);
// Scratch (in floats) that launch_gemm can make use of for this shape; 0 if none.
size_t gemm_splitk_ws_floats(const GemmShape& g);
// Which kernel launch_gemm would pick: 0 = scalar fallback, 1 = MFMA.
int gemm_kernel_kind(const GemmShape& g, const void* A, const void* B, const void* C,
                     const GemmEpilogue& ep = GemmEpilogue());

}  // namespace sub
