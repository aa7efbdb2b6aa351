/* C ABI of libsubstation_amd.so: the fused BERT encoder layer (forward and
 * backward) on AMD MI355X (gfx950).
 *
 * Drop-in for the four symbols the reference's JIT-compiled encoder.so exports
 * (pytorch_module/encoder.cu:304-318) and that pytorch_module/encoder.py:395-403
 * binds with ctypes.  The reference bakes sizes, layouts, dtype and dropout
 * probabilities into the library at compile time (encoder.py:213-376); this
 * library is prebuilt, so the same information arrives through sub_config.
 *
 * All tensors are dense fp16 device buffers owned by the caller, laid out
 * row-major in the dimension order given by their layout string.  Functions
 * returning int give 0 on success and a negative value on error, with the
 * message available from sub_last_error(); nothing aborts the process (the
 * reference's CHECK macro does, pytorch_module/all.cuh:7-13).  A handle must
 * not be used from two threads at once (it carries the RNG step, like the
 * reference's GlobalRandomState, pytorch_module/blocks.cuh:48-51).  Kernels are
 * enqueued on the stream set with sub_set_stream (default: the null stream) and
 * are not synchronised (as pytorch_module/encoder.cu:156,298).
 */
#ifndef SUBSTATION_AMD_H
#define SUBSTATION_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SUB_ABI_VERSION 1
#define SUB_N_PARAMS 12   /* WKQV BKQV WO BO S1 B1 LINB1 LINW1 S2 B2 LINB2 LINW2 */
#define SUB_N_FWD 23      /* forward intermediates, pytorch_module/encoder.py:81 */
#define SUB_N_BWD 14      /* backward intermediates, pytorch_module/encoder.py:111 */

#define SUB_DTYPE_F16 0
#define SUB_ACT_RELU 0
#define SUB_ACT_GELU 1    /* tanh form, substation/transformer.py:11-14 */

/* Dropout sites (word 2 of the Philox counter). */
#define SUB_SITE_SOFTMAX 0
#define SUB_SITE_RESID1 1
#define SUB_SITE_ACT 2
#define SUB_SITE_RESID2 3

/* What pytorch_module/encoder.py:213-376 writes into encoder_parameters.cuh.
 * Names and layouts are listed in the order in which the caller will pass the
 * pointers (the order of the lists in the layouts pickle, encoder.py:229-264).
 * Dimension letters: B batch, J/K query/key position, H heads, P head size,
 * I embedding, U feed-forward width, Q stack index (0=K, 1=Q, 2=V). */
typedef struct sub_config {
    int32_t abi_version;            /* SUB_ABI_VERSION */
    int32_t batch, seq, heads, embed;
    int32_t intermediate;           /* 0 means 4*embed (encoder.py:33) */
    int32_t dtype;                  /* SUB_DTYPE_F16 */
    int32_t activation;             /* SUB_ACT_* */
    float p_softmax, p_resid1, p_act, p_resid2;
    float ln_eps;                   /* 0 means 1e-5 (block_bdrln.cuh:258) */
    uint64_t seed;
    const char* input_layout;       /* of X, a permutation of "BJI" */
    const char* output_layout;      /* of SB2 */
    const char* param_names[SUB_N_PARAMS];
    const char* param_layouts[SUB_N_PARAMS];
    const char* fwd_names[SUB_N_FWD];
    const char* fwd_layouts[SUB_N_FWD];
    const char* bwd_names[SUB_N_BWD];
    const char* bwd_layouts[SUB_N_BWD];
} sub_config;

/* ---- the reference's four exports (pytorch_module/encoder.cu:304-318) ------ */

/* encoder.cu:304 `Encoder* init()`.  Returns an unconfigured handle (NULL on
 * failure); call sub_configure before use, or use init_cfg. */
void* init(void);

/* encoder.cu:316 `void destroy(Encoder*)`. */
void destroy(void* handle);

/* encoder.cu:308 `void encoder_forward(Encoder*, ENCODER_FORWARD_DEF)`:
 * X, the 12 parameters, the 23 forward intermediates, Y (encoder.py:88-93). */
int encoder_forward(void* handle, void* X,
                    void* w0, void* w1, void* w2, void* w3, void* w4, void* w5,
                    void* w6, void* w7, void* w8, void* w9, void* w10, void* w11,
                    void* f0, void* f1, void* f2, void* f3, void* f4, void* f5, void* f6, void* f7,
                    void* f8, void* f9, void* f10, void* f11, void* f12, void* f13, void* f14,
                    void* f15, void* f16, void* f17, void* f18, void* f19, void* f20, void* f21,
                    void* f22, void* Y);

/* encoder.cu:312 `void encoder_backward(Encoder*, ENCODER_BACKWARD_DEF)`:
 * DY, 12 parameter gradients, 14 backward intermediates, 12 parameters,
 * 23 forward intermediates, X, DX (encoder.py:124-130). */
int encoder_backward(void* handle, void* DY,
                     void* dw0, void* dw1, void* dw2, void* dw3, void* dw4, void* dw5,
                     void* dw6, void* dw7, void* dw8, void* dw9, void* dw10, void* dw11,
                     void* b0, void* b1, void* b2, void* b3, void* b4, void* b5, void* b6,
                     void* b7, void* b8, void* b9, void* b10, void* b11, void* b12, void* b13,
                     void* w0, void* w1, void* w2, void* w3, void* w4, void* w5,
                     void* w6, void* w7, void* w8, void* w9, void* w10, void* w11,
                     void* f0, void* f1, void* f2, void* f3, void* f4, void* f5, void* f6, void* f7,
                     void* f8, void* f9, void* f10, void* f11, void* f12, void* f13, void* f14,
                     void* f15, void* f16, void* f17, void* f18, void* f19, void* f20, void* f21,
                     void* f22, void* X, void* DX);

/* ---- configuration (replaces the generated encoder_parameters.cuh) --------- */

void* init_cfg(const sub_config* cfg);               /* init() + sub_configure() */
int sub_configure(void* handle, const sub_config* cfg);
int sub_set_stream(void* handle, void* hip_stream);  /* hipStream_t */
/* Dropout masks are a pure function of (seed, site, step, element); step is
 * incremented by every encoder_forward (blocks.cuh:48-51 advances an offset). */
int sub_set_rng(void* handle, uint64_t seed, uint32_t step);
/* No counterpart in the reference (its generator state lives in device memory
 * already, blocks.cuh:24-51).  For callers that record the launches in a HIP
 * graph: kernel arguments, the step included, are frozen at capture, so replays
 * would repeat the captured masks.  With a counter in device memory set here
 * (one uint32, owned by the caller, NULL to switch off), the step a kernel uses
 * is the host step of sub_set_rng plus *device_step read when the kernel runs,
 * and encoder_forward advances *device_step on the stream instead of the host
 * step. */
int sub_set_rng_counter(void* handle, uint32_t* device_step);
const char* sub_last_error(void);
/* Masked self-attention: the layer of substation/transformer.py:443-546
 * (`decoder`), i.e. the encoder layer with an additive [J,K] mask on the
 * attention scores (fp16 device tensor owned by the caller, layout "JK" or
 * "KJ"; -inf above the diagonal for a causal layer).  As in
 * substation/attention.py:65-68 the mask is added to the raw scores, before the
 * 1/sqrt(P) scaling.  encoder_forward uses it until it is cleared with NULL;
 * encoder_backward needs nothing (masked positions have zero probability).
 * The mask's contents are read by every encoder_forward call (also to find the
 * tiles that are -inf throughout, which the attention kernels pass over) and
 * must stay unchanged until the matching encoder_backward has been issued.
 * Allocates a small table: not to be called during a graph capture. */
int sub_set_attention_mask(void* handle, const void* attn_mask, const char* layout);

/* Options.  SUB_OPT_FUSE_EPILOGUES (default 1): add BKQV in the epilogue of the
 * QKV projection and DRESID1 in the epilogue of the input-gradient projection,
 * where the layouts allow it.  The separate operators aib (block_aib.cuh) and
 * bei (block_bei.cuh) are then not launched and the intermediates WKKWQQWVV and
 * DXATT, which only they consume, are left unwritten.  Set to 0 to materialise
 * every intermediate exactly as pytorch_module/encoder.cu:87-299 does. */
#define SUB_OPT_FUSE_EPILOGUES 1
/* SUB_OPT_FUSE_LN_BACKWARD (default 1): run BackwardScaleBias +
 * BackwardLayerNormResidualDropout (encoder.cu:160-166) as one launch, and
 * ExtendedBackwardScaleBias + BackwardLayerNormResidualDropout +
 * BackwardAttnOutBias (encoder.cu:196-212) as another, where the embedding size
 * (<= 4096; beyond 1024 a row is shared by two or four waves) and the layouts
 * (feature dim contiguous, dense rows) allow it.  Every tensor the
 * separate kernels write is still written, from the same fp16-rounded
 * intermediates; the bias / scale gradients are summed in a different order
 * (fp32), so results can differ from the separate launches in the last bit. */
#define SUB_OPT_FUSE_LN_BACKWARD 2
/* SUB_OPT_FUSE_SCORES (default 1): form the attention scores inside the softmax
 * kernel (QK^T, encoder.cu:104-121) and the gradient of the dropped softmax
 * inside the softmax-backward kernel (dO.V^T, encoder.cu:228-247), for sequence
 * lengths 512 and 1024, head sizes 64 and 128 and feature-contiguous
 * projections.  BETA and DATTN_DROP, which only those kernels consume, are then
 * left unwritten; every other tensor is unchanged.  Set to 0 to materialise
 * them (the Python module does so for debug capture). */
#define SUB_OPT_FUSE_SCORES 3
/* SUB_OPT_FUSE_ATTENTION (default 1): run the whole self-attention -- scores,
 * softmax, dropout and the weighted sum of the values (encoder.cu:104-131), and
 * in the backward pass everything between DGAMMA and the gradients of the
 * projections (encoder.cu:222-262) -- with the scores kept in registers.  None
 * of BETA, ALPHA, ATTN_DROP_MASK, ATTN_DROP, DATTN_DROP and DBETA is then
 * produced; the ALPHA buffer holds two fp32 statistics per score row and the
 * ATTN_DROP_MASK buffer one keep bit per score instead (both buffers must be
 * the ones handed to the matching backward call, as in the reference).  The
 * dropout mask is the same counter-based one as in the separate operators.
 * Needs head size 64 or 128, sequence lengths that are multiples of 128,
 * and feature-contiguous projections (an attention mask set with
 * sub_set_attention_mask is added to the score tiles); otherwise, or with 0,
 * the operators run separately (results then agree to fp16 rounding, not bit
 * for bit, because probabilities are no longer rounded before the weighted sum).
 * Set the option before the forward call and leave it until after the matching
 * backward call.  Value 2 (SUB_FUSE_REQUIRED) makes both calls fail rather
 * than fall back: a caller that has asked sub_attention_in_registers() and got
 * 1 may then pass token allocations (any non-null pointer) for the four tensors
 * that are neither written nor read -- BETA, ATTN_DROP, DATTN_DROP, DBETA --
 * and needs only 8 bytes per score row behind ALPHA and K/8 bytes per score
 * row behind ATTN_DROP_MASK (both 16-byte aligned). */
#define SUB_OPT_FUSE_ATTENTION 4
#define SUB_FUSE_REQUIRED 2
/* SUB_OPT_PAIR_PRODUCTS (default 1): in encoder_backward a data-gradient product
 * and the weight-gradient product next to it (encoder.cu:205-216 DLIN1_LINW1 and
 * DLINW1; :262-276 DXATT and DWKQV), which do not depend on one another, run as
 * one launch with their workgroups interleaved when both have about one 128x128
 * tile per CU: every CU then holds one workgroup of each and one runs while the
 * other waits.  Results are unchanged.  Profiling names: `dXlin1+dWlin1`,
 * `dXQKV-fused+dWQKV-fused`. */
#define SUB_OPT_PAIR_PRODUCTS 5
/* SUB_OPT_RELU_FROM_OUTPUT (default 1).  ReLU layers: the backward pass reads
 * the gate of dropout and ReLU off the forward output DROP2 = relu(LIN1) * mask,
 * which is positive exactly where the mask kept a positive LIN1
 * (block_bdrlb.cuh:72 reads DROP2MASK and LIN1 for it).  encoder_forward then
 * writes neither LIN1 nor DROP2MASK and encoder_backward reads neither: 64 MiB less
 * traffic in each of the two launches at B=8, L=512, E=1024.  Outputs and gradients
 * are bit-identical to those with the option off.  With SUB_OPT_FUSE_EPILOGUES on
 * and DROP2 in BJU order, bias, ReLU and dropout then run in the epilogue of the
 * lin1 product (profiling name `lin1+bad`) and SB1_LINW1 is not written either:
 * the first B*J*U/8 bytes of that buffer then hold one bit per element of DROP2
 * (set where it is positive), in the kernel's own order.  In encoder_backward
 * bdrlb runs in the epilogue of the dXlin2 product (`dXlin2+bdrlb`), which takes
 * its gate from those bits when it is handed the SB1_LINW1 buffer that the
 * handle's latest encoder_forward call wrote and from DROP2 itself otherwise
 * (same results); DDROP2 is not written and DLINB1 sums its terms in another
 * order.
 * GELU layers, where both products qualify for those epilogues, SUB_OPT_FUSE_EPILOGUES
 * is on and LIN1, like DROP2, is in BJU order: bias, GELU and dropout run in the
 * epilogue of lin1, which writes LIN1 (the backward pass needs it) and DROP2 and
 * leaves the keep bits of the dropout, one per element, in the first B*J*U/8 bytes
 * of SB1_LINW1 in place of the DROP2MASK tensor; encoder_backward runs bdrlb
 * (block_bdrlb.cuh:13-146) in the epilogue of dXlin2 from LIN1 and those bits.
 * DROP2MASK, SB1_LINW1 and DDROP2 are not written; results are bit-identical
 * (DLINB1 to rounding).  encoder_backward knows from the options and the pointers
 * it is handed, which are the forward call's, that the bits lie in SB1_LINW1:
 * the option must not change between a forward call and its backward call.
 * Set it to 0 before the forward call when LIN1, DROP2MASK, SB1_LINW1 or
 * DDROP2 are wanted (debug capture). */
#define SUB_OPT_RELU_FROM_OUTPUT 6
/* SUB_OPT_FINISH_IN_PAIR (default 1): the second stage of the column sums of
 * encoder_backward (adding the per-chunk fp32 partials of the bias and
 * LayerNorm-parameter gradients) runs in extra workgroups of the last pair of
 * products of the pass, in the places its tiles leave free on the CUs (two
 * workgroups each), instead of in a launch of its own (same code, same order of
 * additions: bit-identical).  Where that launch also has room for the tiles of
 * the dWout product, dWout runs there with its contraction in one piece and
 * dXout runs alone (DWO then sums its terms in another order than with the
 * option off: equal to rounding).  Profiling names: `dXout`,
 * `dXQKV-fused+dWQKV-fused+dWout`.  Needs SUB_OPT_PAIR_PRODUCTS and the
 * in-register attention (whose kernels produce the DBKQV partials). */
#define SUB_OPT_FINISH_IN_PAIR 7
/* SUB_OPT_SIDE_JOBS (bit mask, default 1).  Bit 0: where the 256x256 tiles of
 * the stacked projections leave CUs idle (192 tiles on 256 CUs at B=8, L=512,
 * E=1024), workgroups behind the tiles of that launch draw the dropout keep bits
 * of the first key tiles of every score row for the attention launch that follows
 * (they depend on nothing but seed, step and position); the attention kernel
 * draws the rest.  Bit 1 (off by default: since that launch stopped being bound
 * by its own vector work the drawing costs it more than it saves the next one):
 * workgroups behind the rows of the first bias-dropout-residual-LayerNorm launch
 * draw the keep bits of lin1's ReLU-dropout epilogue (into the SB1_LINW1 buffer,
 * behind its gate bits).  Same bits, same results.  Needs the in-register
 * attention resp. the `lin1+bad` launch (SUB_OPT_FUSE_EPILOGUES). */
#define SUB_OPT_SIDE_JOBS 8
/* SUB_OPT_PACKED_MASKS (default 1; embedding size a multiple of 8): the masks of
 * the two residual dropouts travel from encoder_forward to encoder_backward as one
 * bit per element (byte (b*J + j)*I/8 + i/8, bit i%8, canonical order whatever
 * the tensor's layout) in the first B*J*I/8 bytes of the DROP1MASK and DROP3MASK
 * buffers, instead of as 0/1 tensors: 7.5 MiB less to write and to read per mask at
 * B=8, L=512, E=1024.  Same results.  Set it to 0 before the forward call when the
 * mask tensors are wanted (debug capture); both calls must see the same value. */
#define SUB_OPT_PACKED_MASKS 9
/* SUB_OPT_SKIP_UNREAD (default 1): intermediates that neither call reads
 * afterwards are not written: ATT keeps the product without its bias (the bias
 * is added in registers, encoder.cu:134-135 writes it back in place), LIN2 is
 * left alone, and where the LayerNorm backward runs as one launch DLN2 and DLN1
 * are left alone.  8 MiB less to write in each of four launches at B=8, L=512,
 * E=1024; outputs and gradients are bit-identical.  Set it to 0 (debug capture
 * does) when those tensors are wanted. */
#define SUB_OPT_SKIP_UNREAD 10
/* SUB_OPT_PRIVATE_LAYOUTS (default 1): when an activation of the configuration is not in the dimension
 * order the fused paths of this library need (token-major rows with the feature dim contiguous: input,
 * output and [B,J,I] tensors BJI, [B,J,U] tensors BJU, scores HBJK, projections QBJHP, attention output
 * BJHP) -- the reference's shipped configurations are feature-major, chosen for V100
 * (pytorch_module/layouts-bert-*.pickle) -- encoder_forward / encoder_backward run the whole layer in those
 * orders: every intermediate lies in the library's order inside the caller's buffer (same number of
 * elements), and the tensors that cross the boundary in another order (input, output, their gradients,
 * weights, weight gradients; weights WKQV QHPI, BKQV QHP, WO IHP, LINW1 UI, LINW2 IU) are copied into it
 * and back by a tiled transposing kernel (entries `relayout-in`, `relayout-out`, `relayout-in-bwd`,
 * `relayout-out-bwd` of the per-launch timing).
 * Outputs and gradients are the same to rounding; saved intermediates are NOT in the configured order
 * (sub_tensor_layout tells the order in use).  The staged copies (input, output, two gradients, the
 * weights and their gradients that differ) are allocated by the first calls.  A configuration whose
 * activations are all in the library's orders runs as it is, whatever its weight orders.  0: every
 * tensor in the configured order, through strided kernels where it must be (what debug capture and
 * a layout search need).  The operator entry points sub_op_* always take the layouts they are given. */
#define SUB_OPT_PRIVATE_LAYOUTS 11
/* *planned = 1 when, with the handle's sizes, layouts and options as they are
 * now, self-attention runs with the scores in registers
 * (given 16-byte aligned tensors).  No counterpart in the reference. */
int sub_attention_in_registers(void* handle, int* planned);
int sub_set_option(void* handle, int option, int value);
/* The present value of an option (a caller that sized LIN1 and DROP2MASK down,
 * see SUB_OPT_RELU_FROM_OUTPUT, checks it before every call). */
int sub_get_option(void* handle, int option, int* value);
/* The dimension order in which encoder_forward / encoder_backward hold a tensor of the configuration
 * ("X", "SB2" or a name of the three lists) inside its buffer: the configured one, or the library's own
 * under SUB_OPT_PRIVATE_LAYOUTS.  out receives a NUL-terminated string of at most 8 letters. */
int sub_tensor_layout(void* handle, const char* name, char out[16]);

/* Array forms of the two calls above: ptrs holds the same pointers in the same
 * order, without the handle (n must be 37 resp. 64). */
int sub_encoder_forward(void* handle, void* const* ptrs, int n);
int sub_encoder_backward(void* handle, void* const* ptrs, int n);

/* Per-operator timing with HIP events on the handle's stream; the counterpart
 * of the NVTX ranges of encoder.cu:32-53.  The launches are the same with timing
 * on as with it off.  sub_profile_read waits for the stream and returns the number
 * of launches of the last encoder_forward call followed, if one has been issued
 * since, by those of the encoder_backward call after it (at most cap are
 * written); reading only after the backward call leaves no host wait between
 * the two passes.  One event is recorded in front of every launch and one at the
 * end of each pass; a launch is timed from its event to the next one. */
int sub_profile_enable(void* handle, int on);
int sub_profile_read(void* handle, int cap, const char** names, float* ms);
/* on = 2 in sub_profile_enable: a one-lane kernel in front of every launch also samples the GPU's
 * shader clock counter and its constant-rate wall clock (no counterpart in the reference).
 * sub_profile_read_clocks returns, for the same launches as sub_profile_read, the shader clock in MHz
 * the GPU held from one sample to the next: the matrix-core peak a launch could have reached scales
 * with it.  The extra kernels lengthen a step by a few microseconds per launch; take durations from a
 * run with on = 1. */
int sub_profile_read_clocks(void* handle, int cap, const char** names, float* mhz);

/* ---- single operators (the units pytorch_module/benchmark.py times) -------- */
/* Sizes come from the handle's configuration; every tensor takes its own layout
 * string.  Vectors of parameters ([I], [U]) are dense. */

/* Scaled-dot-product attention with the scores kept in registers, forward and
 * backward (the chain encoder.cu:104-131 and :222-262 as one operator; with
 * n_keys != n_queries the encoder-decoder attention of
 * substation/transformer.py:288-441, attention.py:31-179).  q, out, d_out, dq:
 * layouts over B, J, H, P; k, v, dk, dv: over B, K, H, P (P innermost; B, H, P from
 * the handle; n_queries, n_keys multiples of 128; head size 64 or 128).
 * out = dropout(softmax(scale * (q.k^T + attn_mask))) . v, keep mask drawn for
 * (site, the handle's seed and step) over the canonical [H,B,J,K] element index.
 * stats: 2*H*B*n_queries floats, keep: H*B*n_queries*n_keys/8 bytes (both 16-byte
 * aligned), written by the forward call and read by the backward call, which
 * also needs the forward call's out.  attn_mask may be null.  These calls fail
 * (nothing is launched) when the sizes, layouts or alignment are not supported. */
int sub_op_attention_forward(void* handle, int n_queries, int n_keys, const void* q, const char* l_q,
                             const void* k, const void* v, const char* l_kv, void* out, const char* l_out,
                             void* stats, void* keep, const void* attn_mask, const char* l_attn_mask,
                             float scale, float p, uint32_t site);
int sub_op_attention_backward(void* handle, int n_queries, int n_keys, const void* q, const char* l_q,
                              const void* k, const void* v, const char* l_kv, const void* out,
                              const char* l_out, const void* d_out, const char* l_dout, void* stats,
                              const void* keep, void* dq, const char* l_dq, void* dk, void* dv,
                              const char* l_dkv, const void* attn_mask, const char* l_attn_mask, float scale);

/* sub_op_attention_backward that also sums dq, dk, dv over samples and positions:
 * dq_bias, dk_bias, dv_bias are [H, P] vectors (null: not wanted; dk_bias and dv_bias
 * both or neither), the gradients of the projection biases
 * (BackwardAttentionInputBiases, block_baib.cuh:15-211, encoder.cu:288-290), formed in
 * the attention launches instead of in launches that read dq, dk, dv again. */
int sub_op_attention_backward_biases(void* handle, int n_queries, int n_keys, const void* q, const char* l_q,
                                     const void* k, const void* v, const char* l_kv, const void* out,
                                     const char* l_out, const void* d_out, const char* l_dout, void* stats,
                                     const void* keep, void* dq, const char* l_dq, void* dk, void* dv,
                                     const char* l_dkv, const void* attn_mask, const char* l_attn_mask, float scale,
                                     void* dq_bias, void* dk_bias, void* dv_bias);

/* block_softmax.cuh:127-188; `scale` multiplies the input (1 in the layer, where
 * the factor is the GEMM's alpha, encoder.cu:116). */
int sub_op_softmax(void* handle, const void* beta, const char* l_beta, void* alpha,
                   const char* l_alpha, void* mask, const char* l_mask, void* drop,
                   const char* l_drop, float scale, float p, uint32_t site);
/* The same with an additive attention mask over (query, key) positions
 * (substation/attention.py:65-68, mask of transformer.py:151-157):
 * alpha = softmax(beta * scale + attn_mask * mask_scale); attn_mask is a [J,K]
 * fp16 tensor in layout "JK" or "KJ", shared by all heads and samples. */
int sub_op_softmax_masked(void* handle, const void* beta, const char* l_beta, void* alpha,
                          const char* l_alpha, void* mask, const char* l_mask, void* drop,
                          const char* l_drop, const void* attn_mask, const char* l_attn_mask,
                          float scale, float mask_scale, float p, uint32_t site);
/* block_bs.cuh:107-156 */
int sub_op_bs(void* handle, const void* alpha, const char* l_alpha, const void* mask,
              const char* l_mask, const void* ddrop, const char* l_ddrop, void* dbeta,
              const char* l_dbeta, float scale);
/* block_bdrln.cuh:287-352; lin may alias in (encoder.cu:134-135) */
int sub_op_bdrln(void* handle, const void* in, const char* l_in, const void* resid,
                 const char* l_resid, const void* linear_bias, const void* scale, const void* bias,
                 void* lin, const char* l_lin, void* mask, const char* l_mask, void* diff,
                 const char* l_diff, void* normed, const char* l_normed, void* out,
                 const char* l_out, void* istd, const char* l_istd, float p, uint32_t site);
/* block_blnrd.cuh:203-259 */
int sub_op_blnrd(void* handle, const void* dout, const char* l_dout, const void* istd,
                 const char* l_istd, const void* diff, const char* l_diff, const void* mask,
                 const char* l_mask, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                 const char* l_d_drop_in);
/* block_bad.cuh:87-145 */
int sub_op_bad(void* handle, const void* in, const char* l_in, const void* bias, void* lin,
               const char* l_lin, void* mask, const char* l_mask, void* out, const char* l_out,
               float p, uint32_t site);
/* block_bsb_ebsb.cuh:178-216 */
int sub_op_bsb(void* handle, const void* in, const char* l_in, const void* scale, const void* dout,
               const char* l_dout, void* din, const char* l_din, void* dscale, void* dbias);
/* block_bsb_ebsb.cuh:376-420 */
int sub_op_ebsb(void* handle, const void* in, const char* l_in, const void* scale,
                const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                const void* dlinear, const char* l_dlinear, void* din, const char* l_din,
                void* dscale, void* dbias, void* dlinear_bias);
/* block_bdrlb.cuh:105-146 */
int sub_op_bdrlb(void* handle, const void* ddrop, const char* l_ddrop, const void* mask,
                 const char* l_mask, const void* lin, const char* l_lin, void* dlinear,
                 const char* l_dlinear, void* dbias);
/* block_baob.cuh:79-97 */
int sub_op_baob(void* handle, const void* datt, const char* l_datt, void* dbo);
/* Operator calls between sub_ops_defer(h, 1) and sub_ops_defer(h, 0) leave the second
 * stage of their column sums (bsb, ebsb, bdrlb, baob, ln_backward: the bias and
 * scale gradients) to one launch that sub_ops_defer(h, 0) issues, as
 * encoder_backward does for its own (encoder.cu:158-299 has one kernel per
 * reduction; no counterpart there).  The gradient vectors are complete only after
 * that call; same bits as without.  When the list (6 entries) or the scratch buffer
 * is full, what is on the list is finished early.  encoder_backward refuses to run
 * in between. */
int sub_ops_defer(void* handle, int on);
/* block_aib.cuh:64-155, on the Q-stacked tensors */
int sub_op_aib(void* handle, const void* in, const char* l_in, const void* bias, const char* l_bias,
               void* out, const char* l_out);
/* block_baib.cuh:161-211, on the Q-stacked tensors */
int sub_op_baib(void* handle, const void* d, const char* l_d, void* dbias, const char* l_dbias);
/* The backward pass around one LayerNorm in one launch where the sizes and layouts
 * allow (rows of up to 1024 contiguous features; the plain form also dense rows of up
 * to 4096), else as the separate operators,
 * with the same results.  extended = 0: block_bsb_ebsb.cuh:12-204 (bsb) followed
 * by block_blnrd.cuh:14-259: g = dout1 * scale, dscale, dbias, then d_ln_in and
 * d_drop_in from g.  extended = 1: block_bsb_ebsb.cuh:206-420 (ebsb: g =
 * (dout1 + dout2) * scale, dlinear_bias = column sums of dlinear), blnrd, and
 * block_baob.cuh:10-97 on d_drop_in (dout_bias).  Pass NULL for the tensors the
 * plain form does not use. */
int sub_op_ln_backward(void* handle, int extended, const void* in, const char* l_in, const void* scale,
                       const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                       const void* dlinear, const char* l_dlinear, const void* istd, const char* l_istd,
                       const void* diff, const char* l_diff, const void* mask, const char* l_mask, void* g,
                       const char* l_g, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                       const char* l_d_drop_in, void* dscale, void* dbias, void* dlinear_bias, void* dout_bias);
/* sub_op_ln_backward for callers that cannot allocate device memory -- code under a
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments; for rows of up to 1024 features the
 * same kernels and bit-identical results.  Rows of 1032 to 4096 features run as the
 * separate operators here, where sub_op_ln_backward may take its one-launch form:
 * the scaled gradient is bit-identical, the other outputs add the same terms in
 * another order and agree to fp16 rounding.  The fp32 partial rows of the column
 * sums (which sub_op_ln_backward keeps
 * in a buffer the handle allocates on first use) live in a 4 MiB array that is part
 * of the library's device image, one copy per GPU for the life of the process.
 * Nothing is allocated or freed.  A call whose partial rows would need more than
 * SUB_STATIC_SCRATCH_BYTES fails with a message, launching nothing; the way the
 * rows are dealt out keeps every shape this operator takes within it (at most 256
 * partial rows of up to 1024 features for each of four sums in the one-launch form,
 * at most 3 MiB for the separate operators on longer rows).  All calls on one GPU, from
 * whatever handle or stream, share the array: calls that may overlap on a GPU race.
 * The first call on a GPU looks the array's address up (no allocation); make it
 * outside a graph capture. */
#define SUB_STATIC_SCRATCH_BYTES (4u << 20)
int sub_op_ln_backward_static(void* handle, int extended, const void* in, const char* l_in, const void* scale,
                              const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                              const void* dlinear, const char* l_dlinear, const void* istd, const char* l_istd,
                              const void* diff, const char* l_diff, const void* mask, const char* l_mask, void* g,
                              const char* l_g, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                              const char* l_d_drop_in, void* dscale, void* dbias, void* dlinear_bias,
                              void* dout_bias);
/* Measurement only, no counterpart in the reference and no handle: `workgroups` workgroups of eight waves
 * (one per CU at 256) each read `iters` chunks of 64 KiB -- the operand bytes of one k-step of a 256 x 256
 * tile -- from the `working_set` bytes at buf (device memory, a multiple of 64 KiB), with asynchronous loads
 * into LDS (to_lds = 1) or plain 128-bit loads into registers (to_lds = 0), every workgroup from a start of
 * its own.  A working set below one XCD's 4 MiB of L2 measures what the L2s deliver to the CUs, a larger one
 * the path beyond them.  to_lds = 2: a copy instead -- every chunk read is also written, to the `working_set`
 * bytes behind the first (buf holds 2 x working_set; nontemporal accesses, as the fused operators use them for
 * tensors on their last read or written for a later pass); to_lds = 3: only those writes (a fill).  In these
 * two forms workgroup w takes chunks w, w + workgroups, ...: with workgroups x iters = working_set / 65536 every
 * chunk is touched once.  *us = duration of the launch (second of two), *mhz = shader clock during it (median
 * over the workgroups of cycle counter / wall counter).  Bytes read (and/or written) = workgroups x iters x
 * 65536.  Allocates and frees a few KiB per call and synchronises the stream. */
int sub_probe_fetch(const void* buf, size_t working_set, int to_lds, int iters, int workgroups, void* stream,
                    float* us, float* mhz);
/* dst (order l_dst) = src (order l_src): the same tensor in another dimension order (any two permutations
 * of the same dims; 128-bit accesses on both sides through 64 x 64 tiles in LDS when the sizes of the two
 * contiguous dims are multiples of 8).  No counterpart in the reference, whose kernels are generated per
 * layout; here it carries tensors across the boundary of SUB_OPT_PRIVATE_LAYOUTS.  src and dst must not overlap. */
int sub_op_relayout(void* handle, const void* src, const char* l_src, void* dst, const char* l_dst);
/* block_bei.cuh:58-106 */
int sub_op_bei(void* handle, const void* dxatt, const char* l_dxatt, const void* dresid1,
               const char* l_dresid1, void* dx, const char* l_dx);
/* gemm.cuh:134-147 `Einsum<Real, lA, lB, lC>::run`: C = alpha * einsum(A, B),
 * dimension roles derived from the three layout strings (einsumparser.h:9-55). */
int sub_op_einsum(void* handle, const void* A, const char* l_A, const void* B, const char* l_B,
                  void* C, const char* l_C, float alpha);
/* The same with an addend in the epilogue: C = alpha * einsum(A, B) + T, where the
 * dims of T are free or batch dims of C (the others broadcast): a projection and
 * its bias (gemm.cuh:134-147 followed by block_aib.cuh:17-155, or the `linear` of
 * substation/transformer.py:41-52 with its bias), or a product added to a residual
 * (block_bei.cuh:12-106).  T may be C (accumulate in place).  Fails when the layouts
 * lead to a kernel that has no epilogue. */
/* The feed-forward activation in the epilogues of the products next to it, as
 * encoder_forward / encoder_backward run them under SUB_OPT_RELU_FROM_OUTPUT:
 * sub_op_einsum_bad: out = dropout(act(einsum(A, B) + bias)) (gemm.cuh:134-147 followed
 * by block_bad.cuh:28-145) with the handle's activation and the keep bits of (seed,
 * step, site, p); `out` in BJU order; `bits` receives B*J*U/8 bytes (ReLU: one bit per
 * output, set where it is positive; GELU: the keep bits) in the kernel's own order, for
 * sub_op_einsum_bdrlb only; GELU also stores the pre-activation to `lin`, laid out like
 * `out` (ReLU: ignored, may be null).
 * sub_op_einsum_bdrlb: dlinear = act'(.) * keep * einsum(A, B) and dbias = its sum over
 * the tokens (gemm.cuh:134-147 followed by block_bdrlb.cuh:13-146); `gate` is the forward
 * output (ReLU) or the pre-activation (GELU), laid out like `dlinear` (BJU), `bits`
 * what sub_op_einsum_bad left.
 * *applied = 0 and nothing launched when the product does not qualify for the kernel
 * that carries these epilogues (whole 256 x 256 tiles for most of the CUs, 16-byte
 * aligned tensors): the caller then runs the product and the operator one after the other. */
int sub_op_einsum_bad(void* handle, const void* A, const char* l_A, const void* B, const char* l_B, const void* bias,
                      const char* l_bias, void* lin, void* out, const char* l_out, void* bits, float p, uint32_t site,
                      int* applied);
int sub_op_einsum_bdrlb(void* handle, const void* A, const char* l_A, const void* B, const char* l_B, const void* gate,
                        const char* l_gate, const void* bits, void* dlinear, const char* l_dlinear, void* dbias,
                        int* applied);
/* Two independent contractions, the first with an optional addend T1 (null: none) as
 * in sub_op_einsum_add, in one launch where the pair qualifies (a data gradient and the
 * weight gradient next to it, as encoder_backward pairs dXlin1 with dWlin1 and dXQKV with
 * dWQKV: gemm.cuh:134-147 twice, encoder.cu:235-239,268-276), else one after the other;
 * *paired (optional) says which.  Same results either way.  Neither output may be an
 * input of the other product. */
int sub_op_einsum_pair(void* handle, const void* A1, const char* l_A1, const void* B1, const char* l_B1,
                       const void* T1, const char* l_T1, void* C1, const char* l_C1, float alpha1,
                       const void* A2, const char* l_A2, const void* B2, const char* l_B2, void* C2,
                       const char* l_C2, float alpha2, int* paired);
int sub_op_einsum_add(void* handle, const void* A, const char* l_A, const void* B, const char* l_B,
                      const void* T, const char* l_T, void* C, const char* l_C, float alpha);

/* ---- host-only helpers (no GPU needed) ------------------------------------- */

/* metahelpers.h:61-78: element strides of `layout` for dims "BJKHPIUQ"
 * (0 for absent dims) under the handle's sizes. */
int sub_layout_strides(void* handle, const char* layout, int64_t strides[8]);
/* einsumparser.h:9-55.  out = {batch, M, N, K, sAM, sAK, sAB0, sBN, sBK, sBB0,
 * sCM, sCN, sCB0, nbatchdims, K0, sAK0, sBK0, kernel_kind (0 scalar, 1 MFMA),
 * nb[3], sAb[3], sBb[3], sCb[3], K1, 0}: up to three batch dims with their own
 * strides (0 where an operand lacks the dim) and K = K0 * K1 (outer x inner
 * contraction group). */
int sub_einsum_classify(void* handle, const char* l_A, const char* l_B, const char* l_C,
                        int64_t out[32]);
/* The 16-bit random fields of canonical elements start .. start+n-1, computed
 * on the host by the same code the kernels run. */
int sub_philox_fields_host(uint64_t seed, uint32_t site, uint32_t step, uint64_t start,
                           uint64_t n, uint16_t* out);
/* Drop threshold used for probability p: keep iff field >= threshold. */
uint32_t sub_dropout_threshold(float p);

#ifdef __cplusplus
}
#endif
#endif /* SUBSTATION_AMD_H */
