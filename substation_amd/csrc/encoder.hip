// Encoder-layer orchestration and the C ABI of libsubstation_amd.so.
// Counterpart of pytorch_module/encoder.cu (struct Encoder, the two operator
// sequences and the four extern "C" exports); the compile-time configuration of
// the generated encoder_parameters.cuh (pytorch_module/encoder.py:213-376) is
// a run-time sub_config here.
#include <hip/hip_runtime.h>

#include <cmath>
#include <map>
#include <algorithm>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/substation_amd.h"
#include "sub_common.hpp"
#include "sub_ops.hpp"

// Scratch of the entry point that allocates nothing (sub_op_ln_backward_static):
// the fp32 partial rows of its column sums live in this array instead of in a
// buffer from hipMalloc.  Every GPU the library runs on holds its own copy, at
// its own address, until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress, never a device address: host code
// hands the resolved pointer (static_scratch() below), and nothing else, to
// kernels.
constexpr size_t kStaticScratchFloats = SUB_STATIC_SCRATCH_BYTES / sizeof(float);     // 4 MiB
static __device__ __align__(256) float scratch[kStaticScratchFloats];

namespace sub {

namespace {

thread_local std::string g_last_error;

// ---------------------------------------------------------------------------
// Tensor tables: names in the reference's pickle order and canonical dims.
// ---------------------------------------------------------------------------
struct TensorDef { const char* name; const char* dims; };

const TensorDef kParams[SUB_N_PARAMS] = {
    {"WKQV", "QPHI"}, {"BKQV", "QPH"}, {"WO", "IPH"}, {"BO", "I"}, {"S1", "I"}, {"B1", "I"},
    {"LINB1", "U"}, {"LINW1", "IU"}, {"S2", "I"}, {"B2", "I"}, {"LINB2", "I"}, {"LINW2", "UI"}};
const TensorDef kFwd[SUB_N_FWD] = {
    {"KKQQVV", "QPHBJ"}, {"WKKWQQWVV", "QPHBJ"}, {"BETA", "HBJK"}, {"ALPHA", "HBJK"},
    {"ATTN_DROP_MASK", "HBJK"}, {"ATTN_DROP", "HBJK"}, {"GAMMA", "PHBJ"}, {"ATT", "BJI"},
    {"DROP1MASK", "BJI"}, {"SB1", "BJI"}, {"SB1_LINW1", "BJU"}, {"DROP2", "BJU"}, {"LIN1", "BJU"},
    {"DROP2_LINW2", "BJI"}, {"LIN2", "BJI"}, {"LN2", "BJI"}, {"LN2STD", "BJ"}, {"LN2DIFF", "BJI"},
    {"DROP2MASK", "BJU"}, {"DROP3MASK", "BJI"}, {"LN1", "BJI"}, {"LN1STD", "BJ"}, {"LN1DIFF", "BJI"}};
const TensorDef kBwd[SUB_N_BWD] = {
    {"DLN2", "BJI"}, {"DRESID2", "BJI"}, {"DLIN2", "BJI"}, {"DDROP2", "BJU"}, {"DLIN1", "BJU"},
    {"DLIN1_LINW1", "BJI"}, {"DLN1", "BJI"}, {"DRESID1", "BJI"}, {"DATT", "BJI"}, {"DXATT", "BJI"},
    {"DGAMMA", "PHBJ"}, {"DATTN_DROP", "HBJK"}, {"DBETA", "HBJK"}, {"DKKQQVV", "QPHBJ"}};

enum P { WKQV, BKQV, WO, BO, S1, B1, LINB1, LINW1, S2, B2, LINB2, LINW2 };
enum F { KKQQVV, WKKWQQWVV, BETA, ALPHA, ATTN_DROP_MASK, ATTN_DROP, GAMMA, ATT, DROP1MASK, SB1,
         SB1_LINW1, DROP2, LIN1, DROP2_LINW2, LIN2, LN2, LN2STD, LN2DIFF, DROP2MASK, DROP3MASK,
         LN1, LN1STD, LN1DIFF };
enum Bw { DLN2, DRESID2, DLIN2, DDROP2, DLIN1, DLIN1_LINW1, DLN1, DRESID1, DATT, DXATT, DGAMMA,
          DATTN_DROP, DBETA, DKKQQVV };

bool same_dims(const Layout& l, const char* dims) {
    size_t n = std::strlen(dims);
    if ((size_t)l.rank != n) return false;
    for (size_t i = 0; i < n; ++i) if (!l.has[dim_of(dims[i])]) return false;
    return true;
}

// ---------------------------------------------------------------------------
// Views
// ---------------------------------------------------------------------------
struct Space {
    RowSpace rs;
    int outer[4];   // logical dims of the four outer slots (-1: unused)
    int rdim;       // logical dim of the row
};

Space make_space(const Sizes& sz, std::initializer_list<int> outer, int rdim) {
    Space s;
    int n[4] = {1, 1, 1, 1};
    int k = 4 - (int)outer.size();
    for (int i = 0; i < 4; ++i) s.outer[i] = -1;
    for (int d : outer) { s.outer[k] = d; n[k] = (int)sz.n[d]; ++k; }
    s.rdim = rdim;
    s.rs.n0 = n[0]; s.rs.n1 = n[1]; s.rs.n2 = n[2]; s.rs.n3 = n[3];
    s.rs.R = (int)sz.n[rdim];
    s.rs.flat = (n[0] == 1 && n[1] == 1 && n[2] == 1) ? 1 : 0;
    return s;
}

// Merges adjacent outer dims that every view walks with one stride
// (s[i] == n[i+1] * s[i+1]), so that the kernels skip the row -> index
// divisions; the canonical row numbering (and with it the dropout mask) is
// unchanged.  `keep` leading outer dims are left alone (kept dims of the column
// reductions).
void flatten(RowSpace& rs, std::initializer_list<View*> views, int keep = 0) {
    int n[4] = {rs.n0, rs.n1, rs.n2, rs.n3};
    auto stride = [](View* v, int i) -> long& {
        return i == 0 ? v->s0 : i == 1 ? v->s1 : i == 2 ? v->s2 : v->s3;
    };
    bool changed = true;
    while (changed) {
        changed = false;
        for (int i = 2; i >= keep && !changed; --i) {
            bool ok = n[i] == 1;
            if (ok) {
                // an extent-1 dim is only worth dropping if a real dim lies outside it
                bool outer = false;
                for (int j = keep; j < i; ++j) outer = outer || n[j] != 1;
                if (!outer) continue;
            } else {
                ok = true;
                for (View* v : views) ok = ok && stride(v, i) == (long)n[i + 1] * stride(v, i + 1);
                if (!ok) continue;
            }
            n[i + 1] *= n[i];
            for (int j = i; j > keep; --j) {
                n[j] = n[j - 1];
                for (View* v : views) stride(v, j) = stride(v, j - 1);
            }
            n[keep] = 1;
            for (View* v : views) stride(v, keep) = 0;
            changed = true;
        }
    }
    rs.n0 = n[0]; rs.n1 = n[1]; rs.n2 = n[2]; rs.n3 = n[3];
    rs.flat = (n[0] == 1 && n[1] == 1 && n[2] == 1) ? 1 : 0;
}

View make_view(const void* p, const Layout& l, const Space& sp) {
    View v;
    v.p = (half_t*)p;
    long so[4];
    for (int i = 0; i < 4; ++i) so[i] = sp.outer[i] >= 0 && l.has[sp.outer[i]] ? l.stride[sp.outer[i]] : 0;
    v.s0 = so[0]; v.s1 = so[1]; v.s2 = so[2]; v.s3 = so[3];
    v.sr = l.has[sp.rdim] ? l.stride[sp.rdim] : 0;
    bool vec = v.sr == 1 && (sp.rs.R % 8 == 0) && ((reinterpret_cast<uintptr_t>(p) & 15) == 0);
    for (int i = 0; i < 4; ++i) vec = vec && (so[i] % 8 == 0);
    v.vec = vec ? 1 : 0;
    return v;
}

// A dense vector indexed by the row dim only ([I] or [U] parameters).
View vector_view(const void* p, int R) {
    View v;
    v.p = (half_t*)p;
    v.s0 = v.s1 = v.s2 = v.s3 = 0;
    v.sr = 1;
    v.vec = (R % 8 == 0) && ((reinterpret_cast<uintptr_t>(p) & 15) == 0) ? 1 : 0;
    return v;
}

// ---------------------------------------------------------------------------
// Handle
// ---------------------------------------------------------------------------
struct GemmPlan {
    GemmShape shape;
    float alpha = 1.f;
    bool ok = false;                  // fused variants only: the plan is usable
    int64_t sM = 0, sN = 0, sb[3] = {0, 0, 0};   // addend strides
};

// G_QKV_BIAS: QKV projection writing KKQQVV directly with BKQV added in the
// epilogue (replaces QKV-fused + aib).  G_DXQKV_RESID: input-gradient projection
// writing DX directly with DRESID1 added (replaces dXQKV-fused + bei).
enum G { G_QKV_BIAS, G_DXQKV_RESID, G_LIN1_BAD, G_DXLIN2_BDRLB, G_QKV, G_QKT, G_GAMMA, G_OUT, G_LIN1, G_LIN2, G_DXLIN2, G_DWLIN2, G_DXLIN1, G_DWLIN1,
         G_DWOUT, G_DXOUT, G_DX1GAMMA, G_DX2GAMMA, G_DX1QKT, G_DX2QKT, G_DXQKV, G_DWQKV, G_COUNT };

// One event in front of every launch: a launch lasts from its event to the next
// one (the next launch's, or the marker that closes a pass: name == nullptr).
struct ProfEntry { const char* name; hipEvent_t a; };

// sub_profile_enable(handle, 2): besides the event, a one-lane kernel in front of every launch stores the
// shader clock counter (s_memtime) and the constant-rate wall clock (s_memrealtime); the ratio of their
// differences between two samples is the shader clock the GPU held during the launch between them.
// The shader clock counter is one per XCD and the eight do not agree, so every sample is taken by a
// number of one-lane workgroups (dealt round-robin over the XCDs), each storing its own pair; two
// samples are then compared pair by pair, and only pairs from the same XCD give a ratio that a clock can
// have (the counters of different XCDs lie far apart).
constexpr int kMaxClockSamples = 256;
constexpr int kClockSlots = 32;
__global__ void k_clock_sample(unsigned long long* slot) {
    slot[2 * blockIdx.x] = __builtin_readcyclecounter();
    slot[2 * blockIdx.x + 1] = wall_clock64();
}

struct Handle {
    bool configured = false;
    Sizes sz;
    int act = ACT_RELU;
    float p_softmax = 0, p_resid1 = 0, p_act = 0, p_resid2 = 0, eps = 1e-5f;
    uint64_t seed = 0;
    uint32_t step = 0;
    hipStream_t stream = nullptr;
    Layout lX, lY;
    Layout lp[SUB_N_PARAMS], lf[SUB_N_FWD], lb[SUB_N_BWD];
    // The dimension orders the caller configured (the orders above are what the launches use: the same, or,
    // under SUB_OPT_PRIVATE_LAYOUTS, the library's own -- see plan_layouts).
    Layout xX, xY;
    Layout xp[SUB_N_PARAMS], xf[SUB_N_FWD], xb[SUB_N_BWD];
    bool private_layouts = true;      // SUB_OPT_PRIVATE_LAYOUTS
    bool staging = false;             // the launches run in the library's own orders
    bool stage_x = false, stage_y = false, stage_p[SUB_N_PARAMS] = {};
    // staged copies in the library's orders: input, output, their gradients, weights and weight gradients
    half_t* sX = nullptr; half_t* sY = nullptr; half_t* sDY = nullptr; half_t* sDX = nullptr;
    half_t* sW[SUB_N_PARAMS] = {}; half_t* sDW[SUB_N_PARAMS] = {};
    // what the last forward call made sX / sW from (the backward call after it reuses them for the same pointers)
    const void* staged_x_from = nullptr; const void* staged_w_from[SUB_N_PARAMS] = {};
    int pos_p[SUB_N_PARAMS], pos_f[SUB_N_FWD], pos_b[SUB_N_BWD];   // internal id -> caller position
    Layout lKK, lQQ, lDKK, lDQQ, lWsub, lBsub;
    GemmPlan gemm[G_COUNT];
    float* ws = nullptr;          // column-reduction partials
    size_t ws_floats = 0;
    size_t ws_need_bwd = 0;       // sum over the backward pass's column reductions
    float* static_ws = nullptr;   // set for the duration of a call that must not allocate: take_ws hands it out
    bool deferring = false;       // backward pass: finish all column reductions in one launch
    bool ops_deferring = false;   // the same across operator calls, between sub_ops_defer(h, 1) and sub_ops_defer(h, 0)
    size_t ws_cursor = 0;
    FinishJobs deferred;
    float* gws = nullptr;         // split-k partials of the small-output contractions
    size_t gws_floats = 0, gws_need = 0;
    bool profiling = false;
    bool profile_clocks = false;      // profiling with clock samples (sub_profile_enable(handle, 2))
    unsigned long long* clock_buf = nullptr;   // kMaxClockSamples pairs (shader clock counter, wall clock)
    uint32_t* step_dev = nullptr;     // optional device-side dropout step (HIP-graph replays)
    const void* attn_mask = nullptr;  // optional additive [J,K] attention mask (caller-owned)
    Layout l_attn_mask;
    void* mask_plan = nullptr;        // what the mask leaves to do (see mask_plan())
    size_t mask_plan_bytes = 0;
    bool mask_plan_built = false;     // a forward pass has filled it for the present mask pointer
    bool fuse_epilogues = true;
    bool fuse_ln_backward = true;
    bool fuse_scores = true;
    int fuse_attention = 1;           // 0 off, 1 where possible, 2 required
    bool pair_products = true;        // a data gradient and the weight gradient next to it in one launch
    bool finish_in_pair = true;       // deferred column sums are finished inside the last pair launch of the backward pass
    bool relu_from_output = true;     // ReLU: the backward gate is read off DROP2; LIN1 and DROP2MASK are not produced
    int side_jobs = 1;                // bit 0: CUs that the stacked projections' tiles leave idle draw attention keep bits;
                                      // bit 1: workgroups behind the first LayerNorm launch draw lin1's keep bits
    bool packed_masks = true;         // DROP1MASK / DROP3MASK travel as one bit per element inside their buffers
    bool skip_unread = true;          // intermediates that neither pass reads are not written (ATT after its bias, LIN2, DLN2, DLN1)
    // where the last forward call's lin1 epilogue left one bit per element of DROP2 (set = positive), or
    // null: the unused SB1_LINW1 buffer of that call.  The backward call reads its gate from there when it
    // is handed the same buffer, and from DROP2 itself otherwise.
    const void* gate_bits_at = nullptr;
    std::vector<ProfEntry> prof;
    size_t prof_used = 0;
    size_t prof_forward = 0;          // entries of the last forward call, kept by the backward call after it

    ~Handle() {
        // A handle may be destroyed (e.g. by a garbage collector) while some other
        // stream of the process is being captured into a HIP graph; freeing this
        // handle's own scratch must not invalidate that capture.
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        const bool swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
        if (ws) (void)hipFree(ws);
        if (gws) (void)hipFree(gws);
        if (mask_plan) (void)hipFree(mask_plan);
        if (clock_buf) (void)hipFree(clock_buf);
        for (half_t* q : {sX, sY, sDY, sDX}) if (q) (void)hipFree(q);
        for (int i = 0; i < SUB_N_PARAMS; ++i) { if (sW[i]) (void)hipFree(sW[i]); if (sDW[i]) (void)hipFree(sDW[i]); }
        for (auto& e : prof) (void)hipEventDestroy(e.a);
        if (swapped) (void)hipThreadExchangeStreamCaptureMode(&mode);
    }
};

void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) fail(std::string(what) + ": " + hipGetErrorString(e));
}

// The address of `scratch` (top of this file) on the current device: resolved
// once per device, with that device current, and kept.
constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

float* static_scratch() {
    int dev = -1;
    hip_check(hipGetDevice(&dev), "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) fail("static scratch: device index out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        hip_check(hipGetSymbolAddress(&p, HIP_SYMBOL(::scratch)), "hipGetSymbolAddress(scratch)");
        if (!p) fail("static scratch: the symbol has no address on this device");
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    return g_scratch_ptr[dev];
}

// The two residual dropout masks as bits (SUB_OPT_PACKED_MASKS): rows must be whole 8-packs.
bool packed_masks(const Handle& h) { return h.packed_masks && h.sz.n[dI] % 8 == 0; }

PhiloxKey make_key(const Handle& h, uint32_t site, float p) {
    PhiloxKey k;
    k.k0 = (uint32_t)h.seed; k.k1 = (uint32_t)(h.seed >> 32);
    k.site = site; k.step = h.step; k.thr = threshold16(p);
    k.step_dev = h.step_dev;
    return k;
}

struct ProfScope {
    Handle& h; bool used = false;
    ProfScope(Handle& h_, const char* name) : h(h_) {
        if (!h.profiling) return;
        if (h.prof_used == h.prof.size()) {
            ProfEntry n{name, nullptr};
            hip_check(hipEventCreate(&n.a), "hipEventCreate");
            h.prof.push_back(n);
        }
        ProfEntry& e = h.prof[h.prof_used++];
        e.name = name;
        hip_check(hipEventRecord(e.a, h.stream), "hipEventRecord");
        if (h.profile_clocks && h.prof_used <= (size_t)kMaxClockSamples)
            hipLaunchKernelGGL(k_clock_sample, dim3(kClockSlots), dim3(1), 0, h.stream, h.clock_buf + 2 * kClockSlots * (h.prof_used - 1));
        used = true;
    }
    // nothing was launched: the entry goes (its event stays in the stream, harmless)
    void cancel() { if (used) { --h.prof_used; used = false; } }
};
// Closes the last launch of a pass.
void prof_mark_end(Handle& h) { ProfScope end(h, nullptr); }

// Allocations happen on the first call of a handle; that call cannot be part
// of a graph capture.
void refuse_capture(const Handle& h, const char* what) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(h.stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone)
        fail(std::string(what) + ": the scratch buffers are allocated by the first forward/backward call, "
             "run one outside the graph capture first");
}

void ensure_ws(Handle& h, size_t floats) {
    if (floats <= h.ws_floats) return;
    refuse_capture(h, "column-sum workspace");
    if (h.ws) hip_check(hipFree(h.ws), "hipFree");
    h.ws = nullptr; h.ws_floats = 0;
    hip_check(hipMalloc((void**)&h.ws, floats * sizeof(float)), "hipMalloc(workspace)");
    h.ws_floats = floats;
}

// Scratch for one column reduction.  While a backward pass defers the finishing
// stage, every reduction gets its own region of the (pre-sized) buffer.
float* take_ws(Handle& h, size_t floats) {
    if (h.static_ws) {
        if (floats > kStaticScratchFloats)
            fail("the column sums of this call need " + std::to_string(floats * sizeof(float)) +
                 " bytes of scratch, more than the " + std::to_string(kStaticScratchFloats * sizeof(float)) +
                 " bytes of the static scratch array");
        return h.static_ws;
    }
    if (!h.deferring) {
        ensure_ws(h, floats);
        return h.ws;
    }
    if (h.ws_cursor + floats > h.ws_floats) {
        // Out of room (operator calls that defer size nothing ahead): finish what is on the list, whose
        // partials the stream has complete by then, and start over at the front of the buffer.
        if (!h.ops_deferring) fail("column-reduction workspace exhausted");
        if (h.deferred.n > 0) launch_colfinish(h.deferred, h.stream);
        h.deferred.n = 0;
        h.ws_cursor = 0;
        // twice the size as well: after a few calls the buffer holds every reduction of a block of calls
        ensure_ws(h, floats > 2 * h.ws_floats ? floats : 2 * h.ws_floats);
    }
    float* p = h.ws + h.ws_cursor;
    h.ws_cursor += (floats + 63) & ~(size_t)63;
    return p;
}
// (a call on the static scratch array has one region for all its reductions: nothing is put off there)
FinishJobs* defer_of(Handle& h) { return h.deferring && !h.static_ws ? &h.deferred : nullptr; }

// ---------------------------------------------------------------------------
// Configuration
// ---------------------------------------------------------------------------
template <int N>
void bind_tensors(const TensorDef (&defs)[N], const char* const* names, const char* const* layouts,
                  const Sizes& sz, Layout* out, int* pos, const char* what) {
    bool seen[N] = {false};
    for (int i = 0; i < N; ++i) {
        if (!names[i] || !layouts[i]) fail(std::string(what) + ": null name or layout");
        int id = -1;
        for (int j = 0; j < N; ++j) if (std::strcmp(names[i], defs[j].name) == 0) id = j;
        if (id < 0) fail(std::string(what) + ": unknown tensor name " + names[i]);
        if (seen[id]) fail(std::string(what) + ": tensor listed twice: " + names[i]);
        seen[id] = true;
        out[id] = make_layout(layouts[i], sz);
        if (!same_dims(out[id], defs[id].dims))
            fail(std::string("layout of ") + names[i] + " must be a permutation of " + defs[id].dims +
                 ", got " + layouts[i]);
        pos[id] = i;
    }
}

void plan_gemm(Handle& h, int id, const Layout& a, const Layout& b, const Layout& c, float alpha,
               const char* name) {
    try {
        h.gemm[id].shape = classify_einsum(a, b, c);
    } catch (const Error& e) {
        fail(std::string(name) + " (" + a.str() + "," + b.str() + "->" + c.str() + "): " + e.what());
    }
    h.gemm[id].alpha = alpha;
}

void plan_layouts(Handle& h, bool own);
void drop_staged(Handle& h);

void configure(Handle& h, const sub_config* c) {
    if (!c) fail("sub_configure: null config");
    if (c->abi_version != SUB_ABI_VERSION) fail("sub_configure: ABI version mismatch");
    if (c->dtype != SUB_DTYPE_F16) fail("sub_configure: only fp16 tensors are supported");
    if (c->batch <= 0 || c->seq <= 0 || c->heads <= 0 || c->embed <= 0) fail("sub_configure: sizes must be positive");
    if (c->embed % c->heads != 0) fail("sub_configure: embed must be a multiple of heads");
    if (c->activation != SUB_ACT_RELU && c->activation != SUB_ACT_GELU) fail("sub_configure: unknown activation");
    const float ps[4] = {c->p_softmax, c->p_resid1, c->p_act, c->p_resid2};
    for (float p : ps) if (!(p >= 0.f && p <= 1.f)) fail("sub_configure: dropout probability outside [0,1]");
    h.configured = false;
    // a handle that is configured again forgets the attention mask of its old sizes
    // (the table of what the mask leaves to do was sized for them)
    if (h.mask_plan) {
        refuse_capture(h, "sub_configure");
        hip_check(hipFree(h.mask_plan), "hipFree(mask plan)");
    }
    h.mask_plan = nullptr; h.mask_plan_bytes = 0; h.mask_plan_built = false; h.attn_mask = nullptr;
    drop_staged(h);
    Sizes sz;
    sz.n[dB] = c->batch; sz.n[dJ] = c->seq; sz.n[dK] = c->seq; sz.n[dH] = c->heads;
    sz.n[dP] = c->embed / c->heads; sz.n[dI] = c->embed;
    sz.n[dU] = c->intermediate > 0 ? c->intermediate : 4 * (int64_t)c->embed; sz.n[dQ] = 3;
    h.sz = sz;
    h.act = c->activation;
    h.p_softmax = c->p_softmax; h.p_resid1 = c->p_resid1; h.p_act = c->p_act; h.p_resid2 = c->p_resid2;
    h.eps = c->ln_eps > 0.f ? c->ln_eps : 1e-5f;
    h.seed = c->seed; h.step = 0;
    h.xX = make_layout(c->input_layout, sz);
    h.xY = make_layout(c->output_layout, sz);
    if (!same_dims(h.xX, "BJI") || !same_dims(h.xY, "BJI")) fail("input/output layout must be a permutation of BJI");
    bind_tensors(kParams, c->param_names, c->param_layouts, sz, h.xp, h.pos_p, "params");
    bind_tensors(kFwd, c->fwd_names, c->fwd_layouts, sz, h.xf, h.pos_f, "forward_interm");
    bind_tensors(kBwd, c->bwd_names, c->bwd_layouts, sz, h.xb, h.pos_b, "backward_interm");
    // the caller's orders must be usable as they are (debug capture and SUB_OPT_PRIVATE_LAYOUTS = 0 run in them)
    plan_layouts(h, false);
    if (h.private_layouts) plan_layouts(h, true);
    h.configured = true;
}

// The dimension orders the launches run in, and everything that follows from them (contraction plans,
// scratch sizes).  own = false: the caller's.  own = true (SUB_OPT_PRIVATE_LAYOUTS): when an activation of the
// caller's configuration is not in the order the fused paths of this library need -- token-major rows with the
// feature dim contiguous; the reference's shipped configurations are feature-major -- every intermediate
// lives in the library's own order inside the caller's buffer (same number of elements), and the tensors that
// cross the boundary (input, output, their gradients, weights, weight gradients) are copied into that order and
// back by k_relayout.  A configuration whose activations are all in the library's orders runs as it is, with
// its own weight orders.
void plan_layouts(Handle& h, bool own) {
    const Sizes& sz = h.sz;
    static const char* const kOwnP[SUB_N_PARAMS] = {"QHPI", "QHP", "IHP", "I", "I", "I", "U", "UI", "I", "I", "I", "IU"};
    static const char* const kOwnF[SUB_N_FWD] = {
        "QBJHP", "QBJHP", "HBJK", "HBJK", "HBJK", "HBJK", "BJHP", "BJI", "BJI", "BJI", "BJU", "BJU", "BJU",
        "BJI", "BJI", "BJI", "BJ", "BJI", "BJU", "BJI", "BJI", "BJ", "BJI"};
    static const char* const kOwnB[SUB_N_BWD] = {
        "BJI", "BJI", "BJI", "BJU", "BJU", "BJI", "BJI", "BJI", "BJI", "BJI", "BJHP", "HBJK", "HBJK", "QBJHP"};
    bool differs = false;
    if (own) {
        differs = h.xX.str() != "BJI" || h.xY.str() != "BJI";
        for (int i = 0; i < SUB_N_FWD; ++i) differs = differs || h.xf[i].str() != kOwnF[i];
        for (int i = 0; i < SUB_N_BWD; ++i) differs = differs || h.xb[i].str() != kOwnB[i];
    }
    h.staging = own && differs;
    h.stage_x = h.stage_y = false;
    for (int i = 0; i < SUB_N_PARAMS; ++i) h.stage_p[i] = false;
    h.staged_x_from = nullptr;
    for (int i = 0; i < SUB_N_PARAMS; ++i) h.staged_w_from[i] = nullptr;
    if (h.staging) {
        h.lX = make_layout("BJI", sz); h.lY = make_layout("BJI", sz);
        h.stage_x = h.xX.str() != "BJI"; h.stage_y = h.xY.str() != "BJI";
        for (int i = 0; i < SUB_N_PARAMS; ++i) {
            h.lp[i] = make_layout(kOwnP[i], sz);
            h.stage_p[i] = h.xp[i].str() != kOwnP[i];
        }
        for (int i = 0; i < SUB_N_FWD; ++i) h.lf[i] = make_layout(kOwnF[i], sz);
        for (int i = 0; i < SUB_N_BWD; ++i) h.lb[i] = make_layout(kOwnB[i], sz);
    } else {
        h.lX = h.xX; h.lY = h.xY;
        for (int i = 0; i < SUB_N_PARAMS; ++i) h.lp[i] = h.xp[i];
        for (int i = 0; i < SUB_N_FWD; ++i) h.lf[i] = h.xf[i];
        for (int i = 0; i < SUB_N_BWD; ++i) h.lb[i] = h.xb[i];
    }

    // Sub-tensors of the Q-stacked tensors (pytorch_module/encoder.py:318-362).
    Layout kq = drop_front(h.lf[KKQQVV], dQ);
    h.lQQ = kq; h.lKK = rename_dim(kq, dJ, dK);
    Layout dkq = drop_front(h.lb[DKKQQVV], dQ);
    h.lDQQ = dkq; h.lDKK = rename_dim(dkq, dJ, dK);
    (void)drop_front(h.lf[WKKWQQWVV], dQ);
    (void)drop_front(h.lp[WKQV], dQ);
    (void)drop_front(h.lp[BKQV], dQ);

    const float a = 1.0f / std::sqrt((float)sz.n[dP]);
    // forward (pytorch_module/encoder.cu:87-157)
    plan_gemm(h, G_QKV, h.lX, h.lp[WKQV], h.lf[WKKWQQWVV], 1.f, "QKV-fused");
    plan_gemm(h, G_QKT, h.lKK, h.lQQ, h.lf[BETA], a, "QKT");
    plan_gemm(h, G_GAMMA, h.lKK, h.lf[ATTN_DROP], h.lf[GAMMA], 1.f, "gamma");
    plan_gemm(h, G_OUT, h.lp[WO], h.lf[GAMMA], h.lf[ATT], 1.f, "out");
    plan_gemm(h, G_LIN1, h.lf[SB1], h.lp[LINW1], h.lf[SB1_LINW1], 1.f, "lin1");
    plan_gemm(h, G_LIN2, h.lf[DROP2], h.lp[LINW2], h.lf[DROP2_LINW2], 1.f, "lin2");
    // backward (pytorch_module/encoder.cu:158-299)
    plan_gemm(h, G_DXLIN2, h.lb[DLIN2], h.lp[LINW2], h.lb[DDROP2], 1.f, "dXlin2");
    plan_gemm(h, G_DWLIN2, h.lb[DLIN2], h.lf[DROP2], h.lp[LINW2], 1.f, "dWlin2");
    plan_gemm(h, G_DXLIN1, h.lb[DLIN1], h.lp[LINW1], h.lb[DLIN1_LINW1], 1.f, "dXlin1");
    plan_gemm(h, G_DWLIN1, h.lb[DLIN1], h.lf[SB1], h.lp[LINW1], 1.f, "dWlin1");
    plan_gemm(h, G_DWOUT, h.lf[GAMMA], h.lb[DATT], h.lp[WO], 1.f, "dWout");
    plan_gemm(h, G_DXOUT, h.lp[WO], h.lb[DATT], h.lb[DGAMMA], 1.f, "dXout");
    plan_gemm(h, G_DX1GAMMA, h.lKK, h.lb[DGAMMA], h.lb[DATTN_DROP], 1.f, "dX1gamma");
    plan_gemm(h, G_DX2GAMMA, h.lb[DGAMMA], h.lf[ATTN_DROP], h.lDKK, 1.f, "dX2gamma");
    plan_gemm(h, G_DX1QKT, h.lKK, h.lb[DBETA], h.lDQQ, a, "dX1QKT");
    plan_gemm(h, G_DX2QKT, h.lQQ, h.lb[DBETA], h.lDKK, a, "dX2QKT");
    plan_gemm(h, G_DXQKV, h.lp[WKQV], h.lb[DKKQQVV], h.lb[DXATT], 1.f, "dXQKV-fused");
    plan_gemm(h, G_DWQKV, h.lX, h.lb[DKKQQVV], h.lp[WKQV], 1.f, "dWQKV-fused");

    // Optional epilogue fusions; they need the addend to be N-contiguous like the
    // output after the kernel's operand swap, which gemm_kernel_kind checks.
    auto plan_fused = [&](int id, const Layout& la, const Layout& lb2, const Layout& lc, const Layout& lt) {
        GemmPlan& p = h.gemm[id];
        p.ok = false;
        try {
            p.shape = classify_einsum(la, lb2, lc);
        } catch (const Error&) {
            return;
        }
        p.alpha = 1.f;
        if (!addend_strides(p.shape, lt, lc, p.sM, p.sN, p.sb)) return;
        GemmEpilogue ep; ep.bias = (const half_t*)16; ep.sbM = p.sM; ep.sbN = p.sN;
        for (int i = 0; i < 3; ++i) ep.sbb[i] = p.sb[i];
        p.ok = gemm_kernel_kind(p.shape, (const void*)16, (const void*)16, (const void*)16, ep) == 1;
    };
    plan_fused(G_QKV_BIAS, h.lX, h.lp[WKQV], h.lf[KKQQVV], h.lp[BKQV]);
    plan_fused(G_DXQKV_RESID, h.lp[WKQV], h.lb[DKKQQVV], h.lX, h.lb[DRESID1]);
    // lin1 with LINB1, ReLU and dropout in its epilogue (writes DROP2; SB1_LINW1 is not produced): DROP2 must be
    // dense in canonical order, since the keep bits are indexed by the canonical element index
    plan_fused(G_LIN1_BAD, h.lf[SB1], h.lp[LINW1], h.lf[DROP2], h.lp[LINB1]);
    if (h.gemm[G_LIN1_BAD].ok) {
        GemmPlan& p = h.gemm[G_LIN1_BAD];
        GemmEpilogue ep; ep.bias = (const half_t*)16; ep.sbM = p.sM; ep.sbN = p.sN; ep.relu_dropout = true;
        p.ok = h.lf[DROP2].str() == "BJU" &&
               gemm_relu_dropout_ok(p.shape, (const void*)16, (const void*)16, (const void*)16, ep);
    }

    // dXlin2 with the ReLU layer's bdrlb in its epilogue (gate read off DROP2, writes DLIN1 and partial column sums for
    // DLINB1; DDROP2 is not produced)
    plan_fused(G_DXLIN2_BDRLB, h.lb[DLIN2], h.lp[LINW2], h.lb[DLIN1], h.lf[DROP2]);
    if (h.gemm[G_DXLIN2_BDRLB].ok) {
        GemmPlan& p = h.gemm[G_DXLIN2_BDRLB];
        GemmEpilogue ep; ep.gate = (const half_t*)16; ep.colsum = (float*)16; ep.sbM = p.sM; ep.sbN = p.sN;
        p.ok = p.sb[0] == 0 && gemm_relu_dropout_ok(p.shape, (const void*)16, (const void*)16, (const void*)16, ep);
    }

    {   // scratch of the five column reductions of one backward pass, side by side
        Space si = make_space(sz, {dB, dJ}, dI), su = make_space(sz, {dB, dJ}, dU);
        Space sq = make_space(sz, {dQ, dH, dB, dJ}, dP);
        RowSpace merged{1, (int)sz.n[dQ], (int)sz.n[dB], (int)sz.n[dJ], (int)(sz.n[dH] * sz.n[dP]), 0};
        size_t baib = colreduce_ws_floats(sq.rs, 1), baib2 = colreduce_ws_floats(merged, 1);
        h.ws_need_bwd = colreduce_ws_floats(si.rs, 2) + colreduce_ws_floats(si.rs, 3) +
                        colreduce_ws_floats(su.rs, 1) + colreduce_ws_floats(si.rs, 1) +
                        (baib > baib2 ? baib : baib2) + 8 * 64;
        // the fused LayerNorm-backward launches replace four of those reductions;
        // size for whichever set is larger
        size_t fused = lnbwd_ws_floats(si.rs, false) + lnbwd_ws_floats(si.rs, true) +
                       colreduce_ws_floats(su.rs, 1) + (baib > baib2 ? baib : baib2) + 8 * 64;
        if (fused > h.ws_need_bwd) h.ws_need_bwd = fused;
        // the attention kernels' partial sums for the projection-bias gradient stand in for baib's
        const size_t attn_bias = (size_t)(3 * sz.n[dH] * sz.n[dB] * ((sz.n[dJ] + 127) / 128) * sz.n[dP]);
        if (attn_bias > (baib > baib2 ? baib : baib2)) h.ws_need_bwd += attn_bias;
        // the partial column sums of dXlin2's epilogue (one row per 128 tokens)
        h.ws_need_bwd += (size_t)((sz.n[dB] * sz.n[dJ] + 127) / 128) * sz.n[dU] + 64;
    }
    h.gws_need = 0;
    for (int i = 0; i < G_COUNT; ++i) {
        size_t n = gemm_splitk_ws_floats(h.gemm[i].shape);
        if (n > h.gws_need) h.gws_need = n;
    }
    // The fp32 scratch of the column reductions is allocated by the first
    // operator that needs it, so that configuring needs no GPU.
}

// ---------------------------------------------------------------------------
// Operators on a handle
// ---------------------------------------------------------------------------
// fp32 scratch for the split contractions of small outputs, grown on demand
void ensure_gws(Handle& h, size_t floats) {
    if (floats <= h.gws_floats) return;
    refuse_capture(h, "split-k workspace");
    if (h.gws) hip_check(hipFree(h.gws), "hipFree");
    h.gws = nullptr; h.gws_floats = 0;
    hip_check(hipMalloc((void**)&h.gws, floats * sizeof(float)), "hipMalloc(split-k workspace)");
    h.gws_floats = floats;
}

void run_gemm(Handle& h, int id, const void* A, const void* B, void* C, const char* name,
              const void* addend = nullptr, GemmSideJob* side = nullptr) {
    ProfScope ps(h, name);
    const GemmPlan& p = h.gemm[id];
    GemmEpilogue ep;
    if (addend) {
        ep.bias = (const half_t*)addend; ep.sbM = p.sM; ep.sbN = p.sN;
        for (int i = 0; i < 3; ++i) ep.sbb[i] = p.sb[i];
    }
    ensure_gws(h, h.gws_need);
    launch_gemm(p.shape, (const half_t*)A, (const half_t*)B, (half_t*)C, p.alpha, ep, h.stream, h.gws,
                h.gws_floats, side);
}

// Two products that do not depend on one another (a data gradient and the weight
// gradient next to it) in one launch where they qualify, else one after the other.
GemmEpilogue addend_epilogue(const GemmPlan& p, const void* addend) {
    GemmEpilogue e;
    if (addend) {
        e.bias = (const half_t*)addend; e.sbM = p.sM; e.sbN = p.sN;
        for (int i = 0; i < 3; ++i) e.sbb[i] = p.sb[i];
    }
    return e;
}

void run_gemm_pair(Handle& h, int id1, const void* A1, const void* B1, void* C1, const char* name1,
                   const void* addend1, int id2, const void* A2, const void* B2, void* C2, const char* name2,
                   const char* pair_name, FinishJobs* tail = nullptr, PairThird* third = nullptr) {
    if (h.pair_products) {
        ProfScope ps(h, pair_name);
        const GemmPlan& p1 = h.gemm[id1];
        const GemmPlan& p2 = h.gemm[id2];
        ensure_gws(h, h.gws_need);
        if (launch_gemm_pair(p1.shape, (const half_t*)A1, (const half_t*)B1, (half_t*)C1, p1.alpha,
                             addend_epilogue(p1, addend1), p2.shape, (const half_t*)A2, (const half_t*)B2,
                             (half_t*)C2, p2.alpha, GemmEpilogue{}, h.stream, h.gws, h.gws_floats, tail, third))
            return;
        ps.cancel();
    }
    run_gemm(h, id1, A1, B1, C1, name1, addend1);
    run_gemm(h, id2, A2, B2, C2, name2);
}

// Would run_gemm_pair with these arguments take `third` into its launch?
bool pair_takes_third(Handle& h, int id1, const void* A1, const void* B1, void* C1, const void* addend1, int id2,
                      const void* A2, const void* B2, void* C2, const PairThird& third) {
    if (!h.pair_products) return false;
    const GemmPlan& p1 = h.gemm[id1];
    const GemmPlan& p2 = h.gemm[id2];
    ensure_gws(h, h.gws_need);
    return gemm_pair_takes_third(p1.shape, (const half_t*)A1, (const half_t*)B1, (half_t*)C1,
                                 addend_epilogue(p1, addend1), p2.shape, (const half_t*)A2, (const half_t*)B2,
                                 (half_t*)C2, GemmEpilogue{}, h.gws, h.gws_floats, third);
}

// Would run_gemm_pair run these two products as one launch?
bool pair_ok(Handle& h, int id1, const void* A1, const void* B1, void* C1, const void* addend1, int id2,
             const void* A2, const void* B2, void* C2) {
    if (!h.pair_products) return false;
    const GemmPlan& p1 = h.gemm[id1];
    const GemmPlan& p2 = h.gemm[id2];
    ensure_gws(h, h.gws_need);
    return gemm_pair_ok(p1.shape, (const half_t*)A1, (const half_t*)B1, (half_t*)C1, addend_epilogue(p1, addend1),
                        p2.shape, (const half_t*)A2, (const half_t*)B2, (half_t*)C2, GemmEpilogue{}, h.gws, h.gws_floats);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

void op_softmax(Handle& h, const void* beta, const Layout& lb, void* alpha, const Layout& la,
                void* mask, const Layout& lm, void* drop, const Layout& ld, float scale, float p,
                uint32_t site, const void* amask = nullptr, const Layout* lam = nullptr,
                float mscale = 1.f) {
    Space sp = make_space(h.sz, {dH, dB, dJ}, dK);
    View vb = make_view(beta, lb, sp), va = make_view(alpha, la, sp), vm = make_view(mask, lm, sp),
         vd = make_view(drop, ld, sp);
    View vam; vam.p = nullptr; vam.s0 = vam.s1 = vam.s2 = vam.s3 = 0; vam.sr = 0; vam.vec = 0;
    if (amask) {
        if (!lam || lam->rank != 2 || !lam->has[dJ] || !lam->has[dK])
            fail("softmax: the attention mask is a [J,K] tensor (layout JK or KJ)");
        vam = make_view(amask, *lam, sp);       // strides 0 along heads and samples
        flatten(sp.rs, {&vb, &va, &vm, &vd, &vam});
    } else {
        flatten(sp.rs, {&vb, &va, &vm, &vd});
    }
    launch_softmax(sp.rs, vb, va, vm, vd, vam, scale, mscale, make_key(h, site, p), h.stream);
}

void op_bs(Handle& h, const void* alpha, const Layout& la, const void* mask, const Layout& lm,
           const void* ddrop, const Layout& ld, void* dbeta, const Layout& lo, float scale) {
    Space sp = make_space(h.sz, {dH, dB, dJ}, dK);
    View va = make_view(alpha, la, sp), vm = make_view(mask, lm, sp), vd = make_view(ddrop, ld, sp),
         vo = make_view(dbeta, lo, sp);
    flatten(sp.rs, {&va, &vm, &vd, &vo});
    launch_bs(sp.rs, va, vm, vd, vo, scale, h.stream);
}

void op_bdrln(Handle& h, const void* in, const Layout& lin_, const void* resid, const Layout& lres,
              const void* linear_bias, const void* scale, const void* bias, void* lin,
              const Layout& llin, void* mask, const Layout& lmask, void* diff, const Layout& ldiff,
              void* normed, const Layout& lnorm, void* out, const Layout& lout, void* istd,
              const Layout& listd, float p, uint32_t site, bool packed_mask = false, bool write_lin = true,
              KeepWordsJob* side = nullptr) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    int R = sp.rs.R;
    View vi = make_view(in, lin_, sp), vr = make_view(resid, lres, sp), vl = make_view(lin, llin, sp),
         vm = make_view(mask, lmask, sp), vd = make_view(diff, ldiff, sp), vn = make_view(normed, lnorm, sp),
         vo = make_view(out, lout, sp), vs = make_view(istd, listd, sp);
    flatten(sp.rs, {&vi, &vr, &vl, &vm, &vd, &vn, &vo, &vs});
    launch_bdrln(sp.rs, vi, vr, vector_view(linear_bias, R), vector_view(scale, R), vector_view(bias, R),
                 vl, vm, vd, vn, vo, vs, make_key(h, site, p), h.eps, h.stream, packed_mask ? (uint8_t*)mask : nullptr,
                 write_lin, side);
}

void op_blnrd(Handle& h, const void* dout, const Layout& ldout, const void* istd, const Layout& listd,
              const void* diff, const Layout& ldiff, const void* mask, const Layout& lmask,
              void* d_ln_in, const Layout& l1, void* d_drop_in, const Layout& l2, bool packed_mask = false) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    View vg = make_view(dout, ldout, sp), vs = make_view(istd, listd, sp), vd = make_view(diff, ldiff, sp),
         vm = make_view(mask, lmask, sp), v1 = make_view(d_ln_in, l1, sp), v2 = make_view(d_drop_in, l2, sp);
    flatten(sp.rs, {&vg, &vs, &vd, &vm, &v1, &v2});
    launch_blnrd(sp.rs, vg, vs, vd, vm, v1, v2, h.stream, packed_mask ? (const uint8_t*)mask : nullptr);
}

void op_bad(Handle& h, const void* in, const Layout& lin_, const void* bias, void* lin,
            const Layout& llin, void* mask, const Layout& lmask, void* out, const Layout& lout,
            float p, uint32_t site, bool out_only = false) {
    Space sp = make_space(h.sz, {dB, dJ}, dU);
    View vi = make_view(in, lin_, sp), vl = make_view(lin, llin, sp), vm = make_view(mask, lmask, sp),
         vo = make_view(out, lout, sp);
    flatten(sp.rs, {&vi, &vl, &vm, &vo});
    launch_bad(sp.rs, vi, vector_view(bias, sp.rs.R), vl, vm, vo, h.act, make_key(h, site, p), h.stream, out_only);
}

void op_bsb(Handle& h, const void* in, const Layout& lin_, const void* scale, const void* dout,
            const Layout& ldout, void* din, const Layout& ldin, void* dscale, void* dbias) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    float* ws = take_ws(h, colreduce_ws_floats(sp.rs, 2));
    launch_bsb(sp.rs, make_view(in, lin_, sp), make_view(dout, ldout, sp), vector_view(scale, sp.rs.R),
               make_view(din, ldin, sp), ColOut{(half_t*)dscale}, ColOut{(half_t*)dbias}, ws, h.stream,
               defer_of(h));
}

void op_ebsb(Handle& h, const void* in, const Layout& lin_, const void* scale, const void* d1,
             const Layout& l1, const void* d2, const Layout& l2, const void* dlinear,
             const Layout& ldl, void* din, const Layout& ldin, void* dscale, void* dbias,
             void* dlinear_bias) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    float* ws = take_ws(h, colreduce_ws_floats(sp.rs, 3));
    launch_ebsb(sp.rs, make_view(in, lin_, sp), make_view(d1, l1, sp), make_view(d2, l2, sp),
                make_view(dlinear, ldl, sp), vector_view(scale, sp.rs.R), make_view(din, ldin, sp),
                ColOut{(half_t*)dscale}, ColOut{(half_t*)dbias}, ColOut{(half_t*)dlinear_bias}, ws,
                h.stream, defer_of(h));
}

void op_bdrlb(Handle& h, const void* ddrop, const Layout& ld, const void* mask, const Layout& lm,
              const void* lin, const Layout& ll, void* dlinear, const Layout& lo, void* dbias) {
    Space sp = make_space(h.sz, {dB, dJ}, dU);
    float* ws = take_ws(h, colreduce_ws_floats(sp.rs, 1));
    launch_bdrlb(sp.rs, make_view(ddrop, ld, sp), make_view(mask, lm, sp), make_view(lin, ll, sp),
                 make_view(dlinear, lo, sp), ColOut{(half_t*)dbias}, h.act, ws, h.stream, defer_of(h));
}

// The ReLU layer's bdrlb with the gate taken from the forward output DROP2 = relu(LIN1) * mask, which is
// positive exactly where the mask kept a positive LIN1 (block_bdrlb.cuh:72 reads the two separately).
void op_bdrlb_from_output(Handle& h, const void* ddrop, const Layout& ld, const void* out, const Layout& lo_,
                          void* dlinear, const Layout& lo, void* dbias) {
    Space sp = make_space(h.sz, {dB, dJ}, dU);
    float* ws = take_ws(h, colreduce_ws_floats(sp.rs, 1));
    launch_bdrlb_from_output(sp.rs, make_view(ddrop, ld, sp), make_view(out, lo_, sp), make_view(dlinear, lo, sp),
                             ColOut{(half_t*)dbias}, ws, h.stream, defer_of(h));
}

// Both passes decide this from the handle alone, so they agree.
bool relu_from_output(const Handle& h) { return h.relu_from_output && h.act == ACT_RELU; }
// GELU: lin1 with bias, activation and dropout in its epilogue (LIN1 and DROP2 written, the keep bits left in the
// SB1_LINW1 buffer instead of a DROP2MASK tensor) and dXlin2 with the backward of that in its epilogue.  Both or
// neither: without DROP2MASK the separate backward operator has nothing to read.
bool gelu_epilogues(const Handle& h) {
    return h.relu_from_output && h.act == ACT_GELU && h.fuse_epilogues && h.gemm[G_LIN1_BAD].ok &&
           h.gemm[G_DXLIN2_BDRLB].ok && h.lf[LIN1].str() == "BJU";
}
// What the forward call adds to that from the tensors it is handed.  The backward call is handed the same ones and
// asks the same question: it knows from the handle's options and these pointers alone whether the keep bits of
// the forward call it belongs to lie in SB1_LINW1 (whichever forward call of the handle that was).
bool lin1_takes_gelu_epilogue(const Handle& h, void* const* W, void* const* F) {
    return gelu_epilogues(h) && aligned16(F[LIN1]) && F[SB1_LINW1] && ((uintptr_t)F[SB1_LINW1] & 3) == 0 &&
           aligned16(W[LINB1]) && aligned16(F[DROP2]) && aligned16(F[SB1]) && aligned16(W[LINW1]);
}

void op_baob(Handle& h, const void* datt, const Layout& l, void* dbo) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    float* ws = take_ws(h, colreduce_ws_floats(sp.rs, 1));
    launch_baob(sp.rs, make_view(datt, l, sp), ColOut{(half_t*)dbo}, ws, h.stream, defer_of(h));
}

// Score rows straight from the projections: `ln` lays out the query-side rows
// ([B,J,H,P]-like), `lm` the key-side rows (its sequence dim is K).
bool score_args(const Handle& h, const void* rows_n, const Layout& ln, const void* rows_m, const Layout& lm,
                float alpha, ScoreArgs& a) {
    if (ln.rank != 4 || lm.rank != 4 || !ln.has[dP] || !lm.has[dP] || ln.stride[dP] != 1 || lm.stride[dP] != 1)
        return false;
    if (!ln.has[dJ] || !lm.has[dK] || !ln.has[dH] || !lm.has[dH] || !ln.has[dB] || !lm.has[dB]) return false;
    a.rows_n = (const half_t*)rows_n; a.rows_m = (const half_t*)rows_m;
    a.n_sh = ln.stride[dH]; a.n_sb = ln.stride[dB]; a.n_sr = ln.stride[dJ];
    a.m_sh = lm.stride[dH]; a.m_sb = lm.stride[dB]; a.m_sr = lm.stride[dK];
    a.alpha = alpha;
    (void)h;
    return true;
}

// QK^T + softmax + dropout in one launch (BETA is not written).
bool op_scores_softmax(Handle& h, const void* qq, const void* kk, void* alpha, const Layout& la, void* mask,
                       const Layout& lm, void* drop, const Layout& ld) {
    if (h.attn_mask) return false;
    ScoreArgs a;
    if (!score_args(h, qq, h.lQQ, kk, h.lKK, h.gemm[G_QKT].alpha, a)) return false;
    Space sp = make_space(h.sz, {dH, dB, dJ}, dK);
    View va = make_view(alpha, la, sp), vm = make_view(mask, lm, sp), vd = make_view(drop, ld, sp);
    return launch_scores_softmax(sp.rs, a, (int)h.sz.n[dP], va, vm, vd,
                                 make_key(h, SUB_SITE_SOFTMAX, h.p_softmax), h.stream);
}

// dO.V^T + softmax backward in one launch (DATTN_DROP is not written).
bool op_dscores_bs(Handle& h, const void* dgamma, const void* vv, const void* alpha, const Layout& la,
                   const void* mask, const Layout& lm, void* dbeta, const Layout& lo) {
    ScoreArgs a;
    if (!score_args(h, dgamma, h.lb[DGAMMA], vv, h.lKK, 1.f, a)) return false;
    Space sp = make_space(h.sz, {dH, dB, dJ}, dK);
    View va = make_view(alpha, la, sp), vm = make_view(mask, lm, sp), vo = make_view(dbeta, lo, sp);
    return launch_dscores_bs(sp.rs, a, (int)h.sz.n[dP], va, vm, vo, h.stream);
}

half_t* sub_q(void* base, const Handle& h, int q) {
    int64_t n = h.sz.n[dP] * h.sz.n[dH] * h.sz.n[dB] * h.sz.n[dJ];
    return (half_t*)base + (int64_t)q * n;
}

// Whole self-attention (scores, softmax, dropout, weighted sum) with the scores
// kept in registers.  The ALPHA buffer then holds, instead of probabilities, two
// fp32 values per score row (log-sum-exp, and in the backward pass the row sum of
// dO o O), and the ATTN_DROP_MASK buffer one keep bit per score.
bool attn_side(const void* p, const Layout& l, int pos_dim, AttnSide& s) {
    if (l.rank != 4 || !l.has[dP] || l.stride[dP] != 1 || !l.has[dH] || !l.has[dB] || !l.has[pos_dim]) return false;
    s.p = (const half_t*)p; s.sh = l.stride[dH]; s.sb = l.stride[dB]; s.sr = l.stride[pos_dim];
    return true;
}

// What sizes, layouts and options say; tensor alignment is checked per call.
bool attention_planned(const Handle& h) {
    if (!h.fuse_attention) return false;
    const Sizes& z = h.sz;
    if (!mha_shape_ok(z.n[dH], z.n[dB], z.n[dJ], z.n[dK], z.n[dP]) || !(h.gemm[G_QKT].alpha > 0.f)) return false;
    AttnSide t;
    return attn_side(nullptr, h.lQQ, dJ, t) && attn_side(nullptr, h.lKK, dK, t) &&
           attn_side(nullptr, h.lf[GAMMA], dJ, t) && attn_side(nullptr, h.lb[DGAMMA], dJ, t) &&
           attn_side(nullptr, h.lDQQ, dJ, t) && attn_side(nullptr, h.lDKK, dK, t) &&
           mha_stat_bytes(z.n[dH], z.n[dB], z.n[dJ]) <=
               (size_t)(z.n[dH] * z.n[dB] * z.n[dJ] * z.n[dK]) * sizeof(half_t);
}

// Decided from what the forward pass sees, so that both passes take the same path.
// With the option at SUB_FUSE_REQUIRED a caller may have handed over token-sized
// stand-ins for the tensors this path does not touch: then there is no way back.
bool attention_fused(const Handle& h, void* const* F, AttnArgs& a) {
    bool ok = attention_planned(h);
    if (ok) {
        const Sizes& z = h.sz;
        a.H = (int)z.n[dH]; a.B = (int)z.n[dB]; a.J = (int)z.n[dJ]; a.K = (int)z.n[dK];
        a.alpha = h.gemm[G_QKT].alpha;
        half_t* KK = sub_q(F[KKQQVV], h, 0); half_t* QQ = sub_q(F[KKQQVV], h, 1);
        half_t* VV = sub_q(F[KKQQVV], h, 2);
        attn_side(QQ, h.lQQ, dJ, a.q); attn_side(KK, h.lKK, dK, a.k); attn_side(VV, h.lKK, dK, a.v);
        attn_side(F[GAMMA], h.lf[GAMMA], dJ, a.o);
        a.lse = (float*)F[ALPHA]; a.dsum = a.lse + (size_t)a.H * a.B * a.J;
        a.keep = (uint32_t*)F[ATTN_DROP_MASK];
        if (h.attn_mask) {
            a.amask = (const half_t*)h.attn_mask;
            a.am_sj = h.l_attn_mask.stride[dJ]; a.am_sk = h.l_attn_mask.stride[dK];
        }
        ok = mha_forward_ok(a, (int)z.n[dP]);
    }
    if (!ok && h.fuse_attention == SUB_FUSE_REQUIRED)
        fail("attention with the scores in registers was required (SUB_OPT_FUSE_ATTENTION = 2) but the sizes, "
             "layouts or tensor alignment rule it out");
    return ok;
}

// The plan of the mask (which tiles it leaves to do, which blocks need the
// addition) is rebuilt from the mask's present contents by every forward pass: the
// caller owns the mask and may have rewritten it.  The backward pass reuses the plan
// of its forward pass, whose mask it has to share anyway (and builds it when this
// handle has run no forward pass since the mask was set).
void mask_plan(Handle& h, AttnArgs& a, bool forward) {
    if (!a.amask || !h.mask_plan) return;
    launch_mha_mask_plan(a, h.mask_plan, forward || !h.mask_plan_built, h.stream);
    h.mask_plan_built = true;
}

// bsb + blnrd (plain) or ebsb + blnrd + baob (extended) in one launch.  Returns
// false, having done nothing, when the shape or the layouts rule the fused
// kernel out; the caller then runs the separate operators.
// How op_lnbwd runs: see LnBwdArgs for the first three; dry = only say whether the launch is possible.
struct LnBwdMode { bool packed_mask = false, write_g = true, move_sum = false, dry = false; };

bool op_lnbwd(Handle& h, bool ext, const void* in, const Layout& lin_, const void* scale, const void* d1,
              const Layout& l1, const void* d2, const Layout& l2, const void* dlinear, const Layout& ldl,
              const void* istd, const Layout& listd, const void* diff, const Layout& ldiff,
              const void* mask, const Layout& lmask, void* g, const Layout& lg, void* d_ln_in,
              const Layout& lo1, void* d_drop_in, const Layout& lo2, void* dscale, void* dbias,
              void* dlinear_bias, void* dout_bias, LnBwdMode mode = {}) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    LnBwdArgs a;
    if (mode.packed_mask) a.mask_bits = (const uint8_t*)mask;
    a.write_g = mode.write_g;
    a.move_sum = mode.move_sum;
    a.in = make_view(in, lin_, sp); a.d1 = make_view(d1, l1, sp);
    a.d2 = ext ? make_view(d2, l2, sp) : a.d1;
    a.dlinear = ext ? make_view(dlinear, ldl, sp) : a.d1;
    a.diff = make_view(diff, ldiff, sp); a.mask = make_view(mask, lmask, sp);
    a.istd = make_view(istd, listd, sp);
    a.g = make_view(g, lg, sp); a.d_ln_in = make_view(d_ln_in, lo1, sp);
    a.d_drop_in = make_view(d_drop_in, lo2, sp);
    flatten(sp.rs, {&a.in, &a.d1, &a.d2, &a.dlinear, &a.diff, &a.mask, &a.istd, &a.g, &a.d_ln_in,
                    &a.d_drop_in});
    a.scale = vector_view(scale, sp.rs.R);
    if (!lnbwd_supported(sp.rs, a, ext)) return false;
    // on the static scratch array, rows beyond 1024 features stay with the separate operators, whose
    // partial rows fit it for every shape (the one-launch form needs up to 256 partial rows of 4096 per sum)
    if (h.static_ws && sp.rs.R > 1024) return false;
    if (mode.dry) return true;
    float* ws = take_ws(h, lnbwd_ws_floats(sp.rs, ext));
    half_t* sums[4] = {(half_t*)dscale, (half_t*)dbias, (half_t*)dlinear_bias, (half_t*)dout_bias};
    launch_lnbwd(sp.rs, a, ext, sums, ws, h.stream, defer_of(h));
    return true;
}

// out[q,p,h,b,j] = in[q,p,h,b,j] + bias[q,p,h].  The row dim is the innermost
// dim of the output when the input is contiguous along it too, else J.
void op_aib(Handle& h, const void* in, const Layout& lin_, const void* bias, const Layout& lbias,
            void* out, const Layout& lout) {
    int r = lout.dims[lout.rank - 1];
    if (lin_.stride[r] != 1) r = dJ;
    int outer[4]; int k = 0;
    const int canon[5] = {dQ, dP, dH, dB, dJ};
    for (int d : canon) if (d != r) outer[k++] = d;
    Space sp = make_space(h.sz, {outer[0], outer[1], outer[2], outer[3]}, r);
    View vi = make_view(in, lin_, sp), vb = make_view(bias, lbias, sp), vo = make_view(out, lout, sp);
    flatten(sp.rs, {&vi, &vb, &vo});
    launch_add(sp.rs, vi, vb, vo, h.stream);
}

// dbias[q,p,h] = sum_{b,j} d[q,p,h,b,j]
void op_baib(Handle& h, const void* d, const Layout& ld, void* dbias, const Layout& lbias) {
    const int64_t P = h.sz.n[dP], H = h.sz.n[dH];
    if (ld.stride[dJ] == 1) {
        // J contiguous: one wave sums the (b, j) block of each (q,p,h)
        Space sp = make_space(h.sz, {dQ, dP, dH, dB}, dJ);
        launch_baib(sp.rs, make_view(d, ld, sp), make_view(dbias, lbias, sp), h.stream);
        return;
    }
    const bool hp_merged = ld.stride[dP] == 1 && ld.stride[dH] == P && lbias.stride[dP] == 1 &&
                           lbias.stride[dH] == P;
    if (hp_merged) {
        // (h,p) is one contiguous run of H*P features in both tensors: a column
        // reduction over (b, j) per q with full-width rows.
        RowSpace rs{1, (int)h.sz.n[dQ], (int)h.sz.n[dB], (int)h.sz.n[dJ], (int)(H * P)};
        View v; v.p = (half_t*)d; v.s0 = 0; v.s1 = ld.stride[dQ]; v.s2 = ld.stride[dB]; v.s3 = ld.stride[dJ];
        v.sr = 1;
        v.vec = ((H * P) % 8 == 0 && v.s1 % 8 == 0 && v.s2 % 8 == 0 && v.s3 % 8 == 0 &&
                 (reinterpret_cast<uintptr_t>(d) & 15) == 0) ? 1 : 0;
        float* ws = take_ws(h, colreduce_ws_floats(rs, 1));
        launch_colsum(rs, v, (half_t*)dbias, 0, lbias.stride[dQ], 1, ws, h.stream, defer_of(h));
        return;
    }
    // general: rows of P features, kept (q,h), summed over (b,j)
    Space sp = make_space(h.sz, {dQ, dH, dB, dJ}, dP);
    float* ws = take_ws(h, colreduce_ws_floats(sp.rs, 1));
    launch_colsum(sp.rs, make_view(d, ld, sp), (half_t*)dbias, lbias.stride[dQ], lbias.stride[dH],
                  lbias.stride[dP], ws, h.stream, defer_of(h));
}

void op_bei(Handle& h, const void* a, const Layout& la, const void* b, const Layout& lb_, void* o,
            const Layout& lo) {
    Space sp = make_space(h.sz, {dB, dJ}, dI);
    View va = make_view(a, la, sp), vb = make_view(b, lb_, sp), vo = make_view(o, lo, sp);
    flatten(sp.rs, {&va, &vb, &vo});
    launch_add(sp.rs, va, vb, vo, h.stream);
}

// ---------------------------------------------------------------------------
// The two operator sequences
// ---------------------------------------------------------------------------
struct FwdPtrs {
    void* X; void* W[SUB_N_PARAMS]; void* F[SUB_N_FWD]; void* Y;
};
struct BwdPtrs {
    void* DY; void* DW[SUB_N_PARAMS]; void* Bk[SUB_N_BWD]; void* W[SUB_N_PARAMS]; void* F[SUB_N_FWD];
    void* X; void* DX;
};

// Advances the device-side dropout step (a vector store by one lane).
__global__ void k_step_increment(uint32_t* step) {
    if (threadIdx.x == 0) step[0] = step[0] + 1u;
}

// A staged copy in the library's own order (SUB_OPT_PRIVATE_LAYOUTS), allocated on first use.
half_t* staged(Handle& h, half_t*& slot, int64_t numel, const char* what) {
    if (!slot) {
        refuse_capture(h, what);
        hip_check(hipMalloc((void**)&slot, (size_t)numel * sizeof(half_t)), what);
    }
    return slot;
}

void drop_staged(Handle& h) {
    bool any = h.sX || h.sY || h.sDY || h.sDX;
    for (int i = 0; i < SUB_N_PARAMS; ++i) any = any || h.sW[i] || h.sDW[i];
    if (!any) return;
    refuse_capture(h, "sub_configure");
    for (half_t** q : {&h.sX, &h.sY, &h.sDY, &h.sDX}) if (*q) { hip_check(hipFree(*q), "hipFree(staged tensor)"); *q = nullptr; }
    for (int i = 0; i < SUB_N_PARAMS; ++i) {
        if (h.sW[i]) { hip_check(hipFree(h.sW[i]), "hipFree(staged weight)"); h.sW[i] = nullptr; }
        if (h.sDW[i]) { hip_check(hipFree(h.sDW[i]), "hipFree(staged weight gradient)"); h.sDW[i] = nullptr; }
    }
}

// The input and the weights in the library's orders: copied when `fresh`, or when the copies at hand were made
// from other pointers than these (a backward call handed other tensors than its forward call).
void stage_inputs(Handle& h, const void* X, void* const* W, const void*& Xs, void** Ws, bool fresh, const char* name) {
    Xs = X;
    for (int i = 0; i < SUB_N_PARAMS; ++i) Ws[i] = W[i];
    bool any = h.stage_x;
    for (int i = 0; i < SUB_N_PARAMS; ++i) any = any || h.stage_p[i];
    if (!any) return;
    ProfScope ps(h, name);
    RelayoutJob jobs[1 + SUB_N_PARAMS];
    int n = 0;
    if (h.stage_x) {
        Xs = staged(h, h.sX, h.lX.numel, "hipMalloc(staged input)");
        if (fresh || h.staged_x_from != X) {
            jobs[n++] = RelayoutJob{h.xX, h.lX, (const half_t*)X, h.sX};
            h.staged_x_from = X;
        }
    }
    for (int i = 0; i < SUB_N_PARAMS; ++i) {
        if (!h.stage_p[i]) continue;
        Ws[i] = staged(h, h.sW[i], h.lp[i].numel, "hipMalloc(staged weight)");
        if (fresh || h.staged_w_from[i] != W[i]) {
            jobs[n++] = RelayoutJob{h.xp[i], h.lp[i], (const half_t*)W[i], h.sW[i]};
            h.staged_w_from[i] = W[i];
        }
    }
    if (n) launch_relayout_batch(jobs, n, h.stream);     // one launch for all of them
    else ps.cancel();
}

void forward(Handle& h, const FwdPtrs& t0) {
    if (!h.configured) fail("encoder_forward: handle is not configured");
    h.prof_used = 0;
    h.prof_forward = 0;
    FwdPtrs t = t0;
    if (h.staging) {
        const void* xs = nullptr;
        stage_inputs(h, t0.X, t0.W, xs, t.W, true, "relayout-in");
        t.X = const_cast<void*>(xs);
        if (h.stage_y) t.Y = staged(h, h.sY, h.lY.numel, "hipMalloc(staged output)");
    }
    void* const* W = t.W; void* const* F = t.F;
    AttnArgs at;
    const bool fused_attention = attention_fused(h, F, at);
    if (h.fuse_epilogues && h.gemm[G_QKV_BIAS].ok && aligned16(W[BKQV]) && aligned16(F[KKQQVV])) {
        // projection + bias in one pass; WKKWQQWVV (the pre-bias copy) is not written.  The CUs its tiles
        // leave idle draw part of the attention's dropout bits, which depend on nothing but the seed.
        GemmSideJob side;
        if (fused_attention && (h.side_jobs & 1)) {
            side.key = make_key(h, SUB_SITE_SOFTMAX, h.p_softmax);
            side.keep = at.keep; side.rows = (uint32_t)((long)at.H * at.B * at.J); side.nk = (uint32_t)at.K;
        }
        run_gemm(h, G_QKV_BIAS, t.X, W[WKQV], F[KKQQVV], "QKV-fused", W[BKQV], &side);
        at.keep_tiles_ready = side.tiles_done;
    } else {
        run_gemm(h, G_QKV, t.X, W[WKQV], F[WKKWQQWVV], "QKV-fused");
        ProfScope ps(h, "aib");
        op_aib(h, F[WKKWQQWVV], h.lf[WKKWQQWVV], W[BKQV], h.lp[BKQV], F[KKQQVV], h.lf[KKQQVV]);
    }
    half_t* KK = sub_q(F[KKQQVV], h, 0); half_t* QQ = sub_q(F[KKQQVV], h, 1); half_t* VV = sub_q(F[KKQQVV], h, 2);
    if (fused_attention) {
        ProfScope ps(h, "attention");
        mask_plan(h, at, true);
        launch_mha_forward(at, (int)h.sz.n[dP], make_key(h, SUB_SITE_SOFTMAX, h.p_softmax), h.stream);
    }
    bool fused_scores = fused_attention;
    if (!fused_attention && h.fuse_scores) {
        ProfScope ps(h, "QKT+softmax");
        fused_scores = op_scores_softmax(h, QQ, KK, F[ALPHA], h.lf[ALPHA], F[ATTN_DROP_MASK],
                                         h.lf[ATTN_DROP_MASK], F[ATTN_DROP], h.lf[ATTN_DROP]);
        if (!fused_scores) ps.cancel();
    }
    if (!fused_scores) {
        run_gemm(h, G_QKT, KK, QQ, F[BETA], "QKT");
        ProfScope ps(h, "softmax");
        op_softmax(h, F[BETA], h.lf[BETA], F[ALPHA], h.lf[ALPHA], F[ATTN_DROP_MASK], h.lf[ATTN_DROP_MASK],
                   F[ATTN_DROP], h.lf[ATTN_DROP], 1.0f, h.p_softmax, SUB_SITE_SOFTMAX, h.attn_mask,
                   &h.l_attn_mask, h.gemm[G_QKT].alpha);
    }
    if (!fused_attention) run_gemm(h, G_GAMMA, VV, F[ATTN_DROP], F[GAMMA], "gamma");
    run_gemm(h, G_OUT, W[WO], F[GAMMA], F[ATT], "out");
    const bool lin1_gelu = lin1_takes_gelu_epilogue(h, W, F);
    const bool lin1_bad = lin1_gelu || (relu_from_output(h) && h.fuse_epilogues && h.gemm[G_LIN1_BAD].ok &&
                                        aligned16(W[LINB1]) && aligned16(F[DROP2]) && aligned16(F[SB1]) && aligned16(W[LINW1]));
    // The keep bits of lin1's ReLU-dropout epilogue depend on nothing but seed, step and position:
    // workgroups behind those of bdrln1, a launch that waits for memory with its vector units idle,
    // draw them, into the SB1_LINW1 buffer (unused with that epilogue) behind its B*J*U/8 bytes of gate bits.
    KeepWordsJob keep_job;
    if (lin1_bad && !lin1_gelu && (h.side_jobs & 2) && aligned16(F[SB1_LINW1])) {
        const GemmPlan& p = h.gemm[G_LIN1_BAD];
        keep_job.key = make_key(h, SUB_SITE_ACT, h.p_act);
        keep_job.M = (uint32_t)p.shape.M; keep_job.N = (uint32_t)p.shape.N;
        if ((size_t)keep_job.M * keep_job.N / 8 % 16 == 0)
            keep_job.out = (uint32_t*)((char*)F[SB1_LINW1] + (size_t)keep_job.M * keep_job.N / 8);
    }
    {
        ProfScope ps(h, "bdrln1");   // adds BO to ATT in place (encoder.cu:134-135)
        op_bdrln(h, F[ATT], h.lf[ATT], t.X, h.lX, W[BO], W[S1], W[B1], F[ATT], h.lf[ATT],
                 F[DROP1MASK], h.lf[DROP1MASK], F[LN1DIFF], h.lf[LN1DIFF], F[LN1], h.lf[LN1],
                 F[SB1], h.lf[SB1], F[LN1STD], h.lf[LN1STD], h.p_resid1, SUB_SITE_RESID1, packed_masks(h), !h.skip_unread,
                 &keep_job);
    }
    if (lin1_bad) {
        // product, bias, activation and dropout in one launch: SB1_LINW1 and DROP2MASK (ReLU: and LIN1) are not produced
        ProfScope ps(h, "lin1+bad");
        const GemmPlan& p = h.gemm[G_LIN1_BAD];
        GemmEpilogue ep;
        ep.bias = (const half_t*)W[LINB1]; ep.sbM = p.sM; ep.sbN = p.sN;
        ep.relu_dropout = true; ep.key = make_key(h, SUB_SITE_ACT, h.p_act);
        if (keep_job.blocks) ep.keep_words = keep_job.out;
        if (F[SB1_LINW1] && ((uintptr_t)F[SB1_LINW1] & 3) == 0) ep.gate_bits_out = (uint32_t*)F[SB1_LINW1];
        h.gate_bits_at = ep.gate_bits_out;
        if (lin1_gelu) { ep.act = ACT_GELU; ep.pre_out = (half_t*)F[LIN1]; }
        launch_gemm(p.shape, (const half_t*)F[SB1], (const half_t*)W[LINW1], (half_t*)F[DROP2], p.alpha, ep, h.stream);
    } else {
    h.gate_bits_at = nullptr;
    run_gemm(h, G_LIN1, F[SB1], W[LINW1], F[SB1_LINW1], "lin1");
    {
        ProfScope ps(h, "bad");
        op_bad(h, F[SB1_LINW1], h.lf[SB1_LINW1], W[LINB1], F[LIN1], h.lf[LIN1], F[DROP2MASK],
               h.lf[DROP2MASK], F[DROP2], h.lf[DROP2], h.p_act, SUB_SITE_ACT, relu_from_output(h));
    }
    }
    run_gemm(h, G_LIN2, F[DROP2], W[LINW2], F[DROP2_LINW2], "lin2");
    {
        ProfScope ps(h, "bdrln2");
        op_bdrln(h, F[DROP2_LINW2], h.lf[DROP2_LINW2], F[SB1], h.lf[SB1], W[LINB2], W[S2], W[B2],
                 F[LIN2], h.lf[LIN2], F[DROP3MASK], h.lf[DROP3MASK], F[LN2DIFF], h.lf[LN2DIFF],
                 F[LN2], h.lf[LN2], t.Y, h.lY, F[LN2STD], h.lf[LN2STD], h.p_resid2, SUB_SITE_RESID2, packed_masks(h), !h.skip_unread);
    }
    if (h.staging && h.stage_y) {
        ProfScope ps(h, "relayout-out");
        launch_relayout(h.lY, h.xY, (const half_t*)t.Y, (half_t*)t0.Y, h.stream);
    }
    prof_mark_end(h);
    if (h.step_dev) {
        hipLaunchKernelGGL(k_step_increment, dim3(1), dim3(64), 0, h.stream, h.step_dev);
        check_launch("dropout step increment");
    } else {
        h.step += 1;
    }
    h.prof_forward = h.prof_used;
}

void backward(Handle& h, const BwdPtrs& t0) {
    if (!h.configured) fail("encoder_backward: handle is not configured");
    // the first backward call after a forward call keeps that call's entries in front of its own
    h.prof_used = h.prof_forward;
    h.prof_forward = 0;
    BwdPtrs t = t0;
    if (h.staging) {
        const void* xs = nullptr;
        stage_inputs(h, t0.X, t0.W, xs, t.W, false, "relayout-in-again");
        t.X = const_cast<void*>(xs);
        if (h.stage_y) {
            ProfScope ps(h, "relayout-in-bwd");
            t.DY = staged(h, h.sDY, h.lY.numel, "hipMalloc(staged output gradient)");
            launch_relayout(h.xY, h.lY, (const half_t*)t0.DY, h.sDY, h.stream);
        }
        if (h.stage_x) t.DX = staged(h, h.sDX, h.lX.numel, "hipMalloc(staged input gradient)");
        for (int i = 0; i < SUB_N_PARAMS; ++i)
            if (h.stage_p[i]) t.DW[i] = staged(h, h.sDW[i], h.lp[i].numel, "hipMalloc(staged weight gradient)");
    }
    // The five bias / scale gradients are only consumed by the caller: their
    // reductions leave fp32 partials in separate scratch regions and one launch
    // at the end of the pass finishes them all (or workgroups of the last pair of
    // products do).  Per-operator timing times this same schedule: the finishing
    // stage is part of the launch that carries it, or an entry of its own.
    if (h.ops_deferring) fail("encoder_backward: column sums are being deferred across operator calls (sub_ops_defer)");
    ensure_ws(h, h.ws_need_bwd);
    h.deferring = true;
    h.ws_cursor = 0;
    h.deferred.n = 0;
    struct Reset { Handle& h; ~Reset() { h.deferring = false; } } reset{h};
    void* const* W = t.W; void* const* F = t.F; void* const* D = t.Bk; void* const* DW = t.DW;
    bool fused = false;
    // the backward passes around the two LayerNorms, each as one launch where possible
    auto ln2_backward = [&](LnBwdMode m) {
        return op_lnbwd(h, false, F[LN2], h.lf[LN2], W[S2], t.DY, h.lY, nullptr, h.lY, nullptr, h.lY,
                        F[LN2STD], h.lf[LN2STD], F[LN2DIFF], h.lf[LN2DIFF], F[DROP3MASK], h.lf[DROP3MASK],
                        D[DLN2], h.lb[DLN2], D[DRESID2], h.lb[DRESID2], D[DLIN2], h.lb[DLIN2],
                        DW[S2], DW[B2], DW[LINB2], nullptr, m);
    };
    auto ln1_backward = [&](LnBwdMode m) {
        return op_lnbwd(h, true, F[LN1], h.lf[LN1], W[S1], D[DRESID2], h.lb[DRESID2], D[DLIN1_LINW1],
                        h.lb[DLIN1_LINW1], D[DLIN2], h.lb[DLIN2], F[LN1STD], h.lf[LN1STD], F[LN1DIFF],
                        h.lf[LN1DIFF], F[DROP1MASK], h.lf[DROP1MASK], D[DLN1], h.lb[DLN1], D[DRESID1],
                        h.lb[DRESID1], D[DATT], h.lb[DATT], DW[S1], DW[B1], DW[LINB2], DW[BO], m);
    };
    LnBwdMode ln_mode;
    ln_mode.packed_mask = packed_masks(h); ln_mode.write_g = !h.skip_unread;
    if (h.fuse_ln_backward) {
        // DLINB2 is the column sum of DLIN2, which the first of the two launches writes and the second
        // would only read for that sum: when both run, the first one sums it
        // (asked with the sum moved: rows beyond 1024 features take the second launch only in that form)
        LnBwdMode probe = ln_mode;
        probe.dry = true; probe.move_sum = true;
        ln_mode.move_sum = ln2_backward(probe) && ln1_backward(probe);
    }
    if (h.fuse_ln_backward) {
        ProfScope ps(h, "bsb+blnrd1");
        fused = ln2_backward(ln_mode);
        if (!fused) ps.cancel();
    }
    if (!fused) {
        {
            ProfScope ps(h, "bsb");
            op_bsb(h, F[LN2], h.lf[LN2], W[S2], t.DY, h.lY, D[DLN2], h.lb[DLN2], DW[S2], DW[B2]);
        }
        {
            ProfScope ps(h, "blnrd1");
            op_blnrd(h, D[DLN2], h.lb[DLN2], F[LN2STD], h.lf[LN2STD], F[LN2DIFF], h.lf[LN2DIFF],
                     F[DROP3MASK], h.lf[DROP3MASK], D[DRESID2], h.lb[DRESID2], D[DLIN2], h.lb[DLIN2], packed_masks(h));
        }
    }
    const bool bits_here = h.gate_bits_at && h.gate_bits_at == F[SB1_LINW1] &&
                           h.gemm[G_LIN1_BAD].shape.M == h.gemm[G_DXLIN2_BDRLB].shape.M &&
                           h.gemm[G_LIN1_BAD].shape.N == h.gemm[G_DXLIN2_BDRLB].shape.N;
    const bool bdrlb_gelu = lin1_takes_gelu_epilogue(h, W, F);       // the forward call's own test: its keep bits lie in SB1_LINW1
    const bool fuse_bdrlb = ((relu_from_output(h) && h.fuse_epilogues && h.gemm[G_DXLIN2_BDRLB].ok && aligned16(F[DROP2])) ||
                             bdrlb_gelu) &&
                            aligned16(D[DLIN1]) && aligned16(D[DLIN2]) && aligned16(W[LINW2]);
    if (bdrlb_gelu && !fuse_bdrlb)
        fail("encoder_backward: the forward call ran lin1 with the GELU epilogue (no DROP2MASK was written), and its "
             "backward epilogue needs 16-byte aligned DLIN1, DLIN2 and LINW2");
    if (fuse_bdrlb) {
        // product, gate and the column sums of the result in one launch: DDROP2 is not produced
        ProfScope ps(h, "dXlin2+bdrlb");
        const GemmPlan& p = h.gemm[G_DXLIN2_BDRLB];
        const int ntc = (int)(p.shape.M / 128), U = (int)p.shape.N;
        float* ws = take_ws(h, (size_t)ntc * U);
        GemmEpilogue ep;
        ep.gate = (const half_t*)(bdrlb_gelu ? F[LIN1] : F[DROP2]); ep.sbM = p.sM; ep.sbN = p.sN; ep.colsum = ws;
        if (bits_here || bdrlb_gelu) ep.gate_bits = (const uint32_t*)F[SB1_LINW1];
        if (bdrlb_gelu) ep.act = ACT_GELU;
        launch_gemm(p.shape, (const half_t*)D[DLIN2], (const half_t*)W[LINW2], (half_t*)D[DLIN1], p.alpha, ep, h.stream);
        FinishJob job{ws, FinishArgs{{(half_t*)DW[LINB1], nullptr, nullptr, nullptr}, 0, 0, 1, 1}, 1, 1, ntc, U};
        finish_or_defer(defer_of(h), job, h.stream);
    } else {
        run_gemm(h, G_DXLIN2, D[DLIN2], W[LINW2], D[DDROP2], "dXlin2");
    }
    // With many tokens the data gradient of linear1 has too many tiles to share a launch with the weight
    // gradient next to it; the two weight gradients of the feed-forward block -- one tile per CU each, their
    // contraction as long as the token count -- then run as a pair of their own on 256 x 128 tiles (a quarter
    // less operand traffic from L2 than alone on 128 x 128 tiles), dWlin2 waiting for dWlin1's operands.
    const bool pair_weights = !pair_ok(h, G_DXLIN1, D[DLIN1], W[LINW1], D[DLIN1_LINW1], nullptr, G_DWLIN1, D[DLIN1], F[SB1],
                                       DW[LINW1]) &&
                              pair_ok(h, G_DWLIN1, D[DLIN1], F[SB1], DW[LINW1], nullptr, G_DWLIN2, D[DLIN2], F[DROP2], DW[LINW2]);
    if (!pair_weights) run_gemm(h, G_DWLIN2, D[DLIN2], F[DROP2], DW[LINW2], "dWlin2");
    if (!fuse_bdrlb) {
        ProfScope ps(h, "bdrlb");
        if (relu_from_output(h))
            op_bdrlb_from_output(h, D[DDROP2], h.lb[DDROP2], F[DROP2], h.lf[DROP2], D[DLIN1], h.lb[DLIN1], DW[LINB1]);
        else
            op_bdrlb(h, D[DDROP2], h.lb[DDROP2], F[DROP2MASK], h.lf[DROP2MASK], F[LIN1], h.lf[LIN1],
                     D[DLIN1], h.lb[DLIN1], DW[LINB1]);
    }
    if (pair_weights) {
        run_gemm(h, G_DXLIN1, D[DLIN1], W[LINW1], D[DLIN1_LINW1], "dXlin1");
        run_gemm_pair(h, G_DWLIN1, D[DLIN1], F[SB1], DW[LINW1], "dWlin1", nullptr,
                      G_DWLIN2, D[DLIN2], F[DROP2], DW[LINW2], "dWlin2", "dWlin1+dWlin2");
    } else {
        run_gemm_pair(h, G_DXLIN1, D[DLIN1], W[LINW1], D[DLIN1_LINW1], "dXlin1", nullptr,
                      G_DWLIN1, D[DLIN1], F[SB1], DW[LINW1], "dWlin1", "dXlin1+dWlin1");
    }
    fused = false;
    if (h.fuse_ln_backward) {
        ProfScope ps(h, "ebsb+blnrd2+baob");
        fused = ln1_backward(ln_mode);
        if (!fused) ps.cancel();
    }
    if (!fused) {
        {
            ProfScope ps(h, "ebsb");
            op_ebsb(h, F[LN1], h.lf[LN1], W[S1], D[DRESID2], h.lb[DRESID2], D[DLIN1_LINW1],
                    h.lb[DLIN1_LINW1], D[DLIN2], h.lb[DLIN2], D[DLN1], h.lb[DLN1], DW[S1], DW[B1], DW[LINB2]);
        }
        {
            ProfScope ps(h, "blnrd2");
            op_blnrd(h, D[DLN1], h.lb[DLN1], F[LN1STD], h.lf[LN1STD], F[LN1DIFF], h.lf[LN1DIFF],
                     F[DROP1MASK], h.lf[DROP1MASK], D[DRESID1], h.lb[DRESID1], D[DATT], h.lb[DATT], packed_masks(h));
        }
        {
            ProfScope ps(h, "baob");
            op_baob(h, D[DATT], h.lb[DATT], DW[BO]);
        }
    }
    AttnArgs at;
    const bool attn_fused = attention_fused(h, F, at);
    const bool fuse_dx = h.fuse_epilogues && h.gemm[G_DXQKV_RESID].ok && aligned16(D[DRESID1]) &&
                         aligned16(t.DX);
    // dWout (64 tiles of 128 x 128 at the bench workload, too few for a launch of its
    // own without splitting its contraction) needs nothing but DATT and feeds nothing:
    // when the last pair of products of the pass has room for its tiles it runs there,
    // unsplit, and dXout runs alone here.
    PairThird dwout;
    bool dwout_later = false;
    if (h.finish_in_pair && attn_fused) {
        const GemmPlan& p3 = h.gemm[G_DWOUT];
        dwout.shape = &p3.shape; dwout.A = (const half_t*)F[GAMMA]; dwout.B = (const half_t*)D[DATT];
        dwout.C = (half_t*)DW[WO]; dwout.alpha = p3.alpha;
        dwout_later = fuse_dx ? pair_takes_third(h, G_DXQKV_RESID, W[WKQV], D[DKKQQVV], t.DX, D[DRESID1], G_DWQKV,
                                                 t.X, D[DKKQQVV], DW[WKQV], dwout)
                              : pair_takes_third(h, G_DXQKV, W[WKQV], D[DKKQQVV], D[DXATT], nullptr, G_DWQKV, t.X,
                                                 D[DKKQQVV], DW[WKQV], dwout);
    }
    if (dwout_later)
        run_gemm(h, G_DXOUT, W[WO], D[DATT], D[DGAMMA], "dXout");
    else
        run_gemm_pair(h, G_DXOUT, W[WO], D[DATT], D[DGAMMA], "dXout", nullptr,
                      G_DWOUT, F[GAMMA], D[DATT], DW[WO], "dWout", "dXout+dWout");
    half_t* KK = sub_q(F[KKQQVV], h, 0); half_t* QQ = sub_q(F[KKQQVV], h, 1); half_t* VV = sub_q(F[KKQQVV], h, 2);
    half_t* DKK = sub_q(D[DKKQQVV], h, 0); half_t* DQQ = sub_q(D[DKKQQVV], h, 1); half_t* DVV = sub_q(D[DKKQQVV], h, 2);
    bool attn_bias = false;
    if (attn_fused) {
        if (!attn_side(D[DGAMMA], h.lb[DGAMMA], dJ, at.d_o) || !attn_side(DQQ, h.lDQQ, dJ, at.dq) ||
            !attn_side(DKK, h.lDKK, dK, at.dk) || !attn_side(DVV, h.lDKK, dK, at.dv))
            fail("encoder_backward: attention layouts changed since the forward pass");
        // the sums over (sample, position) of dQ, dK, dV -- the gradient of the projection
        // biases (BackwardAttentionInputBiases, encoder.cu:288-290) -- start in these launches
        const Layout& lbias = h.lp[BKQV];
        attn_bias = lbias.has[dQ] && lbias.has[dH] && lbias.has[dP];
        const int P = (int)h.sz.n[dP], H = (int)h.sz.n[dH];
        const int ntq = at.B * (at.J / 128), ntk = at.B * (at.K / 128);
        half_t* dbias = (half_t*)DW[BKQV];
        auto finish = [&](float* ws, int ns, int ntc, half_t* o0, half_t* o1) {
            FinishJob job{ws, FinishArgs{{o0, o1, nullptr, nullptr}, 0, lbias.stride[dH], lbias.stride[dP], H}, ns, H,
                          ntc, P};
            finish_or_defer(defer_of(h), job, h.stream);
        };
        {
            ProfScope ps(h, "attention-bwd-dQ");
            mask_plan(h, at, false);
            if (attn_bias) at.bias_q = take_ws(h, (size_t)H * ntq * P);
            launch_mha_backward_dq(at, P, h.stream);
            if (attn_bias) finish(at.bias_q, 1, ntq, dbias + 1 * lbias.stride[dQ], nullptr);
        }
        ProfScope ps(h, "attention-bwd-dKdV");
        if (attn_bias) at.bias_kv = take_ws(h, (size_t)2 * H * ntk * P);
        launch_mha_backward_dkv(at, P, h.stream);
        if (attn_bias) finish(at.bias_kv, 2, ntk, dbias, dbias + 2 * lbias.stride[dQ]);
    } else {
        run_gemm(h, G_DX2GAMMA, D[DGAMMA], F[ATTN_DROP], DVV, "dX2gamma");
        bool fused_scores = false;
        if (h.fuse_scores) {
            ProfScope ps(h, "dX1gamma+bs");
            fused_scores = op_dscores_bs(h, D[DGAMMA], VV, F[ALPHA], h.lf[ALPHA], F[ATTN_DROP_MASK],
                                         h.lf[ATTN_DROP_MASK], D[DBETA], h.lb[DBETA]);
            if (!fused_scores) ps.cancel();
        }
        if (!fused_scores) {
            run_gemm(h, G_DX1GAMMA, VV, D[DGAMMA], D[DATTN_DROP], "dX1gamma");
            ProfScope ps(h, "bs");
            op_bs(h, F[ALPHA], h.lf[ALPHA], F[ATTN_DROP_MASK], h.lf[ATTN_DROP_MASK], D[DATTN_DROP],
                  h.lb[DATTN_DROP], D[DBETA], h.lb[DBETA], 1.0f);
        }
        run_gemm(h, G_DX1QKT, KK, D[DBETA], DQQ, "dX1QKT");
        run_gemm(h, G_DX2QKT, QQ, D[DBETA], DKK, "dX2QKT");
    }
    // The last products of the pass finish the deferred column sums in workgroups of
    // their own launch when every producer of those sums has been launched by now
    // (baib below would add one more).
    FinishJobs* tail = h.deferring && attn_bias && h.finish_in_pair ? &h.deferred : nullptr;
    PairThird* third = dwout_later ? &dwout : nullptr;
    const char* last_name = dwout_later ? "dXQKV-fused+dWQKV-fused+dWout" : "dXQKV-fused+dWQKV-fused";
    if (fuse_dx) {
        // DX = WKQV.DKKQQVV + DRESID1 in one pass; DXATT is not written
        run_gemm_pair(h, G_DXQKV_RESID, W[WKQV], D[DKKQQVV], t.DX, "dXQKV-fused", D[DRESID1],
                      G_DWQKV, t.X, D[DKKQQVV], DW[WKQV], "dWQKV-fused", last_name, tail, third);
    } else {
        run_gemm_pair(h, G_DXQKV, W[WKQV], D[DKKQQVV], D[DXATT], "dXQKV-fused", nullptr,
                      G_DWQKV, t.X, D[DKKQQVV], DW[WKQV], "dWQKV-fused", last_name, tail, third);
    }
    if (dwout_later && !dwout.taken) run_gemm(h, G_DWOUT, F[GAMMA], D[DATT], DW[WO], "dWout");
    if (!attn_bias) {
        ProfScope ps(h, "baib");
        op_baib(h, D[DKKQQVV], h.lb[DKKQQVV], DW[BKQV], h.lp[BKQV]);
    }
    if (!fuse_dx) {
        ProfScope ps(h, "bei");
        op_bei(h, D[DXATT], h.lb[DXATT], D[DRESID1], h.lb[DRESID1], t.DX, h.lX);
    }
    if (h.deferred.n > 0) {
        ProfScope ps(h, "colfinish");
        launch_colfinish(h.deferred, h.stream);
    }
    if (h.staging) {
        bool any = h.stage_x;
        for (int i = 0; i < SUB_N_PARAMS; ++i) any = any || h.stage_p[i];
        if (any) {
            ProfScope ps(h, "relayout-out-bwd");
            RelayoutJob jobs[1 + SUB_N_PARAMS];
            int n = 0;
            if (h.stage_x) jobs[n++] = RelayoutJob{h.lX, h.xX, (const half_t*)t.DX, (half_t*)t0.DX};
            for (int i = 0; i < SUB_N_PARAMS; ++i)
                if (h.stage_p[i]) jobs[n++] = RelayoutJob{h.lp[i], h.xp[i], (const half_t*)t.DW[i], (half_t*)t0.DW[i]};
            launch_relayout_batch(jobs, n, h.stream);
        }
    }
    prof_mark_end(h);
}

void unpack_forward(const Handle& h, void* const* p, FwdPtrs& t) {
    t.X = p[0];
    for (int i = 0; i < SUB_N_PARAMS; ++i) t.W[i] = p[1 + h.pos_p[i]];
    for (int i = 0; i < SUB_N_FWD; ++i) t.F[i] = p[1 + SUB_N_PARAMS + h.pos_f[i]];
    t.Y = p[1 + SUB_N_PARAMS + SUB_N_FWD];
}

void unpack_backward(const Handle& h, void* const* p, BwdPtrs& t) {
    int o = 0;
    t.DY = p[o++];
    for (int i = 0; i < SUB_N_PARAMS; ++i) t.DW[i] = p[o + h.pos_p[i]];
    o += SUB_N_PARAMS;
    for (int i = 0; i < SUB_N_BWD; ++i) t.Bk[i] = p[o + h.pos_b[i]];
    o += SUB_N_BWD;
    for (int i = 0; i < SUB_N_PARAMS; ++i) t.W[i] = p[o + h.pos_p[i]];
    o += SUB_N_PARAMS;
    for (int i = 0; i < SUB_N_FWD; ++i) t.F[i] = p[o + h.pos_f[i]];
    o += SUB_N_FWD;
    t.X = p[o++];
    t.DX = p[o++];
}

template <class Fn>
int guarded(Fn&& fn) {
    try {
        fn();
        return 0;
    } catch (const std::exception& e) {
        g_last_error = e.what();
        return -1;
    } catch (...) {
        g_last_error = "unknown error";
        return -1;
    }
}

Handle& as_handle(void* h) {
    if (!h) fail("null handle");
    return *static_cast<Handle*>(h);
}

Layout L(Handle& h, const char* s) { return make_layout(s, h.sz); }

void need_cfg(const Handle& h) {
    if (!h.configured) fail("handle is not configured");
}

}  // namespace
}  // namespace sub

using namespace sub;

extern "C" {

const char* sub_last_error(void) { return g_last_error.c_str(); }

void* init(void) {
    void* r = nullptr;
    guarded([&] { r = new Handle(); });
    return r;
}

void destroy(void* handle) {
    guarded([&] { delete static_cast<Handle*>(handle); });
}

int sub_configure(void* handle, const sub_config* cfg) {
    return guarded([&] { configure(as_handle(handle), cfg); });
}

void* init_cfg(const sub_config* cfg) {
    void* h = init();
    if (!h) return nullptr;
    if (sub_configure(h, cfg) != 0) {
        std::string keep = g_last_error;
        destroy(h);
        g_last_error = keep;
        return nullptr;
    }
    return h;
}

int sub_set_stream(void* handle, void* hip_stream) {
    return guarded([&] { as_handle(handle).stream = (hipStream_t)hip_stream; });
}

int sub_set_rng(void* handle, uint64_t seed, uint32_t step) {
    return guarded([&] { Handle& h = as_handle(handle); h.seed = seed; h.step = step; });
}

int sub_set_rng_counter(void* handle, uint32_t* device_step) {
    return guarded([&] { as_handle(handle).step_dev = device_step; });
}

int sub_encoder_forward(void* handle, void* const* ptrs, int n) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        if (n != 1 + SUB_N_PARAMS + SUB_N_FWD + 1) fail("sub_encoder_forward: expected 37 pointers");
        need_cfg(h);
        for (int i = 0; i < n; ++i) if (!ptrs[i]) fail("sub_encoder_forward: null tensor pointer");
        FwdPtrs t; unpack_forward(h, ptrs, t);
        forward(h, t);
    });
}

int sub_encoder_backward(void* handle, void* const* ptrs, int n) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        if (n != 1 + 2 * SUB_N_PARAMS + SUB_N_BWD + SUB_N_FWD + 2) fail("sub_encoder_backward: expected 64 pointers");
        need_cfg(h);
        for (int i = 0; i < n; ++i) if (!ptrs[i]) fail("sub_encoder_backward: null tensor pointer");
        BwdPtrs t; unpack_backward(h, ptrs, t);
        backward(h, t);
    });
}

int encoder_forward(void* handle, void* X,
                    void* w0, void* w1, void* w2, void* w3, void* w4, void* w5,
                    void* w6, void* w7, void* w8, void* w9, void* w10, void* w11,
                    void* f0, void* f1, void* f2, void* f3, void* f4, void* f5, void* f6, void* f7,
                    void* f8, void* f9, void* f10, void* f11, void* f12, void* f13, void* f14,
                    void* f15, void* f16, void* f17, void* f18, void* f19, void* f20, void* f21,
                    void* f22, void* Y) {
    void* p[] = {X, w0, w1, w2, w3, w4, w5, w6, w7, w8, w9, w10, w11,
                 f0, f1, f2, f3, f4, f5, f6, f7, f8, f9, f10, f11, f12, f13, f14, f15, f16, f17,
                 f18, f19, f20, f21, f22, Y};
    return sub_encoder_forward(handle, p, (int)(sizeof(p) / sizeof(p[0])));
}

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
                     void* f22, void* X, void* DX) {
    void* p[] = {DY, dw0, dw1, dw2, dw3, dw4, dw5, dw6, dw7, dw8, dw9, dw10, dw11,
                 b0, b1, b2, b3, b4, b5, b6, b7, b8, b9, b10, b11, b12, b13,
                 w0, w1, w2, w3, w4, w5, w6, w7, w8, w9, w10, w11,
                 f0, f1, f2, f3, f4, f5, f6, f7, f8, f9, f10, f11, f12, f13, f14, f15, f16, f17,
                 f18, f19, f20, f21, f22, X, DX};
    return sub_encoder_backward(handle, p, (int)(sizeof(p) / sizeof(p[0])));
}

int sub_get_option(void* handle, int option, int* value) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        if (!value) fail("sub_get_option: null result pointer");
        if (option == SUB_OPT_FUSE_EPILOGUES) *value = h.fuse_epilogues;
        else if (option == SUB_OPT_FUSE_LN_BACKWARD) *value = h.fuse_ln_backward;
        else if (option == SUB_OPT_FUSE_SCORES) *value = h.fuse_scores;
        else if (option == SUB_OPT_FUSE_ATTENTION) *value = h.fuse_attention;
        else if (option == SUB_OPT_PAIR_PRODUCTS) *value = h.pair_products;
        else if (option == SUB_OPT_RELU_FROM_OUTPUT) *value = h.relu_from_output;
        else if (option == SUB_OPT_FINISH_IN_PAIR) *value = h.finish_in_pair;
        else if (option == SUB_OPT_SIDE_JOBS) *value = h.side_jobs;
        else if (option == SUB_OPT_PACKED_MASKS) *value = h.packed_masks;
        else if (option == SUB_OPT_SKIP_UNREAD) *value = h.skip_unread;
        else if (option == SUB_OPT_PRIVATE_LAYOUTS) *value = h.private_layouts;
        else fail("sub_get_option: unknown option");
    });
}

int sub_set_option(void* handle, int option, int value) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        if (option == SUB_OPT_FUSE_EPILOGUES) h.fuse_epilogues = value != 0;
        else if (option == SUB_OPT_FUSE_LN_BACKWARD) h.fuse_ln_backward = value != 0;
        else if (option == SUB_OPT_FUSE_SCORES) h.fuse_scores = value != 0;
        else if (option == SUB_OPT_PAIR_PRODUCTS) h.pair_products = value != 0;
        else if (option == SUB_OPT_RELU_FROM_OUTPUT) h.relu_from_output = value != 0;
        else if (option == SUB_OPT_FINISH_IN_PAIR) h.finish_in_pair = value != 0;
        else if (option == SUB_OPT_SIDE_JOBS) h.side_jobs = value & 3;
        else if (option == SUB_OPT_PACKED_MASKS) h.packed_masks = value != 0;
        else if (option == SUB_OPT_SKIP_UNREAD) h.skip_unread = value != 0;
        else if (option == SUB_OPT_PRIVATE_LAYOUTS) {
            h.private_layouts = value != 0;
            if (h.configured) plan_layouts(h, h.private_layouts);
        }
        else if (option == SUB_OPT_FUSE_ATTENTION) {
            if (value < 0 || value > SUB_FUSE_REQUIRED) fail("sub_set_option: SUB_OPT_FUSE_ATTENTION takes 0, 1 or 2");
            h.fuse_attention = value;
        }
        else fail("sub_set_option: unknown option");
    });
}

int sub_tensor_layout(void* handle, const char* name, char out[16]) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        need_cfg(h);
        if (!name || !out) fail("sub_tensor_layout: null argument");
        std::string l;
        if (!std::strcmp(name, "X")) l = h.lX.str();
        else if (!std::strcmp(name, "SB2")) l = h.lY.str();
        for (int i = 0; i < SUB_N_PARAMS && l.empty(); ++i) if (!std::strcmp(name, kParams[i].name)) l = h.lp[i].str();
        for (int i = 0; i < SUB_N_FWD && l.empty(); ++i) if (!std::strcmp(name, kFwd[i].name)) l = h.lf[i].str();
        for (int i = 0; i < SUB_N_BWD && l.empty(); ++i) if (!std::strcmp(name, kBwd[i].name)) l = h.lb[i].str();
        if (l.empty()) fail(std::string("sub_tensor_layout: unknown tensor name ") + name);
        std::snprintf(out, 16, "%s", l.c_str());
    });
}

int sub_attention_in_registers(void* handle, int* planned) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        need_cfg(h);
        if (!planned) fail("sub_attention_in_registers: null result pointer");
        *planned = attention_planned(h) ? 1 : 0;
    });
}

int sub_profile_enable(void* handle, int on) {
    return guarded([&] {
        Handle& h = as_handle(handle);
        h.profiling = on != 0; h.prof_used = 0;
        h.profile_clocks = on == 2;
        if (h.profile_clocks && !h.clock_buf)
            hip_check(hipMalloc((void**)&h.clock_buf, sizeof(unsigned long long) * 2 * kClockSlots * kMaxClockSamples), "hipMalloc(clock samples)");
        if (h.profile_clocks)       // a slot no workgroup wrote reads as zero and is left out
            hip_check(hipMemset(h.clock_buf, 0, sizeof(unsigned long long) * 2 * kClockSlots * kMaxClockSamples), "hipMemset(clock samples)");
    });
}

int sub_profile_read_clocks(void* handle, int cap, const char** names, float* mhz) {
    int count = 0;
    int rc = guarded([&] {
        Handle& h = as_handle(handle);
        if (!h.profile_clocks || !h.clock_buf) fail("sub_profile_read_clocks: enable profiling with mode 2 first");
        hip_check(hipStreamSynchronize(h.stream), "hipStreamSynchronize");
        std::vector<unsigned long long> v(2 * kClockSlots * kMaxClockSamples);
        hip_check(hipMemcpy(v.data(), h.clock_buf, v.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost), "hipMemcpy");
        int dev = 0, wall_khz = 0;
        hip_check(hipGetDevice(&dev), "hipGetDevice");
        hip_check(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, dev), "hipDeviceGetAttribute");
        for (size_t i = 0; i + 1 < h.prof_used && i + 1 < (size_t)kMaxClockSamples; ++i) {
            if (!h.prof[i].name) continue;
            if (count < cap) {
                // every pair of (slot of this sample, slot of the next) whose ratio is a possible clock
                std::vector<double> r;
                for (int x = 0; x < kClockSlots; ++x) {
                    const unsigned long long* a = &v[2 * (kClockSlots * i + x)];
                    for (int y = 0; y < kClockSlots; ++y) {
                        const unsigned long long* b = &v[2 * (kClockSlots * (i + 1) + y)];
                        if (b[1] <= a[1] || b[0] <= a[0]) continue;
                        const double f = (double)(b[0] - a[0]) / (double)(b[1] - a[1]) * wall_khz * 1e-3;
                        if (f > 300.0 && f < 3000.0) r.push_back(f);
                    }
                }
                std::sort(r.begin(), r.end());
                const int n = (int)r.size();
                const double sum = n ? r[n / 2] * n : 0.0;        // the median
                if (names) names[count] = h.prof[i].name;
                if (mhz) mhz[count] = n ? (float)(sum / n) : 0.f;
            }
            ++count;
        }
    });
    return rc == 0 ? count : rc;
}

int sub_profile_read(void* handle, int cap, const char** names, float* ms) {
    int count = 0;
    int rc = guarded([&] {
        Handle& h = as_handle(handle);
        hip_check(hipStreamSynchronize(h.stream), "hipStreamSynchronize");
        for (size_t i = 0; i + 1 < h.prof_used; ++i) {
            if (!h.prof[i].name) continue;             // the marker between the two passes
            if (count < cap) {
                float t = 0.f;
                hip_check(hipEventElapsedTime(&t, h.prof[i].a, h.prof[i + 1].a), "hipEventElapsedTime");
                if (names) names[count] = h.prof[i].name;
                if (ms) ms[count] = t;
            }
            ++count;
        }
    });
    return rc == 0 ? count : rc;
}

int sub_op_softmax(void* handle, const void* beta, const char* l_beta, void* alpha,
                   const char* l_alpha, void* mask, const char* l_mask, void* drop,
                   const char* l_drop, float scale, float p, uint32_t site) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_softmax(h, beta, L(h, l_beta), alpha, L(h, l_alpha), mask, L(h, l_mask), drop, L(h, l_drop),
                   scale, p, site);
    });
}

int sub_op_softmax_masked(void* handle, const void* beta, const char* l_beta, void* alpha,
                          const char* l_alpha, void* mask, const char* l_mask, void* drop,
                          const char* l_drop, const void* attn_mask, const char* l_attn_mask,
                          float scale, float mask_scale, float p, uint32_t site) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        Layout lam = L(h, l_attn_mask);
        op_softmax(h, beta, L(h, l_beta), alpha, L(h, l_alpha), mask, L(h, l_mask), drop, L(h, l_drop),
                   scale, p, site, attn_mask, &lam, mask_scale);
    });
}

namespace {
// Operands of the attention operators: layouts over (B, J or K, H, P) with the
// numbers of query and key positions given per call (they differ in
// encoder-decoder attention, substation/transformer.py:288-441).
void op_attention_args(Handle& h, int n_queries, int n_keys, const void* q, const char* l_q, const void* k,
                       const void* v, const char* l_kv, const void* out, const char* l_out, void* stats,
                       void* keep, const void* attn_mask, const char* l_attn_mask, float scale, AttnArgs& a) {
    if (n_queries <= 0 || n_keys <= 0) fail("attention: numbers of query and key positions must be positive");
    Sizes z = h.sz;
    z.n[dJ] = n_queries; z.n[dK] = n_keys;
    const Layout lq = make_layout(l_q, z), lkv = make_layout(l_kv, z), lo = make_layout(l_out, z);
    if (!attn_side(q, lq, dJ, a.q) || !attn_side(k, lkv, dK, a.k) || !attn_side(v, lkv, dK, a.v) ||
        !attn_side(out, lo, dJ, a.o))
        fail("attention: q and out take a layout over B, J, H, P and k, v one over B, K, H, P, P innermost");
    a.H = (int)z.n[dH]; a.B = (int)z.n[dB]; a.J = n_queries; a.K = n_keys;
    a.alpha = scale;
    a.lse = (float*)stats; a.dsum = a.lse + (size_t)a.H * a.B * a.J;
    a.keep = (uint32_t*)keep;
    if (attn_mask) {
        const Layout lm = make_layout(l_attn_mask, z);
        if (lm.rank != 2 || !lm.has[dJ] || !lm.has[dK]) fail("attention: the mask layout must be JK or KJ");
        a.amask = (const half_t*)attn_mask; a.am_sj = lm.stride[dJ]; a.am_sk = lm.stride[dK];
    }
}
}  // namespace

int sub_op_attention_forward(void* handle, int n_queries, int n_keys, const void* q, const char* l_q,
                             const void* k, const void* v, const char* l_kv, void* out, const char* l_out,
                             void* stats, void* keep, const void* attn_mask, const char* l_attn_mask,
                             float scale, float p, uint32_t site) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        AttnArgs a;
        op_attention_args(h, n_queries, n_keys, q, l_q, k, v, l_kv, out, l_out, stats, keep, attn_mask,
                          l_attn_mask, scale, a);
        launch_mha_forward(a, (int)h.sz.n[dP], make_key(h, site, p), h.stream);
    });
}

int sub_op_attention_backward(void* handle, int n_queries, int n_keys, const void* q, const char* l_q,
                              const void* k, const void* v, const char* l_kv, const void* out,
                              const char* l_out, const void* d_out, const char* l_dout, void* stats,
                              const void* keep, void* dq, const char* l_dq, void* dk, void* dv,
                              const char* l_dkv, const void* attn_mask, const char* l_attn_mask, float scale) {
    return sub_op_attention_backward_biases(handle, n_queries, n_keys, q, l_q, k, v, l_kv, out, l_out, d_out, l_dout,
                                            stats, keep, dq, l_dq, dk, dv, l_dkv, attn_mask, l_attn_mask, scale,
                                            nullptr, nullptr, nullptr);
}

int sub_op_attention_backward_biases(void* handle, int n_queries, int n_keys, const void* q, const char* l_q,
                                     const void* k, const void* v, const char* l_kv, const void* out,
                                     const char* l_out, const void* d_out, const char* l_dout, void* stats,
                                     const void* keep, void* dq, const char* l_dq, void* dk, void* dv,
                                     const char* l_dkv, const void* attn_mask, const char* l_attn_mask, float scale,
                                     void* dq_bias, void* dk_bias, void* dv_bias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        if ((dk_bias == nullptr) != (dv_bias == nullptr))
            fail("attention backward: dk_bias and dv_bias come from one launch, give both or neither");
        AttnArgs a;
        op_attention_args(h, n_queries, n_keys, q, l_q, k, v, l_kv, out, l_out, stats, const_cast<void*>(keep),
                          attn_mask, l_attn_mask, scale, a);
        Sizes z = h.sz;
        z.n[dJ] = n_queries; z.n[dK] = n_keys;
        if (!attn_side(d_out, make_layout(l_dout, z), dJ, a.d_o) || !attn_side(dq, make_layout(l_dq, z), dJ, a.dq) ||
            !attn_side(dk, make_layout(l_dkv, z), dK, a.dk) || !attn_side(dv, make_layout(l_dkv, z), dK, a.dv))
            fail("attention backward: d_out and dq take a layout over B, J, H, P and dk, dv one over B, K, H, P, "
                 "P innermost");
        // the sums over (sample, position) of dq, dk, dv start in these launches (one partial row per block of
        // 128 positions) and end in the finishing stage of the column sums, deferred or not
        const int P = (int)h.sz.n[dP], H = (int)h.sz.n[dH];
        const int ntq = a.B * (a.J / 128), ntk = a.B * (a.K / 128);
        auto finish = [&](float* ws, int ns, int ntc, void* o0, void* o1) {
            FinishJob job{ws, FinishArgs{{(half_t*)o0, (half_t*)o1, nullptr, nullptr}, 0, P, 1, H}, ns, H, ntc, P};
            finish_or_defer(defer_of(h), job, h.stream);
        };
        if (dq_bias) a.bias_q = take_ws(h, (size_t)H * ntq * P);
        launch_mha_backward_dq(a, P, h.stream);
        if (dq_bias) finish(a.bias_q, 1, ntq, dq_bias, nullptr);
        if (dk_bias) a.bias_kv = take_ws(h, (size_t)2 * H * ntk * P);
        launch_mha_backward_dkv(a, P, h.stream);
        if (dk_bias) finish(a.bias_kv, 2, ntk, dk_bias, dv_bias);
    });
}

int sub_set_attention_mask(void* handle, const void* attn_mask, const char* layout) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        h.mask_plan_built = false;
        if (!attn_mask) { h.attn_mask = nullptr; return; }
        Layout l = L(h, layout);
        if (l.rank != 2 || !l.has[dJ] || !l.has[dK]) fail("sub_set_attention_mask: layout must be JK or KJ");
        h.attn_mask = attn_mask; h.l_attn_mask = l;
        const Sizes& z = h.sz;
        if (z.n[dJ] % 128 == 0 && z.n[dK] % 128 == 0 && !h.mask_plan) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(h.stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
                fail("sub_set_attention_mask: allocates a small table, call it outside the graph capture");
            const size_t bytes = mha_mask_plan_bytes(z.n[dJ], z.n[dK]);
            hip_check(hipMalloc(&h.mask_plan, bytes), "hipMalloc(mask plan)");
            h.mask_plan_bytes = bytes;
        }
    });
}

int sub_op_bs(void* handle, const void* alpha, const char* l_alpha, const void* mask,
              const char* l_mask, const void* ddrop, const char* l_ddrop, void* dbeta,
              const char* l_dbeta, float scale) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_bs(h, alpha, L(h, l_alpha), mask, L(h, l_mask), ddrop, L(h, l_ddrop), dbeta, L(h, l_dbeta), scale);
    });
}

int sub_op_bdrln(void* handle, const void* in, const char* l_in, const void* resid,
                 const char* l_resid, const void* linear_bias, const void* scale, const void* bias,
                 void* lin, const char* l_lin, void* mask, const char* l_mask, void* diff,
                 const char* l_diff, void* normed, const char* l_normed, void* out,
                 const char* l_out, void* istd, const char* l_istd, float p, uint32_t site) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_bdrln(h, in, L(h, l_in), resid, L(h, l_resid), linear_bias, scale, bias, lin, L(h, l_lin),
                 mask, L(h, l_mask), diff, L(h, l_diff), normed, L(h, l_normed), out, L(h, l_out),
                 istd, L(h, l_istd), p, site);
    });
}

int sub_op_blnrd(void* handle, const void* dout, const char* l_dout, const void* istd,
                 const char* l_istd, const void* diff, const char* l_diff, const void* mask,
                 const char* l_mask, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                 const char* l_d_drop_in) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_blnrd(h, dout, L(h, l_dout), istd, L(h, l_istd), diff, L(h, l_diff), mask, L(h, l_mask),
                 d_ln_in, L(h, l_d_ln_in), d_drop_in, L(h, l_d_drop_in));
    });
}

int sub_op_bad(void* handle, const void* in, const char* l_in, const void* bias, void* lin,
               const char* l_lin, void* mask, const char* l_mask, void* out, const char* l_out,
               float p, uint32_t site) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_bad(h, in, L(h, l_in), bias, lin, L(h, l_lin), mask, L(h, l_mask), out, L(h, l_out), p, site);
    });
}

int sub_op_bsb(void* handle, const void* in, const char* l_in, const void* scale, const void* dout,
               const char* l_dout, void* din, const char* l_din, void* dscale, void* dbias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_bsb(h, in, L(h, l_in), scale, dout, L(h, l_dout), din, L(h, l_din), dscale, dbias);
    });
}

int sub_op_ebsb(void* handle, const void* in, const char* l_in, const void* scale,
                const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                const void* dlinear, const char* l_dlinear, void* din, const char* l_din,
                void* dscale, void* dbias, void* dlinear_bias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_ebsb(h, in, L(h, l_in), scale, dout1, L(h, l_dout1), dout2, L(h, l_dout2), dlinear,
                L(h, l_dlinear), din, L(h, l_din), dscale, dbias, dlinear_bias);
    });
}

namespace {
void ln_backward_body(Handle& h, int extended, const void* in, const char* l_in, const void* scale,
                      const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                      const void* dlinear, const char* l_dlinear, const void* istd, const char* l_istd,
                      const void* diff, const char* l_diff, const void* mask, const char* l_mask, void* g,
                      const char* l_g, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                      const char* l_d_drop_in, void* dscale, void* dbias, void* dlinear_bias, void* dout_bias) {
    const bool ext = extended != 0;
    if (ext && (!dout2 || !dlinear || !dlinear_bias || !dout_bias))
        fail("sub_op_ln_backward: the extended form needs dout2, dlinear, dlinear_bias and dout_bias");
    const Layout li = L(h, l_in), l1 = L(h, l_dout1), lis = L(h, l_istd), ldf = L(h, l_diff), lm = L(h, l_mask),
                 lg = L(h, l_g), lo1 = L(h, l_d_ln_in), lo2 = L(h, l_d_drop_in);
    const Layout l2 = ext ? L(h, l_dout2) : l1, ldl = ext ? L(h, l_dlinear) : l1;
    if (op_lnbwd(h, ext, in, li, scale, dout1, l1, dout2, l2, dlinear, ldl, istd, lis, diff, ldf, mask, lm, g, lg,
                 d_ln_in, lo1, d_drop_in, lo2, dscale, dbias, dlinear_bias, dout_bias))
        return;
    // shapes or layouts the one-launch form does not take: the separate operators, same results
    if (ext) op_ebsb(h, in, li, scale, dout1, l1, dout2, l2, dlinear, ldl, g, lg, dscale, dbias, dlinear_bias);
    else op_bsb(h, in, li, scale, dout1, l1, g, lg, dscale, dbias);
    op_blnrd(h, g, lg, istd, lis, diff, ldf, mask, lm, d_ln_in, lo1, d_drop_in, lo2);
    if (ext) op_baob(h, d_drop_in, lo2, dout_bias);
}
}  // namespace

int sub_op_ln_backward(void* handle, int extended, const void* in, const char* l_in, const void* scale,
                       const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                       const void* dlinear, const char* l_dlinear, const void* istd, const char* l_istd,
                       const void* diff, const char* l_diff, const void* mask, const char* l_mask, void* g,
                       const char* l_g, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                       const char* l_d_drop_in, void* dscale, void* dbias, void* dlinear_bias, void* dout_bias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        ln_backward_body(h, extended, in, l_in, scale, dout1, l_dout1, dout2, l_dout2, dlinear, l_dlinear, istd, l_istd,
                         diff, l_diff, mask, l_mask, g, l_g, d_ln_in, l_d_ln_in, d_drop_in, l_d_drop_in, dscale, dbias,
                         dlinear_bias, dout_bias);
    });
}

int sub_op_ln_backward_static(void* handle, int extended, const void* in, const char* l_in, const void* scale,
                              const void* dout1, const char* l_dout1, const void* dout2, const char* l_dout2,
                              const void* dlinear, const char* l_dlinear, const void* istd, const char* l_istd,
                              const void* diff, const char* l_diff, const void* mask, const char* l_mask, void* g,
                              const char* l_g, void* d_ln_in, const char* l_d_ln_in, void* d_drop_in,
                              const char* l_d_drop_in, void* dscale, void* dbias, void* dlinear_bias,
                              void* dout_bias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        // The partial rows go to the static array of the current device.  Each kernel of
        // this call writes every partial it later reads, so nothing has to start at zero;
        // the launches that share the array within the call are ordered by the stream.
        struct Use {
            Handle& h;
            Use(Handle& h_, float* p) : h(h_) { h.static_ws = p; }
            ~Use() { h.static_ws = nullptr; }
        } use(h, static_scratch());
        ln_backward_body(h, extended, in, l_in, scale, dout1, l_dout1, dout2, l_dout2, dlinear, l_dlinear, istd, l_istd,
                         diff, l_diff, mask, l_mask, g, l_g, d_ln_in, l_d_ln_in, d_drop_in, l_d_drop_in, dscale, dbias,
                         dlinear_bias, dout_bias);
    });
}

int sub_op_bdrlb(void* handle, const void* ddrop, const char* l_ddrop, const void* mask,
                 const char* l_mask, const void* lin, const char* l_lin, void* dlinear,
                 const char* l_dlinear, void* dbias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_bdrlb(h, ddrop, L(h, l_ddrop), mask, L(h, l_mask), lin, L(h, l_lin), dlinear, L(h, l_dlinear), dbias);
    });
}

int sub_ops_defer(void* handle, int on) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        if (on) {
            if (h.ops_deferring) return;
            h.ops_deferring = h.deferring = true;
            h.ws_cursor = 0;
            h.deferred.n = 0;
        } else if (h.ops_deferring) {
            h.ops_deferring = h.deferring = false;
            FinishJobs jobs = h.deferred;
            h.deferred.n = 0;
            if (jobs.n > 0) launch_colfinish(jobs, h.stream);
        }
    });
}

int sub_op_baob(void* handle, const void* datt, const char* l_datt, void* dbo) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_baob(h, datt, L(h, l_datt), dbo);
    });
}

int sub_op_aib(void* handle, const void* in, const char* l_in, const void* bias, const char* l_bias,
               void* out, const char* l_out) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_aib(h, in, L(h, l_in), bias, L(h, l_bias), out, L(h, l_out));
    });
}

int sub_op_baib(void* handle, const void* d, const char* l_d, void* dbias, const char* l_dbias) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_baib(h, d, L(h, l_d), dbias, L(h, l_dbias));
    });
}

int sub_op_bei(void* handle, const void* dxatt, const char* l_dxatt, const void* dresid1,
               const char* l_dresid1, void* dx, const char* l_dx) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        op_bei(h, dxatt, L(h, l_dxatt), dresid1, L(h, l_dresid1), dx, L(h, l_dx));
    });
}

int sub_probe_fetch(const void* buf, size_t working_set, int to_lds, int iters, int workgroups, void* stream,
                    float* us, float* mhz) {
    return guarded([&] {
        hipStream_t st = (hipStream_t)stream;
        unsigned long long* stamps = nullptr;
        int* sink = nullptr;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        hip_check(hipMalloc(&stamps, sizeof(unsigned long long) * 4 * (size_t)(workgroups > 0 ? workgroups : 1)), "hipMalloc");
        hip_check(hipMalloc(&sink, 4096), "hipMalloc");
        hip_check(hipEventCreate(&e0), "hipEventCreate");
        hip_check(hipEventCreate(&e1), "hipEventCreate");
        auto release = [&] { (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); (void)hipFree(stamps); (void)hipFree(sink); };
        try {
            float ms = 0.f;
            for (int rep = 0; rep < 2; ++rep) {       // the second launch is the one measured
                hip_check(hipEventRecord(e0, st), "hipEventRecord");
                launch_fetch_probe(buf, working_set, to_lds, iters, workgroups, stamps, sink, st);
                hip_check(hipEventRecord(e1, st), "hipEventRecord");
                hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
                hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
            }
            std::vector<unsigned long long> v(4 * (size_t)workgroups);
            hip_check(hipMemcpy(v.data(), stamps, v.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost), "hipMemcpy");
            int dev = 0, wall_khz = 0;
            hip_check(hipGetDevice(&dev), "hipGetDevice");
            hip_check(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, dev), "hipDeviceGetAttribute");
            std::vector<double> f;
            for (int b = 0; b < workgroups; ++b)
                if (v[4 * b + 3] > v[4 * b + 1] && v[4 * b + 2] > v[4 * b])
                    f.push_back((double)(v[4 * b + 2] - v[4 * b]) / (double)(v[4 * b + 3] - v[4 * b + 1]) * wall_khz * 1e-3);
            std::sort(f.begin(), f.end());
            if (us) *us = ms * 1e3f;
            if (mhz) *mhz = f.empty() ? 0.f : (float)f[f.size() / 2];
        } catch (...) { release(); throw; }
        release();
    });
}

int sub_op_relayout(void* handle, const void* src, const char* l_src, void* dst, const char* l_dst) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        if (!src || !dst) fail("sub_op_relayout: null tensor pointer");
        ProfScope ps(h, "relayout");
        launch_relayout(L(h, l_src), L(h, l_dst), (const half_t*)src, (half_t*)dst, h.stream);
    });
}

int sub_op_einsum(void* handle, const void* A, const char* l_A, const void* B, const char* l_B,
                  void* C, const char* l_C, float alpha) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        GemmShape g = classify_einsum(L(h, l_A), L(h, l_B), L(h, l_C));
        GemmEpilogue ep;
        ensure_gws(h, gemm_splitk_ws_floats(g));
        launch_gemm(g, (const half_t*)A, (const half_t*)B, (half_t*)C, alpha, ep, h.stream, h.gws, h.gws_floats);
    });
}

int sub_op_einsum_add(void* handle, const void* A, const char* l_A, const void* B, const char* l_B,
                      const void* T, const char* l_T, void* C, const char* l_C, float alpha) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        const Layout lc = L(h, l_C), lt = L(h, l_T);
        GemmShape g = classify_einsum(L(h, l_A), L(h, l_B), lc);
        GemmEpilogue ep;
        if (!T) fail("sub_op_einsum_add: null addend");
        if (!addend_strides(g, lt, lc, ep.sbM, ep.sbN, ep.sbb))
            fail(std::string("sub_op_einsum_add: the dims of ") + l_T + " are not free or batch dims of " + l_C +
                 " in one dense run each");
        ep.bias = (const half_t*)T;
        if (gemm_kernel_kind(g, A, B, C, ep) != 1)
            fail("sub_op_einsum_add: these layouts go to the kernel without an epilogue (addend and output "
                 "must be contiguous along the same free dims)");
        ensure_gws(h, gemm_splitk_ws_floats(g));
        launch_gemm(g, (const half_t*)A, (const half_t*)B, (half_t*)C, alpha, ep, h.stream, h.gws, h.gws_floats);
    });
}

int sub_op_einsum_pair(void* handle, const void* A1, const char* l_A1, const void* B1, const char* l_B1,
                       const void* T1, const char* l_T1, void* C1, const char* l_C1, float alpha1,
                       const void* A2, const char* l_A2, const void* B2, const char* l_B2, void* C2,
                       const char* l_C2, float alpha2, int* paired) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        const Layout lc1 = L(h, l_C1);
        GemmShape g1 = classify_einsum(L(h, l_A1), L(h, l_B1), lc1);
        GemmShape g2 = classify_einsum(L(h, l_A2), L(h, l_B2), L(h, l_C2));
        GemmEpilogue ep1;
        if (T1) {
            if (!l_T1 || !addend_strides(g1, L(h, l_T1), lc1, ep1.sbM, ep1.sbN, ep1.sbb))
                fail(std::string("sub_op_einsum_pair: the dims of the addend are not free or batch dims of ") + l_C1 +
                     " in one dense run each");
            ep1.bias = (const half_t*)T1;
            if (gemm_kernel_kind(g1, A1, B1, C1, ep1) != 1)
                fail("sub_op_einsum_pair: these layouts go to the kernel without an epilogue (addend and output "
                     "must be contiguous along the same free dims)");
        }
        size_t need = gemm_splitk_ws_floats(g1), need2 = gemm_splitk_ws_floats(g2);
        ensure_gws(h, need > need2 ? need : need2);
        bool done = h.pair_products &&
                    launch_gemm_pair(g1, (const half_t*)A1, (const half_t*)B1, (half_t*)C1, alpha1, ep1, g2,
                                     (const half_t*)A2, (const half_t*)B2, (half_t*)C2, alpha2, GemmEpilogue{},
                                     h.stream, h.gws, h.gws_floats);
        if (!done) {
            launch_gemm(g1, (const half_t*)A1, (const half_t*)B1, (half_t*)C1, alpha1, ep1, h.stream, h.gws, h.gws_floats);
            launch_gemm(g2, (const half_t*)A2, (const half_t*)B2, (half_t*)C2, alpha2, GemmEpilogue{}, h.stream, h.gws,
                        h.gws_floats);
        }
        if (paired) *paired = done ? 1 : 0;
    });
}

int sub_op_einsum_bad(void* handle, const void* A, const char* l_A, const void* B, const char* l_B, const void* bias,
                      const char* l_bias, void* lin, void* out, const char* l_out, void* bits, float p, uint32_t site,
                      int* applied) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        if (!applied) fail("sub_op_einsum_bad: null `applied`");
        *applied = 0;
        const Layout lc = L(h, l_out);
        GemmShape g = classify_einsum(L(h, l_A), L(h, l_B), lc);
        GemmEpilogue ep;
        if (!bias || !bits || !addend_strides(g, L(h, l_bias), lc, ep.sbM, ep.sbN, ep.sbb)) return;
        ep.bias = (const half_t*)bias;
        ep.relu_dropout = true; ep.key = make_key(h, site, p);
        ep.gate_bits_out = (uint32_t*)bits;
        if (h.act == ACT_GELU) { ep.act = ACT_GELU; ep.pre_out = (half_t*)lin; }
        // the keep bits are indexed by the offset into the output: it has to be dense in canonical order
        if (lc.str() != "BJU" || ((uintptr_t)bits & 3) || !aligned16(bias) || !aligned16(out) || !aligned16(A) ||
            !aligned16(B) || (h.act == ACT_GELU && (!lin || !aligned16(lin))) ||
            !gemm_relu_dropout_ok(g, A, B, out, ep))
            return;
        launch_gemm(g, (const half_t*)A, (const half_t*)B, (half_t*)out, 1.f, ep, h.stream);
        *applied = 1;
    });
}

int sub_op_einsum_bdrlb(void* handle, const void* A, const char* l_A, const void* B, const char* l_B, const void* gate,
                        const char* l_gate, const void* bits, void* dlinear, const char* l_dlinear, void* dbias,
                        int* applied) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        if (!applied) fail("sub_op_einsum_bdrlb: null `applied`");
        *applied = 0;
        const Layout lc = L(h, l_dlinear);
        GemmShape g = classify_einsum(L(h, l_A), L(h, l_B), lc);
        GemmEpilogue ep;
        if (!gate || !bits || !dbias || !addend_strides(g, L(h, l_gate), lc, ep.sbM, ep.sbN, ep.sbb)) return;
        ep.gate = (const half_t*)gate; ep.gate_bits = (const uint32_t*)bits; ep.colsum = (float*)16;
        if (h.act == ACT_GELU) ep.act = ACT_GELU;
        if (lc.str() != "BJU" || ep.sbb[0] != 0 || ((uintptr_t)bits & 3) || !aligned16(gate) || !aligned16(dlinear) ||
            !aligned16(A) || !aligned16(B) || !gemm_relu_dropout_ok(g, A, B, dlinear, ep))
            return;
        const int ntc = (int)(g.M / 128), U = (int)g.N;
        float* ws = take_ws(h, (size_t)ntc * U);
        ep.colsum = ws;
        launch_gemm(g, (const half_t*)A, (const half_t*)B, (half_t*)dlinear, 1.f, ep, h.stream);
        FinishJob job{ws, FinishArgs{{(half_t*)dbias, nullptr, nullptr, nullptr}, 0, 0, 1, 1}, 1, 1, ntc, U};
        finish_or_defer(defer_of(h), job, h.stream);
        *applied = 1;
    });
}

int sub_layout_strides(void* handle, const char* layout, int64_t strides[8]) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        Layout l = L(h, layout);
        for (int d = 0; d < NDIM; ++d) strides[d] = l.has[d] ? l.stride[d] : 0;
    });
}

int sub_einsum_classify(void* handle, const char* l_A, const char* l_B, const char* l_C,
                        int64_t out[32]) {
    return guarded([&] {
        Handle& h = as_handle(handle); need_cfg(h);
        GemmShape g = classify_einsum(L(h, l_A), L(h, l_B), L(h, l_C));
        out[0] = g.batch(); out[1] = g.M; out[2] = g.N; out[3] = g.K();
        out[4] = g.sAM; out[5] = g.sAK1; out[6] = g.sAb[0];
        out[7] = g.sBN; out[8] = g.sBK1; out[9] = g.sBb[0];
        out[10] = g.sCM; out[11] = g.sCN; out[12] = g.sCb[0];
        out[13] = g.nbatch; out[14] = g.K0; out[15] = g.sAK0; out[16] = g.sBK0;
        // alignment of real buffers is unknown here: assume 16-byte aligned bases
        out[17] = gemm_kernel_kind(g, (const void*)16, (const void*)16, (const void*)16);
        for (int i = 0; i < 3; ++i) {
            out[18 + i] = g.nb[i]; out[21 + i] = g.sAb[i]; out[24 + i] = g.sBb[i]; out[27 + i] = g.sCb[i];
        }
        out[30] = g.K1; out[31] = 0;
    });
}

int sub_philox_fields_host(uint64_t seed, uint32_t site, uint32_t step, uint64_t start, uint64_t n,
                           uint16_t* out) {
    return guarded([&] {
        PhiloxKey k{}; k.k0 = (uint32_t)seed; k.k1 = (uint32_t)(seed >> 32); k.site = site; k.step = step; k.thr = 0;
        for (uint64_t i = 0; i < n; ++i) {
            uint64_t e = start + i;
            U4 r = philox_group(k, e >> 3);
            out[i] = (uint16_t)field16(r, (int)(e & 7));
        }
    });
}

uint32_t sub_dropout_threshold(float p) { return threshold16(p); }

}  // extern "C"
