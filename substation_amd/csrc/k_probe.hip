// Measurement only: what the CUs can draw from the L2s and from beyond them with the two load forms
// the contraction kernels use.  The reference has nothing of the kind; the figures it gives are what
// the contraction kernels' operand fetch is priced against.
//
// One workgroup of eight waves per CU; per iteration a workgroup reads one 64 KiB chunk of the working
// set (the bytes of one k-step of a 256 x 256 tile), 1 KiB per wave instruction, each workgroup walking
// the working set from a different start.  A working set below the 4 MiB of one XCD's L2 is answered by
// the L2s, a larger one by the memory-side cache or by HBM.  Two more forms price the memory-bound
// operators: a copy (every chunk read is written to a second region of the same size, the mix of a fused
// operator that reads and writes) and a fill (writes only), with the nontemporal accesses those operators use
// for tensors on their last read or written for a later pass.
#include "sub_ops.hpp"

namespace sub {

namespace {

typedef int i4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) void* global_void_ptr;
typedef __attribute__((address_space(3))) void* lds_void_ptr;

// s_waitcnt immediate that waits for vmcnt <= vm only
constexpr int waitcnt_vm(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | 0x0F70; }

constexpr int PROBE_WAVES = 8, PROBE_CHUNK = 65536, PROBE_NV = PROBE_CHUNK / 1024 / PROBE_WAVES;

// TO_LDS: global_load_lds_dwordx4 into two 64 KiB stages, the chunk before the current one landed before
// the next is requested (what the asynchronous contraction kernel does); otherwise global_load_dwordx4
// into registers, consumed at the end of the iteration (the register-staged kernel's form).
template <bool TO_LDS>
__global__ __launch_bounds__(PROBE_WAVES * 64) void k_fetch_probe(const char* buf, unsigned chunks, int iters,
                                                                  unsigned long long* stamps, int* out) {
    __shared__ __attribute__((aligned(16))) char lds[TO_LDS ? 2 : 1][TO_LDS ? PROBE_CHUNK : 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) {
        stamps[4 * blockIdx.x + 0] = __builtin_readcyclecounter();
        stamps[4 * blockIdx.x + 1] = wall_clock64();
    }
    i4v acc = {0, 0, 0, 0};
    unsigned c = (blockIdx.x * 37u) % chunks;
    for (int it = 0; it < iters; ++it) {
        const char* p = buf + (size_t)c * PROBE_CHUNK + (wave * PROBE_NV) * 1024 + lane * 16;
        if constexpr (TO_LDS) {
#pragma unroll
            for (int i = 0; i < PROBE_NV; ++i)
                __builtin_amdgcn_global_load_lds((global_void_ptr)(p + i * 1024),
                                                 (lds_void_ptr)(lds[it & 1] + (wave * PROBE_NV + i) * 1024), 16, 0, 0);
            __builtin_amdgcn_s_waitcnt(waitcnt_vm(PROBE_NV));
        } else {
            i4v v[PROBE_NV];
#pragma unroll
            for (int i = 0; i < PROBE_NV; ++i) v[i] = *reinterpret_cast<const i4v*>(p + i * 1024);
#pragma unroll
            for (int i = 0; i < PROBE_NV; ++i) acc ^= v[i];
        }
        c = c + 1 < chunks ? c + 1 : 0;
    }
    if constexpr (TO_LDS) {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        __syncthreads();
        acc = *reinterpret_cast<const i4v*>(lds[0] + threadIdx.x * 16);
    }
    if (threadIdx.x == 0) {
        stamps[4 * blockIdx.x + 2] = __builtin_readcyclecounter();
        stamps[4 * blockIdx.x + 3] = wall_clock64();
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) out[threadIdx.x] = acc[0];     // keeps the loads alive
}

// COPY: chunk c of the first `chunks` chunks is read and written to chunk c of the second `chunks`; otherwise
// the chunks are only written.  Every workgroup owns the chunks c = block, block + workgroups, ... so that all
// `chunks` are touched once when iters * workgroups == chunks.
template <bool COPY>
__global__ __launch_bounds__(PROBE_WAVES * 64) void k_stream_probe(char* buf, unsigned chunks, int iters,
                                                                   unsigned long long* stamps) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) {
        stamps[4 * blockIdx.x + 0] = __builtin_readcyclecounter();
        stamps[4 * blockIdx.x + 1] = wall_clock64();
    }
    unsigned c = blockIdx.x % chunks;
    for (int it = 0; it < iters; ++it) {
        const size_t at = (size_t)c * PROBE_CHUNK + (wave * PROBE_NV) * 1024 + lane * 16;
        i4v v[PROBE_NV];
#pragma unroll
        for (int i = 0; i < PROBE_NV; ++i)
            v[i] = COPY ? __builtin_nontemporal_load(reinterpret_cast<const i4v*>(buf + at + i * 1024)) : i4v{it, i, lane, wave};
#pragma unroll
        for (int i = 0; i < PROBE_NV; ++i)
            __builtin_nontemporal_store(v[i], reinterpret_cast<i4v*>(buf + (size_t)chunks * PROBE_CHUNK + at + i * 1024));
        c += gridDim.x;
        if (c >= chunks) c %= chunks;
    }
    if (threadIdx.x == 0) {
        stamps[4 * blockIdx.x + 2] = __builtin_readcyclecounter();
        stamps[4 * blockIdx.x + 3] = wall_clock64();
    }
}

}  // namespace

void launch_fetch_probe(const void* buf, size_t working_set, int form, int iters, int workgroups,
                        unsigned long long* stamps, int* sink, hipStream_t st) {
    const size_t chunks = working_set / PROBE_CHUNK;
    if (!buf || chunks == 0 || chunks > 0xffffffffu) fail("fetch probe: working set of 64 KiB to 256 TiB wanted");
    if (iters <= 0 || workgroups <= 0 || workgroups > 65536) fail("fetch probe: iterations and workgroups must be positive");
    if (form < 0 || form > 3) fail("fetch probe: form 0 (registers), 1 (LDS), 2 (copy) or 3 (fill)");
    if (form >= 2) {
        // (writes the second `working_set` bytes of the buffer)
        if (form == 2)
            hipLaunchKernelGGL(k_stream_probe<true>, dim3(workgroups), dim3(PROBE_WAVES * 64), 0, st, (char*)const_cast<void*>(buf),
                               (unsigned)chunks, iters, stamps);
        else
            hipLaunchKernelGGL(k_stream_probe<false>, dim3(workgroups), dim3(PROBE_WAVES * 64), 0, st, (char*)const_cast<void*>(buf),
                               (unsigned)chunks, iters, stamps);
        check_launch("stream probe");
        return;
    }
    const bool to_lds = form == 1;
    if (to_lds)
        hipLaunchKernelGGL(k_fetch_probe<true>, dim3(workgroups), dim3(PROBE_WAVES * 64), 0, st, (const char*)buf,
                           (unsigned)chunks, iters, stamps, sink);
    else
        hipLaunchKernelGGL(k_fetch_probe<false>, dim3(workgroups), dim3(PROBE_WAVES * 64), 0, st, (const char*)buf,
                           (unsigned)chunks, iters, stamps, sink);
    check_launch("fetch probe");
}

}  // namespace sub
