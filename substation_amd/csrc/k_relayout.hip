// Copies a tensor from one dimension order into another (same logical index space, both dense).
//
// The reference has no such operator: its kernels are generated per layout (pytorch_module/encoder.py:213-376)
// and read whatever order the configuration names.  Here the layer runs in the orders the fused paths of this
// hardware want (token-major rows with the feature dim contiguous) and tensors the caller hands over or gets
// back in another order -- the input, the output, their gradients, the weights and their gradients under the
// reference's shipped feature-major configurations -- cross that boundary through this kernel.
//
// 64 x 64 tiles over (the dim that is contiguous in the source, the dim that is contiguous in the
// destination), 128-bit accesses on both sides, turned around in LDS; when both sides are contiguous along
// the same dim, a plain vector copy with re-computed offsets; a scalar kernel for sizes that are not
// multiples of 8.
#include "sub_ops.hpp"

namespace sub {

namespace {

constexpr int kMaxRank = 5;

struct RelayoutArgs {
    const half_t* src; half_t* dst;
    int rank;                       // dims 0 .. rank-1 in the order below
    // dim 0: contiguous in the source; dim 1: contiguous in the destination (tiled kernel) --
    // or dim 0 contiguous in both (vector kernel); the others in any order
    int n[kMaxRank];
    long ss[kMaxRank], sd[kMaxRank];
};

constexpr int TILE = 64, PITCH = TILE + 2;      // halves; the odd word pitch spreads a column over the banks

__device__ __forceinline__ void relayout_tiled(const RelayoutArgs& a, unsigned b, half_t* tile) {
    const int t0 = (a.n[0] + TILE - 1) / TILE, t1 = (a.n[1] + TILE - 1) / TILE;
    const int i0 = (int)(b % t0) * TILE; b /= t0;
    const int i1 = (int)(b % t1) * TILE; b /= t1;
    long so = 0, dofs = 0;
    for (int d = 2; d < a.rank; ++d) {
        const unsigned i = b % (unsigned)a.n[d]; b /= (unsigned)a.n[d];
        so += (long)i * a.ss[d]; dofs += (long)i * a.sd[d];
    }
    const int tid = threadIdx.x;
    // in: rows along dim 1, 8-packs along dim 0
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int q = tid + k * 256, r = q >> 3, c = (q & 7) * 8;
        if (i1 + r < a.n[1] && i0 + c < a.n[0]) {
            const h8 v = *reinterpret_cast<const h8*>(a.src + so + (long)(i1 + r) * a.ss[1] + (i0 + c));
#pragma unroll
            for (int e = 0; e < 8; ++e) tile[r * PITCH + c + e] = v[e];
        }
    }
    __syncthreads();
    // out: rows along dim 0, 8-packs along dim 1
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int q = tid + k * 256, r = q >> 3, c = (q & 7) * 8;
        if (i0 + r < a.n[0] && i1 + c < a.n[1]) {
            h8 v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = tile[(c + e) * PITCH + r];
            *reinterpret_cast<h8*>(a.dst + dofs + (long)(i0 + r) * a.sd[0] + (i1 + c)) = v;
        }
    }
}

// dim 0 contiguous on both sides: one 8-pack per thread, offsets from the other dims' strides
__device__ __forceinline__ void relayout_vector(const RelayoutArgs& a, unsigned block) {
    long packs = a.n[0] / 8;
    for (int d = 1; d < a.rank; ++d) packs *= a.n[d];
    long q = (long)block * 256 + threadIdx.x;
    if (q >= packs) return;
    const int p0 = a.n[0] / 8;
    long so = (q % p0) * 8, dofs = so;
    q /= p0;
    for (int d = 1; d < a.rank; ++d) {
        const long i = q % a.n[d]; q /= a.n[d];
        so += i * a.ss[d]; dofs += i * a.sd[d];
    }
    *reinterpret_cast<h8*>(a.dst + dofs) = *reinterpret_cast<const h8*>(a.src + so);
}

__device__ __forceinline__ void relayout_scalar(const RelayoutArgs& a, unsigned block) {
    long total = 1;
    for (int d = 0; d < a.rank; ++d) total *= a.n[d];
    long q = (long)block * 256 + threadIdx.x;
    if (q >= total) return;
    long so = 0, dofs = 0;
    for (int d = 0; d < a.rank; ++d) {
        const long i = q % a.n[d]; q /= a.n[d];
        so += i * a.ss[d]; dofs += i * a.sd[d];
    }
    a.dst[dofs] = a.src[so];
}

// Several tensors in one launch: workgroups first[j] .. first[j+1]-1 copy tensor j.
constexpr int kMaxJobs = 8;
enum { MODE_TILED = 0, MODE_VECTOR = 1, MODE_SCALAR = 2 };
struct RelayoutBatch {
    RelayoutArgs a[kMaxJobs];
    int mode[kMaxJobs];
    unsigned first[kMaxJobs + 1];
    int n;
};

__global__ __launch_bounds__(256) void k_relayout(RelayoutBatch b) {
    __shared__ half_t tile[TILE * PITCH];
    int j = 0;
    while (j + 1 < b.n && blockIdx.x >= b.first[j + 1]) ++j;
    const unsigned block = blockIdx.x - b.first[j];
    if (b.mode[j] == MODE_TILED) relayout_tiled(b.a[j], block, tile);
    else if (b.mode[j] == MODE_VECTOR) relayout_vector(b.a[j], block);
    else relayout_scalar(b.a[j], block);
}

// How tensor (ls -> ld) is copied and by how many workgroups.
unsigned plan_relayout(const Layout& ls, const Layout& ld, const half_t* src, half_t* dst, RelayoutArgs& a, int& mode) {
    if (ls.rank != ld.rank || ls.numel != ld.numel) fail("relayout: the two layouts do not name the same tensor");
    if (ls.rank > kMaxRank) fail("relayout: more than five dimensions");
    int cs = -1, cd = -1;           // the logical dims with unit stride (the innermost of extent > 1, else the last)
    for (int i = 0; i < ls.rank; ++i) {
        if (!ld.has[ls.dims[i]] || ld.size[ls.dims[i]] != ls.size[ls.dims[i]])
            fail("relayout: the two layouts do not name the same dimensions");
        if (ls.stride[ls.dims[i]] == 1) cs = ls.dims[i];
        if (ld.stride[ld.dims[i]] == 1) cd = ld.dims[i];
    }
    a.src = src; a.dst = dst; a.rank = ls.rank;
    int order[kMaxRank], k = 0;
    order[k++] = cs;
    if (cd != cs) order[k++] = cd;
    for (int i = ld.rank - 1; i >= 0; --i)       // the rest innermost-of-destination first
        if (ld.dims[i] != cs && ld.dims[i] != cd) order[k++] = ld.dims[i];
    for (int i = 0; i < a.rank; ++i) {
        a.n[i] = (int)ls.size[order[i]]; a.ss[i] = ls.stride[order[i]]; a.sd[i] = ld.stride[order[i]];
    }
    for (int i = a.rank; i < kMaxRank; ++i) { a.n[i] = 1; a.ss[i] = a.sd[i] = 0; }
    const bool aligned = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
    bool vec = aligned && a.n[0] % 8 == 0;
    for (int i = 1; i < a.rank; ++i) vec = vec && a.ss[i] % 8 == 0;
    long blocks;
    if (cd == cs) {
        for (int i = 1; i < a.rank; ++i) vec = vec && a.sd[i] % 8 == 0;
        mode = vec ? MODE_VECTOR : MODE_SCALAR;
        blocks = ((vec ? ls.numel / 8 : ls.numel) + 255) / 256;
    } else {
        vec = vec && a.n[1] % 8 == 0 && a.sd[0] % 8 == 0;
        for (int i = 2; i < a.rank; ++i) vec = vec && a.sd[i] % 8 == 0;
        mode = vec ? MODE_TILED : MODE_SCALAR;
        if (vec) {
            blocks = (long)((a.n[0] + TILE - 1) / TILE) * ((a.n[1] + TILE - 1) / TILE);
            for (int i = 2; i < a.rank; ++i) blocks *= a.n[i];
        } else {
            blocks = (ls.numel + 255) / 256;
        }
    }
    if (blocks > 0x3fffffffL) fail("relayout: tensor too large");
    return (unsigned)blocks;
}

}  // namespace

void launch_relayout_batch(const RelayoutJob* jobs, int n, hipStream_t st) {
    int done = 0;
    while (done < n) {
        RelayoutBatch b;
        b.n = 0; b.first[0] = 0;
        while (done < n && b.n < kMaxJobs) {
            const RelayoutJob& j = jobs[done++];
            if (j.ls.numel == 0) continue;
            const unsigned blocks = plan_relayout(j.ls, j.ld, j.src, j.dst, b.a[b.n], b.mode[b.n]);
            if ((unsigned long)b.first[b.n] + blocks > 0x7fffffffUL) fail("relayout: too many workgroups in one launch");
            b.first[b.n + 1] = b.first[b.n] + blocks;
            ++b.n;
        }
        if (b.n == 0) continue;
        hipLaunchKernelGGL(k_relayout, dim3(b.first[b.n]), dim3(256), 0, st, b);
        check_launch("relayout");
    }
}

void launch_relayout(const Layout& ls, const Layout& ld, const half_t* src, half_t* dst, hipStream_t st) {
    RelayoutJob j{ls, ld, src, dst};
    launch_relayout_batch(&j, 1, st);
}

}  // namespace sub
