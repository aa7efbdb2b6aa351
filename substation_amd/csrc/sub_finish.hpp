// Second stage of the column reductions as a device function, shared by the
// finishing kernel and by the kernels that run it in workgroups of their own
// that would otherwise leave CUs idle.
#pragma once
#include "sub_ops.hpp"

namespace sub {

constexpr int kFinishThreads = 256;      // threads of a workgroup that runs finish_block

// One workgroup of kFinishThreads threads: 32 features x 8 slices of the partial
// rows, the slices combined through `red` (8 x 33 floats of LDS).  bx counts the
// 32-feature groups of job j; groups past its end do nothing.
__device__ __forceinline__ void finish_block(const FinishJob& j, long bx, float (*red)[33]) {
    const int fl = threadIdx.x & 31, sl = threadIdx.x >> 5;
    const long idx = bx * 32 + fl;
    const bool ok = idx < (long)j.ns * j.nbatch * j.R;
    int s = 0, f = 0, z = 0;
    float t = 0.f;
    if (ok) {
        long sz = idx / j.R; f = (int)(idx - sz * j.R);
        s = (int)(sz / j.nbatch); z = (int)(sz - (long)s * j.nbatch);
        const float* p = j.ws + sz * j.ntc * j.R + f;
        // eight independent loads per round trip instead of one
        for (int c = sl; c < j.ntc; c += 64) {
            float v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = c + 8 * k < j.ntc ? p[(long)(c + 8 * k) * j.R] : 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) t += v[k];
        }
    }
    red[sl][fl] = t;
    __syncthreads();
    if (sl == 0 && ok) {
        float tot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) tot += red[i][fl];
        j.fo.out[s][(long)(z / j.fo.n1) * j.fo.ob0 + (long)(z % j.fo.n1) * j.fo.ob1 + (long)f * j.fo.of] = (half_t)tot;
    }
}

// 32-feature groups of the largest job: the x extent of a finishing grid.
inline long finish_groups(const FinishJobs& jobs) {
    long maxn = 0;
    for (int i = 0; i < jobs.n; ++i) {
        long n = (long)jobs.j[i].ns * jobs.j[i].nbatch * jobs.j[i].R;
        if (n > maxn) maxn = n;
    }
    return (maxn + 31) / 32;
}

}  // namespace sub
