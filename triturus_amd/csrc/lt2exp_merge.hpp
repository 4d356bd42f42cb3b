// Merge of an lt2exp contraction that was cut over several workgroups: every split holds a
// partial sum relative to the same shifts ma[r,k] + mb[r,k] (they depend on the column only), so
//   c = (ma + mb) + log(sum over splits of the partial sums),
// added in split order: deterministic, no locks or atomics (the reference merges under a spin
// lock in arrival order, triturus/lt2exp.py:498-506).  Shared by the fp32 and the bf16 kernels.
#pragma once

#include "common.hpp"

namespace trt {

static __global__ __launch_bounds__(256) void lt2exp_merge_kernel(const float *__restrict__ part,
                                                                  const float *__restrict__ shift,
                                                                  float *__restrict__ c, int R, int S, int K,
                                                                  int splits, int64_t sc0, int64_t sc1) {
    const int64_t total = (int64_t)R * S * K;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
        const int k = (int)(e % K);
        const int64_t rs = e / K;
        const int s = (int)(rs % S);
        const int r = (int)(rs / S);
        float sum = 0.f;
        for (int sp = 0; sp < splits; ++sp) sum += part[(int64_t)sp * total + e];
        const float mm = shift[(int64_t)r * K + k] + shift[((int64_t)R + r) * K + k];
        c[(int64_t)r * sc0 + (int64_t)s * sc1 + k] = log_plus(sum, mm);
    }
}

// Launch of the merge: at most 4096 workgroups of 256 threads, grid-stride over R*S*K outputs.
static inline void launch_lt2exp_merge(const float *part, const float *shift, float *c, int64_t R, int64_t S,
                                       int64_t K, int splits, int64_t sc0, int64_t sc1, hipStream_t stream) {
    int64_t blocks = ceil_div(R * S * K, 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(lt2exp_merge_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, part, shift, c, (int)R,
                       (int)S, (int)K, splits, sc0, sc1);
}

}  // namespace trt
