// Merge of an lm2exp contraction that was cut over J: every split s holds its sum relative to
// its own shift m_s (the shift is found while sweeping, so the pieces end with different ones);
//   c = M + log(sum_s part_s * exp(m_s - M)),  M = max_s m_s,
// added in split order: deterministic.  Shared by the fp32 and the bf16 kernels.
#pragma once

#include "common.hpp"

namespace trt {

static __global__ __launch_bounds__(256) void lm2exp_merge_kernel(const float *__restrict__ part,
                                                                  const float *__restrict__ shift,
                                                                  float *__restrict__ c, int R, int I, int K,
                                                                  int splits, int64_t sc0, int64_t sc1) {
    const int64_t total = (int64_t)R * I * K;
    const int64_t rk = (int64_t)R * K;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
        const int k = (int)(e % K);
        const int64_t ri = e / K;
        const int i = (int)(ri % I);
        const int r = (int)(ri / I);
        const float *sh = shift + (int64_t)r * K + k;
        float M = sh[0];
        for (int sp = 1; sp < splits; ++sp) M = max_nan(M, sh[sp * rk]);
        float sum = 0.f;
        for (int sp = 0; sp < splits; ++sp) {
            // exp(m_s - M) in two halves: the factor alone may flush where the product does not
            const float f = exp_shifted(0.5f * (sh[sp * rk] - M));
            sum += part[(int64_t)sp * total + e] * f * f;
        }
        c[(int64_t)r * sc0 + (int64_t)i * sc1 + k] = log_plus(sum, M);
    }
}

// part: [splits][R][I][K] partial sums; shift: [splits][R][K] their shifts.
static inline void launch_lm2exp_merge(const float *part, const float *shift, float *c, int64_t R, int64_t I,
                                       int64_t K, int splits, int64_t sc0, int64_t sc1, hipStream_t stream) {
    int64_t blocks = ceil_div(R * I * K, 256);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(lm2exp_merge_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, part, shift, c, (int)R,
                       (int)I, (int)K, splits, sc0, sc1);
}

}  // namespace trt
