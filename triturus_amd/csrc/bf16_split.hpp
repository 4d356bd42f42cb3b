// Cutting fp32 values into bf16 pieces for the bf16 matrix pipe (shared by lm2exp_bf16.hip and
// lt2exp_bf16.hip): x = x0 + x1 [+ x2], each piece the round-to-nearest bf16 of what the
// previous pieces left.  Two pieces carry 16 significand bits, three carry all 24.
#pragma once

#include "common.hpp"

namespace trt {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));

// two fp32 -> one register of two bf16 (round to nearest even), element 0 in the low half
__device__ __forceinline__ uint32_t pack_bf16(float x0, float x1) {
    floatx2 v = {x0, x1};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf16_lo_as_f32(uint32_t pk) { return __builtin_bit_cast(float, pk << 16); }
__device__ __forceinline__ float bf16_hi_as_f32(uint32_t pk) { return __builtin_bit_cast(float, pk & 0xffff0000u); }

// Cut (x0, x1) into NS bf16 pieces each: out[s] holds piece s of both.  The subtraction is
// exact (the piece agrees with x in its leading bits).  An infinite x leaves inf - inf = NaN
// in the later pieces; with KEEP_INF those are set to 0 so that inf stays inf (two more
// instructions per value: used where the count does not matter).
template <int NS, bool KEEP_INF>
__device__ __forceinline__ void split_pair(float x0, float x1, uint32_t (&out)[NS]) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        out[s] = pack_bf16(x0, x1);
        if (s + 1 < NS) {
            const float f0 = bf16_lo_as_f32(out[s]), f1 = bf16_hi_as_f32(out[s]);
            x0 = (KEEP_INF && __builtin_isinf(f0)) ? 0.f : x0 - f0;
            x1 = (KEEP_INF && __builtin_isinf(f1)) ? 0.f : x1 - f1;
        }
    }
}

}  // namespace trt
