// Shared device helpers for the gfx950 kernels: wave64 primitives, MFMA
// vector types, XCD-aware workgroup numbering.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/triturus_hip.h"

namespace trt {

constexpr int kWave = 64;      // CDNA wavefront width
constexpr int kXcds = 8;       // MI355X: 8 accelerator dies, each with its own L2
constexpr float kClamp = 1e38f;  // max-shift clamp, baselines/lm2exp.py:12

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// The hardware hands consecutive workgroup ids to the 8 XCDs round-robin.
// Renumber so that a run of `total/8` consecutive LOGICAL ids lands on one
// XCD: workgroups that share an operand panel then share one L2.
// `padded_total` must be a multiple of 8; logical ids >= the real total are
// idle (the caller returns early).
__device__ __forceinline__ int64_t xcd_logical_id(int64_t wg, int64_t padded_total) {
    const int64_t per_xcd = padded_total / kXcds;
    return (wg % kXcds) * per_xcd + wg / kXcds;
}

__host__ __device__ __forceinline__ int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

__device__ __forceinline__ float clamp_shift(float m) {
    // NaN-transparent clamp to [-1e38, 1e38] like torch.clamp.
    m = m < -kClamp ? -kClamp : m;
    m = m > kClamp ? kClamp : m;
    return m;
}

// max that lets a NaN through from either side (torch.amax semantics); used
// for the column maxima so a NaN input column yields NaN exactly as the torch
// recipe does.
__device__ __forceinline__ float max_nan(float a, float b) {
    return (a > b || a != a) ? a : b;
}

}  // namespace trt
