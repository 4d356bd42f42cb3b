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

// Host-side cost model for cutting a contraction over several workgroups ("split").
// `tiles` output tiles each need `units` steps of `mfmas_per_unit` MFMA instructions per
// wavefront (64 cycles each on a SIMD).  Unsplit, a tile is one workgroup.  A run lasts as long
// as the busiest of the 256 CUs: it holds q = ceil(workgroups / 256) of them, which share its
// matrix pipe, so it needs q chains' worth of MFMA time -- at 45 % of the MFMA rate when it
// holds a single workgroup (one wavefront per SIMD: nothing hides the LDS, barrier and load
// latencies), 65 % with two, 80 % with three, 90 % from four on.  (Measured: 64 steps of 16
// MFMAs alone on a CU take 62 us, two workgroups of 128 steps 175 us, 512 workgroups of 32 steps
// 43 us; counting whole workgroups matters, 288 tiles take twice as long as 256.)  Split s ways
// the chain shrinks s-fold and the CUs fill up, but the partial sums make a round trip through
// memory and a merge kernel is launched.  Returns the split count (1 = do not split) with the
// smallest estimate; a split must win by 20 %.  The merge constants are pessimistic on purpose
// (2 TB/s, 5 us): splits the model rates as marginal were losses when measured.  per_split_us
// adds a cost per split for callers whose merge is bound by its chain of loads; must_win is the
// fraction of the uncut estimate a cut has to stay under.  eff_few: the rate with one and with
// two workgroups on a CU, for kernels that measure other than 45 % and 65 % there (the 64-row
// lt2exp tile, whose steps hold 32 MFMAs: 67 % and 82 %).
inline int choose_splits(int64_t tiles, int64_t units, int64_t mfmas_per_unit, int64_t out_elems,
                         int min_units_per_split, int max_splits, bool forced, double per_split_us = 0.0,
                         double must_win = 0.8, double eff_one = 0.45, double eff_two = 0.65) {
    constexpr double kCyclesPerUs = 2400.0;
    constexpr int64_t kCuCount = 256;
    const double unit_us = (double)mfmas_per_unit * 64.0 / kCyclesPerUs;
    auto estimate = [&](int sp) {
        const double chain_us = (double)ceil_div(units, sp) * unit_us;  // one workgroup at the full MFMA rate
        const int64_t q = ceil_div(tiles * sp, kCuCount);               // workgroups on the busiest CU
        const double eff = q >= 4 ? 0.9 : (q == 3 ? (eff_two > 0.8 ? 0.88 : 0.8) : (q == 2 ? eff_two : eff_one));
        const double body = (double)q * chain_us / eff;
        const double merge_us =
            sp > 1 ? 5.0 + (double)sp * per_split_us + (double)(sp + 1) * (double)out_elems * 4.0 / 2.0e6 : 0.0;
        return body + merge_us;
    };
    int best = 1;
    double best_us = forced ? 1e300 : must_win * estimate(1);
    for (int sp = 2; sp <= max_splits && (int64_t)sp * min_units_per_split <= units; ++sp) {
        const double us = estimate(sp);
        if (us < best_us) {
            best_us = us;
            best = sp;
        }
    }
    if (forced && best == 1 && units >= 2) best = 2;
    return best;
}

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

// ---- buffer addressing: a 128-bit resource (base, byte extent) in scalar registers,
// a 32-bit per-lane byte offset and a wave-uniform scalar byte offset.  No vector ALU
// instruction is spent on the address, and accesses past the extent are dropped
// (loads return 0) by the hardware.
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
constexpr uint32_t kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, kRsrcFlags);
}
__device__ __forceinline__ float buf_load_f32(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ floatx4 buf_load_f32x4(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
__device__ __forceinline__ void buf_store_f32(float v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, voff, soff, 0);
}
// Write-once output: the non-temporal hint keeps the result stream from evicting the
// operand panels that other workgroups still re-read from L2 (measured: 3 % on lm2exp).
constexpr int kCacheNonTemporal = 2;
__device__ __forceinline__ void buf_store_f32_stream(float v, __amdgpu_buffer_rsrc_t r, uint32_t voff,
                                                     uint32_t soff) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), r, voff, soff, kCacheNonTemporal);
}

// Result stores.  Rows of c that are 16-byte aligned take the non-temporal hint; rows that are not
// leave every line written half by one wavefront and half by its neighbour, and with the hint the
// halves reach memory separately (R=41, I=2636, J=12, K=2223: 413 us against 211 with plain
// stores, which merge in L2; aligned K=2224: 180 with the hint, 224 without).  `streaming` is
// wave-uniform (a kernel argument).
__device__ __forceinline__ void buf_store_f32_out(bool streaming, float v, __amdgpu_buffer_rsrc_t r, uint32_t voff,
                                                  uint32_t soff) {
    if (streaming) buf_store_f32_stream(v, r, voff, soff);
    else buf_store_f32(v, r, voff, soff);
}
inline int rows_16_byte_aligned(const void *c, int64_t s0, int64_t s1) {
    return (s0 % 4 == 0 && s1 % 4 == 0 && (reinterpret_cast<uintptr_t>(c) & 15) == 0) ? 1 : 0;
}

// max of three without NaN canonicalisation moves (a NaN operand is ignored, which is
// what the callers want: see the kernels).
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

// exp(x) for a shifted log-value x = b - m (x <= ~8, possibly -inf or NaN) as one
// multiply and the hardware 2^t instruction.  Relative error <= 2^-23 |x log2(e)| + 1 ulp:
// exact near the maximum, where the sum is decided; results below 2^-126 flush to 0.
// The subtraction b - m is done by the caller in plain fp32 (exact for b close to m);
// folding it into an fma with a pre-scaled m * log2(e) would turn the rounding of that
// product into an absolute exponent error of |m| 2^-24, fatal for |m| >~ 1e9.
__device__ __forceinline__ float exp_shifted(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

// Rescaling running sums by exp(d), d <= 0, when the shift moves up: below about e^-87 the factor
// itself is no longer a normal float (it flushes to zero) although sum * exp(d) may well be one --
// the sums were taken relative to the old shift and can be as large as e^margin times the weights.
// When any lane moves by more than this, the factor is applied as two halves, exp(d/2) twice.
constexpr float kDeepRescale = -80.0f;

// m + log(s) from the hardware log2: log2(0) = -inf gives -inf (m is finite), NaN stays NaN.
__device__ __forceinline__ float log_plus(float s, float m) {
    return __builtin_fmaf(__builtin_amdgcn_logf(s), kLn2, m);
}

}  // namespace trt
