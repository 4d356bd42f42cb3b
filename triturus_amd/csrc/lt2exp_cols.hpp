// lt2exp for layers of few units over many batches: a lane per output column.
//
// With I and J of at most 16 a batch holds at most 256 weights per s, and a call is many batches of
// such crumbs: the MFMA tiles of csrc/lt2exp.hip pad s to 32 rows and j to chunks of 16, and run
// 3-6 times over what memory needs (R=8192, S=I=J=8, K=1024: 469 us for 0.8 GB of a, b, c and w;
// S=I=J=4: 417 us where 74 would do).  Here a lane owns one output column (r, k): it loads its
// I values of a and J values of b (consecutive lanes on consecutive k: whole cache lines), shifts
// and exponentiates them in registers, and then, for every s, contracts them with the batch's
// weights -- which are the same for every lane of the wavefront, so they arrive through scalar
// loads and enter the FMAs as scalar operands: S * I * J FMAs per lane, no LDS, no matrix pipe, no
// padding of s.  The column's results leave as one store per s, again whole lines per wavefront.
// Bound by memory while S * I * J stays under about 7 FMAs per byte the lane moves
// (4 (I + J + S) bytes), by the vector ALU beyond.
#pragma once

#include <cmath>
#include <cstdio>

#include "common.hpp"

namespace trt {

struct Lt2ColsArgs {
    const float *w, *a, *b;
    float *c;
    int R, S, I, J, K;
    int64_t sw0, sw1, sw2, sa0, sa1, sa2, sb0, sb1, sb2, sc0, sc1;
    int k_waves;  // wavefronts per batch: ceil(K / 64)
    int64_t total_waves;
};

constexpr int kColsThreads = 256;

// IMAX, JMAX: I and J rounded up to 4, 8 or 16 -- I = 1 stays 1 -- (register arrays; the rows past I and J hold factors
// of zero and their weights are never read).  EXACT: I = IMAX, J = JMAX and a dense flat axis of w:
// the I * J weights of an s are one run of known length, which the compiler fetches 16 to a scalar
// load instead of one by one.
template <int IMAX, int JMAX, bool EXACT>
static __global__ __launch_bounds__(kColsThreads) void lt2exp_cols_kernel(const Lt2ColsArgs p, const float *__restrict__ w_,
                                                                          const float *__restrict__ a_,
                                                                          const float *__restrict__ b_,
                                                                          float *__restrict__ c_) {
    // (the operands as restrict-qualified arguments of their own: only then may the compiler take
    // the wave-uniform loads of w for scalar loads -- through the struct it must assume that the
    // stores to c can change w, and sends a vector load per weight)
    const int lane = (int)threadIdx.x & (kWave - 1);
    const int64_t wave_id = (int64_t)blockIdx.x * (kColsThreads / kWave) + (int)threadIdx.x / kWave;
    if (wave_id >= p.total_waves) return;  // (wave-uniform)
    // a wavefront stays inside one batch: its weights are wave-uniform
    const int r = __builtin_amdgcn_readfirstlane((int)(wave_id / p.k_waves));
    const int kw = __builtin_amdgcn_readfirstlane((int)(wave_id % p.k_waves));
    const int k = kw * kWave + lane;
    const bool live = k < p.K;
    const int kc = live ? k : p.K - 1;  // (lanes past K compute a copy of the last column and store nothing)

    // (no a: the lm2exp entry -- a contracted plane of 1 x J, a factor of one)
    const float *ak = a_ ? a_ + (int64_t)r * p.sa0 + (int64_t)kc * p.sa2 : nullptr;
    const float *bk = b_ + (int64_t)r * p.sb0 + (int64_t)kc * p.sb2;
    float ea[IMAX], eb[JMAX];
#pragma unroll
    for (int i = 0; i < IMAX; ++i) ea[i] = ak && i < p.I ? ak[(int64_t)i * p.sa1] : -__builtin_inff();
#pragma unroll
    for (int j = 0; j < JMAX; ++j) eb[j] = j < p.J ? bk[(int64_t)j * p.sb1] : -__builtin_inff();
    // (a NaN need not survive the maxima: exp(NaN - m) is NaN for any m and poisons the column)
    float ma = -__builtin_inff(), mb = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < IMAX; ++i) ma = __builtin_fmaxf(ma, ea[i]);
#pragma unroll
    for (int j = 0; j < JMAX; ++j) mb = __builtin_fmaxf(mb, eb[j]);
    ma = ak ? clamp_shift(ma) : 0.f;
    mb = clamp_shift(mb);
#pragma unroll
    for (int i = 0; i < IMAX; ++i) ea[i] = i < p.I ? (ak ? exp_shifted(ea[i] - ma) : 1.f) : 0.f;
#pragma unroll
    for (int j = 0; j < JMAX; ++j) eb[j] = j < p.J ? exp_shifted(eb[j] - mb) : 0.f;
    const float shift = ma + mb;

    const float *wr = w_ + (int64_t)r * p.sw0;  // (wave-uniform: scalar loads)
    float *ck = c_ + (int64_t)r * p.sc0 + k;
    if constexpr (EXACT) {
        for (int s = 0; s < p.S; ++s) {
            const float *ws = wr + (int64_t)s * p.sw1;
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < IMAX; ++i) {
                float t = 0.f;
#pragma unroll
                for (int j = 0; j < JMAX; ++j) t = __builtin_fmaf(ws[i * JMAX + j], eb[j], t);
                sum = __builtin_fmaf(ea[i], t, sum);
            }
            if (live) ck[(int64_t)s * p.sc1] = log_plus(sum, shift);
        }
    } else {
        // any I, J and flat stride: i is a real loop (unrolled over i as well, the offsets of all
        // I * J weights are loop invariants that overflow the scalar registers), so the factors of
        // a wait in LDS, a column per thread.  (Blocks of 2-4 rows without a branch inside -- rows and
        // columns past I and J read again from the last ones under weights selected to zero, so that
        // a block's scalar loads go out together -- were twice as slow: 152 -> 266 us on R=8192,
        // S=I=J=6, K=512.)
        __shared__ float ea_lds[IMAX][kColsThreads];
#pragma unroll
        for (int i = 0; i < IMAX; ++i) ea_lds[i][threadIdx.x] = ea[i];  // (read back by the same thread only)
        const int64_t row = (int64_t)p.J * p.sw2;
        for (int s = 0; s < p.S; ++s) {
            const float *wi = wr + (int64_t)s * p.sw1;
            float sum = 0.f;
#pragma unroll 1
            for (int i = 0; i < p.I; ++i, wi += row) {
                float t = 0.f;
                if (p.sw2 == 1) {  // (wave-uniform) dense rows: four weights to a scalar load, the tail one by one
#pragma unroll
                    for (int jq = 0; jq < JMAX / 4; ++jq) {
                        if (4 * jq + 4 <= p.J) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) t = __builtin_fmaf(wi[4 * jq + e], eb[4 * jq + e], t);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (4 * jq + e < p.J) t = __builtin_fmaf(wi[4 * jq + e], eb[4 * jq + e], t);
                        }
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < JMAX; ++j)
                        if (j < p.J) t = __builtin_fmaf(wi[(int64_t)j * p.sw2], eb[j], t);
                }
                sum = __builtin_fmaf(ea_lds[i][threadIdx.x], t, sum);
            }
            if (live) ck[(int64_t)s * p.sc1] = log_plus(sum, shift);
        }
    }
}

// ---- host side

static inline int cols_pad(int64_t n) { return n <= 4 ? 4 : (n <= 8 ? 8 : 16); }
static inline int cols_pad_i(int64_t n) { return n == 1 ? 1 : cols_pad(n); }

static inline bool cols_applies(int64_t I, int64_t J, int64_t K) { return I <= 16 && J <= 16 && K > 8; }

// Is this kernel the faster one?  The sign of a linear score in log2 units, fitted to 400 timed
// shapes (I, J = 1..16, S = 1..160, K = 9..2048, R up to 60 000, 1-240 MB moved) against what the
// other rules choose (the MFMA tiles, or the kernel that contracts j first) -- the estimate of
// log2(their time / this kernel's):
//   - 0.64 per doubling of the FMAs of a lane (S * I * J, padded as the build runs them),
//   - 0.16 per doubling of K,
//   + 0.92 for the exact-size build (16 weights to a scalar load instead of one),
//   + 0.2 per doubling of the call's work (small calls are bound by their launch either way).
// Taking the kernel by this rule costs 2.2 % over the faster choice per shape (geometric mean
// over the fit's shapes; never taking it 25 %, always taking it 98 %).  Outputs of at most 8
// columns are not asked (a wavefront would hold 8 live lanes; the sweep takes most of them).
static inline double cols_score(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_dense) {
    const int im = cols_pad_i(I), jm = cols_pad(J);
    const bool exact = im == I && jm == J && w_dense;
    const double fmas = (double)S * (double)(exact ? im : I) * (double)jm;
    const double work = 2.0 * (double)R * (double)S * (double)I * (double)J * (double)K;
    return 0.79 - 0.64 * std::log2(fmas) - 0.16 * std::log2((double)K) + (exact ? 0.92 : 0.0) + 0.205 * std::log2(work);
}
static inline bool cols_pays(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_dense) {
    return cols_applies(I, J, K) && cols_score(R, S, I, J, K, w_dense) > 0.0;
}

static inline int cols_kernel_name(int64_t I, int64_t J, bool w_dense, char *buf, size_t buf_bytes) {
    const int im = cols_pad_i(I), jm = cols_pad(J);
    const int n = snprintf(buf, buf_bytes, "trt::lt2exp_cols_kernel<%d, %d, %s>", im, jm,
                           im == I && jm == J && w_dense ? "true" : "false");
    return n > 0 && (size_t)n < buf_bytes ? 0 : TRT_E_RANGE;
}

static int launch_lt2exp_cols(const float *w, const float *a, const float *b, float *c, int64_t R, int64_t S, int64_t I,
                              int64_t J, int64_t K, const int64_t sw[3], const int64_t sa[3], const int64_t sb[3],
                              const int64_t sc[3], hipStream_t stream) {
    Lt2ColsArgs args;
    args.w = w; args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.S = (int)S; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sw0 = sw[0]; args.sw1 = sw[1]; args.sw2 = sw[2];
    args.sa0 = sa[0]; args.sa1 = sa[1]; args.sa2 = sa[2];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.k_waves = (int)ceil_div(K, kWave);
    args.total_waves = R * args.k_waves;
    const int64_t grid = ceil_div(args.total_waves, kColsThreads / kWave);
    if (grid >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    const int im = cols_pad_i(I), jm = cols_pad(J);
    const bool exact = im == I && jm == J && sw[2] == 1;
#define TRT_COLS_LAUNCH(IM_, JM_)                                                                                   \
    do {                                                                                                            \
        if (exact)                                                                                                  \
            hipLaunchKernelGGL((lt2exp_cols_kernel<IM_, JM_, true>), dim3((unsigned)grid), dim3(kColsThreads), 0, stream, args, w, a, b, c);  \
        else                                                                                                        \
            hipLaunchKernelGGL((lt2exp_cols_kernel<IM_, JM_, false>), dim3((unsigned)grid), dim3(kColsThreads), 0, stream, args, w, a, b, c); \
    } while (0)
    if (im == 1) {
        if (jm == 4) TRT_COLS_LAUNCH(1, 4);
        else if (jm == 8) TRT_COLS_LAUNCH(1, 8);
        else TRT_COLS_LAUNCH(1, 16);
    } else if (im == 4) {
        if (jm == 4) TRT_COLS_LAUNCH(4, 4);
        else if (jm == 8) TRT_COLS_LAUNCH(4, 8);
        else TRT_COLS_LAUNCH(4, 16);
    } else if (im == 8) {
        if (jm == 4) TRT_COLS_LAUNCH(8, 4);
        else if (jm == 8) TRT_COLS_LAUNCH(8, 8);
        else TRT_COLS_LAUNCH(8, 16);
    } else {
        if (jm == 4) TRT_COLS_LAUNCH(16, 4);
        else if (jm == 8) TRT_COLS_LAUNCH(16, 8);
        else TRT_COLS_LAUNCH(16, 16);
    }
#undef TRT_COLS_LAUNCH
    return (int)hipGetLastError();
}

}  // namespace trt
