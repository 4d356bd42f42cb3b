// lm2exp for narrow outputs of few rows: one tile per batch, its contraction cut over the wavefronts.
//
// With at most 64 columns and at most 32 rows a batch is a single 32 x 32 (or 32 x 64) tile of
// output under a contraction of J terms, and a call is thousands of such batches.  The tiles of
// csrc/lm2exp.hip set their four wavefronts side by side over 128 columns or stack them over 128
// rows: here three of the four would stand idle, and the fourth walks J alone, one small tile of b
// through LDS per step (R=8192, I=1, J=256, K=16: 177 us for 134 MB of b).  This kernel gives a
// workgroup one batch and each of its four wavefronts a quarter of J.  A wavefront first takes the
// column maxima of its quarter of b -- the four meet in LDS --, then reads the quarter a second time
// (it is 4 to 64 KB and still in L2), exponentiates it where it lands, in the MFMA's B layout
// (lane = column, consecutive lanes on consecutive k: whole cache lines), and multiplies by its
// rows of a, which it reads straight into the A layout (lane = row, 16 bytes per load).  Nothing
// passes through LDS but the four partial tiles at the end, which are added in a fixed order.
#pragma once

#include <cmath>

#include "common.hpp"

namespace trt {

struct Lm2JsplitArgs {
    const float *a, *b;
    float *c;
    int R, I, J, K;
    int64_t sa0, sa1, sb0, sb1, sb2, sc0, sc1;  // (rows of a: dense, 16-byte aligned, J a multiple of 4)
    int n_tiles, i_tiles;
};

constexpr int kJsplitWaves = 4;
constexpr int kJsplitThreads = kJsplitWaves * kWave;

// CT: column blocks of 32 per workgroup (K <= 32 CT)
template <int CT>
static __global__ __launch_bounds__(kJsplitThreads) void lm2exp_jsplit_kernel(const Lm2JsplitArgs p) {
    constexpr int NT = 32 * CT;
    __shared__ __attribute__((aligned(16))) float part[kJsplitWaves][CT][16][kWave];  // the wavefronts' partial tiles
    __shared__ float red[kJsplitWaves][NT];
    __shared__ float shift[NT];

    const int tid = (int)threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int n = lane & 31, half = lane >> 5;
    int wg = (int)blockIdx.x;
    const int it = wg % p.i_tiles;
    wg /= p.i_tiles;
    const int nt = wg % p.n_tiles;
    const int r = wg / p.n_tiles;
    const int k0 = nt * NT, i0 = it * 32;

    // this wavefront's part of j: a quarter, in whole groups of 8
    const int n_groups = (p.J + 7) / 8;
    const int g_lo = n_groups * wave / kJsplitWaves, g_hi = n_groups * (wave + 1) / kJsplitWaves;
    const int j_lo = 8 * g_lo, j_hi = 8 * g_hi < p.J ? 8 * g_hi : p.J;

    // b through a buffer resource: a scalar row offset, a 32-bit lane offset (column and lane half),
    // no 64-bit address arithmetic per load
    const float *br = p.b + (int64_t)r * p.sb0;
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(br, (uint32_t)(((int64_t)(p.J - 1) * p.sb1 + (int64_t)(p.K - 1) * p.sb2 + 1) * 4));
    uint32_t bcol[CT];  // this lane's column of b in bytes (columns past K: the last one again, never stored)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int k = k0 + 32 * ct + n;
        bcol[ct] = (uint32_t)((int64_t)(k < p.K ? k : p.K - 1) * p.sb2) * 4u;
    }
    const uint32_t b_row = (uint32_t)p.sb1 * 4u;  // bytes between two values of j

    // ---- column maxima (a NaN need not survive them: exp(NaN - m) is NaN for any m and poisons
    // its column's sums).  The two lane halves take every other j (j_lo and j_hi are even).
    {
        float m[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) m[ct] = -__builtin_inff();
#pragma unroll 4
        for (int j = j_lo; j < j_hi; j += 2)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                m[ct] = __builtin_fmaxf(m[ct], buf_load_f32(b_rsrc, bcol[ct] + (uint32_t)half * b_row, (uint32_t)j * b_row));
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            m[ct] = __builtin_fmaxf(m[ct], __shfl_xor(m[ct], 32, kWave));
            if (half == 0) red[wave][32 * ct + n] = m[ct];
        }
        __syncthreads();
        if (tid < NT) {
            float y = red[0][tid];
#pragma unroll
            for (int w = 1; w < kJsplitWaves; ++w) y = __builtin_fmaxf(y, red[w][tid]);
            shift[tid] = clamp_shift(y);
        }
        __syncthreads();
    }
    float mk[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) mk[ct] = shift[32 * ct + n];

    // ---- the contraction over this wavefront's groups.  MFMA e of a group takes j = 8 g + 4 half + e:
    // lane (row, half) holds a[row, j], lane (column, half) exp(b[j, column] - m).
    const float *ar = p.a + (int64_t)r * p.sa0;
    const int row = i0 + n;
    const uint32_t a_extent = (uint32_t)(((int64_t)(p.I - 1) * p.sa1 + p.J) * 4);
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(ar, a_extent);
    // (rows past I are read past the extent: zeros)
    const uint32_t a_voff = row < p.I ? (uint32_t)(((int64_t)row * p.sa1 + 4 * half) * 4) : a_extent;
    floatx16 acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[ct][v] = 0.f;

    floatx4 a_next;
    float b_next[CT][4];
    auto issue = [&](int g) {
        a_next = buf_load_f32x4(a_rsrc, a_voff, (uint32_t)(32 * g));
#pragma unroll
        for (int e = 0; e < 4; ++e)  // (past J: zeros or a neighbour's values, never used)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                b_next[ct][e] = buf_load_f32(b_rsrc, bcol[ct] + (uint32_t)(4 * half) * b_row, (uint32_t)(8 * g + e) * b_row);
    };
    if (g_lo < g_hi) issue(g_lo);
    for (int g = g_lo; g < g_hi; ++g) {
        floatx4 av = a_next;
        float bv[CT][4];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[ct][e] = b_next[ct][e];
        if (g + 1 < g_hi) issue(g + 1);
        const int room = p.J - 8 * g - 4 * half;  // values of j of this lane's piece inside the row (the last group may be ragged)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool inside = e < room;
            const float aw = inside ? av[e] : 0.f;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const float f = inside ? exp_shifted(bv[ct][e] - mk[ct]) : 0.f;
                acc[ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(aw, f, acc[ct], 0, 0, 0);
            }
        }
    }

    // ---- the four partial tiles, added in a fixed order; accumulator v of a lane is row
    // 8 (v / 4) + 4 half + v % 4 of the tile, column n
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int v = 0; v < 16; ++v) part[wave][ct][v][lane] = acc[ct][v];
    __syncthreads();
    for (int u = tid; u < CT * 16 * kWave; u += kJsplitThreads) {
        const int l = u & (kWave - 1), v = (u >> 6) & 15, ct = u >> 10;
        const int orow = i0 + 8 * (v / 4) + 4 * (l >> 5) + (v & 3), col = 32 * ct + (l & 31);
        if (orow >= p.I || k0 + col >= p.K) continue;
        float sum = part[0][ct][v][l];
#pragma unroll
        for (int w = 1; w < kJsplitWaves; ++w) sum += part[w][ct][v][l];
        p.c[(int64_t)r * p.sc0 + (int64_t)orow * p.sc1 + k0 + col] = log_plus(sum, shift[col]);
    }
}

// ---- host side

// (rows of a read 16 bytes at a time; J of at least 32 so that every wavefront has a group)
static inline bool jsplit_applies(int64_t I, int64_t J, int64_t K, bool a_aligned) {
    return a_aligned && J % 4 == 0 && J >= 32 && K <= 64 && K > 8;
}

// Is this kernel the faster one?  The sign of a linear score in log2 units fitted to 350 timed
// shapes (I = 1..96, J = 32..4096, K = 9..64, up to 60 000 batches) against lm2exp's own tiles:
// 1.5 doublings ahead to begin with, - 0.44 from 33 columns on (two column blocks per wavefront,
// half the workgroups per compute unit), - 0.31 per doubling of the 32-row tiles of a batch (each
// reads b for itself), - 0.16 per halving of the grid below 1024 workgroups (a workgroup walks a
// quarter of J, however long), - 0.08 per doubling of K, - 0.03 per doubling of J.  2.7 % behind
// the faster choice per shape (never taking it 33 %, always 11 %).
static inline double jsplit_score(int64_t R, int64_t I, int64_t J, int64_t K) {
    const double tiles = (double)ceil_div(I, 32);
    const double lgrid = std::log2((double)R * tiles);
    return 1.51 - 0.08 * std::log2((double)K) - 0.031 * std::log2((double)J) - 0.156 * (lgrid < 10.0 ? 10.0 - lgrid : 0.0) -
           0.311 * std::log2(tiles) - (K > 32 ? 0.44 : 0.0);
}
static inline bool jsplit_pays(int64_t R, int64_t I, int64_t J, int64_t K, bool a_aligned) {
    return jsplit_applies(I, J, K, a_aligned) && jsplit_score(R, I, J, K) > 0.0;
}

static int launch_lm2exp_jsplit(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                                const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], hipStream_t stream) {
    Lm2JsplitArgs args;
    args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sa0 = sa[0]; args.sa1 = sa[1];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    const int ct = K > 32 ? 2 : 1;
    args.n_tiles = (int)ceil_div(K, 32 * ct);
    args.i_tiles = (int)ceil_div(I, 32);
    const int64_t grid = R * args.n_tiles * args.i_tiles;
    if (grid >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    if (ct == 1)
        hipLaunchKernelGGL((lm2exp_jsplit_kernel<1>), dim3((unsigned)grid), dim3(kJsplitThreads), 0, stream, args);
    else
        hipLaunchKernelGGL((lm2exp_jsplit_kernel<2>), dim3((unsigned)grid), dim3(kJsplitThreads), 0, stream, args);
    return (int)hipGetLastError();
}

}  // namespace trt
