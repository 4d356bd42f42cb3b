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
// lm2exp_jsplit16_kernel, below, is the same plan on the 16 x 16 x 4 MFMA for at most 16 rows and 32
// columns.
#pragma once

#include <cmath>
#include <cstdio>

#include "common.hpp"

namespace trt {

struct Lm2JsplitArgs {
    const float *a, *b;
    float *c;
    int R, I, J, K;
    int64_t sa0, sa1, sa2, sb0, sb1, sb2, sc0, sc1;  // (32-row kernel: rows of a dense, 16-byte aligned, J a multiple of 4)
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

// At most 16 rows and at most 32 columns: the same plan on the 16 x 16 x 4 MFMA, whose tile such a
// batch fills (half of a 32 x 32 x 2 tile's rows or columns would be padding, and its MFMAs are a
// quarter of the time here).  Lane (n, q), n = lane % 16, q = lane / 16, holds a[n, j] and
// exp(b[j, n] - m) for j = 4 u + q of MFMA u: 64 lanes read 4 consecutive rows of b, 256
// consecutive bytes where K = 16.  The wavefronts split J in units of 4 (one MFMA), so any J of
// at least 32 is spread evenly; rows of a are read 4 bytes at a time and need no alignment.
// CT: column blocks of 16 per workgroup (K <= 16 CT).  KEEP > 0: J of at most 512 (384 above 16 columns), a wavefront's
// quarter of at most KEEP units: its values of b stay in registers between the maxima and the
// exponentials (b is read once, and the loads of a are in flight across the barrier).
static inline int jsplit16_keep(int64_t J, int64_t K) {  // (0: the wavefronts walk their quarters twice)
    const int64_t share = ceil_div(ceil_div(J, 4), kJsplitWaves);
    for (int keep : {2, 4, 6, 8, 12, 16, 24, 32})
        if (share <= keep) return keep;
    return 0;
}
// AVEC (KEEP a multiple of 4, dense 16-byte aligned rows of a, J a multiple of 4): lane (n, q) reads
// a[n, 4 (u + q) .. + 3] of four units at once, 64 consecutive bytes per row and load (4 bytes at a
// time the 64 lanes of a load touch 16 rows for 16 bytes of each), and the four lanes of a row
// transpose their 4 x 4 values: unit u + e wants a[n, 4 (u + e) + q] on lane (n, q).  Each lane turns
// its four values by its q, one exchange per turn d fetches from lane (n, (q - d) mod 4), and each
// lane turns what it got back.
__device__ __forceinline__ void jsplit_transpose(floatx4 &v, int lane) {
    const int n = lane & 15, q = lane >> 4;
    float w[4], y[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {  // w[d] = v[(d + q) mod 4]
        const float lo = (q & 1) ? v[(d + 1) & 3] : v[d], hi = (q & 1) ? v[(d + 3) & 3] : v[(d + 2) & 3];
        w[d] = (q & 2) ? hi : lo;
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) y[d] = __shfl(w[d], n + 16 * ((q - d) & 3), kWave);
#pragma unroll
    for (int e = 0; e < 4; ++e) {  // v[e] = y[(q - e) mod 4]
        const float lo = (q & 1) ? y[(1 - e) & 3] : y[(0 - e) & 3], hi = (q & 1) ? y[(3 - e) & 3] : y[(2 - e) & 3];
        v[e] = (q & 2) ? hi : lo;
    }
}
template <int CT, int KEEP, bool AVEC>
static __global__ __launch_bounds__(kJsplitThreads) void lm2exp_jsplit16_kernel(const Lm2JsplitArgs p) {
    constexpr int NT = 16 * CT;
    __shared__ float part[kJsplitWaves][CT][4][kWave];  // the wavefronts' partial tiles
    __shared__ float red[kJsplitWaves][NT];
    __shared__ float shift[NT];

    const int tid = (int)threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int n = lane & 15, q = lane >> 4;
    const int r = (int)blockIdx.x;

    // this wavefront's part of j: a quarter, in whole units of 4
    const int n_units = (p.J + 3) / 4;
    const int u_lo = n_units * wave / kJsplitWaves, u_hi = n_units * (wave + 1) / kJsplitWaves;

    const float *br = p.b + (int64_t)r * p.sb0;
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(br, (uint32_t)(((int64_t)(p.J - 1) * p.sb1 + (int64_t)(p.K - 1) * p.sb2 + 1) * 4));
    const uint32_t b_row = (uint32_t)p.sb1 * 4u;  // bytes between two values of j
    uint32_t bcol[CT];  // this lane's column of b and its row q in bytes (columns past K: the last one again, never stored)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int k = 16 * ct + n;
        bcol[ct] = (uint32_t)((int64_t)(k < p.K ? k : p.K - 1) * p.sb2) * 4u + (uint32_t)q * b_row;
    }

    // ---- column maxima: lane (n, q) takes j = 4 u + q (rows past J are read past the extent as
    // zeros and set aside)
    const float *ar = p.a + (int64_t)r * p.sa0;
    const uint32_t a_extent = (uint32_t)(((int64_t)(p.I - 1) * p.sa1 + (int64_t)(p.J - 1) * p.sa2 + 1) * 4);
    const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(ar, a_extent);
    const uint32_t a_col = (uint32_t)p.sa2 * 4u;  // bytes between two values of j
    // (rows past I are read past the extent: zeros)
    const uint32_t a_voff = n < p.I ? (uint32_t)((int64_t)n * p.sa1 * 4) + (uint32_t)q * a_col : a_extent;
    float b_keep[KEEP ? CT : 1][KEEP ? KEEP : 1], a_keep[KEEP ? KEEP : 1];  // (KEEP: -inf and 0 outside the wavefront's units)
    {
        float m[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) m[ct] = -__builtin_inff();
        if constexpr (KEEP > 0) {
#pragma unroll
            for (int t = 0; t < KEEP; ++t) {
                const int u = u_lo + t;
                const bool inside = u < u_hi && 4 * u + q < p.J;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const float v = buf_load_f32(b_rsrc, bcol[ct], (uint32_t)(4 * u) * b_row);
                    b_keep[ct][t] = inside ? v : -__builtin_inff();
                    m[ct] = __builtin_fmaxf(m[ct], b_keep[ct][t]);
                }
            }
            if constexpr (AVEC) {
                static_assert(KEEP % 4 == 0, "four units per load");
                const uint32_t a_voff4 = n < p.I ? a_voff + (uint32_t)(12 * q) : a_extent;  // (unit q of the four: 16 q bytes into the row)
#pragma unroll
                for (int t = 0; t < KEEP; t += 4) {
                    floatx4 v = buf_load_f32x4(a_rsrc, a_voff4, (uint32_t)(16 * (u_lo + t)));
                    jsplit_transpose(v, lane);
#pragma unroll
                    for (int e = 0; e < 4; ++e) a_keep[t + e] = (u_lo + t + e < u_hi && 4 * (u_lo + t + e) + q < p.J) ? v[e] : 0.f;
                }
            } else {
#pragma unroll
                for (int t = 0; t < KEEP; ++t) {
                    const int u = u_lo + t;
                    const float v = buf_load_f32(a_rsrc, a_voff, (uint32_t)(4 * u) * a_col);
                    a_keep[t] = (u < u_hi && 4 * u + q < p.J) ? v : 0.f;
                }
            }
        } else {
#pragma unroll 4
            for (int u = u_lo; u < u_hi; ++u) {
                const bool inside = 4 * u + q < p.J;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const float v = buf_load_f32(b_rsrc, bcol[ct], (uint32_t)(4 * u) * b_row);
                    m[ct] = __builtin_fmaxf(m[ct], inside ? v : -__builtin_inff());
                }
            }
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            m[ct] = __builtin_fmaxf(m[ct], __shfl_xor(m[ct], 16, kWave));
            m[ct] = __builtin_fmaxf(m[ct], __shfl_xor(m[ct], 32, kWave));
            if (q == 0) red[wave][16 * ct + n] = m[ct];
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
    for (int ct = 0; ct < CT; ++ct) mk[ct] = shift[16 * ct + n];

    // ---- the contraction over this wavefront's units, four at a time
    floatx4 acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[ct][v] = 0.f;

    if constexpr (KEEP > 0) {
#pragma unroll
        for (int t = 0; t < KEEP; ++t)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)  // (outside: exp(-inf) = 0 times 0)
                acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_keep[t], exp_shifted(b_keep[ct][t] - mk[ct]), acc[ct], 0, 0, 0);
    } else {
    float a_next[4], b_next[CT][4];
    auto issue = [&](int u) {  // (units past u_hi: a neighbour's values or zeros, never used)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            a_next[e] = buf_load_f32(a_rsrc, a_voff, (uint32_t)(4 * (u + e)) * a_col);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) b_next[ct][e] = buf_load_f32(b_rsrc, bcol[ct], (uint32_t)(4 * (u + e)) * b_row);
        }
    };
    if (u_lo < u_hi) issue(u_lo);
    for (int u = u_lo; u < u_hi; u += 4) {
        float av[4], bv[CT][4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            av[e] = a_next[e];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) bv[ct][e] = b_next[ct][e];
        }
        if (u + 4 < u_hi) issue(u + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool inside = u + e < u_hi && 4 * (u + e) + q < p.J;
            const float aw = inside ? av[e] : 0.f;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const float f = inside ? exp_shifted(bv[ct][e] - mk[ct]) : 0.f;
                acc[ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(aw, f, acc[ct], 0, 0, 0);
            }
        }
    }
    }

    // ---- the four partial tiles, added in a fixed order; accumulator v of a lane is row 4 q + v
    // of the tile, column n
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int v = 0; v < 4; ++v) part[wave][ct][v][lane] = acc[ct][v];
    __syncthreads();
    for (int t = tid; t < CT * 4 * kWave; t += kJsplitThreads) {
        const int l = t & (kWave - 1), v = (t >> 6) & 3, ct = t >> 8;
        const int orow = 4 * (l >> 4) + v, col = 16 * ct + (l & 15);
        if (orow >= p.I || col >= p.K) continue;
        float sum = part[0][ct][v][l];
#pragma unroll
        for (int w = 1; w < kJsplitWaves; ++w) sum += part[w][ct][v][l];
        p.c[(int64_t)r * p.sc0 + (int64_t)orow * p.sc1 + col] = log_plus(sum, shift[col]);
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
// The 16-row kernel (any layout of a): against lm2exp's own tiles on 300 timed shapes (I = 1..16,
// J = 32..4096, half of them no multiple of 4, K = 9..32, up to 60 000 batches) it is 2.0 times
// faster in the geometric mean and behind only on grids of a few dozen batches under contractions of
// thousands of terms, which the tiles cut over J: 1.1 doublings ahead to begin with, + 0.17 per
// doubling of J, - 0.26 per doubling of K, - 0.30 per halving of the grid below 1024 batches
// (0.8 % behind the faster choice per shape; always taking it 0.4 %).  Where both kernels apply it
// is 1.23 times faster than the 32-row one (which is ahead by up to 10 % at I = 16, K = 16: its
// 16-byte loads of a).
static inline bool jsplit16_applies(int64_t I, int64_t J, int64_t K) { return I <= 16 && J >= 32 && K <= 32 && K > 8; }
static inline double jsplit16_score(int64_t R, int64_t J, int64_t K) {
    const double lr = std::log2((double)R);
    return 1.13 - 0.26 * std::log2((double)K) + 0.17 * std::log2((double)J) - 0.30 * (lr < 10.0 ? 10.0 - lr : 0.0);
}
static inline bool jsplit_pays(int64_t R, int64_t I, int64_t J, int64_t K, bool a_aligned) {
    if (jsplit16_applies(I, J, K)) return jsplit16_score(R, J, K) > 0.0;
    return jsplit_applies(I, J, K, a_aligned) && jsplit_score(R, I, J, K) > 0.0;
}
// (the kernel a call that takes this path runs)
// (the 4-byte loads cost by the rows they touch, the transpose the same for any I: measured level
// at about 10 rows, 1.2 to 1.5 times faster at 13 to 16 -- R=4096, I=16, J=256, K=16: 33.7 -> 22.2 us)
static inline bool jsplit16_avec(int64_t I, int64_t J, int64_t K, bool a_aligned) {
    return a_aligned && I >= 12 && J % 4 == 0 && jsplit16_keep(J, K) % 4 == 0 && jsplit16_keep(J, K) > 0;
}
static inline int jsplit_kernel_name(char *buf, size_t bytes, int64_t I, int64_t J, int64_t K, bool a_aligned) {
    if (jsplit16_applies(I, J, K))
        return snprintf(buf, bytes, "trt::lm2exp_jsplit16_kernel<%d, %d, %s>", K > 16 ? 2 : 1, jsplit16_keep(J, K),
                        jsplit16_avec(I, J, K, a_aligned) ? "true" : "false");
    return snprintf(buf, bytes, "trt::lm2exp_jsplit_kernel<%d>", K > 32 ? 2 : 1);
}

static int launch_lm2exp_jsplit(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                                const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], hipStream_t stream) {
    Lm2JsplitArgs args;
    args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sa0 = sa[0]; args.sa1 = sa[1]; args.sa2 = sa[2];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    if (jsplit16_applies(I, J, K)) {
        if (R >= ((int64_t)1 << 31)) return TRT_E_RANGE;
        const bool avec =
            jsplit16_avec(I, J, K, sa[2] == 1 && sa[0] % 4 == 0 && sa[1] % 4 == 0 && (reinterpret_cast<uintptr_t>(a) & 15) == 0);
#define TRT_JSPLIT16_LAUNCH(CT_, KEEP_, AVEC_) \
    hipLaunchKernelGGL((lm2exp_jsplit16_kernel<CT_, KEEP_, AVEC_>), dim3((unsigned)R), dim3(kJsplitThreads), 0, stream, args)
#define TRT_JSPLIT16_AVEC(CT_, KEEP_) \
    if (avec) TRT_JSPLIT16_LAUNCH(CT_, KEEP_, true); else TRT_JSPLIT16_LAUNCH(CT_, KEEP_, false); \
    break;
#define TRT_JSPLIT16_KEEP(CT_) \
    switch (jsplit16_keep(J, K)) { \
        case 2: TRT_JSPLIT16_LAUNCH(CT_, 2, false); break; \
        case 4: TRT_JSPLIT16_AVEC(CT_, 4) \
        case 6: TRT_JSPLIT16_LAUNCH(CT_, 6, false); break; \
        case 8: TRT_JSPLIT16_AVEC(CT_, 8) \
        case 12: TRT_JSPLIT16_AVEC(CT_, 12) \
        case 16: TRT_JSPLIT16_AVEC(CT_, 16) \
        case 24: TRT_JSPLIT16_AVEC(CT_, 24) \
        case 32: TRT_JSPLIT16_AVEC(CT_, 32) \
        default: TRT_JSPLIT16_LAUNCH(CT_, 0, false); break; \
    }
        if (K <= 16) {
            TRT_JSPLIT16_KEEP(1)
        } else {
            TRT_JSPLIT16_KEEP(2)
        }
#undef TRT_JSPLIT16_AVEC
#undef TRT_JSPLIT16_KEEP
#undef TRT_JSPLIT16_LAUNCH
        return (int)hipGetLastError();
    }
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
