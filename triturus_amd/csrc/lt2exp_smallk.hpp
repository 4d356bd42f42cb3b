// lt2exp for outputs of at most 8 columns (K <= 8: one sample, or a handful, per batch -- the
// shape of a serving call).  Such a call is a sweep over w: every weight meets K pairs of factors,
// 2 K flops per 4 bytes, far below what the matrix pipe needs to pay for its 32-column tiles, so
// the MFMA kernels of lt2exp.hip, which stage w through LDS one small tile per step, are bound by
// the latency of those steps (measured: 2-4.5 TB/s of w at K = 1..32).  Here w is streamed with
// 16-byte loads straight into registers, four in flight per lane, and contracted on the vector
// ALU: a lane multiplies its four consecutive weights w[s, i, j..j+3] with the factors
// exp(b[j..j+3, k] - mb[k]) and the sum with exp(a[i, k] - ma[k]), for every k, the factors
// coming from LDS (K x J and I x K floats, computed once per workgroup).  A wavefront owns a
// row s (or, on grids of few rows, a quarter of one) and sums over its lanes at the end.
// No counterpart in the reference, whose kernels tile over K like the MFMA kernels here
// (triturus/lt2exp.py:227-357); the arithmetic contract is the same (baselines/lt2exp.py:15-25).
#pragma once

#include "common.hpp"

namespace trt {

struct Lt2SmallArgs {
    const float *w, *a, *b;
    float *c;
    int R, S, I, J, K;
    int64_t sw0, sw1, sa0, sa1, sa2, sb0, sb1, sb2, sc0, sc1;
    int rows_per_wg;  // rows of S that a workgroup walks
    int s_blocks;     // workgroups per batch
    int once;         // w is too large to be found in a cache by a later call: read-once loads
};

// Sum over the wavefront on the data-parallel-primitive path (six register moves between lanes:
// within quads, within rows of 16, then row to row; lanes without a source read zero); the
// result is complete in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_zero(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true));
}
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v += dpp_or_zero<0xb1, 0xf>(v);   // quad_perm [1,0,3,2]
    v += dpp_or_zero<0x4e, 0xf>(v);   // quad_perm [2,3,0,1]
    v += dpp_or_zero<0x114, 0xf>(v);  // row_shr 4
    v += dpp_or_zero<0x118, 0xf>(v);  // row_shr 8
    v += dpp_or_zero<0x142, 0xa>(v);  // row_bcast 15 into rows 1 and 3
    v += dpp_or_zero<0x143, 0xc>(v);  // row_bcast 31 into rows 2 and 3
    return v;
}

constexpr int kSmallThreads = 256;
constexpr int kSmallWaves = kSmallThreads / kWave;
constexpr int kSmallUnroll = 4;  // 16-byte loads in flight per lane

// KC: columns computed (K padded to 1, 4 or 8).  WPR: wavefronts that share a row (1 or 4).
// ANYJ: J is not a multiple of 4 (but I * J is, so rows of w are still whole 16-byte pieces): the
// four weights of a piece may lie in two rows i, i + 1 of the (i, j) plane, so every weight looks
// its factor of b up by itself and the piece is summed in two parts, one per row of a.
template <int KC, int WPR, bool ANYJ>
static __global__ __launch_bounds__(kSmallThreads) void lt2exp_smallk_kernel(const Lt2SmallArgs p) {
    static_assert(KC == 1 || KC == 4 || KC == 8, "K padded to 1, 4 or 8");
    static_assert(WPR == 1 || WPR == kSmallWaves, "a row per wavefront, or one per workgroup");
    extern __shared__ __attribute__((aligned(16))) float lds[];
    // ANYJ reads the factors of b one by one, consecutive lanes four values of j apart: the plane is
    // stored "transposed by 4" -- j at (j % 4) * Q + j / 4 -- so that those reads fall into consecutive
    // LDS banks instead of every fourth one
    const int Q = (p.J + 3) / 4;              // pitch of a plane: 4 Q >= J floats
    float *ea = lds;                          // [I][KC]: exp(a[i, k] - ma[k])
    float *eb = ea + ((p.I * KC + 3) & ~3);   // [KC][4 Q]: exp(b[j, k] - mb[k]), a plane per column (16-byte aligned)
    float *red = eb + 4 * Q * KC;   // [kSmallThreads] scratch of the reductions
    float *mx = red + kSmallThreads;  // [2][KC]: ma, mb

    const int r = (int)(blockIdx.x / (unsigned)p.s_blocks);
    const int sblk = (int)(blockIdx.x % (unsigned)p.s_blocks);
    const int t = (int)threadIdx.x;
    const int lane = t & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(t / kWave);
    const int k = t % KC;  // the column this thread serves in the prologue (kSmallThreads % KC == 0)
    const float *ar = p.a ? p.a + (int64_t)r * p.sa0 : nullptr;
    const float *br = p.b + (int64_t)r * p.sb0;

    // ---- the sweep's geometry.  A lane's pieces lie 64 * WPR pieces apart; (i, j) of a piece's
    // first weight advances by a fixed step per trip (with J a multiple of 4 the four weights of a
    // piece share their i).  A trip is kSmallUnroll pieces per lane; the loads of the next trip --
    // of the next row, at the end of a row -- are asked for before the current one is contracted,
    // and those of the very first trip before the factors are computed, so that the prologue runs
    // under their latency.
    const int n4 = (p.I * p.J + 3) / 4;                  // 16-byte pieces of a row of w
    const int lane_piece = (WPR == 1 ? 0 : wave * kWave) + lane;
    const int stride_f = 4 * kWave * WPR;                // floats between a lane's consecutive pieces
    const int di = stride_f / p.J, dj = stride_f % p.J;  // wave-uniform
    const int i_first = (4 * lane_piece) / p.J, j_first = (4 * lane_piece) % p.J;
    // ANYJ also takes rows of w that do not start on a 16-byte boundary: a row is then read from the
    // boundary below it, `mis` floats early -- those floats, the end of the row before, are given
    // weight zero -- and (i, j) of a lane's first piece steps back by as many.
    constexpr int kTrip = kSmallUnroll * kWave * WPR;    // pieces of a row that a trip covers
    const int trips_per_row = ((ANYJ ? n4 + 1 : n4) + kTrip - 1) / kTrip;
    const int s_first = sblk * p.rows_per_wg + (WPR == 1 ? wave : 0);
    constexpr int kRowStep = WPR == 1 ? kSmallWaves : 1;
    const int rows_here = WPR == 1 ? (p.rows_per_wg - wave + kSmallWaves - 1) / kSmallWaves : p.rows_per_wg;
    const int rows_left = s_first < p.S ? (p.S - s_first + kRowStep - 1) / kRowStep : 0;
    const int rows_valid = rows_here < rows_left ? rows_here : rows_left;  // wave-uniform
    const float *w_batch = p.w + (int64_t)r * p.sw0;
    auto row_mis = [&](int s) -> int {  // floats between the 16-byte boundary below the row and its start
        if constexpr (!ANYJ) return 0;
        return (int)((reinterpret_cast<uintptr_t>(w_batch + (int64_t)s * p.sw1) >> 2) & 3);
    };
    floatx4 nxt[kSmallUnroll];
    auto issue = [&](int s, int trip) {  // pieces past the row read as zeros
        const int mis = row_mis(s);
        // (whole pieces: what the last one holds beyond the row is given weight zero below)
        const __amdgpu_buffer_rsrc_t w_rsrc =
            make_rsrc(w_batch + (int64_t)s * p.sw1 - mis, (uint32_t)((p.I * p.J + mis + 3) / 4) * 16u);
#pragma unroll
        for (int u = 0; u < kSmallUnroll; ++u) {
            const uint32_t off = (uint32_t)(trip * kTrip + u * kWave * WPR + lane_piece) * 16u;
            nxt[u] = p.once ? __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, off, 0u,
                                                                                                kCacheNonTemporal))
                            : buf_load_f32x4(w_rsrc, off, 0u);
        }
    };
    if (rows_valid > 0) issue(s_first, 0);

    // ---- column maxima of a and b (a NaN need not survive them: exp(NaN - m) is NaN for any m and
    // poisons the sums of its column, as in the torch recipe)
    for (int which = 0; which < 2; ++which) {
        if (which == 0 && !p.a) {  // no factors of a (the lm2exp entry: I = 1, a factor of one)
            if (t < KC) mx[t] = 0.f;
            continue;  // (block-uniform)
        }
        const float *x = which ? br : ar;
        const int64_t s1 = which ? p.sb1 : p.sa1, s2 = which ? p.sb2 : p.sa2;
        const int n = which ? p.J : p.I;
        float m = -__builtin_inff();
        if (k < p.K)
            for (int row = t / KC; row < n; row += kSmallThreads / KC)
                m = __builtin_fmaxf(m, x[(int64_t)row * s1 + (int64_t)k * s2]);
        red[t] = m;
        __syncthreads();
        if (t < KC) {
            float y = -__builtin_inff();
            for (int u = t; u < kSmallThreads; u += KC) y = __builtin_fmaxf(y, red[u]);
            mx[which * KC + t] = clamp_shift(y);
        }
        __syncthreads();
    }
    // ---- factors (columns past K: zero, they are never stored)
    {
        const float mak = mx[k], mbk = mx[KC + k];
        for (int i = t / KC; i < p.I; i += kSmallThreads / KC)
            ea[i * KC + k] = k >= p.K ? 0.f : !p.a ? 1.f : exp_shifted(ar[(int64_t)i * p.sa1 + (int64_t)k * p.sa2] - mak);
        for (int j = t / KC; j < p.J; j += kSmallThreads / KC)
            eb[k * 4 * Q + (ANYJ ? (j & 3) * Q + (j >> 2) : j)] =
                k < p.K ? exp_shifted(br[(int64_t)j * p.sb1 + (int64_t)k * p.sb2] - mbk) : 0.f;
    }
    __syncthreads();

    // ---- the sweep
    for (int rr = 0; rr < rows_valid; ++rr) {
        const int s = s_first + rr * kRowStep;
        float acc[KC];
#pragma unroll
        for (int c = 0; c < KC; ++c) acc[c] = 0.f;
        int i = i_first, j = j_first;
        if constexpr (ANYJ) {
            j -= row_mis(s);
            if (j < 0) {
                j += p.J;
                i -= 1;
            }
        }
        for (int trip = 0; trip < trips_per_row; ++trip) {
            floatx4 wv[kSmallUnroll];
            if constexpr (KC < 8) {
#pragma unroll
                for (int u = 0; u < kSmallUnroll; ++u) wv[u] = nxt[u];
                if (trip + 1 < trips_per_row) issue(s, trip + 1);
                else if (rr + 1 < rows_valid) issue(s + kRowStep, 0);
            } else {
                // (8 columns: the second set of load registers costs a wavefront per SIMD and the LDS
                // reads of the factors, not the loads, bound the trip: measured 5-15 % slower with it)
                if (rr + trip > 0) issue(s, trip);
#pragma unroll
                for (int u = 0; u < kSmallUnroll; ++u) wv[u] = nxt[u];
            }
#pragma unroll
            for (int u = 0; u < kSmallUnroll; ++u) {
                // (a piece past the row: its weights are zeros; i = -1: the floats before the row's start)
                const int ic = i < p.I ? (i < 0 ? 0 : i) : p.I - 1;
                const int jc = i < p.I ? j : 0;
                if constexpr (ANYJ) {
                    // weights 0..m-1 of the piece belong to row i, the others to row i + 1 (J >= 4: at
                    // most one row boundary inside a piece)
                    const int m = p.J - jc;
                    const int ih = i + 1 < p.I ? i + 1 : p.I - 1;
                    const bool before = i < 0, past_lo = i >= p.I, past_hi = i + 1 >= p.I;
                    int at[4];  // where the factor of b of each weight sits in a plane
                    float wl[4], wh[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const bool low = e < m;
                        const int jt = low ? jc + e : e - m;
                        at[e] = (jt & 3) * Q + (jt >> 2);
                        wl[e] = low && !before && !past_lo ? wv[u][e] : 0.f;
                        wh[e] = low || past_hi ? 0.f : wv[u][e];
                    }
                    float fl[KC], fh[KC];
                    if constexpr (KC == 1) {
                        fl[0] = ea[ic];
                        fh[0] = ea[ih];
                    } else {
#pragma unroll
                        for (int q = 0; q < KC / 4; ++q) {
                            const floatx4 v = *reinterpret_cast<const floatx4 *>(&ea[ic * KC + 4 * q]);
                            const floatx4 h2 = *reinterpret_cast<const floatx4 *>(&ea[ih * KC + 4 * q]);
#pragma unroll
                            for (int x = 0; x < 4; ++x) {
                                fl[4 * q + x] = v[x];
                                fh[4 * q + x] = h2[x];
                            }
                        }
                    }
#pragma unroll
                    for (int c = 0; c < KC; ++c) {
                        const float *plane = eb + c * 4 * Q;
                        const float e0 = plane[at[0]], e1 = plane[at[1]], e2 = plane[at[2]], e3 = plane[at[3]];
                        const float lo = wl[0] * e0 + wl[1] * e1 + wl[2] * e2 + wl[3] * e3;
                        const float hi = wh[0] * e0 + wh[1] * e1 + wh[2] * e2 + wh[3] * e3;
                        acc[c] = __builtin_fmaf(fl[c], lo, acc[c]);
                        acc[c] = __builtin_fmaf(fh[c], hi, acc[c]);
                    }
                } else if constexpr (KC == 1) {
                    const floatx4 e = *reinterpret_cast<const floatx4 *>(&eb[jc]);
                    const float dot = wv[u][0] * e[0] + wv[u][1] * e[1] + wv[u][2] * e[2] + wv[u][3] * e[3];
                    acc[0] = __builtin_fmaf(ea[ic], dot, acc[0]);
                } else {
                    float fa[KC];
#pragma unroll
                    for (int q = 0; q < KC / 4; ++q) {
                        const floatx4 v = *reinterpret_cast<const floatx4 *>(&ea[ic * KC + 4 * q]);
                        fa[4 * q] = v[0]; fa[4 * q + 1] = v[1]; fa[4 * q + 2] = v[2]; fa[4 * q + 3] = v[3];
                    }
#pragma unroll
                    for (int c = 0; c < KC; ++c) {
                        const floatx4 e = *reinterpret_cast<const floatx4 *>(&eb[c * 4 * Q + jc]);
                        const float dot = wv[u][0] * e[0] + wv[u][1] * e[1] + wv[u][2] * e[2] + wv[u][3] * e[3];
                        acc[c] = __builtin_fmaf(fa[c], dot, acc[c]);
                    }
                }
                j += dj;
                i += di;
                if (j >= p.J) {
                    j -= p.J;
                    i += 1;
                }
            }
        }
        // ---- sum over the lanes (and, with WPR = 4, over the wavefronts), shift back, log, store
#pragma unroll
        for (int c = 0; c < KC; ++c) acc[c] = wave_sum_lane63(acc[c]);  // complete in lane 63
        if constexpr (WPR == 1) {
            if (lane == kWave - 1) {
                float *crow = p.c + (int64_t)r * p.sc0 + (int64_t)s * p.sc1;
#pragma unroll
                for (int c = 0; c < KC; ++c)
                    if (c < p.K) crow[c] = log_plus(acc[c], mx[c] + mx[KC + c]);
            }
        } else {
            if (lane == kWave - 1)
#pragma unroll
                for (int c = 0; c < KC; ++c) red[wave * KC + c] = acc[c];
            __syncthreads();
            if (t < p.K) {
                float sum = red[t];
                for (int wv2 = 1; wv2 < kSmallWaves; ++wv2) sum += red[wv2 * KC + t];
                p.c[(int64_t)r * p.sc0 + (int64_t)s * p.sc1 + t] = log_plus(sum, mx[t] + mx[KC + t]);
            }
            __syncthreads();  // red is written again by the next row
        }
    }
}

constexpr int64_t kSmallMaxK = 8;
constexpr size_t kSmallMaxLds = 48 * 1024;

static inline int small_kc(int64_t K) { return K <= 1 ? 1 : (K <= 4 ? 4 : 8); }
static inline size_t small_lds_bytes(int64_t I, int64_t J, int64_t K) {
    return ((size_t)(I + (J + 3) / 4 * 4) * small_kc(K) + 4 + kSmallThreads + 2 * 8) * sizeof(float);
}

// Does the call take the sweep?  At most 8 columns; a dense flat axis of w (J a multiple of 4 on
// 16-byte aligned rows: the plain build; any other J > 4 and any row alignment: ANYJ); factors that fit LDS; rows of at
// least 128 weights (256 with more than 4 columns), below which the sum over the lanes at the
// end of a row costs more than the row.  Timed against the matrix-pipe kernels on 300 random
// shapes (K = 1..8, R = 1..256, S = 1..1024, I = 1..300, J = 4..320): the sweep is 1.5-2.8x
// ahead in the median of every class of row length from 256 weights on (up to 11x), whatever
// the number of rows, and these thresholds leave the choice 0.4 % (mean) behind the faster of
// the two (never sweeping: 104 %).
static inline bool smallk_applies(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_aligned,
                                  bool w_dense = true) {
    (void)R;
    (void)S;
    if (K > kSmallMaxK || small_lds_bytes(I, J, K) > kSmallMaxLds) return false;
    if (J % 4 == 0 && w_aligned) return I * J >= (K > 4 ? 256 : 128);
    // (any other J > 4, or rows that do not start on 16-byte boundaries, cost every weight a look-up
    // of its own: level with the matrix-pipe kernels on shorter rows, 0.3x at worst with 8
    // columns; over 120 random shapes the sweep is 1.6x ahead in the median beyond these bounds)
    return w_dense && J > 4 && I * J >= (K > 4 ? 1024 : 256);
}
static inline bool smallk_anyj(int64_t J, bool w_aligned) { return !(J % 4 == 0 && w_aligned); }
static inline int smallk_wpr(int64_t R, int64_t S) { return R * S >= 512 ? 1 : kSmallWaves; }

template <int KC, bool ANYJ>
static int launch_smallk_kc(const Lt2SmallArgs &args, int wpr, size_t lds, unsigned grid, hipStream_t stream) {
    if (wpr == 1)
        hipLaunchKernelGGL((lt2exp_smallk_kernel<KC, 1, ANYJ>), dim3(grid), dim3(kSmallThreads), lds, stream, args);
    else
        hipLaunchKernelGGL((lt2exp_smallk_kernel<KC, kSmallWaves, ANYJ>), dim3(grid), dim3(kSmallThreads), lds, stream,
                           args);
    return (int)hipGetLastError();
}

static int launch_lt2exp_smallk(const float *w, const float *a, const float *b, float *c, int64_t R, int64_t S,
                                int64_t I, int64_t J, int64_t K, const int64_t sw[3], const int64_t sa[3],
                                const int64_t sb[3], const int64_t sc[3], bool w_aligned, hipStream_t stream) {
    Lt2SmallArgs args;
    args.w = w; args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.S = (int)S; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sw0 = sw[0]; args.sw1 = sw[1];
    args.sa0 = sa[0]; args.sa1 = sa[1]; args.sa2 = sa[2];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    const int wpr = smallk_wpr(R, S);
    // a wavefront per row: workgroups of 4..64 rows, some 2048 of them where the rows allow
    int64_t rows = 1;
    if (wpr == 1) {
        rows = ceil_div(ceil_div(R * S, 2048), kSmallWaves) * kSmallWaves;
        if (rows < kSmallWaves) rows = kSmallWaves;
        if (rows > 64) rows = 64;
    }
    // (only a w that the 256 MB memory-side cache cannot hold: the weights of a serving call are the
    // same from call to call, and up to there ordinary loads find part of them again -- 268 MB:
    // 46 us against 50 with read-once loads; 537 MB: 103 against 94)
    args.once = (double)R * (double)S * (double)I * (double)J * 4.0 >= 384.0 * 1048576.0 ? 1 : 0;
    args.rows_per_wg = (int)rows;
    args.s_blocks = (int)ceil_div(S, rows);
    const int64_t grid = R * args.s_blocks;
    if (grid >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    const size_t lds = small_lds_bytes(I, J, K);
    if (!smallk_anyj(J, w_aligned)) {
        switch (small_kc(K)) {
            case 1: return launch_smallk_kc<1, false>(args, wpr, lds, (unsigned)grid, stream);
            case 4: return launch_smallk_kc<4, false>(args, wpr, lds, (unsigned)grid, stream);
            default: return launch_smallk_kc<8, false>(args, wpr, lds, (unsigned)grid, stream);
        }
    }
    switch (small_kc(K)) {
        case 1: return launch_smallk_kc<1, true>(args, wpr, lds, (unsigned)grid, stream);
        case 4: return launch_smallk_kc<4, true>(args, wpr, lds, (unsigned)grid, stream);
        default: return launch_smallk_kc<8, true>(args, wpr, lds, (unsigned)grid, stream);
    }
}

}  // namespace trt
