// lt2exp for gfx950:  c[r,s,k] = log sum_{i,j} w[r,s,i,j] exp(a[r,i,k]) exp(b[r,j,k])
//
// One workgroup owns a (32*RT rows of S) x (32*CT*NWAVES columns of K) tile of
// c[r]; each wavefront owns 32*CT of those columns for all rows.  The
// contraction runs on v_mfma_f32_32x32x2_f32 with
//   A operand = w tile, staged global -> registers -> LDS (double buffered),
//               read back 16 bytes per lane (4 consecutive j);
//   B operand = the shifted Khatri-Rao product exp(a[i,n]-ma[n]) * exp(b[j,n]-mb[n]),
//               formed in registers with ONE multiply per MFMA operand: a lane
//               owns one column n, keeps exp(b[j,n]-mb[n]) for the j of the
//               current j-chunk in VGPRs and multiplies by the scalar
//               exp(a[i,n]-ma[n]) of the current i.
// The I*J*K intermediate of the torch recipe (baselines/lt2exp.py:21-22)
// never exists; every exp is evaluated once per (workgroup, column).
//
// MFMA k-slot mapping (the contraction order is free): within a chunk of
// JC = 8*NQ values of j, MFMA number (q,u) in lane-half h = lane/32 consumes
// j = 8q + 4h + u, so one 16-byte LDS read feeds 4 MFMAs.
//
// Replaces _ker_lt2exp_unsplit / _ker_lt2exp_split, triturus/lt2exp.py:227-357,365-506.

#include "common.hpp"
#include "lt2exp_merge.hpp"
#include "lt2exp_cols.hpp"
#include "lt2exp_rows.hpp"
#include "lt2exp_smallk.hpp"

#include <cstdio>
#include <mutex>

namespace trt {

struct Lt2Args {
    const float *w, *a, *b;
    float *c;         // output (unsplit) -- or partial sums (split)
    float *shift;     // split only: [2][R][K] clamped column maxima
    int R, S, I, J, K;
    int64_t sw0, sw1, sw2, sa0, sa1, sb0, sb1, sc0, sc1;  // sw2: stride of the flat (i, j) axis of w
    int64_t sa2, sb2;  // trailing strides of a and b: a lane owns a column, so they only scale lane offsets
    int s_tiles, n_tiles, splits;
    int iters_per_split;  // (j-chunk, i) iterations per split
    int stream_out;       // rows of c are 16-byte aligned: non-temporal result stores
    int64_t total_wgs, padded_wgs;
};

// WM: wavefronts stacked over rows (1: all NWAVES side by side over columns; 2 or 4 for narrow
// outputs, so that K <= 64 or 32 does not leave most of them idle).
// PJ: packed short rows.  With J = 2, 4 or 8 a chunk of 16 values of j would be mostly padding;
// w is contiguous over (i, j), so the kernel walks that flat axis in chunks of 16 instead: a chunk
// holds 16 / PJ values of i, and MFMA slot f = 8q + 4h + u of it multiplies exp a[i0 + f / PJ]
// by exp b[f % PJ] (the factors of b are the same in every chunk).
// GS: groups of NWAVES wavefronts in the workgroup.  With 2, the two groups own the SAME output
// tile and contract the two halves of the (j-chunk, i) iteration range, each through w tiles
// of its own in LDS; at the end they exchange, through LDS, the half of the accumulators that
// the other group finishes.  A grid of one or two tiles per compute unit then runs with twice
// the wavefronts per SIMD -- what such grids lack (one or two wavefronts per SIMD hide neither
// LDS nor barrier latency) -- without the partial sums ever leaving the compute unit.
template <int RT, int CT, int NQ, int NWAVES, bool VEC, bool SPLIT, int WM = 1, int PJ = 0, int GS = 1>
__global__ __launch_bounds__(NWAVES *kWave *GS, 2 * GS) void lt2exp_kernel(const Lt2Args p) {
    static_assert(PJ == 0 || (VEC && NQ == 2 && (PJ == 2 || PJ == 4 || PJ == 8)), "packed rows: chunks of 16");
    static_assert(GS == 1 || (GS == 2 && VEC && !SPLIT && WM == 1 && PJ == 0 && CT == 1), "paired groups: plain aligned tiles");
    constexpr int NT = NWAVES * kWave;  // threads of a group
    constexpr int WN = NWAVES / WM;
    constexpr int TS = 32 * RT * WM;      // rows of S per workgroup
    constexpr int JC = 8 * NQ;            // j per chunk
    constexpr int LDW = JC + 4;           // padded LDS row (floats): conflict-free 16-byte reads
    constexpr int F4_PER_ROW = JC / 4;
    constexpr int F4_TILE = TS * F4_PER_ROW;              // 16-byte pieces of a w tile
    constexpr int SLOTS = (F4_TILE + NT - 1) / NT;        // of which a thread stages this many
    // REGULAR: a thread keeps its column and steps whole rows from slot to slot; otherwise
    // (chunks of 24 or 48, or tiles smaller than the workgroup) pieces are dealt out linearly
    // and the last slot is only partly filled.
    constexpr bool REGULAR = (NT % F4_PER_ROW == 0) && (F4_TILE % NT == 0);
    constexpr int TN = 32 * CT * WN;

    // (a thread whose last slot lies past the tile stages into a private 16 bytes behind it:
    // the steady state carries no predicates)
    static_assert(GS == 1 || REGULAR, "paired groups stage whole slots");
    __shared__ __attribute__((aligned(16))) float wt_all[GS][2][TS * LDW + (REGULAR ? 0 : 4 * NT)];

    const int64_t L = xcd_logical_id(blockIdx.x, p.padded_wgs);
    if (L >= p.total_wgs) return;
    // The tile coordinates are wave-uniform; the 64-bit divisions below are expanded on
    // the vector ALU, so pin the results back into scalar registers (they feed buffer
    // resources and scalar offsets).
    int64_t rest = L / p.n_tiles;
    const int nt = __builtin_amdgcn_readfirstlane((int)(L % p.n_tiles));
    const int split = __builtin_amdgcn_readfirstlane((int)(rest % p.splits));
    rest /= p.splits;
    const int st = __builtin_amdgcn_readfirstlane((int)(rest % p.s_tiles));
    const int r = __builtin_amdgcn_readfirstlane((int)(rest / p.s_tiles));

    const int grp = GS == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)threadIdx.x / NT);  // wave-uniform
    const int tid = GS == 1 ? (int)threadIdx.x : (int)threadIdx.x - grp * NT;             // within the group
    float(*wt)[TS * LDW + (REGULAR ? 0 : 4 * NT)] = wt_all[grp];
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    const int h = lane / 32;
    const int m = lane % 32;
    const int s0 = st * TS;
    const int wm = wave % WM;
    const int n0 = nt * TN + (wave / WM) * 32 * CT;
    const int wrow0 = wm * 32 * RT;  // first tile row of this wavefront

    int ncol[CT], ncl[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        ncol[ct] = n0 + 32 * ct + m;
        ncl[ct] = ncol[ct] < p.K ? ncol[ct] : p.K - 1;
    }
    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;
    const float *wr = p.w + (int64_t)r * p.sw0;

    // ---- column maxima over the contracted axes (both lane halves share a
    // column: each takes every other row, then they exchange).  A NaN need not
    // survive the maximum: exp(NaN - m) is NaN for any m and poisons the whole
    // output column through the MFMA, as the torch recipe does.
    float ma[CT], mb[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        float x = -__builtin_inff();
#pragma unroll 8
        for (int i = 2 * grp + h; i < p.I; i += 2 * GS) x = __builtin_fmaxf(x, ar[(int64_t)i * p.sa1 + (int64_t)ncl[ct] * p.sa2]);
        x = __builtin_fmaxf(x, __shfl_xor(x, 32, kWave));
        float y = -__builtin_inff();
#pragma unroll 8
        for (int j = 2 * grp + h; j < p.J; j += 2 * GS) y = __builtin_fmaxf(y, br[(int64_t)j * p.sb1 + (int64_t)ncl[ct] * p.sb2]);
        y = __builtin_fmaxf(y, __shfl_xor(y, 32, kWave));
        if (GS == 2) {
            // each group has swept half of the rows: the halves meet in LDS (the tile buffers are
            // not in use yet)
            float *mx = &wt_all[0][0][0];
            if (h == 0) {
                mx[(grp * 2 + 0) * TN + wave * 32 + m] = x;
                mx[(grp * 2 + 1) * TN + wave * 32 + m] = y;
            }
            __syncthreads();
            x = __builtin_fmaxf(x, mx[((grp ^ 1) * 2 + 0) * TN + wave * 32 + m]);
            y = __builtin_fmaxf(y, mx[((grp ^ 1) * 2 + 1) * TN + wave * 32 + m]);
            __syncthreads();
        }
        ma[ct] = clamp_shift(x);
        mb[ct] = clamp_shift(y);
    }

    const int n_jc = PJ ? 1 : (p.J + JC - 1) / JC;
    const int n_i = PJ ? (p.I * p.J + JC - 1) / JC : p.I;  // steps per j-chunk (packed: flat chunks over (i, j))
    const int total_iters = n_jc * n_i;
    int it = split * p.iters_per_split;
    int it_end = it + p.iters_per_split;
    if (it_end > total_iters) it_end = total_iters;
    // paired groups: the first takes the first half of the range (the longer one when the count
    // is odd); both make the same number of trips through the loop, for the barriers' sake
    const int trips = GS == 1 ? it_end - it : (total_iters + 1) / 2;
    if (GS == 2) {
        it = grp * trips;
        it_end = grp == 0 ? trips : total_iters;
    }

    floatx16 acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rt][ct][v] = 0.f;

    // ---- tile staging: global -> registers -> LDS.  FP32 MFMA and the vector ALU do
    // not execute concurrently on this hardware, so the steady state spends no VALU
    // instruction on addresses or masks: the w tile is read through a buffer resource
    // (scalar base + extent, 32-bit lane offset, scalar i/j offset) whose extent ends at
    // the last valid row, so rows past S come back as zeros.  Only a ragged j-chunk
    // (J not a multiple of the chunk) or unaligned w takes the masked path.
    floatx4 stage[SLOTS];
    int srow[SLOTS], sc4[SLOTS];  // tile row and 16-byte column of each slot
    int lds_off[SLOTS];           // where the slot goes in the LDS tile (floats)
    bool sval[SLOTS];
#pragma unroll
    for (int sidx = 0; sidx < SLOTS; ++sidx) {
        if (REGULAR) {
            srow[sidx] = tid / F4_PER_ROW + sidx * (NT / F4_PER_ROW);
            sc4[sidx] = tid % F4_PER_ROW;
            sval[sidx] = true;
        } else {
            const int f = tid + sidx * NT;
            srow[sidx] = f / F4_PER_ROW;
            sc4[sidx] = f % F4_PER_ROW;
            sval[sidx] = f < F4_TILE;
        }
        lds_off[sidx] = sval[sidx] ? srow[sidx] * LDW + 4 * sc4[sidx] : TS * LDW + 4 * tid;
    }
    const int wrows = (p.S - s0) < TS ? (p.S - s0) : TS;
    const float *wtile0 = wr + (int64_t)s0 * p.sw1;
    const __amdgpu_buffer_rsrc_t w_rsrc =
        make_rsrc(wtile0, (uint32_t)(((int64_t)(wrows - 1) * p.sw1 + ((int64_t)p.I * p.J - 1) * p.sw2 + 1) * 4));
    uint32_t woff[SLOTS];
#pragma unroll
    for (int sidx = 0; sidx < SLOTS; ++sidx)
        woff[sidx] = ((uint32_t)srow[sidx] * (uint32_t)p.sw1 + 4u * (uint32_t)sc4[sidx]) * 4u;
    // element-wise staging of the unaligned build (chunks that divide the workgroup evenly)
    constexpr bool ELEM = !VEC && (NT % JC == 0) && ((TS * JC) % NT == 0) && (TS * JC / NT <= 4 * SLOTS);
    constexpr int NE = ELEM ? TS * JC / NT : 1;  // floats per thread
    const int ecol = tid % JC;
    const uint32_t ebase = ((uint32_t)(tid / JC) * (uint32_t)p.sw1 + (uint32_t)ecol * (uint32_t)p.sw2) * 4u;
    // (a slot past the tile loads some valid or out-of-extent address: the value is never used)
    auto load_tile = [&](int i, int jc) {
        // floats of the chunk that belong to this step (packed: of the flat (i, j) axis)
        const int left = PJ ? p.I * p.J - i * JC : p.J - jc * JC;
        const int step = PJ ? JC : p.J;
        const bool full = VEC && (PJ ? left >= JC : jc * JC + JC <= p.J);  // wave-uniform
        if (full) {
            const uint32_t soff = (uint32_t)(i * step + jc * JC) * 4u;
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) stage[sidx] = buf_load_f32x4(w_rsrc, woff[sidx], soff);
        } else if (VEC) {
            // ragged last chunk of aligned rows (J is a multiple of 4): a 16-byte piece is whole
            // or lies past J, where the next i begins: zeros instead
            const uint32_t soff = (uint32_t)(i * step + jc * JC) * 4u;
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) {
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                const floatx4 v = buf_load_f32x4(w_rsrc, woff[sidx], soff);
                stage[sidx] = (PJ ? 4 * sc4[sidx] < left : jc * JC + 4 * sc4[sidx] < p.J) ? v : zero;
            }
        } else if (ELEM) {
            // rows that are not 16-byte aligned: single floats, consecutive lanes on consecutive
            // columns (coalesced), a thread's floats NT / JC rows apart (scalar offsets)
            const uint32_t soff = (uint32_t)(i * p.J + jc * JC) * (uint32_t)p.sw2 * 4u;
            const bool inside = jc * JC + ecol < p.J;
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const float v = buf_load_f32(w_rsrc, ebase, soff + (uint32_t)(e * (NT / JC)) * (uint32_t)p.sw1 * 4u);
                stage[e / 4][e % 4] = inside ? v : 0.f;
            }
        } else {
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) {
                const int row = srow[sidx];
                const int j = jc * JC + 4 * sc4[sidx];
                const float *src = wtile0 + (int64_t)row * p.sw1 + ((int64_t)i * p.J + j) * p.sw2;
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (sval[sidx] && row < wrows) {
                    if (j + 0 < p.J) v[0] = src[0];
                    if (j + 1 < p.J) v[1] = src[p.sw2];
                    if (j + 2 < p.J) v[2] = src[2 * p.sw2];
                    if (j + 3 < p.J) v[3] = src[3 * p.sw2];
                }
                stage[sidx] = v;
            }
        }
    };
    auto store_tile = [&](int buf) {
        if (ELEM) {
#pragma unroll
            for (int e = 0; e < NE; ++e) wt[buf][(tid / JC + e * (NT / JC)) * LDW + ecol] = stage[e / 4][e % 4];
            return;
        }
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) *reinterpret_cast<floatx4 *>(&wt[buf][lds_off[sidx]]) = stage[sidx];
    };

    // a rows for the scalar factor exp(a[i,n] - ma[n]): same addressing scheme
    const __amdgpu_buffer_rsrc_t a_rsrc =
        make_rsrc(ar, (uint32_t)(((int64_t)(p.I - 1) * p.sa1 + (int64_t)(p.K - 1) * p.sa2 + 1) * 4));
    const uint32_t a_row_bytes = (uint32_t)p.sa1 * 4u;
    uint32_t aoff[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) aoff[ct] = (uint32_t)ncl[ct] * (uint32_t)p.sa2 * 4u;

    float eb[CT][4 * NQ];
    auto load_eb = [&](int jc) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int q = 0; q < NQ; ++q)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int j = PJ ? (8 * q + 4 * h + u) % (PJ ? PJ : 1) : jc * JC + 8 * q + 4 * h + u;
                    float raw = -__builtin_inff();
                    if (j < p.J) raw = br[(int64_t)j * p.sb1 + (int64_t)ncl[ct] * p.sb2];
                    eb[ct][4 * q + u] = exp_shifted(raw - mb[ct]);
                }
    };

    // Factors of a per step: one (row i); packed, one per value of i in the chunk that this
    // lane's slots meet: slot f = 8q + 4h + u lies in row f / PJ of the chunk.
    constexpr int EA_N = PJ == 0 ? 1 : (PJ == 2 ? 2 * NQ : NQ);
    constexpr int RPC = PJ ? JC / PJ : 1;  // rows of a per step
    float ea[CT][EA_N], ea_raw[CT][EA_N];
    int erow[EA_N];
#pragma unroll
    for (int e = 0; e < EA_N; ++e) erow[e] = PJ == 8 ? e : (PJ == 4 ? 2 * e + h : (PJ == 2 ? 4 * (e / 2) + 2 * h + e % 2 : 0));
    // (packed: the last chunk may reach past row I - 1: the address is clamped, the factor zero)
    auto load_ea = [&](int i) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int e = 0; e < EA_N; ++e) {
                if (PJ) {
                    int row = i * RPC + erow[e];
                    row = row < p.I ? row : p.I - 1;
                    ea_raw[ct][e] = buf_load_f32(a_rsrc, aoff[ct] + (uint32_t)row * a_row_bytes, 0u);
                } else {
                    ea_raw[ct][e] = buf_load_f32(a_rsrc, aoff[ct], (uint32_t)i * a_row_bytes);
                }
            }
    };
    auto finish_ea = [&](int i) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int e = 0; e < EA_N; ++e) {
                const float x = exp_shifted(ea_raw[ct][e] - ma[ct]);
                ea[ct][e] = (PJ == 0 || i * RPC + erow[e] < p.I) ? x : 0.f;
            }
    };

    // ---- MFMA block over one (i, j-chunk): 4*NQ*RT*CT MFMAs per wavefront
    auto mfma_block = [&](const float *tile) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            floatx4 af[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                af[rt] = *reinterpret_cast<const floatx4 *>(&tile[(32 * rt + m) * LDW + 8 * q + 4 * h]);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const float bop = ea[ct][PJ == 2 ? 2 * q + u / 2 : (PJ ? q : 0)] * eb[ct][4 * q + u];
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[rt][u], bop, acc[rt][ct], 0, 0, 0);
                }
            }
        }
    };

    if constexpr (GS == 1) {
        if (it < it_end) {
            int jc = it / n_i;
            int i = it - jc * n_i;
            load_tile(i, jc);
            load_eb(jc);
            load_ea(i);
            finish_ea(i);
            store_tile(0);
            __syncthreads();

            // Steady state: every iteration prefetches the next tile unconditionally and
            // consumes it before the back edge (no load is ever left in flight across the
            // loop header); the last iteration is peeled.
            int cur = 0;
            for (; it + 1 < it_end; ++it) {
                int ni = i + 1, njc = jc;
                if (ni == n_i) {
                    ni = 0;
                    njc = jc + 1;
                }
                load_tile(ni, njc);
                load_ea(ni);
                __builtin_amdgcn_sched_barrier(0);  // the prefetch is issued before the MFMA block, not sunk into it
                mfma_block(wt[cur] + wrow0 * LDW);
                store_tile(cur ^ 1);
                if (njc != jc) load_eb(njc);
                finish_ea(ni);
                __syncthreads();
                cur ^= 1;
                i = ni;
                jc = njc;
            }
            mfma_block(wt[cur] + wrow0 * LDW);
        }
    } else {
        // Paired groups: the same pipeline, with every step guarded by wave-uniform tests so that
        // both groups meet at every barrier whatever the lengths of their halves.
        // (Measured and not kept: the barrier in the middle of a step's MFMAs, with the fragments
        // of the second half read before it and those of the next tile's first half right after
        // it -- 39.6 us against 38.9 at R=16, S=64, I=J=32, K=2048; with neither stores, loads
        // nor barriers the same loop takes 36.7 us: the MFMAs and the Khatri-Rao multiplies
        // alone run at 89 % of the matrix peak.)
        bool live = it < it_end;
        int jc = live ? it / n_i : 0;
        int i = live ? it - jc * n_i : 0;
        if (live) {
            load_tile(i, jc);
            load_eb(jc);
            load_ea(i);
            finish_ea(i);
            store_tile(0);
        }
        __syncthreads();
        int cur = 0;
        for (int t = 0; t + 1 < trips; ++t) {
            const bool more = it + 1 < it_end;
            int ni = i + 1, njc = jc;
            if (ni == n_i) {
                ni = 0;
                njc = jc + 1;
            }
            if (more) {
                load_tile(ni, njc);
                load_ea(ni);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (live) mfma_block(wt[cur] + wrow0 * LDW);
            if (more) {
                store_tile(cur ^ 1);
                if (njc != jc) load_eb(njc);
                finish_ea(ni);
            }
            __syncthreads();
            cur ^= 1;
            ++it;
            i = ni;
            jc = njc;
            live = more;
        }
        if (live) mfma_block(wt[cur] + wrow0 * LDW);

        // ---- the groups exchange halves of their sums: group g finishes registers 8g .. 8g+7 of
        // every 32 x 32 block (rows 16g + 4h + {0..3, 8..11}) and hands the other eight over.
        __syncthreads();  // the tile buffers are free
        float *xb = &wt_all[0][0][0];
        static_assert(sizeof(wt_all) >= (size_t)GS * NWAVES * RT * 8 * kWave * sizeof(float), "room for the exchange");
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const float theirs = grp == 0 ? acc[rt][0][8 + v] : acc[rt][0][v];
                xb[(((grp * NWAVES + wave) * RT + rt) * 8 + v) * kWave + lane] = theirs;
            }
        __syncthreads();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const float mine = grp == 0 ? acc[rt][0][v] : acc[rt][0][8 + v];
                acc[rt][0][v] = mine + xb[((((grp ^ 1) * NWAVES + wave) * RT + rt) * 8 + v) * kWave + lane];
            }
    }

    // ---- epilogue.  D layout of 32x32x2: register v of lane (h, m) holds
    // row 8*(v/4) + 4*h + v%4, column m.
    if (SPLIT) {
        // partial sums (all splits share ma, mb: they depend on the column only)
        float *part = p.c + ((int64_t)split * p.R + r) * (int64_t)p.S * p.K;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (ncol[ct] >= p.K) continue;
            if (split == 0 && st == 0 && wm == 0 && h == 0) {
                p.shift[(int64_t)r * p.K + ncol[ct]] = ma[ct];
                p.shift[((int64_t)p.R + r) * p.K + ncol[ct]] = mb[ct];
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = s0 + wrow0 + 32 * rt + 8 * (v / 4) + 4 * h + (v % 4);
                    if (row < p.S) part[(int64_t)row * p.K + ncol[ct]] = acc[rt][ct][v];
                }
        }
    } else {
        // Rows past S fall outside the buffer extent and are dropped by the hardware.
        const int crows = p.S - (s0 + wrow0);  // valid rows below this wavefront's first row
        const __amdgpu_buffer_rsrc_t c_rsrc =
            make_rsrc(p.c + (int64_t)r * p.sc0 + (int64_t)(s0 + wrow0) * p.sc1,
                      crows > 0 ? (uint32_t)(((int64_t)(crows - 1) * p.sc1 + p.K) * 4) : 0u);
        const uint32_t c_row_bytes = (uint32_t)p.sc1 * 4u;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (ncol[ct] >= p.K) continue;
            const float mm = ma[ct] + mb[ct];
            const uint32_t co = ((uint32_t)(4 * h) * (uint32_t)p.sc1 + (uint32_t)ncol[ct]) * 4u;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int v = 0; v < 16 / GS; ++v) {
                    // (paired groups: register v of group g is accumulator register 8g + v)
                    const uint32_t trow_c = 32 * rt + 8 * (v / 4) + (v % 4) + (GS == 2 ? 16 * grp : 0);  // + 4h in the lane offset
                    buf_store_f32_out(p.stream_out != 0, log_plus(acc[rt][ct][v], mm), c_rsrc, co,
                                      trow_c * c_row_bytes);
                }
        }
    }
}

// ------------------------------------------------------------------ host
struct Lt2Variant {
    int rt, ct, nq;
    int wm = 1;     // wavefronts stacked over rows
    bool pack = false;  // J = 2, 4 or 8: chunks of 16 over the flat (i, j) axis
    int gs = 1;         // 2: two groups of four wavefronts halve the contraction of one tile between them
};
// variant ids (1-based in the C ABI; 0 = choose by shape)
// (Tiles of two 32-column groups per wavefront -- 64 x 256 and 32 x 256 -- were measured and
// dropped: 64 accumulator registers cost occupancy, 81-85 % of the MFMA peak against 87-89 %.)
static const Lt2Variant kVariants[] = {
    {2, 1, 8},  // 1: 64 x 128 tile, j-chunks of 64
    {2, 1, 4},  // 2: 64 x 128 tile, j-chunks of 32
    {1, 1, 8},  // 3: 32 x 128 tile, j-chunks of 64
    {1, 1, 4},  // 4: 32 x 128 tile, j-chunks of 32
    {1, 1, 2},  // 5..10: j-chunks of 16, 24 and 48 for contractions that chunks of 32 fit badly
    {1, 1, 3},
    {1, 1, 6},
    {2, 1, 2},
    {2, 1, 3},
    {2, 1, 6},
    {1, 1, 4, 4},  // 11: 128 x 32 tile, the 4 wavefronts stacked over rows (outputs of <= 32 columns)
    {1, 1, 4, 2},  // 12: 64 x 64 tile (outputs of <= 64 columns)
    {1, 1, 2, 1, true},  // 13, 14: short rows of w packed into chunks of 16 (other shapes: as 5 and 8)
    {2, 1, 2, 1, true},
    {1, 1, 4, 1, false, 2},  // 15, 16: tiles 4 and 2 with the contraction halved between two groups of
    {2, 1, 4, 1, false, 2},  //         wavefronts in the workgroup (grids of one or two tiles per compute unit)
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
constexpr int kLt2Waves = 4;

// Measured on MI355X at R=64, S=I=J=64, K=4096: the narrow wavefront tile (64 x 32,
// 32 accumulator registers, j-chunks of 32) runs at 87-89 % of the fp32 MFMA peak, the
// 64 x 64 tiles at 81-85 %: occupancy beats operand reuse here.
// Row tile: 32 rows unless the 64-row tile pays.  Its Khatri-Rao multiply is shared by two
// MFMAs, worth 3-6 % per row on contractions of I*J >= 1024 when the tiles divide evenly over
// the CUs (the rule is below, beside the counts it uses);
// everywhere else the 32-row tile is as fast or faster -- twice the workgroups hide more
// latency and balance better (over 288 random shapes: 4-30 % ahead on grids of 1-4 workgroups
// per CU, 27 % (median) when S leaves the last 64-row tile at most half full, e.g. S = 96,
// 160, 208).  (96- and 128-row tiles were measured too: per 32 rows they cost what the 32-row
// tile does.)  Rule checked against the better of the two tiles on those shapes: 0.6 % mean
// regret, 2 shapes of 288 more than 10 % off.
// Short rows that pack: whole rows per chunk of 16, 16-byte pieces that do not straddle the end
// of the flat axis, and more than one chunk.
static bool packs(int64_t I, int64_t J) {
    return (J == 2 || J == 4 || J == 8) && (I * J) % 4 == 0 && I * J >= 32;
}

static int find_lt2_variant(int rt, int nq, bool pack, int gs = 1) {
    for (int v = 0; v < kNumVariants; ++v)
        if (kVariants[v].rt == rt && kVariants[v].ct == 1 && kVariants[v].nq == nq && kVariants[v].wm == 1 &&
            kVariants[v].pack == pack && kVariants[v].gs == gs)
            return v;
    return 0;
}

static int choose_variant(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K) {
    // Outputs of at most 32 (64) columns would leave three (two) of the four wavefronts idle:
    // they are stacked over rows instead (128 x 32 and 64 x 64 tiles).
    // (No lower bound on the number of tiles as lm2exp has: tried, 1.4-2x slower on grids of 64
    // narrow tiles -- a tile's chain of I x J steps is long enough to keep its CU busy.)
    // (Not for short rows that pack: padding such rows to a chunk of 32 costs more than the idle
    // wavefronts -- the packed 128-column tile is 1.1-5x ahead at K = 16..64, J = 2, 4, 8.)
    const bool tall = K <= 32 && S > 64;
    if (!packs(I, J) && (tall || (K <= 64 && S > 32))) {
        const int wm = tall ? 4 : 2;
        for (int v = 0; v < kNumVariants; ++v)
            if (kVariants[v].wm == wm) return v;
    }
    int rt = 1;
    if (S > 32) {
        const int64_t last = S % 64;
        const bool same_padding = last == 0 || last > 32;
        const int64_t ct = ceil_div(K, 128);
        const int64_t n64 = R * ceil_div(S, 64) * ct, n32 = R * ceil_div(S, 32) * ct;
        // The busiest of the 256 CUs decides: it holds ceil(n / 256) tiles, a 64-row tile costs
        // 1.91 32-row tiles.  Measured over 200 shapes with I*J = 1024..16384 and 256..2048
        // 64-row tiles, this ranks the two tiles right: 64 rows are 3-6 % ahead at 448-512, 768,
        // 1024, 2048 tiles, 26 % behind at 320-384 and 14 % behind at 640.  With exactly one
        // 64-row tile per CU the two are level (3-5 % behind launched back to back, 4-5 % ahead
        // on inputs that are not in cache, as the reference's benchmarks time them): 64 rows.
        const int64_t q64 = ceil_div(n64, 256), q32 = ceil_div(n32, 256);
        const int64_t c64 = 191 * q64 * (q64 == 1 ? 104 : 100), c32 = 100 * q32 * 100;
        // (Short contractions, I*J < 1024, were measured level on grids of a few tiles per CU; from
        // four 64-row tiles per CU on they want 64 rows too -- half the workgroups, so half the
        // sweeps, first loads and result stores that a short chain cannot hide: over 44 large
        // grids 7-17 % on every such shape, R=64, S=765, I=5, J=108, K=1739: 897 -> 790 us;
        // R=256, S=52, I=4, J=36, K=2286: 155 -> 132.)
        if (same_padding && (I * J >= 1024 || n64 >= 1024) && c64 < c32) rt = 2;
        // packed rows spend more vector instructions per step (a factor of a per row of the chunk):
        // sharing them between two MFMAs pays from half a wave of workgroups on, whatever the
        // length of the contraction (measured: 6-13 % at 256..2048 tiles, level at 192, from 4 %
        // ahead to 20 % behind at 128, 15 % behind at 20)
        if (same_padding && packs(I, J) && n64 >= 192) rt = 2;
    }
    // j-chunk: the one that pads J least.  Per padded j the chunks cost the same within a few
    // per cent (measured at S = I = 64, K = 4096, R = 64: 15.3 us per j with chunks of 32 or 48,
    // 15.5-16.5 with 16, 15.5-16.1 with 24), so J = 16, 24, 40, 48, 72 run 1.3-2.2x faster on
    // chunks that fit than on chunks of 32 (J = 48: 1059 -> 735 us), also because a last chunk
    // that is only partly filled takes the masked loads.  Ties go to chunks of 32.
    if (packs(I, J)) return find_lt2_variant(rt, 2, true);
    int nq = 4;
    int64_t best = ceil_div(J, 32) * 32 * 100;
    const int cand[3] = {6, 3, 2};
    const int64_t penalty[3] = {100, 103, 109};
    for (int c = 0; c < 3; ++c) {
        // rows of w that are not 16-byte aligned (J not a multiple of 4) are staged float by
        // float, coalesced only for chunks that divide the workgroup evenly: 16 and 32
        if (J % 4 != 0 && cand[c] != 2) continue;
        const int64_t cost = ceil_div(J, 8 * cand[c]) * 8 * cand[c] * penalty[c];
        if (cost < best) {
            best = cost;
            nq = cand[c];
        }
    }
    // 64-row tiles on a large grid (four per CU and more) under a J that whole chunks of 64 fit:
    // chunks of 64 -- half the steps and barriers, and with J = 64 a single j-chunk, so every row
    // of a is loaded and exponentiated once per tile instead of twice.  Timed side by side,
    // alternating: R=64, S=I=J=64, K=4096 975.2 -> 967.2 us (every one of 12 pairs within 1 us
    // of that); R=128, S=I=J=K=256 7675 -> 7560; R=32, S=64, I=128, J=64, K=4096 982 -> 965.  (On
    // small grids the 64-wide chunk's 16 more registers and coarser steps cost up to 25 %.)
    if (rt == 2 && nq == 4 && J % 64 == 0 && R * ceil_div(S, 64) * ceil_div(K, 128) >= 1024) nq = 8;
    return find_lt2_variant(rt, nq, false);
}

template <int RT, int CT, int NQ, bool VEC, bool SPLIT, int WM>
static void launch_one(const Lt2Args &args, hipStream_t stream) {
    hipLaunchKernelGGL((lt2exp_kernel<RT, CT, NQ, kLt2Waves, VEC, SPLIT, WM>), dim3((unsigned)args.padded_wgs),
                       dim3(kLt2Waves * kWave), 0, stream, args);
}

template <int RT, int CT, int NQ, int WM = 1>
static void launch_vs(const Lt2Args &args, bool vec, bool split, hipStream_t stream) {
    if (vec) {
        if (split) launch_one<RT, CT, NQ, true, true, WM>(args, stream);
        else launch_one<RT, CT, NQ, true, false, WM>(args, stream);
    } else {
        if (split) launch_one<RT, CT, NQ, false, true, WM>(args, stream);
        else launch_one<RT, CT, NQ, false, false, WM>(args, stream);
    }
}

template <int RT, int PJ>
static void launch_packed_pj(const Lt2Args &args, bool split, hipStream_t stream) {
    if (split)
        hipLaunchKernelGGL((lt2exp_kernel<RT, 1, 2, kLt2Waves, true, true, 1, PJ>), dim3((unsigned)args.padded_wgs),
                           dim3(kLt2Waves * kWave), 0, stream, args);
    else
        hipLaunchKernelGGL((lt2exp_kernel<RT, 1, 2, kLt2Waves, true, false, 1, PJ>), dim3((unsigned)args.padded_wgs),
                           dim3(kLt2Waves * kWave), 0, stream, args);
}

template <int RT>
static void launch_packed(const Lt2Args &args, bool split, hipStream_t stream) {
    if (args.J == 8) launch_packed_pj<RT, 8>(args, split, stream);
    else if (args.J == 4) launch_packed_pj<RT, 4>(args, split, stream);
    else launch_packed_pj<RT, 2>(args, split, stream);
}

template <int RT>
static void launch_paired(const Lt2Args &args, hipStream_t stream) {
    hipLaunchKernelGGL((lt2exp_kernel<RT, 1, 4, kLt2Waves, true, false, 1, 0, 2>), dim3((unsigned)args.padded_wgs),
                       dim3(2 * kLt2Waves * kWave), 0, stream, args);
}

static void launch_variant(int v, const Lt2Args &args, bool vec, bool split, hipStream_t stream) {
    if (kVariants[v].gs == 2) {  // (the caller has made sure of aligned rows and an uncut contraction)
        if (kVariants[v].rt == 2) launch_paired<2>(args, stream);
        else launch_paired<1>(args, stream);
        return;
    }
    if (kVariants[v].pack) {
        if (kVariants[v].rt == 2) launch_packed<2>(args, split, stream);
        else launch_packed<1>(args, split, stream);
        return;
    }
    switch (v) {
        case 0: launch_vs<2, 1, 8>(args, vec, split, stream); break;
        case 1: launch_vs<2, 1, 4>(args, vec, split, stream); break;
        case 2: launch_vs<1, 1, 8>(args, vec, split, stream); break;
        case 4: launch_vs<1, 1, 2>(args, vec, split, stream); break;
        case 5: launch_vs<1, 1, 3>(args, vec, split, stream); break;
        case 6: launch_vs<1, 1, 6>(args, vec, split, stream); break;
        case 7: launch_vs<2, 1, 2>(args, vec, split, stream); break;
        case 8: launch_vs<2, 1, 3>(args, vec, split, stream); break;
        case 9: launch_vs<2, 1, 6>(args, vec, split, stream); break;
        case 10: launch_vs<1, 1, 4, 4>(args, vec, split, stream); break;
        case 11: launch_vs<1, 1, 4, 2>(args, vec, split, stream); break;
        default: launch_vs<1, 1, 4>(args, vec, split, stream); break;
    }
}

struct SplitPlan {
    bool split;
    int splits;
    int iters_per_split;
    double us = 0.0;  // modelled time of the call (0: this plan comes from a rule, not from the fitted model)
};
static SplitPlan plan_split(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode, int variant);

// Grids of at most two 32-row tiles per compute unit that are not worth cutting over workgroups
// (plan_split) run with the contraction halved between two groups of wavefronts of one
// workgroup instead: 3-27 % faster over 70 random such shapes (R=16, S=64, I=J=32, K=2048: 40.7 ->
// 38.9 us; R=128, S=128, I=64, J=32, K=128: 77 -> 73; R=16, S=32, I=J=32, K=2048: 26.4 -> 24.2).
// 64 rows where the contraction is short (I*J <= 1024) and 64-row tiles fill more than half of
// the CUs, else 32 rows.  Only for aligned rows of w and j-chunks of 32 (the caller checks).
static int paired_variant(int v, int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode) {
    const Lt2Variant &vr = kVariants[v];
    if (mode == TRT_MODE_SPLIT || vr.nq != 4 || vr.pack || vr.wm != 1 || vr.gs != 1) return v;
    const SplitPlan sp = plan_split(R, S, I, J, K, mode, v);
    const int64_t ct = ceil_div(K, 128);
    const int64_t n32 = R * ceil_div(S, 32) * ct, n64 = R * ceil_div(S, 64) * ct;
    if (n32 > 512 || I * ceil_div(J, 32) < 2) return v;
    const int64_t last = S % 64;
    const bool pads_alike = S > 32 && (last == 0 || last > 32);
    if (sp.us > 0.0) {
        // the plan is the fitted model's (plan_split): paired groups are priced by the same model --
        // the whole chain on one CU, which two groups of wavefronts keep at 90 % of the rate
        // (97 % with a second workgroup beside them), half a microsecond for the exchange -- and
        // taken where that is the cheaper plan (timed on 56 shapes of at most 512 tiles: 0.2 %
        // behind the better of the two on average; never pairing would lose 1.8 %)
        const int64_t iters = ceil_div(J, 32) * I;
        auto paired_us = [&](int rt) {
            const int64_t q = ceil_div(rt == 2 ? n64 : n32, 256);
            const double unit_us = (256.0 * 4 * rt + 85.0 + 25.0 * 4) / 2400.0;
            return 6.4 + (double)q * ((double)iters * unit_us + 0.0062 * (double)(I + J)) / (q >= 2 ? 0.97 : 0.9) + 0.5;
        };
        const int rt = (I * J <= 1024 && pads_alike && n64 > 128) ? 2 : 1;
        return paired_us(rt) < sp.us ? find_lt2_variant(rt, 4, false, 2) : v;
    }
    if (sp.split) return v;
    const bool rows64 = I * J <= 1024 && pads_alike && n64 > 128;
    return find_lt2_variant(rows64 ? 2 : 1, 4, false, 2);
}

// A 64 x 64 tile (the wavefronts 2 x 2) in place of the 32 x 128 one where tiles of 128 columns
// would stand half empty: K = 192 is three tiles of 64 columns or two of 128, the second half
// idle.  Taken when the 64 x 64 tiles cover at most 0.8 of the padded area (rows included: they
// pad S to 64), for aligned rows of w and j-chunks of 32 only (the tile has no other build).
// Measured: S=I=J=K=192, batch 1 (one of the reference's benchmark shapes) 61.8 -> 51.3 us;
// R=1, S=535, I=26, J=64, K=136: 18.5 -> 16.5; R=6, S=449, I=10, J=92, K=192: 30.5 -> 27.0;
// R=32, S=60, I=11, J=96, K=192: 25.3 -> 23.2; at 0.88 of the area (R=32, S=41, I=52, J=160,
// K=424) still 5 % ahead, at 0.9 and above level or behind; where paired groups apply they
// stay (R=16, S=382, I=10, J=32, K=184: 16.4 against 17.5).
static int narrow_variant(int v, int64_t S, int64_t K) {
    const Lt2Variant &vr = kVariants[v];
    if (vr.gs != 1 || vr.wm != 1 || vr.pack || vr.nq != 4 || vr.rt != 1 || S <= 32) return v;
    const int64_t area128 = ceil_div(S, 32) * 32 * ceil_div(K, 128) * 128;
    const int64_t area64 = ceil_div(S, 64) * 64 * ceil_div(K, 64) * 64;
    if (5 * area64 > 4 * area128) return v;
    for (int u = 0; u < kNumVariants; ++u)
        if (kVariants[u].wm == 2) return u;
    return v;
}

// Where both apply, the 64 x 64 tile goes first under a long contraction (64 steps and more: R=6,
// S=656, I=40, J=160, K=186 takes 100 us on it, cut, against 129 on paired groups), paired groups
// under a short one (R=16, S=382, I=10, J=32, K=184: 16.4 against 17.5).
static int narrow_or_paired_variant(int v, int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode) {
    const int narrow = narrow_variant(v, S, K);
    if (narrow != v && I * ceil_div(J, 32) >= 64) return narrow;
    return narrow_variant(paired_variant(v, R, S, I, J, K, mode), S, K);
}

// A grid whose contraction is cut over workgroups anyway does not need its tiles to be many: the
// cut fills the CUs, and the 64-row tile's Khatri-Rao multiply serves two MFMAs.  So a 32-row
// tile that would be cut gives way to the 64-row tile of the same j-chunk when S pads alike and
// at least twelve 64-row tiles are left (fewer, and the 32-row tile's finer grain wins: batch 1,
// S=I=J=K=128 29 us against 37).  Measured: R=32, S=I=J=64, K=256 (one of the reference's
// benchmark shapes) 53.8 -> 47.1 us; R=4, S=170, I=90, J=128, K=245 59.9 -> 54.3; R=1, S=570,
// I=26, J=128, K=1309 66.5 -> 61.9; R=32, S=I=J=128, K=256 281 -> 267.
static int tall_variant(int v, int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode) {
    const Lt2Variant &vr = kVariants[v];
    if (mode == TRT_MODE_UNSPLIT || vr.rt != 1 || vr.gs != 1 || vr.wm != 1 || vr.pack || S <= 32) return v;
    const int64_t last = S % 64;
    if (!(last == 0 || last > 32) || R * ceil_div(S, 64) * ceil_div(K, 128) < 12) return v;
    const int tall = find_lt2_variant(2, vr.nq, false);
    if (kVariants[tall].rt != 2 || kVariants[tall].nq != vr.nq) return v;
    return plan_split(R, S, I, J, K, mode, v).split && plan_split(R, S, I, J, K, mode, tall).split ? tall : v;
}

// AUTO follows the reference in kind -- a small output grid with a long contraction is
// split (triturus/lt2exp.py:535 tests R*S*K < 1048576 and I*J > 512) -- but decides with a
// cost model fitted to this machine (measured: R=16 S=64 I=J=32 K=2048, 256 tiles of 32
// iterations, is 1.4x slower split; R=32 S=I=J=48..256 K=256 is 1.3-2.8x faster).
static SplitPlan plan_split(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode, int variant) {
    const Lt2Variant &v = kVariants[variant];
    const int64_t iters = v.pack ? ceil_div(I * J, 8 * v.nq) : ceil_div(J, 8 * v.nq) * I;
    if (mode == TRT_MODE_UNSPLIT || v.gs == 2) return {false, 1, (int)iters};
    const int64_t base = R * ceil_div(S, 32 * v.rt * v.wm) * ceil_div(K, 32 * v.ct * (kLt2Waves / v.wm));
    // 128-column tiles on aligned rows of w: the cut with the least modelled time, where the model
    // is the one fitted for lm2exp's small grids (csrc/lm2exp.hip, choose_tile_and_cut) with this
    // kernel's constants: a step costs its MFMAs plus 85 + 25 nq cycles of vector work, a
    // workgroup's sweeps for the column maxima 6.2 ns per row of a and b, the busiest CU runs
    // q = ceil(workgroups / 256) chains at 73 % of that rate alone, 93.5 % with two, 95 % with
    // three, in full from four on; a launch costs 6.4 us, a cut 4.8 us more plus its partial
    // sums' trip at 3.36 TB/s.  Fitted to cuts of 1..32 timed on 32- and 64-row tiles of 88
    // shapes; on 83 other shapes (166 tiles) the cut it picks is 1.4 % (mean) behind the best
    // one timed, the cut of the model below 4.6 % (R=8, S=296, I=184, J=28, K=1556, 64 rows:
    // 562 us uncut, 435 cut four ways; R=16, S=74, I=55, J=92, K=2372: 488 -> 417).
    if (!v.pack && v.wm == 1 && v.ct == 1 && J % 4 == 0) {
        const double unit_us = (256.0 * v.nq * v.rt + 85.0 + 25.0 * v.nq) / 2400.0;
        const double sweep_us = 0.0062 * (double)(I + J);
        int best = 1;
        double best_us = 1e300, uncut_us = 0.0;
        const bool forced = mode == TRT_MODE_SPLIT && iters >= 2;  // a cut is asked for: two ways at least
        for (int sp = forced ? 2 : 1; sp <= 32; ++sp) {
            if (sp > 1 && 4 * sp > iters && !(forced && sp == 2)) break;  // four steps per workgroup at least
            const int64_t per = ceil_div(iters, sp);
            if (ceil_div(iters, per) != sp) continue;  // the same cut as a smaller count
            const int64_t q = ceil_div(base * sp, 256);
            const double eff = q >= 4 ? 1.0 : (q == 3 ? 0.95 : (q == 2 ? 0.935 : 0.73));
            double us = 6.4 + (double)q * ((double)per * unit_us + sweep_us) / eff;
            if (sp > 1) us += 4.8 + (double)(sp + 1) * (double)(R * S * K) * 4.0 / 3.36e6;
            if (sp == 1) uncut_us = us;
            if (us < best_us) {
                best_us = us;
                best = sp;
            }
        }
        // a cut must win by 3 % (that margin costs nothing on the timed shapes, and on inputs that
        // are not in cache, as the reference's benchmarks time them, a marginal cut loses: R=128,
        // S=I=J=96, K=256 runs 2 % slower cut two ways)
        if (best > 1 && uncut_us > 0.0 && best_us > 0.97 * uncut_us) {
            best = 1;
            best_us = uncut_us;
        }
        if (best <= 1) return {false, 1, (int)iters, best_us};
        return {true, best, (int)ceil_div(iters, best), best_us};
    }
    // (the 64-row tile alone on a CU runs at 67 % of the MFMA rate, two of them at 82 %: measured
    // at R=16 / 32, S=64, I=J=32, K=2048, 40.6 and 66.5 us)
    const bool tall = v.rt >= 2;
    int64_t splits = choose_splits(base, iters, 4 * v.nq * v.rt * v.ct, R * S * K, 4, 32, mode == TRT_MODE_SPLIT, 0.0,
                                   0.8, tall ? 0.67 : 0.45, tall ? 0.82 : 0.65);
    if (splits <= 1) return {false, 1, (int)iters};
    const int64_t per = ceil_div(iters, splits);
    splits = ceil_div(iters, per);
    if (splits <= 1) return {false, 1, (int)iters};
    return {true, (int)splits, (int)per};
}

}  // namespace trt

using namespace trt;

extern "C" int trt_lt2exp_variant_count(void) { return kNumVariants; }

static int resolve_variant(int variant, int64_t R, int64_t S, int64_t I, int64_t J, int64_t K) {
    if (variant >= 1 && variant <= kNumVariants) return variant - 1;
    return choose_variant(R, S, I, J, K);
}

extern "C" size_t trt_lt2exp_workspace_bytes(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode) {
    if (R <= 0 || S <= 0 || I <= 0 || J <= 0 || K <= 0) return 0;
    // the split count depends on the tile shape: size for the largest possible; a call with
    // J = 1 may run with i and j exchanged (trt_lt2exp_f32): room for either
    size_t need = 0;
    for (int pass = 0; pass < 2; ++pass) {
        if (pass == 1) {
            if (!(J == 1 && I > 1)) break;
            J = I;
            I = 1;
        }
        for (int v = 0; v < kNumVariants; ++v) {
            SplitPlan sp = plan_split(R, S, I, J, K, mode, v);
            if (!sp.split) continue;
            size_t b = ((size_t)sp.splits * R * S * K + (size_t)2 * R * K) * sizeof(float);
            if (b > need) need = b;
        }
    }
    return need;
}

namespace trt {
// for trt_lt2exp_bf16, which hands such calls over: would trt_lt2exp_f32 take the sweep of
// csrc/lt2exp_smallk.hpp?
bool lt2exp_takes_sweep(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_aligned, bool w_dense) {
    return smallk_applies(R, S, I, J, K, w_aligned, w_dense);
}
// likewise: would it take the kernel of csrc/lt2exp_cols.hpp (few units, a lane per column)?
bool lt2exp_takes_cols(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_dense, double margin) {
    return cols_applies(I, J, K) && cols_score(R, S, I, J, K, w_dense) > margin;
}
// likewise: would it take the kernel of csrc/lt2exp_rows.hpp (few s per batch)?
// (margin: by how many doublings the fp32 rule's estimate must favour it)
bool lt2exp_takes_rows(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_aligned, bool w_dense,
                       double margin) {
    return rows_score(R, S, I, J, K) > margin && rows_plan(R, S, I, J, K, w_aligned, w_dense).ct != 0;
}
// for trt_lm2exp_f32: c[r, i, k] = log sum_j a[r, i, j] exp(b[r, j, k]) is the same sweep with the
// rows of a as the weights, a contracted plane of 1 x J and no factors on the other side.  Is
// that the faster way?  Only with at most 4 columns and rows of 1024 values and more: lm2exp's
// own tiles stream a at 3.5-4.7 TB/s, and a row ends in a sum over the lanes (timed: R=16, I=4096,
// J=1024: K=1 60 -> 45 us, K=4 58 -> 53, K=8 57 -> 82; R=64, I=64, J=4096, K=1: 37 -> 21;
// rows of 64..256 values: 0.2-0.8x).
bool lm2exp_takes_sweep(int64_t R, int64_t I, int64_t J, int64_t K, bool a_aligned) {
    return K <= 4 && J >= 1024 && J % 4 == 0 && a_aligned && smallk_applies(R, I, 1, J, K, a_aligned);
}
int lm2exp_sweep(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                 const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], hipStream_t stream) {
    const int64_t none[3] = {0, 0, 0};
    return launch_lt2exp_smallk(a, nullptr, b, c, R, I, 1, J, K, sa, none, sb, sc, true, stream);
}
// for trt_lm2exp_f32: lm2exp with J <= 16 is the lane-per-column kernel of csrc/lt2exp_cols.hpp with
// the rows of a as the weights (S = I, a contracted plane of 1 x J, no factors on the other side)
// Taken by the sign of a linear score in log2 units fitted to 350 timed shapes (J = 1..16, I = 1..256,
// K = 9..2048, up to 100 000 batches) against lm2exp's own tiles, which pad i to 32 rows and j to a
// chunk of 32: - 0.46 per doubling of I and - 0.48 per doubling of J (a lane's FMAs), - 0.12 per
// doubling of K, + 0.81 for rows of exactly 4, 8 or 16 dense values (one scalar load per row),
// + 0.2 per doubling of the call's work.  1.9 % behind the faster choice per shape (never taking it
// 34 %, always 41 %): R=8192, I=J=4, K=1024 190 -> 42 us, I=J=8 189 -> 101.
bool lm2exp_takes_cols(int64_t R, int64_t I, int64_t J, int64_t K, bool a_dense, double margin) {
    if (J > 16 || K <= 8) return false;
    const bool exact = (J == 4 || J == 8 || J == 16) && a_dense;
    const double work = 2.0 * (double)R * (double)I * (double)J * (double)K;
    return -1.24 - 0.46 * std::log2((double)I) - 0.475 * std::log2((double)J) - 0.12 * std::log2((double)K) +
               (exact ? 0.81 : 0.0) + 0.196 * std::log2(work) > margin;
}
int lm2exp_cols(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], hipStream_t stream) {
    const int64_t none[3] = {0, 0, 0};
    return launch_lt2exp_cols(a, nullptr, b, c, R, I, 1, J, K, sa, none, sb, sc, stream);
}
int lm2exp_cols_name(int64_t J, bool a_dense, char *buf, size_t buf_bytes) { return cols_kernel_name(1, J, a_dense, buf, buf_bytes); }
int lt2exp_sweep_name(int64_t R, int64_t S, int64_t J, int64_t K, bool w_aligned, char *buf, size_t buf_bytes) {
    const int n = snprintf(buf, buf_bytes, "trt::lt2exp_smallk_kernel<%d, %d, %s>", small_kc(K), smallk_wpr(R, S),
                           smallk_anyj(J, w_aligned) ? "true" : "false");
    return n > 0 && (size_t)n < buf_bytes ? 0 : TRT_E_RANGE;
}
}  // namespace trt

extern "C" int trt_lt2exp_f32(const float *w, const float *a, const float *b, float *c, int64_t R, int64_t S,
                              int64_t I, int64_t J, int64_t K, const int64_t sw[3], const int64_t sa[3],
                              const int64_t sb[3], const int64_t sc[3], int mode, int variant, void *workspace,
                              size_t workspace_bytes, void *stream) {
    if (!w || !a || !b || !c || !sw || !sa || !sb || !sc) return TRT_E_INVALID;
    if (R <= 0 || S <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (mode != TRT_MODE_AUTO && mode != TRT_MODE_SPLIT && mode != TRT_MODE_UNSPLIT) return TRT_E_INVALID;
    if (variant < 0 || variant > kNumVariants) return TRT_E_INVALID;
    if (sw[2] < 0 || sa[2] < 0 || sb[2] < 0 || sc[2] != 1) return TRT_E_LAYOUT;
    for (int d = 0; d < 2; ++d)
        if (sw[d] < 0 || sa[d] < 0 || sb[d] < 0 || sc[d] < 0) return TRT_E_LAYOUT;
    if (sc[1] < K) return TRT_E_LAYOUT;  // output rows must not overlap (stores rely on it)
    const int64_t lim = (int64_t)1 << 30;
    if (R >= lim || S >= lim || I >= lim || J >= lim || K >= lim || I * J >= lim) return TRT_E_RANGE;
    // byte offsets inside one batch slab of w, a and c are 32-bit (buffer addressing)
    if (S * sw[1] + I * J * (sw[2] > 0 ? sw[2] : 1) >= lim || I * sa[1] + K * sa[2] >= lim ||
        J * sb[1] + K * sb[2] >= lim || S * sc[1] + K >= lim)
        return TRT_E_RANGE;

    // A single j under several i: the contraction is symmetric in (i, a) and (j, b), and with
    // J = 1 the same w is an R x S x 1 x I tensor, so the call runs with the roles exchanged
    // (the kernel walks j in chunks and i one at a time: one chunk of I instead of I chunks of 1).
    if (J == 1 && I > 1 && variant == 0)
        return trt_lt2exp_f32(w, b, a, c, R, S, 1, I, K, sw, sb, sa, sc, mode, variant, workspace, workspace_bytes,
                              stream);

    // (a flat axis of w with another stride than 1 -- a sliced view -- is read element by element, in place)
    const bool w_aligned = sw[2] == 1 && (sw[0] % 4 == 0) && (sw[1] % 4 == 0) && ((reinterpret_cast<uintptr_t>(w) & 15) == 0);
    // outputs of at most 8 columns: a sweep over w on the vector ALU (csrc/lt2exp_smallk.hpp); no
    // cut, no workspace, whatever the mode asks for
    if (variant == 0 && smallk_applies(R, S, I, J, K, w_aligned, sw[2] == 1))
        return launch_lt2exp_smallk(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, w_aligned, static_cast<hipStream_t>(stream));
    // layers of few units over many batches: a lane per output column (csrc/lt2exp_cols.hpp); no cut
    // and no workspace either
    if (variant == 0 && cols_pays(R, S, I, J, K, sw[2] == 1))
        return launch_lt2exp_cols(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, static_cast<hipStream_t>(stream));
    // few s per batch: the rows (s, i) of w on the rows of the MFMA, j contracted first
    // (csrc/lt2exp_rows.hpp); no cut and no workspace either
    if (variant == 0 && rows_pays(R, S, I, J, K)) {
        const RowsPlan rp = rows_plan(R, S, I, J, K, w_aligned, sw[2] == 1);
        if (rp.ct) return launch_lt2exp_rows(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, rp, static_cast<hipStream_t>(stream));
    }
    int v = resolve_variant(variant, R, S, I, J, K);
    // packed rows need 16-byte loads along the flat (i, j) axis; any other call runs the same tile unpacked
    if (kVariants[v].pack && !(packs(I, J) && w_aligned)) v = find_lt2_variant(kVariants[v].rt, 2, false);
    if (variant == 0) v = tall_variant(v, R, S, I, J, K, mode);
    if (variant == 0 && (J % 4 == 0) && w_aligned) v = narrow_or_paired_variant(v, R, S, I, J, K, mode);
    // paired groups: aligned rows only, and never under a forced cut over workgroups
    if (kVariants[v].gs == 2 && (!((J % 4 == 0) && w_aligned) || mode == TRT_MODE_SPLIT))
        v = find_lt2_variant(kVariants[v].rt, kVariants[v].nq, false);
    const Lt2Variant &vr = kVariants[v];
    const SplitPlan sp = plan_split(R, S, I, J, K, mode, v);

    Lt2Args args;
    args.w = w; args.a = a; args.b = b;
    args.R = (int)R; args.S = (int)S; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sw0 = sw[0]; args.sw1 = sw[1]; args.sw2 = sw[2];
    args.sa0 = sa[0]; args.sa1 = sa[1]; args.sa2 = sa[2];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.s_tiles = (int)ceil_div(S, 32 * vr.rt * vr.wm);
    args.n_tiles = (int)ceil_div(K, 32 * vr.ct * (kLt2Waves / vr.wm));
    args.splits = sp.splits;
    args.iters_per_split = sp.iters_per_split;
    args.total_wgs = (int64_t)R * args.s_tiles * args.n_tiles * sp.splits;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    args.stream_out = rows_16_byte_aligned(c, sc[0], sc[1]);
    if (args.padded_wgs >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    args.shift = nullptr;
    args.c = c;
    if (sp.split) {
        const size_t need = ((size_t)sp.splits * R * S * K + (size_t)2 * R * K) * sizeof(float);
        if (!workspace || workspace_bytes < need) return TRT_E_WORKSPACE;
        args.c = static_cast<float *>(workspace);
        args.shift = args.c + (size_t)sp.splits * R * S * K;
    }
    // 16-byte loads of w need aligned rows
    const bool vec = (J % 4 == 0) && w_aligned;
    hipStream_t s = static_cast<hipStream_t>(stream);
    launch_variant(v, args, vec, sp.split, s);
    if (sp.split) launch_lt2exp_merge(args.c, args.shift, c, R, S, K, sp.splits, sc[0], sc[1], s);
    return (int)hipGetLastError();
}

// Name of the contraction kernel a trt_lt2exp_f32 call with these arguments launches, as a
// profiler prints it (host only; w_aligned: base and both leading strides of w are multiples
// of 16 bytes).  Benchmarks use it to look their kernel up in profiler output.
extern "C" int trt_lt2exp_kernel_name(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode, int variant,
                                      int w_aligned, char *buf, size_t buf_bytes) {
    if (!buf || buf_bytes == 0 || R <= 0 || S <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (variant < 0 || variant > kNumVariants) return TRT_E_INVALID;
    if (J == 1 && I > 1 && variant == 0) {  // runs with the roles of i and j exchanged
        J = I;
        I = 1;
    }
    // (w_aligned = 0: rows that are not 16-byte aligned, of a dense flat axis)
    if (variant == 0 && smallk_applies(R, S, I, J, K, w_aligned != 0)) return lt2exp_sweep_name(R, S, J, K, w_aligned != 0, buf, buf_bytes);
    if (variant == 0 && cols_pays(R, S, I, J, K, true)) return cols_kernel_name(I, J, true, buf, buf_bytes);
    if (variant == 0 && rows_pays(R, S, I, J, K)) {
        const RowsPlan rp = rows_plan(R, S, I, J, K, w_aligned != 0);
        if (rp.ct) {
            const int n = snprintf(buf, buf_bytes, "trt::lt2exp_rows_kernel<%d, %d, %s>", rp.ct / rp.cts, rp.cts, rp.vec ? "true" : "false");
            return n > 0 && (size_t)n < buf_bytes ? 0 : TRT_E_RANGE;
        }
    }
    int v = resolve_variant(variant, R, S, I, J, K);
    if (kVariants[v].pack && !(packs(I, J) && w_aligned)) v = find_lt2_variant(kVariants[v].rt, 2, false);
    if (variant == 0) v = tall_variant(v, R, S, I, J, K, mode);
    if (variant == 0 && (J % 4 == 0) && w_aligned) v = narrow_or_paired_variant(v, R, S, I, J, K, mode);
    if (kVariants[v].gs == 2 && (!((J % 4 == 0) && w_aligned) || mode == TRT_MODE_SPLIT))
        v = find_lt2_variant(kVariants[v].rt, kVariants[v].nq, false);
    const Lt2Variant &vr = kVariants[v];
    const SplitPlan sp = plan_split(R, S, I, J, K, mode, v);
    const bool vec = vr.pack || ((J % 4 == 0) && w_aligned);
    const int n = snprintf(buf, buf_bytes, "trt::lt2exp_kernel<%d, %d, %d, %d, %s, %s, %d, %d, %d>", vr.rt, vr.ct,
                           vr.pack ? 2 : vr.nq, kLt2Waves, vec ? "true" : "false", sp.split ? "true" : "false", vr.wm,
                           vr.pack ? (int)J : 0, vr.gs);
    return n > 0 && (size_t)n < buf_bytes ? 0 : TRT_E_RANGE;
}

// ---------------------------------------------------------------------------------------------
// trt_lt2exp_f32_static: the same call for callers that cannot allocate (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).  The split-mode workspace --
// partial sums of every split and the two shift vectors -- lives in a file-scope device array
// of kStaticScratchBytes instead of a caller's buffer.  Host code never passes the array's name
// to a kernel (it is a host-side stand-in, not a device address): at the first call on a device
// the address of that device's copy is looked up with hipGetSymbolAddress and kept, and the
// kernels take it as the workspace argument exactly as they take a caller's buffer.  Every
// element of the workspace that the merge kernel reads is written by the contraction kernel of
// the same call first, so nothing has to be cleared between calls; calls that overlap on one
// GPU share the array and race.
namespace trt {
constexpr size_t kStaticScratchBytes = TRT_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void *g_scratch_ptr[kMaxDevices];  // per device: address of that device's copy of `scratch`
static std::mutex g_scratch_mutex;

// Address of the current device's copy of the static scratch array (set-up on first use).
static int static_scratch(void **ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return TRT_E_RANGE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return TRT_E_INVALID;
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}
}  // namespace trt

extern "C" int trt_lt2exp_f32_static(const float *w, const float *a, const float *b, float *c, int64_t R, int64_t S,
                                     int64_t I, int64_t J, int64_t K, const int64_t sw[3], const int64_t sa[3],
                                     const int64_t sb[3], const int64_t sc[3], int mode, int variant, void *stream) {
    if (R <= 0 || S <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    // what the call may need at most (any tile the shape rule can pick): beyond the array, refuse
    const size_t need = trt_lt2exp_workspace_bytes(R, S, I, J, K, mode);
    if (need > trt::kStaticScratchBytes) return TRT_E_SCRATCH;
    void *ws = nullptr;
    if (need > 0) {
        const int st = trt::static_scratch(&ws);
        if (st != 0) return st;
    }
    return trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, variant, ws,
                          need > 0 ? trt::kStaticScratchBytes : 0, stream);
}
