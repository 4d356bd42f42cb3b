// lt2exp with j contracted first: c[r, s, k] = log sum_i exp a[i, k] (sum_j w[s, i, j] exp b[j, k]).
//
// The tiles of csrc/lt2exp.hip put s on the rows of the MFMA and multiply w by the products
// exp a[i, k] exp b[j, k], which the vector ALU makes once per tile of 32..128 values of s: with
// few s per batch most rows of every MFMA are padding and the products are made for nothing
// (R=2048, S=1, I=J=64, K=64: 510 us for 34 MB of w).  Here the rows of the MFMA are the rows
// (s, i) of w -- S I of them per batch, however small S is -- the contracted axis is j alone and
// the B operand is exp(b - mb), kept in LDS for the whole workgroup: no product is formed at all.
// What the MFMA leaves, t[(s, i), k], is multiplied by exp(a[i, k] - ma[k]) and summed over i
// where it sits, in the accumulators (16 rows of a tile per lane, then the two lane halves),
// once per tile of 32 rows.  The flops are those of the other kernel's; its i-by-i outer loop
// turns into this epilogue, 16 FMAs per J / 2 MFMAs.
//
// A workgroup (4 wavefronts) owns a batch r, 32 CT columns of k and a group of up to 16 values of
// s; its wavefronts deal out the tiles (s, 32 values of i) among them.  A lane reads its row of w
// straight from memory into the MFMA's A layout (lane = row, 16 bytes per load, the two lane
// halves on adjacent pieces), 64 values of j ahead of the MFMAs that consume them; w never
// passes through LDS.  The sums of a wavefront's tiles of one s leave through LDS, each
// (wavefront, s) slot written once, and are added in a fixed order: results do not depend on
// timing.
#pragma once

#include <atomic>
#include <cmath>

#include "common.hpp"

namespace trt {

struct Lt2RowsArgs {
    const float *w, *a, *b;
    float *c;
    int R, S, I, J, K;
    int64_t sw0, sw1, sa0, sa1, sa2, sb0, sb1, sb2, sc0, sc1;  // (rows (i) of w: J floats apart, dense)
    int n_tiles;       // tiles of 32 CT columns
    int s_groups;      // workgroups per (r, column tile)
    int s_per_group;   // values of s of a workgroup (at most kRowsMaxS)
    int jp, ip;        // LDS pitches (floats) of a column's factors of b and of a
};

constexpr int kRowsWaves = 4;
constexpr int kRowsThreads = kRowsWaves * kWave;
constexpr int kRowsMaxS = 16;
constexpr int kRowsChunk = 64;                 // values of j per step: 8 loads of 16 bytes per lane
constexpr int kRowsGroups = kRowsChunk / 8;    // groups of 8 values of j (4 MFMAs each)
constexpr int kRowsBlock = 16;                 // loads of a thread in flight in the prologue

// VEC: rows of w of a multiple of 4 floats on 16-byte boundaries, read 16 bytes at a time; otherwise
// (any J, any alignment of a dense w) a lane reads its row float by float -- four times the load
// instructions, each touching 64 cache lines for 4 bytes apiece, which the narrowest column tile
// feels (the loads of four wavefronts then take about as long as their MFMAs) and wider ones do not.
// CT: column blocks of 32 that a unit of work contracts at once.  CTS: the workgroup's tile holds
// CTS times as many, and the units of a tile split them (see below).
// (the second launch bound keeps the register count under what 4, 3 or 2 workgroups per compute
// unit need: a few registers more and a tile of two column blocks loses its third)
template <int CT, int CTS, bool VEC>
static __global__ __launch_bounds__(kRowsThreads, CT == 1 ? (VEC ? 4 : 3) : 3) void lt2exp_rows_kernel(
    const Lt2RowsArgs p) {
    static_assert(CT * CTS <= 4 && (CTS == 1 || CTS == 2 || CTS == 4), "a tile of at most 128 columns");
    constexpr int NT = 32 * CT * CTS;
    constexpr int per_shift = CTS == 4 ? 2 : (CTS == 2 ? 1 : 0);  // units per item: a power of two, at most 4
    extern __shared__ __attribute__((aligned(16))) float lds[];
    // pitches are 4 (mod 8) floats: the 16-byte reads of 8 consecutive lanes (columns) cover all banks
    float *ebT = lds;                                      // [NT][jp]: exp(b[j, n] - mb[n]), zeros past J
    float *eaT = ebT + NT * p.jp;                          // [NT][ip]: exp(a[i, n] - ma[n]), zeros past I
    float *part = eaT + NT * p.ip;                         // [waves][s_per_group][NT]
    float *mx = part + kRowsWaves * p.s_per_group * NT;    // [2][NT]: ma, mb
    float *red = mx + 2 * NT;                              // [2][threads]

    const int tid = (int)threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int n = lane & 31, half = lane >> 5;
    int wg = (int)blockIdx.x;
    const int sg = wg % p.s_groups;
    wg /= p.s_groups;
    const int nt = wg % p.n_tiles;
    const int r = wg / p.n_tiles;
    const int k0 = nt * NT;
    const int s_begin = sg * p.s_per_group;
    const int s_count = p.S - s_begin < p.s_per_group ? p.S - s_begin : p.s_per_group;

    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;
    const float *wr = p.w + (int64_t)r * p.sw0;
    const uint32_t w_extent = (uint32_t)(((int64_t)(p.S - 1) * p.sw1 + (int64_t)p.I * p.J) * 4);
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(wr, w_extent);

    // ---- the work of this wavefront and its loads.  Item q of the workgroup is tile q % n_it of the
    // group's s number q / n_it.  A unit is an item -- or, where the workgroup holds fewer items
    // than wavefronts, one of CTS groups of column blocks of an item, so that the MFMAs of a call of
    // one or two tiles per workgroup run on all four SIMDs instead of one or two (each unit reads
    // the tile's rows of w for itself, from L1).  The wavefront takes units wave, wave + 4, ...; a
    // step is a chunk of 64 values of j of a unit.
    const int n_it = (p.I + 31) / 32;
    const int n_ch = (p.J + kRowsChunk - 1) / kRowsChunk;
    const int items = s_count * n_it;
    const int units = items << per_shift;
    const int my_units = wave < units ? (units - wave + kRowsWaves - 1) / kRowsWaves : 0;
    const int n_groups = (p.J + 7) / 8;  // groups of 8 values of j in a row
    struct Unit {
        int u, s_l, it;  // u: number of the unit in the workgroup
    };
    // (a wavefront's units all have the same column blocks: CTS divides the 4 wavefronts)
    const int cb = (wave & (CTS - 1)) * CT;  // first column block of this wavefront's units
    // (no integer division on the way from one unit to the next: it would cost as much as a
    // quarter of a short tile's MFMAs)
    auto first_unit = [&]() {
        Unit x;
        x.u = wave;
        x.s_l = 0;
        x.it = wave >> per_shift;
        while (x.it >= n_it) {
            x.it -= n_it;
            ++x.s_l;
        }
        return x;
    };
    auto next_unit = [&](const Unit &x) {
        Unit y;
        y.u = x.u + kRowsWaves;
        y.s_l = x.s_l;
        y.it = x.it + ((y.u >> per_shift) - (x.u >> per_shift));
        while (y.it >= n_it) {
            y.it -= n_it;
            ++y.s_l;
        }
        return y;
    };
    floatx4 nxt[kRowsGroups];
    auto issue = [&](const Unit &x, int ch) {
        const int s = s_begin + x.s_l, i = x.it * 32 + n;
        // (rows past I -- they belong to the next s -- are read past the extent: zeros)
        const uint32_t voff = i < p.I ? (uint32_t)(((int64_t)s * p.sw1 + (int64_t)i * p.J + 4 * half) * 4) : w_extent;
        const uint32_t soff = (uint32_t)(ch * kRowsChunk) * 4u;
        const int left = n_groups - ch * kRowsGroups;  // groups of the row from this chunk on
#pragma unroll
        for (int g = 0; g < kRowsGroups; ++g) {
            if (g < left) {
                if constexpr (VEC) {
                    nxt[g] = buf_load_f32x4(w_rsrc, voff + 32u * g, soff);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) nxt[g][e] = buf_load_f32(w_rsrc, voff + 32u * g + 4u * e, soff);
                }
            }
        }
    };
    Unit ahead = first_unit();  // the unit whose first chunk is in flight
    if (my_units > 0) issue(ahead, 0);

    // ---- column maxima of a and b over the contracted axes, then the factors (a NaN need not
    // survive the maximum: exp(NaN - m) is NaN for any m and poisons its column's sums).  A thread
    // owns a column and every G-th row; its loads go out kRowsBlock at a time -- a workgroup with
    // one or two tiles of w lives about as long as this prologue's round trips to memory take --
    // and columns of up to kRowsBlock rows per thread are kept for the factors instead of read twice.
    {
        constexpr int G = kRowsThreads / NT;  // row groups
        const int col = tid % NT, grp = tid / NT;
        const int kc = k0 + col < p.K ? k0 + col : p.K - 1;  // columns past K: computed, never stored
        const float *ac = ar + (int64_t)kc * p.sa2 + (int64_t)grp * p.sa1;
        const float *bc = br + (int64_t)kc * p.sb2 + (int64_t)grp * p.sb1;
        const int64_t a_step = (int64_t)G * p.sa1, b_step = (int64_t)G * p.sb1;
        const int i_pad = n_it * 32, j_pad = n_groups * 8;
        const int na = (p.I - grp + G - 1) / G, nb = (p.J - grp + G - 1) / G;  // rows of this thread
        const bool kept = p.I <= kRowsBlock * G && p.J <= kRowsBlock * G;       // (block-uniform)
        float va[kRowsBlock], vb[kRowsBlock];
        float m_a = -__builtin_inff(), m_b = -__builtin_inff();
        for (int base = 0; base < (kept ? 1 : (p.I + kRowsBlock * G - 1) / (kRowsBlock * G)); ++base) {
#pragma unroll
            for (int u = 0; u < kRowsBlock; ++u)
                va[u] = base * kRowsBlock + u < na ? ac[(int64_t)(base * kRowsBlock + u) * a_step] : -__builtin_inff();
#pragma unroll
            for (int u = 0; u < kRowsBlock; ++u) m_a = __builtin_fmaxf(m_a, va[u]);
        }
        for (int base = 0; base < (kept ? 1 : (p.J + kRowsBlock * G - 1) / (kRowsBlock * G)); ++base) {
#pragma unroll
            for (int u = 0; u < kRowsBlock; ++u)
                vb[u] = base * kRowsBlock + u < nb ? bc[(int64_t)(base * kRowsBlock + u) * b_step] : -__builtin_inff();
#pragma unroll
            for (int u = 0; u < kRowsBlock; ++u) m_b = __builtin_fmaxf(m_b, vb[u]);
        }
        red[tid] = m_a;
        red[kRowsThreads + tid] = m_b;
        __syncthreads();
        if (tid < 2 * NT) {  // (tid / NT: a or b)
            const float *x = red + (tid / NT) * kRowsThreads + tid % NT;
            float y = x[0];
            for (int u = 1; u < G; ++u) y = __builtin_fmaxf(y, x[u * NT]);
            mx[tid] = clamp_shift(y);
        }
        for (int u = tid; u < kRowsWaves * p.s_per_group * NT; u += kRowsThreads) part[u] = 0.f;
        __syncthreads();
        const float mak = mx[col], mbk = mx[NT + col];
        if (kept) {
#pragma unroll
            for (int u = 0; u < kRowsBlock; ++u) {
                const int i = grp + u * G, j = grp + u * G;
                if (i < i_pad) eaT[col * p.ip + i] = i < p.I ? exp_shifted(va[u] - mak) : 0.f;
                if (j < j_pad) ebT[col * p.jp + j] = j < p.J ? exp_shifted(vb[u] - mbk) : 0.f;
            }
            // (the zero rows past the kept ones: I or J just under a multiple of the padding)
            for (int i = grp + kRowsBlock * G; i < i_pad; i += G) eaT[col * p.ip + i] = 0.f;
            for (int j = grp + kRowsBlock * G; j < j_pad; j += G) ebT[col * p.jp + j] = 0.f;
        } else {
#pragma unroll 4
            for (int i = grp; i < i_pad; i += G)
                eaT[col * p.ip + i] = i < p.I ? exp_shifted(ar[(int64_t)i * p.sa1 + (int64_t)kc * p.sa2] - mak) : 0.f;
#pragma unroll 4
            for (int j = grp; j < j_pad; j += G)
                ebT[col * p.jp + j] = j < p.J ? exp_shifted(br[(int64_t)j * p.sb1 + (int64_t)kc * p.sb2] - mbk) : 0.f;
        }
    }
    __syncthreads();

    // ---- the contraction
    const bool ragged = (p.J & 7) != 0;  // the last group of 8 values of j ends past the row: zeros by selection
    float run[CT];                          // sums over the tiles of the current s
    int run_s = -1;
    const int my_cols = 32 * cb + n;
    for (int t = 0; t < my_units; ++t) {
        const Unit x = ahead;
        ahead = next_unit(x);
        const int s_l = x.s_l, it = x.it;
        floatx16 acc[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[ct][v] = 0.f;
        for (int ch = 0; ch < n_ch; ++ch) {
            floatx4 cur[kRowsGroups];
#pragma unroll
            for (int g = 0; g < kRowsGroups; ++g) cur[g] = nxt[g];
            if (ch + 1 < n_ch) issue(x, ch + 1);
            else if (t + 1 < my_units) issue(ahead, 0);
            const int left = n_groups - ch * kRowsGroups;
            const int g0 = ch * kRowsGroups;  // first group of the chunk
#pragma unroll
            for (int g = 0; g < kRowsGroups; ++g) {
                if (g < left) {
                    floatx4 av = cur[g];
                    if (ragged && g0 + g == n_groups - 1) {
                        const int room = p.J - 8 * (n_groups - 1) - 4 * half;  // values of j of this lane's piece inside the row
#pragma unroll
                        for (int e = 0; e < 4; ++e) av[e] = e < room ? av[e] : 0.f;
                    }
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        const floatx4 bv =
                            *reinterpret_cast<const floatx4 *>(&ebT[(32 * (cb + ct) + n) * p.jp + 8 * (g0 + g) + 4 * half]);
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc[ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[e], bv[e], acc[ct], 0, 0, 0);
                    }
                }
            }
        }
        // ---- the tile's rows times the factors of a, summed over i: accumulator v of a lane is
        // row 8 (v / 4) + 4 half + v % 4 of the tile, column n
        if (s_l != run_s) {
            if (run_s >= 0 && half == 0) {
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) part[(wave * p.s_per_group + run_s) * NT + 32 * ct + my_cols] = run[ct];
            }
            run_s = s_l;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) run[ct] = 0.f;
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            float sum = 0.f;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const floatx4 fa = *reinterpret_cast<const floatx4 *>(&eaT[(32 * (cb + ct) + n) * p.ip + it * 32 + 8 * g + 4 * half]);
#pragma unroll
                for (int e = 0; e < 4; ++e) sum = __builtin_fmaf(acc[ct][4 * g + e], fa[e], sum);
            }
            sum += __shfl_xor(sum, 32, kWave);
            run[ct] += sum;
        }
    }
    if (run_s >= 0 && half == 0) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) part[(wave * p.s_per_group + run_s) * NT + 32 * ct + my_cols] = run[ct];
    }
    __syncthreads();

    // ---- the wavefronts' sums in a fixed order, shift back, log, store
    for (int u = tid; u < s_count * NT; u += kRowsThreads) {
        const int s_l = u / NT, col = u % NT;
        if (k0 + col >= p.K) continue;
        float sum = part[s_l * NT + col];
#pragma unroll
        for (int wv = 1; wv < kRowsWaves; ++wv) sum += part[(wv * p.s_per_group + s_l) * NT + col];
        p.c[(int64_t)r * p.sc0 + (int64_t)(s_begin + s_l) * p.sc1 + k0 + col] = log_plus(sum, mx[col] + mx[NT + col]);
    }
}

// ---- host side

constexpr size_t kRowsMaxLds = 64 * 1024;        // (two workgroups on a compute unit)
constexpr size_t kRowsMaxLdsNarrow = 144 * 1024;  // the narrowest column tile may take a compute unit for itself

static inline int rows_pitch(int64_t len, int64_t unit) { return (int)(ceil_div(len, unit) * unit + 4); }
static inline size_t rows_lds_bytes(int64_t I, int64_t J, int ct, int s_per_group) {
    const size_t nt = 32 * (size_t)ct;
    return (nt * (size_t)(rows_pitch(J, 8) + rows_pitch(I, 32)) + (size_t)kRowsWaves * s_per_group * nt + 2 * nt +
            2 * kRowsThreads) * sizeof(float);
}

struct RowsPlan {
    int ct, s_per_group;  // column blocks of the workgroup's tile (0: the kernel does not apply), s per workgroup
    bool vec;             // 16-byte loads of w
    int cts;              // a tile's work cut into cts groups of column blocks (fewer tiles than wavefronts)
};

// Column tile and s per workgroup.  The widest column tile that K fills and LDS holds (w is read
// once per column tile); then as many s per workgroup as leave the grid two workgroups per
// compute unit, where the batch and column tiles alone do not.
static inline RowsPlan rows_plan(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_aligned,
                                 bool w_dense = true) {
    RowsPlan none = {0, 0, false, 1};
    if (!w_dense || J < 8) return none;
    const bool vec = w_aligned && J % 4 == 0;
    int ct = K > 64 ? 4 : (K > 32 ? 2 : 1);
    int spg = (int)(S < kRowsMaxS ? S : kRowsMaxS);
    while (ct > 1 && rows_lds_bytes(I, J, ct, spg) > kRowsMaxLds) ct /= 2;
    if (rows_lds_bytes(I, J, ct, spg) > kRowsMaxLdsNarrow) return none;
    const int64_t n_it = ceil_div(I, 32);
    const int64_t base = R * ceil_div(K, 32 * ct);
    while (spg > 1 && base * ceil_div(S, spg) < 512 && (int64_t)(spg / 2) * n_it >= 8) spg /= 2;
    // fewer tiles than wavefronts in a workgroup: cut a tile's work by column blocks (R=4096, S=1,
    // I=J=32, K=100: 121 -> 48 us; R=2048, S=1, I=J=64, K=256: 144 -> 120).  Cutting the range of j
    // as well, for tiles of a single column block, was slower (K=12: 24 -> 27 us): not done.
    int cts = 1;
    while ((int64_t)spg * n_it * cts < kRowsWaves && cts < ct) cts *= 2;
    return RowsPlan{ct, spg, vec, cts};
}

// Is this kernel the faster one?  Fitted to 1100 timed shapes (S = 1..256, I = 4..512, J = 8..512,
// K = 9..2048, up to 300 MB of w; a quarter of them with J not a multiple of 4) as the sign of a
// linear score in log2 units -- the estimate of log2(time of the s-row tiles / time of this kernel):
//   + per doubling of the padding of s to 32 rows there (0.5, not 1: small calls are bound by
//     latencies on both sides),
//   - 0.65 per doubling of the padding of i to 32 rows here,
//   - 0.18 per doubling of K (more column tiles fill the grid of the s-row tiles),
//   - per halving of J below 32 (the epilogue of a tile, 16 FMAs and 4 LDS reads per column
//     block, against J / 2 MFMAs),
// and, from 13 values of s on, where the padding of s no longer decides, - 0.12 per doubling of
// the work and + 0.25 per halving of K below 64: the s-row tiles run large grids at 100-125
// TFLOP/s, this kernel at 60-95, but a call of less than about a GFLOP is faster here whatever S
// is (R=1, S=I=J=K=128: 30 -> 15 us), and under 64 columns most of the four wavefronts that the
// s-row tiles set side by side over 128 columns stand idle (R=2048, S=16, I=J=64, K=32: 509 ->
// 127 us; S=32, I=J=32, K=32: 137 -> 78).  Such calls need the estimate to favour this kernel by
// 10 % (which keeps calls of a few GFLOP under thousands of columns, where the two run level, on
// the tiles tuned for them).
// Taking the kernel by this rule costs 2.5-3 % over the faster of the two per shape (geometric
// mean over the fit's shapes; never taking it 68 % -- 154 % over the shapes with S <= 12, 23 % over
// 400 shapes with S = 13..128 and K up to 512 --, always taking it 14 %).  The element-load build
// is served by the same rule (the s-row tiles stage such rows element by element too).  Outputs
// of at most 8 columns have been handed to the sweep before this is asked.
static inline double rows_score(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K) {
    const double ws = std::log2(32.0 * (double)ceil_div(S, 32) / (double)S);
    const double wi = std::log2(32.0 * (double)ceil_div(I, 32) / (double)I);
    const double lj = std::log2((double)J), lk = std::log2((double)K);
    const double short_j = lj < 5.0 ? 5.0 - lj : 0.0;
    if (S <= 12) return 1.41 + 0.52 * ws - 0.65 * wi - 0.18 * lk - 0.22 * short_j;
    const double lw = std::log2(2.0 * (double)R * (double)S * (double)I * (double)J * (double)K);
    return 3.62 + 0.36 * ws - 0.65 * wi - 0.27 * short_j - 0.12 * lw + 0.25 * (lk < 6.0 ? 6.0 - lk : 0.0);
}
static inline bool rows_pays(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K) {
    return rows_score(R, S, I, J, K) > 0.0;
}

static int launch_lt2exp_rows(const float *w, const float *a, const float *b, float *c, int64_t R, int64_t S, int64_t I,
                              int64_t J, int64_t K, const int64_t sw[3], const int64_t sa[3], const int64_t sb[3],
                              const int64_t sc[3], const RowsPlan plan, hipStream_t stream) {
    Lt2RowsArgs args;
    args.w = w; args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.S = (int)S; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sw0 = sw[0]; args.sw1 = sw[1];
    args.sa0 = sa[0]; args.sa1 = sa[1]; args.sa2 = sa[2];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.n_tiles = (int)ceil_div(K, 32 * plan.ct);
    args.s_per_group = plan.s_per_group;
    args.s_groups = (int)ceil_div(S, plan.s_per_group);
    args.jp = rows_pitch(J, 8);
    args.ip = rows_pitch(I, 32);
    const int64_t grid = R * args.n_tiles * args.s_groups;
    if (grid >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    const size_t lds = rows_lds_bytes(I, J, plan.ct, plan.s_per_group);
    // (more than 64 KB of LDS must be allowed per kernel and device, once: the first such launch
    // on a device makes that call, every later one -- one inside a stream capture, say -- does not)
    auto launch = [&](auto kernel) -> int {
        if (lds > kRowsMaxLds) {  // (only the narrowest tile goes there)
            static std::atomic<uint64_t> allowed{0};  // (per instance of the kernel: a bit per device)
            int device = 0;
            if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return TRT_E_INVALID;
            if (!(allowed.load(std::memory_order_acquire) >> device & 1)) {
                const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kRowsMaxLdsNarrow);
                if (e != hipSuccess) return (int)e;
                allowed.fetch_or((uint64_t)1 << device, std::memory_order_release);
            }
        }
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kRowsThreads), lds, stream, args);
        return 0;
    };
    int err;
    const int unit_ct = plan.ct / plan.cts;  // column blocks that a unit contracts at once: the kernel's CT
#define TRT_ROWS_LAUNCH(CT_, CTS_) \
    (plan.vec ? launch(&lt2exp_rows_kernel<CT_, CTS_, true>) : launch(&lt2exp_rows_kernel<CT_, CTS_, false>))
    if (plan.cts == 1) err = unit_ct == 1 ? TRT_ROWS_LAUNCH(1, 1) : (unit_ct == 2 ? TRT_ROWS_LAUNCH(2, 1) : TRT_ROWS_LAUNCH(4, 1));
    else if (plan.cts == 2) err = unit_ct == 1 ? TRT_ROWS_LAUNCH(1, 2) : TRT_ROWS_LAUNCH(2, 2);
    else err = TRT_ROWS_LAUNCH(1, 4);
#undef TRT_ROWS_LAUNCH
    if (err) return err;
    return (int)hipGetLastError();
}

}  // namespace trt
