// lt2exp on the bf16 matrix pipe of gfx950, fp32 in and out:
//   c[r,s,k] = log sum_{i,j} w[r,s,i,j] exp(a[r,i,k]) exp(b[r,j,k])
//
// The reference has a reduced-precision mode (TF32 operands, triturus/utils.py:33-44,
// passed to tl.dot at triturus/lt2exp.py:344); gfx950 has no TF32 matrix instruction.
// Its bf16 matrix pipe is 16x faster than the fp32 one, so each fp32 operand is cut
// into NS bf16 pieces (x = x0 + x1 [+ x2], each the bf16 rounding of what the previous
// pieces left) and a product is the sum of the piece products that matter:
//   NS = 2:  x0 y0 + x0 y1 + x1 y0                        3 MFMAs, error ~2^-16 per product
//   NS = 3:  ... + x0 y2 + x1 y1 + x2 y0                  6 MFMAs, error ~2^-23 per product
// accumulated in fp32 by v_mfma_f32_32x32x16_bf16.  Unlike the fp32 MFMA, the bf16 MFMA
// runs beside the vector ALU, so the splitting work is hidden as long as it is shorter
// than the MFMAs it feeds.  To keep it short the Khatri-Rao product is never formed:
//   sum_{i,j} w[s,i,j] ea[i,n] eb[j,n] = sum_i ea[i,n] * ( sum_j w[s,i,j] eb[j,n] )
// so the B operand is eb alone (split once per column tile and j-chunk, reused for every
// i) and the per-i factor ea[i,n] scales the 32 x 32 result tile of each i on its way
// into the running sum (one fma per accumulator register, in fp32).
//
// Tiling as in the fp32 kernel: a workgroup of 4 wavefronts owns 32*RT rows of S and 128
// columns of K, a wavefront 32 of those columns for all rows; w tiles go global ->
// registers -> split -> LDS (double buffered).  (A 2 x 2 arrangement of the wavefronts,
// which halves the LDS reads per MFMA, was measured slower: it needs the B pieces of two
// column tiles in registers and spills.)  MFMA k-slot mapping: element e of lane-half h in k-step ks
// of a chunk is j = 16 ks + 8 h + e for both operands.

#include "bf16_split.hpp"
#include "lt2exp_merge.hpp"

namespace trt {

struct Lt2BfArgs {
    const float *w, *a, *b;
    float *c;      // output (unsplit) -- or partial sums [splits][R][S][K] (split)
    float *shift;  // split only: [2][R][K] clamped column maxima
    int R, S, I, J, K;
    int64_t sw0, sw1, sa0, sa1, sb0, sb1, sc0, sc1;
    int64_t sa2, sb2;  // trailing strides of a and b (a lane owns a column: they only scale lane offsets)
    int64_t sw2;       // stride of the flat (i, j) axis of w: other than 1 in the builds without 16-byte loads only
    int s_tiles, n_tiles, splits;
    int iters_per_split;  // (j-chunk, i) iterations per split
    int stream_out;       // rows of c are 16-byte aligned: non-temporal result stores
    int64_t total_wgs, padded_wgs;
};

template <int RT, int KS, int NS, bool VEC, bool SPLIT = false>
__global__ __launch_bounds__(256, 2) void lt2exp_bf16_kernel(const Lt2BfArgs p) {
    constexpr int NT = 256;
    constexpr int TS = 32 * RT;    // rows of S per workgroup
    constexpr int JC = 16 * KS;    // j per chunk
    constexpr int LDA = JC + 8;    // padded LDS row in bf16 (16 bytes of padding: conflict-free 16-byte reads)
    constexpr int F4_PER_ROW = JC / 4;
    constexpr int F4_TILE = TS * F4_PER_ROW;        // 16-byte pieces of a w tile (fp32)
    constexpr int SLOTS = (F4_TILE + NT - 1) / NT;  // of which a thread stages this many
    // REGULAR: a thread keeps its column and steps whole rows from slot to slot; otherwise
    // (chunks of 48, tiles smaller than the workgroup) pieces are dealt out linearly and the
    // last slot is only partly filled.
    constexpr bool REGULAR = (NT % F4_PER_ROW == 0) && (F4_TILE % NT == 0);
    constexpr int TN = 128;

    // (a thread whose last slot lies past the tile stages into a private 8 bytes behind it: the
    // steady state carries no predicates)
    __shared__ __attribute__((aligned(16))) __bf16 wt[2][NS][TS * LDA + (REGULAR ? 0 : 4 * NT)];

    const int64_t L = xcd_logical_id(blockIdx.x, p.padded_wgs);
    if (L >= p.total_wgs) return;
    int64_t rest = L / p.n_tiles;
    const int nt = __builtin_amdgcn_readfirstlane((int)(L % p.n_tiles));
    const int split = SPLIT ? __builtin_amdgcn_readfirstlane((int)(rest % p.splits)) : 0;
    if (SPLIT) rest /= p.splits;
    const int st = __builtin_amdgcn_readfirstlane((int)(rest % p.s_tiles));
    const int r = __builtin_amdgcn_readfirstlane((int)(rest / p.s_tiles));

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    const int h = lane / 32;
    const int m = lane % 32;
    const int s0 = st * TS;
    const int ncol = nt * TN + wave * 32 + m;
    const int ncl = ncol < p.K ? ncol : p.K - 1;

    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;
    const float *wr = p.w + (int64_t)r * p.sw0;

    // ---- clamped column maxima (baselines/lt2exp.py:15-19): the lane halves take
    // alternate rows and exchange once
    float x = -__builtin_inff();
#pragma unroll 8
    for (int i = h; i < p.I; i += 2) x = __builtin_fmaxf(x, ar[(int64_t)i * p.sa1 + (int64_t)ncl * p.sa2]);
    x = __builtin_fmaxf(x, __shfl_xor(x, 32, kWave));
    const float ma = clamp_shift(x);
    float y = -__builtin_inff();
#pragma unroll 8
    for (int j = h; j < p.J; j += 2) y = __builtin_fmaxf(y, br[(int64_t)j * p.sb1 + (int64_t)ncl * p.sb2]);
    y = __builtin_fmaxf(y, __shfl_xor(y, 32, kWave));
    const float mb = clamp_shift(y);

    // (j-chunk, i) iterations of this workgroup: all of them, or one split's share
    const int n_jc = (p.J + JC - 1) / JC;
    const int it0 = SPLIT ? split * p.iters_per_split : 0;
    int it1 = SPLIT ? it0 + p.iters_per_split : n_jc * p.I;
    if (it1 > n_jc * p.I) it1 = n_jc * p.I;
    const int total_iters = it1 - it0;

    floatx16 total[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) total[rt][v] = 0.f;

    // ---- w tile staging: a buffer resource whose extent ends at the last valid row (rows
    // past S read as zeros), 32-bit lane offsets, the (i, j-chunk) offset in a scalar.
    floatx4 stage[SLOTS];
    int srow[SLOTS], sc4[SLOTS];  // tile row and 16-byte column of each slot
    int lds_off[SLOTS];           // where the slot goes in the LDS tile (bf16 elements)
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
        lds_off[sidx] = sval[sidx] ? srow[sidx] * LDA + 4 * sc4[sidx] : TS * LDA + 4 * tid;
    }
    const int wrows = (p.S - s0) < TS ? (p.S - s0) : TS;
    const float *wtile0 = wr + (int64_t)s0 * p.sw1;
    const __amdgpu_buffer_rsrc_t w_rsrc =
        make_rsrc(wtile0, (uint32_t)(((int64_t)(wrows - 1) * p.sw1 + ((int64_t)p.I * p.J - 1) * p.sw2 + 1) * 4));
    uint32_t woff[SLOTS];
#pragma unroll
    for (int sidx = 0; sidx < SLOTS; ++sidx)
        woff[sidx] = ((uint32_t)srow[sidx] * (uint32_t)p.sw1 + 4u * (uint32_t)sc4[sidx] * (uint32_t)p.sw2) * 4u;
    // pair-wise staging of the unaligned build (chunks that divide the workgroup evenly)
    constexpr bool ELEM = !VEC && (NT % (JC / 2) == 0) && ((TS * JC / 2) % NT == 0) && (TS * JC / 2 / NT <= 2 * SLOTS);
    constexpr int NP = ELEM ? TS * JC / 2 / NT : 1;  // column pairs per thread
    const int ecp = tid % (JC / 2);
    const uint32_t ebase = ((uint32_t)(tid / (JC / 2)) * (uint32_t)p.sw1 + 2u * (uint32_t)ecp * (uint32_t)p.sw2) * 4u;
    const uint32_t wcol_bytes = (uint32_t)p.sw2 * 4u;  // one element of the flat axis further (4 in the builds with 16-byte loads)
    auto load_tile = [&](int i, int jc) __attribute__((always_inline)) {
        const uint32_t soff = (uint32_t)(i * p.J + jc * JC) * wcol_bytes;
        const bool full = VEC && (jc * JC + JC <= p.J);  // wave-uniform
        if (full) {
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) stage[sidx] = buf_load_f32x4(w_rsrc, woff[sidx], soff);
        } else if (VEC) {
            // ragged last chunk of aligned rows (J is a multiple of 4): a 16-byte piece is whole
            // or lies past J, where the next i begins: zeros instead
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) {
                const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
                const floatx4 v = buf_load_f32x4(w_rsrc, woff[sidx], soff);
                stage[sidx] = (jc * JC + 4 * sc4[sidx] < p.J) ? v : zero;
            }
        } else if (ELEM) {
            // rows that are not 16-byte aligned: a thread takes pairs of adjacent columns (one
            // register of two bf16 per piece afterwards), consecutive lanes consecutive pairs, its
            // pairs NT / (JC / 2) rows apart (scalar offsets); what lies past J reads as zero
            const bool in0 = jc * JC + 2 * ecp < p.J, in1 = jc * JC + 2 * ecp + 1 < p.J;
#pragma unroll
            for (int e = 0; e < NP; ++e) {
                const uint32_t so = soff + (uint32_t)(e * (2 * NT / JC)) * (uint32_t)p.sw1 * 4u;
                const float v0 = buf_load_f32(w_rsrc, ebase, so), v1 = buf_load_f32(w_rsrc, ebase + wcol_bytes, so);
                stage[e / 2][2 * (e % 2)] = in0 ? v0 : 0.f;
                stage[e / 2][2 * (e % 2) + 1] = in1 ? v1 : 0.f;
            }
        } else {
            // ragged chunk or unaligned rows: element loads; what lies past J belongs to the
            // next i (or is outside the extent) and is replaced by zero
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) {
                const int j = jc * JC + 4 * sc4[sidx];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = buf_load_f32(w_rsrc, woff[sidx] + wcol_bytes * e, soff);
                    stage[sidx][e] = (j + e < p.J) ? v : 0.f;
                }
            }
        }
    };
    // split the staged fp32 values and write the pieces to LDS (8 bytes per piece and slot)
    auto store_tile = [&](int buf) __attribute__((always_inline)) {
        if (ELEM) {
#pragma unroll
            for (int e = 0; e < NP; ++e) {
                uint32_t pk[NS];
                split_pair<NS, false>(stage[e / 2][2 * (e % 2)], stage[e / 2][2 * (e % 2) + 1], pk);
                const int off = (tid / (JC / 2) + e * (2 * NT / JC)) * LDA + 2 * ecp;
#pragma unroll
                for (int sp = 0; sp < NS; ++sp) *reinterpret_cast<uint32_t *>(&wt[buf][sp][off]) = pk[sp];
            }
            return;
        }
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) {
            uint32_t p01[NS], p23[NS];
            split_pair<NS, false>(stage[sidx][0], stage[sidx][1], p01);
            split_pair<NS, false>(stage[sidx][2], stage[sidx][3], p23);
#pragma unroll
            for (int sp = 0; sp < NS; ++sp) {
                uintx2 v = {p01[sp], p23[sp]};
                *reinterpret_cast<uintx2 *>(&wt[buf][sp][lds_off[sidx]]) = v;
            }
        }
    };

    const __amdgpu_buffer_rsrc_t a_rsrc =
        make_rsrc(ar, (uint32_t)(((int64_t)(p.I - 1) * p.sa1 + (int64_t)(p.K - 1) * p.sa2 + 1) * 4));
    const uint32_t a_row_bytes = (uint32_t)p.sa1 * 4u;
    const uint32_t aoff = (uint32_t)ncl * (uint32_t)p.sa2 * 4u;

    // B operand: exp(b[j,n] - mb[n]) of the current j-chunk, split, in MFMA layout
    uintx4 ebp[NS][KS];
    auto load_eb = [&](int jc) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            float e[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = jc * JC + 16 * ks + 8 * h + u;
                float raw = -__builtin_inff();
                if (j < p.J) raw = br[(int64_t)j * p.sb1 + (int64_t)ncl * p.sb2];
                e[u] = exp_shifted(raw - mb);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                uint32_t pk[NS];
                split_pair<NS, true>(e[2 * u], e[2 * u + 1], pk);
#pragma unroll
                for (int sp = 0; sp < NS; ++sp) ebp[sp][ks][u] = pk[sp];
            }
        }
    };

    if (total_iters > 0) {
        int jc = it0 / p.I;
        int i = it0 - jc * p.I;
        load_tile(i, jc);
        load_eb(jc);
        float ea = exp_shifted(ar[(int64_t)i * p.sa1 + (int64_t)ncl * p.sa2] - ma);
        float ea_raw;
        store_tile(0);
        __syncthreads();

        // ---- one (i, j-chunk) and row tile: inner = w tile x eb (3 or 6 MFMAs per k-step,
        // starting from zero), then total += ea[i,n] * inner
        auto mfma_rows = [&](int buf, int rt, floatx16 &inn) __attribute__((always_inline)) {
            bool first = true;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8 af[NS];
#pragma unroll
                for (int sp = 0; sp < NS; ++sp)
                    af[sp] = *reinterpret_cast<const bf16x8 *>(&wt[buf][sp][(32 * rt + m) * LDA + 16 * ks + 8 * h]);
#pragma unroll
                for (int sa = 0; sa < NS; ++sa)
#pragma unroll
                    for (int sb = 0; sa + sb < NS; ++sb) {
                        const bf16x8 bop = __builtin_bit_cast(bf16x8, ebp[sb][ks]);
                        if (first) {
                            const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f,
                                                   0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                            inn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[sa], bop, zero, 0, 0, 0);
                        } else {
                            inn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[sa], bop, inn, 0, 0, 0);
                        }
                        first = false;
                    }
            }
        };
        // The empty asm pins the fmas to this place in the instruction stream: their results
        // are not needed before the next step, and the compiler would otherwise sink them
        // out of the MFMA block they are meant to overlap with.
        auto scale_add = [&](floatx16 &tot, const floatx16 &inn, float e) __attribute__((always_inline)) {
#pragma unroll
            for (int v = 0; v < 16; ++v) tot[v] = __builtin_fmaf(inn[v], e, tot[v]);
            asm volatile("" : "+v"(tot));
        };

        int cur = 0;
        if constexpr (RT == 2) {
            // Two half-steps per (i, j-chunk).  While the MFMAs of row tile 0 run, the vector
            // ALU adds the previous step's row tile 1 into the running sum; while those of
            // row tile 1 run, it adds row tile 0 and splits the prefetched w tile.
            floatx16 inner0, inner1;
#pragma unroll
            for (int v = 0; v < 16; ++v) inner1[v] = 0.f;
            float ea_old = 0.f;
            for (int it = 0; it + 1 < total_iters; ++it) {
                int ni = i + 1, njc = jc;
                if (ni == p.I) {
                    ni = 0;
                    njc = jc + 1;
                }
                load_tile(ni, njc);
                ea_raw = buf_load_f32(a_rsrc, aoff, (uint32_t)ni * a_row_bytes);
                __builtin_amdgcn_sched_barrier(0);
                mfma_rows(cur, 0, inner0);
                scale_add(total[1], inner1, ea_old);
                __builtin_amdgcn_sched_barrier(0);
                mfma_rows(cur, 1, inner1);
                scale_add(total[0], inner0, ea);
                store_tile(cur ^ 1);
                __builtin_amdgcn_sched_barrier(0);
                ea_old = ea;
                if (njc != jc) load_eb(njc);
                ea = exp_shifted(ea_raw - ma);
                __syncthreads();
                cur ^= 1;
                i = ni;
                jc = njc;
            }
            mfma_rows(cur, 0, inner0);
            scale_add(total[1], inner1, ea_old);
            mfma_rows(cur, 1, inner1);
            scale_add(total[0], inner0, ea);
            scale_add(total[1], inner1, ea);
        } else {
            // One row tile: the same overlap with two result tiles in turn.  While the MFMAs of
            // this step fill one, the vector ALU adds the other (the previous step's) into the
            // running sum; steps are taken in pairs so that both live in fixed registers.
            floatx16 inner_a, inner_b;
#pragma unroll
            for (int v = 0; v < 16; ++v) inner_b[v] = 0.f;
            float ea_old = 0.f;
            auto step = [&](floatx16 &inner_cur, const floatx16 &inner_old) __attribute__((always_inline)) {
                int ni = i + 1, njc = jc;
                if (ni == p.I) {
                    ni = 0;
                    njc = jc + 1;
                }
                load_tile(ni, njc);
                ea_raw = buf_load_f32(a_rsrc, aoff, (uint32_t)ni * a_row_bytes);
                __builtin_amdgcn_sched_barrier(0);
                mfma_rows(cur, 0, inner_cur);
                scale_add(total[0], inner_old, ea_old);
                store_tile(cur ^ 1);
                __builtin_amdgcn_sched_barrier(0);
                ea_old = ea;
                if (njc != jc) load_eb(njc);
                ea = exp_shifted(ea_raw - ma);
                __syncthreads();
                cur ^= 1;
                i = ni;
                jc = njc;
            };
            const int steps = total_iters - 1;  // every step but the last prefetches its successor
            int done = 0;
            for (; done + 2 <= steps; done += 2) {
                step(inner_a, inner_b);
                step(inner_b, inner_a);
            }
            if (done < steps) {
                step(inner_a, inner_b);
                mfma_rows(cur, 0, inner_b);
                scale_add(total[0], inner_a, ea_old);
                scale_add(total[0], inner_b, ea);
            } else {
                mfma_rows(cur, 0, inner_a);
                scale_add(total[0], inner_b, ea_old);
                scale_add(total[0], inner_a, ea);
            }
        }
    }

    // ---- epilogue: register v of lane (h, m) holds row 8*(v/4) + 4*h + v%4, column m
    if (ncol >= p.K) return;
    if (SPLIT) {
        // raw partial sums; all splits share ma, mb (they depend on the column only)
        float *part = p.c + ((int64_t)split * p.R + r) * (int64_t)p.S * p.K;
        if (split == 0 && st == 0 && h == 0) {
            p.shift[(int64_t)r * p.K + ncol] = ma;
            p.shift[((int64_t)p.R + r) * p.K + ncol] = mb;
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = s0 + 32 * rt + 8 * (v / 4) + 4 * h + (v % 4);
                if (row < p.S) part[(int64_t)row * p.K + ncol] = total[rt][v];
            }
        return;
    }
    const int crows = p.S - s0;
    const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(p.c + (int64_t)r * p.sc0 + (int64_t)s0 * p.sc1,
                                                    (uint32_t)(((int64_t)(crows - 1) * p.sc1 + p.K) * 4));
    const uint32_t c_row_bytes = (uint32_t)p.sc1 * 4u;
    const float mm = ma + mb;
    const uint32_t co = ((uint32_t)(4 * h) * (uint32_t)p.sc1 + (uint32_t)ncol) * 4u;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t trow_c = 32 * rt + 8 * (v / 4) + (v % 4);
            buf_store_f32_out(p.stream_out != 0, log_plus(total[rt][v], mm), c_rsrc, co, trow_c * c_row_bytes);
        }
}

template <int RT, int KS, int NS>
static void launch_bf(const Lt2BfArgs &args, bool vec, bool split, hipStream_t stream) {
    const dim3 grid((unsigned)args.padded_wgs), block(256);
    if (vec) {
        if (split) hipLaunchKernelGGL((lt2exp_bf16_kernel<RT, KS, NS, true, true>), grid, block, 0, stream, args);
        else hipLaunchKernelGGL((lt2exp_bf16_kernel<RT, KS, NS, true, false>), grid, block, 0, stream, args);
    } else {
        if (split) hipLaunchKernelGGL((lt2exp_bf16_kernel<RT, KS, NS, false, true>), grid, block, 0, stream, args);
        else hipLaunchKernelGGL((lt2exp_bf16_kernel<RT, KS, NS, false, false>), grid, block, 0, stream, args);
    }
}

template <int NS>
static void launch_bf_shape(const Lt2BfArgs &args, int rt, int ks, bool vec, bool split, hipStream_t stream) {
    if (rt == 2) {
        if (ks == 4) launch_bf<2, 4, NS>(args, vec, split, stream);
        else if (ks == 3) launch_bf<2, 3, NS>(args, vec, split, stream);
        else if (ks == 2) launch_bf<2, 2, NS>(args, vec, split, stream);
        else launch_bf<2, 1, NS>(args, vec, split, stream);
    } else {
        if (ks == 4) launch_bf<1, 4, NS>(args, vec, split, stream);
        else if (ks == 3) launch_bf<1, 3, NS>(args, vec, split, stream);
        else if (ks == 2) launch_bf<1, 2, NS>(args, vec, split, stream);
        else launch_bf<1, 1, NS>(args, vec, split, stream);
    }
}

bool lt2exp_takes_sweep(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_aligned, bool w_dense);  // csrc/lt2exp.hip
bool lt2exp_takes_rows(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_aligned, bool w_dense, double margin);  // csrc/lt2exp.hip
bool lt2exp_takes_cols(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, bool w_dense, double margin);  // csrc/lt2exp.hip

}  // namespace trt

using namespace trt;

// j-chunk (in units of 16) that costs least: padded length of the contraction x cost per padded
// j, measured at S = I = 64, K = 4096, R = 64 with J = 16..144 on 64-row tiles: chunks of 64 cost
// 5.4 us per j with two pieces (9.2 with three), chunks of 48 2 % (4 %) more, of 32 8 % (4 %)
// more, of 16 28 % (13 %) more -- and far more on grids that are latency bound (R = 128,
// S = I = J = 48, K = 256: 85 against 52 us), hence their 35 % (25 %).  Against chunks of 32 or 64
// alone J = 16 runs 2.6x (1.9x) faster, J = 48 1.7x (1.4x), J = 144 1.2x (1.1x).
// When J is not a multiple of 4 every chunk takes element loads, which chunks of 16 bear worst
// (1.9x per padded j over 50 random shapes; 32 and 48 cost 5 % more than 64).
static int bf16_chunk(int64_t J, int pieces) {
    const int64_t penalty[3][4] = {{135, 108, 102, 100}, {125, 104, 104, 100}, {150, 105, 130, 100}};
    const int row = J % 4 != 0 ? 2 : (pieces == 2 ? 0 : 1);
    int best_ks = 4;
    int64_t best = 0;
    for (int ks = 4; ks >= 1; --ks) {
        const int64_t cost = ceil_div(J, 16 * ks) * 16 * ks * penalty[row][ks - 1];
        if (ks == 4 || cost < best) {
            best = cost;
            best_ks = ks;
        }
    }
    return best_ks;
}

// Split count the bf16 path would like for a small grid (32-row tiles): 1 = none.
static int64_t bf16_small_grid_splits(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int pieces, int mode) {
    if (mode == TRT_MODE_UNSPLIT) return 1;
    const int ks = bf16_chunk(J, pieces);
    const int64_t iters = ceil_div(J, 16 * ks) * I;
    const int64_t tiles = R * ceil_div(S, 32) * ceil_div(K, 128);
    if (mode != TRT_MODE_SPLIT && tiles >= 1024) return 1;  // four workgroups per CU: matrix bound as it is
    // The model counts steps in fp32 MFMAs (64 cycles).  A step of this kernel is ks x 3 (or 6) bf16
    // MFMAs of 32 cycles, but on a CU that holds one or two workgroups the splitting and scaling
    // around them is not hidden: measured 0.9 us per step alone on a CU with ks = 4 and two pieces,
    // which the model reproduces with 5/4 of an fp32 MFMA per bf16 MFMA.
    return choose_splits(tiles, iters, (int64_t)ks * (pieces == 2 ? 3 : 6) * 5 / 4, R * S * K, 4, 32,
                         mode == TRT_MODE_SPLIT);
}

static bool bf16_small_grid(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode) {
    const int64_t t32 = R * ceil_div(S, 32) * ceil_div(K, 128);
    return mode == TRT_MODE_SPLIT || t32 < 160 || (t32 <= 256 && I * J > 4096);
}

// Workspace the bf16 entry wants beyond what trt_lt2exp_workspace_bytes reports for the same
// call (callers pass the larger of the two): room for its own cut of a small grid.
extern "C" size_t trt_lt2exp_bf16_workspace_bytes(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int pieces,
                                                  int mode) {
    if (R <= 0 || S <= 0 || I <= 0 || J <= 0 || K <= 0 || (pieces != 2 && pieces != 3)) return 0;
    int64_t splits = bf16_small_grid_splits(R, S, I, J, K, pieces, mode);
    if (J == 1 && I > 1) {  // may run with i and j exchanged (trt_lt2exp_bf16): room for either
        const int64_t swapped = bf16_small_grid_splits(R, S, 1, I, K, pieces, mode);
        if (swapped > splits) splits = swapped;
    }
    return splits >= 2 ? ((size_t)splits * R * S * K + (size_t)2 * R * K) * sizeof(float) : 0;
}

extern "C" int trt_lt2exp_bf16(const float *w, const float *a, const float *b, float *c, int64_t R, int64_t S,
                               int64_t I, int64_t J, int64_t K, const int64_t sw[3], const int64_t sa[3],
                               const int64_t sb[3], const int64_t sc[3], int pieces, int mode, int variant,
                               void *workspace, size_t workspace_bytes, void *stream) {
    if (!w || !a || !b || !c || !sw || !sa || !sb || !sc) return TRT_E_INVALID;
    if (R <= 0 || S <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (pieces != 2 && pieces != 3) return TRT_E_INVALID;
    if (mode != TRT_MODE_AUTO && mode != TRT_MODE_SPLIT && mode != TRT_MODE_UNSPLIT) return TRT_E_INVALID;
    if (variant < 0 || variant > 16) return TRT_E_INVALID;
    if (sw[2] < 0 || sa[2] < 0 || sb[2] < 0 || sc[2] != 1) return TRT_E_LAYOUT;
    for (int d = 0; d < 2; ++d)
        if (sw[d] < 0 || sa[d] < 0 || sb[d] < 0 || sc[d] < 0) return TRT_E_LAYOUT;
    if (sc[1] < K) return TRT_E_LAYOUT;
    const int64_t lim = (int64_t)1 << 30;
    if (R >= lim || S >= lim || I >= lim || J >= lim || K >= lim || I * J >= lim) return TRT_E_RANGE;
    if (S * sw[1] + I * J * (sw[2] > 0 ? sw[2] : 1) >= lim || I * sa[1] + K * sa[2] >= lim || J * sb[1] + K * sb[2] >= lim || S * sc[1] + K >= lim)
        return TRT_E_RANGE;

    // a single j under several i: run with the roles of (i, a) and (j, b) exchanged (see trt_lt2exp_f32)
    if (J == 1 && I > 1 && variant == 0)
        return trt_lt2exp_bf16(w, b, a, c, R, S, 1, I, K, sw, sb, sa, sc, pieces, mode, variant, workspace,
                               workspace_bytes, stream);

    // Outputs of at most 8 columns are a sweep over w, which the fp32 entry runs on the vector ALU
    // (csrc/lt2exp_smallk.hpp): the matrix pipe has nothing to gain there.
    if (variant == 0 && K <= 8 &&
        lt2exp_takes_sweep(R, S, I, J, K, sw[2] == 1 && sw[0] % 4 == 0 && sw[1] % 4 == 0 &&
                                              (reinterpret_cast<uintptr_t>(w) & 15) == 0, sw[2] == 1))
        return trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, 0, workspace, workspace_bytes, stream);

    // Layers of few units over many batches (I, J <= 16): what the fp32 entry gives to its kernel
    // with a lane per output column (csrc/lt2exp_cols.hpp) is bound by memory there, and these tiles
    // pad such calls as the fp32 ones do (150 timed shapes that the fp32 rule takes: 1.36x and 1.27x
    // behind it in the geometric mean with two and three pieces; handing all of them over leaves
    // 1.8 % to the better choice per shape).
    if (variant == 0 && lt2exp_takes_cols(R, S, I, J, K, sw[2] == 1, 0.0))
        return trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, 0, workspace, workspace_bytes, stream);

    // Few s per batch: these tiles, like the fp32 ones, put s on the rows of the MFMA and pad it to
    // 32; the fp32 kernel of csrc/lt2exp_rows.hpp puts the rows (s, i) of w there -- and is the more
    // exact of the two.  It is taken where the fp32 rule's score (log2 of the estimated gain over the
    // fp32 s-row tiles) exceeds a margin fitted to 260 shapes timed on all three paths: up to 12
    // values of s 0.6 against two pieces and 0.4 against three (3.0 and 0.7 % behind the better
    // choice per shape; never handing over 56 and 100 %), beyond that -- calls of little work, bound
    // by latencies in either kernel -- 0.2 and 0 (3.4 and 3.7 %; never 6 and 11 %).
    if (variant == 0 && K > 8 &&
        lt2exp_takes_rows(R, S, I, J, K, sw[2] == 1 && sw[0] % 4 == 0 && sw[1] % 4 == 0 &&
                                             (reinterpret_cast<uintptr_t>(w) & 15) == 0, sw[2] == 1,
                          S <= 12 ? (pieces == 2 ? 0.6 : 0.4) : (pieces == 2 ? 0.2 : 0.0)))
        return trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, 0, workspace, workspace_bytes, stream);

    // Rows of w of 2 or 4 values fill an eighth or a quarter of this kernel's smallest j-chunk;
    // the fp32 kernel walks such rows packed, without padding (measured 1.4-2.5x ahead on
    // R=64 S=64 I=64..128 K=200, R=20 S=200 I=300 K=128; rows of 8: level with two pieces,
    // 5-20 % ahead of three).  Same conditions as trt_lt2exp_f32 applies.
    if (variant == 0 && (J == 2 || J == 4 || (J == 8 && pieces == 3)) && (I * J) % 4 == 0 && I * J >= 32 &&
        sw[0] % 4 == 0 && sw[1] % 4 == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0)
        return trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, 0, workspace, workspace_bytes, stream);

    // Tile and hand-over rules, fitted to 290 random shapes (R 1..128, S 16..512, I, J 8..128,
    // K 64..8192) timed with every tile and on the fp32 path; against the best of those the
    // rules below lose 2.5 % (two pieces) / 1.9 % (three) on average, the previous ones 17 / 14 %.
    //  - A grid of fewer than 160 32-row tiles -- 256 when the contraction is longer than 4096 --
    //    is latency bound, not matrix bound: its contraction is cut over workgroups (32-row tiles,
    //    as many cuts as the cost model asks for and the workspace holds; 1.5-2.5x ahead of the
    //    fp32 path on batch-1 squares of 192..512), and when it is not to be cut the call goes to
    //    the fp32 path.  Mode SPLIT cuts on the bf16 pipe as well.
    //  - 32 rows per workgroup; 64 when that pads S no further and still leaves two workgroups
    //    per CU (the pipelined two-row-tile loop then wins 4-11 %).
    //  - j-chunks of 64, 48, 32 or 16: the one that pads J least, weighed by its cost per j
    //    (bf16_chunk).
    const int64_t ctk = ceil_div(K, 128);
    const int64_t t64 = R * ceil_div(S, 64) * ctk;
    const int64_t s_last = S % 64;
    int rt = (S > 32 && (s_last == 0 || s_last > 32) && t64 >= 512) ? 2 : 1;
    int ks = bf16_chunk(J, pieces);
    const int rule_rt = rt, rule_ks = ks;
    bool split = false, small_grid = false;
    if (variant >= 1) {
        // 1: 64 rows, chunks of 64;  2: 64 rows, 32;  3: 32 rows, 64;  4: 32 rows, 32;
        // 5..8: the same with the contraction cut over workgroups (as far as the workspace allows)
        // 9..12: chunks of 48 and 16 (64 rows: 9, 10; 32 rows: 11, 12);  13..16: the same, cut
        const int tile = (variant - 1) % 4 + 1;
        rt = tile <= 2 ? 2 : 1;
        if (variant <= 8) ks = (tile & 1) ? 4 : 2;
        else ks = (tile & 1) ? 3 : 1;
        split = (variant >= 5 && variant <= 8) || variant >= 13;
    } else {
        // A grid that is not matrix bound as it is has its contraction cut over workgroups on
        // 32-row tiles when the cost model asks for it (below); a small grid that is not to be
        // cut goes to the fp32 path.
        small_grid = bf16_small_grid(R, S, I, J, K, mode);
        if (bf16_small_grid_splits(R, S, I, J, K, pieces, mode) >= 2) {
            split = true;
            rt = 1;
            ks = bf16_chunk(J, pieces);
        }
    }

    // Cutting the (j-chunk, i) iterations over workgroups: partial sums in the workspace
    // ([splits][R][S][K], then the two shift planes), merged in split order.
    int splits = 1, per_split = 0;
    if (split) {
        const int64_t iters = ceil_div(J, 16 * ks) * I;
        const int64_t tiles = R * ceil_div(S, 32 * rt) * ctk;
        const int64_t out = R * S * K;
        const int64_t fit = workspace ? ((int64_t)(workspace_bytes / sizeof(float)) - 2 * R * K) / out : 0;
        int64_t want = variant >= 1
                           ? choose_splits(tiles, iters, (int64_t)ks * (pieces == 2 ? 3 : 6) * rt / 2, out, 4, 32, true)
                           : bf16_small_grid_splits(R, S, I, J, K, pieces, mode);
        if (want > fit) want = fit;
        if (want >= 2) {
            per_split = (int)ceil_div(iters, want);
            splits = (int)ceil_div(iters, per_split);
        }
        split = splits >= 2;
        if (!split && variant == 0) {  // the workspace holds no cut: the uncut tile after all
            rt = rule_rt;
            ks = rule_ks;
        }
    }
    if (small_grid && !split)
        return trt_lt2exp_f32(w, a, b, c, R, S, I, J, K, sw, sa, sb, sc, mode, 0, workspace, workspace_bytes, stream);

    Lt2BfArgs args;
    args.w = w; args.a = a; args.b = b; args.c = c;
    args.shift = nullptr;
    args.splits = splits;
    args.iters_per_split = per_split;
    if (split) {
        args.c = static_cast<float *>(workspace);
        args.shift = args.c + (size_t)splits * R * S * K;
    }
    args.R = (int)R; args.S = (int)S; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sw0 = sw[0]; args.sw1 = sw[1];
    args.sa0 = sa[0]; args.sa1 = sa[1]; args.sa2 = sa[2]; args.sw2 = sw[2];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.s_tiles = (int)ceil_div(S, 32 * rt);
    args.n_tiles = (int)ceil_div(K, 128);
    args.total_wgs = (int64_t)R * args.s_tiles * args.n_tiles * splits;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    args.stream_out = rows_16_byte_aligned(c, sc[0], sc[1]);
    if (args.padded_wgs >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    const bool vec = sw[2] == 1 && (J % 4 == 0) && (sw[0] % 4 == 0) && (sw[1] % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(w) & 15) == 0);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pieces == 2) launch_bf_shape<2>(args, rt, ks, vec, split, s);
    else launch_bf_shape<3>(args, rt, ks, vec, split, s);
    if (split) launch_lt2exp_merge(args.c, args.shift, c, R, S, K, splits, sc[0], sc[1], s);
    return (int)hipGetLastError();
}
