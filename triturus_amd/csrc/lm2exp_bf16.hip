// lm2exp on the bf16 matrix pipe of gfx950, fp32 in and out:
//   c[r,i,k] = log sum_j a[r,i,j] exp(b[r,j,k])
//
// Counterpart of the reference's reduced-precision mode (ALLOW_TF32 passed to tl.dot,
// triturus/lm2exp.py:152, flag triturus/utils.py:33-44).  As in lt2exp_bf16.hip every fp32
// operand is cut into NS bf16 pieces and a product is the sum of the 3 (NS = 2) or 6
// (NS = 3) piece products that matter, accumulated in fp32 by v_mfma_f32_32x32x16_bf16.
//
// A workgroup of 4 wavefronts owns 32*RT rows of I and 128 columns of K; a wavefront owns
// 32 of those columns for all rows.  J is walked in chunks of JC = 16*KS:
//   B operand = exp(b[j,n] - m[n]), evaluated and split in registers (a lane owns one
//               column; element e of lane-half h in k-step ks is j = 16 ks + 8 h + e);
//   A operand = the a tile, global -> registers -> split -> LDS (double buffered).
// The shift m[n] is found while sweeping (one pass over b): it starts as the maximum of the
// column's first chunk and moves up, with the accumulators rescaled, when a later chunk
// exceeds it by more than a margin -- the scheme of the fp32 kernel (lm2exp.hip).
// m is clamped to +-1e38 (baselines/lm2exp.py:12): an all -inf column gives -inf, not NaN.

#include <type_traits>

#include "bf16_split.hpp"
#include "lm2exp_merge.hpp"

namespace trt {


struct Lm2BfArgs {
    const float *a, *b;
    float *c;
    float *part;   // splits > 1: [splits][R][I][K] partial sums
    float *shift;  // splits > 1: [splits][R][K] the shift each partial sum is relative to
    int R, I, J, K;
    int64_t sa0, sa1, sb0, sb1, sc0, sc1;
    int64_t sb2;  // trailing stride of b (a lane owns a column: it only scales the lane offsets)
    int64_t sa2;  // trailing stride of a: other than 1 in the builds without 16-byte loads only
    int i_tiles, n_tiles, splits, chunks_per_split;
    int stream_out;  // rows of c are 16-byte aligned: non-temporal result stores
    int64_t total_wgs, padded_wgs;
};

// PLAIN: no shift, exp or log -- c = a b, the matrix product of trt_mm_bf16.
template <int RT, int KS, int NS, bool VEC, bool PLAIN = false>
__global__ __launch_bounds__(256, 2) void lm2exp_bf16_kernel(const Lm2BfArgs p) {
    constexpr int NT = 256;
    constexpr int TM = 32 * RT;   // rows of I per workgroup
    constexpr int TN = 128;
    constexpr int JC = 16 * KS;
    constexpr int LDA = JC + 8;   // padded LDS row in bf16: conflict-free 16-byte reads
    constexpr int F4_PER_ROW = JC / 4;
    constexpr int ROWS_PER_SLOT = NT / F4_PER_ROW;
    constexpr int SLOTS = TM * F4_PER_ROW / NT;
    static_assert(TM * F4_PER_ROW % NT == 0, "tile must divide over the threads");

    // Distance the shift may lag behind a chunk's maximum before the sums are rescaled.  A wide
    // margin means fewer rescales but a larger argument of exp2, whose error grows with it
    // (~2^-23 |x| log2 e): 32 keeps that below 6e-6, under the 2^-16 of two pieces; three
    // pieces aim at fp32 accuracy and keep the 8 of the fp32 kernel.
    constexpr float kMargin = NS == 2 ? 32.0f : 8.0f;

    extern __shared__ __attribute__((aligned(16))) __bf16 at[];  // [2][NS][TM * LDA]
    auto tile_ptr = [&](int buf, int sp) { return at + (buf * NS + sp) * (TM * LDA); };

    const int64_t L = xcd_logical_id(blockIdx.x, p.padded_wgs);
    if (L >= p.total_wgs) return;
    // Row tiles of one column panel are neighbours in the launch order: they stream the same
    // rows of b at the same time, so the panel comes from HBM once and from L2 afterwards.
    int64_t rest = L / p.i_tiles;
    const int itile = __builtin_amdgcn_readfirstlane((int)(L % p.i_tiles));
    const int split = __builtin_amdgcn_readfirstlane((int)(rest % p.splits));
    rest /= p.splits;
    const int nt = __builtin_amdgcn_readfirstlane((int)(rest % p.n_tiles));
    const int r = __builtin_amdgcn_readfirstlane((int)(rest / p.n_tiles));

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    const int h = lane / 32;
    const int m = lane % 32;
    const int i0 = itile * TM;
    const int ncol = nt * TN + wave * 32 + m;
    const int ncl = ncol < p.K ? ncol : p.K - 1;

    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;

    floatx16 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rt][v] = 0.f;

    // ---- a tile: global -> registers.  Rows past I are clamped to the last valid row (they
    // only feed accumulator rows that are never stored); columns past J must be zeros.
    floatx4 stage[SLOTS];
    const int trow = tid / F4_PER_ROW;
    const int tc4 = tid % F4_PER_ROW;
    uint32_t aoff[SLOTS];
#pragma unroll
    for (int sidx = 0; sidx < SLOTS; ++sidx) {
        int row = i0 + trow + sidx * ROWS_PER_SLOT;
        row = row < p.I ? row : p.I - 1;
        aoff[sidx] = ((uint32_t)(row - i0) * (uint32_t)p.sa1 + 4u * tc4 * (uint32_t)p.sa2) * 4u;
    }
    const float *atile0 = ar + (int64_t)i0 * p.sa1;
    const int arows = (p.I - i0) < TM ? (p.I - i0) : TM;
    const __amdgpu_buffer_rsrc_t a_rsrc =
        make_rsrc(atile0, (uint32_t)(((int64_t)(arows - 1) * p.sa1 + (int64_t)(p.J - 1) * p.sa2 + 1) * 4));
    // pair-wise staging of the unaligned build (chunks that divide the workgroup evenly)
    constexpr bool ELEM = !VEC && (NT % (JC / 2) == 0) && ((TM * JC / 2) % NT == 0) && (TM * JC / 2 / NT <= 2 * SLOTS);
    constexpr int NP = ELEM ? TM * JC / 2 / NT : 1;  // column pairs per thread
    const int ecp = tid % (JC / 2);
    const uint32_t ebase = ((uint32_t)(tid / (JC / 2)) * (uint32_t)p.sa1 + 2u * (uint32_t)ecp * (uint32_t)p.sa2) * 4u;
    const uint32_t acol_bytes = (uint32_t)p.sa2 * 4u;  // one column further (4 in the builds with 16-byte loads)
    auto load_tile = [&](int jc) {
        const uint32_t soff = (uint32_t)(jc * JC) * acol_bytes;  // wave-uniform
        const bool full = VEC && (jc * JC + JC <= p.J);
        if (full) {
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) stage[sidx] = buf_load_f32x4(a_rsrc, aoff[sidx], soff);
        } else if (VEC) {
            // ragged last chunk of aligned rows: what a 16-byte piece holds past J (row padding, the
            // next row, or nothing: outside the extent) is replaced by zeros
            const int j = jc * JC + 4 * tc4;
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) {
                const floatx4 v = buf_load_f32x4(a_rsrc, aoff[sidx], soff);
#pragma unroll
                for (int e = 0; e < 4; ++e) stage[sidx][e] = j + e < p.J ? v[e] : 0.f;
            }
        } else if (ELEM) {
            // rows that are not 16-byte aligned: a thread takes pairs of adjacent columns (one
            // register of two bf16 per piece afterwards), consecutive lanes consecutive pairs, its
            // pairs NT / (JC / 2) rows apart (scalar offsets); rows past I lie outside the extent
            // and read as zeros, as do columns past J
            const bool in0 = jc * JC + 2 * ecp < p.J, in1 = jc * JC + 2 * ecp + 1 < p.J;
#pragma unroll
            for (int e = 0; e < NP; ++e) {
                const uint32_t so = soff + (uint32_t)(e * (2 * NT / JC)) * (uint32_t)p.sa1 * 4u;
                const float v0 = buf_load_f32(a_rsrc, ebase, so), v1 = buf_load_f32(a_rsrc, ebase + acol_bytes, so);
                stage[e / 2][2 * (e % 2)] = in0 ? v0 : 0.f;
                stage[e / 2][2 * (e % 2) + 1] = in1 ? v1 : 0.f;
            }
        } else {
            const int j = jc * JC + 4 * tc4;
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = buf_load_f32(a_rsrc, aoff[sidx] + acol_bytes * e, soff);
                    stage[sidx][e] = (j + e < p.J) ? v : 0.f;
                }
        }
    };
    auto store_tile = [&](int buf) {
        if (ELEM) {
#pragma unroll
            for (int e = 0; e < NP; ++e) {
                uint32_t pk[NS];
                split_pair<NS, false>(stage[e / 2][2 * (e % 2)], stage[e / 2][2 * (e % 2) + 1], pk);
                const int off = (tid / (JC / 2) + e * (2 * NT / JC)) * LDA + 2 * ecp;
#pragma unroll
                for (int sp = 0; sp < NS; ++sp) *reinterpret_cast<uint32_t *>(tile_ptr(buf, sp) + off) = pk[sp];
            }
            return;
        }
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) {
            uint32_t p01[NS], p23[NS];
            split_pair<NS, false>(stage[sidx][0], stage[sidx][1], p01);
            split_pair<NS, false>(stage[sidx][2], stage[sidx][3], p23);
            const int off = (trow + sidx * ROWS_PER_SLOT) * LDA + 4 * tc4;
#pragma unroll
            for (int sp = 0; sp < NS; ++sp) {
                uintx2 v = {p01[sp], p23[sp]};
                *reinterpret_cast<uintx2 *>(tile_ptr(buf, sp) + off) = v;
            }
        }
    };

    // ---- b chunk: global -> registers; rows past J read as -inf
    float braw[KS][8];
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(br, (uint32_t)(((int64_t)(p.J - 1) * p.sb1 + (int64_t)(p.K - 1) * p.sb2 + 1) * 4));
    const uint32_t b_row_bytes = (uint32_t)p.sb1 * 4u;
    const uint32_t boff = ((uint32_t)(8 * h) * (uint32_t)p.sb1 + (uint32_t)ncl * (uint32_t)p.sb2) * 4u;
    auto load_b = [&](int jc) {
        if (jc * JC + JC <= p.J) {  // wave-uniform: a full chunk needs no masks
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    braw[ks][e] = buf_load_f32(b_rsrc, boff, (uint32_t)(jc * JC + 16 * ks + e) * b_row_bytes);
        } else {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float v = buf_load_f32(b_rsrc, boff, (uint32_t)(jc * JC + 16 * ks + e) * b_row_bytes);
                    braw[ks][e] = (jc * JC + 16 * ks + 8 * h + e < p.J) ? v : (PLAIN ? 0.f : -__builtin_inff());
                }
        }
    };
    // Maximum of the chunk's column (both lane halves).  A NaN need not survive here:
    // exp(NaN - m) is NaN for any m and poisons the column through the MFMA.
    auto chunk_max = [&]() {
        float x = max3_raw(braw[0][0], braw[0][1], braw[0][2]);
#pragma unroll
        for (int e = 3; e + 1 < 8 * KS; e += 2) x = max3_raw(x, braw[e / 8][e % 8], braw[(e + 1) / 8][(e + 1) % 8]);
        x = max3_raw(x, braw[KS - 1][7], braw[KS - 1][7]);
        return max3_raw(x, __shfl_xor(x, 32, kWave), x);
    };

    float mref;
    uintx4 ebp[NS][KS];
    // raw chunk -> split MFMA operands, moving the shift first if this chunk towers over it
    auto exp_and_split = [&](auto keep_inf) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                uint32_t pk[NS];
                split_pair<NS, decltype(keep_inf)::value>(exp_shifted(braw[ks][2 * u] - mref),
                                                          exp_shifted(braw[ks][2 * u + 1] - mref), pk);
#pragma unroll
                for (int sp = 0; sp < NS; ++sp) ebp[sp][ks][u] = pk[sp];
            }
    };
    auto shift_and_exp = [&]() {
        if (PLAIN) {  // the B operand is b itself
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    uint32_t pk[NS];
                    split_pair<NS, false>(braw[ks][2 * u], braw[ks][2 * u + 1], pk);
#pragma unroll
                    for (int sp = 0; sp < NS; ++sp) ebp[sp][ks][u] = pk[sp];
                }
            return;
        }
        const float cm = chunk_max();
        const bool need = cm > mref + kMargin;
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
            const float mnew = need ? clamp_shift(cm) : mref;
            const float d = mref - mnew;  // <= 0; 0 in the lanes that stay
            const bool deep = __builtin_amdgcn_ballot_w64(d < kDeepRescale) != 0;  // wave-uniform, rare
            const float sc = exp_shifted(deep ? 0.5f * d : d);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[rt][v] *= sc;
            if (deep) {
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[rt][v] *= sc;
            }
            mref = mnew;
        }
        // exp(b - m) is infinite only for b = +inf (everything else is at most e^margin above
        // the shift): only then do the pieces need the inf - inf guard (rare, wave-uniform)
        if (__builtin_amdgcn_ballot_w64(cm == __builtin_inff()) != 0)
            exp_and_split(std::true_type{});
        else
            exp_and_split(std::false_type{});
    };

    // chunks [jc0, jc1) of this workgroup: all of them unless the contraction is cut over J
    const int n_jc = (p.J + JC - 1) / JC;
    const int jc0 = split * p.chunks_per_split;
    const int jc1 = (jc0 + p.chunks_per_split < n_jc) ? jc0 + p.chunks_per_split : n_jc;

    // ---- prologue: first chunk
    load_tile(jc0);
    load_b(jc0);
    store_tile(0);
    mref = PLAIN ? 0.f : clamp_shift(chunk_max());
    shift_and_exp();
    __syncthreads();

    // Row tiles are taken two at a time (all three of a 96-row tile) so that consecutive MFMAs
    // alternate between accumulators.
    constexpr int RP = RT % 2 == 0 ? 2 : (RT == 3 ? 3 : 1);
    auto mfma_block = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int rt0 = 0; rt0 < RT; rt0 += RP) {
                bf16x8 af[RP][NS];
#pragma unroll
                for (int k = 0; k < RP; ++k)
#pragma unroll
                    for (int sp = 0; sp < NS; ++sp)
                        af[k][sp] = *reinterpret_cast<const bf16x8 *>(tile_ptr(buf, sp) + (32 * (rt0 + k) + m) * LDA +
                                                                      16 * ks + 8 * h);
#pragma unroll
                for (int sa = 0; sa < NS; ++sa)
#pragma unroll
                    for (int sb = 0; sa + sb < NS; ++sb) {
                        const bf16x8 bop = __builtin_bit_cast(bf16x8, ebp[sb][ks]);
#pragma unroll
                        for (int k = 0; k < RP; ++k)
                            acc[rt0 + k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[k][sa], bop, acc[rt0 + k], 0, 0, 0);
                    }
            }
    };

    int cur = 0;
    for (int jc = jc0; jc + 1 < jc1; ++jc) {
        load_tile(jc + 1);
        load_b(jc + 1);
        __builtin_amdgcn_sched_barrier(0);  // the prefetch is issued before the MFMA block
        mfma_block(cur);
        store_tile(cur ^ 1);
        shift_and_exp();
        __syncthreads();
        cur ^= 1;
    }
    mfma_block(cur);

    // ---- epilogue: c = m + log(acc); register v of lane (h, m) holds row 8*(v/4) + 4*h +
    // v%4, column m of its 32 x 32 tile.  Rows past I fall outside the buffer extent.
    if (ncol >= p.K) return;
    if (p.splits > 1) {  // wave-uniform: raw sums and their shift go to the workspace, the merge finishes
        float *part = p.part + (((int64_t)split * p.R + r) * p.I) * (int64_t)p.K;
        if (itile == 0 && h == 0) p.shift[((int64_t)split * p.R + r) * p.K + ncol] = mref;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = i0 + 32 * rt + 8 * (v / 4) + 4 * h + (v % 4);
                if (row < p.I) part[(int64_t)row * p.K + ncol] = acc[rt][v];
            }
        return;
    }
    const int crows = p.I - i0;
    const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(p.c + (int64_t)r * p.sc0 + (int64_t)i0 * p.sc1,
                                                    (uint32_t)(((int64_t)(crows - 1) * p.sc1 + p.K) * 4));
    const uint32_t c_row_bytes = (uint32_t)p.sc1 * 4u;
    const uint32_t co = ((uint32_t)(4 * h) * (uint32_t)p.sc1 + (uint32_t)ncol) * 4u;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t trow_c = 32 * rt + 8 * (v / 4) + (v % 4);
            buf_store_f32_out(p.stream_out != 0, PLAIN ? acc[rt][v] : log_plus(acc[rt][v], mref), c_rsrc, co,
                              trow_c * c_row_bytes);
        }
}

constexpr size_t kBfDefaultLdsLimit = 64 * 1024;

template <int RT, int KS, int NS, bool VEC, bool PLAIN = false>
static int launch_lm_bf_k(const Lm2BfArgs &args, hipStream_t stream) {
    constexpr size_t lds = (size_t)2 * NS * (32 * RT) * (16 * KS + 8) * sizeof(__bf16);
    auto k = lm2exp_bf16_kernel<RT, KS, NS, VEC, PLAIN>;
    if (lds > kBfDefaultLdsLimit) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(k, dim3((unsigned)args.padded_wgs), dim3(256), lds, stream, args);
    return (int)hipGetLastError();
}

template <int RT, int KS>
static int launch_lm_bf(const Lm2BfArgs &args, int pieces, bool vec, hipStream_t stream) {
    if (pieces == 2) return vec ? launch_lm_bf_k<RT, KS, 2, true>(args, stream) : launch_lm_bf_k<RT, KS, 2, false>(args, stream);
    return vec ? launch_lm_bf_k<RT, KS, 3, true>(args, stream) : launch_lm_bf_k<RT, KS, 3, false>(args, stream);
}

struct LmBfVariant {
    int rt, ks;
};
// variant ids are 1-based in the C ABI (0 = choose by shape)
static const LmBfVariant kLmBfVariants[] = {{4, 4}, {4, 2}, {2, 4}, {2, 2}, {1, 4}, {1, 2}, {8, 1}, {8, 2}, {3, 2}};
constexpr int kNumLmBfVariants = sizeof(kLmBfVariants) / sizeof(kLmBfVariants[0]);

bool lm2exp_takes_sweep(int64_t R, int64_t I, int64_t J, int64_t K, bool a_aligned);  // csrc/lt2exp.hip
bool lm2exp_takes_jsplit16(int64_t R, int64_t I, int64_t J, int64_t K);  // csrc/lm2exp.hip

}  // namespace trt

using namespace trt;

extern "C" int trt_lm2exp_bf16_variant_count(void) { return kNumLmBfVariants; }

// Cut of the contraction for grids that do not fill the chip (batch-1 squares and the like):
// `splits` workgroups share one 32 x 128 output tile, each sweeping its own range of 32-wide
// j-chunks with its own running shift; raw sums and shifts go to the workspace and
// lm2exp_merge_kernel finishes.  Returns 1 when the call is not cut.  requested: 0 = by the
// cost model, 1 = never, > 1 = that many (capped by the number of chunks).
static int lm_bf16_cut(int64_t R, int64_t I, int64_t J, int64_t K, int pieces, int requested) {
    if (requested == 1) return 1;
    const int64_t n_jc = ceil_div(J, 32);
    if (n_jc < 2) return 1;
    int64_t sp;
    if (requested > 1) {
        sp = requested > 32 ? 32 : requested;
        if (sp > n_jc) sp = n_jc;
    } else {
        const int64_t tiles = R * ceil_div(I, 32) * ceil_div(K, 128);
        if (tiles >= 1024) return 1;
        // Constants fitted to 150 random shapes of fewer than 1500 tiles timed with every cut of
        // 2..16 on 32- and 64-row tiles: a chunk costs a lone workgroup 0.9 us with two pieces
        // or three (latency, not MFMAs), 0.3 us per split for the merge of a small output (bound
        // by its chain of loads), and a cut that the model rates 10 % ahead is taken.  Against
        // the best measured choice this loses 1.7 %, never cutting 8 % (two pieces) / 5 %.
        sp = choose_splits(tiles, n_jc, 15, R * I * K, 4, 32, false, 0.3, 0.9);
    }
    const int64_t cps = ceil_div(n_jc, sp);
    return (int)ceil_div(n_jc, cps);  // no split is left without a chunk
}

extern "C" size_t trt_lm2exp_bf16_workspace_bytes(int64_t R, int64_t I, int64_t J, int64_t K, int pieces,
                                                  int splits) {
    if (R <= 0 || I <= 0 || J <= 0 || K <= 0 || splits < 0 || (pieces != 2 && pieces != 3)) return 0;
    int64_t sp = lm_bf16_cut(R, I, J, K, pieces, splits);
    if (splits > 1) {  // a forced tile may sweep chunks of 16: room for what any tile would use
        sp = splits > 32 ? 32 : splits;
        if (sp > ceil_div(J, 16)) sp = ceil_div(J, 16);
    }
    return sp > 1 ? (size_t)sp * (size_t)(R * I * K + R * K) * sizeof(float) : 0;
}

extern "C" int trt_lm2exp_bf16(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                               const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], int pieces,
                               int variant, int splits, void *workspace, size_t workspace_bytes, void *stream) {
    if (!a || !b || !c || !sa || !sb || !sc) return TRT_E_INVALID;
    if (R <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (pieces != 2 && pieces != 3) return TRT_E_INVALID;
    if (variant < 0 || variant > kNumLmBfVariants || splits < 0) return TRT_E_INVALID;
    if (sa[2] < 0 || sb[2] < 0 || sc[2] != 1) return TRT_E_LAYOUT;
    for (int d = 0; d < 2; ++d)
        if (sa[d] < 0 || sb[d] < 0 || sc[d] < 0) return TRT_E_LAYOUT;
    if (sc[1] < K) return TRT_E_LAYOUT;  // output rows must not overlap
    const int64_t lim = (int64_t)1 << 30;
    if (R >= lim || I >= lim || J >= lim || K >= lim) return TRT_E_RANGE;
    // byte offsets inside one batch slab are 32-bit (buffer addressing)
    if (I * sa[1] + J * sa[2] >= lim || J * sb[1] + K * sb[2] >= lim || I * sc[1] + K >= lim) return TRT_E_RANGE;

    // Tile and hand-over rules, fitted to 223 random shapes (R 1..256, I, J 16..1024, K 64..8192)
    // timed with every tile and on the fp32 path; against the best of those the rules below lose
    // 5.6 % (two pieces) / 4.3 % (three) on average, the previous ones 19 / 11 %.
    //  - Grids of fewer than 1024 32-row tiles over a long contraction are cut over J when the
    //    cost model (lm_bf16_cut) says so, as far as the workspace allows.
    //  - Uncut grids of fewer than 128 (three pieces: 192) 32-row tiles are latency bound, not
    //    matrix bound, and a contraction of at most 16 (32) is bound by writing c: there the fp32
    //    path (smaller tiles, its own cut over J) is as fast or faster and takes the call.
    //  - j-chunks of 32 (three workgroups fit a CU; chunks of 64 measured 0-17 % behind), except
    //    with two pieces on 64- and 32-row tiles over a contraction of 512 or more (chunks of 64).
    //  - Rows: the candidate (128, 96, 64 or 32 rows; at least 1.5, 1.5, 1, 0 workgroups per CU)
    //    with the least padded rows x cost per row, the cost being 1.2 for 32 rows, 1 for 64, and on
    //    a contraction of 256 or more, where each exp feeds more MFMAs, 0.90 (0.93) for 96 and 0.85
    //    (0.95) for 128 rows; on a shorter one 1 and 1.05.  The 96-row tile (three wavefronts
    //    per SIMD) takes I = 96, 160, 192, 288 and the like: 10-24 % ahead there.
    int v;
    int cut = 1;
    if (variant >= 1) {
        v = variant - 1;
        if (splits > 1) {  // a forced tile with a forced cut (tests and tuning)
            const int64_t jc = 16 * kLmBfVariants[v].ks;
            int64_t sp = splits > 32 ? 32 : splits;
            const int64_t n_jc = ceil_div(J, jc);
            if (sp > n_jc) sp = n_jc;
            cut = (int)ceil_div(n_jc, ceil_div(n_jc, sp));
            const int64_t fit = workspace ? (int64_t)(workspace_bytes / sizeof(float)) / (R * I * K + R * K) : 0;
            if (cut > 1 && cut > fit) return TRT_E_WORKSPACE;
        }
    } else {
        const int64_t ct = ceil_div(K, 128);
        const int64_t n32 = R * ceil_div(I, 32) * ct;
        if (J > (pieces == 2 ? 16 : 32)) {
            cut = lm_bf16_cut(R, I, J, K, pieces, splits);
            const int64_t per_split = R * I * K + R * K;
            const int64_t fit = workspace ? (int64_t)(workspace_bytes / sizeof(float)) / per_split : 0;
            if (cut > fit) cut = fit >= 2 ? lm_bf16_cut(R, I, J, K, pieces, (int)fit) : 1;
        }
        const bool small = n32 < (pieces == 2 ? 128 : 192);
        // where the fp32 path would not cut a contraction of 192..416 either, one launch of
        // 32-row bf16 tiles is 4-15 % ahead of its one launch; where it would, its cut wins on
        // operands that come from HBM (by 4-6 us) and loses on cached ones (by 3 us): left to it
        const bool one_launch = small && splits == 0 && J >= 192 && J <= 416 &&
                                trt_lm2exp_workspace_bytes(R, I, J, K, 0, 0) == 0;
        // outputs of at most 32 columns: the fp32 path has a tile with its wavefronts stacked over rows
        const bool narrow = K <= 32 && I > 64;
        // at most 4 columns under a long contraction: the fp32 entry sweeps a on the vector ALU
        const bool swept = splits <= 1 && lm2exp_takes_sweep(R, I, J, K, sa[2] == 1 && sa[0] % 4 == 0 && sa[1] % 4 == 0 &&
                                                                            (reinterpret_cast<uintptr_t>(a) & 15) == 0);
        // at most 16 rows and 32 columns per batch: one tile per batch, bound by the reads of b
        const bool one_tile = splits <= 1 && lm2exp_takes_jsplit16(R, I, J, K);
        if (narrow || swept || one_tile || (cut == 1 && !one_launch && (splits > 1 || small || J <= (pieces == 2 ? 16 : 32))))
            return trt_lm2exp_f32(a, b, c, R, I, J, K, sa, sb, sc, 0, splits, workspace, workspace_bytes, stream);
        int best_rt = 1;
        int64_t best_cost = ceil_div(I, 32) * 120;
        for (int rt = 2; rt <= 4; ++rt) {
            if (R * ceil_div(I, 32 * rt) * ct < (rt == 2 ? 256 : 384)) continue;  // 1 / 1.5 workgroups per CU
            int64_t per_row = 100;
            if (rt == 3) per_row = J >= 256 ? (pieces == 2 ? 90 : 93) : 100;
            if (rt == 4) per_row = J >= 256 ? (pieces == 2 ? 85 : 95) : 105;
            const int64_t cost = ceil_div(I, 32 * rt) * rt * per_row;
            if (cost <= best_cost) {  // ties go to the larger tile
                best_cost = cost;
                best_rt = rt;
            }
        }
        v = best_rt == 4 ? 1 : (best_rt == 3 ? 8 : (best_rt == 2 ? 3 : 5));  // {4,2}, {3,2}, {2,2}, {1,2}
        if (pieces == 2 && best_rt <= 2 && J >= 512) v -= 1;  // {2,4}, {1,4}: fewer barriers pay on a long contraction
        // two pieces are bound by the vector work on the B operand: 256 rows (each exp feeds 24
        // MFMAs) when I fills them exactly and two workgroups per CU remain (6-25 % at I = 256, 512)
        if (pieces == 2 && best_rt == 4 && I % 256 == 0 && J >= 256 && R * (I / 256) * ct >= 512) v = 7;  // {8,2}
        // the cut is made on 32-row tiles, or on 64-row ones where those still number 64
        if (cut > 1) v = (I > 32 && R * ceil_div(I, 64) * ct >= 64) ? 3 : 5;  // {2,2}, {1,2}
    }
    const LmBfVariant &vr = kLmBfVariants[v];

    Lm2BfArgs args;
    args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sa0 = sa[0]; args.sa1 = sa[1];
    args.sb0 = sb[0]; args.sb1 = sb[1]; args.sb2 = sb[2]; args.sa2 = sa[2];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.i_tiles = (int)ceil_div(I, 32 * vr.rt);
    args.n_tiles = (int)ceil_div(K, 128);
    const int64_t n_jc = ceil_div(J, 16 * vr.ks);
    args.splits = cut;
    args.chunks_per_split = (int)ceil_div(n_jc, cut);
    args.part = cut > 1 ? static_cast<float *>(workspace) : nullptr;
    args.shift = cut > 1 ? args.part + (int64_t)cut * R * I * K : nullptr;
    args.total_wgs = (int64_t)R * args.i_tiles * args.n_tiles * cut;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    args.stream_out = rows_16_byte_aligned(c, sc[0], sc[1]);
    if (args.padded_wgs >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    // (J itself need not be a multiple of 4 when the row stride is: the piece that straddles J
    // is masked by element)
    const bool vec = sa[2] == 1 && (sa[0] % 4 == 0) && (sa[1] % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int status;
    switch (v) {
        case 0: status = launch_lm_bf<4, 4>(args, pieces, vec, s); break;
        case 1: status = launch_lm_bf<4, 2>(args, pieces, vec, s); break;
        case 2: status = launch_lm_bf<2, 4>(args, pieces, vec, s); break;
        case 3: status = launch_lm_bf<2, 2>(args, pieces, vec, s); break;
        case 4: status = launch_lm_bf<1, 4>(args, pieces, vec, s); break;
        case 5: status = launch_lm_bf<1, 2>(args, pieces, vec, s); break;
        case 6: status = launch_lm_bf<8, 1>(args, pieces, vec, s); break;
        case 7: status = launch_lm_bf<8, 2>(args, pieces, vec, s); break;
        default: status = launch_lm_bf<3, 2>(args, pieces, vec, s); break;
    }
    if (status != 0 || cut == 1) return status;
    launch_lm2exp_merge(args.part, args.shift, c, R, I, K, cut, sc[0], sc[1], s);
    return (int)hipGetLastError();
}

// c = a b for row-major fp32 matrices on the bf16 matrix pipe (operands cut into `pieces`
// bf16 pieces, fp32 accumulation): the kernel above without shift, exp and log.  Grids too
// small for it go to trt_mm_f32.  Counterpart of `_ker_mm[grid](..., ALLOW_TF32=True)`,
// triturus/mm.py:199-213.
template <int RT, int KS>
static int launch_mm_bf(const Lm2BfArgs &args, int pieces, bool vec, hipStream_t s) {
    if (pieces == 2)
        return vec ? launch_lm_bf_k<RT, KS, 2, true, true>(args, s) : launch_lm_bf_k<RT, KS, 2, false, true>(args, s);
    return vec ? launch_lm_bf_k<RT, KS, 3, true, true>(args, s) : launch_lm_bf_k<RT, KS, 3, false, true>(args, s);
}

extern "C" int trt_mm_bf16(const float *a, const float *b, float *c, int64_t m, int64_t k, int64_t n, int pieces,
                           void *workspace, size_t workspace_bytes, void *stream) {
    if (!a || !b || !c) return TRT_E_INVALID;
    if (m <= 0 || k <= 0 || n <= 0) return TRT_E_INVALID;
    if (pieces != 2 && pieces != 3) return TRT_E_INVALID;
    const int64_t lim = (int64_t)1 << 30;
    if (m >= lim || k >= lim || n >= lim) return TRT_E_RANGE;
    if (k * n + n >= lim || m * k + k >= lim || m * n + n >= lim) return TRT_E_RANGE;
    const int64_t ct = ceil_div(n, 128);
    const int64_t n128 = ceil_div(m, 128) * ct, n64 = ceil_div(m, 64) * ct;
    int rt;
    if (m > 64 && n128 >= 384) rt = 4;
    else if (m > 32 && n64 >= 256) rt = 2;
    else return trt_mm_f32(a, b, c, m, k, n, 0, 0, workspace, workspace_bytes, stream);
    Lm2BfArgs args;
    args.a = a; args.b = b; args.c = c;
    args.R = 1; args.I = (int)m; args.J = (int)k; args.K = (int)n;
    args.sa0 = m * k; args.sa1 = k;
    args.sb0 = k * n; args.sb1 = n; args.sb2 = 1; args.sa2 = 1;
    args.sc0 = m * n; args.sc1 = n;
    args.i_tiles = (int)ceil_div(m, 32 * rt);
    args.n_tiles = (int)ct;
    args.part = nullptr; args.shift = nullptr;
    args.splits = 1;
    args.chunks_per_split = (int)ceil_div(k, 16);  // at least every chunk
    args.total_wgs = (int64_t)args.i_tiles * args.n_tiles;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    args.stream_out = rows_16_byte_aligned(c, args.sc0, args.sc1);
    const bool vec = (k % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
    hipStream_t s = static_cast<hipStream_t>(stream);
    return rt == 4 ? launch_mm_bf<4, 2>(args, pieces, vec, s) : launch_mm_bf<2, 4>(args, pieces, vec, s);
}
