// lm2exp for gfx950:  c[r,i,k] = log sum_j a[r,i,j] exp(b[r,j,k])
//
// A workgroup of WM x WN wavefronts owns a (32*RT*WM rows of I) x
// (32*CT*WN columns of K) tile of c[r] and walks J in chunks of JC = 8*NQ:
//   B operand = exp(b[j,n] - m[n]), evaluated once per (wavefront, element)
//               straight into the VGPRs the MFMA reads: every lane owns one
//               column n, b never visits LDS;
//   A operand = the a tile, staged global -> registers -> LDS (double
//               buffered) and read back 16 bytes per lane.
// The contraction runs on v_mfma_f32_32x32x2_f32 (IEEE fp32 in, fp32 accumulate),
// MFMA (q,u) of lane-half h consuming j = 8q + 4h + u of the chunk.
//
// The shift m[n].  The result m + log(sum_j a exp(b - m)) does not depend on m, only
// overflow/underflow do, so m need not be the exact column maximum.  This kernel makes one
// sweep over b: m starts as the maximum of the first chunk of the column; when a later chunk's
// maximum exceeds m by more than kRescaleMargin the accumulators of that column are multiplied
// by exp(m_old - m_new) and m moves up.  exp(b - m) therefore never exceeds e^kRescaleMargin, and
// b is read from HBM exactly once.  (The reference kernel sweeps b twice, exact column maximum
// first, triturus/lm2exp.py:125-127; so does the paired-wavefront kernel of lm2exp_pair.hpp,
// which the host prefers where the panel of b stays in cache.)  MODE kPlain: no shift, exp or
// log at all (the mm entry point).
// m is always clamped to +-1e38 (baselines/lm2exp.py:12) so an all -inf
// column gives exp(-inf) = 0, log(0) = -inf: -inf out, never NaN.
//
// Replaces _ker_lm2exp, triturus/lm2exp.py:63-164.  Ragged contracted-axis
// tails are padded with a = 0 and b = -inf (the reference pads b with 0.0,
// triturus/lm2exp.py:143, which can overflow exp(0 - m); not reproduced).

#include "common.hpp"
#include "lm2exp_merge.hpp"

#include <cstdio>

namespace trt {

constexpr float kRescaleMargin = 8.0f;

struct Lm2Args {
    const float *a, *b;
    float *c;
    float *part;   // splits > 1: [splits][R][I][K] partial sums
    float *shift;  // splits > 1: [splits][R][K] the shift each partial sum is relative to
    int R, I, J, K;
    int64_t sa0, sa1, sb0, sb1, sc0, sc1;
    int64_t sa2;  // trailing stride of a (1 for every kernel but the paired-wavefront one)
    int64_t sb2;  // trailing stride of b: a lane owns a column, so it only scales the lane offsets
    int i_tiles, n_tiles, splits, chunks_per_split;
    int stream_out;  // rows of c are 16-byte aligned: non-temporal result stores
    int64_t total_wgs, padded_wgs;
};

// How the shift m[n] is obtained (MODE template parameter of the kernel)
constexpr int kOnline = 1;    // found while sweeping, accumulators rescaled when it moves
constexpr int kPlain = 3;     // no shift, no exp, no log: c = a b (the mm entry point)
constexpr int kPair = 4;      // lm2exp_pair_kernel: exact column maximum first, exp shared by two wavefronts

}  // namespace trt

#include "lm2exp_jsplit.hpp"
#include "lm2exp_pair.hpp"

namespace trt {

template <int RT, int CT, int WM, int WN, int NQ, bool VEC, int MODE>
__global__ __launch_bounds__(WM *WN *kWave, 2) void lm2exp_kernel(const Lm2Args p) {
    constexpr bool ONLINE = MODE == kOnline;
    constexpr int NT = WM * WN * kWave;
    constexpr int TM = 32 * RT * WM;  // rows of I per workgroup
    constexpr int TN = 32 * CT * WN;  // columns of K per workgroup
    constexpr int JC = 8 * NQ;
    constexpr int NB = 4 * NQ;   // b values per lane, column tile and chunk
    constexpr int LDA = JC + 4;  // padded LDS row (floats): conflict-free 16-byte reads
    constexpr int F4_PER_ROW = JC / 4;
    constexpr int F4_TILE = TM * F4_PER_ROW;        // 16-byte pieces of an a tile
    constexpr int SLOTS = (F4_TILE + NT - 1) / NT;  // of which a thread stages this many
    // REGULAR: a thread keeps its column and steps whole rows from slot to slot; otherwise
    // (chunks of 24 or 48, tiles smaller than the workgroup) pieces are dealt out linearly, and
    // a thread whose last slot lies past the tile stages into a private 16 bytes behind the
    // buffers, so that the steady state carries no predicates.
    constexpr bool REGULAR = (NT % F4_PER_ROW == 0) && (F4_TILE % NT == 0);

    constexpr int BUF = TM * LDA + (REGULAR ? 0 : 4 * NT);      // one LDS buffer: the tile, then the private pieces
    extern __shared__ __attribute__((aligned(16))) float at[];  // [2][BUF]

    const int64_t L = xcd_logical_id(blockIdx.x, p.padded_wgs);
    if (L >= p.total_wgs) return;
    // The tile coordinates are wave-uniform; the 64-bit divisions below are expanded on
    // the vector ALU, so pin the results back into scalar registers (they feed buffer
    // resources and scalar offsets).
    int64_t rest = L / p.n_tiles;
    const int nt = __builtin_amdgcn_readfirstlane((int)(L % p.n_tiles));
    const int split = __builtin_amdgcn_readfirstlane((int)(rest % p.splits));
    rest /= p.splits;
    const int itile = __builtin_amdgcn_readfirstlane((int)(rest % p.i_tiles));
    const int r = __builtin_amdgcn_readfirstlane((int)(rest / p.i_tiles));

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int wm = wave % WM;
    const int wn = wave / WM;
    const int lane = tid % kWave;
    const int h = lane / 32;
    const int m = lane % 32;
    const int i0 = itile * TM;
    const int n0 = nt * TN + wn * 32 * CT;
    const int wrow0 = wm * 32 * RT;  // first tile row of this wavefront

    int ncol[CT], ncl[CT];
    uint32_t boff[CT];  // per-lane byte offset inside a wave-uniform row group of b
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        ncol[ct] = n0 + 32 * ct + m;
        ncl[ct] = ncol[ct] < p.K ? ncol[ct] : p.K - 1;
        boff[ct] = ((uint32_t)(4 * h) * (uint32_t)p.sb1 + (uint32_t)ncl[ct] * (uint32_t)p.sb2) * 4u;
    }
    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;

    floatx16 acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rt][ct][v] = 0.f;

    // ---- a tile: global -> registers -> LDS.  Rows past I are clamped to the last
    // valid row instead of masked: they only feed accumulator rows that are never
    // stored.  Columns past J (ragged tail chunk only) must be exact zeros.
    floatx4 stage[SLOTS];
    int sc4[SLOTS];        // 16-byte column of each slot
    int lds_off[SLOTS];    // where the slot goes in an LDS buffer (floats)
    uint32_t aoff[SLOTS];  // per-lane byte offsets from the (wave-uniform) tile origin
#pragma unroll
    for (int sidx = 0; sidx < SLOTS; ++sidx) {
        int trow;
        bool inside = true;
        if (REGULAR) {
            trow = tid / F4_PER_ROW + sidx * (NT / F4_PER_ROW);
            sc4[sidx] = tid % F4_PER_ROW;
        } else {
            const int f = tid + sidx * NT;
            trow = f / F4_PER_ROW;
            sc4[sidx] = f % F4_PER_ROW;
            inside = f < F4_TILE;
        }
        lds_off[sidx] = inside ? trow * LDA + 4 * sc4[sidx] : TM * LDA + 4 * tid;
        int row = i0 + trow;
        row = row < p.I ? row : p.I - 1;
        aoff[sidx] = ((uint32_t)(row - i0) * (uint32_t)p.sa1 + 4u * (uint32_t)sc4[sidx]) * 4u;
    }
    const float *atile0 = ar + (int64_t)i0 * p.sa1;
    const int arows = (p.I - i0) < TM ? (p.I - i0) : TM;  // valid rows of this tile
    const __amdgpu_buffer_rsrc_t a_rsrc =
        make_rsrc(atile0, (uint32_t)(((int64_t)(arows - 1) * p.sa1 + p.J) * 4));
    // element-wise staging of the unaligned build (chunks that divide the workgroup evenly):
    // single floats, consecutive lanes on consecutive columns (coalesced), a thread's floats
    // NT / JC rows apart (scalar offsets); rows past I lie outside the extent and read as zeros
    constexpr bool ELEM = !VEC && (NT % JC == 0) && ((TM * JC) % NT == 0) && (TM * JC / NT <= 4 * SLOTS);
    constexpr int NE = ELEM ? TM * JC / NT : 1;  // floats per thread
    const int ecol = tid % JC;
    const uint32_t ebase = ((uint32_t)(tid / JC) * (uint32_t)p.sa1 + (uint32_t)ecol) * 4u;
    auto load_tile_elem = [&](int jc) {
        const uint32_t soff = (uint32_t)(jc * JC) * 4u;
        const bool inside = jc * JC + ecol < p.J;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const float v = buf_load_f32(a_rsrc, ebase, soff + (uint32_t)(e * (NT / JC)) * (uint32_t)p.sa1 * 4u);
            stage[e / 4][e % 4] = inside ? v : 0.f;
        }
    };
    auto load_tile_full = [&](int jc) {
        if (ELEM) return load_tile_elem(jc);
        const uint32_t soff = (uint32_t)(jc * JC) * 4u;  // wave-uniform
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) {
            if (VEC) {
                stage[sidx] = buf_load_f32x4(a_rsrc, aoff[sidx], soff);
            } else {
                floatx4 v;
                v[0] = buf_load_f32(a_rsrc, aoff[sidx], soff);
                v[1] = buf_load_f32(a_rsrc, aoff[sidx], soff + 4);
                v[2] = buf_load_f32(a_rsrc, aoff[sidx], soff + 8);
                v[3] = buf_load_f32(a_rsrc, aoff[sidx], soff + 12);
                stage[sidx] = v;
            }
        }
    };
    auto load_tile_masked = [&](int jc) {
        if (VEC) {
            // aligned rows: what a 16-byte piece holds past J (row padding, the next row, or
            // nothing: outside the extent) is replaced by zeros
            const uint32_t soff = (uint32_t)(jc * JC) * 4u;
#pragma unroll
            for (int sidx = 0; sidx < SLOTS; ++sidx) {
                const floatx4 v = buf_load_f32x4(a_rsrc, aoff[sidx], soff);
                const int j = jc * JC + 4 * sc4[sidx];
#pragma unroll
                for (int e = 0; e < 4; ++e) stage[sidx][e] = j + e < p.J ? v[e] : 0.f;
            }
            return;
        }
        if (ELEM) return load_tile_elem(jc);
        const char *org = reinterpret_cast<const char *>(atile0 + jc * JC);
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) {
            const int j = jc * JC + 4 * sc4[sidx];
            const float *src = reinterpret_cast<const float *>(org + aoff[sidx]);
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (j + 0 < p.J) v[0] = src[0];
            if (j + 1 < p.J) v[1] = src[1];
            if (j + 2 < p.J) v[2] = src[2];
            if (j + 3 < p.J) v[3] = src[3];
            stage[sidx] = v;
        }
    };
    auto store_tile = [&](int buf) {
        if (ELEM) {
#pragma unroll
            for (int e = 0; e < NE; ++e) at[buf * BUF + (tid / JC + e * (NT / JC)) * LDA + ecol] = stage[e / 4][e % 4];
            return;
        }
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx)
            *reinterpret_cast<floatx4 *>(&at[buf * BUF + lds_off[sidx]]) = stage[sidx];
    };

    // ---- b chunk: global -> registers.  Lane (h, m) takes rows 8q + 4h + u.
    // Full chunks use a wave-uniform row pointer (SGPRs) plus a 32-bit per-lane offset.
    // FP32 MFMA and the vector ALU do not execute concurrently on this hardware, so
    // every VALU instruction in the steady state costs matrix throughput: addresses
    // are kept in scalar registers and exp/log use the bare hardware instructions.
    float braw[CT][NB], eb[CT][NB];
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(br, (uint32_t)(((int64_t)(p.J - 1) * p.sb1 + (int64_t)(p.K - 1) * p.sb2 + 1) * 4));
    const uint32_t b_row_bytes = (uint32_t)p.sb1 * 4u;
    auto load_b_full = [&](int jc) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t soff = (uint32_t)(jc * JC + 8 * q + u) * b_row_bytes;  // wave-uniform
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) braw[ct][4 * q + u] = buf_load_f32(b_rsrc, boff[ct], soff);
            }
    };
    // ragged last chunk: the same loads (what lies past the extent reads as 0, nothing faults),
    // rows past J replaced by -inf
    auto load_b_masked = [&](int jc) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t soff = (uint32_t)(jc * JC + 8 * q + u) * b_row_bytes;  // wave-uniform
                const int j = jc * JC + 8 * q + 4 * h + u;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const float raw = buf_load_f32(b_rsrc, boff[ct], soff);
                    braw[ct][4 * q + u] = j < p.J ? raw : (MODE == kPlain ? 0.f : -__builtin_inff());
                }
            }
    };
    // Maximum of the chunk's column.  A NaN need not survive here: exp(NaN - m) is NaN
    // for any m and poisons the whole output column through the MFMA, which is what
    // the torch recipe gives for a NaN in b.
    auto chunk_max = [&](int ct) {
        float x = max3_raw(braw[ct][0], braw[ct][1], braw[ct][2]);
#pragma unroll
        for (int e = 3; e + 1 < NB; e += 2) x = max3_raw(x, braw[ct][e], braw[ct][e + 1]);
        x = max3_raw(x, braw[ct][NB - 1], braw[ct][NB - 1]);
        return max3_raw(x, __shfl_xor(x, 32, kWave), x);
    };

    float mref[CT];
    // Turn the raw chunk in braw into MFMA operands in eb, moving the shift first if this
    // chunk towers over it (rare, wave-uniform branch).
    auto shift_and_exp = [&]() {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (ONLINE) {
                const float cm = chunk_max(ct);
                const bool need = cm > mref[ct] + kRescaleMargin;
                if (__builtin_amdgcn_ballot_w64(need) != 0) {
                    const float mnew = need ? clamp_shift(cm) : mref[ct];
                    const float d = mref[ct] - mnew;  // <= 0; 0 in the lanes that stay
                    const bool deep = __builtin_amdgcn_ballot_w64(d < kDeepRescale) != 0;  // wave-uniform, rare
                    const float sc = exp_shifted(deep ? 0.5f * d : d);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[rt][ct][v] *= sc;
                    if (deep) {
#pragma unroll
                        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                            for (int v = 0; v < 16; ++v) acc[rt][ct][v] *= sc;
                    }
                    mref[ct] = mnew;
                }
            }
#pragma unroll
            for (int e = 0; e < NB; ++e)
                eb[ct][e] = MODE == kPlain ? braw[ct][e] : exp_shifted(braw[ct][e] - mref[ct]);
        }
    };

    // Chunks [jc0, jc1) of this workgroup (all of them unless the contraction is split
    // over several workgroups); chunks below n_full carry no ragged tail.
    const int n_full = p.J / JC;
    const int n_jc = n_full + ((p.J % JC) != 0 ? 1 : 0);
    const int jc0 = split * p.chunks_per_split;
    const int jc1 = (jc0 + p.chunks_per_split < n_jc) ? jc0 + p.chunks_per_split : n_jc;
    const int full_end = jc1 < n_full ? jc1 : n_full;

    if (MODE == kPlain) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) mref[ct] = 0.f;
    }
    // ---- prologue: first chunk
    if (jc0 < n_full) {
        load_tile_full(jc0);
        load_b_full(jc0);
    } else {
        load_tile_masked(jc0);
        load_b_masked(jc0);
    }
    store_tile(0);
    if (ONLINE) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) mref[ct] = clamp_shift(chunk_max(ct));
    }
    shift_and_exp();
    __syncthreads();

    // Row tiles are taken two at a time (all three of a 96-row tile) so that consecutive
    // MFMAs alternate between accumulators while only two or three A fragments are live.
    constexpr int RP = RT % 2 == 0 ? 2 : (RT == 3 ? 3 : 1);
    // The A fragments of a group of MFMAs are read from LDS one group ahead (two sets of
    // registers), so a group never starts by waiting for its own reads: 7-10 % on the 64-row
    // tile under long contractions (R=1, I=J=K=2048: 158 -> 143 us; R=16, I=J=K=512: 43.4 -> 40.2).
    auto mfma_block = [&](const float *tile) {
        constexpr int GQ = RT / RP;   // groups per quarter chunk
        constexpr int NG = NQ * GQ;   // groups of RP * 4 * CT MFMAs
        constexpr bool AHEAD = RT > 1;  // (the 32-row tile has a single fragment per group and loses 2-7 % by it)
        floatx4 af[2][RP];
#pragma unroll
        for (int k = 0; k < RP; ++k) af[0][k] = *reinterpret_cast<const floatx4 *>(&tile[(32 * k + m) * LDA + 4 * h]);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            if (!AHEAD && g > 0) {
#pragma unroll
                for (int k = 0; k < RP; ++k)
                    af[g & 1][k] = *reinterpret_cast<const floatx4 *>(
                        &tile[(32 * ((g % GQ) * RP + k) + m) * LDA + 8 * (g / GQ) + 4 * h]);
            }
            if (AHEAD && g + 1 < NG) {
                const int qn = (g + 1) / GQ, rn = ((g + 1) % GQ) * RP;
#pragma unroll
                for (int k = 0; k < RP; ++k)
                    af[(g + 1) & 1][k] =
                        *reinterpret_cast<const floatx4 *>(&tile[(32 * (rn + k) + m) * LDA + 8 * qn + 4 * h]);
            }
            const int q = g / GQ, rt0 = (g % GQ) * RP;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int k = 0; k < RP; ++k)
                        acc[rt0 + k][ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            af[g & 1][k][u], eb[ct][4 * q + u], acc[rt0 + k][ct], 0, 0, 0);
        }
    };

    // ---- steady state: prefetch chunk jc+1 unconditionally, contract chunk jc, then
    // consume the prefetch before the back edge; the ragged tail and the last chunk
    // are peeled so the loop body carries no masks.
    int cur = 0;
    int jc = jc0;
    for (; jc + 1 < full_end; ++jc) {
        load_tile_full(jc + 1);
        load_b_full(jc + 1);
        __builtin_amdgcn_sched_barrier(0);  // the prefetch is issued before the MFMA block, not sunk into it
        mfma_block(at + cur * BUF + wrow0 * LDA);
        store_tile(cur ^ 1);
        shift_and_exp();
        __syncthreads();
        cur ^= 1;
    }
    if (jc + 1 < jc1) {  // the next chunk is the masked tail
        load_tile_masked(jc + 1);
        load_b_masked(jc + 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_block(at + cur * BUF + wrow0 * LDA);
        store_tile(cur ^ 1);
        shift_and_exp();
        __syncthreads();
        cur ^= 1;
    }
    mfma_block(at + cur * BUF + wrow0 * LDA);

    // ---- epilogue: c = m + log(acc).  Register v of lane (h, m) holds row
    // 8*(v/4) + 4*h + v%4, column m of its 32 x 32 tile; the row part of the address
    // is wave-uniform apart from the lane half, so it lives in scalar registers.
    // Rows past I fall outside the buffer extent and are dropped by the hardware.
    // With a split contraction the raw sums and their shift go to the workspace instead.
    const bool split_out = p.splits > 1;  // wave-uniform
    const int crows = p.I - (i0 + wrow0);  // valid rows below this wavefront's first row
    float *obase = split_out ? p.part + (((int64_t)split * p.R + r) * p.I + (i0 + wrow0)) * (int64_t)p.K
                             : p.c + (int64_t)r * p.sc0 + (int64_t)(i0 + wrow0) * p.sc1;
    const uint32_t orow = split_out ? (uint32_t)p.K : (uint32_t)p.sc1;
    const __amdgpu_buffer_rsrc_t c_rsrc =
        make_rsrc(obase, crows > 0 ? (uint32_t)(((int64_t)(crows - 1) * orow + p.K) * 4) : 0u);
    const uint32_t c_row_bytes = orow * 4u;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (ncol[ct] >= p.K) continue;
        const uint32_t co = ((uint32_t)(4 * h) * orow + (uint32_t)ncol[ct]) * 4u;
        if (MODE != kPlain && split_out && itile == 0 && wm == 0 && h == 0)
            p.shift[((int64_t)split * p.R + r) * p.K + ncol[ct]] = mref[ct];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t trow = 32 * rt + 8 * (v / 4) + (v % 4);  // + 4h in the lane offset
                if (split_out)  // partial sums are read back by the merge kernel right away
                    buf_store_f32(acc[rt][ct][v], c_rsrc, co, trow * c_row_bytes);
                else if (MODE == kPlain)
                    buf_store_f32_out(p.stream_out != 0, acc[rt][ct][v], c_rsrc, co, trow * c_row_bytes);
                else
                    buf_store_f32_out(p.stream_out != 0, log_plus(acc[rt][ct][v], mref[ct]), c_rsrc, co,
                                      trow * c_row_bytes);
            }
    }
}

// Column maxima m[r,k] = max_j b[r,j,k] (clamped to +-1e38 with CLAMP: the shift of the two-kernel
// variant; a NaN wins).  A workgroup owns 256 columns of one batch (a lane 4 adjacent ones) and
// the rows [split * chunk, (split + 1) * chunk); its 4 wavefronts interleave over those rows and
// combine in LDS.  With splits > 1 the result of a split goes to m + split * R * K and a second
// launch of this kernel reduces over the splits.
// once: b is too large to be found in cache by whoever reads it next; it is read with
// non-temporal loads, and the workgroups of a die take consecutive batches (workgroups go to the
// 8 dies round-robin): 64 x 64 x 4096 in 9.7 us against 11.6.
template <bool CLAMP>
__global__ __launch_bounds__(256) void lm2exp_colmax_kernel(const float *__restrict__ b, float *__restrict__ m, int R,
                                                            int J, int K, int64_t sb0, int64_t sb1, int chunk,
                                                            int once) {
    __shared__ float part[4][256];
    const int blocks_per_batch = (K + 255) / 256;
    const unsigned total = gridDim.x;
    const unsigned logical =
        (once && total % kXcds == 0) ? (blockIdx.x % kXcds) * (total / kXcds) + blockIdx.x / kXcds : blockIdx.x;
    const int kb = logical % blocks_per_batch;
    const int rs = logical / blocks_per_batch;
    const int r = rs % R;
    const int split = rs / R;
    const int k0 = kb * 256;
    const int j0 = split * chunk;
    const int j1 = (j0 + chunk < J) ? j0 + chunk : J;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const float *br = b + (int64_t)r * sb0;
    float x[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = -__builtin_inff();
    const int kc = k0 + 4 * lane;
    const bool vec = kc + 3 < K && (sb1 % 4 == 0) && ((reinterpret_cast<uintptr_t>(br) & 15) == 0);
    int j = j0 + wave;
    if (vec && once) {
        for (; j + 12 < j1; j += 16) {  // four rows of the wavefront in flight
            floatx4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                v[u] = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(br + (int64_t)(j + 4 * u) * sb1 + kc));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) x[e] = max_nan(x[e], v[u][e]);
        }
    }
    for (; j < j1; j += 4) {
        const float *row = br + (int64_t)j * sb1;
        if (vec) {
            const floatx4 v = *reinterpret_cast<const floatx4 *>(row + kc);
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = max_nan(x[e], v[e]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (kc + e < K) x[e] = max_nan(x[e], row[kc + e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) part[wave][4 * lane + e] = x[e];
    __syncthreads();
    const int t = threadIdx.x;
    if (k0 + t < K) {
        const float y = max_nan(max_nan(part[0][t], part[1][t]), max_nan(part[2][t], part[3][t]));
        m[((int64_t)split * R + r) * K + k0 + t] = CLAMP ? clamp_shift(y) : y;
    }
}

// Rows per split of the batched column maxima: enough workgroups for 256 CUs (>= 1024), at
// least 64 rows each, at most 1024 splits.  More than 128 partials per column (few columns
// under a very long axis) are combined in two levels, 64 at a time first.
static int colmax_splits(int64_t R, int64_t J, int64_t K) {
    const int64_t base = R * ceil_div(K, 256);
    int64_t splits = base >= 1024 ? 1 : ceil_div(1024, base);
    if (splits > J / 64) splits = J / 64;
    if (splits > 1024) splits = 1024;
    return splits < 1 ? 1 : (int)splits;
}
static int colmax_mid_splits(int splits) { return splits > 128 ? (splits + 63) / 64 : 1; }

// ------------------------------------------------------------------ host
struct Lm2Variant {
    int rt, ct, wm, wn, nq;
    int mode;
};
// variant ids are 1-based in the C ABI (0 = choose by shape)
static const Lm2Variant kVariants[] = {
    {4, 1, 1, 4, 4, kOnline},   // 1: 128 x 128 tile, 4 waves each 128 x 32 (3 waves/SIMD)
    {4, 1, 1, 8, 4, kOnline},   // 2: 128 x 256 tile, 8 waves each 128 x 32
    {2, 1, 1, 4, 4, kOnline},   // 3: 64 x 128 tile
    {1, 1, 1, 4, 4, kOnline},   // 4: 32 x 128 tile
    {3, 1, 1, 4, 4, kOnline},   // 5: 96 x 128 tile (I = 96, 192, ... without padded rows)
    {4, 1, 1, 4, 2, kOnline},   // 6..11: the 128-, 64- and 32-row tiles with j-chunks of 16 and 24
    {4, 1, 1, 4, 3, kOnline},   //        (chunks of 48 were measured too: 20 more B registers, a
    {2, 1, 1, 4, 2, kOnline},   //        wavefront less per SIMD on the 128-row tile, 5-60 % slower)
    {2, 1, 1, 4, 3, kOnline},
    {1, 1, 1, 4, 2, kOnline},
    {1, 1, 1, 4, 3, kOnline},
    {1, 1, 4, 1, 4, kOnline},   // 12: 128 x 32 tile, the 4 waves stacked over rows (outputs of <= 32 columns)
    {1, 1, 2, 2, 4, kOnline},   // 13: 64 x 64 tile (outputs of <= 64 columns)
    {3, 1, 1, 4, 2, kOnline},   // 14, 15: the 96-row tile with j-chunks of 16 and 24
    {3, 1, 1, 4, 3, kOnline},
    {4, 1, 2, 4, 2, kPair},     // 16: 256 x 128 tile of 2 x 4 wavefronts, exact shift first, exp shared by a pair
    {2, 1, 2, 4, 2, kPair},     // 17: 128 x 128
    {2, 1, 2, 2, 2, kPair},     // 18: 128 x 64 tile of 2 x 2 wavefronts
    {1, 1, 2, 2, 2, kPair},     // 19: 64 x 64
    {3, 1, 2, 2, 2, kPair},     // 20: 192 x 64
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
constexpr size_t kDefaultLdsLimit = 64 * 1024;  // larger dynamic LDS must be opted into per kernel

// Measured on MI355X at R=64, I=J=256, K=4096: the 128-row tiles (64 accumulator
// registers, 3-4 wavefronts per SIMD) beat 256-row tiles of the same kernel (128 accumulator
// registers, 2 per SIMD) although b is then exponentiated once per row tile; so did they beat
// a two-sweep build (exact maximum first: 0.35-0.37 ms against 0.29-0.31 ms) and a two-launch
// build (column maxima by a separate kernel: 0.33 ms).  None of those is kept.
// Smaller grids want smaller row tiles: a 128-row tile amortises each exp over four
// MFMAs, but it only pays when there are enough tiles to keep 256 CUs busy with more
// than one workgroup each.  Rules fitted to sweeps of the variants over the shapes of
// the reference's benchmark grid (batch-1 squares 128..2048; R=64/384, n=256, m=k=64..1024):
//   < 1.5 workgroups of 64 rows per CU and a    the largest tile that leaves >= 128 tiles (the
//   long contraction (J >= 1280)                contraction is then cut over J)
//   some tile leaves >= 1 workgroup per CU      the one with the least modelled time (pick_tile)
//   none does                                   32 x 128   (+12..36 %)
static int find_variant(int rt, int wn, int mode, int nq = 4) {
    for (int v = 0; v < kNumVariants; ++v)
        if (kVariants[v].rt == rt && kVariants[v].ct == 1 && kVariants[v].wm == 1 && kVariants[v].wn == wn &&
            kVariants[v].nq == nq && kVariants[v].mode == mode)
            return v;
    return nq == 4 ? 0 : find_variant(rt, wn, mode);
}

static int find_variant_shape(int rt, int wm, int wn) {
    for (int v = 0; v < kNumVariants; ++v)
        if (kVariants[v].rt == rt && kVariants[v].ct == 1 && kVariants[v].wm == wm && kVariants[v].wn == wn &&
            kVariants[v].nq == 4 && kVariants[v].mode == kOnline)
            return v;
    return 0;
}

static int find_pair_variant(int rt, int wn = 2) {
    for (int v = 0; v < kNumVariants; ++v)
        if (kVariants[v].mode == kPair && kVariants[v].rt == rt && kVariants[v].wn == wn) return v;
    return 0;
}

// j-chunk of the 128-, 64- and 32-row tiles: 32, or 16 or 24 where those pad J less.  Per padded j
// they cost 3-4 % more (R=64, I=256, K=4096: J = 256 takes 281 us on chunks of 32, 287 / 297 on
// 16 / 24), so J = 16, 24, 40, 48, 72, 80, 144, 200 run 17, 8, 15, 13, 16, 12, 9, 6 % faster.
// J not a multiple of 4 (rows of a are then staged by element unless the caller padded them):
// chunks of 32, or of 16 where those shorten the padded contraction to 0.9 or less (J = 37, 45,
// 47: 21-23 % faster; 75, 106: 10-12 %; with less to gain they lose -- a chunk of 16 is twice
// the steps -- R=2, I=87, J=482, K=2925: 21 % slower) and on the 128-row tile, whose 32-wide
// chunk is 16 element loads per thread and step (rt = 4; timed on five such shapes: 4-19 % faster
// on chunks of 16, R=32, I=633, J=273, K=660: 104 -> 84 us).  Chunks of 24 do not divide the
// workgroup evenly and keep the slow staging for such J.
// large: a grid of more than nine 32-row tiles per CU.  There the tiles of 64 rows and more run
// 2 % FASTER on chunks of 16 than on chunks of 32 at equal padding (median over 68 large grids, for
// each of the three tile heights; on small grids they are 0-6 % slower, as above): the penalty of
// the 16-wide chunk turns into a bonus.
static int pick_chunk(int64_t J, int rt = 0, bool large = false) {
    if (J % 4 != 0) return (10 * ceil_div(J, 16) * 16 <= 9 * ceil_div(J, 32) * 32 || rt == 4) ? 2 : 4;
    int nq = 4;
    int64_t best = ceil_div(J, 32) * 32 * 100;
    const int cand[2] = {2, 3};
    const int64_t penalty[2] = {large && rt >= 2 ? 98 : 103, 104};
    for (int c = 0; c < 2; ++c) {
        const int64_t cost = ceil_div(J, 8 * cand[c]) * 8 * cand[c] * penalty[c];
        if (cost < best) {
            best = cost;
            nq = cand[c];
        }
    }
    return nq;
}

// Tile for a grid of R x I rows and K columns among 128 x 128, 96 x 128, 64 x 128, 32 x 128 (rows
// up to 32 * max_rt) and (wide = true) 128 x 256; returns the rows in units of 32 (4, 3, 2, 1; 8
// stands for 128 x 256), or 0 when none of them leaves a workgroup per CU.
// Modelled time: T = tiles per CU (256 CUs), each costing rt MFMA blocks plus an overhead that
// does not shrink with the tile (the exp / shift work of the b chunk, loads, barriers: 0.75
// blocks, less without the exp work), counted in quarter blocks.  A CU holds `res` workgroups at a
// time (3, four of 64-row tiles, six of 32-row tiles, one wide); they share the matrix pipe, so a full round costs
// the sum of its tiles, but a last round with a single workgroup runs at about 2/3 speed (one
// wavefront per SIMD hides little latency) and one with two at ~0.8: a tail penalty, fading when
// T is large (workgroups are dispatched as others finish).  The wide tile costs 6.5 % more per row
// (measured on large grids) and only ever wins by avoiding such a tail.
// Fitted at R=384 and R=64, I=J=64..1024, K=256: ranks the tiles as measured in 26 of 28 shapes
// (both misses within 5 %); I = 96, 160, 192, 288 move to 96 rows (-15..23 %), I = 320 to 64.
static int pick_tile(int64_t R, int64_t I, int64_t K, int overhead_quarters, bool wide, int max_rt = 4,
                     int64_t chunks = 0) {
    const int64_t kFill = 256, kCuCount = 256;  // at least one workgroup per CU
    int best = 0;
    int64_t best_cost = 0;
    const int64_t ct128 = ceil_div(K, 128);
    // Grids of fewer than four 128-row tiles per CU (chunks > 0: the caller contracts that many
    // chunks of 32): the busiest CU decides.  It holds q = ceil(tiles / 256) tiles of
    // chunks * (rt + 1/4) + 3 rt blocks each (the exp work of a chunk does not shrink with the
    // tile; prologue and epilogue do), 10 % more for a tile that is alone on its CU.  Fitted to
    // 155 shapes (I = 128..768, J = 96..640, K = 256..2048, 200..1280 128-row tiles) timed on all
    // four tiles: on the 137 below 1024 tiles the mean regret against the best tile is 0.3 %
    // (the tail model below: 2.4 %, 13 shapes more than 10 % off, e.g. 576-640 tiles of 128 rows
    // where 64 rows are 10 % ahead); from 1024 tiles on short contractions favour the 64-row tile
    // by more than either model says, and the tail model is kept.
    if (chunks > 0 && R * ceil_div(I, 128) * ct128 < 1024) {
        for (int rt = max_rt; rt >= 1; --rt) {
            const int64_t q = ceil_div(R * ceil_div(I, 32 * rt) * ct128, kCuCount);
            const int64_t cost = q * (chunks * (4 * rt + 1) + 12 * rt) * (q == 1 ? 11 : 10);
            if (best == 0 || cost < best_cost) {
                best = rt;
                best_cost = cost;
            }
        }
        return best;
    }
    auto consider = [&](int id, int64_t n, int64_t c, int res) {
        if (n < kFill) return;
        const int64_t T = ceil_div(n, kCuCount);
        const int64_t rem = T % res;
        int64_t tail = 0;  // in 1/20 of a tile
        if (res > 1 && rem == 1) tail = 10;
        else if (res > 1 && rem == 2) tail = res == 3 ? 4 : 6;
        else if (res > 1 && rem == 3) tail = 2;
        if (T > 4) tail = tail * 4 / T;
        const int64_t cost = T * c * 20 + tail * c;
        if (best == 0 || cost < best_cost) {
            best = id;
            best_cost = cost;
        }
    };
    const int64_t ct = ceil_div(K, 128);
    for (int rt = max_rt; rt >= 1; --rt)
        consider(rt, R * ceil_div(I, 32 * rt) * ct, 4 * rt + overhead_quarters, rt == 1 ? 6 : (rt == 2 ? 4 : 3));
    if (wide && max_rt == 4 && K % 256 == 0)
        consider(8, R * ceil_div(I, 128) * (K / 256), (2 * (16 + overhead_quarters) * 213) / 200, 1);
    return best;
}

// 64-column tiles of the paired kernel where tiles of 128 columns would stand partly empty:
// K = 180 is three tiles of 64 columns or two of 128.  Taken when the 64-column tiling covers
// at most 0.85 of the padded columns -- or 0.92 under a long contraction on a tall matrix
// (J >= 256, I >= 512) -- on grids of two such tiles per CU and more; 192 or 128 rows,
// whichever pads I less.  Timed on 48 large grids with
// K = 144..3168: R=384, I=2039, J=420, K=180 1344 -> 1139 us; R=64, I=2085, J=772, K=268
// 688 -> 531; R=128, I=1383, J=1404, K=144 1014 -> 793; R=384, I=358, J=472, K=192 299 -> 234;
// R=16, I=1755, J=268, K=652 (0.92) 120 -> 102; between 0.85 and 0.92 on short contractions
// the 96-row online tile is as good or better, and under J < 128 the online tiles are level or
// ahead whatever the padding (R=32, I=2496, J=112, K=276: 65-67 us on either).  Rows of a that are not 16-byte aligned take them too (R=146, I=586, J=317,
// K=146: 138 -> 112 us; R=45, I=3374, J=211, K=144: 162 -> 126), and smaller grids whose K
// leaves a quarter of the 128-column tiling empty (K = 129..192) take the 64 x 64 tile of the
// same kernel from 100 tiles on (R=3, I=2878, J=587, K=158: 45 -> 32 us; R=6, I=1159, J=2879,
// K=159: 114 -> 95).  Over 200 random shapes with K = 128 m + 1..64 on which every tile was
// timed: 4.7 % -> 2.8 % (mean) behind the best tile.
static int pair64_variant(int64_t R, int64_t I, int64_t J, int64_t K) {
    if (K <= 64) return -1;
    const int64_t c128 = ceil_div(K, 128) * 128, c64 = ceil_div(K, 64) * 64;
    if (J >= 128 && I > 96 && (100 * c64 <= 85 * c128 || (100 * c64 <= 92 * c128 && J >= 256 && I >= 512))) {
        const int rt = ceil_div(I, 192) * 192 <= ceil_div(I, 128) * 128 ? 3 : 2;
        if (R * ceil_div(I, 64 * rt) * (c64 / 64) >= 512) return find_pair_variant(rt, 2);
    }
    if (J >= 192 && I > 64 && 100 * c64 <= 76 * c128 && R * ceil_div(I, 64) * (c64 / 64) >= 100)
        return find_pair_variant(1, 2);
    return -1;
}

static int choose_variant(int64_t R, int64_t I, int64_t J, int64_t K) {
    // Outputs of at most 32 (64) columns would leave three (two) of the four wavefronts of a
    // 128-column tile idle: the wavefronts are stacked over rows instead (128 x 32 and 64 x 64
    // tiles).  R=31, I=2527, J=2423, K=20: 479 -> 269 us; R=26, I=820, J=2949, K=14: 187 -> 91;
    // R=96, I=2932, J=135, K=34: 112 -> 81.
    // Whatever the number of tiles: few of them under a long contraction are cut over J like any
    // other tile, and over 250 random shapes with K = 9..64 (every tile timed) a threshold of 96
    // tiles left the rule 8.6 % (mean) behind the best tile -- R=30, I=283, J=2788, K=10: 72 us on
    // 32 x 128 tiles against 39 -- where taking the narrow tiles throughout stands 4.0 % behind.
    // Large grids of 33..64 columns go to the paired-wavefront kernel's 128 x 64 tile when its
    // 128 rows pad I little more than 64 would (at most 1.1x): the exps of a column shared by two
    // wavefronts, 10-25 % ahead from some 600 tiles of 64 rows on, from 200 under a contraction of
    // 32 chunks and more (R=101, I=1510, J=48, K=48: 23 -> 18 us; R=436, I=89, J=1384, K=46: 127 ->
    // 113; R=14, I=2464, J=2688, K=48: 180 -> 134), which takes the rule to 2.9 % over those 250
    // shapes and 200 others.
    if (K <= 32 && I > 64) return find_variant_shape(1, 4, 1);
    if (K <= 64 && I > 32) {
        const int64_t t64 = R * ceil_div(I, 64);
        if ((t64 >= 600 || (t64 >= 200 && J >= 32 * 31 + 1)) && 10 * ceil_div(I, 128) * 128 <= 11 * ceil_div(I, 64) * 64)
            return find_pair_variant(2, 2);
        return find_variant_shape(1, 2, 2);
    }
    {
        const int pv = pair64_variant(R, I, J, K);
        if (pv >= 0) return pv;
    }
    const int64_t kFill = 384;
    const int64_t ct = ceil_div(K, 128);
    // Large grids of 256-row tiles under a contraction of a few hundred: the paired-wavefront
    // kernel (exact shift first, no rescaling, an exp per workgroup and element).  Its time does
    // not depend on the data; the online kernels rescale whenever a chunk towers over the shift
    // so far, which b ~ N(-50, 20) does in most of the early chunks.  Measured at K = 4096 with
    // that b: R=64 I=J=256 281 us against 293; with b ~ N(0, 1): 280 against 284, R=16 77
    // against 80, R=32 I=1024 K=2048 271 against 280, J = 512 531 against 533; slower with
    // fewer than two tiles per CU (R=8: +9 %), J = 192 (+1 %), or J not a multiple of 4 (+4 %).
    // Both kernels run in steps of the busiest CU's tile count: measured at I = J = 256, K = 1024..
    // 4096, R = 8..64 the paired tile takes 34.3 us per ceil(tiles / 256) and the 128-row tile
    // 18.5 us per ceil(2 tiles / 256), so with 513..640, 769..896 or 1025..1152 paired tiles the
    // online kernel is 4-22 % ahead (576 tiles: 108 against 90-95 us) and the pair is taken only
    // where 1.85 of its steps undercut the online kernel's.
    const int64_t i256 = ceil_div(I, 256);
    const int64_t t256 = R * i256 * ct;
    if (J >= 224 && J <= 512 && J % 4 == 0 && I >= 240 && i256 * 256 * 100 <= I * 107 && t256 >= 512 &&
        185 * ceil_div(t256, 256) <= 100 * ceil_div(2 * t256, 256))
        return find_pair_variant(4, 4);
    const int64_t n128 = R * ceil_div(I, 128) * ct, n64 = R * ceil_div(I, 64) * ct;
    int rt;
    if (I <= 32 || J <= 32) {
        // J <= 32 is a single chunk: a workgroup is load, one MFMA block, log and store in
        // sequence with nothing to overlap inside it, and the call is bound by writing c; many
        // small workgroups hide the most latency (measured 20-35 % ahead of the 128-row tile)
        rt = 1;
    } else if (I <= 64) {
        rt = (n64 >= kFill || J >= 1280) ? 2 : 1;
    } else if (J >= 1280 && n64 < kFill) {
        // at most 1.5 workgroups per CU and a long contraction: it will be cut over J, which
        // fills the chip; take the largest tile that leaves >= 128 tiles
        rt = n128 >= 128 ? 4 : (n64 >= 128 ? 2 : 1);
    } else if ((rt = pick_tile(R, I, K, 3, true, (J <= 64 || (J <= 128 && n128 >= 1024 && n128 < 6144)) ? 2 : 4,
                               ceil_div(J, 32))) != 0) {
        // (two chunks: 64 rows at most (+2..13 %); three or four chunks on 4..24 128-row tiles
        // per CU as well: timed on 47 such shapes the 64-row tile is 1-29 % ahead of the 128-row
        // one on 45 and 1-2 % behind on 2; with more tiles, or longer contractions, 128 rows win)
        if (rt == 8) return find_variant(4, 8, kOnline);
    } else {
        rt = 1;
    }
    return find_variant(rt, 4, kOnline, pick_chunk(J, rt, R * ceil_div(I, 32) * ct > 2304));
}

template <int RT, int CT, int WM, int WN, int NQ, bool VEC, int MODE>
static int launch_k(const Lm2Args &args, hipStream_t stream) {
    constexpr int TM = 32 * RT * WM;
    constexpr int LDA = 8 * NQ + 4;
    constexpr int NT = WM * WN * kWave;
    constexpr bool REGULAR = (NT % (2 * NQ) == 0) && (TM * 2 * NQ % NT == 0);  // as in the kernel
    constexpr size_t lds = (size_t)2 * (TM * LDA + (REGULAR ? 0 : 4 * NT)) * sizeof(float);
    auto k = lm2exp_kernel<RT, CT, WM, WN, NQ, VEC, MODE>;
    if (lds > kDefaultLdsLimit) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(k, dim3((unsigned)args.padded_wgs), dim3(WM * WN * kWave), lds, stream, args);
    return (int)hipGetLastError();
}

template <int RT, int CT, int WM, int WN, int NQ, int MODE>
static int launch_v(const Lm2Args &args, bool vec, hipStream_t stream) {
    return vec ? launch_k<RT, CT, WM, WN, NQ, true, MODE>(args, stream)
               : launch_k<RT, CT, WM, WN, NQ, false, MODE>(args, stream);
}

template <int RT, int WN, int NQ, int LOADA>
static int launch_pair_k(const Lm2Args &args, hipStream_t stream) {
    constexpr int TM = 64 * RT;
    constexpr size_t lds = (size_t)(2 * (2 * NQ) * (TM * 4) + 2 * 2 * WN * 64 * 2 * NQ) * sizeof(float);
    static_assert(lds <= kDefaultLdsLimit, "the paired-wavefront tiles fit the default dynamic LDS limit");
    hipLaunchKernelGGL((lm2exp_pair_kernel<RT, WN, NQ, LOADA>), dim3((unsigned)args.padded_wgs), dim3(128 * WN), lds,
                       stream, args);
    return (int)hipGetLastError();
}

// loada: how the a tile is read (kLoadVec, kLoadByCol, kLoadByRow); lanes along i need a tile
// height that divides the workgroup, which 192 rows do not: such a call reads by column.
template <int RT, int WN>
static int launch_pair(const Lm2Args &args, int loada, hipStream_t stream) {
    if (loada == kLoadVec) return launch_pair_k<RT, WN, 2, kLoadVec>(args, stream);
    if constexpr (RT != 3) {
        if (loada == kLoadByRow) return launch_pair_k<RT, WN, 2, kLoadByRow>(args, stream);
    }
    return launch_pair_k<RT, WN, 2, kLoadByCol>(args, stream);
}

struct Lm2Plan {
    int variant;           // index into kVariants
    int splits;            // workgroups sharing one output tile
    int chunks_per_split;  // j-chunks each of them contracts
};

constexpr int kMaxSplits = 32;

// Small grids under a contraction of some length -- at most nine 32-row tiles per CU, J >= 160,
// 0.1 GFLOP and more -- get the height of their tile and the cut over J chosen TOGETHER, by
// modelled time.  (choose_variant's rules fix the tile first and choose_splits then cuts it; on
// such grids what counts is how many whole workgroups the busiest CU ends up with, which only
// the pair (tile, cut) decides: I=J=K=1536 takes 80 us on 96-row tiles cut four ways -- 768
// workgroups, three per CU -- against 93 on the 128-row tile the rules pick; R=12, I=420, J=2688,
// K=273: 108 against 129.)  The model: a workgroup's chain is its chunks times (MFMAs + the exp
// work of a chunk, which does not shrink with the tile), the busiest of the 256 CUs runs
// q = ceil(workgroups / 256) chains at 77 % of that rate alone, 92 % with two, in full from three
// on, a launch costs 4.8 us, a cut 4.1 us more plus its partial sums' trip through memory at
// 2.46 TB/s.  Constants fitted to 28 tile-and-cut combinations on each of 30 batch-1..3 shapes of
// 640..3072; on 46 other random shapes of the region its pick is 0.9 % (mean) behind the best
// combination measured, the rules' 3.1 %, with the worst case 6 % against 20 %.  Outside the
// region the rules stay: they are ahead on short contractions (J < 160: 2 % against 7 %), on the
// reference's grid shapes below 0.1 GFLOP and where J wants j-chunks of 16 or 24 (the exp work per
// chunk is fitted for chunks of 32 only), and level on larger grids.
struct TileCut {
    int rt, splits;
    double us;
};
static bool joint_region(int64_t R, int64_t I, int64_t J, int64_t K) {
    const int64_t n32 = R * ceil_div(I, 32) * ceil_div(K, 128);
    return K > 64 && I > 32 && J >= 160 && pick_chunk(J) == 4 && n32 <= 2304 &&
           (double)R * (double)I * (double)J * (double)K >= 1e8;
}
// splits_fixed: 0 = any cut, n >= 1 = exactly n (1: uncut)
static TileCut choose_tile_and_cut(int64_t R, int64_t I, int64_t J, int64_t K, int splits_fixed) {
    constexpr int nq = 4;
    const int64_t units = ceil_div(J, 8 * nq);
    TileCut best{1, 1, 1e300};
    for (int rt = 1; rt <= 4; ++rt) {
        const int64_t tiles = R * ceil_div(I, 32 * rt) * ceil_div(K, 128);
        const double unit_us = (256.0 * nq * rt + 107.5 * nq) / 2400.0;
        for (int sp = 1; sp <= kMaxSplits && (sp == 1 || 2 * sp <= units); ++sp) {
            if (splits_fixed && sp != splits_fixed) continue;
            const int64_t per = ceil_div(units, sp);
            if (!splits_fixed && ceil_div(units, per) != sp) continue;  // the same cut as a smaller count
            const int64_t q = ceil_div(tiles * ceil_div(units, per), 256);
            const double eff = q >= 3 ? 1.0 : (q == 2 ? 0.92 : 0.77);
            double us = 4.8 + (double)q * (double)per * unit_us / eff;
            if (sp > 1) us += 4.1 + (double)(sp + 1) * (double)(R * I * K) * 4.0 / 2.46e6;
            if (us < best.us) best = {rt, sp, us};
        }
    }
    return best;
}

// splits_req: 0 = decide here, 1 = never split, n > 1 = split n ways (capped).
// A small grid with a long contraction is cut over J so that the 256 CUs have work:
// e.g. batch 1, I=J=K=1024 is 64 tiles of 128 x 128 but 32 chunks deep.
static Lm2Plan make_plan(int64_t R, int64_t I, int64_t J, int64_t K, int variant, int splits_req) {
    Lm2Plan pl;
    // (the 64-column tiles of the paired kernel go before the joint model, which knows the
    // 128-column tiles only)
    const bool joint = variant < 1 && joint_region(R, I, J, K) && pair64_variant(R, I, J, K) < 0;
    TileCut tc{1, 1, 0.0};
    if (joint) {
        tc = choose_tile_and_cut(R, I, J, K, splits_req);
        if (tc.us >= 1e300) tc = choose_tile_and_cut(R, I, J, K, 0);  // a cut the contraction is too short for
        pl.variant = find_variant(tc.rt, 4, kOnline, pick_chunk(J, tc.rt));
    } else {
        pl.variant = (variant >= 1) ? variant - 1 : choose_variant(R, I, J, K);
    }
    const Lm2Variant &vr = kVariants[pl.variant];
    const int64_t chunks = ceil_div(J, 8 * vr.nq);
    const int64_t base = R * ceil_div(I, 32 * vr.rt * vr.wm) * ceil_div(K, 32 * vr.ct * vr.wn);
    int64_t splits = 1;
    if (vr.mode == kPlain)
        splits = 1;  // this build does not write partial sums
    else if (splits_req == 0 && joint)
        splits = tc.splits;
    else if (splits_req == 0)
        // measured: R=16 I=J=K=512 (256 tiles, 16 chunks) is 1.5x slower split, batch-1
        // squares of 512..1536 are 1.2-1.9x faster; the model below reproduces both
        splits = choose_splits(base, chunks, 4 * vr.nq * vr.rt * vr.ct, R * I * K, 2, kMaxSplits, false);
    else
        splits = splits_req;
    if (splits > kMaxSplits) splits = kMaxSplits;
    if (splits > chunks) splits = chunks;
    if (splits < 1) splits = 1;
    const int64_t per = ceil_div(chunks, splits);
    pl.splits = (int)ceil_div(chunks, per);
    pl.chunks_per_split = (int)per;
    return pl;
}

static size_t plan_workspace(const Lm2Plan &pl, int64_t R, int64_t I, int64_t K) {
    if (pl.splits <= 1) return 0;
    return ((size_t)pl.splits * R * I * K + (size_t)pl.splits * R * K) * sizeof(float);
}

// csrc/lt2exp.hip: the sweep of csrc/lt2exp_smallk.hpp with the rows of a as the weights
bool lm2exp_takes_sweep(int64_t R, int64_t I, int64_t J, int64_t K, bool a_aligned);
int lm2exp_sweep(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                 const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], hipStream_t stream);
int lt2exp_sweep_name(int64_t R, int64_t S, int64_t J, int64_t K, bool w_aligned, char *buf, size_t buf_bytes);
// csrc/lt2exp.hip: the lane-per-column kernel of csrc/lt2exp_cols.hpp with the rows of a as the weights
bool lm2exp_takes_cols(int64_t R, int64_t I, int64_t J, int64_t K, bool a_dense, double margin);
int lm2exp_cols(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J, int64_t K,
                const int64_t sa[3], const int64_t sb[3], const int64_t sc[3], hipStream_t stream);
int lm2exp_cols_name(int64_t J, bool a_dense, char *buf, size_t buf_bytes);

}  // namespace trt

using namespace trt;

extern "C" int trt_lm2exp_variant_count(void) { return kNumVariants; }

extern "C" size_t trt_lm2exp_workspace_bytes(int64_t R, int64_t I, int64_t J, int64_t K, int variant,
                                             int splits) {
    if (R <= 0 || I <= 0 || J <= 0 || K <= 0 || variant < 0 || variant > kNumVariants || splits < 0) return 0;
    return plan_workspace(make_plan(R, I, J, K, variant, splits), R, I, K);
}

namespace trt {
// (for the split-bf16 entry, csrc/lm2exp_bf16.hip: outputs of at most 16 rows and 32 columns per batch
// are bound by the reads of b, not by the matrix pipe, and go to the fp32 entry's kernel for them --
// R=8192, I=1, J=256, K=16: 97 -> 26 us; R=3000, I=7, J=1001, K=11: 145 -> 54; the 32-row kernel against
// the bf16 tiles is 0.6 to 1.2 times their speed and is not handed to)
bool lm2exp_takes_jsplit16(int64_t R, int64_t I, int64_t J, int64_t K) {
    return jsplit16_applies(I, J, K) && jsplit16_score(R, J, K) > 0.0;
}
}  // namespace trt

extern "C" int trt_lm2exp_f32(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J,
                              int64_t K, const int64_t sa[3], const int64_t sb[3], const int64_t sc[3],
                              int variant, int splits, void *workspace, size_t workspace_bytes, void *stream) {
    if (!a || !b || !c || !sa || !sb || !sc) return TRT_E_INVALID;
    if (R <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (variant < 0 || variant > kNumVariants || splits < 0) return TRT_E_INVALID;
    if (sc[2] != 1 || sa[2] < 0 || sb[2] < 0) return TRT_E_LAYOUT;
    for (int d = 0; d < 2; ++d)
        if (sa[d] < 0 || sb[d] < 0 || sc[d] < 0) return TRT_E_LAYOUT;
    if (sc[1] < K || sc[0] < 0) return TRT_E_LAYOUT;  // output rows must not overlap (stores rely on it)
    const int64_t lim = (int64_t)1 << 30;
    if (R >= lim || I >= lim || J >= lim || K >= lim) return TRT_E_RANGE;
    // byte offsets inside one batch slab of a, b and c are 32-bit (buffer addressing)
    if (J * sb[1] + K * sb[2] >= lim || I * sa[1] + J * sa[2] >= lim || I * sc[1] + K >= lim || I * K >= lim)
        return TRT_E_RANGE;

    // at most 4 columns under a long contraction: a sweep over a on the vector ALU
    if (variant == 0 && splits <= 1 &&
        lm2exp_takes_sweep(R, I, J, K, sa[2] == 1 && sa[0] % 4 == 0 && sa[1] % 4 == 0 &&
                                           (reinterpret_cast<uintptr_t>(a) & 15) == 0))
        return lm2exp_sweep(a, b, c, R, I, J, K, sa, sb, sc, static_cast<hipStream_t>(stream));
    // at most 64 columns under few rows per batch: one tile per batch, its contraction cut over the
    // wavefronts (csrc/lm2exp_jsplit.hpp)
    if (variant == 0 && splits <= 1 &&
        jsplit_pays(R, I, J, K, sa[2] == 1 && sa[0] % 4 == 0 && sa[1] % 4 == 0 && (reinterpret_cast<uintptr_t>(a) & 15) == 0))
        return launch_lm2exp_jsplit(a, b, c, R, I, J, K, sa, sb, sc, static_cast<hipStream_t>(stream));
    // a contraction of at most 16 terms over many batches: a lane per output column
    if (variant == 0 && splits <= 1 && lm2exp_takes_cols(R, I, J, K, sa[2] == 1, 0.0))
        return lm2exp_cols(a, b, c, R, I, J, K, sa, sb, sc, static_cast<hipStream_t>(stream));
    Lm2Plan pl = make_plan(R, I, J, K, variant, splits);
    // a trailing stride of a other than 1 (a transposed or strided view): only the
    // paired-wavefront kernel reads such a tile; a call that would take another kernel takes
    // the paired tile of the same height instead, cut over J no further than the caller's
    // workspace (sized without knowledge of the strides) holds
    if (sa[2] != 1 && kVariants[pl.variant].mode != kPair) {
        if (variant >= 1) return TRT_E_LAYOUT;
        const bool narrow = K <= 64;
        const int64_t big_tiles = R * ceil_div(I, 256) * ceil_div(K, 128);
        const int pv = narrow ? find_pair_variant(I > 64 ? 2 : 1, 2)
                       : I > 128 && big_tiles >= 256 ? find_pair_variant(4, 4)
                       : I > 64 ? find_pair_variant(2, 4)
                                : find_pair_variant(1, 2);
        pl = make_plan(R, I, J, K, 1 + pv, splits);
        while (pl.splits > 1 && (!workspace || plan_workspace(pl, R, I, K) > workspace_bytes))
            pl = make_plan(R, I, J, K, 1 + pv, pl.splits - 1);
    }
    const int v = pl.variant;
    const Lm2Variant &vr = kVariants[v];
    Lm2Args args;
    args.a = a; args.b = b; args.c = c;
    args.part = nullptr; args.shift = nullptr;
    args.R = (int)R; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sa0 = sa[0]; args.sa1 = sa[1];
    args.sb0 = sb[0]; args.sb1 = sb[1];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.sa2 = sa[2];
    args.sb2 = sb[2];
    args.i_tiles = (int)ceil_div(I, 32 * vr.rt * vr.wm);
    args.n_tiles = (int)ceil_div(K, 32 * vr.ct * vr.wn);
    args.splits = pl.splits;
    args.chunks_per_split = pl.chunks_per_split;
    args.total_wgs = (int64_t)R * args.i_tiles * args.n_tiles * pl.splits;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    args.stream_out = rows_16_byte_aligned(c, sc[0], sc[1]);
    if (args.padded_wgs >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pl.splits > 1) {
        const size_t need = plan_workspace(pl, R, I, K);
        if (!workspace || workspace_bytes < need) return TRT_E_WORKSPACE;
        args.part = static_cast<float *>(workspace);
        args.shift = args.part + (size_t)pl.splits * R * I * K;
    }
    // (rows of a that start 16-byte aligned: J itself need not be a multiple of 4 when the row
    // stride is -- a padded copy -- since the piece that straddles J is masked by element)
    const bool vec = (sa[0] % 4 == 0) && (sa[1] % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
    int st;
    if (vr.mode == kPair) {
        const int loada = (vec && sa[2] == 1) ? kLoadVec : ((sa[2] != 1 && sa[1] < sa[2]) ? kLoadByRow : kLoadByCol);
        if (vr.wn == 4) {
            st = vr.rt == 4 ? launch_pair<4, 4>(args, loada, s) : launch_pair<2, 4>(args, loada, s);
        } else {
            switch (vr.rt) {
                case 3: st = launch_pair<3, 2>(args, loada, s); break;
                case 2: st = launch_pair<2, 2>(args, loada, s); break;
                default: st = launch_pair<1, 2>(args, loada, s); break;
            }
        }
        if (st != 0 || pl.splits <= 1) return st;
        launch_lm2exp_merge(args.part, args.shift, c, R, I, K, pl.splits, sc[0], sc[1], s);
        return (int)hipGetLastError();
    }
    switch (v) {
        case 0: st = launch_v<4, 1, 1, 4, 4, kOnline>(args, vec, s); break;
        case 1: st = launch_v<4, 1, 1, 8, 4, kOnline>(args, vec, s); break;
        case 2: st = launch_v<2, 1, 1, 4, 4, kOnline>(args, vec, s); break;
        case 3: st = launch_v<1, 1, 1, 4, 4, kOnline>(args, vec, s); break;
        case 5: st = launch_v<4, 1, 1, 4, 2, kOnline>(args, vec, s); break;
        case 6: st = launch_v<4, 1, 1, 4, 3, kOnline>(args, vec, s); break;
        case 7: st = launch_v<2, 1, 1, 4, 2, kOnline>(args, vec, s); break;
        case 8: st = launch_v<2, 1, 1, 4, 3, kOnline>(args, vec, s); break;
        case 9: st = launch_v<1, 1, 1, 4, 2, kOnline>(args, vec, s); break;
        case 10: st = launch_v<1, 1, 1, 4, 3, kOnline>(args, vec, s); break;
        case 11: st = launch_v<1, 1, 4, 1, 4, kOnline>(args, vec, s); break;
        case 12: st = launch_v<1, 1, 2, 2, 4, kOnline>(args, vec, s); break;
        case 13: st = launch_v<3, 1, 1, 4, 2, kOnline>(args, vec, s); break;
        case 14: st = launch_v<3, 1, 1, 4, 3, kOnline>(args, vec, s); break;
        default: st = launch_v<3, 1, 1, 4, 4, kOnline>(args, vec, s); break;
    }
    if (st != 0 || pl.splits <= 1) return st;
    launch_lm2exp_merge(args.part, args.shift, c, R, I, K, pl.splits, sc[0], sc[1], s);
    return (int)hipGetLastError();
}

// Name of the contraction kernel a trt_lm2exp_f32 call with these arguments launches, as a
// profiler prints it (host only; a_vec: a has a unit trailing stride and base and leading
// strides that are multiples of 16 bytes).  Benchmarks use it to look their kernel up in
// profiler output.
extern "C" int trt_lm2exp_kernel_name(int64_t R, int64_t I, int64_t J, int64_t K, int variant, int splits, int a_vec,
                                      char *buf, size_t buf_bytes) {
    if (!buf || buf_bytes == 0 || R <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (variant < 0 || variant > kNumVariants || splits < 0) return TRT_E_INVALID;
    if (variant == 0 && splits <= 1 && lm2exp_takes_sweep(R, I, J, K, a_vec != 0))
        return lt2exp_sweep_name(R, I, J, K, true, buf, buf_bytes);
    if (variant == 0 && splits <= 1 && jsplit_pays(R, I, J, K, a_vec != 0)) {
        const int n = jsplit_kernel_name(buf, buf_bytes, I, J, K, a_vec != 0);
        return n > 0 && (size_t)n < buf_bytes ? 0 : TRT_E_RANGE;
    }
    if (variant == 0 && splits <= 1 && lm2exp_takes_cols(R, I, J, K, true, 0.0)) return lm2exp_cols_name(J, true, buf, buf_bytes);
    const Lm2Variant &vr = kVariants[make_plan(R, I, J, K, variant, splits).variant];
    int n;
    if (vr.mode == kPair)
        n = snprintf(buf, buf_bytes, "trt::lm2exp_pair_kernel<%d, %d, %d, %d>", vr.rt, vr.wn, vr.nq,
                     a_vec ? kLoadVec : kLoadByCol);
    else
        n = snprintf(buf, buf_bytes, "trt::lm2exp_kernel<%d, %d, %d, %d, %d, %s, %d>", vr.rt, vr.ct, vr.wm, vr.wn, vr.nq,
                     a_vec ? "true" : "false", vr.mode);
    return n > 0 && (size_t)n < buf_bytes ? 0 : TRT_E_RANGE;
}

// Batched column maxima m[r,k] = max_j b[r,j,k] of an R x J x K fp32 tensor (a NaN wins, as in
// torch.amax); with `clamp` the result is clamped to +-1e38, which is exactly the shift the
// contraction kernels subtract (baselines/lm2exp.py:11-12, baselines/lt2exp.py:15-19).  Few
// columns under a long reduced axis are cut over J (partial maxima in the workspace, then the
// same kernel over the partials).
extern "C" size_t trt_colmax_batched_workspace_bytes(int64_t R, int64_t J, int64_t K) {
    if (R <= 0 || J <= 0 || K <= 0) return 0;
    const int splits = colmax_splits(R, J, K);
    const int mid = colmax_mid_splits(splits);
    return splits > 1 ? (size_t)(splits + (mid > 1 ? mid : 0)) * R * K * sizeof(float) : 0;
}

extern "C" int trt_colmax_batched_f32(const float *b, float *m, int64_t R, int64_t J, int64_t K,
                                      const int64_t sb[3], int clamp, void *workspace, size_t workspace_bytes,
                                      void *stream) {
    if (!b || !m || !sb) return TRT_E_INVALID;
    if (R <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (sb[2] != 1 || sb[0] < 0 || sb[1] < 0) return TRT_E_LAYOUT;
    const int64_t lim = (int64_t)1 << 30;
    if (R >= lim || J >= lim || K >= lim) return TRT_E_RANGE;
    int splits = colmax_splits(R, J, K);
    const int chunk = (int)ceil_div(J, splits);
    splits = (int)ceil_div(J, chunk);
    const int64_t blocks = R * ceil_div(K, 256) * splits;
    if (blocks >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int once = R * J * K * (int64_t)sizeof(float) >= ((int64_t)32 << 20);  // as the other max reductions
    if (splits > 1) {
        const int mid = colmax_mid_splits(splits);
        if (!workspace || workspace_bytes < (size_t)(splits + (mid > 1 ? mid : 0)) * R * K * sizeof(float))
            return TRT_E_WORKSPACE;
        float *part = static_cast<float *>(workspace);
        hipLaunchKernelGGL(lm2exp_colmax_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, b, part, (int)R, (int)J,
                           (int)K, sb[0], sb[1], chunk, once);
        // reduce over the splits: the partials are an R x splits x K tensor with strides (K, R*K, 1)
        const unsigned blocks2 = (unsigned)(R * ceil_div(K, 256));
        if (mid > 1) {  // 64 partials at a time first
            float *part2 = part + (int64_t)splits * R * K;
            hipLaunchKernelGGL(lm2exp_colmax_kernel<false>, dim3(blocks2 * (unsigned)mid), dim3(256), 0, s, part, part2,
                               (int)R, splits, (int)K, K, R * K, 64, 0);
            part = part2;
            splits = mid;
        }
        if (clamp)
            hipLaunchKernelGGL(lm2exp_colmax_kernel<true>, dim3(blocks2), dim3(256), 0, s, part, m, (int)R, splits, (int)K,
                               K, R * K, splits, 0);
        else
            hipLaunchKernelGGL(lm2exp_colmax_kernel<false>, dim3(blocks2), dim3(256), 0, s, part, m, (int)R, splits,
                               (int)K, K, R * K, splits, 0);
    } else if (clamp) {
        hipLaunchKernelGGL(lm2exp_colmax_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, b, m, (int)R, (int)J,
                           (int)K, sb[0], sb[1], (int)J, once);
    } else {
        hipLaunchKernelGGL(lm2exp_colmax_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, b, m, (int)R, (int)J,
                           (int)K, sb[0], sb[1], (int)J, once);
    }
    return (int)hipGetLastError();
}

namespace trt {

// Sum of the partial products of a matrix product that was cut over k, in split order
// (deterministic).  part: [splits][total]; four elements per lane when VEC.
template <bool VEC>
static __global__ __launch_bounds__(256) void mm_merge_kernel(const float *__restrict__ part, float *__restrict__ c,
                                                              int64_t total, int splits) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    if (VEC) {
        const int64_t quads = total / 4;
        for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < quads; e += stride) {
            float4 sum = reinterpret_cast<const float4 *>(part)[e];
            for (int sp = 1; sp < splits; ++sp) {
                const float4 x = reinterpret_cast<const float4 *>(part + (int64_t)sp * total)[e];
                sum.x += x.x; sum.y += x.y; sum.z += x.z; sum.w += x.w;
            }
            reinterpret_cast<float4 *>(c)[e] = sum;
        }
    } else {
        for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
            float sum = part[e];
            for (int sp = 1; sp < splits; ++sp) sum += part[(int64_t)sp * total + e];
            c[e] = sum;
        }
    }
}

struct MmPlan {
    int rt;      // rows of the tile / 32
    int splits;  // workgroups sharing one output tile (cut over k)
};

// Row tile and cut over k by modelled time.  variant: 0 = any row tile, 1..4 = 32..128 rows.
// splits_req: 0 = any cut, 1 = never cut, n > 1 = cut n ways (capped at kMaxSplits and at one
// 32-wide chunk of k per piece).  The model, fitted to 200 random shapes (m, n = 32..4096,
// k = 64..16384, up to 30 GFLOP) timed on every tile under cuts of 1..32: the busiest CU runs
// q = ceil(workgroups / 256) workgroups of `per` chunks each, a chunk costing 1096 cycles per 32
// rows of the tile plus 306; one or two workgroups on a CU reach 0.84 / 0.98 of that rate, and
// of the 128-row tile three are resident at a time; a launch costs 2.8 us, the merge 3.6 us
// plus its traffic at 3.0 TB/s.  Its pick is 1.9 % (mean) behind the best combination timed,
// the worst 17 %; the uncut rule it replaces was 1.99x (geometric mean) behind.
static MmPlan mm_plan(int64_t m, int64_t k, int64_t n, int variant, int splits_req) {
    const int64_t chunks = ceil_div(k, 32);
    const int64_t ct = ceil_div(n, 128);
    if (splits_req > 1) {  // the count this request comes to
        int64_t sp = splits_req > kMaxSplits ? kMaxSplits : splits_req;
        if (sp > chunks) sp = chunks;
        splits_req = (int)ceil_div(chunks, ceil_div(chunks, sp));
    }
    auto rate = [](int64_t x) { return x >= 3 ? 1.0 : x == 2 ? 0.977 : 0.84; };
    MmPlan best{variant ? variant : 1, 1};
    double best_us = 1e300;
    for (int rt = 1; rt <= 4; ++rt) {
        if (variant ? rt != variant : (rt > 1 && 32 * (rt - 1) >= m)) continue;
        const int64_t tiles = ceil_div(m, 32 * rt) * ct;
        const double unit_us = (1096.0 * rt + 306.0) / 2400.0;
        const int64_t resident = rt == 4 ? 3 : 1 << 20;
        for (int64_t sp = 1; sp <= kMaxSplits; ++sp) {
            if (splits_req ? sp != splits_req : (sp > 1 && 2 * sp > chunks)) continue;
            const int64_t per = ceil_div(chunks, sp);
            if (ceil_div(chunks, per) != sp) continue;  // the same cut as a smaller count
            if (sp > 1 && !splits_req && (double)sp * m * n * 4.0 > (double)(1 << 30)) break;
            const int64_t q = ceil_div(tiles * sp, 256);
            const int64_t full = q / resident, rem = q % resident;
            double us = 2.8 + per * unit_us * (full * resident / rate(resident) + (rem ? rem / rate(rem) : 0.0));
            if (sp > 1) us += 3.6 + (double)(sp + 1) * m * n * 4.0 / 3.03e6;
            if (us < best_us) {
                best_us = us;
                best = MmPlan{rt, (int)sp};
            }
        }
    }
    return best;
}

}  // namespace trt

extern "C" size_t trt_mm_workspace_bytes(int64_t m, int64_t k, int64_t n, int variant, int splits) {
    if (m <= 0 || k <= 0 || n <= 0 || variant < 0 || variant > 4 || splits < 0) return 0;
    const MmPlan pl = mm_plan(m, k, n, variant, splits);
    return pl.splits > 1 ? (size_t)pl.splits * m * n * sizeof(float) : 0;
}

// c = a b for row-major fp32 matrices (m x k times k x n): the contraction kernel above without
// shift, exp and log; small grids are cut over k, the partial products summed in split order.
// Replaces the `_ker_mm[grid](...)` launch, triturus/mm.py:199-213.
extern "C" int trt_mm_f32(const float *a, const float *b, float *c, int64_t m, int64_t k, int64_t n, int variant,
                          int splits, void *workspace, size_t workspace_bytes, void *stream) {
    if (!a || !b || !c) return TRT_E_INVALID;
    if (m <= 0 || k <= 0 || n <= 0) return TRT_E_INVALID;
    if (variant < 0 || variant > 4 || splits < 0) return TRT_E_INVALID;
    const int64_t lim = (int64_t)1 << 30;
    if (m >= lim || k >= lim || n >= lim) return TRT_E_RANGE;
    if (k * n + n >= lim || m * k + k >= lim || m * n + n >= lim) return TRT_E_RANGE;
    MmPlan pl = mm_plan(m, k, n, variant, splits);
    if (pl.splits > 1 && (!workspace || workspace_bytes < (size_t)pl.splits * m * n * sizeof(float))) {
        if (splits > 1) return TRT_E_WORKSPACE;  // an explicit request must be met
        pl.splits = 1;                            // the rule's cut is an optimisation only
    }
    const int rt = pl.rt;
    Lm2Args args;
    args.a = a; args.b = b; args.c = c;
    args.part = pl.splits > 1 ? static_cast<float *>(workspace) : nullptr;
    args.shift = nullptr;
    args.R = 1; args.I = (int)m; args.J = (int)k; args.K = (int)n;
    args.sa0 = m * k; args.sa1 = k;
    args.sb0 = k * n; args.sb1 = n;
    args.sc0 = m * n; args.sc1 = n;
    args.sa2 = 1;
    args.sb2 = 1;
    args.i_tiles = (int)ceil_div(m, 32 * rt);
    args.n_tiles = (int)ceil_div(n, 128);
    args.splits = pl.splits;
    args.chunks_per_split = (int)ceil_div(ceil_div(k, 32), pl.splits);
    args.total_wgs = (int64_t)args.i_tiles * args.n_tiles * pl.splits;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    args.stream_out = rows_16_byte_aligned(c, args.sc0, args.sc1);
    if (args.padded_wgs >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    const bool vec = (k % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
    hipStream_t s = static_cast<hipStream_t>(stream);
    int st;
    if (rt == 4) st = launch_v<4, 1, 1, 4, 4, kPlain>(args, vec, s);
    else if (rt == 3) st = launch_v<3, 1, 1, 4, 4, kPlain>(args, vec, s);
    else if (rt == 2) st = launch_v<2, 1, 1, 4, 4, kPlain>(args, vec, s);
    else st = launch_v<1, 1, 1, 4, 4, kPlain>(args, vec, s);
    if (st != 0 || pl.splits <= 1) return st;
    const int64_t total = m * n;
    const bool vec4 = total % 4 == 0 && ((reinterpret_cast<uintptr_t>(c) | reinterpret_cast<uintptr_t>(workspace)) & 15) == 0;
    int64_t blocks = ceil_div(vec4 ? total / 4 : total, 256);
    if (blocks > 4096) blocks = 4096;
    if (vec4)
        hipLaunchKernelGGL(mm_merge_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, args.part, c, total, pl.splits);
    else
        hipLaunchKernelGGL(mm_merge_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, args.part, c, total, pl.splits);
    return (int)hipGetLastError();
}

