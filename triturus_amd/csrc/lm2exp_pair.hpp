// lm2exp for gfx950, paired-wavefront kernel:  c[r,i,k] = log sum_j a[r,i,j] exp(b[r,j,k])
//
// A workgroup of 2 x WN wavefronts owns a (64*RT rows of I) x (32*WN columns of K) tile of
// c[r]; wavefront (wm, wn) owns rows [32*RT*wm, 32*RT*(wm+1)) and columns [32*wn, 32*wn + 32).
// FP32 MFMA and the vector ALU do not run side by side on this hardware, and a vector
// instruction of one wavefront waits for the matrix instructions that the other wavefronts of
// its SIMD have queued.  So the kernel spends as few vector instructions per MFMA as the
// algorithm allows, and puts those it needs between MFMAs of the same wavefront:
//   * the shift is the exact column maximum, found by one cooperative sweep over the
//     workgroup's panel of b before the contraction (as the reference kernel does,
//     triturus/lm2exp.py:125-127): the main loop carries no running maximum, no branch and no
//     rescaling of accumulators.  The panel (J x 32*WN columns) is read again by the main loop
//     while it is still in cache, which is why the host picks this kernel for moderate J only;
//   * the two wavefronts that share a column panel (wm = 0, 1) each evaluate half of every
//     chunk of exp(b - m') and hand it to the other through LDS, so an exp is taken once per
//     workgroup and element: a quarter of a vector instruction per MFMA with 256-row tiles;
//   * the raw b values are loaded two chunks ahead, so the exps of chunk t + 1 are evaluated
//     between the MFMAs of chunk t.
// The a tile is staged global -> registers -> LDS (double buffered) in 16-byte planes: plane
// c = 2q + h holds, for every tile row, the four values j = 8q + 4h + 0..3 that lane half h
// feeds to the four MFMAs (q, 0..3), so a lane's operand read is one conflict-free 16-byte read.
// The a tile may have any element strides (LOADA): 16-byte loads of aligned unit-stride rows,
// single elements with lanes along j, or single elements with lanes along i (a transposed a).
//
// m is clamped to +-1e38 (baselines/lm2exp.py:12): an all -inf column gives 2^(-inf) = 0 and
// log2(0) = -inf, never NaN.  Replaces _ker_lm2exp, triturus/lm2exp.py:63-164.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace trt {

constexpr int kLoadVec = 0;    // rows of a: unit stride, 16-byte aligned
constexpr int kLoadByCol = 1;  // single elements, consecutive lanes on consecutive j
constexpr int kLoadByRow = 2;  // single elements, consecutive lanes on consecutive i (transposed a)

template <int RT, int WN, int NQ, int LOADA>
__global__ __launch_bounds__(128 * WN, 4) void lm2exp_pair_kernel(const Lm2Args p) {
    static_assert(NQ % 2 == 0, "each wavefront of a pair evaluates half of the chunk");
    constexpr int NT = 128 * WN;  // 2 x WN wavefronts
    constexpr int TM = 64 * RT;   // rows of I per workgroup
    constexpr int TN = 32 * WN;   // columns of K per workgroup
    constexpr int JC = 8 * NQ;    // j per chunk
    constexpr int NH = NQ / 2;    // MFMA groups (of 8 j) per wavefront of a pair
    constexpr int NB = 4 * NH;    // exp values a lane evaluates per chunk
    constexpr int NPL = 2 * NQ;   // 16-byte planes of an a tile
    constexpr int PLANE = TM * 4;            // floats of a plane: TM rows x 4
    constexpr int ABUF = NPL * PLANE;        // floats of one a tile
    constexpr int XBUF = 2 * WN * 64 * NB;   // floats of one exchange buffer: per wavefront, 64 lanes x NB
    constexpr int PIECES = TM * NPL;         // 16-byte pieces of an a tile
    static_assert(PIECES % NT == 0, "every thread stages the same number of pieces");
    constexpr int SLOTS = PIECES / NT;
    constexpr int NE = 4 * SLOTS;  // floats per thread of an a tile
    static_assert(LOADA != kLoadByRow || NT % TM == 0, "lanes along i need a tile height that divides the workgroup");

    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *at = smem;             // [2][ABUF]
    float *xb = smem + 2 * ABUF;  // [2][XBUF]
    // [WN][2][32] column maxima of the two row halves: used before the first barrier of the main
    // loop only, so it shares the second exchange buffer, which is first written after it
    float *mxs = xb + XBUF;
    static_assert(XBUF >= WN * 64, "the column maxima fit the exchange buffer they share");

    // tile coordinates: 32-bit arithmetic (the host keeps the grid below 2^31 workgroups); the
    // generic 64-bit division expands to some hundred scalar instructions per quotient, which
    // every workgroup would pay before its first load
    const uint32_t per_xcd = (uint32_t)p.padded_wgs / kXcds;
    const uint32_t L = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (L >= (uint32_t)p.total_wgs) return;
    uint32_t rest = L / (uint32_t)p.n_tiles;
    const int nt = (int)(L - rest * (uint32_t)p.n_tiles);
    uint32_t rest2 = rest / (uint32_t)p.splits;
    const int split = (int)(rest - rest2 * (uint32_t)p.splits);
    const int r = (int)(rest2 / (uint32_t)p.i_tiles);
    const int itile = (int)(rest2 - (uint32_t)r * (uint32_t)p.i_tiles);
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int wm = wave & 1;
    const int wn = wave >> 1;
    const int lane = tid % kWave;
    const int h = lane / 32;
    const int m = lane % 32;
    const int i0 = itile * TM;
    const int wrow0 = wm * 32 * RT;
    const int ncol = nt * TN + wn * 32 + m;
    const int ncl = ncol < p.K ? ncol : p.K - 1;
    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;

    // chunks [jc0, jc1) of this workgroup (all of them unless the contraction is cut over J)
    const int n_full = p.J / JC;
    const int n_jc = n_full + ((p.J % JC) != 0 ? 1 : 0);
    const int jc0 = split * p.chunks_per_split;
    const int jc1 = (jc0 + p.chunks_per_split < n_jc) ? jc0 + p.chunks_per_split : n_jc;
    const int full_end = jc1 < n_full ? jc1 : n_full;
    const int jbeg = jc0 * JC;
    const int jend = jc1 * JC < p.J ? jc1 * JC : p.J;

    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(br, (uint32_t)(((int64_t)(p.J - 1) * p.sb1 + (int64_t)(p.K - 1) * p.sb2 + 1) * 4));
    const uint32_t b_row_bytes = (uint32_t)p.sb1 * 4u;

    // ---- column maxima of rows [jbeg, jend): the four (wm, h) classes take every fourth row.
    // (Called after the loads of the first chunks have been issued, so that the trips to memory
    // a workgroup starts with overlap.)
    float msh = 0.f;  // the shift: the clamped column maximum
    auto find_shift = [&]() {
        const uint32_t poff = ((uint32_t)h * (uint32_t)p.sb1 + (uint32_t)ncl * (uint32_t)p.sb2) * 4u;
        float x0 = -__builtin_inff(), x1 = x0;
        int j = jbeg + 2 * wm;  // wave-uniform: this lane reads row j + h
        // 64 loads in flight per lane (256 rows of the panel per step), then 8 at a time: the
        // sweep is bound by memory latency, not by the handful of max instructions, so a panel
        // of up to 256 rows costs one trip to memory
        for (; j + 253 < jend; j += 256) {
            float v[64];
#pragma unroll
            for (int t = 0; t < 64; ++t) v[t] = buf_load_f32(b_rsrc, poff, (uint32_t)(j + 4 * t) * b_row_bytes);
#pragma unroll
            for (int t = 0; t < 64; t += 4) {
                x0 = max3_raw(x0, v[t], v[t + 1]);
                x1 = max3_raw(x1, v[t + 2], v[t + 3]);
            }
        }
        for (; j + 29 < jend; j += 32) {
            float v[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) v[t] = buf_load_f32(b_rsrc, poff, (uint32_t)(j + 4 * t) * b_row_bytes);
            x0 = max3_raw(x0, v[0], v[1]);
            x1 = max3_raw(x1, v[2], v[3]);
            x0 = max3_raw(x0, v[4], v[5]);
            x1 = max3_raw(x1, v[6], v[7]);
        }
        for (; j < jend; j += 4) {
            const float v = buf_load_f32(b_rsrc, poff, (uint32_t)j * b_row_bytes);
            x0 = max3_raw(x0, j + h < jend ? v : x0, x0);
        }
        x0 = max3_raw(x0, x1, x0);
        x0 = max3_raw(x0, __shfl_xor(x0, 32, kWave), x0);
        if (h == 0) mxs[(wn * 2 + wm) * 32 + m] = x0;
        __syncthreads();
        const float mx = max3_raw(mxs[(wn * 2) * 32 + m], mxs[(wn * 2 + 1) * 32 + m], x0);
        msh = clamp_shift(mx);
    };

    floatx16 acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rt][v] = 0.f;

    // ---- a tile: global -> registers -> LDS, one chunk ahead.  Rows past I read whatever lies
    // inside the extent of the tile (another row of a, or zeros past it): they only feed
    // accumulator rows that are never stored.  Columns past J (ragged last chunk) must be
    // exact zeros.
    float sa[NE];
    const float *atile0 = ar + (int64_t)i0 * p.sa1;
    const int arows = (p.I - i0) < TM ? (p.I - i0) : TM;
    const __amdgpu_buffer_rsrc_t a_rsrc =
        make_rsrc(atile0, (uint32_t)(((int64_t)(arows - 1) * p.sa1 + (int64_t)(p.J - 1) * p.sa2 + 1) * 4));
    // kLoadVec: piece f = tid + s NT is row f / NPL, plane f % NPL
    // kLoadByCol: element g = tid + e NT is row g / JC, column g % JC = tid % JC
    // kLoadByRow: element g = tid + e NT is row g % TM = tid % TM, column g / TM
    // (kLoadVec: a thread keeps its plane, and its pieces lie NT / NPL rows apart: one lane
    // offset, the slot in the scalar offset of the load and the immediate offset of the LDS
    // write; rows past I lie outside the extent and read as zeros)
    static_assert(NT % NPL == 0, "a thread's pieces share a plane");
    uint32_t aoff[1];
    int lds_off[1];
    int ecol = 0, erow = 0;
    const uint32_t a_slot_bytes = (uint32_t)(NT / NPL) * (uint32_t)p.sa1 * 4u;  // wave-uniform
    if (LOADA == kLoadVec) {
        const int row = tid / NPL, c = tid % NPL;
        lds_off[0] = c * PLANE + row * 4;
        aoff[0] = ((uint32_t)row * (uint32_t)p.sa1 + 4u * (uint32_t)c) * 4u;
    } else if (LOADA == kLoadByCol) {
        ecol = tid % JC;
        erow = tid / JC;
        aoff[0] = ((uint32_t)erow * (uint32_t)p.sa1 + (uint32_t)ecol * (uint32_t)p.sa2) * 4u;
        lds_off[0] = (ecol / 4) * PLANE + erow * 4 + ecol % 4;
    } else {
        erow = tid % TM;
        ecol = tid / TM;
        aoff[0] = ((uint32_t)erow * (uint32_t)p.sa1 + (uint32_t)ecol * (uint32_t)p.sa2) * 4u;
        lds_off[0] = erow * 4;
    }
    auto load_a = [&](int jc, bool masked) {
        if (LOADA == kLoadVec) {
            const uint32_t soff = (uint32_t)(jc * JC) * 4u;
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const floatx4 v = buf_load_f32x4(a_rsrc, aoff[0], soff + (uint32_t)s * a_slot_bytes);
                const int j = jc * JC + 4 * (tid % NPL);
#pragma unroll
                for (int e = 0; e < 4; ++e) sa[4 * s + e] = (!masked || j + e < p.J) ? v[e] : 0.f;
            }
        } else if (LOADA == kLoadByCol) {
            const uint32_t soff = (uint32_t)(jc * JC) * (uint32_t)p.sa2 * 4u;
            const bool inside = !masked || jc * JC + ecol < p.J;
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const float v = buf_load_f32(a_rsrc, aoff[0], soff + (uint32_t)(e * (NT / JC)) * (uint32_t)p.sa1 * 4u);
                sa[e] = inside ? v : 0.f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const int col = jc * JC + e * (NT / TM);  // + ecol: in the lane offset
                const float v = buf_load_f32(a_rsrc, aoff[0], (uint32_t)col * (uint32_t)p.sa2 * 4u);
                sa[e] = (!masked || col + ecol < p.J) ? v : 0.f;
            }
        }
    };
    auto store_a = [&](int buf) {
        float *dst = at + buf * ABUF;
        if (LOADA == kLoadVec) {
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const floatx4 v = {sa[4 * s], sa[4 * s + 1], sa[4 * s + 2], sa[4 * s + 3]};
                *reinterpret_cast<floatx4 *>(&dst[lds_off[0] + s * (NT / NPL) * 4]) = v;
            }
        } else if (LOADA == kLoadByCol) {
#pragma unroll
            for (int e = 0; e < NE; ++e) dst[lds_off[0] + e * (NT / JC) * 4] = sa[e];
        } else {
#pragma unroll
            for (int e = 0; e < NE; ++e) {
                const int col = e * (NT / TM) + ecol;
                dst[lds_off[0] + (col / 4) * PLANE + col % 4] = sa[e];
            }
        }
    };

    // ---- b: this wavefront's half of a chunk, rows 8 (wm NH + qq) + 4h + u, column ncl, raw,
    // two chunks ahead (two register sets that swap roles from step to step)
    const uint32_t boff = ((uint32_t)(4 * h) * (uint32_t)p.sb1 + (uint32_t)ncl * (uint32_t)p.sb2) * 4u;
    auto load_b = [&](float (&raw)[NB], int jc, bool masked) {
#pragma unroll
        for (int qq = 0; qq < NH; ++qq)
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int row = jc * JC + 8 * (wm * NH + qq) + u;  // wave-uniform; + 4h in the lane offset
                const float v = buf_load_f32(b_rsrc, boff, (uint32_t)row * b_row_bytes);
                raw[4 * qq + u] = (!masked || row + 4 * h < p.J) ? v : -__builtin_inff();
            }
    };
    auto exp_one = [&](float raw) { return exp_shifted(raw - msh); };
    float *xmine = xb + (wave * NH) * 256 + lane * 4;
    const float *xpartner = xb + ((wave ^ 1) * NH) * 256 + lane * 4;
    auto publish = [&](const float (&e)[NB], int buf) {
#pragma unroll
        for (int qq = 0; qq < NH; ++qq) {
            const floatx4 v = {e[4 * qq], e[4 * qq + 1], e[4 * qq + 2], e[4 * qq + 3]};
            *reinterpret_cast<floatx4 *>(&xmine[buf * XBUF + qq * 256]) = v;
        }
    };

    // ---- one step.  Chunk t sits in LDS buffer CUR (a tile, partner's exps) and in `ecur`
    // (own exps); `bnext` holds the raw b values of chunk t + 1.  The step issues the loads of
    // the a tile of chunk t + 1 and of the b values of chunk t + 2 (into `bfree`), contracts
    // chunk t -- own half of the exps first, then the partner's -- with the exps of chunk
    // t + 1 evaluated between the MFMAs of the own half (into `enext`), and moves chunk t + 1
    // to LDS buffer CUR ^ 1.  FAST: all those chunks exist and are full, no tests.
    const int rd_own = (2 * (wm * NH) + h) * PLANE + (wrow0 + m) * 4;
    const int rd_partner = (2 * ((wm ^ 1) * NH) + h) * PLANE + (wrow0 + m) * 4;
    // Two register sets that swap roles from step to step, picked by the step's parity (a
    // compile-time index: the sets must stay in registers): ee[CUR] the own exps of chunk t,
    // ee[CUR ^ 1] those of chunk t + 1; bb[CUR ^ 1] the raw b values of chunk t + 1, bb[CUR]
    // free for those of chunk t + 2.
    float ee[2][NB], bb[2][NB];
    auto step = [&](auto cur_c, auto fast_c, int t) {
        constexpr int CUR = decltype(cur_c)::value;
        constexpr bool FAST = decltype(fast_c)::value;
        float (&ecur)[NB] = ee[CUR];
        float (&enext)[NB] = ee[CUR ^ 1];
        const float (&bnext)[NB] = bb[CUR ^ 1];
        float (&bfree)[NB] = bb[CUR];
        const bool more = FAST || t + 1 < jc1;  // wave-uniform
        if (FAST) {
            load_a(t + 1, false);
            load_b(bfree, t + 2, false);
        } else {
            if (more) {
                if (t + 1 >= n_full) load_a(t + 1, true);
                else load_a(t + 1, false);
            }
            if (t + 2 < jc1) {
                if (t + 2 >= n_full) load_b(bfree, t + 2, true);
                else load_b(bfree, t + 2, false);
            }
        }
        // The MFMAs of the step come in groups of 4 RP: RP row tiles (their a fragments, one
        // 16-byte read each) times the four j of one MFMA group; groups [0, NG / 2) use the
        // wavefront's own exps, the others the partner's.  The fragments of a group are read
        // while the group before it runs, and one exp of chunk t + 1 follows every other
        // group of the first half.
        constexpr int RP = RT % 2 == 0 ? 2 : 1;      // row tiles per group
        constexpr int NG = 2 * NH * (RT / RP);       // groups per step
        const float *tile = at + CUR * ABUF;
        floatx4 ebp[NH];
#pragma unroll
        for (int qq = 0; qq < NH; ++qq) ebp[qq] = *reinterpret_cast<const floatx4 *>(&xpartner[CUR * XBUF + qq * 256]);
        auto read_frags = [&](floatx4 (&af)[RP], int g) {
            const int half = g / (NG / 2), gg = g % (NG / 2);
            const int qq = gg / (RT / RP), rt0 = (gg % (RT / RP)) * RP;
#pragma unroll
            for (int k = 0; k < RP; ++k)
                af[k] = *reinterpret_cast<const floatx4 *>(
                    &tile[(half ? rd_partner : rd_own) + 2 * qq * PLANE + 32 * (rt0 + k) * 4]);
        };
        floatx4 afa[RP], afb[RP];
        read_frags(afa, 0);
        __builtin_amdgcn_sched_barrier(0);  // the loads are issued before the MFMA block, not sunk into it
        int nexp = 0;  // exps of chunk t + 1 evaluated so far (compile-time after unrolling)
        auto run_group = [&](const floatx4 (&af)[RP], floatx4 (&afn)[RP], int g) {
            const int half = g / (NG / 2), gg = g % (NG / 2);
            const int qq = gg / (RT / RP), rt0 = (gg % (RT / RP)) * RP;
            if (g + 1 < NG) read_frags(afn, g + 1);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int k = 0; k < RP; ++k)
                    acc[rt0 + k] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        af[k][u], half ? ebp[qq][u] : ecur[4 * qq + u], acc[rt0 + k], 0, 0, 0);
                // NB exps over the 2 NG u-pairs of the first half
                // (the count advances whether or not there is a next chunk: it must stay a
                // compile-time index, or the register sets become arrays in scratch memory)
                if (half == 0 && (u % 2 == 1 || NB > NG) && nexp < NB) {
                    if (more) enext[nexp] = exp_one(bnext[nexp]);
                    ++nexp;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (g == NG / 2 - 1) {
                for (; nexp < NB; ++nexp)
                    if (more) enext[nexp] = exp_one(bnext[nexp]);
                if (more) publish(enext, CUR ^ 1);
            }
        };
#pragma unroll
        for (int g = 0; g < NG; g += 2) {
            run_group(afa, afb, g);
            run_group(afb, afa, g + 1);
        }
        if (more) {
            store_a(CUR ^ 1);
            __syncthreads();
        }
    };

    // ---- prologue: the first chunk (a tile and b values) and the b values of the second
    using std::integral_constant;
    float (&e0)[NB] = ee[0], (&b0)[NB] = bb[0], (&b1)[NB] = bb[1];
    if (jc0 >= n_full) {
        load_a(jc0, true);
        load_b(b0, jc0, true);
    } else {
        load_a(jc0, false);
        load_b(b0, jc0, false);
    }
    if (jc0 + 1 < jc1) {
        if (jc0 + 1 >= n_full) load_b(b1, jc0 + 1, true);
        else load_b(b1, jc0 + 1, false);
    }
    find_shift();
    store_a(0);
#pragma unroll
    for (int e = 0; e < NB; ++e) e0[e] = exp_one(b0[e]);
    publish(e0, 0);
    __syncthreads();
    // ---- steady state, two steps per trip (LDS buffers and register sets swap roles); the
    // last chunks, the ragged one among them, take the steps with tests
    int t = jc0;
    for (; t + 3 < full_end; t += 2) {
        step(integral_constant<int, 0>{}, integral_constant<bool, true>{}, t);
        step(integral_constant<int, 1>{}, integral_constant<bool, true>{}, t + 1);
    }
    while (t < jc1) {
        step(integral_constant<int, 0>{}, integral_constant<bool, false>{}, t);
        if (++t >= jc1) break;
        step(integral_constant<int, 1>{}, integral_constant<bool, false>{}, t);
        ++t;
    }

    // ---- epilogue: c = m + log(acc).  Register v of lane (h, m) holds row
    // 8 (v / 4) + 4h + v % 4, column m of its 32 x 32 tile.  Rows past I fall outside the
    // buffer extent and are dropped by the hardware.  With a cut contraction the raw sums and
    // their shift go to the workspace instead.
    const bool split_out = p.splits > 1;  // wave-uniform
    const int crows = p.I - (i0 + wrow0);
    float *obase = split_out ? p.part + (((int64_t)split * p.R + r) * p.I + (i0 + wrow0)) * (int64_t)p.K
                             : p.c + (int64_t)r * p.sc0 + (int64_t)(i0 + wrow0) * p.sc1;
    const uint32_t orow = split_out ? (uint32_t)p.K : (uint32_t)p.sc1;
    const __amdgpu_buffer_rsrc_t c_rsrc =
        make_rsrc(obase, crows > 0 ? (uint32_t)(((int64_t)(crows - 1) * orow + p.K) * 4) : 0u);
    const uint32_t c_row_bytes = orow * 4u;
    if (ncol < p.K) {
        const uint32_t co = ((uint32_t)(4 * h) * orow + (uint32_t)ncol) * 4u;
        if (split_out && itile == 0 && wm == 0 && h == 0) p.shift[((int64_t)split * p.R + r) * p.K + ncol] = msh;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t trow = 32 * rt + 8 * (v / 4) + (v % 4);  // + 4h in the lane offset
                if (split_out)  // partial sums are read back by the merge kernel right away
                    buf_store_f32(acc[rt][v], c_rsrc, co, trow * c_row_bytes);
                else
                    buf_store_f32_out(p.stream_out != 0, log_plus(acc[rt][v], msh), c_rsrc, co, trow * c_row_bytes);
            }
    }
}

}  // namespace trt
