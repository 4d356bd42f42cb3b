// lm2exp for gfx950:  c[r,i,k] = log sum_j a[r,i,j] exp(b[r,j,k])
//
// A workgroup of WM x WN wavefronts owns a (32*RT*WM rows of I) x
// (32*CT*WN columns of K) tile of c[r].  Each wavefront first takes the
// maximum of its b columns over all J (every lane owns one column, the two
// lane halves take alternate rows and exchange once), then walks J in chunks
// of JC = 8*NQ:
//   B operand = exp(b[j,n] - m[n]), evaluated once per (wavefront, element)
//               straight into the VGPRs the MFMA reads: b never visits LDS;
//   A operand = the a tile, staged global -> registers -> LDS (double
//               buffered) and read back 16 bytes per lane.
// The contraction runs on v_mfma_f32_32x32x2_f32 (IEEE fp32 in, fp32 accumulate),
// MFMA (q,u) of lane-half h consuming j = 8q + 4h + u of the chunk.
// Epilogue: m[n] + log(acc); acc == 0 (all -inf column, or zero row of a)
// gives -inf, never NaN, because m is clamped to +-1e38 first.
//
// Replaces _ker_lm2exp, triturus/lm2exp.py:63-164.  Ragged contracted-axis
// tails are padded with a = 0 and b = -inf (the reference pads b with 0.0,
// triturus/lm2exp.py:143, which can overflow exp(0 - m); not reproduced).

#include "common.hpp"

namespace trt {

struct Lm2Args {
    const float *a, *b;
    float *c;
    int R, I, J, K;
    int64_t sa0, sa1, sb0, sb1, sc0, sc1;
    int i_tiles, n_tiles;
    int64_t total_wgs, padded_wgs;
};

template <int RT, int CT, int WM, int WN, int NQ, bool VEC>
__global__ __launch_bounds__(WM *WN *kWave, 2) void lm2exp_kernel(const Lm2Args p) {
    constexpr int NT = WM * WN * kWave;
    constexpr int TM = 32 * RT * WM;  // rows of I per workgroup
    constexpr int TN = 32 * CT * WN;  // columns of K per workgroup
    constexpr int JC = 8 * NQ;
    constexpr int LDA = JC + 4;  // padded LDS row (floats)
    constexpr int F4_PER_ROW = JC / 4;
    constexpr int SLOTS = TM * F4_PER_ROW / NT;
    static_assert(TM * F4_PER_ROW % NT == 0, "tile must divide over the threads");

    extern __shared__ __attribute__((aligned(16))) float at[];  // [2][TM * LDA]

    const int64_t L = xcd_logical_id(blockIdx.x, p.padded_wgs);
    if (L >= p.total_wgs) return;
    const int nt = (int)(L % p.n_tiles);
    const int64_t rest = L / p.n_tiles;
    const int itile = (int)(rest % p.i_tiles);
    const int r = (int)(rest / p.i_tiles);

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
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        ncol[ct] = n0 + 32 * ct + m;
        ncl[ct] = ncol[ct] < p.K ? ncol[ct] : p.K - 1;
    }
    const float *ar = p.a + (int64_t)r * p.sa0;
    const float *br = p.b + (int64_t)r * p.sb0;

    // ---- sweep 1: column maxima of b over all J
    float mx[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        float x0 = -__builtin_inff(), x1 = x0, x2 = x0, x3 = x0;
        int j = h;
        for (; j + 6 < p.J; j += 8) {
            const float *bp = br + (int64_t)j * p.sb1 + ncl[ct];
            x0 = max_nan(x0, bp[0]);
            x1 = max_nan(x1, bp[2 * p.sb1]);
            x2 = max_nan(x2, bp[4 * p.sb1]);
            x3 = max_nan(x3, bp[6 * p.sb1]);
        }
        for (; j < p.J; j += 2) x0 = max_nan(x0, br[(int64_t)j * p.sb1 + ncl[ct]]);
        float x = max_nan(max_nan(x0, x1), max_nan(x2, x3));
        x = max_nan(x, __shfl_xor(x, 32, kWave));
        mx[ct] = clamp_shift(x);
    }

    floatx16 acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[rt][ct][v] = 0.f;

    floatx4 stage[SLOTS];
    auto load_tile = [&](int jc) {
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) {
            const int f = tid + sidx * NT;
            const int row = f / F4_PER_ROW;
            const int c4 = f % F4_PER_ROW;
            const int j = jc * JC + 4 * c4;
            const bool row_ok = (i0 + row) < p.I;
            const float *src = ar + (int64_t)(i0 + row) * p.sa1 + j;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if (VEC) {
                if (row_ok && j < p.J) v = *reinterpret_cast<const floatx4 *>(src);
            } else {
                if (row_ok) {
                    if (j + 0 < p.J) v[0] = src[0];
                    if (j + 1 < p.J) v[1] = src[1];
                    if (j + 2 < p.J) v[2] = src[2];
                    if (j + 3 < p.J) v[3] = src[3];
                }
            }
            stage[sidx] = v;
        }
    };
    auto store_tile = [&](int buf) {
        float *dst = at + buf * (TM * LDA);
#pragma unroll
        for (int sidx = 0; sidx < SLOTS; ++sidx) {
            const int f = tid + sidx * NT;
            const int row = f / F4_PER_ROW;
            const int c4 = f % F4_PER_ROW;
            *reinterpret_cast<floatx4 *>(&dst[row * LDA + 4 * c4]) = stage[sidx];
        }
    };

    float braw[CT][4 * NQ], eb[CT][4 * NQ];
    auto load_b = [&](int jc) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int q = 0; q < NQ; ++q)
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int j = jc * JC + 8 * q + 4 * h + u;
                    float raw = -__builtin_inff();
                    if (j < p.J) raw = br[(int64_t)j * p.sb1 + ncl[ct]];
                    braw[ct][4 * q + u] = raw;
                }
    };
    auto exp_b = [&]() {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int e = 0; e < 4 * NQ; ++e) eb[ct][e] = expf(braw[ct][e] - mx[ct]);
    };

    const int n_jc = (p.J + JC - 1) / JC;
    load_tile(0);
    load_b(0);
    store_tile(0);
    exp_b();
    __syncthreads();

    int cur = 0;
    for (int jc = 0; jc < n_jc; ++jc) {
        const bool has_next = (jc + 1) < n_jc;
        if (has_next) {
            load_tile(jc + 1);
            load_b(jc + 1);
        }
        const float *tile = at + cur * (TM * LDA) + wrow0 * LDA;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            floatx4 af[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                af[rt] = *reinterpret_cast<const floatx4 *>(&tile[(32 * rt + m) * LDA + 8 * q + 4 * h]);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[rt][u], eb[ct][4 * q + u],
                                                                          acc[rt][ct], 0, 0, 0);
        }
        if (has_next) {
            store_tile(cur ^ 1);
            exp_b();
        }
        __syncthreads();
        cur ^= 1;
    }

    // ---- epilogue: register v of lane (h, m) holds row 8*(v/4) + 4*h + v%4, column m
    float *cr = p.c + (int64_t)r * p.sc0;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (ncol[ct] >= p.K) continue;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = i0 + wrow0 + 32 * rt + 8 * (v / 4) + 4 * h + (v % 4);
                if (row < p.I) cr[(int64_t)row * p.sc1 + ncol[ct]] = mx[ct] + logf(acc[rt][ct][v]);
            }
    }
}

// ------------------------------------------------------------------ host
struct Lm2Variant {
    int rt, ct, wm, wn, nq;
};
static const Lm2Variant kVariants[] = {
    {8, 1, 1, 8, 4},  // 256 x 256 tile, 8 waves each 256 x 32
    {4, 2, 2, 4, 4},  // 256 x 256 tile, 8 waves each 128 x 64
    {8, 1, 1, 4, 4},  // 256 x 128 tile, 4 waves each 256 x 32
    {4, 1, 1, 4, 4},  // 128 x 128 tile, 4 waves each 128 x 32
    {2, 2, 1, 4, 4},  // 64 x 256 tile, 4 waves each 64 x 64
    {2, 1, 1, 4, 4},  // 64 x 128 tile
    {1, 1, 1, 4, 4},  // 32 x 128 tile
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
constexpr size_t kDefaultLdsLimit = 64 * 1024;  // larger dynamic LDS must be opted into per kernel

static int choose_variant(int64_t R, int64_t I, int64_t J, int64_t K) {
    (void)J;
    int v;
    if (I > 128) v = 0;
    else if (I > 64) v = 3;
    else if (I > 32) v = 4;
    else v = 6;
    // fall back to narrower column tiles when the grid would leave CUs idle
    if (v == 0 && R * ceil_div(I, 256) * ceil_div(K, 256) < 256) v = 2;
    if (v == 4 && R * ceil_div(I, 64) * ceil_div(K, 256) < 256) v = 5;
    return v;
}

template <int RT, int CT, int WM, int WN, int NQ>
static int launch_v(const Lm2Args &args, bool vec, hipStream_t stream) {
    constexpr int TM = 32 * RT * WM;
    constexpr int LDA = 8 * NQ + 4;
    constexpr size_t lds = (size_t)2 * TM * LDA * sizeof(float);
    hipError_t e;
    if (vec) {
        auto k = lm2exp_kernel<RT, CT, WM, WN, NQ, true>;
        if (lds > kDefaultLdsLimit) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
        }
        hipLaunchKernelGGL(k, dim3((unsigned)args.padded_wgs), dim3(WM * WN * kWave), lds, stream, args);
    } else {
        auto k = lm2exp_kernel<RT, CT, WM, WN, NQ, false>;
        if (lds > kDefaultLdsLimit) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
        }
        hipLaunchKernelGGL(k, dim3((unsigned)args.padded_wgs), dim3(WM * WN * kWave), lds, stream, args);
    }
    return (int)hipGetLastError();
}

}  // namespace trt

using namespace trt;

extern "C" int trt_lm2exp_variant_count(void) { return kNumVariants; }

extern "C" int trt_lm2exp_f32(const float *a, const float *b, float *c, int64_t R, int64_t I, int64_t J,
                              int64_t K, const int64_t sa[3], const int64_t sb[3], const int64_t sc[3],
                              int variant, void *stream) {
    if (!a || !b || !c || !sa || !sb || !sc) return TRT_E_INVALID;
    if (R <= 0 || I <= 0 || J <= 0 || K <= 0) return TRT_E_INVALID;
    if (variant < 0 || variant > kNumVariants) return TRT_E_INVALID;
    if (sa[2] != 1 || sb[2] != 1 || sc[2] != 1) return TRT_E_LAYOUT;
    for (int d = 0; d < 2; ++d)
        if (sa[d] < 0 || sb[d] < 0 || sc[d] < 0) return TRT_E_LAYOUT;
    const int64_t lim = (int64_t)1 << 30;
    if (R >= lim || I >= lim || J >= lim || K >= lim) return TRT_E_RANGE;

    const int v = (variant >= 1) ? variant - 1 : choose_variant(R, I, J, K);
    const Lm2Variant &vr = kVariants[v];
    Lm2Args args;
    args.a = a; args.b = b; args.c = c;
    args.R = (int)R; args.I = (int)I; args.J = (int)J; args.K = (int)K;
    args.sa0 = sa[0]; args.sa1 = sa[1];
    args.sb0 = sb[0]; args.sb1 = sb[1];
    args.sc0 = sc[0]; args.sc1 = sc[1];
    args.i_tiles = (int)ceil_div(I, 32 * vr.rt * vr.wm);
    args.n_tiles = (int)ceil_div(K, 32 * vr.ct * vr.wn);
    args.total_wgs = (int64_t)R * args.i_tiles * args.n_tiles;
    args.padded_wgs = ceil_div(args.total_wgs, kXcds) * kXcds;
    if (args.padded_wgs >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    const bool vec = (J % 4 == 0) && (sa[0] % 4 == 0) && (sa[1] % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(a) & 15) == 0);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (v) {
        case 0: return launch_v<8, 1, 1, 8, 4>(args, vec, s);
        case 1: return launch_v<4, 2, 2, 4, 4>(args, vec, s);
        case 2: return launch_v<8, 1, 1, 4, 4>(args, vec, s);
        case 3: return launch_v<4, 1, 1, 4, 4>(args, vec, s);
        case 4: return launch_v<2, 2, 1, 4, 4>(args, vec, s);
        case 5: return launch_v<2, 1, 1, 4, 4>(args, vec, s);
        default: return launch_v<1, 1, 1, 4, 4>(args, vec, s);
    }
}
