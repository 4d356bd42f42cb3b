// matmax / vmax / vamax for gfx950: every element is read once from HBM with
// 16-byte coalesced loads, reduced in registers, then across the 64-lane
// wavefront, then across the workgroup through LDS.  Large inputs take one
// streaming launch plus one tiny combine launch over per-workgroup partials.
//
// Semantics follow torch, the oracle the reference tests use
// (tests/max.py:13,22,32): NaN propagates; argmax ties go to the lowest index
// and a NaN reports the first NaN.
//
// Replaces: _ker_vamax / _ker_vmax / _ker_matmax, triturus/max.py:8-32,62-93,125-168.

#include "common.hpp"

#include <hip/hip_fp16.h>

namespace trt {

// ---------------------------------------------------------------- elements
template <int DT>
struct Elem;
template <>
struct Elem<TRT_F32> {
    using T = float;
    using C = float;
    __device__ static C up(T v) { return v; }
    __device__ static T down(C v) { return v; }
};
template <>
struct Elem<TRT_F64> {
    using T = double;
    using C = double;
    __device__ static C up(T v) { return v; }
    __device__ static T down(C v) { return v; }
};
template <>
struct Elem<TRT_F16> {
    using T = _Float16;
    using C = float;
    __device__ static C up(T v) { return (float)v; }
    __device__ static T down(C v) { return (_Float16)v; }
};
template <>
struct Elem<TRT_BF16> {
    using T = uint16_t;
    using C = float;
    __device__ static C up(T v) { return __uint_as_float(((uint32_t)v) << 16); }
    __device__ static T down(C v) { return (uint16_t)(__float_as_uint(v) >> 16); }
};

template <typename C>
__device__ __forceinline__ C neg_inf();
template <>
__device__ __forceinline__ float neg_inf<float>() { return -__builtin_inff(); }
template <>
__device__ __forceinline__ double neg_inf<double>() { return -__builtin_inf(); }

constexpr int64_t kNoIdx = INT64_MAX;

template <typename C>
__device__ __forceinline__ C vmax_nan(C a, C b) {
    return (a > b || a != a) ? a : b;
}

// Is candidate (v, i) preferred over (bv, bi)?  NaN beats numbers; equal
// values (or two NaNs) go to the lower index.
template <typename C>
__device__ __forceinline__ bool prefer(C v, int64_t i, C bv, int64_t bi) {
    const bool vn = v != v, bn = bv != bv;
    const bool strictly = (v > bv) || (vn && !bn);
    const bool same = (v == bv) || (vn && bn);
    return strictly || (same && i < bi);
}

template <typename C>
__device__ __forceinline__ C shfl_xor_c(C v, int off) { return __shfl_xor(v, off, kWave); }

__device__ __forceinline__ int64_t shfl_xor_i64(int64_t v, int off) {
    int lo = __shfl_xor((int)(uint32_t)(uint64_t)v, off, kWave);
    int hi = __shfl_xor((int)(uint32_t)((uint64_t)v >> 32), off, kWave);
    return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint64_t)(uint32_t)lo);
}

template <typename C>
__device__ __forceinline__ C wave_max(C v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = vmax_nan(v, shfl_xor_c(v, off));
    return v;
}

template <typename C>
__device__ __forceinline__ void wave_argmax(C &v, int64_t &i) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        C ov = shfl_xor_c(v, off);
        int64_t oi = shfl_xor_i64(i, off);
        if (prefer(ov, oi, v, i)) {
            v = ov;
            i = oi;
        }
    }
}

// 16-byte vector of T
template <typename T>
struct alignas(16) Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T e[N];
};

// ------------------------------------------------------------------- vmax
constexpr int kVmaxThreads = 256;
constexpr int kVmaxMaxBlocks = 2048;
constexpr int kVmaxUnroll = 4;

// FINAL: the launch has a single workgroup, which writes the result itself (short vectors
// take one launch instead of two).
template <int DT, bool WITH_IDX, bool FINAL>
__global__ __launch_bounds__(kVmaxThreads) void vmax_stage1(
    const typename Elem<DT>::T *__restrict__ x, int64_t n, int64_t head, int64_t nvec,
    typename Elem<DT>::C *__restrict__ pval, int64_t *__restrict__ pidx,
    typename Elem<DT>::T *__restrict__ out_val, int64_t *__restrict__ out_idx) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int VN = V::N;

    C best = neg_inf<C>();
    int64_t bidx = kNoIdx;
    auto feed = [&](C c, int64_t i) {
        // indices arrive in increasing order within a thread: strict compare
        // keeps the first occurrence.
        const bool take = (c > best) || (c != c && best == best);
        best = take ? c : best;
        if (WITH_IDX) bidx = take ? i : bidx;
    };

    const int tid = threadIdx.x;
    if (blockIdx.x == 0 && tid < head) feed(E::up(x[tid]), tid);

    // Workgroups walk the vector in contiguous blocks of kVmaxUnroll * kVmaxThreads 16-byte
    // pieces (block-cyclic over the grid): measured 6.3 TB/s against 4.7 TB/s for the same
    // loads spread a whole grid apart.  Indices still increase within a thread.
    const V *xv = reinterpret_cast<const V *>(x + head);
    constexpr int64_t kBlock = (int64_t)kVmaxUnroll * kVmaxThreads;
    const int64_t full_blocks = nvec / kBlock;
    for (int64_t blk = blockIdx.x; blk < full_blocks; blk += gridDim.x) {
        const int64_t v = blk * kBlock + tid;
        V buf[kVmaxUnroll];
#pragma unroll
        for (int u = 0; u < kVmaxUnroll; ++u) buf[u] = xv[v + u * kVmaxThreads];
#pragma unroll
        for (int u = 0; u < kVmaxUnroll; ++u) {
            const int64_t base = head + (v + u * kVmaxThreads) * VN;
#pragma unroll
            for (int e = 0; e < VN; ++e) feed(E::up(buf[u].e[e]), base + e);
        }
    }
    // the last, partial block goes to the workgroup whose turn it would be
    if ((int64_t)blockIdx.x == full_blocks % gridDim.x) {
        for (int64_t v = full_blocks * kBlock + tid; v < nvec; v += kVmaxThreads) {
            V buf = xv[v];
            const int64_t base = head + v * VN;
#pragma unroll
            for (int e = 0; e < VN; ++e) feed(E::up(buf.e[e]), base + e);
        }
    }
    const int64_t tail0 = head + nvec * VN;
    if (blockIdx.x == 0 && tail0 + tid < n) feed(E::up(x[tail0 + tid]), tail0 + tid);

    __shared__ C sval[kVmaxThreads / kWave];
    __shared__ int64_t sidx[kVmaxThreads / kWave];
    if (WITH_IDX) {
        wave_argmax(best, bidx);
    } else {
        best = wave_max(best);
    }
    const int wave = tid / kWave;
    if (lane_id() == 0) {
        sval[wave] = best;
        sidx[wave] = bidx;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kVmaxThreads / kWave; ++w) {
            if (WITH_IDX) {
                if (prefer(sval[w], sidx[w], best, bidx)) {
                    best = sval[w];
                    bidx = sidx[w];
                }
            } else {
                best = vmax_nan(best, sval[w]);
            }
        }
        if (FINAL) {
            *out_val = E::down(best);
            // every element is -inf: the first one is the answer, as in torch.max
            if (WITH_IDX) *out_idx = (bidx == kNoIdx) ? 0 : bidx;
        } else {
            pval[blockIdx.x] = best;
            if (WITH_IDX) pidx[blockIdx.x] = bidx;
        }
    }
}

template <int DT, bool WITH_IDX>
__global__ __launch_bounds__(kVmaxThreads) void vmax_stage2(
    const typename Elem<DT>::C *__restrict__ pval, const int64_t *__restrict__ pidx, int nparts,
    typename Elem<DT>::T *__restrict__ out_val, int64_t *__restrict__ out_idx) {
    using E = Elem<DT>;
    using C = typename E::C;
    C best = neg_inf<C>();
    int64_t bidx = kNoIdx;
    const int tid = threadIdx.x;
    for (int p = tid; p < nparts; p += kVmaxThreads) {
        C v = pval[p];
        if (WITH_IDX) {
            int64_t i = pidx[p];
            if (prefer(v, i, best, bidx)) {
                best = v;
                bidx = i;
            }
        } else {
            best = vmax_nan(best, v);
        }
    }
    __shared__ C sval[kVmaxThreads / kWave];
    __shared__ int64_t sidx[kVmaxThreads / kWave];
    if (WITH_IDX) {
        wave_argmax(best, bidx);
    } else {
        best = wave_max(best);
    }
    const int wave = tid / kWave;
    if (lane_id() == 0) {
        sval[wave] = best;
        sidx[wave] = bidx;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kVmaxThreads / kWave; ++w) {
            if (WITH_IDX) {
                if (prefer(sval[w], sidx[w], best, bidx)) {
                    best = sval[w];
                    bidx = sidx[w];
                }
            } else {
                best = vmax_nan(best, sval[w]);
            }
        }
        *out_val = E::down(best);
        // Every element is -inf (nothing compared greater than the initial
        // value): the first element is the answer, as in torch.max.
        if (WITH_IDX) *out_idx = (bidx == kNoIdx) ? 0 : bidx;
    }
}

static int vmax_blocks(int64_t nvec) {
    int64_t b = ceil_div(nvec, (int64_t)kVmaxThreads * kVmaxUnroll);
    if (b < 1) b = 1;
    if (b > kVmaxMaxBlocks) b = kVmaxMaxBlocks;
    return (int)b;
}

static size_t elem_size(int dtype) {
    switch (dtype) {
        case TRT_F32: return 4;
        case TRT_F64: return 8;
        case TRT_F16: return 2;
        case TRT_BF16: return 2;
        default: return 0;
    }
}

// workspace layout: [kVmaxMaxBlocks x 8-byte value slots][kVmaxMaxBlocks x int64]; vectors
// short enough for one workgroup need none
static bool vmax_single_block(int64_t n, int dtype) {
    const int64_t vn = 16 / (int64_t)elem_size(dtype);
    return n <= (int64_t)kVmaxThreads * kVmaxUnroll * vn * 2;
}
static size_t vmax_ws_bytes(int64_t n, int dtype) {
    return vmax_single_block(n, dtype) ? 0 : (size_t)kVmaxMaxBlocks * 16;
}

template <int DT>
static int vmax_launch(const void *x, int64_t n, void *out_val, int64_t *out_idx, void *ws,
                       hipStream_t stream) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    constexpr int VN = 16 / (int)sizeof(T);
    const T *xp = static_cast<const T *>(x);
    // elements before the first 16-byte boundary
    const uintptr_t addr = reinterpret_cast<uintptr_t>(xp);
    int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(T));
    if (head > n) head = n;
    const int64_t nvec = (n - head) / VN;
    T *ov = static_cast<T *>(out_val);
    if (vmax_single_block(n, DT)) {
        if (out_idx)
            hipLaunchKernelGGL((vmax_stage1<DT, true, true>), dim3(1), dim3(kVmaxThreads), 0, stream, xp, n, head,
                               nvec, (C *)nullptr, (int64_t *)nullptr, ov, out_idx);
        else
            hipLaunchKernelGGL((vmax_stage1<DT, false, true>), dim3(1), dim3(kVmaxThreads), 0, stream, xp, n, head,
                               nvec, (C *)nullptr, (int64_t *)nullptr, ov, out_idx);
        return (int)hipGetLastError();
    }
    const int blocks = vmax_blocks(nvec);
    C *pval = static_cast<C *>(ws);
    int64_t *pidx = reinterpret_cast<int64_t *>(static_cast<char *>(ws) + (size_t)kVmaxMaxBlocks * 8);
    if (out_idx) {
        hipLaunchKernelGGL((vmax_stage1<DT, true, false>), dim3(blocks), dim3(kVmaxThreads), 0, stream, xp, n,
                           head, nvec, pval, pidx, ov, out_idx);
        hipLaunchKernelGGL((vmax_stage2<DT, true>), dim3(1), dim3(kVmaxThreads), 0, stream, pval, pidx,
                           blocks, ov, out_idx);
    } else {
        hipLaunchKernelGGL((vmax_stage1<DT, false, false>), dim3(blocks), dim3(kVmaxThreads), 0, stream, xp, n,
                           head, nvec, pval, pidx, ov, out_idx);
        hipLaunchKernelGGL((vmax_stage2<DT, false>), dim3(1), dim3(kVmaxThreads), 0, stream, pval, pidx,
                           blocks, ov, out_idx);
    }
    return (int)hipGetLastError();
}

// ----------------------------------------------------------------- matmax
constexpr int kMatThreads = 256;
constexpr int kMatWaves = kMatThreads / kWave;

// Row maxima (reduction along the contiguous axis).  One wavefront per
// (row, column-chunk); lanes walk the row with VN-wide loads.
template <int DT, bool VEC>
__global__ __launch_bounds__(kMatThreads) void rowmax_kernel(
    const typename Elem<DT>::T *__restrict__ x, int64_t ld, int64_t m, int64_t n, int64_t chunk,
    int64_t splits, typename Elem<DT>::T *__restrict__ y, int64_t ldy) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int VN = V::N;
    const int wave = threadIdx.x / kWave;
    const int lane = lane_id();
    const int64_t split = blockIdx.x % splits;
    const int64_t row = (blockIdx.x / splits) * kMatWaves + wave;
    if (row >= m) return;
    const int64_t c0 = split * chunk;
    const int64_t c1 = (c0 + chunk < n) ? c0 + chunk : n;
    const T *xr = x + row * ld;
    C best = neg_inf<C>();
    if (VEC) {
        // ld, c0 and the base address are multiples of 16 bytes here
        const int64_t nv = (c1 - c0) / VN;
        const V *xv = reinterpret_cast<const V *>(xr + c0);
        int64_t v = lane;
        for (; v + 3 * kWave < nv; v += 4 * kWave) {
            V b0 = xv[v], b1 = xv[v + kWave], b2 = xv[v + 2 * kWave], b3 = xv[v + 3 * kWave];
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                best = vmax_nan(best, E::up(b0.e[e]));
                best = vmax_nan(best, E::up(b1.e[e]));
                best = vmax_nan(best, E::up(b2.e[e]));
                best = vmax_nan(best, E::up(b3.e[e]));
            }
        }
        for (; v < nv; v += kWave) {
            V b0 = xv[v];
#pragma unroll
            for (int e = 0; e < VN; ++e) best = vmax_nan(best, E::up(b0.e[e]));
        }
        for (int64_t c = c0 + nv * VN + lane; c < c1; c += kWave) best = vmax_nan(best, E::up(xr[c]));
    } else {
        for (int64_t c = c0 + lane; c < c1; c += kWave) best = vmax_nan(best, E::up(xr[c]));
    }
    best = wave_max(best);
    if (lane == 0) y[row * ldy + split] = E::down(best);
}

// Row maxima of long rows: one workgroup per row, its 256 lanes walking the row in contiguous
// blocks of 4 x 256 16-byte pieces (16 KiB).  Contiguous blocks per workgroup stream faster
// than four wavefronts on four different rows (measured on 16384^2 fp32: 174 us against 189 us).
template <int DT>
__global__ __launch_bounds__(kMatThreads) void rowmax_wide_kernel(const typename Elem<DT>::T *__restrict__ x,
                                                                  int64_t ld, int64_t n,
                                                                  typename Elem<DT>::T *__restrict__ y) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int VN = V::N;
    const int tid = threadIdx.x;
    const T *xr = x + (int64_t)blockIdx.x * ld;
    const V *xv = reinterpret_cast<const V *>(xr);
    const int64_t nv = n / VN;
    C best = neg_inf<C>();
    int64_t v = tid;
    for (; v + 3 * kMatThreads < nv; v += 4 * kMatThreads) {
        V b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) b[u] = xv[v + u * kMatThreads];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < VN; ++e) best = vmax_nan(best, E::up(b[u].e[e]));
    }
    for (; v < nv; v += kMatThreads) {
        V b0 = xv[v];
#pragma unroll
        for (int e = 0; e < VN; ++e) best = vmax_nan(best, E::up(b0.e[e]));
    }
    for (int64_t c = nv * VN + tid; c < n; c += kMatThreads) best = vmax_nan(best, E::up(xr[c]));
    best = wave_max(best);
    __shared__ C part[kMatWaves];
    if (lane_id() == 0) part[tid / kWave] = best;
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int w = 1; w < kMatWaves; ++w) best = vmax_nan(best, part[w]);
        y[blockIdx.x] = E::down(best);
    }
}

// Column maxima (reduction along the strided axis).  Each thread owns CN
// adjacent columns; the 4 wavefronts of a workgroup interleave over the rows
// of the workgroup's row chunk and combine through LDS.
template <int DT, bool VEC>
__global__ __launch_bounds__(kMatThreads) void colmax_kernel(
    const typename Elem<DT>::T *__restrict__ x, int64_t ld, int64_t m, int64_t n, int64_t rchunk,
    int64_t colblocks, typename Elem<DT>::T *__restrict__ y, int64_t ldy) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int CN = VEC ? V::N : 1;
    const int wave = threadIdx.x / kWave;
    const int lane = lane_id();
    const int64_t cb = blockIdx.x % colblocks;
    const int64_t split = blockIdx.x / colblocks;
    const int64_t col = (cb * kWave + lane) * CN;
    const int64_t r0 = split * rchunk;
    const int64_t r1 = (r0 + rchunk < m) ? r0 + rchunk : m;
    C best[CN];
#pragma unroll
    for (int e = 0; e < CN; ++e) best[e] = neg_inf<C>();
    if (col < n) {
        const T *xc = x + col;
        if (VEC) {
            int64_t r = r0 + wave;
            for (; r + 3 * kMatWaves < r1; r += 4 * kMatWaves) {
                V b0 = *reinterpret_cast<const V *>(xc + r * ld);
                V b1 = *reinterpret_cast<const V *>(xc + (r + kMatWaves) * ld);
                V b2 = *reinterpret_cast<const V *>(xc + (r + 2 * kMatWaves) * ld);
                V b3 = *reinterpret_cast<const V *>(xc + (r + 3 * kMatWaves) * ld);
#pragma unroll
                for (int e = 0; e < CN; ++e) {
                    best[e] = vmax_nan(best[e], E::up(b0.e[e]));
                    best[e] = vmax_nan(best[e], E::up(b1.e[e]));
                    best[e] = vmax_nan(best[e], E::up(b2.e[e]));
                    best[e] = vmax_nan(best[e], E::up(b3.e[e]));
                }
            }
            for (; r < r1; r += kMatWaves) {
                V b0 = *reinterpret_cast<const V *>(xc + r * ld);
#pragma unroll
                for (int e = 0; e < CN; ++e) best[e] = vmax_nan(best[e], E::up(b0.e[e]));
            }
        } else {
            for (int64_t r = r0 + wave; r < r1; r += kMatWaves)
                best[0] = vmax_nan(best[0], E::up(xc[r * ld]));
        }
    }
    __shared__ C sm[kMatWaves][kWave * CN];
#pragma unroll
    for (int e = 0; e < CN; ++e) sm[wave][lane * CN + e] = best[e];
    __syncthreads();
    if (wave == 0 && col < n) {
#pragma unroll
        for (int e = 0; e < CN; ++e) {
            C b = best[e];
            for (int w = 1; w < kMatWaves; ++w) b = vmax_nan(b, sm[w][lane * CN + e]);
            if (col + e < n) y[split * ldy + col + e] = E::down(b);
        }
    }
}

struct MatPlan {
    int64_t splits;  // partial results per output element (1: written straight to y)
    int64_t chunk;   // reduced-axis elements per partial
};

constexpr int64_t kTargetWaves = 4096;

// Rows of at least 16 KiB, enough of them to fill the chip, 16-byte aligned: one workgroup
// per row (rowmax_wide_kernel), no partial results.  (The same idea for axis 0 -- a
// workgroup on 4 KiB of each row -- measured no better at 16384^2 and worse at 8192^2.)
template <int DT>
static bool rowmax_wide(const void *x, int64_t m, int64_t n) {
    using T = typename Elem<DT>::T;
    constexpr int VN = 16 / (int)sizeof(T);
    return m >= 1024 && n * (int64_t)sizeof(T) >= 16384 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
           (n % VN) == 0 && m < ((int64_t)1 << 31);
}

static MatPlan rowmax_plan(int64_t m, int64_t n, int vn) {
    // enough (row, chunk) wavefronts to fill 256 CUs; chunks of >= 2048
    // elements, a multiple of the vector width.
    int64_t splits = ceil_div(kTargetWaves, m);
    const int64_t max_splits = n / 2048 > 0 ? n / 2048 : 1;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int64_t chunk = ceil_div(n, splits);
    chunk = ceil_div(chunk, (int64_t)(vn * kWave)) * (vn * kWave);
    splits = ceil_div(n, chunk);
    return {splits, chunk};
}

static MatPlan colmax_plan(int64_t m, int64_t n, int cn) {
    const int64_t colblocks = ceil_div(n, (int64_t)kWave * cn);
    int64_t splits = ceil_div(kTargetWaves / kMatWaves, colblocks);
    const int64_t max_splits = m / 32 > 0 ? m / 32 : 1;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    int64_t rchunk = ceil_div(m, splits);
    splits = ceil_div(m, rchunk);
    return {splits, rchunk};
}

// Partial column maxima are combined by the same kernel; more than 128 rows of them (tall,
// narrow matrices: few column blocks, so many row splits) go through an intermediate level of
// 64-row pieces instead of one workgroup walking them all.
static int64_t combine_splits(int64_t rows) { return rows > 128 ? ceil_div(rows, (int64_t)64) : 1; }

template <int DT>
static bool vec_ok(const void *p, int64_t ld) {
    constexpr int VN = 16 / (int)sizeof(typename Elem<DT>::T);
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && (ld % VN) == 0;
}

template <int DT>
static void rowmax_launch(const typename Elem<DT>::T *x, int64_t ld, int64_t m, int64_t n, MatPlan p,
                          typename Elem<DT>::T *y, int64_t ldy, hipStream_t stream) {
    const int64_t blocks = p.splits * ceil_div(m, (int64_t)kMatWaves);
    if (vec_ok<DT>(x, ld))
        hipLaunchKernelGGL((rowmax_kernel<DT, true>), dim3((unsigned)blocks), dim3(kMatThreads), 0, stream,
                           x, ld, m, n, p.chunk, p.splits, y, ldy);
    else
        hipLaunchKernelGGL((rowmax_kernel<DT, false>), dim3((unsigned)blocks), dim3(kMatThreads), 0, stream,
                           x, ld, m, n, p.chunk, p.splits, y, ldy);
}

template <int DT>
static void colmax_launch(const typename Elem<DT>::T *x, int64_t ld, int64_t m, int64_t n, bool vec,
                          MatPlan p, typename Elem<DT>::T *y, int64_t ldy, hipStream_t stream) {
    constexpr int VN = 16 / (int)sizeof(typename Elem<DT>::T);
    const int64_t colblocks = ceil_div(n, (int64_t)kWave * (vec ? VN : 1));
    const int64_t blocks = colblocks * p.splits;
    if (vec)
        hipLaunchKernelGGL((colmax_kernel<DT, true>), dim3((unsigned)blocks), dim3(kMatThreads), 0, stream,
                           x, ld, m, n, p.chunk, colblocks, y, ldy);
    else
        hipLaunchKernelGGL((colmax_kernel<DT, false>), dim3((unsigned)blocks), dim3(kMatThreads), 0, stream,
                           x, ld, m, n, p.chunk, colblocks, y, ldy);
}

template <int DT>
static size_t matmax_ws(int64_t m, int64_t n, int axis) {
    using T = typename Elem<DT>::T;
    constexpr int VN = 16 / (int)sizeof(T);
    if (axis == 1) {
        MatPlan p = rowmax_plan(m, n, VN);
        return p.splits > 1 ? (size_t)(m * p.splits) * sizeof(T) : 0;
    }
    // worst case over the vector / scalar column paths, plus the intermediate level
    MatPlan pv = colmax_plan(m, n, VN), ps = colmax_plan(m, n, 1);
    int64_t s = pv.splits > ps.splits ? pv.splits : ps.splits;
    if (s <= 1) return 0;
    const int64_t s2 = combine_splits(s);
    return (size_t)((s + (s2 > 1 ? s2 : 0)) * n) * sizeof(T);
}

template <int DT>
static int matmax_launch(const void *xv, void *yv, int64_t m, int64_t n, int axis, void *ws,
                         size_t ws_bytes, hipStream_t stream) {
    using T = typename Elem<DT>::T;
    constexpr int VN = 16 / (int)sizeof(T);
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    T *part = static_cast<T *>(ws);
    if (matmax_ws<DT>(m, n, axis) > ws_bytes) return TRT_E_WORKSPACE;
    if (matmax_ws<DT>(m, n, axis) > 0 && ws == nullptr) return TRT_E_WORKSPACE;
    if (axis == 1 && rowmax_wide<DT>(x, m, n)) {
        hipLaunchKernelGGL((rowmax_wide_kernel<DT>), dim3((unsigned)m), dim3(kMatThreads), 0, stream, x, n, n, y);
    } else if (axis == 1) {
        MatPlan p = rowmax_plan(m, n, VN);
        if (p.splits == 1) {
            rowmax_launch<DT>(x, n, m, n, p, y, 1, stream);
        } else {
            rowmax_launch<DT>(x, n, m, n, p, part, p.splits, stream);
            MatPlan p2{1, p.splits};
            rowmax_launch<DT>(part, p.splits, m, p.splits, p2, y, 1, stream);
        }
    } else {
        const bool vec = vec_ok<DT>(x, n);
        MatPlan p = colmax_plan(m, n, vec ? VN : 1);
        if (p.splits == 1) {
            colmax_launch<DT>(x, n, m, n, vec, p, y, n, stream);
        } else {
            colmax_launch<DT>(x, n, m, n, vec, p, part, n, stream);
            int64_t rows = p.splits;
            const int64_t s2 = combine_splits(rows);
            if (s2 > 1) {  // intermediate level behind the first partials (sized by matmax_ws)
                MatPlan pc{s2, 64};
                T *part2 = part + rows * n;
                colmax_launch<DT>(part, n, rows, n, vec_ok<DT>(part, n), pc, part2, n, stream);
                part = part2;
                rows = s2;
            }
            MatPlan p2{1, rows};
            colmax_launch<DT>(part, n, rows, n, vec_ok<DT>(part, n), p2, y, n, stream);
        }
    }
    return (int)hipGetLastError();
}

// Largest workgroup count among the launches of a matmax call (same plans as matmax_launch).
static int64_t matmax_max_blocks(int64_t m, int64_t n, int axis, int dtype) {
    const int vn = 16 / (int)elem_size(dtype);
    if (axis == 1) {
        // one workgroup per row (long rows), or one per 4 rows and column chunk
        const int64_t wide = m;
        const int64_t split = rowmax_plan(m, n, vn).splits * ceil_div(m, (int64_t)kMatWaves);
        return wide > split ? wide : split;
    }
    int64_t most = 0;
    for (int cn = 1; cn <= vn; cn += vn - 1 > 0 ? vn - 1 : 1) {  // the scalar and the vector column paths
        const int64_t colblocks = ceil_div(n, (int64_t)kWave * cn);
        const int64_t splits = colmax_plan(m, n, cn).splits;
        const int64_t s2 = combine_splits(splits);
        const int64_t blocks = colblocks * (splits > s2 ? splits : s2);
        if (blocks > most) most = blocks;
    }
    return most;
}

}  // namespace trt

using namespace trt;

extern "C" size_t trt_vmax_workspace_bytes(int64_t n, int dtype) {
    return (elem_size(dtype) && n > 0) ? vmax_ws_bytes(n, dtype) : 0;
}

extern "C" int trt_vmax(const void *x, int64_t n, int dtype, void *out_val, int64_t *out_idx,
                        void *workspace, size_t workspace_bytes, void *stream) {
    if (!x || !out_val || n <= 0 || !elem_size(dtype)) return TRT_E_INVALID;
    const size_t need = vmax_ws_bytes(n, dtype);
    if (need && (!workspace || workspace_bytes < need)) return TRT_E_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(x) % elem_size(dtype)) != 0) return TRT_E_LAYOUT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case TRT_F32: return vmax_launch<TRT_F32>(x, n, out_val, out_idx, workspace, s);
        case TRT_F64: return vmax_launch<TRT_F64>(x, n, out_val, out_idx, workspace, s);
        case TRT_F16: return vmax_launch<TRT_F16>(x, n, out_val, out_idx, workspace, s);
        default: return vmax_launch<TRT_BF16>(x, n, out_val, out_idx, workspace, s);
    }
}

extern "C" size_t trt_matmax_workspace_bytes(int64_t m, int64_t n, int axis, int dtype) {
    if (m <= 0 || n <= 0 || (axis != 0 && axis != 1)) return 0;
    switch (dtype) {
        case TRT_F32: return matmax_ws<TRT_F32>(m, n, axis);
        case TRT_F64: return matmax_ws<TRT_F64>(m, n, axis);
        case TRT_F16: return matmax_ws<TRT_F16>(m, n, axis);
        case TRT_BF16: return matmax_ws<TRT_BF16>(m, n, axis);
        default: return 0;
    }
}

extern "C" int trt_matmax(const void *x, void *y, int64_t m, int64_t n, int axis, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream) {
    if (!x || !y || m <= 0 || n <= 0 || (axis != 0 && axis != 1) || !elem_size(dtype))
        return TRT_E_INVALID;
    if ((reinterpret_cast<uintptr_t>(x) % elem_size(dtype)) != 0) return TRT_E_LAYOUT;
    if (m > (int64_t)1 << 40 || n > (int64_t)1 << 40) return TRT_E_RANGE;
    // workgroup ids are 32-bit: every launch of the call must stay below 2^31 workgroups
    if (matmax_max_blocks(m, n, axis, dtype) >= ((int64_t)1 << 31)) return TRT_E_RANGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case TRT_F32: return matmax_launch<TRT_F32>(x, y, m, n, axis, workspace, workspace_bytes, s);
        case TRT_F64: return matmax_launch<TRT_F64>(x, y, m, n, axis, workspace, workspace_bytes, s);
        case TRT_F16: return matmax_launch<TRT_F16>(x, y, m, n, axis, workspace, workspace_bytes, s);
        default: return matmax_launch<TRT_BF16>(x, y, m, n, axis, workspace, workspace_bytes, s);
    }
}

// ------------------------------------------------------------ copy kernel
// One contiguous block of 4 * 256 16-byte pieces per workgroup, non-temporal both ways.
__global__ __launch_bounds__(256) void copy16_kernel(const trt::uintx4 *__restrict__ src,
                                                     trt::uintx4 *__restrict__ dst, size_t nvec) {
    const size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
    trt::uintx4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (base + u * 256 < nvec) v[u] = __builtin_nontemporal_load(&src[base + u * 256]);
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (base + u * 256 < nvec) __builtin_nontemporal_store(v[u], &dst[base + u * 256]);
}

extern "C" int trt_copy_bytes(const void *src, void *dst, size_t nbytes, void *stream) {
    if (!src || !dst || nbytes == 0 || (nbytes & 15)) return TRT_E_INVALID;
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) return TRT_E_LAYOUT;
    const size_t nvec = nbytes / 16;
    const size_t blocks = (nvec + 1023) / 1024;
    if (blocks >= ((size_t)1 << 31)) return TRT_E_RANGE;
    hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const trt::uintx4 *>(src), static_cast<trt::uintx4 *>(dst), nvec);
    return (int)hipGetLastError();
}
