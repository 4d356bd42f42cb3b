// matmax / vmax / vamax for gfx950: every element is read once from HBM with
// 16-byte coalesced loads, reduced in registers, then across the 64-lane
// wavefront, then across the workgroup through LDS.  A reduction is one launch:
// the workgroups leave partial results in the caller's workspace and the one that
// finishes last combines them (unaligned or very wide matrices keep a tree of
// two or three launches, colmax_kernel / rowmax_kernel).
//
// Semantics follow torch, the oracle the reference tests use
// (tests/max.py:13,22,32): NaN propagates; argmax ties go to the lowest index
// and a NaN reports the first NaN.
//
// Replaces: _ker_vamax / _ker_vmax / _ker_matmax, triturus/max.py:8-32,62-93,125-168.

#include <type_traits>

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

// max that ignores a NaN operand (both NaN: NaN), one instruction without canonicalisation moves
__device__ __forceinline__ float max_ignoring_nan(float a, float b) { return max3_raw(a, b, b); }
__device__ __forceinline__ double max_ignoring_nan(double a, double b) { return __builtin_fmax(a, b); }
__device__ __forceinline__ float max3_ignoring_nan(float a, float b, float c) { return max3_raw(a, b, c); }
__device__ __forceinline__ double max3_ignoring_nan(double a, double b, double c) {
    return __builtin_fmax(__builtin_fmax(a, b), c);
}

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

// ---- wavefront reductions on the data-parallel-primitive path: six register moves between
// lanes (within quads, within rows of 16, then row to row) instead of six round trips through
// the LDS permute unit; the result is complete in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v) {
    const int x = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(x, x, CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move(double v) {
    const uint64_t x = __builtin_bit_cast(uint64_t, v);
    const int lo = (int)(uint32_t)x, hi = (int)(uint32_t)(x >> 32);
    const uint32_t l2 = (uint32_t)__builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
    const uint32_t h2 = (uint32_t)__builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
    return __builtin_bit_cast(double, ((uint64_t)h2 << 32) | l2);
}
__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ double read_lane(double v, int lane) {
    const uint64_t x = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)x, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(x >> 32), lane);
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

// Maximum over the wavefront (a NaN wins), the same value in every lane.
template <typename C>
__device__ __forceinline__ C wave_max(C v) {
    v = vmax_nan(v, dpp_move<0xb1, 0xf>(v));   // quad_perm [1,0,3,2]
    v = vmax_nan(v, dpp_move<0x4e, 0xf>(v));   // quad_perm [2,3,0,1]
    v = vmax_nan(v, dpp_move<0x114, 0xf>(v));  // row_shr 4
    v = vmax_nan(v, dpp_move<0x118, 0xf>(v));  // row_shr 8
    v = vmax_nan(v, dpp_move<0x142, 0xa>(v));  // row_bcast 15 into rows 1 and 3
    v = vmax_nan(v, dpp_move<0x143, 0xc>(v));  // row_bcast 31 into rows 2 and 3
    return read_lane(v, 63);
}

__device__ __forceinline__ int64_t read_lane(int64_t v, int lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(uint64_t)v, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), lane);
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int64_t min_with_moved(int64_t v) {
    const int lo = (int)(uint32_t)(uint64_t)v, hi = (int)(uint32_t)((uint64_t)v >> 32);
    const uint32_t l2 = (uint32_t)__builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
    const uint32_t h2 = (uint32_t)__builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
    const int64_t o = (int64_t)(((uint64_t)h2 << 32) | l2);
    return o < v ? o : v;
}

// (Maximum, lowest index among the lanes that hold it) over the wavefront, in every lane: the
// value by wave_max, then the smallest index of the lanes that hold it by the same six moves
// (a fixed cost whether one lane holds the maximum or all of them do).
template <typename C>
__device__ __forceinline__ void wave_argmax(C &v, int64_t &i) {
    const C m = wave_max(v);
    const bool mine = (v == m) || (v != v && m != m);
    int64_t j = mine ? i : kNoIdx;
    j = min_with_moved<0xb1, 0xf>(j);
    j = min_with_moved<0x4e, 0xf>(j);
    j = min_with_moved<0x114, 0xf>(j);
    j = min_with_moved<0x118, 0xf>(j);
    j = min_with_moved<0x142, 0xa>(j);
    j = min_with_moved<0x143, 0xc>(j);
    const int64_t best = read_lane(j, 63);
    // the value as the winning lane holds it (-0.0 and +0.0 compare equal: the bits of the
    // element at the reported index are what torch.max returns)
    const uint64_t winner = __builtin_amdgcn_ballot_w64(mine && i == best);
    v = read_lane(v, __builtin_ctzll(winner ? winner : 1));
    i = best;
}

// 16-byte vector of T
template <typename T>
struct alignas(16) Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T e[N];
};

// ------------------------------------------------------------------- vmax
constexpr int kVmaxThreads = 256;
constexpr int kVmaxMaxBlocks = 512;  // two workgroups per compute unit; each walks several blocks
constexpr int kVmaxUnroll = 8;
constexpr int kVmaxGroup = 32;  // workgroups that draw from one arrival counter

// Arrival counters ("tickets") at the head of a max workspace: a launch whose workgroups leave
// partial results takes one ticket per workgroup; the workgroup that draws the last one
// combines the partials and puts the counter back to its idle value.  The counters must be idle
// before the first call that uses a workspace (trt_max_workspace_init) and every call leaves
// them idle, so one launch does the work of two and the library still keeps no state of its own.
// A counter is a 64-bit word: a fixed tag in the upper half, the number of arrivals in the lower.
// A workgroup that draws a word with another tag, or a count its launch cannot have produced,
// knows that the workspace was never prepared or has been written over: it elects nobody and
// writes a NaN (index -1) where the result belongs, so that a broken workspace shows in the
// output instead of leaving it unwritten.
constexpr size_t kTicketBytes = TRT_MAX_TICKET_BYTES;
using Ticket = unsigned long long;
constexpr Ticket kTicketTag = (Ticket)0x7452544Bu << 32;  // "tRTK": idle counter = tag, no arrivals
// Counters that different groups of workgroups draw from sit 256 bytes apart: device-scope atomics on
// one memory line are served one after the other (measured ~10 ns each), on different lines side by side.
constexpr int kTicketStride = 256 / (int)sizeof(Ticket);
constexpr int kMaxTickets = (int)(kTicketBytes / 256);
// drawn: what the counter held before this workgroup's arrival; of: arrivals the launch makes
__device__ __forceinline__ bool ticket_last(Ticket drawn, int of) { return drawn == (kTicketTag | (Ticket)(of - 1)); }
__device__ __forceinline__ bool ticket_sound(Ticket drawn, int of) {
    return (drawn >> 32) == (kTicketTag >> 32) && (unsigned)drawn < (unsigned)of;
}
static_assert(kVmaxMaxBlocks / kVmaxGroup < kMaxTickets, "one counter per group and one for the groups");

// The partials of the other workgroups were written on other compute units (and other dies,
// each with its own L2), so partials and tickets are device-scope atomic accesses, which go
// past the caches that are not coherent across the device.  A device-scope FENCE would do as
// well but writes back and invalidates whole caches, once per workgroup: measured 120 us
// instead of 12 us on a 64 MiB vector.  Between its partial stores and its ticket a wavefront
// waits for the stores to be acknowledged (a workgroup-scope release: a wait, no cache action).
// Partial results themselves travel as 16-byte buffer accesses with the device-scope bit (sc1)
// of the cache policy.  A wavefront's device-scope accesses do not overlap one another -- each
// costs a trip of some 170 ns (measured: the last workgroup's time grows by that much per load
// instruction) -- so a partial is one 16-byte record, not a word per field.
constexpr int kDeviceScope = 16;
__device__ __forceinline__ Ticket take_ticket(Ticket *ticket) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    return __hip_atomic_fetch_add(ticket, (Ticket)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The same for a whole wavefront that has stored: lane 0 draws, the others wait with it.
__device__ __forceinline__ Ticket take_ticket_wave(Ticket *ticket) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    Ticket t = 0;
    if (lane_id() == 0) t = __hip_atomic_fetch_add(ticket, (Ticket)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return t;
}
__device__ __forceinline__ void ticket_idle(Ticket *ticket) {  // ready for the next call
    __hip_atomic_store(ticket, kTicketTag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Workgroups go to the 8 dies (each with an L2 of its own) round-robin: logical position of a
// workgroup such that each die owns a run of consecutive positions.  A column reduction hands
// each die whole row splits -- all column blocks of them -- and not one column block of every
// split (rows a power of two apart map to the same few channels of a die's L2: measured 14.6 us
// against 18.2 us on a 4096 x 4096 fp32 matrix); a sweep of a vector gives each die one
// contiguous eighth.
constexpr int kDies = 8;
__device__ __forceinline__ int64_t die_major(int64_t block, int64_t total) {
    return (total % kDies == 0) ? (block % kDies) * (total / kDies) + block / kDies : block;
}

// One 16-byte piece.  ONCE: a non-temporal load, for operands too large to be found in L2 by a
// later call (kStreamBytes): the sweep of a 64 MiB operand then runs at 7.0-7.5 TB/s where
// ordinary loads of the same pattern reach 6.1, provided the engine clock is up (at the few
// hundred MHz of a GPU that has just been idle the two are level).  Operands that fit L2 keep
// ordinary loads: read again by the next call, they are served from L2 (16 MiB: 5.6 us against
// 6.8 with non-temporal loads).
constexpr int64_t kStreamBytes = (int64_t)32 << 20;
template <bool ONCE, class V>
__device__ __forceinline__ V load_piece(const V *p) {
    static_assert(sizeof(V) == 16, "a 16-byte piece");
    if constexpr (ONCE) {
        const uintx4 bits = __builtin_nontemporal_load(reinterpret_cast<const uintx4 *>(p));
        V v;
        __builtin_memcpy(&v, &bits, 16);
        return v;
    } else {
        return *p;
    }
}
using OnceT = std::true_type;
using AgainT = std::false_type;

// Max and first-occurrence argmax in one launch.  Every 16-byte piece costs a couple of vector
// instructions: the maximum of its elements (NaN ignored), one unordered test per pair of elements
// to notice NaNs, and a compare-and-select of (value, piece number) -- the position inside the
// piece is worked out once, at the end, by reading the winning piece again.  A wavefront that has
// seen a NaN repeats its share element by element with the exact rule (a NaN wins, first one
// reported), which costs nothing on inputs without NaN.
// FINAL: the launch has a single workgroup, which writes the result itself.
template <int DT, bool WITH_IDX, bool FINAL>
__global__ __launch_bounds__(kVmaxThreads) void vmax_kernel(
    const typename Elem<DT>::T *__restrict__ x, int64_t n, int64_t head, int64_t nvec,
    int64_t share_q, int share_rem, int once, uintx4 *prec, Ticket *ticket,
    typename Elem<DT>::T *__restrict__ out_val, int64_t *__restrict__ out_idx) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int VN = V::N;
    const int tid = threadIdx.x;
    const V *xv = reinterpret_cast<const V *>(x + head);
    constexpr int64_t kBlock = (int64_t)kVmaxUnroll * kVmaxThreads;
    const int64_t full_blocks = nvec / kBlock;

    // ---- fast sweep: best piece maximum and the number of the piece (in this thread's
    // visiting order) that first reached it
    C bv = neg_inf<C>();
    unsigned bk = 0xffffffffu;  // no piece yet
    V bpiece;                   // the piece itself: its elements decide the position at the end
#pragma unroll
    for (int e = 0; e < VN; ++e) bpiece.e[e] = T();
    bool saw_nan = false;
    auto piece_max = [&](const V &b, C &m, bool &un) {
        C c[VN];
#pragma unroll
        for (int e = 0; e < VN; ++e) c[e] = E::up(b.e[e]);
        m = c[0];
#pragma unroll
        for (int e = 1; e < VN; ++e) m = max_ignoring_nan(m, c[e]);
#pragma unroll
        for (int e = 0; e + 1 < VN; e += 2) un |= __builtin_isunordered(c[e], c[e + 1]);
    };
    // The vector is cut into blocks of kVmaxUnroll * kVmaxThreads 16-byte pieces; a workgroup
    // takes a run of consecutive blocks (share_q of them, one more for the first share_rem
    // workgroups), and the workgroups of a die take consecutive runs, so each die streams one
    // contiguous eighth of the vector.  Measured on 64 MiB: 9.6 us for the bare sweep against
    // 10.5 with the blocks dealt round-robin over the grid (and 11.1 with ordinary loads).
    // Piece numbers increase with the index within a thread.
    const int64_t logical = die_major(blockIdx.x, gridDim.x);
    const int64_t first_block = logical * share_q + (logical < share_rem ? logical : share_rem);
    const int64_t end_block = first_block + share_q + (logical < share_rem ? 1 : 0);
    unsigned k = 0;
    auto sweep = [&](auto once_tag) {
        for (int64_t blk = first_block; blk < end_block; ++blk) {
            const int64_t v = blk * kBlock + tid;
            V buf[kVmaxUnroll];
#pragma unroll
            for (int u = 0; u < kVmaxUnroll; ++u)
                buf[u] = load_piece<decltype(once_tag)::value>(&xv[v + u * kVmaxThreads]);
            // every load of the block is issued before the first piece is looked at
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kVmaxUnroll; ++u) {
                C m;
                piece_max(buf[u], m, saw_nan);
                const bool take = m > bv;
                bv = take ? m : bv;
                if (WITH_IDX) {
                    bk = take ? k + u : bk;
#pragma unroll
                    for (int e = 0; e < VN; ++e) bpiece.e[e] = take ? buf[u].e[e] : bpiece.e[e];
                }
            }
            k += kVmaxUnroll;
        }
    };
    if (once) sweep(OnceT{});
    else sweep(AgainT{});
    const unsigned in_full = k;  // pieces of whole blocks come first in the visiting order
    // the last, partial block goes to the workgroup of the last run
    const bool has_tail_block = logical == (int64_t)gridDim.x - 1;
    if (has_tail_block) {
        for (int64_t v = full_blocks * kBlock + tid; v < nvec; v += kVmaxThreads) {
            C m;
            const V b = xv[v];
            piece_max(b, m, saw_nan);
            const bool take = m > bv;
            bv = take ? m : bv;
            if (WITH_IDX) {
                bk = take ? k : bk;
#pragma unroll
                for (int e = 0; e < VN; ++e) bpiece.e[e] = take ? b.e[e] : bpiece.e[e];
            }
            ++k;
        }
    }
    // piece number -> absolute piece index (the inverse of the two loops above)
    auto piece_index = [&](unsigned kk) -> int64_t {
        if (kk < in_full)
            return (first_block + (int64_t)(kk / kVmaxUnroll)) * kBlock + tid +
                   (int64_t)(kk % kVmaxUnroll) * kVmaxThreads;
        return full_blocks * kBlock + tid + (int64_t)(kk - in_full) * kVmaxThreads;
    };

    C best = neg_inf<C>();
    int64_t bidx = kNoIdx;
    auto feed = [&](C c, int64_t i) {  // exact rule, any order
        if (prefer(c, i, best, bidx)) {
            best = c;
            bidx = i;
        }
    };
    if (__builtin_amdgcn_ballot_w64(saw_nan) != 0) {
        // ---- a NaN somewhere in this wavefront's share: element by element, exact rule
        for (int64_t blk = first_block; blk < end_block; ++blk)
            for (int u = 0; u < kVmaxUnroll; ++u) {
                const int64_t v = blk * kBlock + tid + u * kVmaxThreads;
                const V b = xv[v];
#pragma unroll
                for (int e = 0; e < VN; ++e) feed(E::up(b.e[e]), head + v * VN + e);
            }
        if (has_tail_block)
            for (int64_t v = full_blocks * kBlock + tid; v < nvec; v += kVmaxThreads) {
                const V b = xv[v];
#pragma unroll
                for (int e = 0; e < VN; ++e) feed(E::up(b.e[e]), head + v * VN + e);
            }
    } else if (bk != 0xffffffffu || !WITH_IDX) {
        // ---- the winning piece: its first element equal to the maximum (the element's own
        // bits are reported: -0.0 and +0.0 compare equal)
        best = bv;
        if (WITH_IDX) {
            const int64_t v = piece_index(bk);
#pragma unroll
            for (int e = VN - 1; e >= 0; --e) {
                const C c = E::up(bpiece.e[e]);
                if (c == bv) {
                    best = c;
                    bidx = head + v * VN + e;
                }
            }
        }
    } else if (k > 0) {
        // ---- no piece rose above -inf: every element of this thread's share is -inf, and the
        // first of them is its candidate (a later tail element must not win the tie)
        bidx = head + piece_index(0) * VN;
    }
    // elements before the first and after the last whole 16-byte piece
    if (blockIdx.x == 0 && tid < head) feed(E::up(x[tid]), tid);
    const int64_t tail0 = head + nvec * VN;
    if (blockIdx.x == 0 && tail0 + tid < n) feed(E::up(x[tail0 + tid]), tail0 + tid);

    __shared__ C sval[kVmaxThreads / kWave];
    __shared__ int64_t sidx[kVmaxThreads / kWave];
    __shared__ bool last_block;
    auto wave_reduce = [&]() {
        if (WITH_IDX) {
            wave_argmax(best, bidx);
        } else {
            best = wave_max(best);
        }
    };
    auto block_reduce = [&]() {  // result in thread 0
        wave_reduce();
        if (lane_id() == 0) {
            sval[tid / kWave] = best;
            sidx[tid / kWave] = bidx;
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
        }
    };
    auto write_result = [&]() {
        *out_val = E::down(best);
        // every element is -inf: the first one is the answer, as in torch.max
        if (WITH_IDX) *out_idx = (bidx == kNoIdx) ? 0 : bidx;
    };
    block_reduce();
    if (FINAL) {
        if (tid == 0) write_result();
        return;
    }
    // ---- "the last to arrive combines", counted at two levels: the last workgroup of a group of
    // kVmaxGroup draws from the counter of the groups, and the last of those combines all the
    // partials.  (One counter for all workgroups would serialise a burst of device-scope atomics
    // at the end of the sweep; combining group by group would add a round trip of partials.)
    const int nblocks = (int)gridDim.x;
    const int group = blockIdx.x / kVmaxGroup;
    const int ngroups = (nblocks + kVmaxGroup - 1) / kVmaxGroup;
    const int gfirst = group * kVmaxGroup;
    const int gsize = nblocks - gfirst < kVmaxGroup ? nblocks - gfirst : kVmaxGroup;
    union Record {
        struct {
            C val;  // (a 4-byte value leaves the rest of its 8-byte slot unused)
            int64_t idx;
        } f;
        uintx4 bits;
    };
    static_assert(sizeof(Record) == 16, "one 16-byte access per partial");
    const __amdgpu_buffer_rsrc_t prsrc = make_rsrc(prec, (uint32_t)kVmaxMaxBlocks * 16u);
    Ticket *tick1 = ticket + group * kTicketStride;
    Ticket *tick2 = ticket + (kMaxTickets - 1) * kTicketStride;
    if (tid == 0) {
        // the partial: one 16-byte record (value in an 8-byte slot, index)
        Record rec;
        rec.f.val = best;
        rec.f.idx = bidx;
        __builtin_amdgcn_raw_buffer_store_b128(rec.bits, prsrc, (uint32_t)blockIdx.x * 16u, 0, kDeviceScope);
        Ticket drawn = take_ticket(tick1);
        bool sound = ticket_sound(drawn, gsize);
        bool last = ticket_last(drawn, gsize);
        if (last) {
            drawn = take_ticket(tick2);
            sound = ticket_sound(drawn, ngroups);
            last = ticket_last(drawn, ngroups);
            ticket_idle(tick1);
        }
        if (!sound) {  // counters that no launch of this library left behind: say so in the result
            *out_val = E::down((C)__builtin_nanf(""));
            if (WITH_IDX) *out_idx = -1;
        }
        last_block = last;
    }
    __syncthreads();
    if (!last_block) return;
    best = neg_inf<C>();
    bidx = kNoIdx;
    // every partial is asked for before the first is looked at: one round trip, not one per partial
    constexpr int kPer = (kVmaxMaxBlocks + kVmaxThreads - 1) / kVmaxThreads;
    // (a slot past the last workgroup is replaced by slot 0: seeing a partial twice changes nothing)
    Record pr[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const int i = tid + u * kVmaxThreads;
        pr[u].bits = __builtin_amdgcn_raw_buffer_load_b128(prsrc, (uint32_t)(i < nblocks ? i : 0) * 16u, 0, kDeviceScope);
    }
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        if (WITH_IDX) {
            feed(pr[u].f.val, pr[u].f.idx);
        } else {
            best = vmax_nan(best, pr[u].f.val);
        }
    }
    block_reduce();
    if (tid == 0) {
        write_result();
        ticket_idle(tick2);
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

// workspace layout: [tickets][kVmaxMaxBlocks x 16-byte records (value slot, int64 index)];
// vectors short enough for one workgroup need none
static bool vmax_single_block(int64_t n, int dtype) {
    const int64_t vn = 16 / (int64_t)elem_size(dtype);
    return n <= (int64_t)kVmaxThreads * kVmaxUnroll * vn * 2;
}
static size_t vmax_ws_bytes(int64_t n, int dtype) {
    return vmax_single_block(n, dtype) ? 0 : kTicketBytes + (size_t)kVmaxMaxBlocks * 16;
}

template <int DT>
static int vmax_launch(const void *x, int64_t n, void *out_val, int64_t *out_idx, void *ws,
                       hipStream_t stream) {
    using E = Elem<DT>;
    using T = typename E::T;
    constexpr int VN = 16 / (int)sizeof(T);
    const T *xp = static_cast<const T *>(x);
    // elements before the first 16-byte boundary
    const uintptr_t addr = reinterpret_cast<uintptr_t>(xp);
    int64_t head = (int64_t)(((16 - (addr & 15)) & 15) / sizeof(T));
    if (head > n) head = n;
    const int64_t nvec = (n - head) / VN;
    const int64_t full_blocks = nvec / ((int64_t)kVmaxUnroll * kVmaxThreads);  // whole blocks of pieces
    T *ov = static_cast<T *>(out_val);
    if (vmax_single_block(n, DT)) {
        if (out_idx)
            hipLaunchKernelGGL((vmax_kernel<DT, true, true>), dim3(1), dim3(kVmaxThreads), 0, stream, xp, n, head,
                               nvec, full_blocks, 0, 0, (uintx4 *)nullptr, (Ticket *)nullptr, ov, out_idx);
        else
            hipLaunchKernelGGL((vmax_kernel<DT, false, true>), dim3(1), dim3(kVmaxThreads), 0, stream, xp, n, head,
                               nvec, full_blocks, 0, 0, (uintx4 *)nullptr, (Ticket *)nullptr, ov, out_idx);
        return (int)hipGetLastError();
    }
    const int blocks = vmax_blocks(nvec);
    const int64_t share_q = full_blocks / blocks;
    const int share_rem = (int)(full_blocks % blocks);
    const int once = n * (int64_t)sizeof(T) >= kStreamBytes;
    Ticket *ticket = static_cast<Ticket *>(ws);
    uintx4 *prec = reinterpret_cast<uintx4 *>(static_cast<char *>(ws) + kTicketBytes);
    if (out_idx)
        hipLaunchKernelGGL((vmax_kernel<DT, true, false>), dim3(blocks), dim3(kVmaxThreads), 0, stream, xp, n, head,
                           nvec, share_q, share_rem, once, prec, ticket, ov, out_idx);
    else
        hipLaunchKernelGGL((vmax_kernel<DT, false, false>), dim3(blocks), dim3(kVmaxThreads), 0, stream, xp, n, head,
                           nvec, share_q, share_rem, once, prec, ticket, ov, out_idx);
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
    int64_t splits, int once, typename Elem<DT>::T *__restrict__ y, int64_t ldy) {
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
        auto sweep = [&](auto once_tag) {
            constexpr bool ONCE = decltype(once_tag)::value;
            for (; v + 3 * kWave < nv; v += 4 * kWave) {
                V b0 = load_piece<ONCE>(&xv[v]), b1 = load_piece<ONCE>(&xv[v + kWave]),
                  b2 = load_piece<ONCE>(&xv[v + 2 * kWave]), b3 = load_piece<ONCE>(&xv[v + 3 * kWave]);
#pragma unroll
                for (int e = 0; e < VN; ++e) {
                    best = vmax_nan(best, E::up(b0.e[e]));
                    best = vmax_nan(best, E::up(b1.e[e]));
                    best = vmax_nan(best, E::up(b2.e[e]));
                    best = vmax_nan(best, E::up(b3.e[e]));
                }
            }
        };
        if (once) sweep(OnceT{});
        else sweep(AgainT{});
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
                                                                  int64_t ld, int64_t n, int once,
                                                                  typename Elem<DT>::T *__restrict__ y) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int VN = V::N;
    const int tid = threadIdx.x;
    const int64_t row = die_major(blockIdx.x, gridDim.x);  // each die streams a run of consecutive rows
    const T *xr = x + row * ld;
    const V *xv = reinterpret_cast<const V *>(xr);
    const int64_t nv = n / VN;
    C best = neg_inf<C>();
    int64_t v = tid;
    auto sweep = [&](auto once_tag) {
        for (; v + 3 * kMatThreads < nv; v += 4 * kMatThreads) {
            V b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) b[u] = load_piece<decltype(once_tag)::value>(&xv[v + u * kMatThreads]);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < VN; ++e) best = vmax_nan(best, E::up(b[u].e[e]));
        }
    };
    if (once) sweep(OnceT{});
    else sweep(AgainT{});
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
        y[row] = E::down(best);
    }
}

// Column maxima (reduction along the strided axis).  Each thread owns CN
// adjacent columns; the 4 wavefronts of a workgroup interleave over the rows
// of the workgroup's row chunk and combine through LDS.
// Row splits leave partial rows that further launches of this kernel combine; matrices that
// colmax_fused_kernel covers take that one-launch path instead.
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
    const int64_t logical = die_major(blockIdx.x, gridDim.x);
    const int64_t cb = logical % colblocks;
    const int64_t split = logical / colblocks;
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

// Column maxima in one launch, for 16-byte-aligned matrices whose row splits number at most
// kColFusedSplits: as colmax_kernel, then the workgroup of a column block that finishes last
// combines the block's partial rows (device-scope 8-byte accesses, see take_ticket) and writes y.
// VPL: 16-byte vectors per lane.  With 2 a wavefront reads 2 KiB of a row at a time and a
// workgroup owns 512 (fp32) columns: measured on 4096 x 4096 fp32 with 128 rows per workgroup,
// the sweep alone takes 12.9 us against 13.3 us with 1 KiB pieces (16384^2: 173 against 182 us);
// the host picks it for large matrices only (colmax_fused_plan).
constexpr int kColFusedSplits = 32;
constexpr int kColFusedUnroll = 8;  // 16-byte loads in flight per lane
template <int DT, int VPL>
__global__ __launch_bounds__(kMatThreads) void colmax_fused_kernel(
    const typename Elem<DT>::T *__restrict__ x, int64_t ld, int64_t m, int64_t n, int64_t rchunk,
    int colblocks, int splits, int once, unsigned long long *part, Ticket *ticket,
    typename Elem<DT>::T *__restrict__ y) {
    using E = Elem<DT>;
    using T = typename E::T;
    using C = typename E::C;
    using V = Vec16<T>;
    constexpr int VN = V::N;
    constexpr int CN = VPL * VN;                    // columns per lane: VPL pieces, kWave * VN columns apart
    constexpr int ROWS = kColFusedUnroll / VPL;     // rows in flight per wavefront
    const int wave = threadIdx.x / kWave;
    const int lane = lane_id();
    const int logical = (int)die_major(blockIdx.x, gridDim.x);
    const int cb = logical % colblocks;
    const int split = logical / colblocks;
    const int64_t col = ((int64_t)cb * VPL * kWave + lane) * VN;  // of the lane's first piece
    const int64_t r0 = split * rchunk;
    const int64_t r1 = (r0 + rchunk < m) ? r0 + rchunk : m;
    bool have[VPL];  // the piece lies inside the matrix (n is a multiple of VN here)
#pragma unroll
    for (int p = 0; p < VPL; ++p) have[p] = col + (int64_t)p * kWave * VN < n;
    C best[CN];
#pragma unroll
    for (int e = 0; e < CN; ++e) best[e] = neg_inf<C>();
    // A piece that lies past the matrix is read from a valid place instead (the lane's first
    // piece, or column 0) and never written to y: the sweep carries no predicates.
    const T *xc = x + (have[0] ? col : 0);
    int64_t poff[VPL];
#pragma unroll
    for (int p = 0; p < VPL; ++p) poff[p] = have[p] ? (int64_t)p * kWave * VN : 0;
    // One vector instruction per element: a maximum of three that ignores NaN takes two rows
    // at a time, and one unordered test per pair of rows remembers, per column, whether a NaN
    // went by; the flag is folded into the value once, after the sweep (NaN wins).
    bool un[CN];
#pragma unroll
    for (int e = 0; e < CN; ++e) un[e] = false;
    auto fold2 = [&](const V &b0, const V &b1, int p) {
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            const C c0 = E::up(b0.e[e]), c1 = E::up(b1.e[e]);
            best[p * VN + e] = max3_ignoring_nan(best[p * VN + e], c0, c1);
            un[p * VN + e] |= __builtin_isunordered(c0, c1);
        }
    };
    auto fold = [&](const V &b, int p) { fold2(b, b, p); };
    auto settle = [&]() {  // a column that has seen a NaN is NaN
#pragma unroll
        for (int e = 0; e < CN; ++e) {
            best[e] = un[e] ? (C)__builtin_nanf("") : best[e];
            un[e] = false;
        }
    };
    static_assert(ROWS % 2 == 0, "rows are folded in pairs");
    int64_t r = r0 + wave;
    auto sweep = [&](auto once_tag) {
        for (; r + (ROWS - 1) * kMatWaves < r1; r += ROWS * kMatWaves) {
            V b[ROWS][VPL];
#pragma unroll
            for (int u = 0; u < ROWS; ++u)
#pragma unroll
                for (int p = 0; p < VPL; ++p)
                    b[u][p] = load_piece<decltype(once_tag)::value>(
                        reinterpret_cast<const V *>(xc + (r + u * kMatWaves) * ld + poff[p]));
            __builtin_amdgcn_sched_barrier(0);  // all loads of the step are under way before the first is looked at
#pragma unroll
            for (int u = 0; u < ROWS; u += 2)
#pragma unroll
                for (int p = 0; p < VPL; ++p) fold2(b[u][p], b[u + 1][p], p);
        }
    };
    if (once) sweep(OnceT{});
    else sweep(AgainT{});
    for (; r < r1; r += kMatWaves) {
#pragma unroll
        for (int p = 0; p < VPL; ++p) fold(*reinterpret_cast<const V *>(xc + r * ld + poff[p]), p);
    }
    __shared__ C sm[kMatWaves][kWave * CN];
    __shared__ bool last_block;
    auto across_waves = [&]() {  // wave 0 ends up with the maxima of the workgroup
        settle();
#pragma unroll
        for (int e = 0; e < CN; ++e) sm[wave][e * kWave + lane] = best[e];
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int e = 0; e < CN; ++e)
                for (int w = 1; w < kMatWaves; ++w) best[e] = vmax_nan(best[e], sm[w][e * kWave + lane]);
        }
    };
    across_waves();
    // a partial row: VPL x 16 bytes per lane of wave 0, as 8-byte words (piece p, half q: word 2p + q)
    constexpr int WORDS = 2 * VPL;
    const int64_t words_per_row = (int64_t)colblocks * kWave * WORDS;
    union Piece {
        V v;
        unsigned long long w[2];
    };
    // (partials travel as 16-byte buffer accesses with the device-scope bit: the last workgroup's
    // trips to memory cost by the instruction, and this halves their number)
    const __amdgpu_buffer_rsrc_t prsrc = make_rsrc(part, (uint32_t)(words_per_row * splits * 8));
    const uint32_t plane = (uint32_t)(((int64_t)cb * kWave + lane) * WORDS * 8);
    if (wave == 0) {
#pragma unroll
        for (int p = 0; p < VPL; ++p) {
            Piece u;
#pragma unroll
            for (int e = 0; e < VN; ++e) u.v.e[e] = E::down(best[p * VN + e]);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, u), prsrc, plane + 16u * p,
                                                   (uint32_t)(split * words_per_row * 8), kDeviceScope);
        }
        const Ticket drawn = take_ticket_wave(ticket + cb * kTicketStride);
        if (lane == 0) last_block = ticket_last(drawn, splits);
        // counters that no launch of this library left behind: NaN in this block's part of y
        const bool broken = __builtin_amdgcn_readfirstlane((int)!ticket_sound(drawn, splits)) != 0;
        if (broken) {
#pragma unroll
            for (int p = 0; p < VPL; ++p) {
                if (!have[p]) continue;
                V out;
#pragma unroll
                for (int e = 0; e < VN; ++e) out.e[e] = E::down((C)__builtin_nanf(""));
                *reinterpret_cast<V *>(y + col + (int64_t)p * kWave * VN) = out;
            }
        }
    }
    __syncthreads();
    if (!last_block) return;
    // the last workgroup of the column block: wavefront w takes splits w, w + 4, ...; all loads
    // of a batch are asked for before the first is looked at
    constexpr int kBatch = kColFusedSplits / kMatWaves;  // all splits in one batch: one round trip (a trip costs over 1 us here)
#pragma unroll
    for (int e = 0; e < CN; ++e) best[e] = neg_inf<C>();
    // (a split past the last one is replaced by split 0: folding a row twice changes nothing,
    // and the loads carry no predicates)
#pragma unroll
    for (int s0 = 0; s0 < kColFusedSplits; s0 += kBatch * kMatWaves) {
        if (s0 >= splits) break;  // wave-uniform
        uintx4 w[kBatch][VPL];
#pragma unroll
        for (int q = 0; q < kBatch; ++q) {
            const int sp = s0 + wave + q * kMatWaves;
            const uint32_t soff = (uint32_t)((sp < splits ? sp : 0) * words_per_row * 8);  // wave-uniform
#pragma unroll
            for (int p = 0; p < VPL; ++p)
                w[q][p] = __builtin_amdgcn_raw_buffer_load_b128(prsrc, plane + 16u * p, soff, kDeviceScope);
        }
#pragma unroll
        for (int q = 0; q < kBatch; q += 2)
#pragma unroll
            for (int p = 0; p < VPL; ++p)
                fold2(__builtin_bit_cast(Piece, w[q][p]).v, __builtin_bit_cast(Piece, w[q + 1][p]).v, p);
    }
    __syncthreads();  // sm is reused
    across_waves();
    if (wave == 0) {
#pragma unroll
        for (int p = 0; p < VPL; ++p) {
            if (!have[p]) continue;
            V out;
#pragma unroll
            for (int e = 0; e < VN; ++e) out.e[e] = E::down(best[p * VN + e]);
            *reinterpret_cast<V *>(y + col + (int64_t)p * kWave * VN) = out;
        }
        if (lane == 0) ticket_idle(ticket + cb * kTicketStride);
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

// One-launch column maxima (colmax_fused_kernel): two workgroups per compute unit when the
// matrix allows, every split at least 32 rows, at most kColFusedSplits splits and one arrival
// counter per column block.  splits < 2: not applicable.
struct FusedPlan {
    int vpl;        // 16-byte pieces per lane (0: the one-launch path does not apply)
    int colblocks;  // workgroups across a row
    int splits;     // workgroups down a column
    int64_t chunk;  // rows per split
};
static FusedPlan colmax_fused_plan(int64_t m, int64_t n, int vn) {
    FusedPlan none{0, 0, 1, m};
    if (n % vn != 0) return none;  // whole 16-byte pieces only (y is written in pieces)
    // Two pieces per lane for matrices of 256 MiB and more, where that still leaves a workgroup
    // of at least 128 rows per CU: the sweep is 5 % faster (16384^2 fp32: 175 against 182 us),
    // but the last workgroup of a column block then has twice the partial words to fetch, and
    // those device-scope loads are slow (4096^2 fp32: 3.6 us against 1.3 us, 16.7 us in all
    // against 14.6 us).
    const bool large = m * n * (16 / vn) >= ((int64_t)1 << 28);
    for (int vpl = large ? 2 : 1; vpl >= 1; --vpl) {
        const int64_t colblocks = ceil_div(n, (int64_t)kWave * vn * vpl);
        if (colblocks > kMaxTickets) continue;
        int64_t splits = ceil_div((int64_t)(vpl == 2 ? 256 : 512), colblocks);
        if (splits > kColFusedSplits) splits = kColFusedSplits;
        if (splits > m / 32) splits = m / 32;
        if (splits < 2) continue;
        const int64_t rchunk = ceil_div(m, splits);
        if (vpl == 2 && (rchunk < 128 || colblocks * splits < 192)) continue;
        return {vpl, (int)colblocks, (int)ceil_div(m, rchunk), rchunk};
    }
    return none;
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
                          typename Elem<DT>::T *y, int64_t ldy, hipStream_t stream, int once = 0) {
    const int64_t blocks = p.splits * ceil_div(m, (int64_t)kMatWaves);
    if (vec_ok<DT>(x, ld))
        hipLaunchKernelGGL((rowmax_kernel<DT, true>), dim3((unsigned)blocks), dim3(kMatThreads), 0, stream,
                           x, ld, m, n, p.chunk, p.splits, once, y, ldy);
    else
        hipLaunchKernelGGL((rowmax_kernel<DT, false>), dim3((unsigned)blocks), dim3(kMatThreads), 0, stream,
                           x, ld, m, n, p.chunk, p.splits, once, y, ldy);
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

// workspace: [tickets][partials]
template <int DT>
static size_t matmax_ws(int64_t m, int64_t n, int axis) {
    using T = typename Elem<DT>::T;
    constexpr int VN = 16 / (int)sizeof(T);
    if (axis == 1) {
        MatPlan p = rowmax_plan(m, n, VN);
        return p.splits > 1 ? kTicketBytes + (size_t)(m * p.splits) * sizeof(T) : 0;
    }
    // worst case over the vector / scalar column paths, plus the intermediate level
    MatPlan pv = colmax_plan(m, n, VN), ps = colmax_plan(m, n, 1);
    const FusedPlan pf = colmax_fused_plan(m, n, VN);
    const size_t fused = pf.vpl ? (size_t)pf.splits * pf.colblocks * kWave * 16 * pf.vpl : 0;
    int64_t s = pv.splits > ps.splits ? pv.splits : ps.splits;
    size_t tree = 0;
    if (s > 1) {
        const int64_t s2 = combine_splits(s);
        tree = (size_t)((s + (s2 > 1 ? s2 : 0)) * n) * sizeof(T);
    }
    const size_t most = fused > tree ? fused : tree;
    return most ? kTicketBytes + most : 0;
}

template <int DT>
static int matmax_launch(const void *xv, void *yv, int64_t m, int64_t n, int axis, void *ws,
                         size_t ws_bytes, hipStream_t stream) {
    using T = typename Elem<DT>::T;
    constexpr int VN = 16 / (int)sizeof(T);
    const T *x = static_cast<const T *>(xv);
    T *y = static_cast<T *>(yv);
    T *part = reinterpret_cast<T *>(static_cast<char *>(ws) + kTicketBytes);
    if (matmax_ws<DT>(m, n, axis) > ws_bytes) return TRT_E_WORKSPACE;
    if (matmax_ws<DT>(m, n, axis) > 0 && ws == nullptr) return TRT_E_WORKSPACE;
    const int once = m * n * (int64_t)sizeof(T) >= kStreamBytes;  // too large to be found in L2 again
    if (axis == 1 && rowmax_wide<DT>(x, m, n)) {
        hipLaunchKernelGGL((rowmax_wide_kernel<DT>), dim3((unsigned)m), dim3(kMatThreads), 0, stream, x, n, n, once,
                           y);
    } else if (axis == 1) {
        MatPlan p = rowmax_plan(m, n, VN);
        if (p.splits == 1) {
            rowmax_launch<DT>(x, n, m, n, p, y, 1, stream, once);
        } else {
            rowmax_launch<DT>(x, n, m, n, p, part, p.splits, stream, once);
            MatPlan p2{1, p.splits};
            rowmax_launch<DT>(part, p.splits, m, p.splits, p2, y, 1, stream);
        }
    } else {
        const bool vec = vec_ok<DT>(x, n);
        MatPlan p = colmax_plan(m, n, vec ? VN : 1);
        const FusedPlan pf = colmax_fused_plan(m, n, VN);
        const bool fused = vec && (reinterpret_cast<uintptr_t>(y) & 15) == 0;  // y is written in 16-byte pieces
        if (fused && pf.vpl == 2) {
            hipLaunchKernelGGL((colmax_fused_kernel<DT, 2>), dim3((unsigned)(pf.colblocks * pf.splits)),
                               dim3(kMatThreads), 0, stream, x, n, m, n, pf.chunk, pf.colblocks, pf.splits, once,
                               reinterpret_cast<unsigned long long *>(part), static_cast<Ticket *>(ws), y);
        } else if (fused && pf.vpl == 1) {
            hipLaunchKernelGGL((colmax_fused_kernel<DT, 1>), dim3((unsigned)(pf.colblocks * pf.splits)),
                               dim3(kMatThreads), 0, stream, x, n, m, n, pf.chunk, pf.colblocks, pf.splits, once,
                               reinterpret_cast<unsigned long long *>(part), static_cast<Ticket *>(ws), y);
        } else if (p.splits == 1) {
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
    // counters are 8-byte atomics, partial results 16-byte accesses
    if (need && (reinterpret_cast<uintptr_t>(workspace) & 15)) return TRT_E_LAYOUT;
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
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 15)) return TRT_E_LAYOUT;
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

// Arrival counters of a max workspace set idle, by a kernel (a caller that prepares its
// workspaces while a stream is being captured into a graph needs no memset node).
__global__ __launch_bounds__(256) void idle_tickets_kernel(trt::Ticket *ticket) {
    for (unsigned i = threadIdx.x; i < trt::kTicketBytes / sizeof(trt::Ticket); i += 256) ticket[i] = trt::kTicketTag;
}

extern "C" int trt_max_workspace_init(void *workspace, size_t workspace_bytes, void *stream) {
    if (!workspace || workspace_bytes < trt::kTicketBytes) return TRT_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 15) return TRT_E_LAYOUT;
    hipLaunchKernelGGL(idle_tickets_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<trt::Ticket *>(workspace));
    return (int)hipGetLastError();
}

// Debugging aid: waits for `stream`, copies the counters to the host and looks at them.
extern "C" int trt_max_workspace_check(const void *workspace, size_t workspace_bytes, void *stream) {
    if (!workspace || workspace_bytes < trt::kTicketBytes) return TRT_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 15) return TRT_E_LAYOUT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t err = hipStreamSynchronize(s);
    if (err != hipSuccess) return (int)err;
    static thread_local trt::Ticket host[trt::kTicketBytes / sizeof(trt::Ticket)];
    err = hipMemcpy(host, workspace, trt::kTicketBytes, hipMemcpyDeviceToHost);
    if (err != hipSuccess) return (int)err;
    for (size_t i = 0; i < trt::kTicketBytes / sizeof(trt::Ticket); ++i)
        if (host[i] != trt::kTicketTag) return TRT_E_STATE;
    return TRT_OK;
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
