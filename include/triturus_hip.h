/*
 * triturus_hip.h -- C ABI of the gfx950 (MI355X) log-space contraction library.
 *
 * Every entry point takes raw DEVICE pointers, sizes, element strides and a
 * hipStream_t (as void*).  The library allocates nothing, keeps no state,
 * never synchronises (trt_max_workspace_check, a debugging aid, excepted) and never throws: each call enqueues its kernels on the
 * given stream and returns an int status
 *      0            success
 *      < 0          argument / layout error (TRT_E_*), nothing was enqueued
 *      > 0          a hipError_t reported by the launch
 * Outputs and workspaces are owned by the caller.
 *
 * The reference (loreloc/triturus) has no FFI: its boundary for this path is
 * the Triton kernel launch made by each Python wrapper.  Each function below
 * names the reference launch site it replaces (path:line in the reference).
 *
 * Letters: R = batch; lm2exp contracts J; lt2exp contracts (I, J); K is the
 * trailing, contiguous "column" axis of every log-space operand.
 */
#ifndef TRITURUS_HIP_H
#define TRITURUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRT_ABI_VERSION 9

#define TRT_OK 0
#define TRT_E_INVALID (-1)   /* null pointer, non-positive size, bad enum   */
#define TRT_E_LAYOUT (-2)    /* stride pattern the kernels do not handle    */
#define TRT_E_WORKSPACE (-3) /* workspace missing or smaller than required  */
#define TRT_E_RANGE (-4)     /* a size exceeds what the index math supports */
#define TRT_E_SCRATCH (-5)   /* the call needs more than the library's static scratch holds */
#define TRT_E_STATE (-6)     /* trt_max_workspace_check: arrival counters not idle           */

/* Element types of the max reductions (triturus/max.py:37,98,178 accept any
 * floating dtype). */
#define TRT_F32 0
#define TRT_F64 1
#define TRT_F16 2
#define TRT_BF16 3

/* lt2exp launch modes (triturus/lt2exp.py:534-541). */
#define TRT_MODE_AUTO 0
#define TRT_MODE_SPLIT 1
#define TRT_MODE_UNSPLIT 2

/* ABI version of the loaded library (== TRT_ABI_VERSION it was built with). */
int trt_version(void);

/* Static, human-readable text for a status returned by any call below. */
const char *trt_error_string(int status);

/*
 * c[r,i,k] = log sum_j a[r,i,j] * exp(b[r,j,k])            (fp32)
 * a: R x I x J linear-space, b: R x J x K log-space, c: R x I x K.
 * sa/sb/sc: element strides of the three axes, all non-negative (zero: an
 * expanded operand).  a and b may have any strides, as the reference forwards them to its
 * kernel (triturus/lm2exp.py:190-198): a transposed or column-strided operand is read in
 * place (a lane owns a column of b, so its trailing stride only scales the lane's offsets;
 * fastest with a unit trailing stride, where a half-wave reads 128-byte row segments).  The
 * trailing stride of c must be 1 (TRT_E_LAYOUT otherwise); its two leading strides are
 * free.  Replaces the `_ker_lm2exp[grid](...)` launch,
 * triturus/lm2exp.py:186-205; arithmetic contract baselines/lm2exp.py:11-14 (column
 * max clamped to +-1e38, an all -inf column gives -inf, never NaN).
 * variant: 0 = choose by shape; 1..trt_lm2exp_variant_count() force a tile shape and
 * kernel (experiments, tests); a forced variant that is not one of the paired-wavefront
 * tiles (the last five) needs sa[2] == 1.
 * splits: the contraction over J may be cut over several workgroups whose partial
 * sums are merged by a second kernel in a fixed order (deterministic): 0 = decide
 * by shape (small grids with a long contraction), 1 = never, n = n ways.  The
 * reference has no such mode for lm2exp.  When it splits, the call needs a
 * workspace of trt_lm2exp_workspace_bytes(R, I, J, K, variant, splits) bytes
 * (0 when it does not split: pass NULL, 0).  With variant 0, splits <= 1, at most 4 columns,
 * J >= 1024 a multiple of 4 and 16-byte aligned rows of a, a is streamed once on the vector ALU
 * (the few-column kernel of trt_lt2exp_f32) and no workspace is used.  With variant 0,
 * splits <= 1, more than 8 columns and J <= 16 over many batches, every output column gets a lane
 * of its own (the few-unit kernel of trt_lt2exp_f32) where that is the faster way; likewise no
 * workspace.  With at most 64 columns under few rows per batch and J >= 32 (above 16 rows or 32
 * columns: J a multiple of 4 and 16-byte aligned rows of a), a workgroup takes a batch's one
 * tile and cuts its contraction over its wavefronts (likewise).  trt_lm2exp_kernel_name tells which kernel a call takes.
 */
int trt_lm2exp_f32(const float *a, const float *b, float *c,
                   int64_t R, int64_t I, int64_t J, int64_t K,
                   const int64_t sa[3], const int64_t sb[3], const int64_t sc[3],
                   int variant, int splits, void *workspace, size_t workspace_bytes,
                   void *stream);
size_t trt_lm2exp_workspace_bytes(int64_t R, int64_t I, int64_t J, int64_t K,
                                  int variant, int splits);
int trt_lm2exp_variant_count(void);

/*
 * c[r,s,k] = log sum_{i,j} w[r,s,i,j] * exp(a[r,i,k]) * exp(b[r,j,k])   (fp32)
 * w: R x S x (I*J) linear-space (the reference flattens the two trailing axes
 * with w.view(batch, m, -1), triturus/lt2exp.py:549, so sw has 3 entries),
 * a: R x I x K, b: R x J x K log-space, c: R x S x K.  The trailing stride of c
 * must be 1; w, a and b take any non-negative strides, as the reference's kernels do
 * (triturus/lt2exp.py:577-585, :606-620): a flat axis of w with another stride than 1
 * -- a sliced view -- is read in place, element by element, and so are transposed or
 * column-strided a and b (a lane owns a column: the stride scales its offsets).  Replaces the `_ker_lt2exp_unsplit[grid](...)` launch,
 * triturus/lt2exp.py:601-629, and the `_ker_lt2exp_split[grid](...)` launch,
 * triturus/lt2exp.py:564-597; arithmetic contract baselines/lt2exp.py:15-25.
 * mode: TRT_MODE_*.  AUTO decides like the reference does -- by the size of the
 * output grid and the length of the contraction (triturus/lt2exp.py:535 uses
 * R*S*K < 1048576 and I*J > 512) -- with thresholds measured on MI355X: it
 * splits when the unsplit grid would leave many compute units idle and the
 * contraction is long enough to pay for the merge.  SPLIT partitions
 * the contracted (i,j) range over several workgroups and merges the partial
 * sums deterministically; it needs a workspace of
 * trt_lt2exp_workspace_bytes(...) bytes (UNSPLIT needs none: pass NULL, 0).
 * variant: 0 = choose by shape; 1..trt_lt2exp_variant_count() force a tile shape
 * and j-chunk (tests, tuning).  With J = 1 and variant 0 the call runs with the
 * roles of (i, a) and (j, b) exchanged; with J = 2, 4 or 8, I*J a multiple of 4
 * and 16-byte aligned rows of w (base, sw[0], sw[1]) the kernel walks (i, j) as
 * one flat axis, so short rows cost no padding.  With at most 8 columns (K <= 8), a dense flat
 * axis of w (sw[2] == 1) and rows of at least 128 weights (256 for K > 4; 256 / 1024 unless J is a
 * multiple of 4 and the rows are 16-byte aligned, and then J > 4), variant 0 streams w once on
 * the vector ALU instead (no cut, no workspace used, whatever the mode).  With few s per
 * batch (about a dozen at most), or little work altogether, and a dense flat axis of w
 * (16 bytes at a time where J is a multiple of 4 and the rows are 16-byte aligned, float by
 * float otherwise), variant 0 contracts j first, with the rows (s, i) of w on the rows of the
 * matrix instruction (likewise no cut and no workspace).  With I and J of at most 16 over many
 * batches (and more than 8 columns), variant 0 gives every output column a lane of its own and
 * contracts on the vector ALU where that is the faster way (likewise).  trt_lt2exp_kernel_name
 * tells which kernel a call takes.
 */
int trt_lt2exp_f32(const float *w, const float *a, const float *b, float *c,
                   int64_t R, int64_t S, int64_t I, int64_t J, int64_t K,
                   const int64_t sw[3], const int64_t sa[3], const int64_t sb[3],
                   const int64_t sc[3], int mode, int variant,
                   void *workspace, size_t workspace_bytes, void *stream);
size_t trt_lt2exp_workspace_bytes(int64_t R, int64_t S, int64_t I, int64_t J,
                                  int64_t K, int mode);
int trt_lt2exp_variant_count(void);

#define TRT_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
/*
 * trt_lt2exp_f32 without a workspace argument, for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  No counterpart in the reference (whose wrapper allocates its lock and output
 * with torch, triturus/lt2exp.py:544-562).  The split-mode workspace (partial sums and
 * shifts) lives in a device array inside the library of TRT_STATIC_SCRATCH_BYTES bytes
 * (16 MiB; every GPU the library runs on holds its copy until the process ends).  The call
 * allocates and frees nothing.  A shape whose split mode may need more than that
 * (trt_lt2exp_workspace_bytes(R, S, I, J, K, mode) > TRT_STATIC_SCRATCH_BYTES) is refused
 * with TRT_E_SCRATCH and nothing is enqueued; TRT_MODE_UNSPLIT needs no scratch at all.  The
 * first call on a device looks up the address of that device's copy of the array (make it
 * outside graph capture).  All calls on one GPU share the array: calls that overlap in time
 * (two streams, two threads) race; calls enqueued on one stream do not.  Nothing in the array
 * has to be cleared between calls.  Results are bit-identical to trt_lt2exp_f32.
 */
int trt_lt2exp_f32_static(const float *w, const float *a, const float *b, float *c,
                          int64_t R, int64_t S, int64_t I, int64_t J, int64_t K,
                          const int64_t sw[3], const int64_t sa[3], const int64_t sb[3],
                          const int64_t sc[3], int mode, int variant, void *stream);

/*
 * The same contraction as trt_lt2exp_f32 (fp32 tensors in and out, same layouts and status
 * codes and strides) on the bf16 matrix pipe: every fp32 operand is cut into `pieces` bf16
 * pieces and a product is the sum of the piece products that matter, accumulated in fp32.
 *   pieces = 2 (TRT_PIECES_BF16X3): 3 MFMAs per product, relative error ~2^-16 per product
 *   pieces = 3 (TRT_PIECES_BF16X6): 6 MFMAs per product, relative error ~2^-23 per product
 * This is the library's counterpart of the reference's reduced-precision mode
 * (ALLOW_TF32 passed to tl.dot, triturus/lt2exp.py:344, flag triturus/utils.py:33-44):
 * gfx950 has no TF32 matrix instruction; two bf16 pieces are more accurate than TF32
 * (2^-11) and several times faster than the fp32 matrix pipe.  The call takes the same mode
 * and workspace (trt_lt2exp_workspace_bytes) as trt_lt2exp_f32: with variant 0 a grid too
 * small to be matrix bound has its contraction cut over workgroups (as the mode and the
 * workspace allow) or is handed to trt_lt2exp_f32, and so are rows of w of 2 or 4 values
 * (8 with three pieces) that the fp32 kernel packs.  variant: 0 = choose by shape, 1..4 and
 * 9..12 force a bf16 tile shape, 5..8 and 13..16 the same tiles with the contraction cut
 * (experiments, tests).
 */
#define TRT_PIECES_BF16X3 2
#define TRT_PIECES_BF16X6 3
int trt_lt2exp_bf16(const float *w, const float *a, const float *b, float *c,
                    int64_t R, int64_t S, int64_t I, int64_t J, int64_t K,
                    const int64_t sw[3], const int64_t sa[3], const int64_t sb[3],
                    const int64_t sc[3], int pieces, int mode, int variant,
                    void *workspace, size_t workspace_bytes, void *stream);
/* Workspace for trt_lt2exp_bf16: the larger of this and trt_lt2exp_workspace_bytes. */
size_t trt_lt2exp_bf16_workspace_bytes(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K,
                                       int pieces, int mode);

/*
 * trt_lm2exp_f32 on the bf16 matrix pipe, in the same way (ALLOW_TF32 at
 * triturus/lm2exp.py:152 is the reference's counterpart): same tensors, layouts, strides and
 * status codes; pieces as above.  splits as for trt_lm2exp_f32: 0 = decide by shape, 1 = never,
 * > 1 = cut the contraction that many times (capped by its length).  With variant 0, a grid too
 * small to be matrix bound has its contraction cut over workgroups (as the workspace allows) or
 * is handed to trt_lm2exp_f32, so the workspace is the larger of
 * trt_lm2exp_bf16_workspace_bytes(R, I, J, K, pieces, splits) and
 * trt_lm2exp_workspace_bytes(R, I, J, K, 0, splits).
 * variant: 0 = choose by shape, 1..trt_lm2exp_bf16_variant_count() force a bf16 tile shape
 * (cut only when splits > 1).
 */
int trt_lm2exp_bf16(const float *a, const float *b, float *c,
                    int64_t R, int64_t I, int64_t J, int64_t K,
                    const int64_t sa[3], const int64_t sb[3], const int64_t sc[3],
                    int pieces, int variant, int splits,
                    void *workspace, size_t workspace_bytes, void *stream);
/* Workspace for trt_lm2exp_bf16's own cut over J: the larger of this and
 * trt_lm2exp_workspace_bytes(R, I, J, K, 0, splits) serves every path the call may take. */
size_t trt_lm2exp_bf16_workspace_bytes(int64_t R, int64_t I, int64_t J, int64_t K,
                                       int pieces, int splits);
int trt_lm2exp_bf16_variant_count(void);

/*
 * Workspaces of the max reductions (trt_matmax, trt_vmax) start with arrival counters: the
 * workgroup that finishes last combines the partial results of all of them, so a reduction is
 * one launch.  The first TRT_MAX_TICKET_BYTES of such a workspace must be prepared with
 * trt_max_workspace_init before the first call that uses it (a hipMemset to zero does NOT do:
 * an idle counter carries a tag); every call leaves the counters idle, so a workspace is
 * prepared once and reused from call to call -- by one stream at a time: calls that overlap in
 * time need workspaces of their own.  Workspaces must be 16-byte aligned (TRT_E_LAYOUT).
 * What a broken contract looks like: a reduction that finds a counter without the tag (a
 * workspace never prepared, or written over) or with more arrivals than its launch makes
 * elects no combining workgroup and writes NaN -- with index -1 from trt_vmax -- where the
 * result belongs (the launch itself cannot report a status: it is asynchronous); the counters
 * stay as they are until trt_max_workspace_init runs again.  Two calls that use one workspace
 * at the same time are detected only when their counts happen to overshoot.
 */
#define TRT_MAX_TICKET_BYTES 65536
/* Sets the arrival counters of a max workspace idle with a small kernel on `stream` (no memset
 * node: safe to record into a HIP graph).  No counterpart in the reference, whose reductions
 * launch once per level.  workspace_bytes < TRT_MAX_TICKET_BYTES: TRT_E_WORKSPACE. */
int trt_max_workspace_init(void *workspace, size_t workspace_bytes, void *stream);
/* Debugging aid, no counterpart in the reference: waits for `stream` (this one call of the
 * library synchronises), reads the counters back and returns TRT_E_STATE unless all of them
 * are idle -- which they are between any two reductions of a sound program. */
int trt_max_workspace_check(const void *workspace, size_t workspace_bytes, void *stream);

/* *capture_id = the identity of the HIP graph capture `stream` is in, 0 when it is in none.  Host
 * only; no counterpart in the reference.  A caller that keeps one max workspace per stream
 * needs it to give every capture a workspace (and a trt_max_workspace_init node) of its own:
 * a workspace prepared while capturing is idle only when the graph runs. */
int trt_stream_capture_id(void *stream, unsigned long long *capture_id);

/*
 * Max of a contiguous m x n row-major matrix along axis 0 (y has n entries)
 * or axis 1 (y has m entries).  NaN propagates as in torch.amax.  Replaces the
 * multi-launch `_ker_matmax` tree, triturus/max.py:190-225.  workspace:
 * trt_matmax_workspace_bytes(m, n, axis, dtype) bytes (may be 0).
 */
int trt_matmax(const void *x, void *y, int64_t m, int64_t n, int axis, int dtype,
               void *workspace, size_t workspace_bytes, void *stream);
size_t trt_matmax_workspace_bytes(int64_t m, int64_t n, int axis, int dtype);

/*
 * Batched column maxima m[r,k] = max_j b[r,j,k] of an R x J x K fp32 tensor
 * (element strides sb, trailing stride 1); m is R x K, contiguous.  A NaN in a
 * column gives NaN, like torch.amax(b, dim=1).  With clamp != 0 the maxima are
 * clamped to +-1e38: exactly the shift that the contraction recipes subtract
 * (baselines/lm2exp.py:11-12, baselines/lt2exp.py:15-19).  The reference has the 2-D reduction only
 * (`matmax`, triturus/max.py:125-188); this is its batched form along axis 1.
 * workspace: trt_colmax_batched_workspace_bytes(R, J, K) bytes (0 unless few
 * columns stand under a long reduced axis, which is then cut over J).
 */
int trt_colmax_batched_f32(const float *b, float *m, int64_t R, int64_t J, int64_t K,
                           const int64_t sb[3], int clamp, void *workspace, size_t workspace_bytes,
                           void *stream);
size_t trt_colmax_batched_workspace_bytes(int64_t R, int64_t J, int64_t K);

/*
 * Max and first-occurrence argmax (int64) of a contiguous vector of n
 * elements; a NaN wins and reports the first NaN, as torch.max(x, 0) does.
 * out_idx may be NULL (value only: the reference's vamax).  Replaces the
 * `_ker_vmax` / `_ker_vamax` launch loops, triturus/max.py:108-121 and
 * :46-58.  workspace: trt_vmax_workspace_bytes(n, dtype) bytes.
 */
int trt_vmax(const void *x, int64_t n, int dtype, void *out_val, int64_t *out_idx,
             void *workspace, size_t workspace_bytes, void *stream);
size_t trt_vmax_workspace_bytes(int64_t n, int dtype);

/*
 * c = a b for contiguous row-major fp32 matrices, a: m x k, b: k x n, c: m x n, in IEEE fp32
 * on the fp32 matrix pipe (the lm2exp contraction kernel without shift, exp and log).
 * Replaces the `_ker_mm[grid](...)` launch, triturus/mm.py:199-213.  Not on the log-space
 * path: provided so that the reference's module surface is complete.
 * variant: 0 = row tile by rule, 1..4 = tiles of 32..128 rows.  splits: 0 = the library
 * decides whether to cut the product over k (grids of few tiles), 1 = never, n > 1 = n ways
 * (capped at 32 and at 32 values of k per piece); the partial products are summed in split
 * order by a second launch, so the result is deterministic.  workspace:
 * trt_mm_workspace_bytes(m, k, n, variant, splits) bytes, 16-byte aligned; without it a cut
 * the library chose itself is dropped and an explicit one fails with TRT_E_WORKSPACE.
 */
int trt_mm_f32(const float *a, const float *b, float *c, int64_t m, int64_t k, int64_t n,
               int variant, int splits, void *workspace, size_t workspace_bytes, void *stream);
size_t trt_mm_workspace_bytes(int64_t m, int64_t k, int64_t n, int variant, int splits);

/*
 * trt_mm_f32 on the bf16 matrix pipe with split operands (pieces as for trt_lt2exp_bf16;
 * counterpart of ALLOW_TF32 at triturus/mm.py:212).  Grids too small for the bf16 kernels
 * are handed to trt_mm_f32 with the workspace (trt_mm_workspace_bytes(m, k, n, 0, 0) bytes).
 */
int trt_mm_bf16(const float *a, const float *b, float *c, int64_t m, int64_t k, int64_t n,
                int pieces, void *workspace, size_t workspace_bytes, void *stream);

/*
 * r = x + y for contiguous vectors of n elements of `dtype` (TRT_F32 ...).  Replaces the
 * `_ker_vadd[grid](...)` launch, triturus/add.py:45.  Same remark as trt_mm_f32.
 */
int trt_vadd(const void *x, const void *y, void *r, int64_t n, int dtype, void *stream);

/*
 * Name of the contraction kernel that a trt_lt2exp_f32 / trt_lm2exp_f32 call with these sizes
 * and choices launches, written to buf as a profiler prints it (e.g.
 * "trt::lt2exp_kernel<2, 1, 4, 4, true, false, 1, 0>").  Host only.  w_aligned / a_vec: the
 * operand's base and leading strides are multiples of 16 bytes (and a has a unit trailing
 * stride).  No counterpart in the reference: benchmarks use it to find their kernel in
 * profiler output.
 */
int trt_lt2exp_kernel_name(int64_t R, int64_t S, int64_t I, int64_t J, int64_t K, int mode,
                           int variant, int w_aligned, char *buf, size_t buf_bytes);
int trt_lm2exp_kernel_name(int64_t R, int64_t I, int64_t J, int64_t K, int variant, int splits,
                           int a_vec, char *buf, size_t buf_bytes);

/*
 * Plain device-to-device copy kernel of nbytes (multiple of 16, 16-byte
 * aligned pointers).  No counterpart in the reference: it is the known-size
 * kernel that hardware byte counters are calibrated against.
 */
int trt_copy_bytes(const void *src, void *dst, size_t nbytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TRITURUS_HIP_H */
