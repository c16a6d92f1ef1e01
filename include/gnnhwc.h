/*
 * gnnhwc.h -- C ABI of libgnnhwc_hip.so: channels-last (NHWC) GroupNorm forward / backward
 * with a fused activation, for AMD gfx950 (MI355X).
 *
 * This is the drop-in boundary for the reference's raw kernel interface
 *   run_gn_fwd_kernels<T> / run_gn_bwd_kernels<T>   (src/gnnhwc/csrc/gn_kernel.h:11-41)
 * which its op glue calls from gn_nhwc_fwd / gn_nhwc_bwd (src/gnnhwc/csrc/custom_gn.cpp:10-89).
 * The template parameter T becomes a runtime dtype code, `int` sizes become int64_t, the implicit
 * "current CUDA stream" becomes an explicit hipStream_t, and the scratch memory the reference takes
 * from the caching allocator inside the host driver (gn_kernel.cu:461,954-1001) becomes a
 * caller-provided workspace whose size is queried up front.  No torch types appear here.
 *
 * Tensor layout (identical to the reference's permuted views, custom_gn.cpp:24,64-65):
 *   x, y, dy, dx : (N, R, C) contiguous, C fastest; R = product of all spatial dims.
 *   weight, bias, dweight, dbias : (C) in `param_dtype`; weight/bias may be NULL (gamma=1, beta=0).
 *   mean, rstd   : (N, G) in `stats_dtype`.
 * All pointers are device pointers on the device that is current for the calling thread.
 * Calls are asynchronous on `stream` and never synchronise.  gnnhwc_fwd / gnnhwc_bwd allocate no device memory: the
 * caller brings the workspace.  Concurrent calls on different streams are safe as long as each call has its own
 * workspace.
 *
 * State the library keeps (none of it affects results): a per-thread error string; and, for the single-launch
 * kernels (see gnnhwc_set_resident), process-wide: the on / off switch, per device the stream of the last
 * single-launch call and one event that orders a call on another stream behind it, a 64-byte host-pinned status
 * word (allocated with hipHostMalloc at the first single-launch call of the process; see gnnhwc_resident_status), one 8-byte generation cell per
 * device inside the library's image (used by launches recorded into HIP graphs), a pool of events while
 * gnnhwc_profile_enable is on, and a device buffer of 64 KiB when GNNHWC_TRACE is set in the environment.
 * A caller that must see no allocation at all after start-up either makes one warm-up call per device first or
 * switches the single-launch kernels off.
 *
 * Every entry point returns GNNHWC_OK (0) or a negative error code; gnnhwc_last_error() describes the
 * most recent failure on the calling thread.  Nothing is launched when an error is returned.
 */
#ifndef GNNHWC_H
#define GNNHWC_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes -- the four types of AT_DISPATCH_FLOATING_TYPES_AND2(Half, BFloat16, ...)
 * (custom_gn.cpp:29-33, 73-77). */
enum {
  GNNHWC_F32 = 0,
  GNNHWC_F64 = 1,
  GNNHWC_F16 = 2,
  GNNHWC_BF16 = 3
};

/* activation codes -- same integers as GN_NHWC.act_code (custom_gn.py:52-59) and the
 * act_fn_option switch of the reference host drivers (gn_kernel.cu:419-436, 911-929). */
enum {
  GNNHWC_ACT_IDENTITY = 0,
  GNNHWC_ACT_RELU = 1,
  GNNHWC_ACT_SILU = 2,
  GNNHWC_ACT_GELU = 3,
  GNNHWC_ACT_GELU_TANH = 4
};

enum {
  GNNHWC_OK = 0,
  GNNHWC_ERR_INVALID_ARGUMENT = -1, /* bad shape / dtype / activation / null pointer          */
  GNNHWC_ERR_WORKSPACE = -2,        /* workspace null, misaligned or smaller than required     */
  GNNHWC_ERR_LAUNCH = -3            /* the HIP runtime rejected a launch (message has details) */
};

/* Library version, (major << 16) | minor. */
int gnnhwc_version(void);

/* Human-readable description of the last error on this thread ("" if none). */
const char *gnnhwc_last_error(void);

/*
 * Bytes of device workspace gnnhwc_fwd / gnnhwc_bwd need for this problem (0 is never returned
 * for a valid shape; returns 0 and sets the error string for an invalid one).  The workspace must
 * be 256-byte aligned; its contents on entry are ignored and are undefined on return.
 * Replaces: raw_alloc of the Welford scratch (gn_kernel.cu:461) and of the seven backward
 * scratch buffers (gn_kernel.cu:954,973-974,998-1001).
 */
size_t gnnhwc_fwd_workspace_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype);
size_t gnnhwc_bwd_workspace_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype);

/*
 * Forward: per-(n, group) mean / rstd = 1/sqrt(var + eps) (biased variance), then
 *   y = act((x - mean) * rstd * weight + bias).
 * Replaces run_gn_fwd_kernels<T> (gn_kernel.h:11-24; gn_kernel.cu:439-531).
 *   dtype        : type of x and y.
 *   param_dtype  : type of weight and bias (the reference requires it to equal dtype,
 *                  custom_gn.cpp:35; here GNNHWC_F32 parameters with F16/BF16 data are also accepted).
 *   stats_dtype  : type mean / rstd are written in; equal to dtype, or GNNHWC_F32 for F16/BF16 data.
 * Statistics are always accumulated and applied in fp32 (fp64 for F64) whatever stats_dtype is.
 * Inference: mean and / or rstd may be NULL when the caller does not need them (no backward will follow), and
 * y may be the same buffer as x (every element of x is read before the element of y that replaces it is written).
 */
int gnnhwc_fwd(const void *x, const void *weight, const void *bias,
               void *y, void *mean, void *rstd,
               int64_t N, int64_t R, int64_t C, int64_t G,
               double eps, int act,
               int dtype, int param_dtype, int stats_dtype,
               void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * Forward of float data with y written in a 16-bit type (no counterpart in the reference, where y has the type of x,
 * custom_gn.cpp:28, and the cast for a half-precision consumer is a separate elementwise pass).  For the
 * GroupNorm -> activation -> convolution step of a network whose convolutions run in half precision on a float
 * residual stream: y leaves in the convolution's type, each value rounded once from the fp32 result, so the forward
 * writes S/2 instead of S bytes and the cast kernel (1.5 S more traffic) disappears.
 *   dtype   : GNNHWC_F32 (type of x).
 *   y_dtype : GNNHWC_F16 or GNNHWC_BF16 (type of y); GNNHWC_F32 makes this gnnhwc_fwd.  Anything else, or another
 *             dtype with a y_dtype different from it, is GNNHWC_ERR_INVALID_ARGUMENT.
 * y must not be the buffer of x when the types differ.  Everything else as gnnhwc_fwd (same workspace size).
 * The backward that follows is gnnhwc_bwd_cast, which reads the 16-bit gradient of y as it is.
 */
int gnnhwc_fwd_cast(const void *x, const void *weight, const void *bias,
                    void *y, void *mean, void *rstd,
                    int64_t N, int64_t R, int64_t C, int64_t G,
                    double eps, int act,
                    int dtype, int param_dtype, int stats_dtype, int y_dtype,
                    void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * Forward with the additions that precede the normalisation fused in (no counterpart in the reference, whose
 * callers add in a separate pass: in a diffusion ResNet block `h + temb[:, :, None, None]` before the second
 * norm, and `shortcut + h` before the next block's first norm).  The tensor that is normalised is
 *   s = x + residual + channel_bias[n][c]          (fp32 arithmetic, rounded to dtype once)
 * i.e. exactly what an elementwise addition in dtype would have handed to gnnhwc_fwd; y, mean and rstd are those
 * of gnnhwc_fwd applied to s.
 *   residual      : (N, R, C) in dtype, or NULL.
 *   channel_bias  : (N, C) in channel_bias_dtype (dtype, or GNNHWC_F32 for F16/BF16 data), or NULL.
 *   sum_out       : (N, R, C) in dtype; receives s.  May be NULL when the caller does not need the sum, and may be
 *                   the same buffer as x or residual (in-place accumulation); must differ from y.
 * With all three NULL this is gnnhwc_fwd.  Workspace: gnnhwc_fwd_workspace_bytes.  y may alias x or residual.
 * A later backward takes s as its x (gnnhwc_bwd knows nothing of the additions: the gradient of s is the gradient
 * of x and of residual, and its sum over R is the gradient of channel_bias).
 */
int gnnhwc_fwd_add(const void *x, const void *residual, const void *channel_bias, void *sum_out,
                   const void *weight, const void *bias,
                   void *y, void *mean, void *rstd,
                   int64_t N, int64_t R, int64_t C, int64_t G,
                   double eps, int act,
                   int dtype, int param_dtype, int stats_dtype, int channel_bias_dtype,
                   void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * Forward that allocates nothing (no counterpart in the reference, whose host driver takes its scratch from the
 * caching allocator on every call, gn_kernel.cu:461,530).  For callers that cannot allocate device memory or have
 * nobody to allocate for them: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same results contract and arguments as gnnhwc_fwd without the workspace: the per-tile partial statistics live in
 * GNNHWC_STATIC_SCRATCH_BYTES of device memory that is part of the library's image (every device the library runs on
 * holds its own copy until the process ends; the first call on a device looks its address up, nothing is allocated
 * then or later, and no event, host-pinned word or other library state is created).  It always runs the multi-launch
 * kernels (statistics, then normalise + activation: x is read twice), whose scratch needs no clearing: every word a
 * launch reads has been written by the launch before it in the same call.
 *   - A problem whose partial statistics need more than the scratch holds is rejected with GNNHWC_ERR_WORKSPACE and
 *     nothing is launched; gnnhwc_fwd_static_scratch_bytes tells how much a problem needs (0 for an invalid shape).
 *   - All calls on one device share that device's scratch: calls that overlap in time on one device (two streams,
 *     two host threads, two concurrently replayed graphs) race and give undefined statistics.  Calls that follow
 *     each other on one stream are safe.
 *   - Per-kernel timing (gnnhwc_profile_enable) is ignored by this entry point.
 */
#define GNNHWC_STATIC_SCRATCH_BYTES (4u << 20)
size_t gnnhwc_fwd_static_scratch_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype);
int gnnhwc_fwd_static(const void *x, const void *weight, const void *bias,
                      void *y, void *mean, void *rstd,
                      int64_t N, int64_t R, int64_t C, int64_t G,
                      double eps, int act,
                      int dtype, int param_dtype, int stats_dtype,
                      void *stream /* hipStream_t */);

/*
 * Backward: given dy and the forward's inputs and statistics, recomputes the activation gradient and
 * returns dx (N,R,C), dweight (C) and dbias (C).
 * Replaces run_gn_bwd_kernels<T> (gn_kernel.h:26-41; gn_kernel.cu:932-1055).
 *   dweight / dbias are written in param_dtype; either may be NULL to skip it.
 *   dx may be the buffer of dy (every element of dy is read before the element of dx in its place is written); it must
 *   not be the buffer of x.
 */
int gnnhwc_bwd(const void *dy, const void *x, const void *weight, const void *bias,
               const void *mean, const void *rstd,
               void *dx, void *dweight, void *dbias,
               int64_t N, int64_t R, int64_t C, int64_t G, int act,
               int dtype, int param_dtype, int stats_dtype,
               void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * Backward of float data whose incoming gradient is stored in a 16-bit type (no counterpart in the reference, where dy
 * has the type of x, custom_gn.cpp:64-65): the training half of gnnhwc_fwd_cast.  dy is widened in registers as it is
 * loaded; no separate pass over it, and dy costs S/2 instead of S bytes of traffic.
 *   dtype    : GNNHWC_F32 (type of x and dx).
 *   dy_dtype : GNNHWC_F16 or GNNHWC_BF16 (type of dy); GNNHWC_F32 makes this gnnhwc_bwd.  Anything else, or another
 *              dtype with a dy_dtype different from it, is GNNHWC_ERR_INVALID_ARGUMENT.
 * dx must not be the buffer of dy when the types differ.  Results are bit for bit those of gnnhwc_bwd on dy widened to
 * float.  Everything else as gnnhwc_bwd (same workspace size).
 */
int gnnhwc_bwd_cast(const void *dy, const void *x, const void *weight, const void *bias,
                    const void *mean, const void *rstd,
                    void *dx, void *dweight, void *dbias,
                    int64_t N, int64_t R, int64_t C, int64_t G, int act,
                    int dtype, int param_dtype, int stats_dtype, int dy_dtype,
                    void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * Channels-first layout: x, y, dy, dx are (N, C, R) contiguous, R fastest.  The reference has no kernel for it:
 * GN_NHWC.forward hands such input to torch's GroupNorm and applies the activation in a second pass
 * (custom_gn.py:75-79); these entry points give the same results with the activation fused (forward: two launches,
 * x read twice; backward: two, x and dy read twice).  Arguments, dtypes, NULL conventions and errors are those of gnnhwc_fwd /
 * gnnhwc_bwd, except that C comes before R; y may alias x.  Workspace: gnnhwc_nchw_workspace_bytes.
 */
size_t gnnhwc_nchw_workspace_bytes(int64_t N, int64_t C, int64_t R, int64_t G, int dtype, int backward);
int gnnhwc_fwd_nchw(const void *x, const void *weight, const void *bias,
                    void *y, void *mean, void *rstd,
                    int64_t N, int64_t C, int64_t R, int64_t G,
                    double eps, int act,
                    int dtype, int param_dtype, int stats_dtype,
                    void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);
int gnnhwc_bwd_nchw(const void *dy, const void *x, const void *weight, const void *bias,
                    const void *mean, const void *rstd,
                    void *dx, void *dweight, void *dbias,
                    int64_t N, int64_t C, int64_t R, int64_t G, int act,
                    int dtype, int param_dtype, int stats_dtype,
                    void *workspace, size_t workspace_bytes, void *stream /* hipStream_t */);

/*
 * Kernel selection (no counterpart in the reference).  By default a problem whose tensors fit in the
 * register files of one launch is run by the single-launch kernels (x and dy are read from memory once;
 * workgroups exchange partial results while resident), anything else by the multi-launch streaming
 * kernels.  A single-launch kernel is fastest with the device to itself: calls of one process on
 * different streams are ordered by the library (a call on another stream than the previous single-launch
 * call of the device first makes its stream wait, on the device, for what has been submitted to that
 * previous stream).  Where the device is shared all the same (launches recorded into graphs that are replayed
 * concurrently, other processes), the kernels still produce correct results, more slowly (see
 * gnnhwc_resident_status below); gnnhwc_set_resident(0) (or GNNHWC_DISABLE_RESIDENT=1 in the environment)
 * selects the streaming kernels, which do not care.  Process-wide; returns the previous setting.
 */
int gnnhwc_set_resident(int on);

/*
 * Per-kernel timing for benchmarks (no counterpart in the reference, which relies on an external
 * profiler, prof.py:1-39).  While enabled, every kernel the library launches on this thread carries a
 * pair of HIP events bound to its own dispatch on the launch stream, so that their difference is the
 * kernel's begin-to-end time on the device.  gnnhwc_profile_collect synchronises those events and
 * reports, for each kernel kind, the number of launches and the summed duration in milliseconds since
 * the last collect, then clears the record.  Kinds: 0 fwd statistics, 1 fwd statistics compaction
 * (many row tiles only), 2 fwd apply, 3 bwd reduce, 4 bwd compaction (many row tiles only), 5 bwd dx,
 * 6 single-launch fwd, 7 single-launch bwd, 8 the plain copy of gnnhwc_debug_copy, 9 the elementwise pre-addition
 * of gnnhwc_fwd_add's multi-launch form, 10 single-launch fwd with the pre-addition fused in, 11-14 the channels-first
 * kernels (fwd statistics, fwd apply, bwd reduce, bwd dx with dgamma / dbeta).
 */
#define GNNHWC_NUM_KERNEL_KINDS 15
int gnnhwc_profile_enable(int on);
int gnnhwc_profile_collect(int64_t *launches /* [GNNHWC_NUM_KERNEL_KINDS] */,
                           double *total_ms /* [GNNHWC_NUM_KERNEL_KINDS] */);
const char *gnnhwc_kernel_kind_name(int kind);

/*
 * What the single-launch kernels do when their workgroups cannot all run at once (no counterpart in the reference,
 * whose independent launches, gn_kernel.cu:439-536 and 932-1060, have no such state -- and neither has this library: no
 * call fails or returns wrong numbers because of it).  The workgroups of such a kernel wait for each other's partial
 * results with a bounded number of polls.  If a wait expires (another stream, a concurrently replayed graph or another
 * process holds part of the device, so that some workgroups have not been scheduled yet), the waiting workgroup stops
 * waiting: it takes the partial results that have arrived, recomputes the missing ones from the call's own inputs,
 * reads its rows again and stores its results.  Every workgroup publishes its own partial results before it waits, so
 * the workgroups scheduled later find everything: the kernel always ends, and y, mean, rstd, dx, dweight, dbias are
 * correct to the same tolerances as always -- the call only takes longer (milliseconds instead of microseconds when
 * many workgroups had to recompute).
 *   - gnnhwc_resident_status() returns 1 if that has happened in any single-launch kernel of this process since the
 *     last query, else 0, and clears the note.  It never reports an error and does not synchronise: ask once the work
 *     in question has completed.  A caller that sees 1 often may prefer gnnhwc_set_resident(0) for that workload
 *     (the multi-launch kernels need no co-residency); nothing switches by itself.
 *   - gnnhwc_debug_set_spin_limit sets the number of polls per wait (about a microsecond each) and returns the
 *     previous value: negative restores the default (1024), except -2, which makes every wait expire at its first poll
 *     whether or not the data had arrived and every partial result be recomputed; tests use that to exercise the
 *     recovery, every kernel still exits normally.  With -2, outputs must not replace inputs in place (a recomputation
 *     that ignores what has arrived may read rows another workgroup has already overwritten; in normal operation a
 *     recomputed value is only used if its workgroup has provably not written anything yet).
 */
int gnnhwc_resident_status(void);
int gnnhwc_debug_set_spin_limit(int polls);

/*
 * Which kernels the calling thread's most recent gnnhwc_fwd / _fwd_add / _fwd_cast / gnnhwc_bwd call launched (no
 * counterpart in the reference; for benchmarks and tests that must know what they measured).  out[7] receives: the
 * kernel kind (6, 7 or 10: a single-launch kernel; -1: the multi-launch kernels), rows per lane of the register tile,
 * rows of the x window of a backward that keeps g' only (0: x is kept too), 1 if the two-level exchange was used,
 * the number of launches the call was cut into (over groups of samples), workgroups of the last of them, rows of x
 * that backward parks in LDS between its two passes.
 */
int gnnhwc_debug_last_launch(int64_t *out /* [7] */);

/*
 * Plain device-to-device copy of `bytes` (a multiple of 16; 16-byte aligned pointers) by a kernel with the
 * same block size and access width as the GroupNorm kernels and no arithmetic.  No counterpart in the
 * reference.  Benchmarks use it as the practical ceiling a two-stream kernel can reach at a given size, and
 * as the dispatch of known size that calibrates hardware memory-traffic counters.
 */
int gnnhwc_debug_copy(void *dst, const void *src, size_t bytes, void *stream /* hipStream_t */);

/*
 * The load phase of a single-launch kernel on its own (no counterpart in the reference): every lane of a grid of
 * (row tiles, 128-byte chunks, samples) workgroups requests rows_per_lane (4, 8, 16, 22 or 32) rows of 16 bytes of x --
 * and of dy unless it is NULL -- up front, in those kernels' tile geometry, and nothing else happens.  A yardstick like
 * gnnhwc_debug_copy: a single-launch kernel cannot have its rows sooner than this kernel ends.  row_bytes: bytes of one
 * row of the (N, R, C) tensor, a multiple of 128.  sink: 4 writable bytes or NULL.  Timed as kernel kind 8.
 */
int gnnhwc_debug_load_tile(const void *x, const void *dy, void *sink, int64_t N, int64_t R, int64_t row_bytes,
                           int rows_per_lane, void *stream /* hipStream_t */);

/*
 * The tiling the multi-launch kernels would use for a problem (no counterpart in the reference, whose
 * calc_block_params, gn_kernel.cu:37-60, is internal too); nothing is launched, no GPU is needed.  For tests of the
 * host-side planning.  vector: 1 = 16-byte lane vectors (C must be a multiple of 16 / sizeof(dtype)), 0 = scalar
 * kernels; backward: 0 / 1.  out[12] receives: elements per lane vector, lane vectors per row, lane vectors of a
 * row per workgroup, chunks along C, rows per step, rows per tile, tiles per sample, most groups a chunk
 * intersects, workgroups per launch, 1 if a compaction launch runs between producer and consumer, bytes of
 * workspace this tiling needs, channels per group.
 */
int gnnhwc_debug_plan(int64_t N, int64_t R, int64_t C, int64_t G, int dtype, int vector, int backward,
                      int64_t *out /* [12] */);

/*
 * In-kernel timeline of the single-launch kernels, for tuning (no counterpart in the reference; its
 * nearest relative is the DEBUG(...) launch-parameter printf, gn_kernel.cu:13-19).  Only in
 * libgnnhwc_hip_trace.so, the same library compiled with the stamps (the library proper has none: even switched
 * off they cost every launch time, and there this call returns an error).  With GNNHWC_TRACE=1 (stamps wait for
 * outstanding memory operations) or 2 (they do not) in the environment at the first call, thread 0 of every
 * workgroup of a single-launch kernel writes a 100 MHz wall-clock stamp at up to 8 phase boundaries.  This call
 * synchronises the device and copies `count` 64-bit words, laid out [workgroup][8], from the most recent such launch.
 */
int gnnhwc_debug_read_trace(unsigned long long *out, int64_t count);

#ifdef __cplusplus
}
#endif
#endif /* GNNHWC_H */
