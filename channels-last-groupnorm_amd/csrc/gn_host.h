// Host-side interface between the C ABI (gn_api.hip) and the per-element-type kernel launchers
// (gn_inst.hip, compiled once per type).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>
#include <tuple>
#include <utility>
#include "../../include/gnnhwc.h"
#include "gn_plan.h"

namespace gn {

enum KernelKind {
  kKindFwdStats = 0,
  kKindFwdStatsCompact = 1,
  kKindFwdApply = 2,
  kKindBwdReduce = 3,
  kKindBwdCompact = 4,
  kKindBwdDx = 5,
  kKindFusedFwd = 6,
  kKindFusedBwd = 7,
  kKindCopy = 8,
  kKindAdd = 9,        // elementwise pre-addition of the multi-launch fused-addition forward
  kKindFusedFwdAdd = 10,  // single-launch forward with the pre-addition fused in
  kKindNchwStats = 11,    // channels-first layout: forward statistics, forward apply, backward reduce,
  kKindNchwApply = 12,    // backward dx (+ dgamma / dbeta)
  kKindNchwBwdReduce = 13,
  kKindNchwBwdDx = 14,
  kNumKinds = 15
};
static_assert(kNumKinds == GNNHWC_NUM_KERNEL_KINDS, "kernel kinds out of step with include/gnnhwc.h");

struct FwdArgs {
  const void *x, *w, *b;
  AddArgs add;  // all null: plain forward
  bool has_add() const { return add.residual || add.channel_bias || add.sum_out; }
  void *y, *mean, *rstd;
  double eps;
  int act, pdtype, sdtype;
  int ydtype;  // type y is stored in: the data type, or for float data GN_F16 / GN_BF16
  void *ws;
  hipStream_t stream;
  Plan plan;
  bool streaming_only = false;  // multi-launch kernels whatever the size (the entry point that must not allocate)
};
struct BwdArgs {
  const void *dy, *x, *w, *b, *mean, *rstd;
  void *dx, *dw, *db;
  int act, pdtype, sdtype;
  int dydtype;  // type dy is stored in: the data type, or for float data GN_F16 / GN_BF16
  void *ws;
  hipStream_t stream;
  Plan plan;
};

// One call on a channels-first tensor (N, C, R contiguous): forward (x -> y, mean_out, rstd_out) or backward
// (dy, x, mean, rstd -> dx, dw, db).
struct NchwArgs {
  bool backward, vector;  // vector: 16-byte lane vectors (R a multiple of the vector width, aligned pointers)
  const void *x, *dy, *w, *b, *mean, *rstd;
  void *y, *dx, *dw, *db, *mean_out, *rstd_out;
  int64_t N, C, R, G;
  double eps;
  int act, pdtype, sdtype;
  void *ws;
  hipStream_t stream;
};
// Elements of one chunk of a channel row: 64 lanes x vec elements x 4 lane vectors (kNchwUnroll in gn_nchw.h).
inline int nchw_chunk_len(int vec) { return 64 * vec * 4; }
// Accumulation-type elements of the per-chunk partials: 3 planes forward, 2 backward, of [N * C][chunks] ...
inline size_t nchw_partial_elems(int64_t N, int64_t C, int64_t R, int vec, bool backward) {
  const int64_t chunks = (R + nchw_chunk_len(vec) - 1) / nchw_chunk_len(vec);
  return ((size_t)(backward ? 2 : 3) * (size_t)(N * C * chunks) + 63) / 64 * 64;
}
// ... and of the whole workspace: behind them, 2 planes [N * G] for the per-slab records of the compaction launch
// (at most N * C elements each, whatever G is).
inline size_t nchw_workspace_elems(int64_t N, int64_t C, int64_t R, int vec, bool backward) {
  return nchw_partial_elems(N, C, R, vec, backward) + 2 * (size_t)(N * C);
}

// Workspace layout, in elements of the accumulation type (float, or double for f64 data).
struct FwdWorkspace {
  size_t part, compact, total;  // element offsets; total = element count
};
struct BwdWorkspace {
  size_t partC, partG, compactC, compactG, total;
};
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline FwdWorkspace fwd_workspace(const Plan &p) {
  FwdWorkspace w;
  w.part = 0;
  w.compact = align_up((size_t)p.N * p.tiles * p.nchunk * p.G * 3, 64);  // 3 planes [N][nchunk][G][tiles]
  w.total = w.compact + align_up((size_t)p.N * p.G * 3, 64);
  return w;
}
inline BwdWorkspace bwd_workspace(const Plan &p) {
  BwdWorkspace w;
  w.partC = 0;
  w.partG = align_up((size_t)p.N * p.tiles * p.C * 2, 64);
  w.compactC = w.partG + align_up((size_t)p.N * p.tiles * p.nchunk * p.G * 2, 64);
  w.compactG = w.compactC + align_up((size_t)p.N * p.C * 2, 64);
  w.total = w.compactG + align_up((size_t)p.N * p.G * 2, 64);
  return w;
}
// Every layout of the workspace (streaming or single-launch, forward or backward) leaves its first 256 bytes unused.
constexpr size_t kWorkspaceHeader = 256;
// The resident kernels keep their partial results and one flag per workgroup in the same workspace.
constexpr int kMaxResidentBlocks = 4 * kNumCU;
inline size_t resident_rec_bytes(int64_t G) { return (size_t)16 * G * kMaxResidentBlocks; }
// Final records of the two-level exchange, one per (sample, group) of a launch: a launch has at most kMaxResidentBlocks samples.
inline size_t resident_frec_bytes(int64_t G) { return (size_t)16 * G * kMaxResidentBlocks; }
inline size_t resident_fwd_bytes(int64_t G) {
  return kWorkspaceHeader + align_up(resident_rec_bytes(G), 256) + align_up(resident_frec_bytes(G), 256);
}
// All-to-all or two-level exchange: records a workgroup would poll in the all-to-all form (tiles x chunks per group x
// groups per chunk); beyond this bound the polling traffic of the whole launch rivals the tensor itself.
constexpr int kTwoLevelRecords = 1024;
inline bool two_level_exchange(const Plan &p) {
  const int chunk_channels = p.lpr * p.vec;
  const int64_t per_group = (int64_t)p.tiles * ((p.D - 1) / chunk_channels + 2);
  return per_group * p.gmax > kTwoLevelRecords && p.tiles > 1;
}
// chunk_channels = channels per workgroup (lpr * vec): N * tiles * C = workgroups * chunk_channels
// A tensor of several samples that is too large for one single-launch kernel may still be run as up to
// kMaxBatches such launches over consecutive groups of samples (samples share nothing but dgamma / dbeta).
constexpr int kMaxBatches = 4;
// Channel records of the backward, 16 bytes per (sample, tile, channel): one launch's worth is at most
// chunk_channels * kMaxResidentBlocks of them, and there is room for the launches of a batched call up to a bound.
inline size_t resident_crec_bytes(int64_t chunk_channels) {
  const size_t one = (size_t)16 * chunk_channels * kMaxResidentBlocks;
  const size_t many = one * kMaxBatches < ((size_t)16 << 20) ? one * kMaxBatches : ((size_t)16 << 20);
  return align_up(one > many ? one : many, 256);
}
inline size_t resident_bwd_bytes(int64_t chunk_channels, int64_t G) {
  return kWorkspaceHeader + resident_crec_bytes(chunk_channels) + align_up(resident_rec_bytes(G), 256) +
         align_up(resident_frec_bytes(G), 256);
}
// A fresh nonzero 64-bit value per call (gn_api.hip).
unsigned long long next_epoch();
// Epoch source of launches that are being recorded into a HIP graph.  captured_epoch() leaves `generation` null
// when `stream` is not capturing; otherwise it points at the library's per-device generation word, and the
// kernel that increments it has been recorded on `stream` if this is the first such launch of the capture.
// Returns false if the stream is capturing but the word is not available (the caller then records the
// multi-launch kernels instead).
struct CapturedEpoch {
  const unsigned long long *generation = nullptr;
  unsigned long long next_sequence() const;  // differs between the captured launches of one graph
};
bool captured_epoch(hipStream_t stream, CapturedEpoch &out);
// Two single-launch kernels must not share the device: each needs all of its workgroups resident at once.  Kernels
// of one stream follow each other anyway; when a call arrives on another stream than the previous single-launch
// call of the device, this makes the new stream wait for everything submitted so far on the previous one (an
// event recorded there, no host synchronisation).  The object also serialises the host-side bookkeeping and the
// enqueueing of the launches it guards, so it lives until they have been submitted.  Launches that are being
// recorded into a graph are not ordered this way.
class ResidentOrder {
 public:
  ResidentOrder(hipStream_t stream, bool capturing);
  ~ResidentOrder();
  ResidentOrder(const ResidentOrder &) = delete;
  ResidentOrder &operator=(const ResidentOrder &) = delete;

 private:
  bool locked_;
};
// Which single-launch kernel the calling thread's most recent call used (gnnhwc_debug_last_launch): rows per lane, rows of
// the x window (0: none), rows of x parked in LDS, two-level exchange, launches the call was cut into, workgroups of the
// last launch.
void note_resident_launch(int kind, int rows_per_lane, int window_rows, int parked_rows, int two_level, int launches,
                          int64_t workgroups);
void note_streaming_call();
bool resident_enabled();
// Device buffer for in-kernel timestamps when GNNHWC_TRACE=1, else null.
unsigned long long *trace_buffer();
bool trace_waits();  // GNNHWC_TRACE=1: stamps wait for memory; GNNHWC_TRACE=2: they do not
// Host-pinned word the single-launch kernels set on a timed-out wait (null if it cannot be allocated: then the
// single-launch kernels are not used), and the note that a kernel has been given it.
unsigned long long *resident_status();
void mark_resident_launch();
int resident_spin_limit();
int resident_min_rows();  // tuning knob (environment): smallest rows-per-lane variant the single-launch path may pick

// Consumers merge the tile partials of their own groups in their prologue when every lane has at most kEarly
// entries to fetch; otherwise a compaction kernel runs in between and leaves one entry per group.
inline bool needs_compaction(const Plan &p) {
  const int chunk_channels = p.lpr * p.vec;
  const int64_t per_group = (int64_t)p.tiles * ((p.D - 1) / chunk_channels + 2);
  const int lanes = merge_lanes_for(p.gmax);
  return lanes < 1 || per_group > (int64_t)kEarly * lanes;
}
// Whether a chunk's groups fit one merge round at all (more than kBlock groups per chunk do not; those plans
// use the general looping merge).
inline bool one_round_merge(const Plan &p) { return pow2_at_least(p.gmax) <= kBlock; }

// Per-kernel timing (gn_api.hip).  When profiling is enabled on this thread, profile_events hands out a
// start / stop event pair that the launch binds to the kernel's own dispatch: their difference is the
// kernel's begin-to-end time on the device, the quantity a kernel trace reports, with no dispatch gap.
bool profile_events(int kind, hipEvent_t *start, hipEvent_t *stop);

// GNNHWC_COOPERATIVE=1 (measurement only): the single-launch kernels go through hipLaunchCooperativeKernel, the
// runtime's own guarantee that a grid is resident as a whole, instead of a plain launch.
bool cooperative_launches();
template <typename... KArgs, size_t... I>
inline void launch_cooperative(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t stream, std::tuple<KArgs...> &vals,
                               std::index_sequence<I...>) {
  void *argv[] = {(void *)&std::get<I>(vals)...};
  (void)hipLaunchCooperativeKernel((const void *)kernel, grid, block, argv, 0, stream);
}
template <typename... KArgs, typename... Args>
inline void launch(int kind, void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t stream, Args &&...args) {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if ((kind == kKindFusedFwd || kind == kKindFusedBwd || kind == kKindFusedFwdAdd) && cooperative_launches()) {
    std::tuple<KArgs...> vals(static_cast<KArgs>(args)...);
    const bool timed = profile_events(kind, &e0, &e1);  // (events around the launch, not bound to the dispatch)
    if (timed) (void)hipEventRecord(e0, stream);
    launch_cooperative(kernel, grid, block, stream, vals, std::index_sequence_for<KArgs...>{});
    if (timed) (void)hipEventRecord(e1, stream);
    return;
  }
  if (profile_events(kind, &e0, &e1))
    hipExtLaunchKernelGGL(kernel, grid, block, 0, stream, e0, e1, 0, static_cast<KArgs>(args)...);
  else
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, static_cast<KArgs>(args)...);
}

// Return hipSuccess or the first launch error.
template <typename T> hipError_t launch_fwd(const FwdArgs &a);
template <typename T> hipError_t launch_bwd(const BwdArgs &a);

hipError_t launch_fwd_f32(const FwdArgs &a);
hipError_t launch_fwd_f64(const FwdArgs &a);
hipError_t launch_fwd_f16(const FwdArgs &a);
hipError_t launch_fwd_bf16(const FwdArgs &a);
hipError_t launch_bwd_f32(const BwdArgs &a);
hipError_t launch_bwd_f64(const BwdArgs &a);
hipError_t launch_bwd_f16(const BwdArgs &a);
hipError_t launch_bwd_bf16(const BwdArgs &a);
hipError_t launch_nchw_f32(const NchwArgs &a);
hipError_t launch_nchw_f64(const NchwArgs &a);
hipError_t launch_nchw_f16(const NchwArgs &a);
hipError_t launch_nchw_bf16(const NchwArgs &a);

}  // namespace gn
