// Host-side interface between the C ABI (gn_api.hip) and the per-element-type kernel launchers
// (gn_inst.hip, compiled once per type).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include "gn_plan.h"

namespace gn {

enum KernelKind {
  kKindFwdStats = 0,
  kKindFwdStatsFinalize = 1,
  kKindFwdApply = 2,
  kKindBwdReduce = 3,
  kKindBwdFinalize = 4,
  kKindBwdDx = 5,
  kKindFusedFwd = 6,
  kKindFusedBwd = 7,
  kNumKinds = 8
};

struct FwdArgs {
  const void *x, *w, *b;
  void *y, *mean, *rstd;
  double eps;
  int act, pdtype, sdtype;
  void *ws;
  hipStream_t stream;
  Plan plan;
};
struct BwdArgs {
  const void *dy, *x, *w, *b, *mean, *rstd;
  void *dx, *dw, *db;
  int act, pdtype, sdtype;
  void *ws;
  hipStream_t stream;
  Plan plan;
};

// Workspace layout, in elements of the accumulation type (float, or double for f64 data).
struct FwdWorkspace {
  size_t part, mean, rstd, total;  // element offsets; total = element count
};
struct BwdWorkspace {
  size_t part, sums, coef, total;
};
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline FwdWorkspace fwd_workspace(const Plan &p) {
  FwdWorkspace w;
  w.part = 0;
  w.mean = align_up((size_t)p.N * p.tiles * p.nchunk * p.G * 3, 64);
  w.rstd = w.mean + align_up((size_t)p.N * p.G, 64);
  w.total = w.rstd + align_up((size_t)p.N * p.G, 64);
  return w;
}
inline BwdWorkspace bwd_workspace(const Plan &p) {
  BwdWorkspace w;
  w.part = 0;
  w.sums = align_up((size_t)p.N * p.tiles * p.C * 2, 64);
  w.coef = w.sums + align_up((size_t)p.N * p.C * 2, 64);
  w.total = w.coef + align_up((size_t)p.N * p.G * 2, 64);
  return w;
}

// Bracket one kernel launch with HIP events when profiling is enabled on this thread (gn_api.hip).
void profile_before(int kind, hipStream_t stream);
void profile_after(int kind, hipStream_t stream);
struct ProfileScope {
  int kind;
  hipStream_t stream;
  ProfileScope(int k, hipStream_t s) : kind(k), stream(s) { profile_before(kind, stream); }
  ~ProfileScope() { profile_after(kind, stream); }
};

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

}  // namespace gn
