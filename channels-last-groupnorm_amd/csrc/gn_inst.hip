// Kernel instantiations and launch sequences for ONE element type, selected with -DGN_INST_DTYPE=0..3
// (f32, f64, f16, bf16).  Built four times so the four types compile in parallel.
#include "gn_host.h"
#include "gn_kernels.h"

#ifndef GN_INST_DTYPE
#error "compile with -DGN_INST_DTYPE=<0|1|2|3>"
#endif

namespace gn {

#if GN_INST_DTYPE == 0
typedef float elem_t;
#define GN_SUFFIX f32
#elif GN_INST_DTYPE == 1
typedef double elem_t;
#define GN_SUFFIX f64
#elif GN_INST_DTYPE == 2
typedef f16_t elem_t;
#define GN_SUFFIX f16
#else
typedef bf16_t elem_t;
#define GN_SUFFIX bf16
#endif
#define GN_CAT2(a, b) a##b
#define GN_CAT(a, b) GN_CAT2(a, b)

namespace {

typedef acc_t<elem_t> A;
constexpr int kVec = vec_of<elem_t>::value;

template <int VEC, int ACT> void launch_apply(const FwdArgs &a, const A *ws_mean, const A *ws_rstd) {
  const Plan &p = a.plan;
  hipLaunchKernelGGL((apply_kernel<elem_t, VEC, ACT>), dim3((unsigned)p.nblocks), dim3(kBlock), 0, a.stream,
                     (const elem_t *)a.x, (elem_t *)a.y, ws_mean, ws_rstd, a.w, a.b, a.pdtype, p);
}
template <int VEC> void launch_apply_act(const FwdArgs &a, const A *ws_mean, const A *ws_rstd) {
  switch (a.act) {
    case GN_ACT_IDENTITY: launch_apply<VEC, GN_ACT_IDENTITY>(a, ws_mean, ws_rstd); break;
    case GN_ACT_RELU: launch_apply<VEC, GN_ACT_RELU>(a, ws_mean, ws_rstd); break;
    case GN_ACT_SILU: launch_apply<VEC, GN_ACT_SILU>(a, ws_mean, ws_rstd); break;
    case GN_ACT_GELU: launch_apply<VEC, GN_ACT_GELU>(a, ws_mean, ws_rstd); break;
    default: launch_apply<VEC, GN_ACT_GELU_TANH>(a, ws_mean, ws_rstd); break;
  }
}

template <int VEC> hipError_t fwd_impl(const FwdArgs &a) {
  const Plan &p = a.plan;
  const FwdWorkspace ws = fwd_workspace(p);
  A *base = (A *)a.ws;
  A *part = base + ws.part, *ws_mean = base + ws.mean, *ws_rstd = base + ws.rstd;
  {
    ProfileScope s(kKindFwdStats, a.stream);
    hipLaunchKernelGGL((stats_kernel<elem_t, VEC>), dim3((unsigned)p.nblocks), dim3(kBlock), 0, a.stream,
                       (const elem_t *)a.x, part, p);
  }
  {
    ProfileScope s(kKindFwdStatsFinalize, a.stream);
    const int64_t items = p.N * p.G;
    const unsigned grid = (unsigned)((items + kBlock / 64 - 1) / (kBlock / 64));
    hipLaunchKernelGGL((stats_finalize_kernel<A>), dim3(grid), dim3(kBlock), 0, a.stream, (const A *)part, ws_mean,
                       ws_rstd, a.mean, a.rstd, a.sdtype, (A)a.eps, p);
  }
  {
    ProfileScope s(kKindFwdApply, a.stream);
    launch_apply_act<VEC>(a, ws_mean, ws_rstd);
  }
  return hipGetLastError();
}

template <int VEC, int ACT> void launch_bwd_act(const BwdArgs &a) {
  const Plan &p = a.plan;
  const BwdWorkspace ws = bwd_workspace(p);
  A *base = (A *)a.ws;
  A *part = base + ws.part, *sums = base + ws.sums, *coef = base + ws.coef;
  {
    ProfileScope s(kKindBwdReduce, a.stream);
    hipLaunchKernelGGL((bwd_reduce_kernel<elem_t, VEC, ACT>), dim3((unsigned)p.nblocks), dim3(kBlock), 0, a.stream,
                       (const elem_t *)a.x, (const elem_t *)a.dy, a.mean, a.rstd, a.sdtype, a.w, a.b, a.pdtype, part, p);
  }
  {
    ProfileScope s(kKindBwdFinalize, a.stream);
    hipLaunchKernelGGL((bwd_finalize_kernel<A>), dim3((unsigned)(p.N * p.G)), dim3(kBlock), 0, a.stream,
                       (const A *)part, a.mean, a.rstd, a.sdtype, a.w, a.pdtype, sums, coef, p);
  }
  {
    ProfileScope s(kKindBwdDx, a.stream);
    const unsigned extra = (unsigned)((p.C + kBlock - 1) / kBlock);
    hipLaunchKernelGGL((bwd_dx_kernel<elem_t, VEC, ACT>), dim3((unsigned)p.nblocks + extra), dim3(kBlock), 0, a.stream,
                       (const elem_t *)a.x, (const elem_t *)a.dy, (elem_t *)a.dx, a.mean, a.rstd, a.sdtype, a.w, a.b,
                       a.pdtype, (const A *)sums, (const A *)coef, a.dw, a.db, p);
  }
}
template <int VEC> hipError_t bwd_impl(const BwdArgs &a) {
  switch (a.act) {
    case GN_ACT_IDENTITY: launch_bwd_act<VEC, GN_ACT_IDENTITY>(a); break;
    case GN_ACT_RELU: launch_bwd_act<VEC, GN_ACT_RELU>(a); break;
    case GN_ACT_SILU: launch_bwd_act<VEC, GN_ACT_SILU>(a); break;
    case GN_ACT_GELU: launch_bwd_act<VEC, GN_ACT_GELU>(a); break;
    default: launch_bwd_act<VEC, GN_ACT_GELU_TANH>(a); break;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t GN_CAT(launch_fwd_, GN_SUFFIX)(const FwdArgs &a) {
  return a.plan.vec == 1 ? fwd_impl<1>(a) : fwd_impl<kVec>(a);
}
hipError_t GN_CAT(launch_bwd_, GN_SUFFIX)(const BwdArgs &a) {
  return a.plan.vec == 1 ? bwd_impl<1>(a) : bwd_impl<kVec>(a);
}

}  // namespace gn
