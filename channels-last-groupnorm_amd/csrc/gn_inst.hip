// Kernel instantiations and launch sequences for ONE element type, selected with -DGN_INST_DTYPE=0..3
// (f32, f64, f16, bf16).  Built four times so the four types compile in parallel.
#include "gn_host.h"
#include "gn_kernels.h"

#ifndef GN_INST_DTYPE
#error "compile with -DGN_INST_DTYPE=<0|1|2|3>"
#endif

namespace gn {

// wide_param_t: the other type weight / bias may have (f32 parameters with 16-bit data)
#if GN_INST_DTYPE == 0
typedef float elem_t;
typedef float wide_param_t;
#define GN_SUFFIX f32
#elif GN_INST_DTYPE == 1
typedef double elem_t;
typedef double wide_param_t;
#define GN_SUFFIX f64
#elif GN_INST_DTYPE == 2
typedef f16_t elem_t;
typedef float wide_param_t;
#define GN_SUFFIX f16
#else
typedef bf16_t elem_t;
typedef float wide_param_t;
#define GN_SUFFIX bf16
#endif
#define GN_CAT2(a, b) a##b
#define GN_CAT(a, b) GN_CAT2(a, b)

namespace {

typedef acc_t<elem_t> A;
constexpr int kVec = vec_of<elem_t>::value;

dim3 tile_grid(const Plan &p, int extra_x) {
  return dim3((unsigned)(p.tiles + extra_x), (unsigned)p.nchunk, (unsigned)(p.N < 65535 ? p.N : 65535));
}

template <typename PT, int VEC, int ACT> void launch_apply(const FwdArgs &a, const A *part, const PartialGeo &q) {
  const Plan &p = a.plan;
  hipLaunchKernelGGL((apply_kernel<elem_t, PT, VEC, ACT>), tile_grid(p, 0), dim3(kBlock), 0, a.stream, (const elem_t *)a.x,
                     (elem_t *)a.y, part, q, a.w, a.b, a.mean, a.rstd, a.sdtype, (A)a.eps, p);
}
template <typename PT, int VEC> void launch_apply_act(const FwdArgs &a, const A *part, const PartialGeo &q) {
  switch (a.act) {
    case GN_ACT_IDENTITY: launch_apply<PT, VEC, GN_ACT_IDENTITY>(a, part, q); break;
    case GN_ACT_RELU: launch_apply<PT, VEC, GN_ACT_RELU>(a, part, q); break;
    case GN_ACT_SILU: launch_apply<PT, VEC, GN_ACT_SILU>(a, part, q); break;
    case GN_ACT_GELU: launch_apply<PT, VEC, GN_ACT_GELU>(a, part, q); break;
    default: launch_apply<PT, VEC, GN_ACT_GELU_TANH>(a, part, q); break;
  }
}

template <int VEC> hipError_t fwd_impl(const FwdArgs &a) {
  const Plan &p = a.plan;
  const FwdWorkspace ws = fwd_workspace(p);
  A *base = (A *)a.ws;
  A *part = base + ws.part, *compact = base + ws.compact;
  PartialGeo q = {p.tiles, p.nchunk, p.lpr * p.vec};
  {
    ProfileScope s(kKindFwdStats, a.stream);
    hipLaunchKernelGGL((stats_kernel<elem_t, VEC>), tile_grid(p, 0), dim3(kBlock), 0, a.stream, (const elem_t *)a.x, part, p);
  }
  const A *src = part;
  if (needs_compaction(p)) {
    ProfileScope s(kKindFwdStatsCompact, a.stream);
    const int64_t items = p.N * p.G;
    const unsigned grid = (unsigned)((items + kBlock / 64 - 1) / (kBlock / 64));
    hipLaunchKernelGGL((stats_compact_kernel<A>), dim3(grid), dim3(kBlock), 0, a.stream, (const A *)part, compact, q, p);
    q = PartialGeo{1, 1, (int)p.C};
    src = compact;
  }
  {
    ProfileScope s(kKindFwdApply, a.stream);
    if (a.pdtype == GN_INST_DTYPE) launch_apply_act<elem_t, VEC>(a, src, q);
    else launch_apply_act<wide_param_t, VEC>(a, src, q);
  }
  return hipGetLastError();
}

template <typename PT, int VEC, int ACT> void launch_bwd_act(const BwdArgs &a) {
  const Plan &p = a.plan;
  const BwdWorkspace ws = bwd_workspace(p);
  A *base = (A *)a.ws;
  A *partC = base + ws.partC, *partG = base + ws.partG, *compactC = base + ws.compactC, *compactG = base + ws.compactG;
  PartialGeo q = {p.tiles, p.nchunk, p.lpr * p.vec};
  {
    ProfileScope s(kKindBwdReduce, a.stream);
    hipLaunchKernelGGL((bwd_reduce_kernel<elem_t, PT, VEC, ACT>), tile_grid(p, 0), dim3(kBlock), 0, a.stream,
                       (const elem_t *)a.x, (const elem_t *)a.dy, a.mean, a.rstd, a.sdtype, a.w, a.b, partC, partG, p);
  }
  const A *srcC = partC, *srcG = partG;
  if (needs_compaction(p)) {
    ProfileScope s(kKindBwdCompact, a.stream);
    const int nG = (int)((p.N * p.G + kBlock / 64 - 1) / (kBlock / 64));
    const int64_t nC = (p.N * p.C + 31) / 32;
    hipLaunchKernelGGL((bwd_compact_kernel<A>), dim3((unsigned)(nG + nC)), dim3(kBlock), 0, a.stream, (const A *)partC,
                       (const A *)partG, compactC, compactG, q, nG, p);
    q = PartialGeo{1, 1, (int)p.C};
    srcC = compactC;
    srcG = compactG;
  }
  {
    ProfileScope s(kKindBwdDx, a.stream);
    hipLaunchKernelGGL((bwd_dx_kernel<elem_t, PT, VEC, ACT>), tile_grid(p, 1), dim3(kBlock), 0, a.stream,
                       (const elem_t *)a.x, (const elem_t *)a.dy, (elem_t *)a.dx, a.mean, a.rstd, a.sdtype, a.w, a.b, srcC,
                       srcG, q, a.dw, a.db, p);
  }
}
template <typename PT, int VEC> void bwd_act(const BwdArgs &a) {
  switch (a.act) {
    case GN_ACT_IDENTITY: launch_bwd_act<PT, VEC, GN_ACT_IDENTITY>(a); break;
    case GN_ACT_RELU: launch_bwd_act<PT, VEC, GN_ACT_RELU>(a); break;
    case GN_ACT_SILU: launch_bwd_act<PT, VEC, GN_ACT_SILU>(a); break;
    case GN_ACT_GELU: launch_bwd_act<PT, VEC, GN_ACT_GELU>(a); break;
    default: launch_bwd_act<PT, VEC, GN_ACT_GELU_TANH>(a); break;
  }
}
template <int VEC> hipError_t bwd_impl(const BwdArgs &a) {
  if (a.pdtype == GN_INST_DTYPE) bwd_act<elem_t, VEC>(a);
  else bwd_act<wide_param_t, VEC>(a);
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
