// Channels-first kernels (gn_nchw.h) instantiated and launched for ONE element type, selected with
// -DGN_INST_DTYPE=0..3 (f32, f64, f16, bf16).
#include "gn_host.h"
#include "gn_nchw.h"

#ifndef GN_INST_DTYPE
#error "compile with -DGN_INST_DTYPE=<0|1|2|3>"
#endif

namespace gn {

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

NchwGeo geometry(const NchwArgs &a, int vec) {
  NchwGeo q;
  q.N = a.N; q.C = a.C; q.R = a.R;
  q.G = (int)a.G;
  q.D = (int)(a.C / a.G);
  q.chunk_len = nchw_chunk_len(vec);
  q.chunks = (int)((a.R + q.chunk_len - 1) / q.chunk_len);
  q.rows = a.N * a.C;
  return q;
}
unsigned wave_grid(int64_t waves) { return (unsigned)((waves + kBlock / 64 - 1) / (kBlock / 64)); }

template <typename PT, int VEC, int ACT> void fwd_launch(const NchwArgs &a, const NchwGeo &q) {
  A *part = (A *)a.ws;
  const unsigned grid = wave_grid(q.rows * q.chunks);
  launch(kKindNchwStats, (nchw_stats_kernel<elem_t, VEC>), dim3(grid), dim3(kBlock), a.stream, (const elem_t *)a.x, part, q);
  A *compact = nullptr;
  if ((int64_t)q.D * q.chunks > kNchwMergeInline) {  // many partials per slab: merge each slab once, not once per wavefront
    compact = part + nchw_partial_elems(a.N, a.C, a.R, VEC, false);
    launch(kKindNchwStats, (nchw_stats_compact_kernel<A>), dim3(wave_grid(q.N * q.G)), dim3(kBlock), a.stream, (const A *)part,
           compact, q);
  }
  launch(kKindNchwApply, (nchw_apply_kernel<elem_t, PT, VEC, ACT>), dim3(grid), dim3(kBlock), a.stream, (const elem_t *)a.x,
         (elem_t *)a.y, (const A *)part, (const A *)compact, a.w, a.b, a.mean_out, a.rstd_out, a.sdtype, (A)a.eps, q);
}
template <typename PT, int VEC, int ACT> void bwd_launch(const NchwArgs &a, const NchwGeo &q) {
  A *part = (A *)a.ws;
  const unsigned grid = wave_grid(q.rows * q.chunks);
  launch(kKindNchwBwdReduce, (nchw_bwd_reduce_kernel<elem_t, PT, VEC, ACT>), dim3(grid), dim3(kBlock), a.stream,
         (const elem_t *)a.x, (const elem_t *)a.dy, a.mean, a.rstd, a.sdtype, a.w, a.b, part, q);
  A *compact = nullptr;
  if ((int64_t)q.D * q.chunks > kNchwMergeInline) {
    compact = part + nchw_partial_elems(a.N, a.C, a.R, VEC, true);
    launch(kKindNchwBwdReduce, (nchw_bwd_compact_kernel<A, PT>), dim3(wave_grid(q.N * q.G)), dim3(kBlock), a.stream,
           (const A *)part, a.w, compact, q);
  }
  launch(kKindNchwBwdDx, (nchw_bwd_dx_kernel<elem_t, PT, VEC, ACT>), dim3(grid), dim3(kBlock), a.stream, (const elem_t *)a.x,
         (const elem_t *)a.dy, (elem_t *)a.dx, a.mean, a.rstd, a.sdtype, a.w, a.b, (const A *)part, (const A *)compact, a.dw,
         a.db, q);
}
template <typename PT, int VEC> void dispatch_act(const NchwArgs &a, const NchwGeo &q) {
  switch (a.act) {
    case GN_ACT_IDENTITY: a.backward ? bwd_launch<PT, VEC, GN_ACT_IDENTITY>(a, q) : fwd_launch<PT, VEC, GN_ACT_IDENTITY>(a, q); break;
    case GN_ACT_RELU: a.backward ? bwd_launch<PT, VEC, GN_ACT_RELU>(a, q) : fwd_launch<PT, VEC, GN_ACT_RELU>(a, q); break;
    case GN_ACT_SILU: a.backward ? bwd_launch<PT, VEC, GN_ACT_SILU>(a, q) : fwd_launch<PT, VEC, GN_ACT_SILU>(a, q); break;
    case GN_ACT_GELU: a.backward ? bwd_launch<PT, VEC, GN_ACT_GELU>(a, q) : fwd_launch<PT, VEC, GN_ACT_GELU>(a, q); break;
    default: a.backward ? bwd_launch<PT, VEC, GN_ACT_GELU_TANH>(a, q) : fwd_launch<PT, VEC, GN_ACT_GELU_TANH>(a, q); break;
  }
}
template <int VEC> void dispatch_pt(const NchwArgs &a) {
  const NchwGeo q = geometry(a, VEC);
  if (a.pdtype == GN_INST_DTYPE) dispatch_act<elem_t, VEC>(a, q);
  else dispatch_act<wide_param_t, VEC>(a, q);
}

}  // namespace

hipError_t GN_CAT(launch_nchw_, GN_SUFFIX)(const NchwArgs &a) {
  if (a.vector) dispatch_pt<kVec>(a);
  else dispatch_pt<1>(a);
  return hipGetLastError();
}

}  // namespace gn
