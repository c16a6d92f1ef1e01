// Channels-first (N, C, R contiguous, R fastest) GroupNorm + activation, forward and backward.
//
// The reference has no kernel for this layout: GN_NHWC.forward hands channels-first input to torch's GroupNorm
// and applies the activation in a second pass (src/gnnhwc/custom_gn.py:75-79).  Here the same result comes from
// two launches forward (x is read twice, y written once) and two backward, with the activation fused.
//
// In this layout a (sample, group) slab is D * R contiguous elements and a channel is a contiguous row of R, so
// the unit of work is one wavefront on one chunk of one row: its 64 lanes read consecutive 16-byte vectors, every
// element of the chunk shares gamma / beta / mean / rstd, and the chunk's sums reduce inside the wavefront with
// DPP moves -- no LDS, no barriers.  Partial results are laid out [N * C][chunks] so that the partials of a slab
// (D consecutive rows) are one contiguous run.  The algebra is that of the channels-last kernels
// (gn_kernel.cu:598-618, 717-727, 783-800, 868-871; Welford.h:8-21,66-72 for the statistics).
#pragma once
#include "gn_kernels.h"

namespace gn {

constexpr int kNchwUnroll = 4;  // lane vectors of a chunk per lane
struct NchwGeo {
  int64_t N, C, R;
  int G, D;
  int chunk_len;  // elements per chunk = 64 * VEC * kNchwUnroll
  int chunks;     // chunks per row = ceil(R / chunk_len)
  int64_t rows;   // N * C
};

// The chunk this wavefront works on; false past the end of the grid.
struct NchwPos {
  int64_t row;  // n * C + c
  int64_t n;
  int c, g, k, lane;
  int64_t base;  // element offset of the row
  int e0;        // first element of the chunk inside the row
};
__device__ __forceinline__ bool nchw_pos(const NchwGeo &q, NchwPos &p) {
  const int64_t wid = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (wid >= q.rows * q.chunks) return false;
  p.row = wid / q.chunks;
  p.k = (int)(wid - p.row * q.chunks);
  p.n = p.row / q.C;
  p.c = (int)(p.row - p.n * q.C);
  p.g = p.c / q.D;
  p.lane = threadIdx.x & 63;
  p.base = p.row * q.R;
  p.e0 = p.k * q.chunk_len;
  return true;
}
// Element index (inside the row) of lane vector u of this lane, and whether it lies inside the row.
template <int VEC> __device__ __forceinline__ int nchw_elem(const NchwPos &p, int u) { return p.e0 + (u * 64 + p.lane) * VEC; }

// ---------------------------------------------------------------------------------------------
// Forward pass 1: (count, mean, M2) of every chunk.   part: 3 planes [N * C][chunks]
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void nchw_stats_kernel(const T *__restrict__ x, acc_t<T> *__restrict__ part, NchwGeo q) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  NchwPos p;
  if (!nchw_pos(q, p)) return;
  const T *row = x + p.base;
  typename LV::raw_t buf[kNchwUnroll];
  const int last = (int)((q.R - 1) / VEC * VEC);  // a vector that is certainly inside the row
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const int e = nchw_elem<VEC>(p, u);
    buf[u] = LV::load(row + (e < q.R ? e : last));
  }
  // sums about the chunk's first element: it lies inside the data, so nothing cancels
  A pv[VEC];
  LV::unpack(LV::load(row + p.e0), pv);
  const A K = pv[0];
  A s1 = (A)0, s2 = (A)0, cnt = (A)0;
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const bool in = nchw_elem<VEC>(p, u) < q.R;
    A v[VEC];
    LV::unpack(buf[u], v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A d = in ? v[j] - K : (A)0;
      s1 += d;
      s2 += d * d;
    }
    cnt += in ? (A)VEC : (A)0;
  }
  segment_sum2(s1, s2, 64);
  cnt = segment_sum(cnt, 64);
  if (p.lane == 0) {
    const int64_t plane = q.rows * q.chunks;
    const int64_t slot = p.row * q.chunks + p.k;
    const A dm = s1 * fast_rcp(cnt);
    part[slot] = cnt;
    part[plane + slot] = K + dm;
    part[2 * plane + slot] = s2 - s1 * dm;
  }
}

// Merge the D * chunks partial triples of slab (n, g) with the 64 lanes of a wavefront (pivot form of the exact
// two-pass merge); every lane returns the slab's mean and M2.
template <typename A>
__device__ __forceinline__ void nchw_merge_slab(const A *__restrict__ part, const NchwGeo &q, int64_t n, int g, int lane,
                                                A &mean, A &m2) {
  const int64_t plane = q.rows * q.chunks;
  const int64_t first = (n * q.C + (int64_t)g * q.D) * q.chunks;
  const int64_t P = (int64_t)q.D * q.chunks;
  A nl = (A)0, kl = (A)0, s1 = (A)0, s2 = (A)0;
  for (int64_t i = lane; i < P; i += 64) {
    const A cn = part[first + i], mu = part[plane + first + i], mm = part[2 * plane + first + i];
    if (nl == (A)0) kl = mu;
    const A d = mu - kl;
    nl += cn;
    s1 += cn * d;
    s2 += mm + cn * d * d;
  }
  const A inv = nl > (A)0 ? fast_rcp(nl) : (A)0;
  const A mean_l = kl + s1 * inv;
  const A m2_l = s2 - s1 * s1 * inv;
  const A K = __shfl(mean_l, 0, 64);  // lane 0 always has an entry
  const A d = mean_l - K;
  A t0 = nl, t1 = nl * d, t2 = m2_l + nl * d * d;
  t0 = segment_sum(t0, 64);
  segment_sum2(t1, t2, 64);
  const A dm = t1 * fast_rcp(t0);
  mean = K + dm;
  m2 = t2 - t1 * dm;
}

// A slab has D * chunks partials and as many wavefronts, each of which needs the slab's merged result: merged by every
// wavefront in its own prologue that is D * chunks reads per wavefront, fine for the usual few dozen (one launch
// saved) and quadratic for one group of many long rows.  Beyond kNchwMergeInline partials per slab a compaction launch
// of one wavefront per slab runs in between and leaves one record per slab, which the consumers read instead.
constexpr int kNchwMergeInline = 256;
// forward: (mean, M2) per slab -> out: 2 planes [N * G]
template <typename A>
__global__ __launch_bounds__(kBlock) void nchw_stats_compact_kernel(const A *__restrict__ part, A *__restrict__ out, NchwGeo q) {
  const int64_t item = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (item >= q.N * q.G) return;
  const int64_t n = item / q.G;
  A mean, m2;
  nchw_merge_slab<A>(part, q, n, (int)(item - n * q.G), threadIdx.x & 63, mean, m2);
  if ((threadIdx.x & 63) == 0) {
    out[item] = mean;
    out[q.N * q.G + item] = m2;
  }
}
// The slab's group sums A = sum_c gamma_c S1_c and B = sum_c gamma_c S2_c from its D * chunks partials (64 lanes).
template <typename A, typename PT>
__device__ __forceinline__ void nchw_group_sums(const A *__restrict__ part, const void *w, const NchwGeo &q, int64_t n, int g,
                                                int lane, A &ta, A &tb) {
  const int64_t plane = q.rows * q.chunks;
  const int64_t first = (n * q.C + (int64_t)g * q.D) * q.chunks;
  const int64_t P = (int64_t)q.D * q.chunks;
  ta = (A)0;
  tb = (A)0;
  for (int64_t i = lane; i < P; i += 64) {
    const int cl = (int)(i / q.chunks);
    const A gm = w ? load_param<PT, A>(w, g * q.D + cl) : (A)1;
    ta += gm * part[first + i];
    tb += gm * part[plane + first + i];
  }
  segment_sum2(ta, tb, 64);
}
// backward: (A, B) per slab -> out: 2 planes [N * G]
template <typename A, typename PT>
__global__ __launch_bounds__(kBlock) void nchw_bwd_compact_kernel(const A *__restrict__ part, const void *w, A *__restrict__ out,
                                                                  NchwGeo q) {
  const int64_t item = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (item >= q.N * q.G) return;
  const int64_t n = item / q.G;
  A ta, tb;
  nchw_group_sums<A, PT>(part, w, q, n, (int)(item - n * q.G), threadIdx.x & 63, ta, tb);
  if ((threadIdx.x & 63) == 0) {
    out[item] = ta;
    out[q.N * q.G + item] = tb;
  }
}

// ---------------------------------------------------------------------------------------------
// Forward pass 2: every wavefront merges its slab's partials (or reads the slab's compacted record), then y = act(x * a + b) on its chunk with
// a = rstd * gamma_c, b = beta_c - mean * a.  The wavefront on the first chunk of a slab reports mean / rstd.
// ---------------------------------------------------------------------------------------------
template <typename T, typename PT, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void nchw_apply_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                            const acc_t<T> *__restrict__ part, const acc_t<T> *__restrict__ compact,
                                                            const void *w, const void *b, void *mean_out, void *rstd_out,
                                                            int sdtype, acc_t<T> eps, NchwGeo q) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  NchwPos p;
  if (!nchw_pos(q, p)) return;
  const T *row = x + p.base;
  typename LV::raw_t buf[kNchwUnroll];
  const int last = (int)((q.R - 1) / VEC * VEC);
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const int e = nchw_elem<VEC>(p, u);
    buf[u] = LV::load(row + (e < q.R ? e : last));
  }
  const A gamma = w ? load_param<PT, A>(w, p.c) : (A)1;
  const A beta = b ? load_param<PT, A>(b, p.c) : (A)0;
  A mean, m2;
  if (compact) {
    mean = compact[p.n * q.G + p.g];
    m2 = compact[q.N * q.G + p.n * q.G + p.g];
  } else {
    nchw_merge_slab<A>(part, q, p.n, p.g, p.lane, mean, m2);
  }
  const A rs = fast_rsqrt(m2 * fast_rcp((A)q.D * (A)q.R) + eps);
  if (p.lane == 0 && p.k == 0 && p.c == p.g * q.D) {
    if (mean_out) store_scalar<A>(mean_out, p.n * q.G + p.g, sdtype, mean);
    if (rstd_out) store_scalar<A>(rstd_out, p.n * q.G + p.g, sdtype, rs);
  }
  const A sa = rs * gamma, sb = beta - mean * sa;
  T *out = y + p.base;
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const int e = nchw_elem<VEC>(p, u);
    if (e < q.R) {
      A v[VEC];
      LV::unpack(buf[u], v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = act_fwd<ACT, A>(v[j] * sa + sb);
      store_streaming<LV>(out + e, LV::pack(v));
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 1: S1 = sum g' x and S2 = sum g' of every chunk, g' = dy * act'(x a + b).
//   part: 2 planes [N * C][chunks]
// ---------------------------------------------------------------------------------------------
template <typename T, typename PT, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void nchw_bwd_reduce_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                                 const void *mean, const void *rstd, int sdtype, const void *w,
                                                                 const void *b, acc_t<T> *__restrict__ part, NchwGeo q) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  NchwPos p;
  if (!nchw_pos(q, p)) return;
  typename LV::raw_t bx[kNchwUnroll], bd[kNchwUnroll];
  const int last = (int)((q.R - 1) / VEC * VEC);
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const int e = nchw_elem<VEC>(p, u);
    const int64_t o = p.base + (e < q.R ? e : last);
    bx[u] = LV::load(x + o);
    bd[u] = LV::load(dy + o);
  }
  const A gamma = w ? load_param<PT, A>(w, p.c) : (A)1;
  const A beta = b ? load_param<PT, A>(b, p.c) : (A)0;
  const A mu = load_scalar<A>(mean, p.n * q.G + p.g, sdtype);
  const A rs = load_scalar<A>(rstd, p.n * q.G + p.g, sdtype);
  const A sa = rs * gamma, sb = beta - mu * sa;
  A s1 = (A)0, s2 = (A)0;
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const bool in = nchw_elem<VEC>(p, u) < q.R;
    A vx[VEC], vd[VEC];
    LV::unpack(bx[u], vx);
    LV::unpack(bd[u], vd);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A g = in ? vd[j] * act_bwd<ACT, A>(vx[j] * sa + sb) : (A)0;
      s1 += g * vx[j];
      s2 += g;
    }
  }
  segment_sum2(s1, s2, 64);
  if (p.lane == 0) {
    const int64_t slot = p.row * q.chunks + p.k;
    part[slot] = s1;
    part[q.rows * q.chunks + slot] = s2;
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 2: dx = a g' + coef1 x + coef2 with the group coefficients of compute_bwd_scale_biases
// (gn_kernel.cu:786-800), which every wavefront rebuilds from its slab's partials:
//   A = sum_c gamma_c S1_c,  B = sum_c gamma_c S2_c,  s = 1 / (D R),
//   coef1 = (mean B - A) s rstd^3,  coef2 = -mean coef1 - B s rstd.
// ---------------------------------------------------------------------------------------------
template <typename T, typename PT, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void nchw_bwd_dx_kernel(const T *__restrict__ x, const T *__restrict__ dy, T *__restrict__ dx,
                                                             const void *mean, const void *rstd, int sdtype, const void *w,
                                                             const void *b, const acc_t<T> *__restrict__ part,
                                                             const acc_t<T> *__restrict__ compact, void *dw, void *db, NchwGeo q) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  NchwPos p;
  if (!nchw_pos(q, p)) return;
  typename LV::raw_t bx[kNchwUnroll], bd[kNchwUnroll];
  const int last = (int)((q.R - 1) / VEC * VEC);
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const int e = nchw_elem<VEC>(p, u);
    const int64_t o = p.base + (e < q.R ? e : last);
    bx[u] = LV::load(x + o);
    bd[u] = LV::load(dy + o);
  }
  const A gamma = w ? load_param<PT, A>(w, p.c) : (A)1;
  const A beta = b ? load_param<PT, A>(b, p.c) : (A)0;
  const A mu = load_scalar<A>(mean, p.n * q.G + p.g, sdtype);
  const A rs = load_scalar<A>(rstd, p.n * q.G + p.g, sdtype);
  // dgamma_c = sum_n (S1 - mean S2) rstd and dbeta_c = sum_n S2 (compute_dweight_dbias, gn_kernel.cu:695-728) over
  // the N * chunks partials of channel c: the wavefront on the channel's first chunk in the first sample does it
  if (p.n == 0 && p.k == 0 && (dw || db)) {
    const int64_t plane = q.rows * q.chunks;
    A t1 = (A)0, t2 = (A)0;
    const int64_t entries = q.N * q.chunks;
    for (int64_t i = p.lane; i < entries; i += 64) {
      const int64_t nn = i / q.chunks;
      const int kk = (int)(i - nn * q.chunks);
      const int64_t slot = (nn * q.C + p.c) * q.chunks + kk;
      const A s1 = part[slot], s2 = part[plane + slot];
      const A m = load_scalar<A>(mean, nn * q.G + p.g, sdtype);
      const A r = load_scalar<A>(rstd, nn * q.G + p.g, sdtype);
      t1 += (s1 - m * s2) * r;
      t2 += s2;
    }
    segment_sum2(t1, t2, 64);
    if (p.lane == 0) {
      if (dw) store_param<PT, A>(dw, p.c, t1);
      if (db) store_param<PT, A>(db, p.c, t2);
    }
  }
  // group sums from the slab's D * chunks partials (or the slab's compacted record)
  A ta, tb;
  if (compact) {
    ta = compact[p.n * q.G + p.g];
    tb = compact[q.N * q.G + p.n * q.G + p.g];
  } else {
    nchw_group_sums<A, PT>(part, w, q, p.n, p.g, p.lane, ta, tb);
  }
  const A s = fast_rcp((A)q.D * (A)q.R);
  const A c1 = (mu * tb - ta) * s * rs * rs * rs;
  const A c2 = -mu * c1 - tb * s * rs;
  const A sa = rs * gamma, sb = beta - mu * sa;
  T *out = dx + p.base;
#pragma unroll
  for (int u = 0; u < kNchwUnroll; ++u) {
    const int e = nchw_elem<VEC>(p, u);
    if (e < q.R) {
      A vx[VEC], vd[VEC];
      LV::unpack(bx[u], vx);
      LV::unpack(bd[u], vd);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const A g = vd[j] * act_bwd<ACT, A>(vx[j] * sa + sb);
        vd[j] = sa * g + (c1 * vx[j] + c2);
      }
      store_streaming<LV>(out + e, LV::pack(vd));
    }
  }
}

}  // namespace gn
