// The streaming GroupNorm kernels (templates; instantiated once per element type in gn_inst.hip).
//
//   forward : stats_kernel -> stats_finalize_kernel -> apply_kernel
//   backward: bwd_reduce_kernel -> bwd_finalize_kernel -> bwd_dx_kernel
//
// Every large kernel walks the same Plan: a workgroup owns a tile of consecutive rows of one sample,
// each lane owns VEC fixed channels and reads/writes them with one 128-bit access per row, so a
// wavefront touches whole contiguous rows.  Cross-lane and cross-workgroup reductions use fixed
// trees and per-tile partial buffers, never floating-point atomics, so results are bit-identical
// from run to run (the reference has the same property, it contains no atomics either).
#pragma once
#include "gn_device.h"

namespace gn {

template <typename T> using acc_t = typename acc_of<T>::type;

// rows of a tile of `len` rows handled by lane-row ty: ty, ty + rpi, ...
__device__ __forceinline__ int rows_of(int len, int rpi, int ty) { return len > ty ? (len - ty + rpi - 1) / rpi : 0; }

struct LanePos {
  TileCoord tc;
  int ty, tx, cvi;   // lane row, lane column inside the chunk, lane-vector index inside the row
  int len;           // rows in this tile
  int64_t row0;      // first row of the tile (inside the sample)
  bool active;
};
__device__ __forceinline__ LanePos lane_pos(const Plan &p, bool reversed) {
  LanePos l;
  l.tc = decode_block(p, blockIdx.x, reversed);
  const int tid = threadIdx.x;
  l.ty = tid / p.lpr;
  l.tx = tid - l.ty * p.lpr;
  l.cvi = l.tc.chunk * p.lpr + l.tx;
  l.row0 = (int64_t)l.tc.tile * p.tile_rows;
  const int64_t rem = p.R - l.row0;
  l.len = rem < p.tile_rows ? (int)rem : p.tile_rows;
  l.active = l.ty < p.rpi && l.cvi < p.cv;
  return l;
}

// a = rstd * gamma, b = beta - mean * a: normalise + affine as one FMA per element
// (same folding as src/gnnhwc/csrc/gn_kernel.cu:350-379, 601-602, 783-784).
template <typename A, int VEC>
__device__ __forceinline__ void affine_coeffs(const Plan &p, const LanePos &l, const void *mean, const void *rstd,
                                              int sdtype, const void *w, const void *b, int pdtype, A (&sa)[VEC],
                                              A (&sb)[VEC]) {
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int c = l.cvi * VEC + j;
    const int g = c / p.D;
    const int64_t ng = l.tc.n * p.G + g;
    const A mu = load_scalar<A>(mean, ng, sdtype);
    const A rs = load_scalar<A>(rstd, ng, sdtype);
    const A gamma = w ? load_scalar<A>(w, c, pdtype) : (A)1;
    const A beta = b ? load_scalar<A>(b, c, pdtype) : (A)0;
    sa[j] = rs * gamma;
    sb[j] = beta - mu * sa[j];
  }
}

// ---------------------------------------------------------------------------------------------
// Forward pass 1: per-tile (count, mean, M2) of every group the tile touches.
// Does the work of compute_stats_pt1 (src/gnnhwc/csrc/gn_kernel.cu:132-224).  Each lane folds
// kUnroll rows at a time with an exact two-pass mean / sum-of-squares on the values it holds in
// registers and merges that block into its running moments (one reciprocal per kUnroll rows instead
// of the per-element division of WelfordOps::reduce, Welford.h:30-42).
//   part : [N][tiles][nchunk][G][3] accumulation type; only the groups a chunk intersects are written.
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void stats_kernel(const T *__restrict__ x, acc_t<T> *__restrict__ part, Plan p) {
  using A = acc_t<T>;
  __shared__ A sm_mean[kBlock * VEC];
  __shared__ A sm_m2[kBlock * VEC];
  const LanePos l = lane_pos(p, false);
  const int W = p.lpr * VEC;

  if (l.active) {
    A mean[VEC], m2[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) { mean[j] = (A)0; m2[j] = (A)0; }
    A cnt = (A)0;
    const T *px = x + ((l.tc.n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC);
    const int64_t step = (int64_t)p.rpi * p.C;
    int lr = l.ty;
    for (; lr + (kUnroll - 1) * p.rpi < l.len; lr += kUnroll * p.rpi) {
      A v[kUnroll][VEC];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) LaneVec<T, VEC, false>::load(px + u * step, v[u]);
      px += kUnroll * step;
      const A n = cnt + (A)kUnroll;
      const A f = (A)kUnroll * fast_rcp(n);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        A s = v[0][j];
#pragma unroll
        for (int u = 1; u < kUnroll; ++u) s += v[u][j];
        const A mb = s * ((A)1 / (A)kUnroll);
        A q = (A)0;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) { const A d = v[u][j] - mb; q += d * d; }
        const A d = mb - mean[j];
        mean[j] += d * f;
        m2[j] += q + d * d * cnt * f;
      }
      cnt = n;
    }
    for (; lr < l.len; lr += p.rpi) {
      A v[VEC];
      LaneVec<T, VEC, false>::load(px, v);
      px += step;
      cnt += (A)1;
      const A inv = fast_rcp(cnt);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const A d = v[j] - mean[j];
        mean[j] += d * inv;
        m2[j] += d * (v[j] - mean[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      sm_mean[l.ty * W + l.tx * VEC + j] = mean[j];
      sm_m2[l.ty * W + l.tx * VEC + j] = m2[j];
    }
  }
  __syncthreads();

  // merge the per-(lane row, channel) moments of each group this chunk intersects: 16 lanes per group
  const int cstart = l.tc.chunk * p.lpr * VEC;
  const int lanes_here = p.cv - l.tc.chunk * p.lpr < p.lpr ? p.cv - l.tc.chunk * p.lpr : p.lpr;
  const int cend = cstart + lanes_here * VEC;
  const int g_lo = cstart / p.D, g_hi = (cend - 1) / p.D;
  const int ng = g_hi - g_lo + 1;
  constexpr int L = 16;
  constexpr int NSUB = kBlock / L;
  const int sub = threadIdx.x / L, sl = threadIdx.x % L;
  for (int base = 0; base < ng; base += NSUB) {
    const int gi = base + sub;
    const int g = g_lo + gi;
    Moments<A> m = {(A)0, (A)0, (A)0};
    if (gi < ng) {
      const int ca = (g * p.D > cstart ? g * p.D : cstart) - cstart;
      const int cb = ((g + 1) * p.D < cend ? (g + 1) * p.D : cend) - cstart;
      for (int ety = 0; ety < p.rpi; ++ety) {
        const int rc = rows_of(l.len, p.rpi, ety);
        if (rc == 0) break;
        for (int c = ca + sl; c < cb; c += L) {
          const Moments<A> e = {(A)rc, sm_mean[ety * W + c], sm_m2[ety * W + c]};
          m = merge(m, e);
        }
      }
    }
    m = segment_merge(m, L);
    if (gi < ng && sl == 0) {
      const int64_t slot = ((l.tc.n * p.tiles + l.tc.tile) * p.nchunk + l.tc.chunk) * p.G + g;
      part[slot * 3 + 0] = m.n;
      part[slot * 3 + 1] = m.mean;
      part[slot * 3 + 2] = m.m2;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Forward pass 2: merge the tile partials of one (n, g) per wavefront, in slot order, and produce
// mean and rstd = 1 / sqrt(M2 / n + eps).  Does the work of compute_stats_pt2
// (src/gnnhwc/csrc/gn_kernel.cu:226-292), except that the accumulation-type copies kept in the
// workspace (ws_mean / ws_rstd) feed the apply kernel, so rounding mean / rstd to a 16-bit output
// type (gn_kernel.cu:290-291) does not touch y.
// ---------------------------------------------------------------------------------------------
template <typename A>
__global__ __launch_bounds__(kBlock) void stats_finalize_kernel(const A *__restrict__ part, A *__restrict__ ws_mean,
                                                                A *__restrict__ ws_rstd, void *mean_out, void *rstd_out,
                                                                int sdtype, A eps, Plan p) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (kBlock / 64) + wave;
  const bool valid = item < p.N * p.G;
  Moments<A> m = {(A)0, (A)0, (A)0};
  if (valid) {
    const int64_t n = item / p.G;
    const int g = (int)(item - n * p.G);
    const int chunk_w = p.lpr * p.vec;
    const int k_lo = (g * p.D) / chunk_w, k_hi = ((g + 1) * p.D - 1) / chunk_w;
    const int nk = k_hi - k_lo + 1;
    const int entries = p.tiles * nk;
    for (int e = lane; e < entries; e += 64) {
      const int t = e / nk, k = k_lo + (e - t * nk);
      const int64_t slot = ((n * p.tiles + t) * p.nchunk + k) * p.G + g;
      const Moments<A> q = {part[slot * 3 + 0], part[slot * 3 + 1], part[slot * 3 + 2]};
      m = merge(m, q);
    }
  }
  m = segment_merge(m, 64);
  if (valid && lane == 0) {
    const A var = m.m2 / m.n;
    const A rs = (A)1 / sqrt(var + eps);
    ws_mean[item] = m.mean;
    ws_rstd[item] = rs;
    store_scalar<A>(mean_out, item, sdtype, m.mean);
    store_scalar<A>(rstd_out, item, sdtype, rs);
  }
}

// ---------------------------------------------------------------------------------------------
// Forward pass 3: y = act(x * a + b).  Does the work of scale_shift_kernel
// (src/gnnhwc/csrc/gn_kernel.cu:305-412) for every shape with one code path (no R % 8 fast / slow split).
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void apply_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                       const acc_t<T> *__restrict__ ws_mean,
                                                       const acc_t<T> *__restrict__ ws_rstd, const void *w, const void *b,
                                                       int pdtype, Plan p) {
  using A = acc_t<T>;
  const LanePos l = lane_pos(p, true);
  if (!l.active) return;
  constexpr int acc_dtype = sizeof(A) == 8 ? GN_F64 : GN_F32;
  A sa[VEC], sb[VEC];
  affine_coeffs<A, VEC>(p, l, ws_mean, ws_rstd, acc_dtype, w, b, pdtype, sa, sb);
  const int64_t off = (l.tc.n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
  const T *px = x + off;
  T *py = y + off;
  const int64_t step = (int64_t)p.rpi * p.C;
  int lr = l.ty;
  for (; lr + (kUnroll - 1) * p.rpi < l.len; lr += kUnroll * p.rpi) {
    A v[kUnroll][VEC];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) LaneVec<T, VEC, true>::load(px + u * step, v[u]);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[u][j] = act_fwd<ACT, A>(v[u][j] * sa[j] + sb[j]);
      LaneVec<T, VEC, true>::store(py + u * step, v[u]);
    }
    px += kUnroll * step;
    py += kUnroll * step;
  }
  for (; lr < l.len; lr += p.rpi) {
    A v[VEC];
    LaneVec<T, VEC, true>::load(px, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = act_fwd<ACT, A>(v[j] * sa[j] + sb[j]);
    LaneVec<T, VEC, true>::store(py, v);
    px += step;
    py += step;
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 1: per-tile, per-channel S1 = sum g * x and S2 = sum g with g = dy * act'(x a + b)
// recomputed from x.  Does the work of width_reduce (src/gnnhwc/csrc/gn_kernel.cu:557-646).
//   part : [N][tiles][C][2] accumulation type.
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void bwd_reduce_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                            const void *mean, const void *rstd, int sdtype, const void *w,
                                                            const void *b, int pdtype, acc_t<T> *__restrict__ part,
                                                            Plan p) {
  using A = acc_t<T>;
  __shared__ A sm1[kBlock * VEC];
  __shared__ A sm2[kBlock * VEC];
  const LanePos l = lane_pos(p, false);
  const int W = p.lpr * VEC;
  if (l.active) {
    A sa[VEC], sb[VEC], s1[VEC], s2[VEC];
    affine_coeffs<A, VEC>(p, l, mean, rstd, sdtype, w, b, pdtype, sa, sb);
#pragma unroll
    for (int j = 0; j < VEC; ++j) { s1[j] = (A)0; s2[j] = (A)0; }
    const int64_t off = (l.tc.n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
    const T *px = x + off;
    const T *pdy = dy + off;
    const int64_t step = (int64_t)p.rpi * p.C;
    int lr = l.ty;
    for (; lr + (kUnroll - 1) * p.rpi < l.len; lr += kUnroll * p.rpi) {
      A vx[kUnroll][VEC], vd[kUnroll][VEC];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        LaneVec<T, VEC, false>::load(px + u * step, vx[u]);
        LaneVec<T, VEC, false>::load(pdy + u * step, vd[u]);
      }
      px += kUnroll * step;
      pdy += kUnroll * step;
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const A g = vd[u][j] * act_bwd<ACT, A>(vx[u][j] * sa[j] + sb[j]);
          s1[j] += g * vx[u][j];
          s2[j] += g;
        }
      }
    }
    for (; lr < l.len; lr += p.rpi) {
      A vx[VEC], vd[VEC];
      LaneVec<T, VEC, false>::load(px, vx);
      LaneVec<T, VEC, false>::load(pdy, vd);
      px += step;
      pdy += step;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const A g = vd[j] * act_bwd<ACT, A>(vx[j] * sa[j] + sb[j]);
        s1[j] += g * vx[j];
        s2[j] += g;
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      sm1[l.ty * W + l.tx * VEC + j] = s1[j];
      sm2[l.ty * W + l.tx * VEC + j] = s2[j];
    }
  }
  __syncthreads();
  const int cstart = l.tc.chunk * p.lpr * VEC;
  const int lanes_here = p.cv - l.tc.chunk * p.lpr < p.lpr ? p.cv - l.tc.chunk * p.lpr : p.lpr;
  const int wch = lanes_here * VEC;
  for (int c = threadIdx.x; c < wch; c += kBlock) {
    A t1 = (A)0, t2 = (A)0;
    for (int ety = 0; ety < p.rpi; ++ety) {
      t1 += sm1[ety * W + c];
      t2 += sm2[ety * W + c];
    }
    const int64_t idx = ((l.tc.n * p.tiles + l.tc.tile) * p.C + cstart + c) * 2;
    part[idx] = t1;
    part[idx + 1] = t2;
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 2, one workgroup per (n, g): sum the tile partials of the group's channels
// (height_reduce, src/gnnhwc/csrc/gn_kernel.cu:648-693), then
//   A = sum_c gamma_c S1_c, B = sum_c gamma_c S2_c, s = 1 / (D R),
//   coef1 = (mean B - A) s rstd^3, coef2 = -mean coef1 - B s rstd
// (compute_bwd_scale_biases, gn_kernel.cu:730-801).
//   sums : [N][C][2]   coef : [N][G][2]
// ---------------------------------------------------------------------------------------------
template <typename A>
__global__ __launch_bounds__(kBlock) void bwd_finalize_kernel(const A *__restrict__ part, const void *mean,
                                                              const void *rstd, int sdtype, const void *w, int pdtype,
                                                              A *__restrict__ sums, A *__restrict__ coef, Plan p) {
  __shared__ A red[2 * (kBlock / 64)];
  const int64_t n = blockIdx.x / p.G;
  const int g = (int)(blockIdx.x - n * p.G);
  int L = 1;
  while (L < p.tiles && L < 64) L <<= 1;
  const int per_pass = kBlock / L;
  const int sub = threadIdx.x / L, sl = threadIdx.x % L;
  A ga = (A)0, gb = (A)0;  // this thread's share of A and B (only segment leaders contribute)
  for (int base = 0; base < p.D; base += per_pass) {
    const int i = base + sub;
    A s1 = (A)0, s2 = (A)0;
    const int c = g * p.D + i;
    if (i < p.D) {
      for (int t = sl; t < p.tiles; t += L) {
        const int64_t idx = ((n * p.tiles + t) * p.C + c) * 2;
        s1 += part[idx];
        s2 += part[idx + 1];
      }
    }
    s1 = segment_sum(s1, L);
    s2 = segment_sum(s2, L);
    if (i < p.D && sl == 0) {
      sums[(n * p.C + c) * 2] = s1;
      sums[(n * p.C + c) * 2 + 1] = s2;
      const A gamma = w ? load_scalar<A>(w, c, pdtype) : (A)1;
      ga += gamma * s1;
      gb += gamma * s2;
    }
  }
  ga = segment_sum(ga, 64);
  gb = segment_sum(gb, 64);
  if ((threadIdx.x & 63) == 0) {
    red[2 * (threadIdx.x >> 6)] = ga;
    red[2 * (threadIdx.x >> 6) + 1] = gb;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    A ta = (A)0, tb = (A)0;
    for (int wv = 0; wv < kBlock / 64; ++wv) { ta += red[2 * wv]; tb += red[2 * wv + 1]; }
    const int64_t ng = n * p.G + g;
    const A mu = load_scalar<A>(mean, ng, sdtype);
    const A rs = load_scalar<A>(rstd, ng, sdtype);
    const A s = (A)1 / ((A)p.D * (A)p.R);
    const A c1 = (mu * tb - ta) * s * rs * rs * rs;
    coef[ng * 2] = c1;
    coef[ng * 2 + 1] = -mu * c1 - tb * s * rs;
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 3: dx = a g + coef1 x + coef2 with g recomputed as in pass 1.  Does the work of
// dx_elem_kernel (src/gnnhwc/csrc/gn_kernel.cu:803-905).  The last ceil(C / 256) workgroups of the grid
// instead produce dgamma_c = sum_n (S1 - mean S2) rstd and dbeta_c = sum_n S2
// (compute_dweight_dbias, gn_kernel.cu:695-728).
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) void bwd_dx_kernel(const T *__restrict__ x, const T *__restrict__ dy,
                                                        T *__restrict__ dx, const void *mean, const void *rstd,
                                                        int sdtype, const void *w, const void *b, int pdtype,
                                                        const acc_t<T> *__restrict__ sums,
                                                        const acc_t<T> *__restrict__ coef, void *dw, void *db, Plan p) {
  using A = acc_t<T>;
  if ((int64_t)blockIdx.x >= p.nblocks) {
    const int64_t c = ((int64_t)blockIdx.x - p.nblocks) * kBlock + threadIdx.x;
    if (c < p.C) {
      const int g = (int)(c / p.D);
      A t1 = (A)0, t2 = (A)0;
      for (int64_t n = 0; n < p.N; ++n) {
        const A mu = load_scalar<A>(mean, n * p.G + g, sdtype);
        const A rs = load_scalar<A>(rstd, n * p.G + g, sdtype);
        const A s1 = sums[(n * p.C + c) * 2], s2 = sums[(n * p.C + c) * 2 + 1];
        t1 += (s1 - mu * s2) * rs;
        t2 += s2;
      }
      if (dw) store_scalar<A>(dw, c, pdtype, t1);
      if (db) store_scalar<A>(db, c, pdtype, t2);
    }
    return;
  }
  const LanePos l = lane_pos(p, true);
  if (!l.active) return;
  A sa[VEC], sb[VEC], c1[VEC], c2[VEC];
  affine_coeffs<A, VEC>(p, l, mean, rstd, sdtype, w, b, pdtype, sa, sb);
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const int g = (l.cvi * VEC + j) / p.D;
    c1[j] = coef[(l.tc.n * p.G + g) * 2];
    c2[j] = coef[(l.tc.n * p.G + g) * 2 + 1];
  }
  const int64_t off = (l.tc.n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
  const T *px = x + off;
  const T *pdy = dy + off;
  T *pdx = dx + off;
  const int64_t step = (int64_t)p.rpi * p.C;
  int lr = l.ty;
  for (; lr + (kUnroll - 1) * p.rpi < l.len; lr += kUnroll * p.rpi) {
    A vx[kUnroll][VEC], vd[kUnroll][VEC];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      LaneVec<T, VEC, true>::load(px + u * step, vx[u]);
      LaneVec<T, VEC, true>::load(pdy + u * step, vd[u]);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const A g = vd[u][j] * act_bwd<ACT, A>(vx[u][j] * sa[j] + sb[j]);
        vd[u][j] = sa[j] * g + (c1[j] * vx[u][j] + c2[j]);
      }
      LaneVec<T, VEC, true>::store(pdx + u * step, vd[u]);
    }
    px += kUnroll * step;
    pdy += kUnroll * step;
    pdx += kUnroll * step;
  }
  for (; lr < l.len; lr += p.rpi) {
    A vx[VEC], vd[VEC];
    LaneVec<T, VEC, true>::load(px, vx);
    LaneVec<T, VEC, true>::load(pdy, vd);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A g = vd[j] * act_bwd<ACT, A>(vx[j] * sa[j] + sb[j]);
      vd[j] = sa[j] * g + (c1[j] * vx[j] + c2[j]);
    }
    LaneVec<T, VEC, true>::store(pdx, vd);
    px += step;
    pdy += step;
    pdx += step;
  }
}

}  // namespace gn
