// The streaming GroupNorm kernels (templates; instantiated once per element type in gn_inst.hip).
//
//   forward : stats_kernel -> [stats_compact_kernel] -> apply_kernel
//   backward: bwd_reduce_kernel -> [bwd_compact_kernel] -> bwd_dx_kernel
//
// Every large kernel walks the same Plan: a workgroup owns a tile of consecutive rows of one sample and
// a chunk of whole 128-byte lines of each row; each lane owns VEC fixed channels and moves them with
// one 128-bit access per row, two batches of rows in flight at a time.  The producers (stats,
// bwd_reduce) leave one partial result per tile; the consumers (apply, bwd_dx) merge the partials of
// the groups they touch in their own prologue, while their first loads are already in flight, so there
// is no separate finalize launch unless a sample has so many tiles that the merge is first compacted
// by the bracketed kernels.  All reductions use fixed trees and per-tile buffers, never floating-point
// atomics: results are bit-identical from run to run (the reference has the same property, it contains
// no atomics either).
#pragma once
#include <type_traits>

#include "gn_device.h"

namespace gn {

template <typename T> using acc_t = typename acc_of<T>::type;

struct LanePos {
  int64_t n;
  int tile, chunk;
  int ty, tx, cvi;   // lane row, lane column inside the chunk, lane-vector index inside the row
  int len;           // rows in this tile
  int64_t row0;      // first row of the tile (inside the sample)
  int cstart, wch;   // first channel and number of channels of this chunk
  int g_lo, ng;      // first group and number of groups the chunk intersects
  int rows_base, rows_rem;  // lane row ty owns rows_base + (ty < rows_rem) rows of the tile
  int rows;          // rows of the tile this lane owns (0 for an idle lane)
  bool active;
};
// `reversed` walks the row tiles from the far end in blocks of eight: the second pass of a two-pass
// operation then starts on the tiles the first pass touched last, while tile t stays on XCD t mod 8.
// `salt` is zero.  A caller that needs the position a second time, late in a kernel, passes a zero the compiler
// cannot see through, so that the position is computed again there instead of being kept in registers all the way.
// POW2: the chunk width p.lpr (and with it p.rpi) is known to be a power of two: shifts instead of divisions, and the two
// divisors need not be loaded.
template <bool POW2 = false>
__device__ __forceinline__ LanePos lane_pos(const Plan &p, int64_t n, bool reversed, int salt = 0) {
  LanePos l;
  l.n = n;
  int t = blockIdx.x + salt;
  if (reversed) {
    const int full = p.tiles & ~7;
    if (t < full) t = full - 8 - (t & ~7) + (t & 7);
  }
  l.tile = t;
  l.chunk = blockIdx.y + salt;
  const int tid = threadIdx.x + salt;
  const int lpr_log2 = __builtin_ctz(p.lpr);
  l.ty = POW2 ? tid >> lpr_log2 : div_by(tid, p.by_lpr);
  l.tx = POW2 ? tid & (p.lpr - 1) : tid - l.ty * p.lpr;
  l.cvi = l.chunk * p.lpr + l.tx;
  l.row0 = (int64_t)l.tile * p.tile_rows;
  const int64_t rem = p.R - l.row0;
  l.len = rem < p.tile_rows ? (int)rem : p.tile_rows;
  l.rows_base = POW2 ? l.len >> __builtin_ctz(p.rpi) : div_by(l.len, p.by_rpi);
  l.rows_rem = POW2 ? l.len & (p.rpi - 1) : l.len - l.rows_base * p.rpi;
  l.cstart = l.chunk * p.lpr * p.vec;
  const int lanes_here = p.cv - l.chunk * p.lpr < p.lpr ? p.cv - l.chunk * p.lpr : p.lpr;
  l.wch = lanes_here * p.vec;
  l.g_lo = div_by(l.cstart, p.by_D);
  l.ng = div_by(l.cstart + l.wch - 1, p.by_D) - l.g_lo + 1;
  l.active = l.ty < p.rpi && l.cvi < p.cv;
  l.rows = l.active ? l.rows_base + (l.ty < l.rows_rem ? 1 : 0) : 0;
  return l;
}

// A lane walks its rows in batches of U and keeps two batches of raw vectors in registers: while batch b
// is being consumed the loads of batch b + 1 are already in flight.  issue(sel, b) starts the loads of
// batch b into buffer `sel` (std::integral_constant 0 / 1); consume(sel, b) uses them.  The caller issues
// batch 0 itself, before any prologue it wants to hide behind those loads.
// Row u of batch b is the lane's row min(b U + u, rows - 1): the trailing batch re-reads the last row
// instead of branching, consumers that accumulate weight such duplicates with 0, consumers that store
// simply store the same values again.
// `nb` must be uniform over the workgroup (lanes with fewer rows clamp), and every issue inside the steady
// state is unconditional: a load issued under a branch would force the waits that follow the join to
// assume it may not have happened, i.e. to drain the queue, and the two batches would no longer overlap.
template <typename ISSUE, typename CONSUME>
__device__ __forceinline__ void double_buffered(int nb, ISSUE &&issue, CONSUME &&consume) {
  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  int b = 0;
  while (b + 2 < nb) {
    issue(B1{}, b + 1);
    consume(B0{}, b);
    issue(B0{}, b + 2);
    consume(B1{}, b + 1);
    b += 2;
  }
  if (nb - b == 2) {
    issue(B1{}, b + 1);
    consume(B0{}, b);
    consume(B1{}, b + 1);
  } else if (nb - b == 1) {
    consume(B0{}, b);
  }
}
// Batches every active lane of the workgroup walks: the lane rows with the most rows set the count.
template <int U> __device__ __forceinline__ int block_batches(const Plan &p, const LanePos &l) {
  const int rows_blk = div_by(l.len + p.rpi - 1, p.by_rpi);
  return (rows_blk + U - 1) / U;
}
__device__ __forceinline__ int clamp_row(int idx, int rows) { return idx < rows ? idx : rows - 1; }

// Partial results are ordinary cached data between two launches, but inside a resident launch they are
// exchanged between workgroups on different XCDs, whose L2 caches are not coherent with each other.
// COH selects device-scope accesses (write-through stores, cache-bypassing loads), which makes the
// exchange work without any L2 write-back / invalidate fence.
template <bool COH, typename A> __device__ __forceinline__ A ld_part(const A *p) {
  if constexpr (COH) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else return *p;
}
template <bool COH, typename A> __device__ __forceinline__ void st_part(A *p, A v) {
  if constexpr (COH) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

template <typename PT, typename A> __device__ __forceinline__ A load_param(const void *p, int64_t i) {
  A v[1];
  LaneVec<PT, 1>::unpack(LaneVec<PT, 1>::load((const PT *)p + i), v);
  return v[0];
}
template <typename PT, typename A> __device__ __forceinline__ void store_param(void *p, int64_t i, A x) {
  const A v[1] = {x};
  LaneVec<PT, 1>::store((PT *)p + i, LaneVec<PT, 1>::pack(v));
}

// The incoming gradient of a backward on float data may be stored in a 16-bit type (DY16; dydtype GN_F16 or GN_BF16: the
// layer that produced it ran in half precision).  A lane vector of it is 8 bytes, carried in the first half of the raw
// register vector until it is unpacked; widening happens in registers, no separate pass over dy.
template <typename T, int VEC, bool DY16>
__device__ __forceinline__ typename LaneVec<T, VEC>::raw_t load_dy(const T *dy, int64_t e) {
  if constexpr (!DY16) {
    return LaneVec<T, VEC>::load(dy + e);
  } else {
    static_assert(sizeof(T) == 4, "a 16-bit gradient accompanies float data only");
    const uint16_t *h = (const uint16_t *)dy + e;
    if constexpr (VEC == 4) {
      const u32x2 v = *(const u32x2 *)h;
      const uint32_t lo = v.x, hi = v.y;
      return f32x4{__builtin_bit_cast(float, lo), __builtin_bit_cast(float, hi), 0.f, 0.f};
    } else {
      return __builtin_bit_cast(float, (uint32_t)*h);
    }
  }
}
__device__ __forceinline__ float widen_16(uint32_t bits16, int dydtype) {
  const float b = bf16_bits_to_float(bits16 << 16);
  const float h = (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
  return dydtype == GN_BF16 ? b : h;
}
template <typename T, int VEC, bool DY16>
__device__ __forceinline__ void unpack_dy(typename LaneVec<T, VEC>::raw_t raw, acc_t<T> (&v)[VEC], int dydtype) {
  if constexpr (!DY16) {
    LaneVec<T, VEC>::unpack(raw, v);
  } else if constexpr (VEC == 4) {
    const float r0 = raw.x, r1 = raw.y;
    const uint32_t lo = __builtin_bit_cast(uint32_t, r0), hi = __builtin_bit_cast(uint32_t, r1);
    v[0] = widen_16(lo & 0xffffu, dydtype);
    v[1] = widen_16(lo >> 16, dydtype);
    v[2] = widen_16(hi & 0xffffu, dydtype);
    v[3] = widen_16(hi >> 16, dydtype);
  } else {
    v[0] = widen_16(__builtin_bit_cast(uint32_t, raw) & 0xffffu, dydtype);
  }
}
// One element of it (recovery paths, scalar code).
template <typename T, bool DY16> __device__ __forceinline__ float load_dy_scalar(const T *dy, int64_t e, int dydtype) {
  float v[1];
  unpack_dy<T, 1, DY16>(load_dy<T, 1, DY16>(dy, e), v, dydtype);
  return v[0];
}

// Per-group tile partials are stored as planes of one field each, laid out [N][nchunk][G][tiles]: the
// entries a consumer merges for one group (all tiles of the one or two chunks that hold the group) are
// contiguous, so the merge reads them with coalesced loads.
__device__ __forceinline__ int64_t group_slot(const PartialGeo &q, int G, int64_t n, int t, int k, int g) {
  return ((n * q.nchunk + k) * G + g) * q.tiles + t;
}
__device__ __forceinline__ int64_t group_plane(const PartialGeo &q, int G, int64_t N) {
  return N * q.nchunk * G * q.tiles;
}
// Chunks [k_lo, k_lo + nk) of the producer hold pieces of group g.
__device__ __forceinline__ void group_chunks(const PartialGeo &q, int D, int g, int &k_lo, int &nk) {
  k_lo = div_by(g * D, q.by_chunk);
  nk = div_by((g + 1) * D - 1, q.by_chunk) - k_lo + 1;
}
// Lanes per group for a consumer's looping merge of tile partials (general path).
__device__ __forceinline__ int merge_lanes(const PartialGeo &q, int D) {
  return pow2_ceil_clamped(q.tiles * (div_by(D - 1, q.by_chunk) + 2), 64);
}

// Early fetch of tile partials: every group of the chunk gets `L` lanes in a single round, and each lane
// loads its (at most kEarly) entries of NF fields into registers.  The loads are issued before the lane's
// first data loads, so they are not queued behind them; they are consumed after those loads are in flight.
template <typename A, int NF> struct EarlyPartials {
  A v[kEarly][NF];  // as loaded: entry i is meaningful only if have(i) (the others were read from entry 0 of the buffer)
  int L, gi, sl, P;
  bool valid;
  __device__ __forceinline__ bool have(int i) const { return sl + i * L < P; }
};
template <typename A, int NF, bool COH>
__device__ __forceinline__ void fetch_partials(EarlyPartials<A, NF> &e, const A *__restrict__ part, int64_t plane,
                                               const PartialGeo &q, const Plan &p, const LanePos &l) {
  int gp = 1;
  while (gp < p.gmax) gp <<= 1;
  e.L = kBlock / gp < 64 ? kBlock / gp : 64;
  e.gi = threadIdx.x >> __builtin_ctz(e.L);  // L is a power of two
  e.sl = threadIdx.x & (e.L - 1);
  e.valid = e.gi < l.ng;
  const int g = l.g_lo + e.gi;
  int k_lo = 0, nk = 1;
  if (e.valid) group_chunks(q, p.D, g, k_lo, nk);
  e.P = e.valid ? q.tiles * nk : 0;
  const int64_t base = group_slot(q, p.G, l.n, 0, k_lo, g);
  const int64_t kstride = (int64_t)p.G * q.tiles;
  // all addresses first, then nothing but loads: any control flow between the loads (the division below may
  // branch) or any use of a loaded value here would make the compiler wait for them before the caller's next loads
  int64_t slot[kEarly];
#pragma unroll
  for (int i = 0; i < kEarly; ++i) {
    const int en = e.sl + i * e.L;
    const bool have = en < e.P;
    const int k = have ? div_by(en, q.by_tiles) : 0, t = have ? en - k * q.tiles : 0;
    slot[i] = have ? base + k * kstride + t : 0;  // entry 0 exists: the load needs no guard
  }
#pragma unroll
  for (int i = 0; i < kEarly; ++i) {
#pragma unroll
    for (int f = 0; f < NF; ++f) e.v[i][f] = ld_part<COH>(part + f * plane + slot[i]);
  }
}
// (count, mean, M2) entries -> merged triple (pivot form), available in every lane of the group's segment.
template <typename A> __device__ __forceinline__ Moments<A> reduce_moments(const EarlyPartials<A, 3> &e) {
  A nl = (A)0, s1 = (A)0, s2 = (A)0;
  const A kl = e.have(0) ? e.v[0][1] : (A)0;
#pragma unroll
  for (int i = 0; i < kEarly; ++i) {
    const bool h = e.have(i);
    const A cn = h ? e.v[i][0] : (A)0;
    const A d = h ? e.v[i][1] - kl : (A)0;
    nl += cn;
    s1 += cn * d;
    s2 += (h ? e.v[i][2] : (A)0) + cn * d * d;
  }
  const A inv = nl > (A)0 ? fast_rcp(nl) : (A)0;
  const A mean_l = kl + s1 * inv;
  const A m2_l = s2 - s1 * s1 * inv;
  const A K = __shfl(mean_l, (int)(threadIdx.x & 63 & ~(e.L - 1)), 64);
  const A d = mean_l - K;
  A t0 = nl, t1 = nl * d, t2 = m2_l + nl * d * d;
  t0 = segment_sum(t0, e.L);
  segment_sum2(t1, t2, e.L);
  Moments<A> r;
  r.n = t0;
  const A dm = e.valid ? t1 * fast_rcp(t0) : (A)0;
  r.mean = K + dm;
  r.m2 = t2 - t1 * dm;
  return r;
}
template <typename A> __device__ __forceinline__ void reduce_sums(const EarlyPartials<A, 2> &e, A &ta, A &tb) {
  ta = (A)0;
  tb = (A)0;
#pragma unroll
  for (int i = 0; i < kEarly; ++i) {
    const bool h = e.have(i);
    ta += h ? e.v[i][0] : (A)0;
    tb += h ? e.v[i][1] : (A)0;
  }
  segment_sum2(ta, tb, e.L);
}
// Channels [ca, cb) (relative to the chunk) of group g that lie inside the chunk.
__device__ __forceinline__ void group_span(const Plan &p, const LanePos &l, int g, int &ca, int &cb) {
  ca = (g * p.D > l.cstart ? g * p.D : l.cstart) - l.cstart;
  cb = ((g + 1) * p.D < l.cstart + l.wch ? (g + 1) * p.D : l.cstart + l.wch) - l.cstart;
}

// ---------------------------------------------------------------------------------------------
// Running per-channel statistics of one lane over its rows of the tile.  Each batch of rows is folded
// with an exact two-pass mean / sum of squares on the values held in registers and merged into the
// running moments with Chan's update: one reciprocal per batch instead of the per-element division of
// WelfordOps::reduce (src/gnnhwc/csrc/Welford.h:30-42).
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC, int U>
__device__ __forceinline__ void fold_batch(const typename LaneVec<T, VEC>::raw_t (&raw)[U], int m, acc_t<T> &cnt,
                                           acc_t<T> (&mean)[VEC], acc_t<T> (&m2)[VEC]) {
  using A = acc_t<T>;
  A s[VEC], qq[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) { s[j] = (A)0; qq[j] = (A)0; }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const A keep = u < m ? (A)1 : (A)0;
    A v[VEC];
    LaneVec<T, VEC>::unpack(raw[u], v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) s[j] += keep * v[j];
  }
  const A mf = (A)m;
  const A inv_m = fast_rcp(mf);
#pragma unroll
  for (int j = 0; j < VEC; ++j) s[j] *= inv_m;  // batch mean
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const A keep = u < m ? (A)1 : (A)0;
    A v[VEC];
    LaneVec<T, VEC>::unpack(raw[u], v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) { const A d = v[j] - s[j]; qq[j] += keep * d * d; }
  }
  const A nn = cnt + mf;
  const A f = mf * fast_rcp(nn);
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const A d = s[j] - mean[j];
    mean[j] += d * f;
    m2[j] += qq[j] + d * d * cnt * f;
  }
  cnt = nn;
}

template <typename T, int VEC, int U>
__device__ __forceinline__ void lane_stats(const T *__restrict__ x, const Plan &p, const LanePos &l,
                                           acc_t<T> (&mean)[VEC], acc_t<T> (&m2)[VEC]) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
#pragma unroll
  for (int j = 0; j < VEC; ++j) { mean[j] = (A)0; m2[j] = (A)0; }
  A cnt = (A)0;
  const int rows = l.rows;
  const int nb = block_batches<U>(p, l);
  if (rows == 0) return;
  const T *base = x + ((l.n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC);
  const int64_t step = (int64_t)p.rpi * p.C;
  typename LV::raw_t buf0[U], buf1[U];
  auto issue = [&](auto sel, int b) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const T *src = base + (int64_t)clamp_row(b * U + u, rows) * step;
      if constexpr (decltype(sel)::value == 0) buf0[u] = LV::load(src);
      else buf1[u] = LV::load(src);
    }
  };
  auto consume = [&](auto sel, int b) {
    int m = rows - b * U;
    m = m < 0 ? 0 : (m > U ? U : m);
    if (m == 0) return;  // only in the last batch of a lane row that is one row short
    if constexpr (decltype(sel)::value == 0) fold_batch<T, VEC, U>(buf0, m, cnt, mean, m2);
    else fold_batch<T, VEC, U>(buf1, m, cnt, mean, m2);
  };
  issue(std::integral_constant<int, 0>{}, 0);
  double_buffered(nb, issue, consume);
}

// Sum of col[0], col[stride], ... (n entries) with eight reads in flight: the loop is latency bound otherwise.
template <typename A> __device__ __forceinline__ A column_sum(const A *col, int stride, int n) {
  A t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = (A)0;
  int r = 0;
  for (; r + 8 <= n; r += 8) {
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] += col[(r + i) * stride];
  }
  for (; r < n; ++r) t[0] += col[r * stride];
  return ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
}

// Merge the per-lane moments of a workgroup into one (count, mean, M2) triple per group of the chunk and
// hand each to emit(g, count, mean, M2) (called by one lane per group).
// Chan's pairwise update (Welford.h:44-65) costs several operations per value and step; instead every
// lane re-expresses its moments as plain sums about a pivot shared by its channel column (the mean of the
// column's first lane row, so the pivot lies inside the data and nothing cancels),
//   S1 = n (mean - K),   S2 = M2 + n (mean - K)^2,
// which add across lane rows with one LDS read and one addition each; the channels of a group, whose pivots
// differ, are then merged about the group's first pivot.
template <typename A, int VEC, typename EMIT>
__device__ __forceinline__ void block_group_moments(const Plan &p, const LanePos &l, const A (&mean)[VEC],
                                                    const A (&m2)[VEC], A *sm_s1, A *sm_s2, EMIT &&emit) {
  __shared__ A sm_k[kBlock * VEC];
  const int W = p.lpr * VEC;
  const int col0 = l.tx * VEC;
  if (l.active && l.ty == 0) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) sm_k[col0 + j] = mean[j];
  }
  __syncthreads();
  if (l.active) {
    const A cnt = (A)l.rows;
    const int at = (l.ty * p.lpr + l.tx) * VEC;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A d = mean[j] - sm_k[col0 + j];
      const A t = cnt * d;
      sm_s1[at + j] = t;
      sm_s2[at + j] = m2[j] + t * d;
    }
  }
  __syncthreads();
  for (int col = threadIdx.x; col < 2 * l.wch; col += kBlock) {
    const bool second = col >= l.wch;
    A *arr = second ? sm_s2 : sm_s1;
    const int c = second ? col - l.wch : col;
    arr[c] = column_sum(arr + c, W, p.rpi);  // replaces lane row 0 of the column (only this thread touches the column)
  }
  __syncthreads();
  const int nc_max = p.D < l.wch ? p.D : l.wch;
  const int L = pow2_ceil_clamped(nc_max, 16);  // lanes per group: a DPP row at most
  const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
  const int seg = spread_segment(L), sl = threadIdx.x & (L - 1);
  const A nrows = (A)l.len;
  for (int base = 0; base < l.ng; base += nseg) {
    const int gi = base + seg;
    const int g = l.g_lo + gi;
    const bool valid = gi < l.ng;
    int ca = 0, cb = 0;
    if (valid) group_span(p, l, g, ca, cb);
    const A K = valid ? sm_k[ca] : (A)0;
    A s1 = (A)0, s2 = (A)0;
    for (int c = ca + sl; c < cb; c += L) {
      const A dk = sm_k[c] - K;
      const A a1 = sm_s1[c];
      s1 += a1 + nrows * dk;
      s2 += sm_s2[c] + dk * ((A)2 * a1 + nrows * dk);
    }
    segment_sum2(s1, s2, L);
    if (valid && sl == 0) {
      const A total = (A)(cb - ca) * nrows;
      const A dm = s1 * fast_rcp(total);
      emit(g, total, K + dm, s2 - s1 * dm);
    }
  }
  __syncthreads();  // the LDS arrays may be reused by the caller
}

// Sum the per-lane (s1, s2) pairs of a workgroup over its lane rows: afterwards sm1[c], sm2[c] hold the
// tile's sums for channel c of the chunk (c < wch).
template <typename A, int VEC>
__device__ __forceinline__ void block_channel_sums(const Plan &p, const LanePos &l, const A (&s1)[VEC], const A (&s2)[VEC],
                                                   A *sm1, A *sm2) {
  const int W = p.lpr * VEC;
  if (l.active) {
    const int at = (l.ty * p.lpr + l.tx) * VEC;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      sm1[at + j] = s1[j];
      sm2[at + j] = s2[j];
    }
  }
  __syncthreads();
  for (int col = threadIdx.x; col < 2 * l.wch; col += kBlock) {
    const bool second = col >= l.wch;
    A *arr = second ? sm2 : sm1;
    const int c = second ? col - l.wch : col;
    arr[c] = column_sum(arr + c, W, p.rpi);  // replaces lane row 0 of the column (only this thread touches the column)
  }
  __syncthreads();
}

// ---------------------------------------------------------------------------------------------
// Pre-addition of the multi-launch forward: dst = x + residual + channel_bias[n][c], rounded to T once, on the
// tiles of the streaming kernels.  dst may be x or the residual (a lane reads the elements it writes first, and no
// other lane touches them).  `safe` is any readable 64 bytes (the workspace).
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void add_kernel(const T *__restrict__ x, AddArgs add, T *dst, const void *safe, Plan p) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  constexpr int U = 4;  // rows of a lane in flight
  const T *rp = (const T *)add.residual;
  for (int64_t n = blockIdx.z; n < p.N; n += gridDim.z) {
    const LanePos l = lane_pos(p, n, false);
    if (l.rows == 0) continue;
    A tb[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      tb[j] = add.channel_bias ? load_scalar_flat<A>(add.channel_bias, n * p.C + (int64_t)l.cvi * VEC + j, add.channel_bias_dtype, safe)
                               : (A)0;
    const int64_t base = (n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
    const int64_t step = (int64_t)p.rpi * p.C;
    for (int r0 = 0; r0 < l.rows; r0 += U) {
      typename LV::raw_t bx[U], br[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t o = base + (int64_t)clamp_row(r0 + u, l.rows) * step;
        bx[u] = LV::load(x + o);
        br[u] = LV::load((rp ? rp : x) + o);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (r0 + u < l.rows) {
          A vx[VEC], vr[VEC];
          LV::unpack(bx[u], vx);
          LV::unpack(br[u], vr);
#pragma unroll
          for (int j = 0; j < VEC; ++j) vx[j] = (vx[j] + (rp ? vr[j] : (A)0)) + tb[j];
          LV::store(dst + base + (int64_t)(r0 + u) * step, LV::pack(vx));
        }
      }
    }
  }
}

// The same without a channel addend: dst = x + residual is a flat elementwise sum, four lane vectors per thread and
// step (nvec = number of lane vectors of the tensor).
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void add_flat_kernel(const T *__restrict__ x, const T *residual, T *dst, int64_t nvec) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  constexpr int U = 4;
  const int64_t stride = (int64_t)gridDim.x * kBlock;
  for (int64_t i0 = (int64_t)blockIdx.x * kBlock + threadIdx.x; i0 < nvec; i0 += U * stride) {
    typename LV::raw_t bx[U], br[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = i0 + u * stride;
      const int64_t e = (i < nvec ? i : i0) * VEC;
      bx[u] = LV::load(x + e);
      br[u] = LV::load(residual + e);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = i0 + u * stride;
      if (i < nvec) {
        A vx[VEC], vr[VEC];
        LV::unpack(bx[u], vx);
        LV::unpack(br[u], vr);
#pragma unroll
        for (int j = 0; j < VEC; ++j) vx[j] += vr[j];
        LV::store(dst + i * VEC, LV::pack(vx));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Forward pass 1: per-tile (count, mean, M2) of every group the tile touches.
// Does the work of compute_stats_pt1 (src/gnnhwc/csrc/gn_kernel.cu:132-224).
//   part : 3 planes [N][nchunk][G][tiles]; only the groups a chunk intersects are written.
// ---------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void stats_kernel(
    const T *__restrict__ x, acc_t<T> *__restrict__ part, Plan p) {
  using A = acc_t<T>;
  __shared__ A sm_mean[kBlock * VEC];
  __shared__ A sm_m2[kBlock * VEC];
  const PartialGeo q = producer_geo(p);
  const int64_t plane = group_plane(q, p.G, p.N);
  for (int64_t n = blockIdx.z; n < p.N; n += gridDim.z) {
    const LanePos l = lane_pos(p, n, false);
    A mean[VEC], m2[VEC];
    lane_stats<T, VEC, kUnrollFwd>(x, p, l, mean, m2);
    block_group_moments<A, VEC>(p, l, mean, m2, sm_mean, sm_m2, [&](int g, A cnt, A mu, A s2) {
      const int64_t slot = group_slot(q, p.G, n, l.tile, l.chunk, g);
      part[slot] = cnt;
      part[plane + slot] = mu;
      part[2 * plane + slot] = s2;
    });
  }
}

// Merge the P = tiles * (chunks holding a piece of g) partial triples of group g with `L` lanes; every
// lane of the segment returns the merged triple.  One pass over the entries (all loads independent, one
// memory round trip): each lane folds its entries about the mean of its first one, then the lanes are
// merged about the first lane's mean (the pivot form of the two-pass merge).
template <typename A, bool COH>
__device__ __forceinline__ Moments<A> merge_group_partials(const A *__restrict__ part, int64_t plane, const PartialGeo &q,
                                                           int G, int D, int64_t n, int g, bool valid, int L, int sl) {
  int k_lo = 0, nk = 1;
  if (valid) group_chunks(q, D, g, k_lo, nk);
  const int P = valid ? q.tiles * nk : 0;
  // entries of chunk k_lo .. k_lo + nk - 1 are contiguous runs of q.tiles values each
  const int64_t base = group_slot(q, G, n, 0, k_lo, g);
  const int64_t kstride = (int64_t)G * q.tiles;
  A nl = (A)0, kl = (A)0, s1 = (A)0, s2 = (A)0;
  for (int e = sl; e < P; e += L) {
    const int k = div_by(e, q.by_tiles), t = e - k * q.tiles;
    const int64_t slot = base + k * kstride + t;
    const A cn = ld_part<COH>(part + slot);
    const A mu = ld_part<COH>(part + plane + slot);
    const A mm = ld_part<COH>(part + 2 * plane + slot);
    if (nl == (A)0) kl = mu;
    const A d = mu - kl;
    nl += cn;
    s1 += cn * d;
    s2 += mm + cn * d * d;
  }
  const A inv = nl > (A)0 ? fast_rcp(nl) : (A)0;
  const A mean_l = kl + s1 * inv;
  const A m2_l = s2 - s1 * s1 * inv;
  const A K = __shfl(mean_l, (int)(threadIdx.x & 63 & ~(L - 1)), 64);
  const A d = mean_l - K;
  A t0 = nl, t1 = nl * d, t2 = m2_l + nl * d * d;
  t0 = segment_sum(t0, L);
  segment_sum2(t1, t2, L);
  Moments<A> r;
  r.n = t0;
  const A dm = valid ? t1 * fast_rcp(t0) : (A)0;
  r.mean = K + dm;
  r.m2 = t2 - t1 * dm;
  return r;
}

// ---------------------------------------------------------------------------------------------
// Optional forward pass 1b (only when a sample has too many tiles for the consumers to merge
// themselves): one wavefront per (n, g) merges the tile partials into a single triple.
//   out : 3 planes [N][G]
// ---------------------------------------------------------------------------------------------
template <typename A>
__global__ __launch_bounds__(kBlock) void stats_compact_kernel(const A *__restrict__ part, A *__restrict__ out,
                                                               PartialGeo q, Plan p) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (kBlock / 64) + wave;
  const bool valid = item < p.N * p.G;
  const int64_t n = valid ? item / p.G : 0;
  const int g = valid ? (int)(item - n * p.G) : 0;
  const Moments<A> m = merge_group_partials<A, false>(part, group_plane(q, p.G, p.N), q, p.G, p.D, n, g, valid, 64, lane);
  if (valid && lane == 0) {
    const int64_t oplane = p.N * p.G;
    out[item] = m.n;
    out[oplane + item] = m.mean;
    out[2 * oplane + item] = m.m2;
  }
}

// Consumer prologue of the forward: merge the tile partials of the chunk's groups into mean / rstd
// (compute_stats_pt2, src/gnnhwc/csrc/gn_kernel.cu:226-292: rstd = 1 / sqrt(M2 / n + eps)), leave them in
// LDS indexed by (g - g_lo), and let the workgroups of row tile 0 report them to the caller's outputs.
template <typename A, bool COH>
__device__ __forceinline__ void merge_chunk_stats(const A *__restrict__ part, const PartialGeo &q, const Plan &p,
                                                  const LanePos &l, A eps, A *sm_mu, A *sm_rs, void *mean_out,
                                                  void *rstd_out, int sdtype) {
  const int L = merge_lanes(q, p.D);
  const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
  const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
  const int64_t plane = group_plane(q, p.G, p.N);
  for (int base = 0; base < l.ng; base += nseg) {
    const int gi = base + seg;
    const bool valid = gi < l.ng;
    const int g = l.g_lo + gi;
    const Moments<A> m = merge_group_partials<A, COH>(part, plane, q, p.G, p.D, l.n, g, valid, L, sl);
    if (valid && sl == 0) {
      const A rs = fast_rsqrt(m.m2 * fast_rcp(m.n) + eps);
      sm_mu[gi] = m.mean;
      sm_rs[gi] = rs;
      if (l.tile == 0 && g * p.D >= l.cstart) {  // the chunk where the group starts reports it
        if (mean_out) store_scalar<A>(mean_out, l.n * p.G + g, sdtype, m.mean);
        if (rstd_out) store_scalar<A>(rstd_out, l.n * p.G + g, sdtype, rs);
      }
    }
  }
  __syncthreads();
}
// Backward: the caller's mean / rstd of the chunk's groups, staged in LDS the same way.  In two steps, so that
// the loads can be issued ahead of a kernel's bulk loads and waited for on their own while those are in flight:
// fetch (no control flow around the loads of the usual case, one group per thread) and commit (LDS writes).
template <typename A> struct StagedStats {
  A mu, rs;
};
template <typename A>
__device__ __forceinline__ StagedStats<A> fetch_chunk_stats(const void *mean, const void *rstd, int sdtype, const Plan &p,
                                                            const LanePos &l, A *sm_mu, A *sm_rs, const void *safe) {
  for (int gi = threadIdx.x + kBlock; gi < l.ng; gi += kBlock) {  // more groups than threads: rare, done up front
    sm_mu[gi] = load_scalar<A>(mean, l.n * p.G + l.g_lo + gi, sdtype);
    sm_rs[gi] = load_scalar<A>(rstd, l.n * p.G + l.g_lo + gi, sdtype);
  }
  const int gi = (int)threadIdx.x < l.ng ? threadIdx.x : l.ng - 1;
  StagedStats<A> st;
  st.mu = load_scalar_flat<A>(mean, l.n * p.G + l.g_lo + gi, sdtype, safe);
  st.rs = load_scalar_flat<A>(rstd, l.n * p.G + l.g_lo + gi, sdtype, safe);
  return st;
}
template <typename A>
__device__ __forceinline__ void commit_chunk_stats(const StagedStats<A> &st, const LanePos &l, A *sm_mu, A *sm_rs) {
  if ((int)threadIdx.x < l.ng) {
    sm_mu[threadIdx.x] = st.mu;
    sm_rs[threadIdx.x] = st.rs;
  }
}

// gamma / beta of the lane's channels, requested early (next to the first data loads, so that their latency is
// hidden behind whatever the kernel has to wait for anyway) and without control flow: a load under a branch
// makes the compiler drain every outstanding load where the branch joins.  Absent parameters are read from
// `safe` (any readable 64 bytes) and replaced by 1 / 0; c is the lane's first channel, already clamped into range.
template <typename A, typename PT, int VEC>
__device__ __forceinline__ void lane_params_flat(int c, const void *w, const void *b, const void *safe, A (&gamma)[VEC],
                                                 A (&beta)[VEC]) {
  const PT *wp = w ? (const PT *)w + c : (const PT *)safe;
  const PT *bp = b ? (const PT *)b + c : (const PT *)safe;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const A gv = load_param<PT, A>(wp, j);
    const A bv = load_param<PT, A>(bp, j);
    gamma[j] = w ? gv : (A)1;
    beta[j] = b ? bv : (A)0;
  }
}
// Addresses that are valid for every lane of the workgroup, idle ones included (they re-read the tile's first
// row and the row's last lane vector), so that loads need no guard; `rows` is at least 1 for the row clamp.
struct SafeLane {
  int64_t off;  // element offset of the lane's first row
  int c;        // first channel of the lane vector
  int rows;     // max(rows of the lane, 1)
  bool live;    // the lane owns at least one row
};
template <int VEC> __device__ __forceinline__ SafeLane safe_lane(const Plan &p, const LanePos &l, int64_t n) {
  SafeLane s;
  s.live = l.rows > 0;
  const int cvi = l.cvi < p.cv ? l.cvi : p.cv - 1;
  s.c = cvi * VEC;
  s.off = (n * p.R + l.row0 + (s.live ? l.ty : 0)) * p.C + s.c;
  s.rows = s.live ? l.rows : 1;
  return s;
}
// a = rstd * gamma, b = beta - mean * a: normalise + affine as one FMA per element (same folding as
// src/gnnhwc/csrc/gn_kernel.cu:350-379, 601-602, 783-784).  Group statistics come from LDS; optional
// per-group extras (the backward's coef1 / coef2) are fetched alongside.  On return sa / sb replace gamma / beta.
// Per-channel copies of two per-group LDS arrays (indexed by group inside the chunk) for the lane's VEC channels.
// When a group has at least VEC channels the lane's channels lie in at most two groups: four LDS reads and a select
// per channel instead of two reads and the bookkeeping of the group boundary per channel.
template <typename A, int VEC>
__device__ __forceinline__ void lane_group_pairs(const Plan &p, const LanePos &l, const A *sm_a, const A *sm_b, A (&va)[VEC],
                                                 A (&vb)[VEC]) {
  const int c = l.cvi * VEC;
  int gi = div_by(c, p.by_D);
  int rem = c - gi * p.D;
  gi -= l.g_lo;
  if (VEC > 1 && p.D >= VEC) {
    const int split = p.D - rem;               // channels j < split lie in group gi, the others in gi + 1
    const int gj = split < VEC ? gi + 1 : gi;  // (no second group: read the first again, never past the chunk's groups)
    const A a0 = sm_a[gi], b0 = sm_b[gi], a1 = sm_a[gj], b1 = sm_b[gj];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const bool first = j < split;
      va[j] = first ? a0 : a1;
      vb[j] = first ? b0 : b1;
    }
  } else {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      va[j] = sm_a[gi];
      vb[j] = sm_b[gi];
      ++rem;
      const bool wrap = rem == p.D;
      rem = wrap ? 0 : rem;
      gi += wrap ? 1 : 0;
    }
  }
}
template <typename A, int VEC, bool EXTRA>
__device__ __forceinline__ void lane_coeffs(const Plan &p, const LanePos &l, const A *sm_mu, const A *sm_rs,
                                            const A *sm_c1, const A *sm_c2, A (&sa)[VEC], A (&sb)[VEC], A (&c1)[VEC],
                                            A (&c2)[VEC]) {
  A mu[VEC], rs[VEC];
  lane_group_pairs<A, VEC>(p, l, sm_mu, sm_rs, mu, rs);
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    sa[j] = rs[j] * sa[j];
    sb[j] = sb[j] - mu[j] * sa[j];
  }
  if (EXTRA) lane_group_pairs<A, VEC>(p, l, sm_c1, sm_c2, c1, c2);
}

// ---------------------------------------------------------------------------------------------
// Forward pass 2: y = act(x * a + b) (scale_shift_kernel, src/gnnhwc/csrc/gn_kernel.cu:305-412), for every
// shape with one code path (no R % 8 fast / slow split).  y is computed from the unrounded mean / rstd
// whatever type the reported statistics have (cf. gn_kernel.cu:290-291).
// ---------------------------------------------------------------------------------------------
template <typename T, typename PT, int VEC, int ACT>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void apply_kernel(
    const T *__restrict__ x, T *__restrict__ y, const acc_t<T> *__restrict__ part, PartialGeo q, const void *w,
    const void *b, void *mean_out, void *rstd_out, int sdtype, int ydtype, acc_t<T> eps, Plan p) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  constexpr int U = kUnrollFwd;
  __shared__ A sm_mu[kBlock * VEC];
  __shared__ A sm_rs[kBlock * VEC];
  const bool one_round = pow2_at_least(p.gmax) <= kBlock;
  for (int64_t n = blockIdx.z; n < p.N; n += gridDim.z) {
    const LanePos l = lane_pos(p, n, true);
    const int rows = l.rows;
    const int nb = block_batches<U>(p, l);
    const SafeLane sfl = safe_lane<VEC>(p, l, n);
    const int64_t off = sfl.off;
    const int64_t step = (int64_t)p.rpi * p.C;
    typename LV::raw_t buf0[U], buf1[U];
    A sa[VEC], sb[VEC], unused1[VEC], unused2[VEC];
    auto issue = [&](auto sel, int bi) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const T *src = x + off + (int64_t)clamp_row(bi * U + u, sfl.rows) * step;
        if constexpr (decltype(sel)::value == 0) buf0[u] = LV::load(src);
        else buf1[u] = LV::load(src);
      }
    };
    auto consume = [&](auto sel, int bi) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        A v[VEC];
        if constexpr (decltype(sel)::value == 0) LV::unpack(buf0[u], v);
        else LV::unpack(buf1[u], v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = act_fwd<ACT, A>(v[j] * sa[j] + sb[j]);
        if (bi * U + u < rows) store_result<T, VEC>(y, off + (int64_t)(bi * U + u) * step, v, ydtype);
      }
    };
    // order of issue: the few small loads the prologue depends on first, then the first batch of x, so that
    // the small ones are not queued behind the bulk traffic of every workgroup; no load of the prologue sits under
    // a branch (idle lanes read valid addresses too), so each wait below covers exactly the loads it needs
    // (the early fetch runs even when the general merge below will be used: a branch here would make the compiler
    // wait for these loads before it issues the next ones)
    EarlyPartials<A, 3> early;
    fetch_partials<A, 3, false>(early, part, group_plane(q, p.G, p.N), q, p, l);
    lane_params_flat<A, PT, VEC>(sfl.c, w, b, part, sa, sb);
    issue_order_fence();
    issue(std::integral_constant<int, 0>{}, 0);
    if (one_round) {
      const Moments<A> m = reduce_moments<A>(early);
      if (early.valid && early.sl == 0) {
        const int g = l.g_lo + early.gi;
        const A rs = fast_rsqrt(m.m2 * fast_rcp(m.n) + eps);
        sm_mu[early.gi] = m.mean;
        sm_rs[early.gi] = rs;
        if (l.tile == 0 && g * p.D >= l.cstart) {  // the chunk where the group starts reports it
          if (mean_out) store_scalar<A>(mean_out, n * p.G + g, sdtype, m.mean);
          if (rstd_out) store_scalar<A>(rstd_out, n * p.G + g, sdtype, rs);
        }
      }
      __syncthreads();
    } else {
      merge_chunk_stats<A, false>(part, q, p, l, eps, sm_mu, sm_rs, mean_out, rstd_out, sdtype);
    }
    if (rows > 0) {
      lane_coeffs<A, VEC, false>(p, l, sm_mu, sm_rs, nullptr, nullptr, sa, sb, unused1, unused2);
      double_buffered(nb, issue, consume);
    }
    __syncthreads();  // sm_mu / sm_rs are rewritten for the next sample of a wrapped grid
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 1: per tile, per channel S1 = sum g x and S2 = sum g with g = dy * act'(x a + b)
// recomputed from x (width_reduce, src/gnnhwc/csrc/gn_kernel.cu:557-646), and per tile, per group
// A = sum_c gamma_c S1_c and B = sum_c gamma_c S2_c (the group sums of compute_bwd_scale_biases,
// gn_kernel.cu:786-797).
//   partC : [N][tiles][C][2]      partG : 2 planes [N][nchunk][G][tiles]
// ---------------------------------------------------------------------------------------------
template <typename T, typename PT, int VEC, int ACT, bool DY16 = false>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void bwd_reduce_kernel(
    const T *__restrict__ x, const T *__restrict__ dy, const void *mean, const void *rstd, int sdtype, const void *w,
    const void *b, acc_t<T> *__restrict__ partC, acc_t<T> *__restrict__ partG, Plan p, int dydtype) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  constexpr int U = kUnrollBwd;
  __shared__ A sm1[kBlock * VEC];
  __shared__ A sm2[kBlock * VEC];
  __shared__ A sm_mu[kBlock * VEC];
  __shared__ A sm_rs[kBlock * VEC];
  const PartialGeo q = producer_geo(p);
  const int64_t plane = group_plane(q, p.G, p.N);
  for (int64_t n = blockIdx.z; n < p.N; n += gridDim.z) {
    const LanePos l = lane_pos(p, n, false);
    const int rows = l.rows;
    const int nb = block_batches<U>(p, l);
    const SafeLane sfl = safe_lane<VEC>(p, l, n);
    const int64_t off = sfl.off;
    const int64_t step = (int64_t)p.rpi * p.C;
    typename LV::raw_t bx0[U], bx1[U], bd0[U], bd1[U];
    A sa[VEC], sb[VEC], s1[VEC], s2[VEC], unused1[VEC], unused2[VEC];
    auto issue = [&](auto sel, int bi) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t o = off + (int64_t)clamp_row(bi * U + u, sfl.rows) * step;
        if constexpr (decltype(sel)::value == 0) { bx0[u] = LV::load(x + o); bd0[u] = load_dy<T, VEC, DY16>(dy, o); }
        else { bx1[u] = LV::load(x + o); bd1[u] = load_dy<T, VEC, DY16>(dy, o); }
      }
    };
    auto consume = [&](auto sel, int bi) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const A keep = bi * U + u < rows ? (A)1 : (A)0;
        A vx[VEC], vd[VEC];
        if constexpr (decltype(sel)::value == 0) { LV::unpack(bx0[u], vx); unpack_dy<T, VEC, DY16>(bd0[u], vd, dydtype); }
        else { LV::unpack(bx1[u], vx); unpack_dy<T, VEC, DY16>(bd1[u], vd, dydtype); }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const A g = keep * vd[j] * act_bwd<ACT, A>(vx[j] * sa[j] + sb[j]);
          s1[j] += g * vx[j];
          s2[j] += g;
        }
      }
    };
    // small loads first, then the bulk, none of them under a branch: the statistics are waited for on their own
    const StagedStats<A> st = fetch_chunk_stats<A>(mean, rstd, sdtype, p, l, sm_mu, sm_rs, partC);
    lane_params_flat<A, PT, VEC>(sfl.c, w, b, partC, sa, sb);
    // gamma of the channel this thread publishes in the epilogue, fetched now: off the tile's serial tail
    A gamma0;
    {
      const int cg = (int)threadIdx.x < l.wch ? threadIdx.x : 0;
      const PT *gp = w ? (const PT *)w + l.cstart + cg : (const PT *)partC;
      const A gv = load_param<PT, A>(gp, 0);
      gamma0 = w ? gv : (A)1;
    }
    issue_order_fence();
    issue(std::integral_constant<int, 0>{}, 0);
    commit_chunk_stats<A>(st, l, sm_mu, sm_rs);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < VEC; ++j) { s1[j] = (A)0; s2[j] = (A)0; }
    if (rows > 0) {
      lane_coeffs<A, VEC, false>(p, l, sm_mu, sm_rs, nullptr, nullptr, sa, sb, unused1, unused2);
      double_buffered(nb, issue, consume);
    }
    block_channel_sums<A, VEC>(p, l, s1, s2, sm1, sm2);
    // per channel: publish the tile sums; keep gamma-weighted copies for the group sums
    // (a thread's first channel uses the gamma fetched in the prologue: no load in this serial tail)
    if ((int)threadIdx.x < l.wch) {
      const int c = threadIdx.x;
      const A t1 = sm1[c], t2 = sm2[c];
      const int64_t idx = ((n * p.tiles + l.tile) * p.C + l.cstart + c) * 2;
      partC[idx] = t1;
      partC[idx + 1] = t2;
      sm1[c] = gamma0 * t1;
      sm2[c] = gamma0 * t2;
    }
    for (int c = threadIdx.x + kBlock; c < l.wch; c += kBlock) {
      const A t1 = sm1[c], t2 = sm2[c];
      const int64_t idx = ((n * p.tiles + l.tile) * p.C + l.cstart + c) * 2;
      partC[idx] = t1;
      partC[idx + 1] = t2;
      const A gamma = w ? load_param<PT, A>(w, l.cstart + c) : (A)1;
      sm1[c] = gamma * t1;
      sm2[c] = gamma * t2;
    }
    __syncthreads();
    {
      const int L = pow2_ceil_clamped(p.D < l.wch ? p.D : l.wch, 64);
      const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
      const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
      for (int base = 0; base < l.ng; base += nseg) {
        const int gi = base + seg;
        const int g = l.g_lo + gi;
        const bool valid = gi < l.ng;
        int ca = 0, cb = 0;
        if (valid) group_span(p, l, g, ca, cb);
        A ta = (A)0, tb = (A)0;
        for (int c = ca + sl; c < cb; c += L) { ta += sm1[c]; tb += sm2[c]; }
        ta = segment_sum(ta, L);
        tb = segment_sum(tb, L);
        if (valid && sl == 0) {
          const int64_t slot = group_slot(q, p.G, n, l.tile, l.chunk, g);
          partG[slot] = ta;
          partG[plane + slot] = tb;
        }
      }
    }
    __syncthreads();
  }
}

// Sum the tile partials (A, B) of group g with L lanes; every lane of the segment gets the sums.
template <typename A, bool COH>
__device__ __forceinline__ void sum_group_partials(const A *__restrict__ partG, int64_t plane, const PartialGeo &q, int G,
                                                   int D, int64_t n, int g, bool valid, int L, int sl, A &ta, A &tb) {
  int k_lo = 0, nk = 1;
  if (valid) group_chunks(q, D, g, k_lo, nk);
  const int P = valid ? q.tiles * nk : 0;
  const int64_t base = group_slot(q, G, n, 0, k_lo, g);
  const int64_t kstride = (int64_t)G * q.tiles;
  ta = (A)0;
  tb = (A)0;
  for (int e = sl; e < P; e += L) {
    const int k = div_by(e, q.by_tiles), t = e - k * q.tiles;
    const int64_t slot = base + k * kstride + t;
    ta += ld_part<COH>(partG + slot);
    tb += ld_part<COH>(partG + plane + slot);
  }
  ta = segment_sum(ta, L);
  tb = segment_sum(tb, L);
}

// ---------------------------------------------------------------------------------------------
// Optional backward pass 1b (many tiles per sample): sum the tile partials once.
//   blocks [0, nG)      : one wavefront per (n, g)         -> outG 2 planes [N][G]
//   blocks [nG, nG + nC): kBlock / cpb lanes per (n, c)    -> outC [N][C][2]   (height_reduce, gn_kernel.cu:648-693)
// ---------------------------------------------------------------------------------------------
template <typename A>
__global__ __launch_bounds__(kBlock) void bwd_compact_kernel(const A *__restrict__ partC, const A *__restrict__ partG,
                                                             A *__restrict__ outC, A *__restrict__ outG, PartialGeo q,
                                                             int nG_blocks, int cpb, Plan p) {
  if ((int)blockIdx.x < nG_blocks) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * (kBlock / 64) + wave;
    const bool valid = item < p.N * p.G;
    const int64_t n = valid ? item / p.G : 0;
    const int g = valid ? (int)(item - n * p.G) : 0;
    A ta, tb;
    sum_group_partials<A, false>(partG, group_plane(q, p.G, p.N), q, p.G, p.D, n, g, valid, 64, lane, ta, tb);
    if (valid && lane == 0) {
      outG[item] = ta;
      outG[p.N * p.G + item] = tb;
    }
    return;
  }
  // channel sums: cpb channels per workgroup (a power of two chosen by the host so that a small N C still
  // yields many workgroups), kBlock / cpb tile slices; consecutive lanes read consecutive channels
  const int cl = threadIdx.x & (cpb - 1), ts = threadIdx.x / cpb;
  const int slices = kBlock / cpb;
  const int64_t nc = ((int64_t)blockIdx.x - nG_blocks) * cpb + cl;
  __shared__ A red[2][kBlock];
  const bool valid = nc < p.N * p.C;
  A t1 = (A)0, t2 = (A)0;
  if (valid) {
    const int64_t n = nc / p.C, c = nc - n * p.C;
    const A *src = partC + ((n * q.tiles) * p.C + c) * 2;
    const int64_t tstride = p.C * 2;
    int t = ts;
    for (; t + 3 * slices < q.tiles; t += 4 * slices) {  // four independent loads in flight per lane
      A a[4], b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        a[u] = src[(int64_t)(t + u * slices) * tstride];
        b[u] = src[(int64_t)(t + u * slices) * tstride + 1];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) { t1 += a[u]; t2 += b[u]; }
    }
    for (; t < q.tiles; t += slices) {
      t1 += src[(int64_t)t * tstride];
      t2 += src[(int64_t)t * tstride + 1];
    }
  }
  red[0][threadIdx.x] = t1;
  red[1][threadIdx.x] = t2;
  __syncthreads();
  for (int h = slices >> 1; h > 0; h >>= 1) {
    if (ts < h) {
      red[0][threadIdx.x] += red[0][threadIdx.x + h * cpb];
      red[1][threadIdx.x] += red[1][threadIdx.x + h * cpb];
    }
    __syncthreads();
  }
  if (valid && ts == 0) {
    outC[nc * 2] = red[0][cl];
    outC[nc * 2 + 1] = red[1][cl];
  }
}

// ---------------------------------------------------------------------------------------------
// Backward pass 2: sum the tile partials A, B of the chunk's groups, s = 1 / (D R),
//   coef1 = (mean B - A) s rstd^3, coef2 = -mean coef1 - B s rstd      (gn_kernel.cu:798-800)
//   dx = a g + coef1 x + coef2, g recomputed as in pass 1                (dx_elem_kernel, gn_kernel.cu:803-905)
// One extra column of workgroups (blockIdx.x == tiles, sample 0 only) produces, for the channels of its
// chunk, dgamma_c = sum_n (S1 - mean S2) rstd and dbeta_c = sum_n S2 (compute_dweight_dbias, gn_kernel.cu:695-728).
// ---------------------------------------------------------------------------------------------
template <typename T, typename PT, int VEC, int ACT, bool DY16 = false>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void bwd_dx_kernel(
    const T *__restrict__ x, const T *__restrict__ dy, T *__restrict__ dx, const void *mean, const void *rstd, int sdtype,
    const void *w, const void *b, const acc_t<T> *__restrict__ partC, const acc_t<T> *__restrict__ partG, PartialGeo q,
    void *dw, void *db, Plan p, int dydtype) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  constexpr int U = kUnrollBwd;
  const bool one_round = pow2_at_least(p.gmax) <= kBlock;
  __shared__ A sm_c1[kBlock * VEC];
  __shared__ A sm_c2[kBlock * VEC];
  __shared__ A sm_mu[kBlock * VEC];
  __shared__ A sm_rs[kBlock * VEC];
  if ((int)blockIdx.x == p.tiles) {
    if (blockIdx.z != 0 || (!dw && !db)) return;
    const int cstart = blockIdx.y * p.lpr * p.vec;
    const int lanes_here = p.cv - (int)blockIdx.y * p.lpr < p.lpr ? p.cv - (int)blockIdx.y * p.lpr : p.lpr;
    const int wch = lanes_here * p.vec;
    // threads are laid out (tile slice, channel): consecutive threads read consecutive channels
    const int cw = wch < kBlock ? wch : kBlock;  // channels handled per pass
    const int nsl = kBlock / cw;                 // tile slices
    const int cl = threadIdx.x % cw, ts = threadIdx.x / cw;
    for (int cbase = 0; cbase < wch; cbase += cw) {
      const int c = cstart + cbase + cl;
      A t1 = (A)0, t2 = (A)0;
      if (cbase + cl < wch && ts < nsl) {
        const int g = div_by(c, p.by_D);
        for (int64_t n = 0; n < p.N; ++n) {
          A s1 = (A)0, s2 = (A)0;
          for (int t = ts; t < q.tiles; t += nsl) {
            const int64_t idx = ((n * q.tiles + t) * p.C + c) * 2;
            s1 += partC[idx];
            s2 += partC[idx + 1];
          }
          const A mu = load_scalar<A>(mean, n * p.G + g, sdtype);
          const A rs = load_scalar<A>(rstd, n * p.G + g, sdtype);
          t1 += (s1 - mu * s2) * rs;
          t2 += s2;
        }
      }
      __syncthreads();
      if (ts < nsl) { sm_c1[ts * cw + cl] = t1; sm_c2[ts * cw + cl] = t2; }
      __syncthreads();
      if (ts == 0 && cbase + cl < wch) {
        A r1 = (A)0, r2 = (A)0;
        for (int s = 0; s < nsl; ++s) { r1 += sm_c1[s * cw + cl]; r2 += sm_c2[s * cw + cl]; }
        if (dw) store_param<PT, A>(dw, c, r1);
        if (db) store_param<PT, A>(db, c, r2);
      }
    }
    return;
  }
  const int64_t plane = group_plane(q, p.G, p.N);
  for (int64_t n = blockIdx.z; n < p.N; n += gridDim.z) {
    const LanePos l = lane_pos(p, n, true);
    const int rows = l.rows;
    const int nb = block_batches<U>(p, l);
    const SafeLane sfl = safe_lane<VEC>(p, l, n);
    const int64_t off = sfl.off;
    const int64_t step = (int64_t)p.rpi * p.C;
    typename LV::raw_t bx0[U], bx1[U], bd0[U], bd1[U];
    A sa[VEC], sb[VEC], c1[VEC], c2[VEC];
    auto issue = [&](auto sel, int bi) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t o = off + (int64_t)clamp_row(bi * U + u, sfl.rows) * step;
        if constexpr (decltype(sel)::value == 0) { bx0[u] = LV::load(x + o); bd0[u] = load_dy<T, VEC, DY16>(dy, o); }
        else { bx1[u] = LV::load(x + o); bd1[u] = load_dy<T, VEC, DY16>(dy, o); }
      }
    };
    auto consume = [&](auto sel, int bi) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        A vx[VEC], vd[VEC];
        if constexpr (decltype(sel)::value == 0) { LV::unpack(bx0[u], vx); unpack_dy<T, VEC, DY16>(bd0[u], vd, dydtype); }
        else { LV::unpack(bx1[u], vx); unpack_dy<T, VEC, DY16>(bd1[u], vd, dydtype); }
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const A g = vd[j] * act_bwd<ACT, A>(vx[j] * sa[j] + sb[j]);
          vd[j] = sa[j] * g + (c1[j] * vx[j] + c2[j]);
        }
        if (bi * U + u < rows) store_streaming<LV>(dx + off + (int64_t)(bi * U + u) * step, LV::pack(vd));
      }
    };
    EarlyPartials<A, 2> early;
    A emu = (A)0, ers = (A)0;
    {
      // unconditional, also when the general merge below will be used: a branch here would make the compiler wait
      // for these loads before it issues the next ones
      fetch_partials<A, 2, false>(early, partG, plane, q, p, l);
      const int64_t gidx = early.valid ? n * p.G + l.g_lo + early.gi : 0;  // entry 0 exists: no guard on the loads
      emu = load_scalar_flat<A>(mean, gidx, sdtype, partC);
      ers = load_scalar_flat<A>(rstd, gidx, sdtype, partC);
    }
    lane_params_flat<A, PT, VEC>(sfl.c, w, b, partC, sa, sb);
    issue_order_fence();
    issue(std::integral_constant<int, 0>{}, 0);  // in flight while the group sums are merged
    if (one_round) {
      A ta, tb;
      reduce_sums<A>(early, ta, tb);
      if (early.valid && early.sl == 0) {
        const A s = fast_rcp((A)p.D * (A)p.R);
        const A k1 = (emu * tb - ta) * s * ers * ers * ers;
        sm_mu[early.gi] = emu;
        sm_rs[early.gi] = ers;
        sm_c1[early.gi] = k1;
        sm_c2[early.gi] = -emu * k1 - tb * s * ers;
      }
    } else {
      const int L = merge_lanes(q, p.D);
      const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
      const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
      for (int base = 0; base < l.ng; base += nseg) {
        const int gi = base + seg;
        const bool valid = gi < l.ng;
        const int g = l.g_lo + gi;
        A ta, tb;
        sum_group_partials<A, false>(partG, plane, q, p.G, p.D, n, g, valid, L, sl, ta, tb);
        if (valid && sl == 0) {
          const A mu = load_scalar<A>(mean, n * p.G + g, sdtype);
          const A rs = load_scalar<A>(rstd, n * p.G + g, sdtype);
          const A s = fast_rcp((A)p.D * (A)p.R);
          const A k1 = (mu * tb - ta) * s * rs * rs * rs;
          sm_mu[gi] = mu;
          sm_rs[gi] = rs;
          sm_c1[gi] = k1;
          sm_c2[gi] = -mu * k1 - tb * s * rs;
        }
      }
    }
    __syncthreads();
    if (rows > 0) {
      lane_coeffs<A, VEC, true>(p, l, sm_mu, sm_rs, sm_c1, sm_c2, sa, sb, c1, c2);
      double_buffered(nb, issue, consume);
    }
    __syncthreads();
  }
}

}  // namespace gn
