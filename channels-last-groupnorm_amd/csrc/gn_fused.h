// Single-launch ("resident") GroupNorm kernels: the whole activation tensor is held in the register
// files of the workgroups of one launch, so x (and dy) are read from memory exactly once.
//
//   forward : load tile -> per-tile group moments -> publish -> wait for the tiles that share my
//             groups -> merge -> y = act(x a + b) from registers
//   backward: load tile (x, dy) -> per-tile channel / group sums -> publish -> wait -> merge ->
//             dx from registers; the workgroups of row tile 0 of sample 0 also finish dgamma / dbeta
//
// The launch must be small enough for every workgroup to be resident at once (the host checks this
// against the occupancy the runtime reports and otherwise uses the streaming kernels): a workgroup
// spins on data written by other workgroups of the same launch.
//
// Exchange protocol.  The XCDs' L2 caches are not coherent with each other, and the fences that would
// make ordinary stores visible across them (L2 write-back / invalidate) cost tens of microseconds when
// every workgroup issues them.  So everything that crosses workgroups is written with device-scope
// (write-through) stores and read with device-scope (cache-bypassing) loads, and no fence is used.
//  * Everything that crosses workgroups travels as a 16-byte record {value0, value1, epoch (64 bit)} written by a
//    single 128-bit store and read by a single 128-bit load: per (sample, chunk, group, tile) for the group
//    statistics / group sums, and in the backward per (sample, tile, channel) for the sums that feed dgamma / dbeta.
//    A consumer that sees this call's epoch in a record takes the values it loaded with it.  The epoch is a fresh
//    64-bit value per call, so the workspace never needs clearing, there are no flags, and one memory round trip
//    carries both "ready" and the data.
//    This relies on an aligned 128-bit device-scope store being observed as a whole by an aligned 128-bit
//    device-scope load (single-copy atomicity of a 16-byte access inside one 64-byte sector of the memory channel
//    that owns it).  The instruction set does not promise it in writing; if it did not hold, a consumer could pair a
//    fresh epoch with stale values.  The epoch therefore sits in the LAST two words of the record: a torn access
//    that delivered the words in address order would show stale epoch words, not stale values.
// Polling is bounded (SyncArea::max_spins).  A wait that expires records the epoch in a host-visible status word and
// poisons what depended on it with NaN, and the kernel carries on: the grid always drains.  Only fp32-accumulating
// element types use these kernels (a record has room for two 32-bit values); float64 data takes the streaming kernels.
#pragma once
#include "gn_kernels.h"

namespace gn {

constexpr int kRecFast = 2;  // records a lane keeps in registers while polling
constexpr int kForcedTimeout = -2;  // poll limit that makes every wait give up at once (tests of the failure path)
constexpr int kTailFast = 2;  // channel records a lane of the dgamma / dbeta stage requests ahead of the dx phase
constexpr int kMaxResidentBlocksDev = 4 * kNumCU;

struct SyncArea {
  void *recs;                 // 16-byte records, laid out [N][nchunk][G][tiles]
  unsigned rec_bytes;
  void *crecs;                // backward: 16-byte records {S1, S2, epoch} per (sample, tile, channel) of the whole tensor
  unsigned crec_bytes;
  void *frecs;                // 16-byte records {value0, value1, epoch} per (sample, group): results of the second level
  unsigned frec_bytes;        // (two_level != 0 only)
  int two_level;              // host side only: selects the TWO_LEVEL instantiation of the kernel
  unsigned long long epoch;   // value that marks "written in this call"
  const unsigned long long *generation;  // device counter that replaces the epoch in captured launches (resident_epoch)
  unsigned long long *status; // set to the epoch if a wait of this call timed out
  int max_spins;              // polls allowed per wait
  unsigned long long *trace;  // optional [workgroup][kTracePoints] timestamps (100 MHz wall clock), else null
  int trace_wait;             // stamps wait for outstanding memory operations first
};
constexpr int kTracePoints = 8;
__device__ __forceinline__ void trace_point(const SyncArea &s, int point, float after = 0.f) {
#if GN_TRACE
  if (!s.trace) return;
  // either stamp a phase once its memory operations have completed, or (trace_wait == 0) leave the kernel's
  // own overlap alone and only order the stamp behind the value `after`
  if (s.trace_wait) __builtin_amdgcn_s_waitcnt(0);
  asm volatile("" ::"v"(after));
  if (threadIdx.x == 0) {
    const int64_t b = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
    if (b < kMaxResidentBlocksDev) s.trace[b * kTracePoints + point] = wall_clock64();
  }
#else
  (void)s;
  (void)point;
  (void)after;
#endif
}

// A launch recorded into a HIP graph is replayed with identical kernel arguments, so the host cannot give
// each replay a fresh epoch.  The first captured launch of a capture therefore records a one-thread kernel in
// front of itself that increments a generation word owned by the library (one per device), and the epoch of a
// captured launch is that generation combined with a sequence number the host fixed at capture time (in
// s.epoch): the generation differs between any two replays of any graphs, the sequence number between the
// launches of one graph.  Bit 63 keeps the two families apart: set for captured launches, clear for the host's.
constexpr int kCapturedSeqBits = 24;
__device__ __forceinline__ SyncArea resident_epoch(SyncArea s) {
  constexpr unsigned long long kCaptured = 1ull << 63;
  if (s.generation)
    s.epoch = kCaptured | (*s.generation << kCapturedSeqBits) | (s.epoch & ((1ull << kCapturedSeqBits) - 1));
  else s.epoch &= ~kCaptured;
  if (s.epoch == 0) s.epoch = 1;
  return s;
}

// 128-bit device-scope accesses through a raw buffer descriptor (cache policy sc1)
constexpr int kAuxDeviceScope = 16;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t record_buffer(const SyncArea &s) {
  return __builtin_amdgcn_make_buffer_rsrc(s.recs, 0, (int)s.rec_bytes, 0x27000);
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t channel_record_buffer(const SyncArea &s) {
  return __builtin_amdgcn_make_buffer_rsrc(s.crecs, 0, (int)s.crec_bytes, 0x27000);
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t final_record_buffer(const SyncArea &s) {
  return __builtin_amdgcn_make_buffer_rsrc(s.frecs, 0, (int)s.frec_bytes, 0x27000);
}
__device__ __forceinline__ void record_store(__amdgpu_buffer_rsrc_t r, int64_t idx, float v0, float v1,
                                             unsigned long long epoch) {
  const u32x4 rec = {__builtin_bit_cast(unsigned, v0), __builtin_bit_cast(unsigned, v1), (unsigned)epoch,
                     (unsigned)(epoch >> 32)};
  __builtin_amdgcn_raw_buffer_store_b128(rec, r, (int)(idx * 16), 0, kAuxDeviceScope);
}
__device__ __forceinline__ u32x4 record_load(__amdgpu_buffer_rsrc_t r, int64_t idx) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)(idx * 16), 0, kAuxDeviceScope);
}
__device__ __forceinline__ bool record_ready(const u32x4 &rec, unsigned long long epoch) {
  return rec.z == (unsigned)epoch && rec.w == (unsigned)(epoch >> 32);
}

// Elements behind record (tile t, chunk k, group g): the rows of the tile times the channels of g in chunk k.
// (32-bit arithmetic: channel indices and the rows of a tile fit, and 64-bit multiplies are slow here)
__device__ __forceinline__ float record_count(const Plan &p, int t, int k, int g) {
  const int cc = p.lpr * p.vec;
  const int c_lo = g * p.D > k * cc ? g * p.D : k * cc;
  int c_hi = (g + 1) * p.D < (k + 1) * cc ? (g + 1) * p.D : (k + 1) * cc;
  if (c_hi > (int)p.C) c_hi = (int)p.C;
  const int64_t rem = p.R - (int64_t)t * p.tile_rows;  // t * tile_rows: one 32 x 32 -> 64 multiply
  const int rows = rem < p.tile_rows ? (int)rem : p.tile_rows;
  return (float)(c_hi - c_lo) * (float)rows;
}
// Slot of a record, in 32 bits with 24-bit multiplies: a single-launch kernel has at most kMaxResidentBlocksDev
// workgroups, so (n nchunk + k) and tiles are small, and the host only sizes the record area for G below 2^20.
__device__ __forceinline__ int record_slot(const PartialGeo &q, int G, int n, int t, int k, int g) {
  const int col = __mul24(n, q.nchunk) + k;
  return __mul24(__mul24(col, G) + g, q.tiles) + t;
}

// What a result is replaced by when a wait expired: not a number, so that the call's output cannot pass for one.
__device__ __forceinline__ float poison() { return __builtin_nanf(""); }
// Two-level exchange.  With T row tiles per sample every workgroup polls T records for each group of its chunk: fine for a
// few dozen tiles, but the polling traffic grows with T squared (512 tiles x 16 groups: 8192 records per workgroup, as many
// bytes as the tensor itself per round of polls).  Beyond a bound set by the host, each group's tile records are instead
// merged ONCE, by the workgroup that owns the group -- tile (group index inside the chunk) mod T of the chunk in which
// the group starts -- with all 256 lanes, and published as one final record per (sample, group) that everybody polls.
// One more round trip, a few thousand times less traffic.
__device__ __forceinline__ bool owns_group(const Plan &p, const LanePos &l, int gi) {
  return (l.g_lo + gi) * p.D >= l.cstart && gi - div_by(gi, p.by_tiles) * p.tiles == l.tile;
}
// Sum of two values over the 256 lanes of the workgroup (fixed tree: wavefront, then the four wavefronts in order);
// every lane gets the result.  Uses 8 floats of LDS at `scratch`; the caller's other LDS data is not touched.
template <typename A> __device__ __forceinline__ void block_sum2(A &a, A &b, A *scratch) {
  segment_reduce2(a, b, 64);
  __syncthreads();  // scratch may still be read from a previous use
  if ((int)(threadIdx.x & 63) == segment_leader<A>(64)) {
    scratch[threadIdx.x >> 6] = a;
    scratch[4 + (threadIdx.x >> 6)] = b;
  }
  __syncthreads();
  a = (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
  b = (scratch[4] + scratch[5]) + (scratch[6] + scratch[7]);
}
// Wait for the final record of (sample, group) slot; false (and NaN values) if the wait expires.
__device__ __forceinline__ void poll_final(const SyncArea &s, __amdgpu_buffer_rsrc_t fb, int slot, float &v0, float &v1) {
  int spins = 0;
  while (true) {
    const u32x4 rec = record_load(fb, slot);
    if (record_ready(rec, s.epoch) && s.max_spins != kForcedTimeout) {
      const unsigned u0 = rec.x, u1 = rec.y;
      v0 = __builtin_bit_cast(float, u0);
      v1 = __builtin_bit_cast(float, u1);
      return;
    }
    if (++spins > s.max_spins) {
      *s.status = s.epoch;
      v0 = poison();
      v1 = poison();
      return;
    }
    __builtin_amdgcn_s_sleep(2);
  }
}
// Collect the records of group g (all tiles of the chunks that hold a piece of it) with L lanes: each lane polls its
// own records until they carry this call's epoch, kRecFast at a time (they stay in registers: the round trip that
// finds them ready also brings their values), and hands (value0, value1, count) of each to body.  If a wait expires,
// the lane's records are not this call's: body is handed NaN values first, so that whatever the caller accumulates
// cannot pass for a result.
template <typename BODY>
__device__ __forceinline__ void for_group_records(const SyncArea &s, __amdgpu_buffer_rsrc_t rb, const PartialGeo &q,
                                                  const Plan &p, int64_t n, int g, bool valid, int L, int sl, BODY &&body) {
  int k_lo = 0, nk = 1;
  if (valid) group_chunks(q, p.D, g, k_lo, nk);
  const int P = valid ? q.tiles * nk : 0;
  const int base = record_slot(q, p.G, (int)n, 0, k_lo, g);
  const int kstride = __mul24(p.G, q.tiles);
  int spins = 0;
  for (int e0 = sl; e0 < P; e0 += kRecFast * L) {
    u32x4 rec[kRecFast];
    bool have[kRecFast];
    int idx[kRecFast];
    int kk[kRecFast], tt[kRecFast];
#pragma unroll
    for (int i = 0; i < kRecFast; ++i) {
      const int e = e0 + i * L;
      have[i] = e < P;
      kk[i] = have[i] ? div_by(e, q.by_tiles) : 0;
      tt[i] = have[i] ? e - kk[i] * q.tiles : 0;
      idx[i] = base + __mul24(kk[i], kstride) + tt[i];
    }
    while (true) {
      bool ok = true;
#pragma unroll
      for (int i = 0; i < kRecFast; ++i) rec[i] = record_load(rb, idx[i]);
#pragma unroll
      for (int i = 0; i < kRecFast; ++i) ok = ok && (!have[i] || record_ready(rec[i], s.epoch));
      if (s.max_spins == kForcedTimeout) ok = false;
      if (ok) break;
      if (++spins > s.max_spins) {
        *s.status = s.epoch;
        body(poison(), poison(), 1.0f);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
#pragma unroll
    for (int i = 0; i < kRecFast; ++i) {
      if (have[i]) {
        // copy the lanes out first: __builtin_bit_cast applied directly to a vector element reads element 0
        const unsigned u0 = rec[i].x, u1 = rec[i].y;
        body(__builtin_bit_cast(float, u0), __builtin_bit_cast(float, u1), record_count(p, tt[i], k_lo + kk[i], g));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Resident forward.  NV = register capacity in rows per lane.  Statistics follow the same definitions
// as the streaming kernels (count / mean / M2, biased variance, rstd = 1 / sqrt(var + eps);
// src/gnnhwc/csrc/Welford.h:8-21,66-72, gn_kernel.cu:175,254,291); the per-lane moments are taken in one pass, as
// sums about the lane's own first row.
//   records : {mean, M2, epoch} per (n, chunk, group, tile)
// ---------------------------------------------------------------------------------------------
// ADD: 0 plain forward; 1 a per-(sample, channel) addend only (same register budget as the plain kernel);
// 2 a residual tensor, with or without the addend (holds two tiles while it combines them, like the backward).
constexpr int kAddNone = 0, kAddChannel = 1, kAddResidual = 2;
// Occupancy the register budget is sized for.
constexpr int fused_fwd_waves(int nv, int add) {
  return add == kAddResidual ? (nv <= 4 ? 4 : nv <= 8 ? 3 : nv <= 16 ? 2 : 1) : (nv <= 8 ? 4 : nv <= 16 ? 3 : 2);
}
// TWO_LEVEL: the exchange of a launch with many row tiles per sample (two_level_exchange on the host).  A template
// parameter, not a run-time switch: the code of the form a launch does not use would sit in the middle of the path every
// workgroup executes once, and these kernels are sensitive to their own size.
template <typename T, typename PT, int VEC, int ACT, int NV, int ADD, bool TWO_LEVEL>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(fused_fwd_waves(NV, ADD)))) void fused_fwd_kernel(
    const T *__restrict__ x, T *__restrict__ y, SyncArea sync_arg, const void *w, const void *b, void *mean_out,
    void *rstd_out, int sdtype, int ydtype, acc_t<T> eps, AddArgs add, Plan p) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  const SyncArea sync = resident_epoch(sync_arg);
  __shared__ A sm0[kBlock * VEC];
  __shared__ A sm1[kBlock * VEC];
  const PartialGeo q = producer_geo(p);
  const int64_t n = blockIdx.z;
  const LanePos l = lane_pos(p, n, false);
  const int rows = l.rows;
  const int64_t off = (n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
  const int64_t step = (int64_t)p.rpi * p.C;
  typename LV::raw_t buf[NV];
  trace_point(sync, 0);
  // gamma / beta are needed only after the exchange, but they are requested first and without any branch: a load
  // under a branch makes the compiler drain every outstanding load where the branch joins, and then the statistics
  // below could not start on the first rows while the later ones are still arriving
  A sa[VEC], sb[VEC];
  {
    const int cvi = l.cvi < p.cv ? l.cvi : p.cv - 1;
    lane_params_flat<A, PT, VEC>(cvi * VEC, w, b, sync.recs, sa, sb);
  }
  // ADD: the per-(sample, channel) addend of the lane's channels, requested with the parameters and without branches
  A tb[VEC];
  if constexpr (ADD != kAddNone) {
    const int cvi = l.cvi < p.cv ? l.cvi : p.cv - 1;
    const void *cb = add.channel_bias ? add.channel_bias : sync.recs;
    const int64_t cb0 = add.channel_bias ? n * p.C + (int64_t)cvi * VEC : 0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A v = load_scalar_flat<A>(cb, add.channel_bias ? cb0 + j : 0, add.channel_bias_dtype, sync.recs);
      tb[j] = add.channel_bias ? v : (A)0;
    }
  }
  issue_order_fence();
  if (rows > 0) {
    // every load is unconditional (rows past the lane's last one re-read it): the waits that follow can then
    // count loads exactly, and row u is processed while rows u + 1 ... are still in flight
    if constexpr (ADD == kAddResidual) {
      // (an absent residual would re-read x and be discarded, so that the loads stay free of branches; the host
      // picks the channel-only variant for that case)
      const T *rp = add.residual ? (const T *)add.residual : x;
      const bool has_r = add.residual != nullptr;
      typename LV::raw_t rbuf[NV];
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        const int64_t o = off + (int64_t)clamp_row(u, rows) * step;
        buf[u] = LV::load(x + o);
        rbuf[u] = LV::load(rp + o);
      }
      T *so = (T *)add.sum_out;
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        A vx[VEC], vr[VEC];
        LV::unpack(buf[u], vx);
        LV::unpack(rbuf[u], vr);
#pragma unroll
        for (int j = 0; j < VEC; ++j) vx[j] = (vx[j] + (has_r ? vr[j] : (A)0)) + tb[j];
        buf[u] = LV::pack(vx);  // rounded to T once: the statistics and y are those of the stored sum
        if (so && u < rows) store_streaming<LV>(so + off + (int64_t)u * step, buf[u]);
      }
    } else {
#pragma unroll
      for (int u = 0; u < NV; ++u) buf[u] = LV::load(x + off + (int64_t)clamp_row(u, rows) * step);
      if constexpr (ADD == kAddChannel) {
        T *so = (T *)add.sum_out;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
          A vx[VEC];
          LV::unpack(buf[u], vx);
#pragma unroll
          for (int j = 0; j < VEC; ++j) vx[j] += tb[j];
          buf[u] = LV::pack(vx);
          if (so && u < rows) store_streaming<LV>(so + off + (int64_t)u * step, buf[u]);
        }
      }
    }
  }
  // everything up to the exchange is on the critical path of the whole group; what follows it is not: a wavefront
  // still working towards the exchange goes before one (of another workgroup on the same SIMD) that is past it
  __builtin_amdgcn_s_setprio(2);
  A mean[VEC], m2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) { mean[j] = (A)0; m2[j] = (A)0; }
  if (rows > 0) {
    // One pass, taken row by row as the rows arrive: sums of the deviations from the lane's own first row (a value
    // of the data, so nothing cancels: the pivot form of the moments) and of their squares.  Nothing but a few
    // operations per channel is left to do once the last row is there.
    A k[VEC], s1[VEC], s2[VEC];
    LV::unpack(buf[0], k);
#pragma unroll
    for (int j = 0; j < VEC; ++j) { s1[j] = (A)0; s2[j] = (A)0; }
    // rows past the lane's last one (only in the last tile of a sample) are replaced by the pivot row, whose deviation
    // is exactly zero: one loop serves full and partial tiles, and a full tile only skips this block
    if (rows != NV) {
#pragma unroll
      for (int u = 1; u < NV; ++u)
        if (u >= rows) buf[u] = buf[0];
    }
#pragma unroll
    for (int u = 1; u < NV; ++u) {
      A v[VEC];
      LV::unpack(buf[u], v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const A d = v[j] - k[j];
        s1[j] += d;
        s2[j] += d * d;
      }
    }
    const A inv = fast_rcp((A)rows);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A dm = s1[j] * inv;
      mean[j] = k[j] + dm;
      m2[j] = s2[j] - s1[j] * dm;
    }
  }
  const __amdgpu_buffer_rsrc_t rb = record_buffer(sync);
  trace_point(sync, 1, (float)m2[0]);
  // the reduction and the exchange are one chain of dependent steps that every workgroup of the group waits for:
  // let these wavefronts go first on a SIMD they share with wavefronts of other workgroups that are still streaming
  __builtin_amdgcn_s_setprio(3);
  block_group_moments<A, VEC>(p, l, mean, m2, sm0, sm1, [&](int g, A cnt, A mu, A s2) {
    (void)cnt;  // the consumers recompute it from the geometry
    record_store(rb, record_slot(q, p.G, (int)n, l.tile, l.chunk, g), mu, s2, sync.epoch);
  });
  trace_point(sync, 2);
  if constexpr (TWO_LEVEL) {
    // second level: the groups this workgroup owns, one at a time with all 256 lanes (usually one group or none)
    const __amdgpu_buffer_rsrc_t fb = final_record_buffer(sync);
    const A total = (A)p.D * (A)p.R;
    __shared__ A sm_x[12];
    for (int gi = l.tile; gi < l.ng; gi += p.tiles) {  // uniform over the workgroup
      if (!owns_group(p, l, gi)) continue;
      const int g = l.g_lo + gi;
      A nl = (A)0, kl = (A)0, s1 = (A)0, s2 = (A)0;
      for_group_records(sync, rb, q, p, n, g, true, kBlock, threadIdx.x, [&](float mu, float mm, float cnt) {
        if (nl == (A)0) kl = mu;
        const A d = mu - kl;
        nl += cnt;
        s1 += cnt * d;
        s2 += mm + cnt * d * d;
      });
      const A inv = nl > (A)0 ? fast_rcp(nl) : (A)0;
      const A mean_l = kl + s1 * inv;
      const A m2_l = s2 - s1 * s1 * inv;
      __syncthreads();
      if (threadIdx.x == 0) sm_x[8] = mean_l;  // lane 0 always has a record: the pivot of the merge across lanes
      __syncthreads();
      const A K = sm_x[8];
      const A d = nl > (A)0 ? mean_l - K : (A)0;
      A t1 = nl * d, t2 = m2_l + nl * d * d;
      block_sum2(t1, t2, sm_x);
      if (threadIdx.x == 0) {
        const A dm = t1 * fast_rcp(total);
        const A gmean = K + dm;
        const A rs = fast_rsqrt((t2 - t1 * dm) * fast_rcp(total) + eps);
        record_store(fb, (int)n * p.G + g, gmean, rs, sync.epoch);
        if (mean_out) store_scalar<A>(mean_out, n * p.G + g, sdtype, gmean);
        if (rstd_out) store_scalar<A>(rstd_out, n * p.G + g, sdtype, rs);
      }
    }
    // everybody: one final record per group of the chunk
    for (int gi = threadIdx.x; gi < l.ng; gi += kBlock) {
      float gmean, rs;
      poll_final(sync, fb, (int)n * p.G + l.g_lo + gi, gmean, rs);
      sm0[gi] = gmean;
      sm1[gi] = rs;
    }
    __syncthreads();
  } else {
    // merge the records of the chunk's groups (exact two-pass form, compute_stats_pt2's job:
    // src/gnnhwc/csrc/gn_kernel.cu:226-292); rstd = 1 / sqrt(M2 / n + eps)
    const int L = merge_lanes(q, p.D);
    const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
    const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
    const A total = (A)p.D * (A)p.R;  // elements of a group
    for (int base = 0; base < l.ng; base += nseg) {
      const int gi = base + seg;
      const bool valid = gi < l.ng;
      const int g = l.g_lo + gi;
      // each lane folds its records about the mean of its first one ...
      A nl = (A)0, kl = (A)0, s1 = (A)0, s2 = (A)0;
      for_group_records(sync, rb, q, p, n, g, valid, L, sl, [&](float mu, float mm, float cnt) {
        if (nl == (A)0) kl = mu;
        const A d = mu - kl;
        nl += cnt;
        s1 += cnt * d;
        s2 += mm + cnt * d * d;
      });
      const A inv = nl > (A)0 ? fast_rcp(nl) : (A)0;
      const A mean_l = kl + s1 * inv;
      const A m2_l = s2 - s1 * s1 * inv;
      // ... and the lanes are merged about the first lane's mean
      const A K = __shfl(mean_l, (int)(threadIdx.x & 63 & ~(L - 1)), 64);
      const A d = mean_l - K;
      A t1 = nl * d, t2 = m2_l + nl * d * d;
      segment_reduce2(t1, t2, L);
      if (valid && sl == segment_leader<A>(L)) {
        const A dm = t1 * fast_rcp(total);
        const A gmean = K + dm;
        const A rs = fast_rsqrt((t2 - t1 * dm) * fast_rcp(total) + eps);
        sm0[gi] = gmean;
        sm1[gi] = rs;
        if (l.tile == 0 && g * p.D >= l.cstart) {
          if (mean_out) store_scalar<A>(mean_out, n * p.G + g, sdtype, gmean);
          if (rstd_out) store_scalar<A>(rstd_out, n * p.G + g, sdtype, rs);
        }
      }
    }
    __syncthreads();
  }
  __builtin_amdgcn_s_setprio(0);
  trace_point(sync, 3);
  if (rows > 0) {
    A unused1[VEC], unused2[VEC];
    lane_coeffs<A, VEC, false>(p, l, sm0, sm1, nullptr, nullptr, sa, sb, unused1, unused2);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      if (u < rows) {
        A v[VEC];
        pin(buf[u]);
        LV::unpack(buf[u], v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = act_fwd<ACT, A>(v[j] * sa[j] + sb[j]);
        store_result<T, VEC>(y, off + (int64_t)u * step, v, ydtype);
      }
    }
  }
  trace_point(sync, 4);
}

// ---------------------------------------------------------------------------------------------
// Resident backward.  Same algebra as bwd_reduce_kernel + bwd_dx_kernel
// (src/gnnhwc/csrc/gn_kernel.cu:598-618, 717-727, 783-800, 868-871), with x and dy read once.
//   group records   : {A, B, epoch} per (n, chunk, group, tile) of this launch
//   channel records : {S1, S2, epoch} per (n, tile, channel) of the whole tensor (they feed dgamma / dbeta)
// ---------------------------------------------------------------------------------------------
// XW: 0 keeps the tile of x in registers next to the tile of g' (NV rows each).  XW > 0 keeps g' only and streams x
// through a window of XW rows, twice: once for the sums and once, in the opposite direction (so that the window's
// last rows serve both passes), for dx.  That form holds a tensor half again as large at the price of reading
// (NV - XW) / NV of x a second time: 4 - XW / NV tensors of traffic, against the 5 of the multi-launch backward.
constexpr int fused_bwd_waves(int nv, int xw) {
  return xw > 0 ? (nv <= 24 ? 3 : 2) : (nv <= 4 ? 4 : nv <= 8 ? 3 : nv <= 22 ? 2 : 1);
}
template <typename T, typename PT, int VEC, int ACT, int NV, bool TWO_LEVEL, int XW = 0>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(fused_bwd_waves(NV, XW)))) void fused_bwd_kernel(
    const T *__restrict__ x, const T *__restrict__ dy, T *__restrict__ dx, const void *mean, const void *rstd, int sdtype,
    const void *w, const void *b, SyncArea sync_arg, void *dw, void *db, const void *mean_all, const void *rstd_all,
    int64_t n0, int64_t n_all, Plan p) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  const SyncArea sync = resident_epoch(sync_arg);
  __shared__ A sm1[kBlock * VEC];
  __shared__ A sm2[kBlock * VEC];
  __shared__ A sm_mu[kBlock * VEC];
  __shared__ A sm_rs[kBlock * VEC];
  const PartialGeo q = producer_geo(p);
  const int64_t n = blockIdx.z;
  const LanePos l = lane_pos(p, n, false);
  const __amdgpu_buffer_rsrc_t rb = record_buffer(sync);
  const __amdgpu_buffer_rsrc_t rbc = channel_record_buffer(sync);
  const void *safe = sync.recs;  // readable bytes for loads that only exist to keep the prologue free of branches
  const int rows = l.rows;
  const SafeLane sfl = safe_lane<VEC>(p, l, n);
  const int64_t off = sfl.off;
  const int64_t step = (int64_t)p.rpi * p.C;
  constexpr int NX = XW > 0 ? XW : NV;  // rows of x held at a time; row u lives in bx[u % NX]
  static_assert(XW >= 0 && XW <= NV, "window within the tile");
  typename LV::raw_t bx[NX], bd[NV];
  auto row_offset = [&](int u) { return off + (int64_t)clamp_row(u, sfl.rows) * step; };
  // XW > 0: rows are requested all through the kernel, so their addresses must be cheap to form again: the tile's
  // (uniform) base plus a 32-bit byte offset per lane and row (the host admits only tiles below 2 GiB)
  const int64_t tile_base = (n * p.R + l.row0) * p.C;
  const unsigned lane_byte0 = (unsigned)(((sfl.live ? l.ty : 0) * p.C + sfl.c) * (int)sizeof(T));
  const unsigned step_bytes = (unsigned)(p.rpi * p.C * (int)sizeof(T));
  // (every pass forms them from its own opaque copy of the three terms: offsets kept from one pass for the next
  // would cost a register per row)
  struct RowTerms { unsigned lane0, step; int rows; };
  auto fresh_terms = [&]() {
    RowTerms t{lane_byte0, step_bytes, sfl.rows};
    pin(t.lane0);
    pin(t.step);
    pin(t.rows);
    return t;
  };
  auto tile_row = [&](const T *base, const RowTerms &t, int u) {
    return (const T *)((const char *)(base + tile_base) + (t.lane0 + (unsigned)clamp_row(u, t.rows) * t.step));
  };
  trace_point(sync, 0);
  // the small loads go first: loads return in order, so the statistics and parameters, which the first row's
  // arithmetic needs, must not queue behind the whole tile.  Nothing here is under a branch (idle lanes read valid
  // addresses too), so every later wait counts exactly the loads it needs.
  const StagedStats<A> st = fetch_chunk_stats<A>(mean, rstd, sdtype, p, l, sm_mu, sm_rs, safe);
  A sa[VEC], sb[VEC], c1[VEC], c2[VEC];
  lane_params_flat<A, PT, VEC>(sfl.c, w, b, safe, sa, sb);
  // gamma of the channel this thread handles when the tile's per-channel sums are published: fetched now, so that
  // the load is not part of the serial section between the sums and the record exchange
  A gamma0;
  {
    const int cg = (int)threadIdx.x < l.wch ? threadIdx.x : 0;
    const PT *gp = w ? (const PT *)w + l.cstart + cg : (const PT *)safe;
    const A gv = load_param<PT, A>(gp, 0);
    gamma0 = w ? gv : (A)1;
  }
  issue_order_fence();
  if constexpr (XW == 0) {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int64_t o = row_offset(u);
      bx[u] = LV::load(x + o);
      bd[u] = LV::load(dy + o);
    }
  } else {
    // the window of x first (row 0's arithmetic needs it), then all of dy; the rest of x follows row by row below
    const RowTerms t0 = fresh_terms();
#pragma unroll
    for (int u = 0; u < XW; ++u) bx[u] = LV::load(tile_row(x, t0, u));
#pragma unroll
    for (int u = 0; u < NV; ++u) bd[u] = LV::load(tile_row(dy, t0, u));
  }
  commit_chunk_stats<A>(st, l, sm_mu, sm_rs);
  __builtin_amdgcn_s_setprio(2);  // towards the exchange: ahead of wavefronts that are already past theirs
  __syncthreads();
  trace_point(sync, 1);
  {
    A s1[VEC], s2[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) { s1[j] = (A)0; s2[j] = (A)0; }
    if (rows > 0) {
      lane_coeffs<A, VEC, false>(p, l, sm_mu, sm_rs, nullptr, nullptr, sa, sb, c1, c2);
      // dy is not needed again: its registers keep g' = dy * act'(z) for the dx phase (for 16-bit data
      // rounded to T, the rounding an unfused activation backward applies to the same quantity).
      // Rows past the lane's last one (only in the last tile of a sample; they re-read a valid row of x) get dy = 0,
      // hence g' = 0 and no contribution: one loop serves full and partial tiles, and a full tile only skips this block.
      if (rows != NV) {
        const typename LV::raw_t zero = {};
#pragma unroll
        for (int u = 0; u < NV; ++u)
          if (u >= rows) bd[u] = zero;
      }
      const RowTerms t1 = fresh_terms();
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        A vx[VEC], vd[VEC];
        pin(bx[u % NX]);  // one row at a time: cheap activations otherwise tempt the scheduler into unpacking many
        pin(bd[u]);       // rows ahead, which costs more registers than the tile itself
        LV::unpack(bx[u % NX], vx);
        LV::unpack(bd[u], vd);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if constexpr (XW > 0 && VEC >= 4) {
            // half a row at a time: the temporaries of a costly derivative for a whole row do not fit beside the tile
            if (j == VEC / 2) {
#pragma unroll
              for (int i = 0; i < VEC / 2; ++i) { pin(vd[i]); pin(s1[i]); pin(s2[i]); }
#pragma unroll
              for (int i = VEC / 2; i < VEC; ++i) { pin(vx[i]); pin(vd[i]); }
            }
          }
          const A g = vd[j] * act_bwd<ACT, A>(vx[j] * sa[j] + sb[j]);
          s1[j] += g * vx[j];
          s2[j] += g;
          vd[j] = g;
        }
        bd[u] = LV::pack(vd);
        if constexpr (XW > 0) {
          // the sums are brought up to date row by row: left alone, the scheduler postpones the chains of the window's
          // last rows to the end and keeps their unpacked g' alive until then
#pragma unroll
          for (int j = 0; j < VEC; ++j) { pin(s1[j]); pin(s2[j]); }
          pin(bd[u]);  // packed here and now (the conversion otherwise sinks towards the dx phase, g' staying unpacked)
          if (u + XW < NV) {
            issue_order_fence();  // not before the rows ahead of it are consumed: the slot is the register budget
            bx[u % NX] = LV::load(tile_row(x, t1, u + XW));  // the slot's next row
          }
        }
      }
    }
    trace_point(sync, 6, (float)(s1[0] + s2[0]));
    __builtin_amdgcn_s_setprio(3);  // as in the forward: the serial chain to the exchange goes first
    block_channel_sums<A, VEC>(p, l, s1, s2, sm1, sm2);
  }
  // (channel records are indexed in 32 bits: their area is a few megabytes)
  const int crec_row = __mul24(__mul24((int)(n0 + n), p.tiles) + l.tile, (int)p.C) + l.cstart;
  // publish the tile's per-channel sums and keep gamma-weighted copies for the group sums; the first channel of a
  // thread uses the gamma fetched in the prologue (no load in this serial section), wider chunks load the rest
  if ((int)threadIdx.x < l.wch) {
    const int c = threadIdx.x;
    const A t1 = sm1[c], t2 = sm2[c];
    record_store(rbc, crec_row + c, t1, t2, sync.epoch);
    sm1[c] = gamma0 * t1;
    sm2[c] = gamma0 * t2;
  }
  for (int c = threadIdx.x + kBlock; c < l.wch; c += kBlock) {
    const A t1 = sm1[c], t2 = sm2[c];
    record_store(rbc, crec_row + c, t1, t2, sync.epoch);
    const A gamma = w ? load_param<PT, A>(w, l.cstart + c) : (A)1;
    sm1[c] = gamma * t1;
    sm2[c] = gamma * t2;
  }
  __syncthreads();
  {
    const int L = pow2_ceil_clamped(p.D < l.wch ? p.D : l.wch, 64);
    const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
    const int seg = spread_segment(L), sl = threadIdx.x & (L - 1);
    for (int base = 0; base < l.ng; base += nseg) {
      const int gi = base + seg;
      const int g = l.g_lo + gi;
      const bool valid = gi < l.ng;
      int ca = 0, cb = 0;
      if (valid) group_span(p, l, g, ca, cb);
      A ta = (A)0, tb = (A)0;
      for (int c = ca + sl; c < cb; c += L) { ta += sm1[c]; tb += sm2[c]; }
      segment_reduce2(ta, tb, L);
      if (valid && sl == segment_leader<A>(L)) record_store(rb, record_slot(q, p.G, (int)n, l.tile, l.chunk, g), ta, tb, sync.epoch);
    }
  }
  __syncthreads();
  trace_point(sync, 2);
  if constexpr (TWO_LEVEL) {
    // second level (see owns_group): the groups this workgroup owns, one at a time with all 256 lanes
    const __amdgpu_buffer_rsrc_t fb = final_record_buffer(sync);
    __shared__ A sm_x[8];
    for (int gi = l.tile; gi < l.ng; gi += p.tiles) {  // uniform over the workgroup
      if (!owns_group(p, l, gi)) continue;
      const int g = l.g_lo + gi;
      A ta = (A)0, tb = (A)0;
      for_group_records(sync, rb, q, p, n, g, true, kBlock, threadIdx.x, [&](float ra, float rbv, float) {
        ta += ra;
        tb += rbv;
      });
      block_sum2(ta, tb, sm_x);
      if (threadIdx.x == 0) {
        const A mu = sm_mu[gi];
        const A rs = sm_rs[gi];
        const A s = fast_rcp((A)p.D * (A)p.R);
        const A k1 = (mu * tb - ta) * s * rs * rs * rs;
        record_store(fb, (int)n * p.G + g, k1, -mu * k1 - tb * s * rs, sync.epoch);
      }
    }
    for (int gi = threadIdx.x; gi < l.ng; gi += kBlock) {
      float k1, k2;
      poll_final(sync, fb, (int)n * p.G + l.g_lo + gi, k1, k2);
      sm1[gi] = k1;
      sm2[gi] = k2;
    }
  } else {
    const int L = merge_lanes(q, p.D);
    const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
    const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
    for (int base = 0; base < l.ng; base += nseg) {
      const int gi = base + seg;
      const bool valid = gi < l.ng;
      const int g = l.g_lo + gi;
      A ta = (A)0, tb = (A)0;
      for_group_records(sync, rb, q, p, n, g, valid, L, sl, [&](float ra, float rbv, float) {
        ta += ra;
        tb += rbv;
      });
      segment_reduce2(ta, tb, L);
      if (valid && sl == segment_leader<A>(L)) {
        const A mu = sm_mu[gi];
        const A rs = sm_rs[gi];
        const A s = fast_rcp((A)p.D * (A)p.R);
        const A k1 = (mu * tb - ta) * s * rs * rs * rs;
        sm1[gi] = k1;
        sm2[gi] = -mu * k1 - tb * s * rs;
      }
    }
  }
  __syncthreads();
  // dgamma / dbeta (compute_dweight_dbias, gn_kernel.cu:695-728).  The workgroups of this launch's first sample
  // share the channels of their chunk: a segment of L lanes per channel sums the channel records of every
  // (sample, row tile) pair of the whole tensor.  The records of this launch validate themselves by their epoch
  // (no flags, no waiting for store acknowledgements anywhere); those of earlier launches over other groups of
  // samples are complete because those launches have ended.  The first kTailFast records of a lane are requested
  // here, so that their latency passes behind the dx phase below, and checked after it.
  __builtin_amdgcn_s_setprio(0);
  const bool tail = n == 0 && (dw || db);
  const int pairs = (int)n_all * p.tiles;
  const int TL = pow2_ceil_clamped(pairs, 64);
  const int tlg = __builtin_ctz(TL);
  const int cpp = kBlock >> tlg;  // channels per pass of the workgroup
  const int tslot = threadIdx.x >> tlg, tsl = threadIdx.x & (TL - 1);
  const bool tail_lane = tail && l.tile * cpp + tslot < l.wch;
  const int tail_c = l.cstart + (tail_lane ? l.tile * cpp + tslot : 0);
  const int tail_g = div_by(tail_c, p.by_D);
  u32x4 trec[kTailFast];
  A tmu[kTailFast], trs[kTailFast];
  if (tail) {
#pragma unroll
    for (int i = 0; i < kTailFast; ++i) {
      const int e = tsl + i * TL;
      const int nn = e < pairs ? div_by(e, p.by_tiles) : 0;
      const int t = e < pairs ? e - nn * p.tiles : 0;
      trec[i] = record_load(rbc, __mul24(__mul24(nn, p.tiles) + t, (int)p.C) + tail_c);
      tmu[i] = load_scalar_flat<A>(mean_all, nn * p.G + tail_g, sdtype, safe);
      trs[i] = load_scalar_flat<A>(rstd_all, nn * p.G + tail_g, sdtype, safe);
    }
  }
  trace_point(sync, 3);
  if (rows > 0) {
    lane_group_pairs<A, VEC>(p, l, sm1, sm2, c1, c2);
    if constexpr (XW == 0) {
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        if (u < rows) {
          A vx[VEC], vd[VEC];
          pin(bx[u]);
          LV::unpack(bx[u], vx);
          LV::unpack(bd[u], vd);  // g'
#pragma unroll
          for (int j = 0; j < VEC; ++j) vd[j] = sa[j] * vd[j] + (c1[j] * vx[j] + c2[j]);
          store_streaming<LV>(dx + off + (int64_t)u * step, LV::pack(vd));
        }
      }
    } else {
      // from the last row down: the window still holds rows NV - XW ... NV - 1 of the first pass, and every slot is
      // refilled with the row XW below it as soon as its row is done (unconditionally: the waits count loads exactly)
      const RowTerms t2 = fresh_terms();
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int u = NV - 1 - k;
        A vx[VEC], vd[VEC];
        pin(bx[u % NX]);
        pin(bd[u]);
        LV::unpack(bx[u % NX], vx);
        LV::unpack(bd[u], vd);  // g'
#pragma unroll
        for (int j = 0; j < VEC; ++j) vd[j] = sa[j] * vd[j] + (c1[j] * vx[j] + c2[j]);
        if (u < rows) store_streaming<LV>((T *)tile_row(dx, t2, u), LV::pack(vd));
        if (u >= XW) {
          issue_order_fence();
          bx[u % NX] = LV::load(tile_row(x, t2, u - XW));
        }
      }
    }
  }
  trace_point(sync, 4);
  if (tail) {
    int spins = 0;
    for (int cb = l.tile * cpp; cb < l.wch; cb += p.tiles * cpp) {
      const bool first = cb == l.tile * cpp;
      const int cc = cb + tslot;
      const bool valid = cc < l.wch;
      const int c = l.cstart + (valid ? cc : 0);
      const int g = div_by(c, p.by_D);
      A t1 = (A)0, t2 = (A)0;
      // one (sample, tile) pair: wait until its record is this launch's (if it is this launch's to write) and add it
      auto add = [&](int e, u32x4 rec, A mu, A rs) {
        const int64_t nn = div_by(e, p.by_tiles);
        const int t = e - (int)nn * p.tiles;
        while (valid && nn >= n0 && (!record_ready(rec, sync.epoch) || sync.max_spins == kForcedTimeout)) {
          if (++spins > sync.max_spins) {
            *sync.status = sync.epoch;
            t1 = poison();  // dgamma / dbeta of this channel say so
            t2 = poison();
            break;
          }
          __builtin_amdgcn_s_sleep(2);
          rec = record_load(rbc, (nn * p.tiles + t) * p.C + c);
        }
        const unsigned u0 = rec.x, u1 = rec.y;
        const A s1 = __builtin_bit_cast(float, u0), s2 = __builtin_bit_cast(float, u1);
        t1 += (s1 - mu * s2) * rs;
        t2 += s2;
      };
      int e = tsl;
      if (first) {  // the records requested before the dx phase
#pragma unroll
        for (int i = 0; i < kTailFast; ++i) {
          if (e < pairs) add(e, trec[i], tmu[i], trs[i]);
          e += TL;
        }
      }
      for (; e < pairs; e += TL) {
        const int64_t nn = div_by(e, p.by_tiles);
        const int t = e - (int)nn * p.tiles;
        add(e, record_load(rbc, (nn * p.tiles + t) * p.C + c), load_scalar<A>(mean_all, nn * p.G + g, sdtype),
            load_scalar<A>(rstd_all, nn * p.G + g, sdtype));
      }
      if (!valid) { t1 = (A)0; t2 = (A)0; }
      segment_reduce2(t1, t2, TL);
      if (valid && tsl == segment_leader<A>(TL)) {
        if (dw) store_param<PT, A>(dw, c, t1);
        if (db) store_param<PT, A>(db, c, t2);
      }
    }
    trace_point(sync, 5);
  }
}

}  // namespace gn
