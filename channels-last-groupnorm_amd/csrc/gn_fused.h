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
//    An aligned 128-bit device-scope store is expected to be observed as a whole by an aligned 128-bit device-scope
//    load (single-copy atomicity of a 16-byte access inside one 64-byte sector of the memory channel that owns it),
//    but the instruction set does not promise that in writing, so the protocol does not depend on it: the record
//    validates itself.  Its third word is the low half of the epoch folded with a hash of the two values (record_hash),
//    its fourth the high half: whichever words of a torn access are the stale ones, the record fails validation and
//    is polled again.
// Polling is bounded (SyncArea::max_spins).  When a wait of any lane expires (the workgroup that owes it a record is
// not resident yet: something else holds part of the device), the whole workgroup leaves the fast path at the next
// barrier and finishes its tile the slow way (recover_* below): it takes the records that have arrived, RECOMPUTES the
// others from the kernel's inputs, reads its own rows again from memory and stores its results; a host-visible status
// word notes that it happened.  Every workgroup publishes its own records before it waits for anybody else's, so
// workgroups that are scheduled later still find everything they need: the grid always drains and every output is
// correct, only later.  Only fp32-accumulating element types use these kernels (a record has room for two 32-bit
// values); float64 data takes the streaming kernels.
#pragma once
#include "gn_kernels.h"

namespace gn {

constexpr int kRecFast = 2;  // records a lane keeps in registers while polling
constexpr int kForcedTimeout = -2;  // poll limit that makes every wait give up at once, ready or not, and every record be
                                    // recomputed (tests of the recovery path)
constexpr int kTailFast = 2;  // channel records a lane of the dgamma / dbeta stage requests ahead of the dx phase
constexpr int kMaxResidentBlocksDev = 4 * kNumCU;
// ADD (forward with fused additions): 0 plain forward; 1 a per-(sample, channel) addend only (same register budget as the plain kernel);
// 2 a residual tensor, with or without the addend (holds two tiles while it combines them, like the backward).
constexpr int kAddNone = 0, kAddChannel = 1, kAddResidual = 2;
// The sum of a forward with fused additions is stored while the rows arrive -- unless it replaces one of its own
// inputs in place: then it is stored after the exchange, with y, so that a workgroup that has not published its record
// has not overwritten anything a recomputation of that record would read.
template <typename T> __device__ __forceinline__ bool sum_after_exchange(const T *x, const AddArgs &add) {
  return add.sum_out != nullptr && ((const void *)add.sum_out == (const void *)x || (const void *)add.sum_out == add.residual);
}

struct SyncArea {
  void *area;                 // the 16-byte records of the launch, three arrays inside one region of area_bytes bytes:
  unsigned area_bytes;
  unsigned rec_first;         // index of the first of the records laid out [N][nchunk][G][tiles]
  unsigned crec_first;        // backward: records {S1, S2, epoch} per (sample, tile, channel) of the whole tensor
  unsigned frec_first;        // records {value0, value1, epoch} per (sample, group): results of the second level
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
// One array of records: the buffer descriptor of the whole region (the same for the three arrays, so that it occupies
// four scalar registers once) and the index of the array's first record in it.
struct RecordArray {
  __amdgpu_buffer_rsrc_t rsrc;
  int first;
};
__device__ __forceinline__ __amdgpu_buffer_rsrc_t record_region(const SyncArea &s) {
  return __builtin_amdgcn_make_buffer_rsrc(s.area, 0, (int)s.area_bytes, 0x27000);
}
__device__ __forceinline__ RecordArray record_buffer(const SyncArea &s) { return {record_region(s), (int)s.rec_first}; }
__device__ __forceinline__ RecordArray channel_record_buffer(const SyncArea &s) { return {record_region(s), (int)s.crec_first}; }
__device__ __forceinline__ RecordArray final_record_buffer(const SyncArea &s) { return {record_region(s), (int)s.frec_first}; }
// The third word of a record carries the low half of the epoch folded with a hash of the two values: a record whose four
// words were not written together (an access observed in pieces, should that ever happen) does not validate, whichever
// of its words are the stale ones, and is simply polled again.
__device__ __forceinline__ unsigned record_hash(unsigned u0, unsigned u1) { return u0 ^ __builtin_amdgcn_alignbit(u1, u1, 13); }
__device__ __forceinline__ void record_store(const RecordArray &r, int64_t idx, float v0, float v1, unsigned long long epoch) {
  const unsigned u0 = __builtin_bit_cast(unsigned, v0), u1 = __builtin_bit_cast(unsigned, v1);
  const u32x4 rec = {u0, u1, (unsigned)epoch ^ record_hash(u0, u1), (unsigned)(epoch >> 32)};
  __builtin_amdgcn_raw_buffer_store_b128(rec, r.rsrc, ((int)idx + r.first) * 16, 0, kAuxDeviceScope);
}
__device__ __forceinline__ u32x4 record_load(const RecordArray &r, int64_t idx) {
  return __builtin_amdgcn_raw_buffer_load_b128(r.rsrc, ((int)idx + r.first) * 16, 0, kAuxDeviceScope);
}
__device__ __forceinline__ bool record_ready(const u32x4 &rec, unsigned long long epoch) {
  return (rec.z ^ record_hash(rec.x, rec.y)) == (unsigned)epoch && rec.w == (unsigned)(epoch >> 32);
}

// Lanes per group for the exchange: a lane takes kRecFast records per round trip, so half as many lanes as a group has
// records serve it in one round -- and twice as many groups of the chunk are merged side by side, which for chunks that
// hold many small groups (64 channels of groups of 10) saves the second pass over the groups and its round trip.
__device__ __forceinline__ int exchange_lanes(const PartialGeo &q, int D) {
  const int records = q.tiles * (div_by(D - 1, q.by_chunk) + 2);
  return pow2_ceil_clamped((records + kRecFast - 1) / kRecFast, 64);
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
__device__ __forceinline__ void record_values(const u32x4 &rec, float &v0, float &v1) {
  // copy the lanes out first: __builtin_bit_cast applied directly to a vector element reads element 0
  const unsigned u0 = rec.x, u1 = rec.y;
  v0 = __builtin_bit_cast(float, u0);
  v1 = __builtin_bit_cast(float, u1);
}
// Wait for the final record of (sample, group) slot.  If the wait expires, `late` is set and the values mean nothing.
__device__ __forceinline__ void poll_final(const SyncArea &s, RecordArray fb, int slot, float &v0, float &v1,
                                           bool &late) {
  int spins = 0;
  while (true) {
    const u32x4 rec = record_load(fb, slot);
    record_values(rec, v0, v1);
    if (record_ready(rec, s.epoch) && s.max_spins != kForcedTimeout) return;
    if (__builtin_expect(++spins > s.max_spins, 0)) {
      late = true;
      return;
    }
    __builtin_amdgcn_s_sleep(2);
  }
}
// Collect the records of group g (all tiles of the chunks that hold a piece of it) with L lanes: each lane polls its
// own records until they carry this call's epoch, kRecFast at a time (they stay in registers: the round trip that
// finds them ready also brings their values), and hands (value0, value1, count) of each to body.  If the lane's
// wait expires, `late` is set and the lane stops: what it has accumulated means nothing, and the workgroup takes the
// recovery path at its next barrier.
template <typename BODY>
__device__ __forceinline__ void for_group_records(const SyncArea &s, RecordArray rb, const PartialGeo &q,
                                                  const Plan &p, int64_t n, int g, bool valid, int L, int sl, bool &late,
                                                  BODY &&body) {
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
      if (__builtin_expect(++spins > s.max_spins, 0)) {
        late = true;
        return;
      }
      __builtin_amdgcn_s_sleep(2);
    }
#pragma unroll
    for (int i = 0; i < kRecFast; ++i) {
      if (have[i]) {
        float v0, v1;
        record_values(rec[i], v0, v1);
        body(v0, v1, record_count(p, tt[i], k_lo + kk[i], g));
      }
    }
  }
}

// ---- recovery: a workgroup one of whose waits expired finishes its tile without the fast path -----------------------
// Cold code, reached by a branch that is uniform over the workgroup, after which the registers of the fast path are
// dead (the tile is read again from memory).  The workgroup walks the records it needs, 256 at a time: those that
// have arrived are taken, each of the others is recomputed from the kernel's inputs by all 256 lanes together, with
// sums in double precision (so that sums of another shape than the fast path's fixed trees lose nothing against
// them).  A recomputed value is used only if the record has STILL not arrived afterwards: then its workgroup had
// not published when the recomputation finished reading, hence had not started to write results either (a
// workgroup does not store results before it has seen its own record through memory, with all the others) -- which
// matters when the output replaces an input in place.  If the record has arrived meanwhile, the record is taken.
struct RecoveryLds {
  float v0[kBlock], v1[kBlock];  // a round of records: values, and whether they had arrived
  int ok[kBlock];
  double sums[8];                // cross-wavefront stage of block_sum2_f64
  int late;                      // set by any lane whose wait expired (the fast path reads it after a barrier)
  int late_tail;                 // the same for the waits of the dgamma / dbeta stage
};
// Rows [r0, r1) of row tile t and channels [c_lo, c_hi) of group g inside chunk k: the elements behind a record.
struct RecordSpan {
  int64_t r0, r1;
  int c_lo, c_hi;
};
__device__ __forceinline__ RecordSpan record_span(const Plan &p, int t, int k, int g) {
  const int cc = p.lpr * p.vec;
  RecordSpan sp;
  sp.c_lo = g * p.D > k * cc ? g * p.D : k * cc;
  sp.c_hi = (g + 1) * p.D < (k + 1) * cc ? (g + 1) * p.D : (k + 1) * cc;
  if (sp.c_hi > (int)p.C) sp.c_hi = (int)p.C;
  sp.r0 = (int64_t)t * p.tile_rows;
  sp.r1 = sp.r0 + p.tile_rows < p.R ? sp.r0 + p.tile_rows : p.R;
  return sp;
}
// Sum of two doubles over the 256 lanes (fixed tree); every lane gets the totals.
__device__ __forceinline__ void block_sum2_f64(double &a, double &b, double *scratch) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const double oa = __shfl_xor(a, m, 64), ob = __shfl_xor(b, m, 64);
    a += oa;
    b += ob;
  }
  __syncthreads();  // scratch may still be read from a previous use
  if ((threadIdx.x & 63) == 0) {
    scratch[threadIdx.x >> 6] = a;
    scratch[4 + (threadIdx.x >> 6)] = b;
  }
  __syncthreads();
  a = (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
  b = (scratch[4] + scratch[5]) + (scratch[6] + scratch[7]);
}
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
// The kernel's argument block, read again from the kernarg segment through a pointer the compiler cannot see through.
// A kernel's arguments are loaded where it starts; code at its far end that used those copies would keep them in
// scalar registers (or spill and restore them) all the way through the fast path.  P must be the kernel's only parameter.
template <typename P> __device__ __forceinline__ P reread_kernel_args() {
  static_assert(sizeof(P) % 4 == 0, "whole 32-bit words");
  const __attribute__((address_space(4))) uint32_t *src =
      (const __attribute__((address_space(4))) uint32_t *)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(src));
  P a;
  uint32_t *dst = (uint32_t *)&a;
#pragma unroll
  for (unsigned i = 0; i < sizeof(P) / 4; ++i) dst[i] = src[i];
  return a;
}
// A zero the compiler cannot see through (see lane_pos).
__device__ __forceinline__ int opaque_zero() {
  int z = 0;
  asm volatile("" : "+s"(z));
  return z;
}
__device__ __forceinline__ float uniform(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
}
// One round of the walk: lane i loads record slot_of(e0 + i) (for e0 + i < count) and the round's values and arrival
// flags are left in LDS for everybody.  arrived(e, rec) decides whether a loaded record counts as there.
template <typename SLOT, typename ARRIVED>
__device__ __forceinline__ void load_record_round(RecordArray rb, RecoveryLds &r, int e0, int count, SLOT &&slot_of,
                                                  ARRIVED &&arrived) {
  const int e = e0 + (int)threadIdx.x;
  const bool have = e < count;
  const u32x4 rec = record_load(rb, have ? slot_of(e) : slot_of(e0));
  __syncthreads();  // the previous round has been consumed
  record_values(rec, r.v0[threadIdx.x], r.v1[threadIdx.x]);
  r.ok[threadIdx.x] = have && arrived(e, rec) ? 1 : 0;
  __syncthreads();
}
// After a recomputation (every lane holds the same v0, v1): look at the record once more and prefer it if it has
// arrived meanwhile.  Uniform over the workgroup.
__device__ __forceinline__ void prefer_arrived(const SyncArea &s, RecordArray rb, RecoveryLds &r, int64_t slot,
                                               float &v0, float &v1) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // every input the recomputation read is here before the record is read again
  __syncthreads();
  if (threadIdx.x == 0) {
    const u32x4 again = record_load(rb, slot);
    r.ok[0] = record_ready(again, s.epoch) && s.max_spins != kForcedTimeout ? 1 : 0;
    record_values(again, r.v0[0], r.v1[0]);
  }
  __syncthreads();
  if (uniform(r.ok[0])) {
    v0 = uniform(r.v0[0]);
    v1 = uniform(r.v1[0]);
  }
  __syncthreads();  // r.*[0] may be rewritten
}

// Element (row r, channel c) of sample n of the tensor a forward normalises: x, or with fused additions the sum
// (x + residual) + channel_bias rounded to T once, exactly as the fast path forms it.
template <typename T, int ADD>
__device__ __forceinline__ float normalised_input(const T *x, const AddArgs &add, const Plan &p, int64_t n, int64_t r, int c) {
  using L1 = LaneVec<T, 1>;
  const int64_t e = (n * p.R + r) * p.C + c;
  float v[1];
  L1::unpack(L1::load(x + e), v);
  if constexpr (ADD != kAddNone) {
    float vr[1] = {0.f};
    if (add.residual) L1::unpack(L1::load((const T *)add.residual + e), vr);
    const float tb = add.channel_bias ? load_scalar<float>(add.channel_bias, n * p.C + c, add.channel_bias_dtype) : 0.f;
    v[0] = (v[0] + vr[0]) + tb;
    const typename L1::raw_t packed = L1::pack(v);
    L1::unpack(packed, v);
  }
  return v[0];
}
// {mean, M2} of the elements behind forward record (t, k, g) of sample n, by the whole workgroup.
template <typename T, int ADD>
__device__ __forceinline__ void recompute_fwd_record(const T *x, const AddArgs &add, const Plan &p, int64_t n, int t, int k,
                                                     int g, double *scratch, float &mu, float &m2) {
  const RecordSpan sp = record_span(p, t, k, g);
  const int nc = sp.c_hi - sp.c_lo;
  const int64_t cnt = (sp.r1 - sp.r0) * nc;
  const double K = normalised_input<T, ADD>(x, add, p, n, sp.r0, sp.c_lo);
  double s1 = 0.0, s2 = 0.0;
#pragma nounroll
  for (int64_t i = threadIdx.x; i < cnt; i += kBlock) {
    const int64_t r = i / nc;
    const int c = (int)(i - r * nc);
    const double d = (double)normalised_input<T, ADD>(x, add, p, n, sp.r0 + r, sp.c_lo + c) - K;
    s1 += d;
    s2 += d * d;
  }
  block_sum2_f64(s1, s2, scratch);
  const double dm = s1 / (double)cnt;
  mu = (float)(K + dm);
  m2 = (float)(s2 - s1 * dm);
}
// gamma, and the normalisation coefficients a = rstd gamma, b = beta - mean a, of channel c.
template <typename PT>
__device__ __forceinline__ void channel_coeffs(const void *w, const void *b, int c, float mu, float rs, float &gamma, float &a,
                                               float &bb) {
  gamma = w ? load_param<PT, float>(w, c) : 1.f;
  const float beta = b ? load_param<PT, float>(b, c) : 0.f;
  a = rs * gamma;
  bb = beta - mu * a;
}
// Backward group record (t, k, g) of the sample at xs / dys: {sum_c gamma_c sum g' x, sum_c gamma_c sum g'} with
// g' = dy act'(x a_c + b_c), by the whole workgroup.  mu, rs: the group's statistics.
// Pointer to element e of a gradient that is stored in T or (DY16) in a 16-bit type, as a T pointer that load_dy accepts.
template <typename T, bool DY16> __device__ __forceinline__ const T *dy_at(const T *dy, int64_t e) {
  return DY16 ? (const T *)((const uint16_t *)dy + e) : dy + e;
}
template <typename T, typename PT, int ACT, bool DY16>
__device__ __forceinline__ void recompute_bwd_record(const T *xs, const T *dys, int dydtype, const void *w, const void *b,
                                                     const Plan &p, int t, int k, int g, float mu, float rs, double *scratch,
                                                     float &va, float &vb) {
  using L1 = LaneVec<T, 1>;
  const RecordSpan sp = record_span(p, t, k, g);
  const int nc = sp.c_hi - sp.c_lo;
  const int64_t cnt = (sp.r1 - sp.r0) * nc;
  double ta = 0.0, tb = 0.0;
#pragma nounroll
  for (int64_t i = threadIdx.x; i < cnt; i += kBlock) {
    const int64_t r = i / nc;
    const int c = sp.c_lo + (int)(i - r * nc);
    float gamma, a, bb, vx[1];
    channel_coeffs<PT>(w, b, c, mu, rs, gamma, a, bb);
    L1::unpack(L1::load(xs + (sp.r0 + r) * p.C + c), vx);
    const float vd = load_dy_scalar<T, DY16>(dys, (sp.r0 + r) * p.C + c, dydtype);
    const float gp = vd * act_bwd<ACT, float>(vx[0] * a + bb);
    ta += (double)gamma * ((double)gp * (double)vx[0]);
    tb += (double)gamma * (double)gp;
  }
  block_sum2_f64(ta, tb, scratch);
  va = (float)ta;
  vb = (float)tb;
}
// Backward channel record (tile t, channel c) of the sample at xs / dys: {sum g' x, sum g'} over the tile's rows.
template <typename T, int ACT, bool DY16>
__device__ __forceinline__ void recompute_channel_record(const T *xs, const T *dys, int dydtype, const Plan &p, int t, int c,
                                                         float a, float bb, double *scratch, float &v0, float &v1) {
  using L1 = LaneVec<T, 1>;
  const int64_t r0 = (int64_t)t * p.tile_rows;
  const int64_t r1 = r0 + p.tile_rows < p.R ? r0 + p.tile_rows : p.R;
  double S1 = 0.0, S2 = 0.0;
#pragma nounroll
  for (int64_t r = r0 + threadIdx.x; r < r1; r += kBlock) {
    float vx[1];
    L1::unpack(L1::load(xs + r * p.C + c), vx);
    const float vd = load_dy_scalar<T, DY16>(dys, r * p.C + c, dydtype);
    const float gp = vd * act_bwd<ACT, float>(vx[0] * a + bb);
    S1 += (double)gp * (double)vx[0];
    S2 += (double)gp;
  }
  block_sum2_f64(S1, S2, scratch);
  v0 = (float)S1;
  v1 = (float)S2;
}
// The records of group g of sample n, one after the other (uniform over the workgroup): body(v0, v1, count) gets each,
// as it arrived or as recompute(t, k, v0, v1) rebuilt it.
template <typename BODY, typename RECOMPUTE>
__device__ __forceinline__ void recover_group_records(const SyncArea &s, RecordArray rb, RecoveryLds &r,
                                                      const PartialGeo &q, const Plan &p, int64_t n, int g, BODY &&body,
                                                      RECOMPUTE &&recompute) {
  int k_lo = 0, nk = 1;
  group_chunks(q, p.D, g, k_lo, nk);
  const int P = q.tiles * nk;
  auto slot_of = [&](int e) {
    const int kk = e / q.tiles;
    return record_slot(q, p.G, (int)n, e - kk * q.tiles, k_lo + kk, g);
  };
#pragma nounroll
  for (int e0 = 0; e0 < P; e0 += kBlock) {
    load_record_round(rb, r, e0, P, slot_of,
                      [&](int, const u32x4 &rec) { return record_ready(rec, s.epoch) && s.max_spins != kForcedTimeout; });
    const int m = P - e0 < kBlock ? P - e0 : kBlock;
#pragma nounroll
    for (int i = 0; i < m; ++i) {
      const int e = e0 + i;
      const int kk = e / q.tiles;
      const int t = e - kk * q.tiles, k = k_lo + kk;
      float v0 = uniform(r.v0[i]), v1 = uniform(r.v1[i]);
      if (!uniform(r.ok[i])) {
        recompute(t, k, v0, v1);
        prefer_arrived(s, rb, r, slot_of(e), v0, v1);
      }
      body(v0, v1, record_count(p, t, k, g));
    }
  }
}

// The rest of a forward workgroup's work after an expired wait: the statistics of the chunk's groups from the tile
// records (or from the input where they are missing), then the workgroup's own rows, read again from memory.
template <typename T, typename PT, int VEC, int ACT, int ADD, bool TWO_LEVEL>
__device__ __forceinline__ void recover_fwd(const T *x, T *y, const SyncArea &sync, const void *w, const void *b, void *mean_out,
                                            void *rstd_out, int sdtype, int ydtype, float eps, const AddArgs &add, const Plan &p,
                                            RecoveryLds &r, float *sm_mu, float *sm_rs) {
  using LV = LaneVec<T, VEC>;
  const int salt = opaque_zero();
  const int64_t n = blockIdx.z + salt;
  const LanePos l = lane_pos<true>(p, n, false, salt);  // again: nothing of the fast path's is kept alive for this path
  const PartialGeo q = producer_geo(p);
  const RecordArray rb = record_buffer(sync);
  if (threadIdx.x == 0) *sync.status = sync.epoch;
#pragma nounroll
  for (int gi = 0; gi < l.ng; ++gi) {
    const int g = l.g_lo + gi;
    double nl = 0.0, K = 0.0, s1 = 0.0, s2 = 0.0;
    recover_group_records(
        sync, rb, r, q, p, n, g,
        [&](float mu, float mm, float cnt) {
          if (nl == 0.0) K = mu;
          const double d = (double)mu - K;
          nl += cnt;
          s1 += cnt * d;
          s2 += mm + cnt * d * d;
        },
        [&](int t, int k, float &v0, float &v1) { recompute_fwd_record<T, ADD>(x, add, p, n, t, k, g, r.sums, v0, v1); });
    const double dm = s1 / nl;
    const float gmean = (float)(K + dm);
    const float rs = (float)(1.0 / sqrt((s2 - s1 * dm) / nl + (double)eps));
    if (threadIdx.x == 0) {
      sm_mu[gi] = gmean;
      sm_rs[gi] = rs;
      const bool owner = TWO_LEVEL ? owns_group(p, l, gi) : l.tile == 0 && g * p.D >= l.cstart;
      if (owner) {
        if (mean_out) store_scalar<float>(mean_out, n * p.G + g, sdtype, gmean);
        if (rstd_out) store_scalar<float>(rstd_out, n * p.G + g, sdtype, rs);
        // (two-level exchange: the workgroups that wait for this group's final record get it after all)
        if (TWO_LEVEL) record_store(final_record_buffer(sync), (int)n * p.G + g, gmean, rs, sync.epoch);
      }
    }
  }
  __syncthreads();
  if (l.rows > 0) {
    float sa[VEC], sb[VEC], unused1[VEC], unused2[VEC], tb[VEC];
    lane_params_flat<float, PT, VEC>(l.cvi * VEC, w, b, sync.area, sa, sb);
    lane_coeffs<float, VEC, false>(p, l, sm_mu, sm_rs, nullptr, nullptr, sa, sb, unused1, unused2);
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      tb[j] = ADD != kAddNone && add.channel_bias
                  ? load_scalar<float>(add.channel_bias, n * p.C + (int64_t)l.cvi * VEC + j, add.channel_bias_dtype)
                  : 0.f;
    const int64_t off = (n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
    const int64_t step = (int64_t)p.rpi * p.C;
    const bool sum_late = sum_after_exchange<T>(x, add);
#pragma nounroll
    for (int u = 0; u < l.rows; ++u) {
      float v[VEC];
      typename LV::raw_t raw = LV::load(x + off + (int64_t)u * step);
      LV::unpack(raw, v);
      if constexpr (ADD != kAddNone) {
        float vr[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) vr[j] = 0.f;
        if (add.residual) LV::unpack(LV::load((const T *)add.residual + off + (int64_t)u * step), vr);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = (v[j] + vr[j]) + tb[j];
        raw = LV::pack(v);
        if (add.sum_out && sum_late) store_streaming<LV>((T *)add.sum_out + off + (int64_t)u * step, raw);
        LV::unpack(raw, v);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = act_fwd<ACT, float>(v[j] * sa[j] + sb[j]);
      store_result<T, VEC>(y, off + (int64_t)u * step, v, ydtype);
    }
  }
}

// The same for a backward workgroup, up to and including its rows of dx: the group sums of the chunk's groups from the
// tile records (or from x and dy where they are missing) give the coefficients, then dx row by row from memory.
template <typename T, typename PT, int VEC, int ACT, bool TWO_LEVEL, bool DY16>
__device__ __forceinline__ void recover_bwd_dx(const T *x, const T *dy, T *dx, int dydtype, const void *mean, const void *rstd,
                                               int sdtype, const void *w, const void *b, const SyncArea &sync, const Plan &p,
                                               RecoveryLds &r, const float *sm_mu, const float *sm_rs, float *sm_k1,
                                               float *sm_k2) {
  using LV = LaneVec<T, VEC>;
  const int salt = opaque_zero();
  const int64_t n = blockIdx.z + salt;
  const LanePos l = lane_pos<true>(p, n, false, salt);  // again: nothing of the fast path's is kept alive for this path
  const PartialGeo q = producer_geo(p);
  const RecordArray rb = record_buffer(sync);
  if (threadIdx.x == 0) *sync.status = sync.epoch;
  const int64_t sample = n * p.R * p.C;
#pragma nounroll
  for (int gi = 0; gi < l.ng; ++gi) {
    const int g = l.g_lo + gi;
    const float mu = uniform(sm_mu[gi]), rs = uniform(sm_rs[gi]);
    double ta = 0.0, tb = 0.0;
    recover_group_records(
        sync, rb, r, q, p, n, g,
        [&](float ra, float rbv, float) {
          ta += ra;
          tb += rbv;
        },
        [&](int t, int k, float &v0, float &v1) {
          recompute_bwd_record<T, PT, ACT, DY16>(x + sample, dy_at<T, DY16>(dy, sample), dydtype, w, b, p, t, k, g, mu, rs, r.sums, v0, v1);
        });
    const double sc = 1.0 / ((double)p.D * (double)p.R);
    const double k1 = ((double)mu * tb - ta) * sc * (double)rs * (double)rs * (double)rs;
    const double k2 = -(double)mu * k1 - tb * sc * (double)rs;
    __syncthreads();
    if (threadIdx.x == 0) {
      sm_k1[gi] = (float)k1;
      sm_k2[gi] = (float)k2;
      if (TWO_LEVEL && owns_group(p, l, gi)) record_store(final_record_buffer(sync), (int)n * p.G + g, (float)k1, (float)k2, sync.epoch);
    }
  }
  __syncthreads();
  if (l.rows > 0) {
    float sa[VEC], sb[VEC], c1[VEC], c2[VEC];
    lane_params_flat<float, PT, VEC>(l.cvi * VEC, w, b, sync.area, sa, sb);
    lane_coeffs<float, VEC, true>(p, l, sm_mu, sm_rs, sm_k1, sm_k2, sa, sb, c1, c2);
    const int64_t off = (n * p.R + l.row0 + l.ty) * p.C + (int64_t)l.cvi * VEC;
    const int64_t step = (int64_t)p.rpi * p.C;
#pragma nounroll
    for (int u = 0; u < l.rows; ++u) {
      float vx[VEC], vd[VEC];
      LV::unpack(LV::load(x + off + (int64_t)u * step), vx);
      unpack_dy<T, VEC, DY16>(load_dy<T, VEC, DY16>(dy, off + (int64_t)u * step), vd, dydtype);
#pragma unroll
      for (int j = 0; j < VEC; ++j) vd[j] = vd[j] * act_bwd<ACT, float>(vx[j] * sa[j] + sb[j]);
      // (g' passes through T as on the fast path, where it waits in registers in packed form)
      const typename LV::raw_t gp = LV::pack(vd);
      LV::unpack(gp, vd);
#pragma unroll
      for (int j = 0; j < VEC; ++j) vd[j] = sa[j] * vd[j] + (c1[j] * vx[j] + c2[j]);
      store_streaming<LV>(dx + off + (int64_t)u * step, LV::pack(vd));
    }
  }
}

// Which channels a workgroup of the launch's first sample finishes dgamma / dbeta for.  The C channels are cut into
// blocks of cpp channels (cpp lanes segments of a workgroup work side by side, each with as many lanes as there are
// (sample, tile) pairs, 64 at most); block s lies in chunk s / bpc.  Workgroup (tile, chunk) takes the blocks
// chunk * tiles + tile, that + tiles * nchunk, ...: the blocks go to the workgroups with the LOWEST linear index, the
// first to be dispatched and the first to be done with their own rows, whatever chunk the block belongs to -- a
// workgroup dispatched last (on a CU that serves two others first) then has nothing left to do after its dx.
struct TailBlocks {
  int first, stride, total;  // this workgroup's blocks: first, first + stride, ... below total
  int bpc_log2;              // log2 of the blocks per chunk
  int chunk_channels;        // channels of a full chunk
};
__device__ __forceinline__ TailBlocks tail_blocks(const Plan &p, const LanePos &l, int cpp) {
  TailBlocks t;
  t.chunk_channels = p.lpr * p.vec;  // a power of two (the host admits no other chunk width), as is cpp
  const int bpc = t.chunk_channels > cpp ? t.chunk_channels >> __builtin_ctz(cpp) : 1;
  t.bpc_log2 = __builtin_ctz(bpc);
  t.first = l.chunk * p.tiles + l.tile;
  t.stride = p.tiles * p.nchunk;
  t.total = p.nchunk << t.bpc_log2;
  return t;
}
// Block s: its first channel and how many of its cpp channels exist (the last chunk of a row may be narrower).
__device__ __forceinline__ void tail_block_channels(const Plan &p, const TailBlocks &t, int s, int cpp, int &c0, int &count) {
  const int k = s >> t.bpc_log2;
  c0 = k * t.chunk_channels + (s & ((1 << t.bpc_log2) - 1)) * cpp;
  const int chunk_end = (k + 1) * t.chunk_channels < (int)p.C ? (k + 1) * t.chunk_channels : (int)p.C;
  count = chunk_end - c0 < cpp ? chunk_end - c0 : cpp;
  if (count < 0) count = 0;
}

// dgamma / dbeta of the channels this workgroup finishes, after an expired wait of that stage: every channel record
// of the whole tensor that feeds them is taken as it arrived, or rebuilt from x and dy.  Records of samples before n0
// were written by launches that have ended.  x / dy point at sample n0.
template <typename T, typename PT, int ACT, bool DY16>
__device__ __forceinline__ void recover_bwd_tail(const T *x, const T *dy, int dydtype, const void *w, const void *b, const void *mean_all,
                                                 const void *rstd_all, int sdtype, const SyncArea &sync, const Plan &p,
                                                 RecoveryLds &r, int64_t n0, int64_t n_all, void *dw, void *db) {
  const int salt = opaque_zero();
  const LanePos l = lane_pos<true>(p, blockIdx.z + salt, false, salt);
  const int cpp = kBlock / pow2_ceil_clamped((int)n_all * p.tiles, 64);  // channels per pass of the workgroup, as on the fast path
  const RecordArray rbc = channel_record_buffer(sync);
  if (threadIdx.x == 0) *sync.status = sync.epoch;
  const int pairs = (int)n_all * p.tiles;
  const TailBlocks tb = tail_blocks(p, l, cpp);
#pragma nounroll
  for (int s = tb.first; s < tb.total; s += tb.stride) {
    int c0, count;
    tail_block_channels(p, tb, s, cpp, c0, count);
#pragma nounroll
    for (int cc = 0; cc < count; ++cc) {
      const int c = c0 + cc;
      const int g = c / p.D;
      double t1 = 0.0, t2 = 0.0;
      auto slot_of = [&](int e) { return e * (int)p.C + c; };  // e = sample * tiles + tile
#pragma nounroll
      for (int e0 = 0; e0 < pairs; e0 += kBlock) {
        load_record_round(rbc, r, e0, pairs, slot_of, [&](int e, const u32x4 &rec) {
          return e / p.tiles < n0 || (record_ready(rec, sync.epoch) && sync.max_spins != kForcedTimeout);
        });
        const int m = pairs - e0 < kBlock ? pairs - e0 : kBlock;
#pragma nounroll
        for (int i = 0; i < m; ++i) {
          const int e = e0 + i;
          const int nn = e / p.tiles, t = e - nn * p.tiles;
          const float mu = load_scalar<float>(mean_all, (int64_t)nn * p.G + g, sdtype);
          const float rs = load_scalar<float>(rstd_all, (int64_t)nn * p.G + g, sdtype);
          float v0 = uniform(r.v0[i]), v1 = uniform(r.v1[i]);
          if (!uniform(r.ok[i])) {
            float gamma, a, bb;
            channel_coeffs<PT>(w, b, c, mu, rs, gamma, a, bb);
            const int64_t sample = (int64_t)(nn - n0) * p.R * p.C;
            recompute_channel_record<T, ACT, DY16>(x + sample, dy_at<T, DY16>(dy, sample), dydtype, p, t, c, a, bb, r.sums, v0, v1);
            prefer_arrived(sync, rbc, r, slot_of(e), v0, v1);
          }
          t1 += ((double)v0 - (double)mu * (double)v1) * (double)rs;
          t2 += (double)v1;
        }
      }
      if (threadIdx.x == 0) {
        if (dw) store_param<PT, float>(dw, c, (float)t1);
        if (db) store_param<PT, float>(db, c, (float)t2);
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
// Occupancy the register budget is sized for.
// (with a residual: the tile plus a window of residual_window(nv) rows of the residual)
constexpr int residual_window(int nv) { return nv <= 8 ? nv : 8; }
constexpr int fused_fwd_waves(int nv, int add) {
  return add == kAddResidual ? (nv <= 4 ? 4 : nv <= 16 ? 3 : 2) : (nv <= 8 ? 4 : nv <= 16 ? 3 : 2);
}
// TWO_LEVEL: the exchange of a launch with many row tiles per sample (two_level_exchange on the host).  A template
// parameter, not a run-time switch: the code of the form a launch does not use would sit in the middle of the path every
// workgroup executes once, and these kernels are sensitive to their own size.

// Rows of a backward tile that a lane requests before it starts on the first one; row u + upfront_rows follows when
// row u has been consumed.  A CU serves the requests of its workgroups first come, first served: with every row
// requested up front, the workgroup that came second gets its first row when the first one has its last, and then has
// the arithmetic of its whole tile (15 operations and two transcendentals per element) ahead of it with nothing left to
// overlap it.  Requested a few rows at a time, the requests of the workgroups of a CU interleave and all of them work
// through their rows while rows are still arriving.  Four rows of x and of dy in flight per lane are what keeps the
// memory system as busy as the whole tile did (measured: 3, 5, 6, 8 and 11 are all slower); the form that streams x
// through a window keeps six of each.  The forward is left alone: it has a quarter of the arithmetic per row, and with
// fewer rows in flight its rows only arrive later (c3c: 18.7 -> 21.7 us with 8 of 16 rows up front, 29 us with 4).
constexpr int kUpfrontRows = 4;
constexpr int kUpfrontWindowRows = 6;
constexpr int upfront_rows(int nv) { return nv > kUpfrontRows ? kUpfrontRows : nv; }

// The single parameter of the forward kernel (one block, so that the recovery path can read it again: reread_kernel_args).
struct FusedFwdParams {
  const void *x;
  void *y;
  SyncArea sync;
  const void *w, *b;
  void *mean_out, *rstd_out;
  int sdtype, ydtype;
  float eps;
  int pad_;
  AddArgs add;
  Plan p;
};
template <typename T, typename PT, int VEC, int ACT, int NV, int ADD, bool TWO_LEVEL>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(fused_fwd_waves(NV, ADD)))) void fused_fwd_kernel(
    const FusedFwdParams args) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  const T *__restrict__ x = (const T *)args.x;
  const void *w = args.w, *b = args.b;
  const AddArgs &add = args.add;
  const Plan &p = args.p;
  const SyncArea sync = resident_epoch(args.sync);
  __shared__ A sm0[kBlock * VEC];
  __shared__ A sm1[kBlock * VEC];
  __shared__ RecoveryLds recovery;
  if (threadIdx.x == 0) recovery.late = 0;  // (several barriers lie between this and the first lane that may set it)
  bool late = false;                        // a wait of this lane expired
  const PartialGeo q = producer_geo(p);
  const int64_t n = blockIdx.z;
  const LanePos l = lane_pos<true>(p, n, false);
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
    lane_params_flat<A, PT, VEC>(cvi * VEC, w, b, sync.area, sa, sb);
  }
  // ADD: the per-(sample, channel) addend of the lane's channels, requested with the parameters and without branches
  A tb[VEC];
  if constexpr (ADD != kAddNone) {
    const int cvi = l.cvi < p.cv ? l.cvi : p.cv - 1;
    const void *cb = add.channel_bias ? add.channel_bias : sync.area;
    const int64_t cb0 = add.channel_bias ? n * p.C + (int64_t)cvi * VEC : 0;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const A v = load_scalar_flat<A>(cb, add.channel_bias ? cb0 + j : 0, add.channel_bias_dtype, sync.area);
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
      // The residual passes through a window of RW rows: row u + RW is requested into the slot of row u as soon as that
      // row has been added, so the kernel holds NV + RW rows at most, not 2 NV -- which is what lets a tensor of the
      // size of the plain forward's (x alone fills the registers) still run as one launch with its residual.
      constexpr int RW = residual_window(NV);
      const T *rp = add.residual ? (const T *)add.residual : x;
      const bool has_r = add.residual != nullptr;
      typename LV::raw_t rbuf[RW];
#pragma unroll
      for (int u = 0; u < RW; ++u) rbuf[u] = LV::load(rp + off + (int64_t)clamp_row(u, rows) * step);
#pragma unroll
      for (int u = 0; u < NV; ++u) buf[u] = LV::load(x + off + (int64_t)clamp_row(u, rows) * step);
      T *so = sum_after_exchange<T>(x, add) ? nullptr : (T *)add.sum_out;
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        A vx[VEC], vr[VEC];
        LV::unpack(buf[u], vx);
        LV::unpack(rbuf[u % RW], vr);
#pragma unroll
        for (int j = 0; j < VEC; ++j) vx[j] = (vx[j] + (has_r ? vr[j] : (A)0)) + tb[j];
        buf[u] = LV::pack(vx);  // rounded to T once: the statistics and y are those of the stored sum
        if (so && u < rows) store_streaming<LV>(so + off + (int64_t)u * step, buf[u]);
        if (u + RW < NV) {
          issue_order_fence();  // not before the row it replaces has been used: the slot is the register budget
          rbuf[u % RW] = LV::load(rp + off + (int64_t)clamp_row(u + RW, rows) * step);
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < NV; ++u) buf[u] = LV::load(x + off + (int64_t)clamp_row(u, rows) * step);
      if constexpr (ADD == kAddChannel) {
        T *so = sum_after_exchange<T>(x, add) ? nullptr : (T *)add.sum_out;
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
  const RecordArray rb = record_buffer(sync);
  trace_point(sync, 1, (float)m2[0]);
  // the reduction and the exchange are one chain of dependent steps that every workgroup of the group waits for:
  // let these wavefronts go first on a SIMD they share with wavefronts of other workgroups that are still streaming
  __builtin_amdgcn_s_setprio(3);
  block_group_moments<A, VEC>(p, l, mean, m2, sm0, sm1, [&](int g, A cnt, A mu, A s2) {
    (void)cnt;  // the consumers recompute it from the geometry
    record_store(rb, record_slot(q, p.G, (int)n, l.tile, l.chunk, g), mu, s2, sync.epoch);
  });
  trace_point(sync, 2);
  // Each of the two phases that follow works on its own copy of the kernel's arguments, read again where the phase
  // begins: what the phases before it loaded need not stay in scalar registers (or be spilled and restored) all the way.
  const unsigned long long epoch = sync.epoch;
  {
  const FusedFwdParams args = reread_kernel_args<FusedFwdParams>();
  const Plan &p = args.p;
  const PartialGeo q = producer_geo(p);
  SyncArea sync = args.sync;
  sync.epoch = epoch;
  const RecordArray rb = record_buffer(sync);
  void *mean_out = args.mean_out, *rstd_out = args.rstd_out;
  const int sdtype = args.sdtype;
  const A eps = args.eps;
  if constexpr (TWO_LEVEL) {
    // second level: the groups this workgroup owns, one at a time with all 256 lanes (usually one group or none)
    const RecordArray fb = final_record_buffer(sync);
    const A total = (A)p.D * (A)p.R;
    __shared__ A sm_x[12];
    for (int gi = l.tile; gi < l.ng; gi += p.tiles) {  // uniform over the workgroup
      if (!owns_group(p, l, gi)) continue;
      const int g = l.g_lo + gi;
      A nl = (A)0, kl = (A)0, s1 = (A)0, s2 = (A)0;
      for_group_records(sync, rb, q, p, n, g, true, kBlock, threadIdx.x, late, [&](float mu, float mm, float cnt) {
        if (nl == (A)0) kl = mu;
        const A d = mu - kl;
        nl += cnt;
        s1 += cnt * d;
        s2 += mm + cnt * d * d;
      });
      const A inv = nl > (A)0 ? fast_rcp(nl) : (A)0;
      const A mean_l = kl + s1 * inv;
      const A m2_l = s2 - s1 * s1 * inv;
      if (late) recovery.late = 1;
      __syncthreads();
      if (threadIdx.x == 0) sm_x[8] = mean_l;  // lane 0 always has a record: the pivot of the merge across lanes
      __syncthreads();
      const A K = sm_x[8];
      const A d = nl > (A)0 ? mean_l - K : (A)0;
      A t1 = nl * d, t2 = m2_l + nl * d * d;
      block_sum2(t1, t2, sm_x);
      if (threadIdx.x == 0 && recovery.late == 0) {  // (after an expired wait the sums mean nothing: the recovery publishes)
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
      poll_final(sync, fb, (int)n * p.G + l.g_lo + gi, gmean, rs, late);
      sm0[gi] = gmean;
      sm1[gi] = rs;
    }
    if (late) recovery.late = 1;
    __syncthreads();
  } else {
    // merge the records of the chunk's groups (exact two-pass form, compute_stats_pt2's job:
    // src/gnnhwc/csrc/gn_kernel.cu:226-292); rstd = 1 / sqrt(M2 / n + eps)
    const int L = exchange_lanes(q, p.D);
    const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
    const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
    const A total = (A)p.D * (A)p.R;  // elements of a group
    for (int base = 0; base < l.ng; base += nseg) {
      const int gi = base + seg;
      const bool valid = gi < l.ng;
      const int g = l.g_lo + gi;
      // each lane folds its records about the mean of its first one ...
      A nl = (A)0, kl = (A)0, s1 = (A)0, s2 = (A)0;
      for_group_records(sync, rb, q, p, n, g, valid, L, sl, late, [&](float mu, float mm, float cnt) {
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
    if (late) recovery.late = 1;
    __syncthreads();
  }
  }
  __builtin_amdgcn_s_setprio(0);
  const FusedFwdParams args2 = reread_kernel_args<FusedFwdParams>();
  if (__builtin_expect(uniform(recovery.late) != 0, 0)) {
    // a wait expired somewhere in this workgroup: what the lanes hold means nothing.  Start again from memory.
    SyncArea ks = args2.sync;
    ks.epoch = epoch;
    recover_fwd<T, PT, VEC, ACT, ADD, TWO_LEVEL>((const T *)args2.x, (T *)args2.y, ks, args2.w, args2.b, args2.mean_out,
                                                 args2.rstd_out, args2.sdtype, args2.ydtype, args2.eps, args2.add, args2.p,
                                                 recovery, sm0, sm1);
    return;
  }
  trace_point(sync, 3);
  if (rows > 0) {
    const Plan &p = args2.p;
    const T *x = (const T *)args2.x;
    T *y = (T *)args2.y;
    const AddArgs &add = args2.add;
    const int ydtype = args2.ydtype;
    const int64_t step = (int64_t)p.rpi * p.C;
    A unused1[VEC], unused2[VEC];
    lane_coeffs<A, VEC, false>(p, l, sm0, sm1, nullptr, nullptr, sa, sb, unused1, unused2);
    const bool sum_late = ADD != kAddNone && sum_after_exchange<T>(x, add);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      if (u < rows) {
        A v[VEC];
        pin(buf[u]);
        if constexpr (ADD != kAddNone) {
          if (sum_late) store_streaming<LV>((T *)add.sum_out + off + (int64_t)u * step, buf[u]);
        }
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
// XL > 0 (with XW > 0): the first XL rows of x, which the second pass reaches last, are parked in LDS when the first
// pass is done with them (16 bytes per lane and row: XL x 4 KB per workgroup, LDS that the register-bound occupancy of
// these kernels leaves idle) and read back from there: only NV - XW - XL rows are read from memory a second time.
constexpr int fused_bwd_waves(int nv, int xw) {
  return xw > 0 ? (nv <= 24 ? 3 : 2) : (nv <= 4 ? 4 : nv <= 8 ? 3 : nv <= 22 ? 2 : 1);
}
// The single parameter of the backward kernel (see FusedFwdParams).  x, dy, dx, mean, rstd: this launch's samples;
// mean_all, rstd_all: the whole tensor's; n0: index of this launch's first sample in the tensor, n_all: its samples.
struct FusedBwdParams {
  const void *x, *dy;
  void *dx;
  const void *mean, *rstd;
  const void *w, *b;
  SyncArea sync;
  void *dw, *db;
  const void *mean_all, *rstd_all;
  int64_t n0, n_all;
  int sdtype;
  int dydtype;  // type dy is stored in: the data type, or for float data GN_F16 / GN_BF16 (kernels instantiated with DY16)
  Plan p;
};
// Statistics slots in LDS of a backward kernel: one per group of the chunk.  The kernels with parked rows need their LDS
// for those and serve chunks of at most kBlock channels (the host checks), hence at most kBlock groups.
constexpr int fused_bwd_stat_slots(int vec, int xl) { return xl > 0 ? kBlock : kBlock * vec; }
template <typename T, typename PT, int VEC, int ACT, int NV, bool TWO_LEVEL, int XW = 0, int XL = 0, bool DY16 = false>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(fused_bwd_waves(NV, XW)))) void fused_bwd_kernel(
    const FusedBwdParams args) {
  using A = acc_t<T>;
  using LV = LaneVec<T, VEC>;
  const T *__restrict__ x = (const T *)args.x;
  const T *__restrict__ dy = (const T *)args.dy;
  const void *mean = args.mean, *rstd = args.rstd, *w = args.w, *b = args.b;
  const int64_t n0 = args.n0;
  const int sdtype = args.sdtype;
  const Plan &p = args.p;
  const SyncArea sync = resident_epoch(args.sync);
  __shared__ A sm1[kBlock * VEC];
  __shared__ A sm2[kBlock * VEC];
  __shared__ A sm_mu[fused_bwd_stat_slots(VEC, XL)];
  __shared__ A sm_rs[fused_bwd_stat_slots(VEC, XL)];
  __shared__ typename LV::raw_t parked[XL > 0 ? XL : 1][kBlock];  // rows 0 .. XL - 1 of x between the two passes
  static_assert(XL == 0 || (XW > 0 && XW + XL <= NV), "parked rows lie below the window's last position");
  __shared__ RecoveryLds recovery;
  if (threadIdx.x == 0) {  // (several barriers lie between this and the first lane that may set either)
    recovery.late = 0;
    recovery.late_tail = 0;
  }
  bool late = false;  // a wait of this lane expired
  const PartialGeo q = producer_geo(p);
  const int64_t n = blockIdx.z;
  const LanePos l = lane_pos<true>(p, n, false);
  const RecordArray rb = record_buffer(sync);
  const RecordArray rbc = channel_record_buffer(sync);
  const void *safe = sync.area;  // readable bytes for loads that only exist to keep the prologue free of branches
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
  // (a 16-bit gradient beside float data: the same element offsets at half the bytes)
  auto dy_row = [&](const RowTerms &t, int u) {
    const unsigned bytes = t.lane0 + (unsigned)clamp_row(u, t.rows) * t.step;
    return DY16 ? (const T *)((const char *)dy + tile_base * 2 + (bytes >> 1)) : (const T *)((const char *)(dy + tile_base) + bytes);
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
  // NB rows of x and dy are requested up front, row u + NB as soon as row u has been consumed (see upfront_rows)
  constexpr int NB = XW == 0 ? upfront_rows(NV) : NV;
  constexpr int NBW = XW > 0 ? (kUpfrontWindowRows < NV ? kUpfrontWindowRows : NV) : NV;  // the same for dy beside a window of x
  constexpr int NBX = XW > 0 ? (kUpfrontWindowRows < XW ? kUpfrontWindowRows : XW) : 0;    // and for the window itself
  if constexpr (XW == 0) {
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int64_t o = row_offset(u);
      bx[u] = LV::load(x + o);
      bd[u] = load_dy<T, VEC, DY16>(dy, o);
    }
  } else {
    // the window of x first (row 0's arithmetic needs it), then all of dy; the rest of x follows row by row below
    const RowTerms t0 = fresh_terms();
#pragma unroll
    for (int u = 0; u < NBX; ++u) bx[u] = LV::load(tile_row(x, t0, u));
#pragma unroll
    for (int u = 0; u < NBW; ++u) bd[u] = load_dy<T, VEC, DY16>(dy_row(t0, u), 0);
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
        for (int u = 0; u < (XW > 0 ? NBW : NB); ++u)
          if (u >= rows) bd[u] = zero;
      }
      const RowTerms t1 = fresh_terms();
#pragma unroll
      for (int u = 0; u < NV; ++u) {
        A vx[VEC], vd[VEC];
        if constexpr (NB < NV || NBW < NV) {
          // (rows requested later are zeroed when their turn comes)
          if (u >= (XW > 0 ? NBW : NB) && rows != NV && u >= rows) bd[u] = typename LV::raw_t{};
        }
        pin(bx[u % NX]);  // one row at a time: cheap activations otherwise tempt the scheduler into unpacking many
        pin(bd[u]);       // rows ahead, which costs more registers than the tile itself
        LV::unpack(bx[u % NX], vx);
        unpack_dy<T, VEC, DY16>(bd[u], vd, args.dydtype);
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
        if constexpr (XW == 0 && NB < NV) {
          if (u + NB < NV) {
            issue_order_fence();  // in program order behind the row just consumed
            const int64_t o = row_offset(u + NB);
            bx[u + NB] = LV::load(x + o);
            bd[u + NB] = load_dy<T, VEC, DY16>(dy, o);
          }
        }
        if constexpr (XW > 0) {
          // the sums are brought up to date row by row: left alone, the scheduler postpones the chains of the window's
          // last rows to the end and keeps their unpacked g' alive until then
#pragma unroll
          for (int j = 0; j < VEC; ++j) { pin(s1[j]); pin(s2[j]); }
          pin(bd[u]);  // packed here and now (the conversion otherwise sinks towards the dx phase, g' staying unpacked)
          if constexpr (XL > 0) {
            if (u < XL) parked[u][threadIdx.x] = bx[u % NX];
          }
          if (u + NBX < NV) {
            issue_order_fence();  // not before the rows ahead of it are consumed: the slot is the register budget
            bx[(u + NBX) % NX] = LV::load(tile_row(x, t1, u + NBX));  // (its slot held row u + NBX - NX, consumed long ago)
          }
          if constexpr (NBW < NV) {
            if (u + NBW < NV) bd[u + NBW] = load_dy<T, VEC, DY16>(dy_row(t1, u + NBW), 0);
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
  // The rest of the kernel works on its own copy of the kernel's arguments, read again here: what the phases before it
  // loaded need not stay in scalar registers (or be spilled and restored) all the way.
  const unsigned long long epoch = sync.epoch;
  {
  const FusedBwdParams args = reread_kernel_args<FusedBwdParams>();
  const T *x = (const T *)args.x;
  T *dx = (T *)args.dx;
  void *dw = args.dw, *db = args.db;
  const void *mean_all = args.mean_all, *rstd_all = args.rstd_all;
  const int64_t n0 = args.n0, n_all = args.n_all;
  const int sdtype = args.sdtype;
  const Plan &p = args.p;
  const PartialGeo q = producer_geo(p);
  SyncArea sync = args.sync;
  sync.epoch = epoch;
  const RecordArray rb = record_buffer(sync), rbc = channel_record_buffer(sync);
  const void *safe = sync.area;
  if constexpr (TWO_LEVEL) {
    // second level (see owns_group): the groups this workgroup owns, one at a time with all 256 lanes
    const RecordArray fb = final_record_buffer(sync);
    __shared__ A sm_x[8];
    for (int gi = l.tile; gi < l.ng; gi += p.tiles) {  // uniform over the workgroup
      if (!owns_group(p, l, gi)) continue;
      const int g = l.g_lo + gi;
      A ta = (A)0, tb = (A)0;
      for_group_records(sync, rb, q, p, n, g, true, kBlock, threadIdx.x, late, [&](float ra, float rbv, float) {
        ta += ra;
        tb += rbv;
      });
      if (late) recovery.late = 1;
      block_sum2(ta, tb, sm_x);
      if (threadIdx.x == 0 && recovery.late == 0) {  // (after an expired wait the sums mean nothing: the recovery publishes)
        const A mu = sm_mu[gi];
        const A rs = sm_rs[gi];
        const A s = fast_rcp((A)p.D * (A)p.R);
        const A k1 = (mu * tb - ta) * s * rs * rs * rs;
        record_store(fb, (int)n * p.G + g, k1, -mu * k1 - tb * s * rs, sync.epoch);
      }
    }
    for (int gi = threadIdx.x; gi < l.ng; gi += kBlock) {
      float k1, k2;
      poll_final(sync, fb, (int)n * p.G + l.g_lo + gi, k1, k2, late);
      sm1[gi] = k1;
      sm2[gi] = k2;
    }
  } else {
    const int L = exchange_lanes(q, p.D);
    const int nseg = kBlock >> __builtin_ctz(L);  // L is a power of two
    const int seg = threadIdx.x >> __builtin_ctz(L), sl = threadIdx.x & (L - 1);
    for (int base = 0; base < l.ng; base += nseg) {
      const int gi = base + seg;
      const bool valid = gi < l.ng;
      const int g = l.g_lo + gi;
      A ta = (A)0, tb = (A)0;
      for_group_records(sync, rb, q, p, n, g, valid, L, sl, late, [&](float ra, float rbv, float) {
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
  if (late) recovery.late = 1;
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
  if (__builtin_expect(uniform(recovery.late) != 0, 0)) {
    // a wait expired somewhere in this workgroup: what the lanes hold means nothing.  Coefficients, dx and (the
    // workgroups that finish dgamma / dbeta) the channel sums again, from memory.
    const FusedBwdParams ka = reread_kernel_args<FusedBwdParams>();
    SyncArea ks = ka.sync;
    ks.epoch = epoch;
    recover_bwd_dx<T, PT, VEC, ACT, TWO_LEVEL, DY16>((const T *)ka.x, (const T *)ka.dy, (T *)ka.dx, ka.dydtype, ka.mean, ka.rstd,
                                                     ka.sdtype, ka.w, ka.b, ks, ka.p, recovery, sm_mu, sm_rs, sm1, sm2);
    if (blockIdx.z == 0 && (ka.dw || ka.db))
      recover_bwd_tail<T, PT, ACT, DY16>((const T *)ka.x, (const T *)ka.dy, ka.dydtype, ka.w, ka.b, ka.mean_all, ka.rstd_all, ka.sdtype,
                                         ks, ka.p, recovery, ka.n0, ka.n_all, ka.dw, ka.db);
    return;
  }
  const int tslot = threadIdx.x >> tlg, tsl = threadIdx.x & (TL - 1);
  const TailBlocks tb = tail_blocks(p, l, cpp);
  int tail_c0 = 0, tail_count = 0;
  if (tail && tb.first < tb.total) tail_block_channels(p, tb, tb.first, cpp, tail_c0, tail_count);
  const bool tail_lane = tslot < tail_count;
  const int tail_c = tail_lane ? tail_c0 + tslot : 0;
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
        if (XL > 0 && u < XL) {
          // (a parked row: written and read by the same lane, no barrier needed)
          typename LV::raw_t back = parked[u][threadIdx.x];
          pin(back);
          LV::unpack(back, vx);
        } else {
          pin(bx[u % NX]);
          LV::unpack(bx[u % NX], vx);
        }
        pin(bd[u]);
        LV::unpack(bd[u], vd);  // g'
#pragma unroll
        for (int j = 0; j < VEC; ++j) vd[j] = sa[j] * vd[j] + (c1[j] * vx[j] + c2[j]);
        if (u < rows) store_streaming<LV>((T *)tile_row(dx, t2, u), LV::pack(vd));
        if (u >= XW && u - XW >= XL) {
          issue_order_fence();
          bx[u % NX] = LV::load(tile_row(x, t2, u - XW));
        }
      }
    }
  }
  trace_point(sync, 4);
  if (tail) {
    int spins = 0;
    late = false;
    for (int s = tb.first; s < tb.total; s += tb.stride) {
      const bool first = s == tb.first;
      int c0, count;
      tail_block_channels(p, tb, s, cpp, c0, count);
      const bool valid = tslot < count;
      const int c = valid ? c0 + tslot : 0;
      const int g = div_by(c, p.by_D);
      A t1 = (A)0, t2 = (A)0;
      // one (sample, tile) pair: wait until its record is this launch's (if it is this launch's to write) and add it
      auto add = [&](int e, u32x4 rec, A mu, A rs) {
        const int64_t nn = div_by(e, p.by_tiles);
        const int t = e - (int)nn * p.tiles;
        while (valid && nn >= n0 && (!record_ready(rec, sync.epoch) || sync.max_spins == kForcedTimeout)) {
          if (__builtin_expect(++spins > sync.max_spins, 0)) {
            late = true;  // the sums of this channel mean nothing: the workgroup recomputes its channels below
            break;
          }
          __builtin_amdgcn_s_sleep(2);
          rec = record_load(rbc, (nn * p.tiles + t) * p.C + c);
        }
        A s1, s2;
        record_values(rec, s1, s2);
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
    if (late) recovery.late_tail = 1;
    __syncthreads();
    if (__builtin_expect(uniform(recovery.late_tail) != 0, 0)) {
      const FusedBwdParams ka = reread_kernel_args<FusedBwdParams>();
      SyncArea ks = ka.sync;
      ks.epoch = epoch;
      recover_bwd_tail<T, PT, ACT, DY16>((const T *)ka.x, (const T *)ka.dy, ka.dydtype, ka.w, ka.b, ka.mean_all, ka.rstd_all, ka.sdtype,
                                         ks, ka.p, recovery, ka.n0, ka.n_all, ka.dw, ka.db);
    }
  }
  }
}

}  // namespace gn
