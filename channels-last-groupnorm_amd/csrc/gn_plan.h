// Launch plan shared by host and device code: how an (N, R, C) channels-last slab is cut into
// workgroup tiles.  Plays the role of the reference's calc_block_params / closest_factor
// (src/gnnhwc/csrc/gn_kernel.cu:37-60,121-128) but is built around 128-bit lane vectors and
// 256-thread workgroups instead of <=128-thread blocks over a virtual H x W factorisation.
#pragma once
// GN_TRACE = 1 compiles the phase stamps of the single-launch kernels in (libgnnhwc_hip_trace.so).  The library proper is
// built without them: even switched off at run time they cost registers, basic-block boundaries and code on the path
// every launch executes (measured: 2 % of the SD-UNet sweep).
#ifndef GN_TRACE
#define GN_TRACE 0
#endif
#include <stdint.h>

namespace gn {

enum { GN_F32 = 0, GN_F64 = 1, GN_F16 = 2, GN_BF16 = 3 };
enum { GN_ACT_IDENTITY = 0, GN_ACT_RELU = 1, GN_ACT_SILU = 2, GN_ACT_GELU = 3, GN_ACT_GELU_TANH = 4 };

constexpr int kBlock = 256;         // threads per workgroup (4 wavefronts)
constexpr int kUnrollFwd = 4;       // independent row loads in flight per lane, one-input kernels
constexpr int kUnrollBwd = 2;       // ... two-input kernels (x and dy)
constexpr int kNumCU = 256;         // MI355X
constexpr int kTargetBlocks = 768;  // ~3 workgroups per CU, what the streaming kernels' registers allow: one resident wave
constexpr int kEarly = 4;            // tile partials a lane of a consumer workgroup fetches ahead of its data

// Division by a launch constant without the integer-division sequence (a few dozen instructions on this hardware, all
// of them latency in a workgroup's prologue) and without a branch: with L = ceil(log2 d) and
// magic = floor(2^32 (2^L - d) / d) + 1,
//   t = umulhi(magic, n),   n / d = (t + ((n - t) >> min(L, 1))) >> max(L - 1, 0)
// for every 0 <= n < 2^32 and 1 <= d < 2^31 (Granlund and Montgomery, "Division by invariant integers using
// multiplication", 1994, section 4).  No fallback means no cold code and no extra basic blocks in the kernels.
struct Divisor {
  int d;
  unsigned magic;
  int sh1, sh2;
};
__host__ __device__ inline Divisor make_divisor(int64_t d, int64_t /*largest dividend: any value below 2^32 is fine*/) {
  Divisor v;
  v.d = (int)d;
  const uint64_t ud = (uint64_t)(d < 1 ? 1 : d);
  int L = 0;
  while (((uint64_t)1 << L) < ud) ++L;
  v.magic = (unsigned)(((((uint64_t)1 << L) - ud) << 32) / ud + 1);
  v.sh1 = L < 1 ? L : 1;
  v.sh2 = L > 1 ? L - 1 : 0;
  return v;
}
__host__ __device__ __forceinline__ int div_by(int n, const Divisor &v) {
  const unsigned un = (unsigned)n;
#if defined(__HIP_DEVICE_COMPILE__)
  const unsigned t = __umulhi(v.magic, un);
#else
  const unsigned t = (unsigned)(((uint64_t)v.magic * un) >> 32);
#endif
  return (int)((t + ((un - t) >> v.sh1)) >> v.sh2);
}

// One workgroup owns `tile_rows` consecutive rows of one sample and one chunk of `lpr` lane vectors
// (lpr * vec channels) of every such row.  Inside the workgroup thread t handles lane vector
// (t % lpr) of rows (t / lpr), (t / lpr) + rpi, ...: every lane keeps the same channels for the whole
// tile, so per-channel affine coefficients and per-channel partial sums live in registers.
// Grid: x = row tile, y = channel chunk, z = sample (z wraps when N exceeds the grid limit).
struct Plan {
  int64_t N, R, C;
  int G, D;         // groups, channels per group
  int vec;          // elements per lane vector (16 bytes / sizeof(T), or 1 for the scalar path)
  int cv;           // lane vectors per row = C / vec
  int lpr;          // lane vectors of a row handled by one workgroup (<= kBlock)
  int nchunk;       // workgroups side by side along C = ceil(cv / lpr)
  int rpi;          // rows covered per step = kBlock / lpr
  int tile_rows;    // rows per workgroup tile
  int tiles;        // row tiles per sample = ceil(R / tile_rows)
  int gmax;         // most groups any chunk intersects
  int64_t nblocks;  // N * tiles * nchunk
  Divisor by_lpr, by_rpi, by_D, by_tiles, by_chunk;  // lpr, rpi, D, tiles, lpr * vec (set_divisors)
};
// Fill the divisors from the other fields (again after any change of the tiling).
inline void set_divisors(Plan &p) {
  p.by_lpr = make_divisor(p.lpr, kBlock);
  p.by_rpi = make_divisor(p.rpi, (int64_t)p.tile_rows + p.rpi);
  p.by_D = make_divisor(p.D, 2 * p.C);
  const int64_t wide = p.N > p.nchunk + 1 ? p.N : p.nchunk + 1;
  p.by_tiles = make_divisor(p.tiles, wide * p.tiles);
  p.by_chunk = make_divisor((int64_t)p.lpr * p.vec, p.C + p.D);
}

// Pre-additions of the forward (fused-addition variant): the tensor that is normalised is s = x + residual + channel_bias[n][c],
// rounded to T once (what an unfused elementwise addition in T would hand to the normalisation); s is written to
// sum_out if that is given.  Any of the three pointers may be null.
struct AddArgs {
  const void *residual;      // (N, R, C) in T
  const void *channel_bias;  // (N, C) in channel_bias_dtype
  int channel_bias_dtype;
  void *sum_out;             // (N, R, C) in T
};

// Geometry of a buffer of per-tile partial results as the consumer sees it: either the producer's own
// (tiles, nchunk), or (1, 1) after the compaction kernel has merged all tiles of a sample.
struct PartialGeo {
  int tiles, nchunk;
  int chunk_channels;  // channels per chunk of the producer (lpr * vec); C when compacted
  Divisor by_tiles, by_chunk;
};
// The producer's own geometry, and the one a compaction kernel leaves behind.
__host__ __device__ inline PartialGeo producer_geo(const Plan &p) {
  PartialGeo q;
  q.tiles = p.tiles;
  q.nchunk = p.nchunk;
  q.chunk_channels = p.lpr * p.vec;
  q.by_tiles = p.by_tiles;
  q.by_chunk = p.by_chunk;
  return q;
}
inline PartialGeo compacted_geo(const Plan &p) {
  PartialGeo q;
  q.tiles = 1;
  q.nchunk = 1;
  q.chunk_channels = (int)p.C;
  q.by_tiles = make_divisor(1, 0);
  q.by_chunk = make_divisor(p.C, p.C + p.D);
  return q;
}

// A consumer workgroup merges the tile partials of all groups of its chunk in one round: merge_lanes lanes
// per group, each fetching at most kEarly entries.  The host checks that this covers the plan and
// otherwise runs the compaction kernel first (which leaves one entry per group).
__host__ __device__ inline int pow2_at_least(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}
__host__ __device__ inline int merge_lanes_for(int gmax) {
  const int l = kBlock / pow2_at_least(gmax);
  return l > 64 ? 64 : l;
}

}  // namespace gn
