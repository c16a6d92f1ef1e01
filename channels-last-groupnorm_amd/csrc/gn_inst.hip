// Kernel instantiations and launch sequences for ONE element type, selected with -DGN_INST_DTYPE=0..3
// (f32, f64, f16, bf16).  Built four times so the four types compile in parallel.
#include "gn_host.h"
#include <algorithm>

#include "gn_fused.h"
#include "gn_kernels.h"

#ifndef GN_INST_DTYPE
#error "compile with -DGN_INST_DTYPE=<0|1|2|3>"
#endif
// One data type's kernels are spread over three translation units so that they compile in parallel:
// part 0 the forward, part 1 the backward, part 2 the forward with fused additions (single-launch variants).
#ifndef GN_INST_PART
#error "compile with -DGN_INST_PART=<0|1|2>"
#endif
#define GN_PART_FWD (GN_INST_PART == 0)
#define GN_PART_BWD (GN_INST_PART == 1)
#define GN_PART_ADD (GN_INST_PART == 2)

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

#if GN_PART_FWD
template <typename PT, int VEC, int ACT> void launch_apply(const FwdArgs &a, const A *part, const PartialGeo &q) {
  const Plan &p = a.plan;
  launch(kKindFwdApply, (apply_kernel<elem_t, PT, VEC, ACT>), tile_grid(p, 0), dim3(kBlock), a.stream, (const elem_t *)a.x,
         (elem_t *)a.y, part, q, a.w, a.b, a.mean, a.rstd, a.sdtype, a.ydtype, (A)a.eps, p);
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
#endif  // GN_PART_FWD

// ---- resident (single-launch) path ----------------------------------------------------------------
// Workgroups that can be resident at once for a kernel: occupancy reported by the runtime times the CUs.
template <typename K> int resident_slots(K kernel) {
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kBlock, 0) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  const int slots = per_cu * cus;
  return slots < kMaxResidentBlocks ? slots : kMaxResidentBlocks;
}

// Row tiling of a resident launch with a register capacity of nv rows per lane: tiles of exactly nv rows per
// lane (all loads useful; only the last tile of a sample may be short), every workgroup resident.
// Returns false if it does not fit.
bool resident_tiling(const Plan &base, int64_t samples, int nv, int slots, Plan &out) {
  const int64_t columns = samples * base.nchunk;
  if (slots <= 0 || columns > slots || samples > 65535) return false;
  if (base.G > 8192 || base.C >= (1 << 23)) return false;  // the kernels index their records with 24-bit multiplies
  if ((base.lpr & (base.lpr - 1)) != 0) return false;  // ... and find a lane's row and column by shifts
  const int64_t rows = (int64_t)nv * base.rpi;
  const int64_t tiles = (base.R + rows - 1) / rows;
  if (columns * tiles > slots) return false;
  out = base;
  out.N = samples;
  out.tile_rows = (int)rows;
  out.tiles = (int)tiles;
  out.nblocks = columns * tiles;
  set_divisors(out);
  return true;
}


struct ResidentWorkspace {
  SyncArea sync;
};
// Captured launches take their per-replay epoch from the library's generation word and a sequence number.
void arm_generation(ResidentWorkspace &r, const CapturedEpoch &c) {
  r.sync.generation = c.generation;
  if (c.generation) r.sync.epoch = c.next_sequence();
}
ResidentWorkspace resident_fwd_ws(void *ws, const Plan &p) {
  ResidentWorkspace r;
  char *base = (char *)ws + kWorkspaceHeader;
  r.sync.area = base;
  r.sync.area_bytes = (unsigned)(resident_fwd_bytes(p.G) - kWorkspaceHeader);
  r.sync.rec_first = 0;
  r.sync.frec_first = (unsigned)(align_up(resident_rec_bytes(p.G), 256) / 16);
  r.sync.crec_first = 0;  // (no channel records in the forward)
  r.sync.two_level = two_level_exchange(p) ? 1 : 0;
  r.sync.status = resident_status();
  r.sync.generation = nullptr;
  r.sync.max_spins = resident_spin_limit();
  r.sync.epoch = next_epoch();
  r.sync.trace = trace_buffer();
  r.sync.trace_wait = trace_waits() ? 1 : 0;
  return r;
}
ResidentWorkspace resident_bwd_ws(void *ws, const Plan &p) {
  ResidentWorkspace r;
  char *base = (char *)ws + kWorkspaceHeader;
  const size_t cc = (size_t)p.lpr * p.vec;
  r.sync.area = base;
  r.sync.area_bytes = (unsigned)(resident_bwd_bytes(cc, p.G) - kWorkspaceHeader);
  r.sync.crec_first = 0;  // channel records of the whole tensor, [N][tiles][C]
  r.sync.rec_first = (unsigned)(resident_crec_bytes(cc) / 16);
  r.sync.frec_first = (unsigned)((resident_crec_bytes(cc) + align_up(resident_rec_bytes(p.G), 256)) / 16);
  r.sync.two_level = two_level_exchange(p) ? 1 : 0;
  r.sync.status = resident_status();
  r.sync.generation = nullptr;
  r.sync.max_spins = resident_spin_limit();
  r.sync.epoch = next_epoch();
  r.sync.trace = trace_buffer();
  r.sync.trace_wait = trace_waits() ? 1 : 0;
  return r;
}

// How many consecutive single-launch kernels over groups of samples still beat the streaming pair.  Each launch
// pays a fixed latency of roughly 9 microseconds in the backward but moves 3 S bytes instead of the pair's 5 S
// (about 5.4 bytes per nanosecond either way, and about 14 us fixed for the pair); measured on (N, 320, 128, 128)
// bf16: two launches equal the pair at N = 4 and beat it by 14 % at N = 6, three launches by 6 % at N = 8.
// In the forward the pair only moves 3 S against 2 S, and two launches measured 5 % slower than the pair: never split.
int worthwhile_batches(const Plan &p, bool backward) {
  if (!backward) return 1;
  const double s_mb = (double)p.N * p.R * p.C * sizeof(elem_t) / 1e6;
  const double k = (14.0 + 0.405 * s_mb) / 9.0;
  const int kk = k < 1.0 ? 1 : (int)k;
  return kk < kMaxBatches ? kk : kMaxBatches;
}
size_t stat_size(int sdtype) { return sdtype == GN_F32 ? 4 : sdtype == GN_F64 ? 8 : 2; }

#if !GN_PART_BWD
// One NV variant, the tensor cut into `batches` launches over consecutive samples (1: the whole tensor).
template <typename PT, int ACT, int NV, int ADD> bool try_resident_fwd_nv(const FwdArgs &a, int batches) {
  if (NV < resident_min_rows()) return false;
  auto kernel_all = fused_fwd_kernel<elem_t, PT, kVec, ACT, NV, ADD, false>;  // every workgroup polls every tile
  auto kernel_two = fused_fwd_kernel<elem_t, PT, kVec, ACT, NV, ADD, true>;   // two-level exchange (many tiles)
  static const int slots = std::min(resident_slots(kernel_all), resident_slots(kernel_two));
  const int64_t per = (a.plan.N + batches - 1) / batches;
  Plan p;
  if (!resident_tiling(a.plan, per, NV, slots, p)) return false;
  if (!resident_status()) return false;
  CapturedEpoch cap;
  if (!captured_epoch(a.stream, cap)) return false;
  ResidentOrder order(a.stream, cap.generation != nullptr);
  mark_resident_launch();
  const int64_t sample = a.plan.R * a.plan.C;
  for (int64_t n0 = 0; n0 < a.plan.N; n0 += per) {
    Plan pb = p;
    if (a.plan.N - n0 < per) resident_tiling(a.plan, a.plan.N - n0, NV, slots, pb);  // the last, shorter group
    ResidentWorkspace r = resident_fwd_ws(a.ws, pb);  // the launches follow each other on the stream: same records
    arm_generation(r, cap);
    AddArgs add = a.add;  // this group of samples' part of the addends
    if (add.residual) add.residual = (const elem_t *)add.residual + n0 * sample;
    if (add.sum_out) add.sum_out = (elem_t *)add.sum_out + n0 * sample;
    if (add.channel_bias) add.channel_bias = (const char *)add.channel_bias + n0 * a.plan.C * stat_size(add.channel_bias_dtype);
    FusedFwdParams k = {};
    k.x = (const elem_t *)a.x + n0 * sample;
    k.y = (char *)a.y + n0 * sample * stat_size(a.ydtype);
    k.sync = r.sync;
    k.w = a.w;
    k.b = a.b;
    k.mean_out = a.mean ? (char *)a.mean + n0 * a.plan.G * stat_size(a.sdtype) : nullptr;
    k.rstd_out = a.rstd ? (char *)a.rstd + n0 * a.plan.G * stat_size(a.sdtype) : nullptr;
    k.sdtype = a.sdtype;
    k.ydtype = a.ydtype;
    k.eps = (float)a.eps;
    k.add = add;
    k.p = pb;
    launch(ADD != kAddNone ? kKindFusedFwdAdd : kKindFusedFwd, r.sync.two_level ? kernel_two : kernel_all, tile_grid(pb, 0),
           dim3(kBlock), a.stream, k);
    note_resident_launch(ADD != kAddNone ? kKindFusedFwdAdd : kKindFusedFwd, NV, 0, 0, r.sync.two_level, batches, pb.nblocks);
  }
  return true;
}
template <typename PT, int ACT, int ADD> bool try_resident_fwd_add(const FwdArgs &a) {
  // never cut into several launches: with a residual the alternative (an elementwise sum, then the plain forward)
  // measured faster than two single-launch kernels
  const int wb = worthwhile_batches(a.plan, false);
  const int most = a.plan.N < wb ? (int)a.plan.N : wb;
  for (int b = 1; b <= most; ++b)
    if (try_resident_fwd_nv<PT, ACT, 4, ADD>(a, b) || try_resident_fwd_nv<PT, ACT, 8, ADD>(a, b) ||
        try_resident_fwd_nv<PT, ACT, 16, ADD>(a, b) || try_resident_fwd_nv<PT, ACT, 32, ADD>(a, b))
      return true;
  return false;
}
template <typename PT, int ACT> bool try_resident_fwd_act(const FwdArgs &a) {
#if GN_PART_ADD
  // a sum of x and a channel addend alone, or a copy of x (sum_out only), needs no second tile
  return a.add.residual ? try_resident_fwd_add<PT, ACT, kAddResidual>(a) : try_resident_fwd_add<PT, ACT, kAddChannel>(a);
#else
  return try_resident_fwd_add<PT, ACT, kAddNone>(a);
#endif
}
template <typename PT> bool try_resident_fwd_pt(const FwdArgs &a) {
  switch (a.act) {
    case GN_ACT_IDENTITY: return try_resident_fwd_act<PT, GN_ACT_IDENTITY>(a);
    case GN_ACT_RELU: return try_resident_fwd_act<PT, GN_ACT_RELU>(a);
    case GN_ACT_SILU: return try_resident_fwd_act<PT, GN_ACT_SILU>(a);
    case GN_ACT_GELU: return try_resident_fwd_act<PT, GN_ACT_GELU>(a);
    default: return try_resident_fwd_act<PT, GN_ACT_GELU_TANH>(a);
  }
}
}  // namespace
// the single-launch forward with fused additions lives in part 2
bool GN_CAT(try_resident_fwd_added_, GN_SUFFIX)(const FwdArgs &a);
namespace {
bool try_resident_fwd(const FwdArgs &a) {
  if constexpr (sizeof(A) != 4) {
    return false;  // no single-launch kernels for 64-bit data
  } else {
    if (!resident_enabled() || a.plan.vec == 1) return false;
#if GN_PART_FWD
    if (a.has_add()) return GN_CAT(try_resident_fwd_added_, GN_SUFFIX)(a);
#endif
    return a.pdtype == GN_INST_DTYPE ? try_resident_fwd_pt<elem_t>(a) : try_resident_fwd_pt<wide_param_t>(a);
  }
}

#endif  // !GN_PART_BWD

#if GN_PART_BWD
// dy stored in a 16-bit type while the data are float (only the float instantiation has such kernels)
constexpr bool kHasDy16 = GN_INST_DTYPE == 0;
template <typename PT, int ACT, int NV, int XW, int XL, bool DY16> bool try_resident_bwd_one(const BwdArgs &a, int batches);
template <typename PT, int ACT, int NV, int XW = 0, int XL = 0> bool try_resident_bwd_nv(const BwdArgs &a, int batches) {
  if (a.dydtype != GN_INST_DTYPE) {
    if constexpr (kHasDy16) return try_resident_bwd_one<PT, ACT, NV, XW, XL, true>(a, batches);
    else return false;
  }
  return try_resident_bwd_one<PT, ACT, NV, XW, XL, false>(a, batches);
}
template <typename PT, int ACT, int NV, int XW, int XL, bool DY16> bool try_resident_bwd_one(const BwdArgs &a, int batches) {
  if (NV < resident_min_rows()) return false;
  // (kernels that park rows of x in LDS have statistics slots for chunks of at most kBlock channels)
  if (XL > 0 && a.plan.lpr * a.plan.vec > kBlock) return false;
  auto kernel_all = fused_bwd_kernel<elem_t, PT, kVec, ACT, NV, false, XW, XL, DY16>;
  auto kernel_two = fused_bwd_kernel<elem_t, PT, kVec, ACT, NV, true, XW, XL, DY16>;
  static const int slots = std::min(resident_slots(kernel_all), resident_slots(kernel_two));
  const int64_t per = (a.plan.N + batches - 1) / batches;
  Plan p;
  if (!resident_tiling(a.plan, per, NV, slots, p)) return false;
  // (the windowed form addresses the rows of a tile by 32-bit byte offsets from the tile's first row)
  if (XW > 0 && (int64_t)p.tile_rows * p.C * (int64_t)sizeof(elem_t) >= ((int64_t)1 << 31)) return false;
  // the channel records of every sample stay in the workspace until the last launch has summed them
  const size_t crec_need = (size_t)a.plan.N * p.tiles * a.plan.C * 16;
  if (crec_need > resident_crec_bytes((int64_t)p.lpr * p.vec)) return false;
  if (!resident_status()) return false;
  CapturedEpoch cap;
  if (!captured_epoch(a.stream, cap)) return false;
  ResidentOrder order(a.stream, cap.generation != nullptr);
  mark_resident_launch();
  const int64_t sample = a.plan.R * a.plan.C;
  const size_t ssz = stat_size(a.sdtype);
  for (int64_t n0 = 0; n0 < a.plan.N; n0 += per) {
    Plan pb = p;
    if (a.plan.N - n0 < per) resident_tiling(a.plan, a.plan.N - n0, NV, slots, pb);  // the last, shorter group
    pb.tiles = p.tiles;  // same row tiling in every group (it depends on R and NV only)
    ResidentWorkspace r = resident_bwd_ws(a.ws, pb);
    arm_generation(r, cap);
    const bool last = n0 + per >= a.plan.N;
    FusedBwdParams k = {};
    k.x = (const elem_t *)a.x + n0 * sample;
    k.dy = (const char *)a.dy + n0 * sample * stat_size(a.dydtype);
    k.dydtype = a.dydtype;
    k.dx = (elem_t *)a.dx + n0 * sample;
    k.mean = (const char *)a.mean + n0 * a.plan.G * ssz;
    k.rstd = (const char *)a.rstd + n0 * a.plan.G * ssz;
    k.w = a.w;
    k.b = a.b;
    k.sync = r.sync;
    k.dw = last ? a.dw : nullptr;
    k.db = last ? a.db : nullptr;
    k.mean_all = a.mean;
    k.rstd_all = a.rstd;
    k.n0 = n0;
    k.n_all = a.plan.N;
    k.sdtype = a.sdtype;
    k.p = pb;
    launch(kKindFusedBwd, r.sync.two_level ? kernel_two : kernel_all, tile_grid(pb, 0), dim3(kBlock), a.stream, k);
    note_resident_launch(kKindFusedBwd, NV, XW, XL, r.sync.two_level, batches, pb.nblocks);
  }
  return true;
}
template <typename PT, int ACT> bool try_resident_bwd_act(const BwdArgs &a) {
  const int most = a.plan.N < worthwhile_batches(a.plan, true) ? (int)a.plan.N : worthwhile_batches(a.plan, true);
  for (int b = 1; b <= most; ++b) {
    if (try_resident_bwd_nv<PT, ACT, 4>(a, b) || try_resident_bwd_nv<PT, ACT, 8>(a, b) ||
        try_resident_bwd_nv<PT, ACT, 16>(a, b) || try_resident_bwd_nv<PT, ACT, 22>(a, b) ||
        try_resident_bwd_nv<PT, ACT, 32>(a, b))
      return true;
    // too large for two tiles in registers: the form that keeps g' and reads most of x twice, before the tensor is cut
    // into more launches (measured on bf16 (N, 320, 128, 128): 32.6 against 39.3 us at N = 5, 37.2 against 43.4 at N = 6)
    // (window: what the registers leave beside 32 rows of g', 16 rows for 16-bit data; parked: the rows of x that two
    // workgroups per CU can keep in LDS beside their reduction arrays, 14 x 4 KB for 16-bit data, 16 x 4 KB for float)
    constexpr int window = sizeof(elem_t) == 2 ? 16 : 12;
    constexpr int parked = sizeof(elem_t) == 2 ? 14 : 16;
    if (try_resident_bwd_nv<PT, ACT, 32, window, parked>(a, b) || try_resident_bwd_nv<PT, ACT, 36, 8, parked>(a, b)) return true;
  }
  return false;
}
template <typename PT> bool try_resident_bwd_pt(const BwdArgs &a) {
  switch (a.act) {
    case GN_ACT_IDENTITY: return try_resident_bwd_act<PT, GN_ACT_IDENTITY>(a);
    case GN_ACT_RELU: return try_resident_bwd_act<PT, GN_ACT_RELU>(a);
    case GN_ACT_SILU: return try_resident_bwd_act<PT, GN_ACT_SILU>(a);
    case GN_ACT_GELU: return try_resident_bwd_act<PT, GN_ACT_GELU>(a);
    default: return try_resident_bwd_act<PT, GN_ACT_GELU_TANH>(a);
  }
}
bool try_resident_bwd(const BwdArgs &a) {
  if constexpr (sizeof(A) != 4) {
    return false;
  } else {
    if (!resident_enabled() || a.plan.vec == 1) return false;
    return a.pdtype == GN_INST_DTYPE ? try_resident_bwd_pt<elem_t>(a) : try_resident_bwd_pt<wide_param_t>(a);
  }
}

#endif  // GN_PART_BWD

#if GN_PART_FWD
template <int VEC> hipError_t fwd_impl(const FwdArgs &a) {
  if (VEC != 1 && !a.streaming_only && try_resident_fwd(a)) return hipGetLastError();
  note_streaming_call();
  if (a.has_add()) {
    // multi-launch form: materialise the sum (in sum_out, or in y when the caller does not want it), then
    // normalise it from there (in place when it sits in y)
    const Plan &p = a.plan;
    elem_t *dst = (elem_t *)(a.add.sum_out ? a.add.sum_out : a.y);
    if (a.add.residual && !a.add.channel_bias) {
      const int64_t nvec = p.N * p.R * p.C / VEC;
      const int64_t want = (nvec + 4 * kBlock - 1) / (4 * kBlock);
      const unsigned grid = (unsigned)(want < 8 * kNumCU ? (want > 0 ? want : 1) : 8 * kNumCU);
      launch(kKindAdd, (add_flat_kernel<elem_t, VEC>), dim3(grid), dim3(kBlock), a.stream, (const elem_t *)a.x,
             (const elem_t *)a.add.residual, dst, nvec);
    } else {
      launch(kKindAdd, (add_kernel<elem_t, VEC>), tile_grid(p, 0), dim3(kBlock), a.stream, (const elem_t *)a.x, a.add, dst,
             (const void *)a.ws, p);
    }
    FwdArgs plain = a;
    plain.x = dst;
    plain.add = AddArgs{nullptr, nullptr, a.add.channel_bias_dtype, nullptr};
    return fwd_impl<VEC>(plain);
  }
  const Plan &p = a.plan;
  const FwdWorkspace ws = fwd_workspace(p);
  A *base = (A *)((char *)a.ws + kWorkspaceHeader);
  A *part = base + ws.part, *compact = base + ws.compact;
  PartialGeo q = producer_geo(p);
  {
    launch(kKindFwdStats, (stats_kernel<elem_t, VEC>), tile_grid(p, 0), dim3(kBlock), a.stream, (const elem_t *)a.x, part, p);
  }
  const A *src = part;
  if (needs_compaction(p)) {
    const int64_t items = p.N * p.G;
    const unsigned grid = (unsigned)((items + kBlock / 64 - 1) / (kBlock / 64));
    launch(kKindFwdStatsCompact, (stats_compact_kernel<A>), dim3(grid), dim3(kBlock), a.stream, (const A *)part, compact, q, p);
    q = compacted_geo(p);
    src = compact;
  }
  {
    if (a.pdtype == GN_INST_DTYPE) launch_apply_act<elem_t, VEC>(a, src, q);
    else launch_apply_act<wide_param_t, VEC>(a, src, q);
  }
  return hipGetLastError();
}

#endif  // GN_PART_FWD

#if GN_PART_BWD
template <typename PT, int VEC, int ACT, bool DY16> void launch_bwd_act(const BwdArgs &a) {
  const Plan &p = a.plan;
  const BwdWorkspace ws = bwd_workspace(p);
  A *base = (A *)((char *)a.ws + kWorkspaceHeader);
  A *partC = base + ws.partC, *partG = base + ws.partG, *compactC = base + ws.compactC, *compactG = base + ws.compactG;
  PartialGeo q = producer_geo(p);
  {
    launch(kKindBwdReduce, (bwd_reduce_kernel<elem_t, PT, VEC, ACT, DY16>), tile_grid(p, 0), dim3(kBlock), a.stream,
                       (const elem_t *)a.x, (const elem_t *)a.dy, a.mean, a.rstd, a.sdtype, a.w, a.b, partC, partG, p, a.dydtype);
  }
  const A *srcC = partC, *srcG = partG;
  if (needs_compaction(p)) {
    const int nG = (int)((p.N * p.G + kBlock / 64 - 1) / (kBlock / 64));
    int cpb = 32;  // channels per workgroup: fewer when N C is small, so that about a CU's worth of workgroups exist
    while (cpb > 2 && p.N * p.C / cpb < kNumCU) cpb >>= 1;
    const int64_t nC = (p.N * p.C + cpb - 1) / cpb;
    launch(kKindBwdCompact, (bwd_compact_kernel<A>), dim3((unsigned)(nG + nC)), dim3(kBlock), a.stream, (const A *)partC,
           (const A *)partG, compactC, compactG, q, nG, cpb, p);
    q = compacted_geo(p);
    srcC = compactC;
    srcG = compactG;
  }
  {
    launch(kKindBwdDx, (bwd_dx_kernel<elem_t, PT, VEC, ACT, DY16>), tile_grid(p, 1), dim3(kBlock), a.stream,
                       (const elem_t *)a.x, (const elem_t *)a.dy, (elem_t *)a.dx, a.mean, a.rstd, a.sdtype, a.w, a.b, srcC,
                       srcG, q, a.dw, a.db, p, a.dydtype);
  }
}
template <typename PT, int VEC, bool DY16> void bwd_act_dy(const BwdArgs &a) {
  switch (a.act) {
    case GN_ACT_IDENTITY: launch_bwd_act<PT, VEC, GN_ACT_IDENTITY, DY16>(a); break;
    case GN_ACT_RELU: launch_bwd_act<PT, VEC, GN_ACT_RELU, DY16>(a); break;
    case GN_ACT_SILU: launch_bwd_act<PT, VEC, GN_ACT_SILU, DY16>(a); break;
    case GN_ACT_GELU: launch_bwd_act<PT, VEC, GN_ACT_GELU, DY16>(a); break;
    default: launch_bwd_act<PT, VEC, GN_ACT_GELU_TANH, DY16>(a); break;
  }
}
template <typename PT, int VEC> void bwd_act(const BwdArgs &a) {
  if constexpr (kHasDy16) {
    if (a.dydtype != GN_INST_DTYPE) return bwd_act_dy<PT, VEC, true>(a);
  }
  bwd_act_dy<PT, VEC, false>(a);
}
template <int VEC> hipError_t bwd_impl(const BwdArgs &a) {
  if (VEC != 1 && try_resident_bwd(a)) return hipGetLastError();
  note_streaming_call();
  if (a.pdtype == GN_INST_DTYPE) bwd_act<elem_t, VEC>(a);
  else bwd_act<wide_param_t, VEC>(a);
  return hipGetLastError();
}

#endif  // GN_PART_BWD

}  // namespace

#if GN_PART_FWD
hipError_t GN_CAT(launch_fwd_, GN_SUFFIX)(const FwdArgs &a) {
  return a.plan.vec == 1 ? fwd_impl<1>(a) : fwd_impl<kVec>(a);
}
#elif GN_PART_BWD
hipError_t GN_CAT(launch_bwd_, GN_SUFFIX)(const BwdArgs &a) {
  return a.plan.vec == 1 ? bwd_impl<1>(a) : bwd_impl<kVec>(a);
}
#else
bool GN_CAT(try_resident_fwd_added_, GN_SUFFIX)(const FwdArgs &a) { return try_resident_fwd(a); }
#endif

}  // namespace gn
