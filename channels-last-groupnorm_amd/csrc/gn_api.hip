// C ABI of libgnnhwc_hip.so (declared in include/gnnhwc.h): argument validation, launch planning,
// element-type dispatch and the optional per-kernel event timing.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "../../include/gnnhwc.h"
#include "gn_host.h"

namespace gn {
namespace {

thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int env_int(const char *name, int fallback) {
  const char *v = getenv(name);
  return (v && *v) ? atoi(v) : fallback;
}

int elem_size(int dtype) {
  switch (dtype) {
    case GN_F32: return 4;
    case GN_F64: return 8;
    case GN_F16: return 2;
    case GN_BF16: return 2;
    default: return 0;
  }
}
const char *dtype_name(int dtype) {
  static const char *names[] = {"f32", "f64", "f16", "bf16"};
  return (dtype >= 0 && dtype < 4) ? names[dtype] : "?";
}

// Cut (N, R, C) into workgroup tiles.  `vec` is 16 / sizeof(T) for the 128-bit path or 1 for the
// scalar path; `streams` is the number of activation-sized tensors a tile reads (1 forward, 2 backward).
//
// Chunk width: a workgroup reads `lpr` lane vectors (lpr * 16 bytes) of each row.  Narrow chunks mean
// tall tiles for the same number of workgroups, and the per-tile partial results (one entry per group
// or channel and tile) shrink with the number of row tiles; so the narrowest chunk that still covers
// whole 128-byte lines, divides the row evenly and leaves no lane idle is preferred.
// Rows per tile: chosen so that a large tensor yields about `target` workgroups and a small one still
// yields as many workgroups as it has lane rows, down to one row per lane.
Plan make_plan(int64_t N, int64_t R, int64_t C, int64_t G, int vec, int streams) {
  static const int forced_lpr = env_int("GNNHWC_LPR", 0);
  static const int forced_fwd_steps = env_int("GNNHWC_FWD_STEPS", 0);
  static const int forced_bwd_steps = env_int("GNNHWC_BWD_STEPS", 0);
  const int forced_steps = streams == 1 ? forced_fwd_steps : forced_bwd_steps;
  static const int forced_target = env_int("GNNHWC_TARGET_BLOCKS", 0);
  Plan p;
  p.N = N; p.R = R; p.C = C;
  p.G = (int)G;
  p.D = (int)(C / G);
  p.vec = vec;
  p.cv = (int)(C / vec);
  int lpr = 0;
  if (forced_lpr > 0 && forced_lpr <= kBlock && forced_lpr <= p.cv) {
    lpr = forced_lpr;
  } else if (vec > 1) {
    static const int preferred[] = {8, 16, 32, 64, 128, 256, 4, 2};  // half and quarter lines only as a last resort
    for (int d : preferred)
      if (p.cv % d == 0) { lpr = d; break; }
  }
  if (lpr == 0) {  // no even cut into whole cache lines: take the whole row, or equal-ish chunks of a long one
    const int nchunk = (p.cv + kBlock - 1) / kBlock;
    lpr = (p.cv + nchunk - 1) / nchunk;
  }
  p.lpr = lpr;
  p.nchunk = (p.cv + lpr - 1) / lpr;
  p.rpi = kBlock / lpr;
  const int64_t lane_rows = (R + p.rpi - 1) / p.rpi;  // steps needed to walk one sample
  const int64_t units = N * p.nchunk * lane_rows;     // workgroups if each took a single step
  const int64_t target = forced_target > 0 ? forced_target : kTargetBlocks;
  const int unroll = streams == 1 ? kUnrollFwd : kUnrollBwd;
  int64_t k;
  if (forced_steps > 0) {
    k = forced_steps;
  } else {
    // few, tall tiles: about `target` workgroups in all (one resident wave of them), so that the consumers' merge
    // of tile partials stays short -- and, where that still leaves every CU busy, few enough tiles per group for
    // the consumers to merge them in their prologue instead of a compaction launch in between
    int64_t tiles_wanted = (target + N * p.nchunk - 1) / (N * p.nchunk);
    if (forced_target == 0) {
      const int chunk_channels = lpr * vec;
      const int64_t groups_touched = (chunk_channels + p.D - 2) / p.D + 1;
      const int lanes = merge_lanes_for((int)(groups_touched < G ? groups_touched : G));
      const int64_t tiles_merged = lanes < 1 ? 0 : (int64_t)kEarly * lanes / ((p.D - 1) / chunk_channels + 2);
      if (tiles_wanted > tiles_merged && tiles_merged * N * p.nchunk >= kTargetBlocks / 2) tiles_wanted = tiles_merged;
    }
    if (tiles_wanted < 1) tiles_wanted = 1;
    k = (lane_rows + tiles_wanted - 1) / tiles_wanted;
    if (k < unroll) {
      k = units / kNumCU;  // small problem: keep every CU busy before making tiles taller
      if (k < 1) k = 1;
      if (k > unroll) k = unroll;
    } else {
      k = (k + unroll - 1) / unroll * unroll;  // whole batches: no load slot of the last batch is wasted
    }
  }
  if (k > lane_rows) k = lane_rows;
  p.tile_rows = (int)(k * p.rpi);
  p.tiles = (int)((R + p.tile_rows - 1) / p.tile_rows);
  p.nblocks = N * p.tiles * p.nchunk;
  set_divisors(p);
  {
    const int chunk_channels = p.lpr * vec;
    const int64_t g = (chunk_channels + p.D - 2) / p.D + 1;  // groups a window of chunk_channels can touch
    p.gmax = (int)(g < G ? g : G);
  }
  static const int debug = env_int("GNNHWC_DEBUG_PLAN", 0);
  if (debug)
    fprintf(stderr, "[gnnhwc] plan(%s) N=%lld R=%lld C=%lld G=%d D=%d vec=%d cv=%d lpr=%d nchunk=%d rpi=%d tile_rows=%d tiles=%d nblocks=%lld\n",
            streams == 1 ? "fwd" : "bwd", (long long)N, (long long)R, (long long)C, p.G, p.D, p.vec, p.cv, p.lpr,
            p.nchunk, p.rpi, p.tile_rows, p.tiles, (long long)p.nblocks);
  return p;
}

int check_shape(int64_t N, int64_t R, int64_t C, int64_t G, int dtype) {
  if (elem_size(dtype) == 0) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown dtype code %d", dtype);
  if (N < 0 || R < 0 || C <= 0 || G <= 0)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "invalid shape N=%lld R=%lld C=%lld G=%lld", (long long)N, (long long)R,
                (long long)C, (long long)G);
  if (C % G != 0)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "num_channels (%lld) must be divisible by num_groups (%lld)", (long long)C,
                (long long)G);
  if (C > (1 << 24) || N > ((int64_t)1 << 31) || R > ((int64_t)1 << 40) ||
      (double)N * (double)R * (double)C > 4.0e18)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "shape N=%lld R=%lld C=%lld is beyond the supported index range",
                (long long)N, (long long)R, (long long)C);
  return GNNHWC_OK;
}
int check_dtypes(int dtype, int pdtype, int sdtype) {
  const bool half = dtype == GN_F16 || dtype == GN_BF16;
  if (!(pdtype == dtype || (half && pdtype == GN_F32)))
    return fail(GNNHWC_ERR_INVALID_ARGUMENT,
                "weight/bias dtype %s does not match data dtype %s (only f32 parameters with f16/bf16 data may differ)",
                dtype_name(pdtype), dtype_name(dtype));
  if (!(sdtype == dtype || (half && sdtype == GN_F32)))
    return fail(GNNHWC_ERR_INVALID_ARGUMENT,
                "mean/rstd dtype %s does not match data dtype %s (only f32 statistics with f16/bf16 data may differ)",
                dtype_name(sdtype), dtype_name(dtype));
  return GNNHWC_OK;
}
bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

size_t acc_size(int dtype) { return dtype == GN_F64 ? 8 : 4; }
size_t max_size(size_t a, size_t b) { return a > b ? a : b; }
size_t fwd_ws_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype, bool streaming_only = false) {
  const int vec = 16 / elem_size(dtype);
  size_t need = fwd_workspace(make_plan(N, R, C, G, 1, 1)).total;
  size_t resident = 0;
  if (C % vec == 0) {
    const size_t v = fwd_workspace(make_plan(N, R, C, G, vec, 1)).total;
    if (v > need) need = v;
    resident = dtype == GN_F64 || streaming_only ? 0 : resident_fwd_bytes(G);
  }
  return max_size(kWorkspaceHeader + need * acc_size(dtype), resident);
}
size_t bwd_ws_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype) {
  const int vec = 16 / elem_size(dtype);
  size_t need = bwd_workspace(make_plan(N, R, C, G, 1, 2)).total;
  size_t resident = 0;
  if (C % vec == 0) {
    const Plan pv = make_plan(N, R, C, G, vec, 2);
    const size_t v = bwd_workspace(pv).total;
    if (v > need) need = v;
    resident = dtype == GN_F64 ? 0 : resident_bwd_bytes((int64_t)pv.lpr * vec, G);
  }
  return max_size(kWorkspaceHeader + need * acc_size(dtype), resident);
}

__global__ void fill_zero_kernel(void *p, int64_t n, int dtype) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  switch (dtype) {
    case GN_F32: ((float *)p)[i] = 0.f; break;
    case GN_F64: ((double *)p)[i] = 0.0; break;
    default: ((uint16_t *)p)[i] = 0; break;
  }
}

// Plain 16-byte-per-lane copy: the yardstick the library's kernels are measured against (same block size,
// same access width, no arithmetic), and the known-size dispatch that calibrates memory-traffic counters.
__global__ __launch_bounds__(256) void copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int64_t n16) {
  const int64_t base = ((int64_t)blockIdx.x * 4) * 256 + threadIdx.x;
  uint4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int64_t i = base + (int64_t)u * 256;
    v[u] = src[i < n16 ? i : n16 - 1];
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int64_t i = base + (int64_t)u * 256;
    if (i < n16) dst[i] = v[u];
  }
}

// The load phase of a single-launch kernel on its own: every lane requests NV rows of 16 bytes of x (and of dy) up front,
// in the tile geometry of the 128-byte-chunk plans (lane = (row t / 8, column t % 8); row u of a lane is 32 rows below
// row u - 1), and nothing else happens.  A yardstick like copy_kernel: no single-launch kernel can have its rows
// sooner than this kernel ends.
template <int NV, bool TWO>
__global__ __launch_bounds__(256) void load_tile_kernel(const char *__restrict__ x, const char *__restrict__ dy, unsigned *sink,
                                                        int64_t R, int64_t row_bytes) {
  const int ty = threadIdx.x >> 3, tx = threadIdx.x & 7;
  const int64_t first = (int64_t)blockIdx.x * NV * 32 + ty;
  const int64_t off = ((int64_t)blockIdx.z * R + first) * row_bytes + (int64_t)blockIdx.y * 128 + tx * 16;
  uint4 bx[NV], bd[NV];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int64_t o = off + (first + 32 * u < R ? 32 * u : 0) * row_bytes;
    bx[u] = *(const uint4 *)(x + (first < R ? o : 0));
    if (TWO) bd[u] = *(const uint4 *)(dy + (first < R ? o : 0));
  }
  unsigned acc = 0;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    acc ^= bx[u].x ^ bx[u].y ^ bx[u].z ^ bx[u].w;
    if (TWO) acc ^= bd[u].x ^ bd[u].y ^ bd[u].z ^ bd[u].w;
  }
  if (acc == 0x9E3779B9u && sink) *sink = acc;  // (keeps the loads alive; practically never taken)
}
template <int NV> void launch_load_tile(const void *x, const void *dy, void *sink, dim3 grid, hipStream_t stream, int64_t R,
                                        int64_t row_bytes) {
  if (dy) launch(kKindCopy, load_tile_kernel<NV, true>, grid, dim3(256), stream, (const char *)x, (const char *)dy, (unsigned *)sink, R, row_bytes);
  else launch(kKindCopy, load_tile_kernel<NV, false>, grid, dim3(256), stream, (const char *)x, (const char *)dy, (unsigned *)sink, R, row_bytes);
}

// ---- per-kernel event timing ----
struct Timed {
  int kind;
  hipEvent_t start, stop;
};
thread_local bool g_profile = false;
thread_local std::vector<Timed> g_timed;
thread_local std::vector<hipEvent_t> g_event_pool;

hipEvent_t get_event() {
  if (!g_event_pool.empty()) {
    hipEvent_t e = g_event_pool.back();
    g_event_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}

}  // namespace

unsigned long long next_epoch() {
  static std::atomic<unsigned long long> counter{0};
  static const unsigned long long seed = []() {
    unsigned long long v = (unsigned long long)time(nullptr) * 0x9E3779B97F4A7C15ull;
    v ^= (unsigned long long)(uintptr_t)&counter << 17;
    return v | 1ull;
  }();
  // odd multiplier: distinct counters give distinct epochs; never 0
  unsigned long long e = seed + 0x9E3779B97F4A7C15ull * (counter.fetch_add(1) + 1);
  return e ? e : 1ull;
}
// ---- epochs of captured launches -------------------------------------------------------------------------
// One generation word per device, in the library's own device memory (each device holds its own copy of the
// array below at its own address; host code only ever uses the address hipGetSymbolAddress returns for the
// current device, never the array's name).
static __device__ __align__(256) unsigned long long g_generation_cell[32];
__global__ void bump_generation_kernel(unsigned long long *generation) { *generation += 1; }
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_capture_mutex;
unsigned long long *g_generation_ptr[kMaxDevices];
bool g_generation_tried[kMaxDevices];
unsigned long long g_last_capture[kMaxDevices];
bool g_have_last_capture[kMaxDevices];
std::atomic<unsigned long long> g_capture_sequence{0};
}  // namespace
unsigned long long CapturedEpoch::next_sequence() const { return g_capture_sequence.fetch_add(1) + 1; }
bool captured_epoch(hipStream_t stream, CapturedEpoch &out) {
  out.generation = nullptr;
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  if (hipStreamGetCaptureInfo(stream, &st, &id) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // not a capturing stream as far as the runtime can tell
  }
  if (st == hipStreamCaptureStatusNone) return true;
  if (st != hipStreamCaptureStatusActive) return false;  // invalidated capture: record nothing that depends on it
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return false;
  }
  std::lock_guard<std::mutex> lock(g_capture_mutex);
  if (!g_generation_tried[dev]) {
    g_generation_tried[dev] = true;
    // looking a symbol up is not a stream operation, but keep the capture from seeing it as one
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_generation_cell)) != hipSuccess) {
      (void)hipGetLastError();
      p = nullptr;
    }
    if (swapped) (void)hipThreadExchangeStreamCaptureMode(&mode);
    g_generation_ptr[dev] = (unsigned long long *)p;
  }
  unsigned long long *word = g_generation_ptr[dev];
  if (!word) return false;
  if (!g_have_last_capture[dev] || g_last_capture[dev] != id) {
    hipLaunchKernelGGL(bump_generation_kernel, dim3(1), dim3(1), 0, stream, word);
    if (hipGetLastError() != hipSuccess) return false;
    g_have_last_capture[dev] = true;
    g_last_capture[dev] = id;
  }
  out.generation = word;
  return true;
}

// ---- one single-launch kernel at a time per device ----------------------------------------------------------
namespace {
std::mutex g_order_mutex;
hipStream_t g_order_stream[kMaxDevices];
bool g_order_have[kMaxDevices];
hipEvent_t g_order_event[kMaxDevices];
}  // namespace
ResidentOrder::ResidentOrder(hipStream_t stream, bool capturing) : locked_(false) {
  if (capturing) return;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return;
  }
  g_order_mutex.lock();
  locked_ = true;
  if (g_order_have[dev] && g_order_stream[dev] != stream) {
    hipEvent_t &ev = g_order_event[dev];
    if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      ev = nullptr;
    }
    // the event covers everything submitted to the previous stream so far, the last single-launch kernel included;
    // a previous stream that has started recording a graph since is left alone (an event recorded there would
    // become part of that graph)
    hipStreamCaptureStatus prev = hipStreamCaptureStatusNone;
    const bool known = hipStreamIsCapturing(g_order_stream[dev], &prev) == hipSuccess;
    if (ev && known && prev == hipStreamCaptureStatusNone && hipEventRecord(ev, g_order_stream[dev]) == hipSuccess) {
      if (hipStreamWaitEvent(stream, ev, 0) != hipSuccess) (void)hipGetLastError();
    } else {
      (void)hipGetLastError();  // e.g. the previous stream no longer exists
    }
  }
  g_order_stream[dev] = stream;
  g_order_have[dev] = true;
}
ResidentOrder::~ResidentOrder() {
  if (locked_) g_order_mutex.unlock();
}

bool trace_waits() {
  static const bool w = env_int("GNNHWC_TRACE", 0) != 2;
  return w;
}
unsigned long long *trace_buffer() {
#if !GN_TRACE
  return nullptr;  // this build's kernels have no stamps
#endif
  static unsigned long long *buf = []() -> unsigned long long * {
    if (env_int("GNNHWC_TRACE", 0) == 0) return nullptr;
    void *p = nullptr;
    const size_t bytes = (size_t)kMaxResidentBlocks * 8 * sizeof(unsigned long long);
    if (hipMalloc(&p, bytes) != hipSuccess) return nullptr;
    (void)hipMemset(p, 0, bytes);
    return (unsigned long long *)p;
  }();
  return buf;
}
// Host-pinned, device-visible word that a single-launch kernel sets when one of its bounded waits expires (its
// workgroups were not all resident at once, and it recomputed the records it was waiting for): gnnhwc_resident_status.
unsigned long long *resident_status() {
  static unsigned long long *word = []() -> unsigned long long * {
    // the first call may come while the thread is capturing a graph: allocation is legal there in relaxed mode
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    void *h = nullptr;
    if (hipHostMalloc(&h, 64, hipHostMallocPortable | hipHostMallocMapped) != hipSuccess) {
      (void)hipGetLastError();
      h = nullptr;
    }
    if (swapped) (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (h) memset(h, 0, 64);
    return (unsigned long long *)h;
  }();
  return word;
}
std::atomic<bool> g_status_live{false};  // resident_status() has been handed to a kernel
void mark_resident_launch() { g_status_live.store(true, std::memory_order_relaxed); }

int resident_min_rows() {
  static const int v = env_int("GNNHWC_RESIDENT_MIN_ROWS", 0);
  return v;
}
// Polls per wait.  A poll is a device-scope round trip and a short sleep, about a microsecond, so a lane waits about a
// millisecond for workgroups that are not resident yet before it recomputes their records itself -- which costs a few
// milliseconds per launch: waiting about as long as the recovery takes, and no longer.
constexpr int kDefaultSpinLimit = 1 << 10;
std::atomic<int> g_spin_limit{kDefaultSpinLimit};
int resident_spin_limit() { return g_spin_limit.load(std::memory_order_relaxed); }

thread_local int64_t g_last_launch[7] = {-1, 0, 0, 0, 0, 0, 0};
void note_resident_launch(int kind, int rows_per_lane, int window_rows, int parked_rows, int two_level, int launches,
                          int64_t workgroups) {
  g_last_launch[0] = kind;
  g_last_launch[1] = rows_per_lane;
  g_last_launch[2] = window_rows;
  g_last_launch[3] = two_level;
  g_last_launch[4] = launches;
  g_last_launch[5] = workgroups;
  g_last_launch[6] = parked_rows;
}
void note_streaming_call() { g_last_launch[0] = -1; }
bool cooperative_launches() {
  static const bool v = env_int("GNNHWC_COOPERATIVE", 0) != 0;
  return v;
}
std::atomic<int> g_resident{-1};  // -1: follow the environment
bool resident_enabled() {
  static const int off = env_int("GNNHWC_DISABLE_RESIDENT", 0);
  const int v = g_resident.load(std::memory_order_relaxed);
  return v < 0 ? off == 0 : v != 0;
}

bool profile_events(int kind, hipEvent_t *start, hipEvent_t *stop) {
  if (!g_profile) return false;
  Timed t;
  t.kind = kind;
  t.start = get_event();
  t.stop = get_event();
  if (!t.start || !t.stop) return false;
  g_timed.push_back(t);
  *start = t.start;
  *stop = t.stop;
  return true;
}

}  // namespace gn

using namespace gn;

// A single-launch kernel some of whose waits expired has recomputed what it was waiting for: its results are right, it
// only took longer.  The status word records that it happened; reading clears it.
static int degraded_since_last_query() {
  if (!g_status_live.load(std::memory_order_relaxed)) return 0;
  volatile unsigned long long *w = resident_status();
  if (!w || *w == 0) return 0;
  *w = 0;
  return 1;
}

// ---- forward that allocates nothing -------------------------------------------------------------------------
// The scratch memory of the multi-launch forward (per-tile partial statistics) in the library's own device image:
// every device the library runs on holds its own copy of this array, at its own address, until the process ends.
// Host code never uses the array's name as an address: static_scratch() asks the runtime for the current device's
// copy once and hands that pointer on.
static __device__ __align__(256) unsigned char scratch[GNNHWC_STATIC_SCRATCH_BYTES];
namespace {
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];
bool g_scratch_tried[kMaxDevices];
// Address of the current device's copy of `scratch` (null, with the error string set, if it cannot be had).
void *static_scratch() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    fail(GNNHWC_ERR_LAUNCH, "no current device for the library's scratch memory (%s)", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_tried[dev]) {
    // looking a symbol up is not a stream operation, but a capture in progress on this thread must not see it as one
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    const bool swapped = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
    void *ptr = nullptr;
    e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (swapped) (void)hipThreadExchangeStreamCaptureMode(&mode);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      fail(GNNHWC_ERR_LAUNCH, "hipGetSymbolAddress for the library's scratch memory failed: %s", hipGetErrorString(e));
      return nullptr;  // not marked as tried: a later call asks again
    }
    g_scratch_ptr[dev] = ptr;
    g_scratch_tried[dev] = true;
  }
  if (!g_scratch_ptr[dev]) fail(GNNHWC_ERR_LAUNCH, "the library's scratch memory has no address on device %d", dev);
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" {

int gnnhwc_version(void) { return (1 << 16) | 0; }

const char *gnnhwc_last_error(void) { return g_error; }

size_t gnnhwc_fwd_workspace_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype) {
  if (check_shape(N, R, C, G, dtype) != GNNHWC_OK) return 0;
  if (N == 0 || R == 0) return 256;
  return align_up(fwd_ws_bytes(N, R, C, G, dtype), 256);
}
size_t gnnhwc_bwd_workspace_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype) {
  if (check_shape(N, R, C, G, dtype) != GNNHWC_OK) return 0;
  if (N == 0 || R == 0) return 256;
  return align_up(bwd_ws_bytes(N, R, C, G, dtype), 256);
}

static int forward(const void *x, const AddArgs &add, const void *weight, const void *bias, void *y, void *mean, void *rstd,
                   int64_t N, int64_t R, int64_t C, int64_t G, double eps, int act, int dtype, int param_dtype,
                   int stats_dtype, void *workspace, size_t workspace_bytes, void *stream, bool streaming_only = false,
                   int y_dtype = -1) {
  int rc = check_shape(N, R, C, G, dtype);
  if (rc != GNNHWC_OK) return rc;
  rc = check_dtypes(dtype, param_dtype, stats_dtype);
  if (rc != GNNHWC_OK) return rc;
  if (act < GN_ACT_IDENTITY || act > GN_ACT_GELU_TANH)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown activation code %d", act);
  if (y_dtype < 0) y_dtype = dtype;
  if (y_dtype != dtype && !(dtype == GN_F32 && (y_dtype == GN_F16 || y_dtype == GN_BF16)))
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "y_dtype %d with dtype %d: y is written in dtype, or as F16 / BF16 for F32 data",
                y_dtype, dtype);
  if (N == 0 || R == 0) return GNNHWC_OK;  // nothing to normalise; mean / rstd of an empty slab are left untouched
  if (!x || !y) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "x and y must not be null");
  if (y_dtype != dtype && y == x) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "y of another type than x cannot replace x in place");
  const size_t need = streaming_only ? align_up(fwd_ws_bytes(N, R, C, G, dtype, true), 256) : gnnhwc_fwd_workspace_bytes(N, R, C, G, dtype);
  if (!workspace || !aligned16(workspace) || workspace_bytes < need)
    return fail(GNNHWC_ERR_WORKSPACE, "forward workspace must be 16-byte aligned and at least %zu bytes (got %p, %zu bytes)",
                need, workspace, workspace_bytes);
  const int vec = 16 / elem_size(dtype);
  const bool vector_ok = C % vec == 0 && aligned16(x) && aligned16(y) && aligned16(add.residual) && aligned16(add.sum_out);
  FwdArgs a;
  a.streaming_only = streaming_only;
  a.add = add;
  a.x = x; a.w = weight; a.b = bias; a.y = y; a.mean = mean; a.rstd = rstd;
  a.eps = eps; a.act = act; a.pdtype = param_dtype; a.sdtype = stats_dtype; a.ydtype = y_dtype;
  a.ws = workspace; a.stream = (hipStream_t)stream;
  a.plan = make_plan(N, R, C, G, vector_ok ? vec : 1, 1);
  if (a.plan.nchunk > 65535) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "too many channels for this build (C = %lld)", (long long)C);
  hipError_t e;
  switch (dtype) {
    case GN_F32: e = launch_fwd_f32(a); break;
    case GN_F64: e = launch_fwd_f64(a); break;
    case GN_F16: e = launch_fwd_f16(a); break;
    default: e = launch_fwd_bf16(a); break;
  }
  if (e != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "forward launch failed: %s", hipGetErrorString(e));
  return GNNHWC_OK;
}

int gnnhwc_fwd(const void *x, const void *weight, const void *bias, void *y, void *mean, void *rstd, int64_t N,
               int64_t R, int64_t C, int64_t G, double eps, int act, int dtype, int param_dtype, int stats_dtype,
               void *workspace, size_t workspace_bytes, void *stream) {
  const AddArgs none = {nullptr, nullptr, GN_F32, nullptr};
  return forward(x, none, weight, bias, y, mean, rstd, N, R, C, G, eps, act, dtype, param_dtype, stats_dtype, workspace,
                 workspace_bytes, stream);
}

int gnnhwc_fwd_cast(const void *x, const void *weight, const void *bias, void *y, void *mean, void *rstd, int64_t N,
                    int64_t R, int64_t C, int64_t G, double eps, int act, int dtype, int param_dtype, int stats_dtype,
                    int y_dtype, void *workspace, size_t workspace_bytes, void *stream) {
  if (y_dtype < GN_F32 || y_dtype > GN_BF16) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown y_dtype code %d", y_dtype);
  const AddArgs none = {nullptr, nullptr, GN_F32, nullptr};
  return forward(x, none, weight, bias, y, mean, rstd, N, R, C, G, eps, act, dtype, param_dtype, stats_dtype, workspace,
                 workspace_bytes, stream, false, y_dtype);
}

size_t gnnhwc_fwd_static_scratch_bytes(int64_t N, int64_t R, int64_t C, int64_t G, int dtype) {
  if (check_shape(N, R, C, G, dtype) != GNNHWC_OK) return 0;
  if (N == 0 || R == 0) return 256;
  return align_up(fwd_ws_bytes(N, R, C, G, dtype, true), 256);
}

int gnnhwc_fwd_static(const void *x, const void *weight, const void *bias, void *y, void *mean, void *rstd, int64_t N,
                      int64_t R, int64_t C, int64_t G, double eps, int act, int dtype, int param_dtype, int stats_dtype,
                      void *stream) {
  int rc = check_shape(N, R, C, G, dtype);
  if (rc != GNNHWC_OK) return rc;
  void *ptr = nullptr;
  if (N > 0 && R > 0) {  // (an empty problem launches nothing and needs no scratch; its other arguments are still checked)
    const size_t need = gnnhwc_fwd_static_scratch_bytes(N, R, C, G, dtype);
    if (need > (size_t)GNNHWC_STATIC_SCRATCH_BYTES)
      return fail(GNNHWC_ERR_WORKSPACE,
                  "gnnhwc_fwd_static: this problem needs %zu bytes of scratch memory, the library's own holds %zu; use "
                  "gnnhwc_fwd with a caller-provided workspace", need, (size_t)GNNHWC_STATIC_SCRATCH_BYTES);
    ptr = static_scratch();
    if (!ptr) return GNNHWC_ERR_LAUNCH;
  }
  // no per-launch events here (creating one allocates): timing is off for the duration of this call
  const bool profiling = g_profile;
  g_profile = false;
  const AddArgs none = {nullptr, nullptr, GN_F32, nullptr};
  rc = forward(x, none, weight, bias, y, mean, rstd, N, R, C, G, eps, act, dtype, param_dtype, stats_dtype, ptr,
               (size_t)GNNHWC_STATIC_SCRATCH_BYTES, stream, true);
  g_profile = profiling;
  return rc;
}

int gnnhwc_fwd_add(const void *x, const void *residual, const void *channel_bias, void *sum_out, const void *weight,
                   const void *bias, void *y, void *mean, void *rstd, int64_t N, int64_t R, int64_t C, int64_t G,
                   double eps, int act, int dtype, int param_dtype, int stats_dtype, int channel_bias_dtype,
                   void *workspace, size_t workspace_bytes, void *stream) {
  if (channel_bias && channel_bias_dtype != dtype && !(channel_bias_dtype == GN_F32 && (dtype == GN_F16 || dtype == GN_BF16)))
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "channel_bias_dtype must equal dtype, or be F32 for F16/BF16 data");
  if (sum_out && sum_out == y)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "sum_out and y must be different buffers");
  const AddArgs add = {residual, channel_bias, channel_bias ? channel_bias_dtype : GN_F32, sum_out};
  return forward(x, add, weight, bias, y, mean, rstd, N, R, C, G, eps, act, dtype, param_dtype, stats_dtype, workspace,
                 workspace_bytes, stream);
}

static int backward(const void *dy, const void *x, const void *weight, const void *bias, const void *mean, const void *rstd,
                    void *dx, void *dweight, void *dbias, int64_t N, int64_t R, int64_t C, int64_t G, int act, int dtype,
                    int param_dtype, int stats_dtype, int dy_dtype, void *workspace, size_t workspace_bytes, void *stream) {
  int rc = check_shape(N, R, C, G, dtype);
  if (rc != GNNHWC_OK) return rc;
  rc = check_dtypes(dtype, param_dtype, stats_dtype);
  if (rc != GNNHWC_OK) return rc;
  if (dy_dtype != dtype && !(dtype == GN_F32 && (dy_dtype == GN_F16 || dy_dtype == GN_BF16)))
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "dy_dtype %d with dtype %d: dy is read in dtype, or as F16 / BF16 for F32 data",
                dy_dtype, dtype);
  if (act < GN_ACT_IDENTITY || act > GN_ACT_GELU_TANH)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown activation code %d", act);
  if (N == 0 || R == 0) {
    // no elements: the parameter gradients are empty sums
    const unsigned grid = (unsigned)((C + 255) / 256);
    if (dweight) hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, dweight, C, param_dtype);
    if (dbias) hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, dbias, C, param_dtype);
    const hipError_t e0 = hipGetLastError();
    if (e0 != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "backward launch failed: %s", hipGetErrorString(e0));
    return GNNHWC_OK;
  }
  if (!dy || !x || !mean || !rstd || !dx)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "dy, x, mean, rstd and dx must not be null");
  const size_t need = gnnhwc_bwd_workspace_bytes(N, R, C, G, dtype);
  if (!workspace || !aligned16(workspace) || workspace_bytes < need)
    return fail(GNNHWC_ERR_WORKSPACE, "backward workspace must be 16-byte aligned and at least %zu bytes (got %p, %zu bytes)",
                need, workspace, workspace_bytes);
  const int vec = 16 / elem_size(dtype);
  if (dy_dtype != dtype && dx == dy) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "dx of another type than dy cannot replace dy in place");
  const bool vector_ok = C % vec == 0 && aligned16(x) && aligned16(dy) && aligned16(dx);
  BwdArgs a;
  a.dydtype = dy_dtype;
  a.dy = dy; a.x = x; a.w = weight; a.b = bias; a.mean = mean; a.rstd = rstd;
  a.dx = dx; a.dw = dweight; a.db = dbias;
  a.act = act; a.pdtype = param_dtype; a.sdtype = stats_dtype;
  a.ws = workspace; a.stream = (hipStream_t)stream;
  a.plan = make_plan(N, R, C, G, vector_ok ? vec : 1, 2);
  if (a.plan.nchunk > 65535) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "too many channels for this build (C = %lld)", (long long)C);
  if (N * G > 0x7fffffffLL) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "N * G too large");
  hipError_t e;
  switch (dtype) {
    case GN_F32: e = launch_bwd_f32(a); break;
    case GN_F64: e = launch_bwd_f64(a); break;
    case GN_F16: e = launch_bwd_f16(a); break;
    default: e = launch_bwd_bf16(a); break;
  }
  if (e != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "backward launch failed: %s", hipGetErrorString(e));
  return GNNHWC_OK;
}

int gnnhwc_bwd(const void *dy, const void *x, const void *weight, const void *bias, const void *mean, const void *rstd,
               void *dx, void *dweight, void *dbias, int64_t N, int64_t R, int64_t C, int64_t G, int act, int dtype,
               int param_dtype, int stats_dtype, void *workspace, size_t workspace_bytes, void *stream) {
  return backward(dy, x, weight, bias, mean, rstd, dx, dweight, dbias, N, R, C, G, act, dtype, param_dtype, stats_dtype, dtype,
                  workspace, workspace_bytes, stream);
}

int gnnhwc_bwd_cast(const void *dy, const void *x, const void *weight, const void *bias, const void *mean, const void *rstd,
                    void *dx, void *dweight, void *dbias, int64_t N, int64_t R, int64_t C, int64_t G, int act, int dtype,
                    int param_dtype, int stats_dtype, int dy_dtype, void *workspace, size_t workspace_bytes, void *stream) {
  if (dy_dtype < GN_F32 || dy_dtype > GN_BF16) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown dy_dtype code %d", dy_dtype);
  return backward(dy, x, weight, bias, mean, rstd, dx, dweight, dbias, N, R, C, G, act, dtype, param_dtype, stats_dtype, dy_dtype,
                  workspace, workspace_bytes, stream);
}

int gnnhwc_profile_enable(int on) {
  g_profile = on != 0;
  return GNNHWC_OK;
}

int gnnhwc_profile_collect(int64_t *launches, double *total_ms) {
  if (!launches || !total_ms) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "null output array");
  for (int k = 0; k < GNNHWC_NUM_KERNEL_KINDS; ++k) { launches[k] = 0; total_ms[k] = 0.0; }
  int rc = GNNHWC_OK;
  for (const Timed &t : g_timed) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(t.stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, t.start, t.stop);
    if (e == hipSuccess) {
      launches[t.kind] += 1;
      total_ms[t.kind] += ms;
    } else {
      rc = fail(GNNHWC_ERR_LAUNCH, "event timing failed: %s", hipGetErrorString(e));
    }
    g_event_pool.push_back(t.start);
    g_event_pool.push_back(t.stop);
  }
  g_timed.clear();
  return rc;
}

int gnnhwc_resident_status(void) { return degraded_since_last_query(); }

int gnnhwc_set_resident(int on) {
  const int before = resident_enabled() ? 1 : 0;
  g_resident.store(on ? 1 : 0, std::memory_order_relaxed);
  return before;
}

int gnnhwc_debug_set_spin_limit(int polls) {
  if (polls < 0 && polls != -2) polls = kDefaultSpinLimit;  // -2: every wait takes the recovery path at once, ready or not
  return g_spin_limit.exchange(polls, std::memory_order_relaxed);
}

int gnnhwc_debug_read_trace(unsigned long long *out, int64_t count) {
#if !GN_TRACE
  return fail(GNNHWC_ERR_INVALID_ARGUMENT, "this library is built without trace points: load libgnnhwc_hip_trace.so "
              "(the Python binding does when GNNHWC_TRACE is set in the environment)");
#endif
  unsigned long long *buf = trace_buffer();
  if (!buf) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "tracing is off (set GNNHWC_TRACE=1 before the first call)");
  const int64_t cap = (int64_t)kMaxResidentBlocks * 8;
  if (!out || count <= 0 || count > cap) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "trace read of %lld words (capacity %lld)", (long long)count, (long long)cap);
  const hipError_t e = hipMemcpy(out, buf, (size_t)count * sizeof(unsigned long long), hipMemcpyDeviceToHost);
  if (e != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "trace read failed: %s", hipGetErrorString(e));
  return GNNHWC_OK;
}

int gnnhwc_debug_last_launch(int64_t *out) {
  if (!out) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "null output array");
  for (int i = 0; i < 7; ++i) out[i] = g_last_launch[i];
  return GNNHWC_OK;
}

int gnnhwc_debug_load_tile(const void *x, const void *dy, void *sink, int64_t N, int64_t R, int64_t row_bytes, int rows_per_lane,
                           void *stream) {
  if (!x || N <= 0 || R <= 0 || row_bytes <= 0 || row_bytes % 128 != 0 || N > 65535 || row_bytes / 128 > 65535 || ((uintptr_t)x | (uintptr_t)dy) % 16 != 0)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "load_tile: rows of a multiple of 128 bytes, at most 65535 samples and chunks, aligned pointers");
  const int64_t tiles = (R + (int64_t)rows_per_lane * 32 - 1) / ((int64_t)rows_per_lane * 32);
  const dim3 grid((unsigned)tiles, (unsigned)(row_bytes / 128), (unsigned)N);
  switch (rows_per_lane) {
    case 4: launch_load_tile<4>(x, dy, sink, grid, (hipStream_t)stream, R, row_bytes); break;
    case 8: launch_load_tile<8>(x, dy, sink, grid, (hipStream_t)stream, R, row_bytes); break;
    case 16: launch_load_tile<16>(x, dy, sink, grid, (hipStream_t)stream, R, row_bytes); break;
    case 22: launch_load_tile<22>(x, dy, sink, grid, (hipStream_t)stream, R, row_bytes); break;
    case 32: launch_load_tile<32>(x, dy, sink, grid, (hipStream_t)stream, R, row_bytes); break;
    default: return fail(GNNHWC_ERR_INVALID_ARGUMENT, "load_tile: rows_per_lane must be 4, 8, 16, 22 or 32");
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "load_tile launch failed: %s", hipGetErrorString(e));
  return GNNHWC_OK;
}

int gnnhwc_debug_copy(void *dst, const void *src, size_t bytes, void *stream) {
  if (!dst || !src || bytes == 0 || bytes % 16 != 0 || ((uintptr_t)dst | (uintptr_t)src) % 16 != 0)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "copy of %zu bytes: pointers and size must be non-null multiples of 16", bytes);
  const int64_t n16 = (int64_t)(bytes / 16);
  const int64_t grid = (n16 + 1023) / 1024;
  if (grid > 0x7fffffff) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "copy of %zu bytes is too large", bytes);
  launch(kKindCopy, copy_kernel, dim3((unsigned)grid), dim3(256), (hipStream_t)stream, (const uint4 *)src, (uint4 *)dst, n16);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "copy launch failed: %s", hipGetErrorString(e));
  return GNNHWC_OK;
}

// ---- channels-first layout -----------------------------------------------------------------------------------
static int nchw_vec(int dtype, int64_t R, const void *a, const void *b, const void *c) {
  const int vec = 16 / elem_size(dtype);
  return (R % vec == 0 && aligned16(a) && aligned16(b) && aligned16(c)) ? vec : 1;
}
size_t gnnhwc_nchw_workspace_bytes(int64_t N, int64_t C, int64_t R, int64_t G, int dtype, int backward) {
  if (check_shape(N, R, C, G, dtype) != GNNHWC_OK) return 0;
  if (N == 0 || R == 0) return 256;
  // the scalar kernels have the most chunks per row: enough for either path
  return align_up(nchw_workspace_elems(N, C, R, 1, backward != 0) * acc_size(dtype), 256);
}
static int nchw_call(NchwArgs &a, int dtype, void *workspace, size_t workspace_bytes, const char *what) {
  const size_t need = gnnhwc_nchw_workspace_bytes(a.N, a.C, a.R, a.G, dtype, a.backward ? 1 : 0);
  if (!workspace || !aligned16(workspace) || workspace_bytes < need)
    return fail(GNNHWC_ERR_WORKSPACE, "%s workspace must be 16-byte aligned and at least %zu bytes (got %p, %zu bytes)", what,
                need, workspace, workspace_bytes);
  // the kernels index the elements of one row, and its chunks, with 32-bit integers
  if (a.R > 0x7fffffffLL - 4096)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "%s: rows of %lld elements are beyond the supported range", what, (long long)a.R);
  const int vec = a.vector ? 16 / (int)elem_size(dtype) : 1;
  const int64_t chunks = (a.R + nchw_chunk_len(vec) - 1) / nchw_chunk_len(vec);
  if ((double)a.N * (double)a.C * (double)chunks / 4.0 > 2.0e9)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "%s: too many rows for one launch (N C = %lld)", what, (long long)(a.N * a.C));
  if ((double)(a.C / a.G) * (double)chunks >= 2147483648.0)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "%s: a group of %lld rows of %lld elements is beyond the supported range", what,
                (long long)(a.C / a.G), (long long)a.R);
  a.ws = workspace;
  hipError_t e;
  switch (dtype) {
    case GN_F32: e = launch_nchw_f32(a); break;
    case GN_F64: e = launch_nchw_f64(a); break;
    case GN_F16: e = launch_nchw_f16(a); break;
    default: e = launch_nchw_bf16(a); break;
  }
  if (e != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "%s launch failed: %s", what, hipGetErrorString(e));
  return GNNHWC_OK;
}

int gnnhwc_fwd_nchw(const void *x, const void *weight, const void *bias, void *y, void *mean, void *rstd, int64_t N,
                    int64_t C, int64_t R, int64_t G, double eps, int act, int dtype, int param_dtype, int stats_dtype,
                    void *workspace, size_t workspace_bytes, void *stream) {
  int rc = check_shape(N, R, C, G, dtype);
  if (rc != GNNHWC_OK) return rc;
  rc = check_dtypes(dtype, param_dtype, stats_dtype);
  if (rc != GNNHWC_OK) return rc;
  if (act < GN_ACT_IDENTITY || act > GN_ACT_GELU_TANH)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown activation code %d", act);
  if (N == 0 || R == 0) return GNNHWC_OK;
  if (!x || !y) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "x and y must not be null");
  NchwArgs a = {};
  a.backward = false;
  a.vector = nchw_vec(dtype, R, x, y, nullptr) > 1;
  a.x = x; a.w = weight; a.b = bias; a.y = y; a.mean_out = mean; a.rstd_out = rstd;
  a.N = N; a.C = C; a.R = R; a.G = G;
  a.eps = eps; a.act = act; a.pdtype = param_dtype; a.sdtype = stats_dtype;
  a.stream = (hipStream_t)stream;
  return nchw_call(a, dtype, workspace, workspace_bytes, "channels-first forward");
}

int gnnhwc_bwd_nchw(const void *dy, const void *x, const void *weight, const void *bias, const void *mean, const void *rstd,
                    void *dx, void *dweight, void *dbias, int64_t N, int64_t C, int64_t R, int64_t G, int act, int dtype,
                    int param_dtype, int stats_dtype, void *workspace, size_t workspace_bytes, void *stream) {
  int rc = check_shape(N, R, C, G, dtype);
  if (rc != GNNHWC_OK) return rc;
  rc = check_dtypes(dtype, param_dtype, stats_dtype);
  if (rc != GNNHWC_OK) return rc;
  if (act < GN_ACT_IDENTITY || act > GN_ACT_GELU_TANH)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "unknown activation code %d", act);
  if (N == 0 || R == 0) {
    const unsigned grid = (unsigned)((C + 255) / 256);
    if (dweight) hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, dweight, C, param_dtype);
    if (dbias) hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, dbias, C, param_dtype);
    const hipError_t e0 = hipGetLastError();
    if (e0 != hipSuccess) return fail(GNNHWC_ERR_LAUNCH, "backward launch failed: %s", hipGetErrorString(e0));
    return GNNHWC_OK;
  }
  if (!dy || !x || !mean || !rstd || !dx)
    return fail(GNNHWC_ERR_INVALID_ARGUMENT, "dy, x, mean, rstd and dx must not be null");
  if (N * G > 0x7fffffffLL) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "N * G too large");
  NchwArgs a = {};
  a.backward = true;
  a.vector = nchw_vec(dtype, R, x, dy, dx) > 1;
  a.x = x; a.dy = dy; a.w = weight; a.b = bias; a.mean = mean; a.rstd = rstd;
  a.dx = dx; a.dw = dweight; a.db = dbias;
  a.N = N; a.C = C; a.R = R; a.G = G;
  a.eps = 0.0; a.act = act; a.pdtype = param_dtype; a.sdtype = stats_dtype;
  a.stream = (hipStream_t)stream;
  return nchw_call(a, dtype, workspace, workspace_bytes, "channels-first backward");
}

int gnnhwc_debug_plan(int64_t N, int64_t R, int64_t C, int64_t G, int dtype, int vector, int backward, int64_t *out) {
  if (!out) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "null output array");
  const int rc = check_shape(N, R, C, G, dtype);
  if (rc != GNNHWC_OK) return rc;
  if (N == 0 || R == 0) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "empty problem: nothing is planned");
  const int vec = 16 / elem_size(dtype);
  if (vector && C % vec != 0) return fail(GNNHWC_ERR_INVALID_ARGUMENT, "C = %lld is not a multiple of the vector width %d", (long long)C, vec);
  const Plan p = make_plan(N, R, C, G, vector ? vec : 1, backward ? 2 : 1);
  const size_t elems = backward ? bwd_workspace(p).total : fwd_workspace(p).total;
  out[0] = p.vec; out[1] = p.cv; out[2] = p.lpr; out[3] = p.nchunk; out[4] = p.rpi; out[5] = p.tile_rows;
  out[6] = p.tiles; out[7] = p.gmax; out[8] = p.nblocks; out[9] = needs_compaction(p) ? 1 : 0;
  out[10] = (int64_t)(kWorkspaceHeader + elems * acc_size(dtype));
  out[11] = p.D;
  return GNNHWC_OK;
}

const char *gnnhwc_kernel_kind_name(int kind) {
  static const char *names[GNNHWC_NUM_KERNEL_KINDS] = {"fwd_stats", "fwd_stats_compact", "fwd_apply", "bwd_reduce",
                                                       "bwd_compact", "bwd_dx", "fused_fwd", "fused_bwd", "copy",
                                                       "fwd_add", "fused_fwd_add",
                                                       "nchw_stats", "nchw_apply", "nchw_bwd_reduce", "nchw_bwd_dx"};
  return (kind >= 0 && kind < GNNHWC_NUM_KERNEL_KINDS) ? names[kind] : "";
}

}  // extern "C"
