// Device selection, the library stream, buffers, copies, events and scratch.
#include "internal.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <map>
#include <unordered_map>
#include <vector>

namespace mg {

// entry points called so far (every one of them takes the lock first): lets the per-launch timing
// tell whether anything can have been enqueued between two timed launches
static std::atomic<unsigned long long> g_api_calls{0};

std::recursive_mutex &api_mutex() {
  static std::recursive_mutex m;
  ++g_api_calls;
  return m;
}

static thread_local char g_error[512] = "";

static const char *g_plan = "";

void note_plan(const char *text) { g_plan = text ? text : ""; }

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t err, const char *what, const char *file, int line) {
  const char *base = strrchr(file, '/');
  int code = (err == hipErrorOutOfMemory || err == hipErrorMemoryAllocation) ? MG_ERR_OOM
             : (err == hipErrorNoDevice || err == hipErrorInvalidDevice)     ? MG_ERR_NO_DEVICE
                                                                             : MG_ERR_HIP;
  (void)hipGetLastError();  // clear the sticky error so that later calls start clean
  return fail(code, "%s:%d: %s -> %s (%s)", base ? base + 1 : file, line, what, hipGetErrorName(err),
              hipGetErrorString(err));
}

Runtime &runtime() {
  static Runtime r;
  return r;
}

int workspace(size_t nbytes, void **ptr) {
  Runtime &rt = runtime();
  if (nbytes > rt.workspace_bytes) {
    // Work already enqueued may still be reading the old block.
    MG_HIP(hipStreamSynchronize(rt.stream));
    if (rt.workspace) MG_HIP(hipFree(rt.workspace));
    rt.workspace = nullptr;
    rt.workspace_bytes = 0;
    size_t want = (nbytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    MG_HIP(hipMalloc(&rt.workspace, want));
    rt.workspace_bytes = want;
  }
  *ptr = rt.workspace;
  return MG_OK;
}

// ---- per-launch timing -------------------------------------------------------------------
// One event after every timed launch; the event after the launch before it serves as its start
// when nothing else can have been enqueued in between (the earlier scope ended in this entry
// point or in the one called just before it) -- an event record costs a few microseconds of
// stream time, which for launches of 5 - 20 us is a large part of what is being measured.
namespace {
struct TimingRecord {
  int tag;
  size_t start, stop;  // indices into Timing::events
};
struct Timing {
  bool on = false;
  bool paused = false;             // on, but the launches of the moment are not recorded
  std::vector<hipEvent_t> events;  // created once and reused
  std::vector<TimingRecord> records;
  size_t used_events = 0, used = 0;
  bool open = false;               // between timing_begin and timing_end
  size_t open_start = 0;
  int open_tag = 0;
  bool chain = false;              // the last thing enqueued by a timed scope was events[last_stop]
  size_t last_stop = 0;
  unsigned long long chain_call = 0;
} g_timing;
// the next unused event, recorded on the library stream; false if none could be created
bool record_next_event(size_t *index) {
  if (g_timing.used_events == g_timing.events.size()) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
      (void)hipGetLastError();
      g_timing.on = false;
      return false;
    }
    g_timing.events.push_back(e);
  }
  *index = g_timing.used_events++;
  (void)hipEventRecord(g_timing.events[*index], runtime().stream);
  return true;
}
}  // namespace

void timing_begin(int tag) {
  if (!g_timing.on || g_timing.paused) return;
  const unsigned long long call = g_api_calls.load();
  g_timing.open_tag = tag;
  if (g_timing.chain && call - g_timing.chain_call <= 1) {
    g_timing.open_start = g_timing.last_stop;
    g_timing.open = true;
    return;
  }
  g_timing.open = record_next_event(&g_timing.open_start);
}

void timing_end() {
  if (!g_timing.on || !g_timing.open) return;
  g_timing.open = false;
  size_t stop = 0;
  if (!record_next_event(&stop)) return;
  TimingRecord r{g_timing.open_tag, g_timing.open_start, stop};
  if (g_timing.used == g_timing.records.size())
    g_timing.records.push_back(r);
  else
    g_timing.records[g_timing.used] = r;
  ++g_timing.used;
  g_timing.chain = true;
  g_timing.last_stop = stop;
  g_timing.chain_call = g_api_calls.load();
}

static void timing_reset() {
  g_timing.used = 0;
  g_timing.used_events = 0;
  g_timing.open = false;
  g_timing.chain = false;
}

static void timing_release() {
  for (hipEvent_t e : g_timing.events) (void)hipEventDestroy(e);
  g_timing.events.clear();
  g_timing.records.clear();
  timing_reset();
  g_timing.on = false;
}

__global__ void fill_zero_kernel(uint32_t *p, size_t nwords) {
  size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = size_t(gridDim.x) * blockDim.x;
  for (; i < nwords; i += step) p[i] = 0u;
}

// 16 bytes per lane, grid-stride: the plain copy that bandwidth figures are
// calibrated against.
__global__ void __launch_bounds__(256) copy16_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
  size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = size_t(gridDim.x) * blockDim.x;
  for (; i < n16; i += step) dst[i] = src[i];
}

__global__ void fill_zero_bytes_kernel(uint8_t *p, size_t n) {
  size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace mg

using namespace mg;

#define MG_LOCK() std::lock_guard<std::recursive_mutex> mg_guard_(::mg::api_mutex())

// ---- matrix-core rate probe ---------------------------------------------------------
namespace {
// Streams for the memory probe: every 16-byte piece of `big` is stored (or loaded); piece i
// goes with piece i / share of `small`, so the second stream is 1 / share of the first.
__global__ void __launch_bounds__(256) stream_store_kernel(float4 *big, const float4 *small, long long pieces, int share) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= pieces) return;
  float4 v = make_float4(1.f, 2.f, 3.f, 4.f);
  if (share > 0) v = small[i / share];
  v.x += 1.f;
  big[i] = v;
}

__global__ void __launch_bounds__(256) stream_load_kernel(const float4 *big, float4 *small, long long pieces, int share) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= pieces) return;
  const float4 v = big[i];
  // without a second stream the value still has to arrive: the store below never happens for finite data
  if (share > 0 ? i % share == 0 : (v.x != v.x && v.y == 123.25f)) small[share > 0 ? i / share : 0] = v;
}

typedef float probe_f32x4 __attribute__((ext_vector_type(4)));
typedef double probe_f64x4 __attribute__((ext_vector_type(4)));

// 16 independent accumulator tiles (8 for the 4-register fp64 tile) per wave, operands
// fixed in registers: the loop is MFMA instructions and a counter, nothing else.
template <int KIND>
__global__ void __launch_bounds__(256) mfma_probe_kernel(double *sink, int iters) {
  const double seed = 1.0 + 1e-3 * (threadIdx.x & 63);
  double total = 0;
  if constexpr (KIND == 0) {
    probe_f32x4 acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = probe_f32x4{0, 0, 0, 0};
    const float a = (float)seed, b = (float)(2.0 - seed);
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
    for (int i = 0; i < 16; ++i) total += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  } else if constexpr (KIND == 1) {
    probe_f64x4 acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = probe_f64x4{0, 0, 0, 0};
    const double a = seed, b = 2.0 - seed;
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, acc[i], 0, 0, 0);
    for (int i = 0; i < 8; ++i) total += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  } else {
    double acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = 0;
    const double a = seed, b = 2.0 - seed;
    for (int it = 0; it < iters; ++it)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f64_4x4x4f64(a, b, acc[i], 0, 0, 0);
    for (int i = 0; i < 16; ++i) total += acc[i];
  }
  sink[blockIdx.x * 256 + threadIdx.x] = total;
}
}  // namespace

// Blocks given back with mg_free are kept and handed out again: hipMalloc costs tens of
// microseconds and hipFree waits for the whole device, once per result of every operation.
// Everything the library does to a block is ordered on its one stream, so a block may be
// reused as soon as it is given back: whatever was enqueued on it before runs first.
namespace {
struct BlockPool {
  std::multimap<size_t, void *> idle;           // size -> block, not in use
  std::unordered_map<void *, size_t> size_of;   // every block of the pool, in use or idle
  size_t idle_bytes = 0;
  bool off = false;                             // MYGRAD_HIP_POOL=0: plain hipMalloc / hipFree
  bool pinned = false;                          // blocks of pinned host memory (hipHostMalloc)
};
BlockPool &pool() {
  static BlockPool p;
  return p;
}
// Pinned host blocks (results are downloaded into them): allocating and releasing 100 MB
// of pinned memory costs about as much as copying it over the link.
BlockPool &host_pool() {
  static BlockPool p;
  p.pinned = true;
  return p;
}
size_t pool_round(size_t n) {
  const size_t unit = n <= (size_t(1) << 20) ? 512 : (size_t(1) << 21);
  return (n + unit - 1) / unit * unit;
}
// Gives idle blocks back to the driver until at most `keep` bytes of them are left.
void pool_trim(size_t keep, BlockPool &bp = pool()) {
  if (bp.idle_bytes <= keep) return;
  (void)hipStreamSynchronize(runtime().stream);  // work enqueued before the blocks were given back
  while (bp.idle_bytes > keep && !bp.idle.empty()) {
    auto largest = std::prev(bp.idle.end());
    if (bp.pinned)
      (void)hipHostFree(largest->second);
    else
      (void)hipFree(largest->second);
    bp.idle_bytes -= largest->first;
    bp.size_of.erase(largest->second);
    bp.idle.erase(largest);
  }
}
}  // namespace

extern "C" {

const char *mg_last_error(void) { return g_error; }

const char *mg_last_plan(void) {
  MG_LOCK();
  return g_plan;
}

int mg_init(int device) {
  MG_LOCK();
  Runtime &rt = runtime();
  if (rt.ready) {
    if (device >= 0 && device != rt.device)
      return fail(MG_ERR_BAD_ARG, "already initialised on device %d, asked for %d", rt.device, device);
    return MG_OK;
  }
  int count = 0;
  hipError_t err = hipGetDeviceCount(&count);
  if (err != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return fail(MG_ERR_NO_DEVICE, "no HIP device visible (%s)", err == hipSuccess ? "count == 0" : hipGetErrorName(err));
  }
  if (device < 0) device = 0;
  if (device >= count) return fail(MG_ERR_NO_DEVICE, "device %d requested but only %d visible", device, count);
  MG_HIP(hipSetDevice(device));
  MG_HIP(hipGetDeviceProperties(&rt.props, device));
  if (strncmp(rt.props.gcnArchName, "gfx950", 6) != 0)
    return fail(MG_ERR_NO_DEVICE, "device %d is %s; this library carries gfx950 code only", device,
                rt.props.gcnArchName);
  if (int rc = resolve_static_scratch(device)) return rc;
  MG_HIP(hipStreamCreateWithFlags(&rt.stream, hipStreamNonBlocking));
  {
    const char *flag = getenv("MYGRAD_HIP_POOL");
    pool().off = flag && flag[0] == '0';
  }
  rt.device = device;
  rt.ready = true;
  return MG_OK;
}

int mg_shutdown(void) {
  MG_LOCK();
  Runtime &rt = runtime();
  if (!rt.ready) return MG_OK;
  MG_HIP(hipStreamSynchronize(rt.stream));
  release_conv_plans();
  timing_release();
  if (rt.workspace) MG_HIP(hipFree(rt.workspace));
  rt.workspace = nullptr;
  rt.workspace_bytes = 0;
  pool_trim(0);  // idle blocks go back to the driver; blocks still held by callers stay theirs
  pool_trim(0, host_pool());
  MG_HIP(hipStreamDestroy(rt.stream));
  rt.stream = nullptr;
  rt.ready = false;
  rt.device = -1;
  return MG_OK;
}

int mg_device_info(mg_device_info_t *info) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!info) return fail(MG_ERR_BAD_ARG, "info is null");
  const hipDeviceProp_t &p = runtime().props;
  memset(info, 0, sizeof *info);
  strncpy(info->name, p.gcnArchName, sizeof info->name - 1);
  info->compute_units = p.multiProcessorCount;
  info->clock_khz = p.clockRate;
  info->wavefront = p.warpSize;
  info->lds_bytes_per_block = (int32_t)p.sharedMemPerBlock;
  info->hbm_bytes = (int64_t)p.totalGlobalMem;
  info->l2_bytes = p.l2CacheSize;
  info->memory_clock_khz = p.memoryClockRate;
  info->memory_bus_bits = p.memoryBusWidth;
  return MG_OK;
}

int mg_malloc(void **dptr, size_t nbytes) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!dptr) return fail(MG_ERR_BAD_ARG, "dptr is null");
  *dptr = nullptr;
  if (nbytes == 0) nbytes = 256;  // keep a distinct, valid pointer for empty tensors
  BlockPool &bp = pool();
  if (bp.off) {
    MG_HIP(hipMalloc(dptr, nbytes));
    return MG_OK;
  }
  const size_t want = pool_round(nbytes);
  auto fit = bp.idle.lower_bound(want);
  if (fit != bp.idle.end() && fit->first <= want + want / 4) {  // at most a quarter of it unused
    *dptr = fit->second;
    bp.idle_bytes -= fit->first;
    bp.idle.erase(fit);
    return MG_OK;
  }
  hipError_t err = hipMalloc(dptr, want);
  if ((err == hipErrorOutOfMemory || err == hipErrorMemoryAllocation) && bp.idle_bytes > 0) {
    (void)hipGetLastError();
    pool_trim(0);
    err = hipMalloc(dptr, want);
  }
  if (err != hipSuccess) {
    *dptr = nullptr;
    return hip_fail(err, "hipMalloc", __FILE__, __LINE__);
  }
  bp.size_of[*dptr] = want;
  return MG_OK;
}

int mg_free(void *dptr) {
  MG_LOCK();
  if (!dptr) return MG_OK;
  BlockPool &bp = pool();
  auto known = bp.size_of.find(dptr);
  if (!runtime().ready) {
    // a block that outlived mg_shutdown: there is no stream left to order its reuse on,
    // so it goes straight back to the driver (hipFree waits for the device)
    if (known != bp.size_of.end()) bp.size_of.erase(known);
    MG_HIP(hipFree(dptr));
    return MG_OK;
  }
  if (known == bp.size_of.end()) {
    // not from the pool: hipFree waits for the device, so no kernel can still be using it
    MG_HIP(hipFree(dptr));
    return MG_OK;
  }
  bp.idle.emplace(known->second, dptr);
  bp.idle_bytes += known->second;
  // keep at most a quarter of the device's memory idle
  const size_t limit = runtime().props.totalGlobalMem / 4;
  if (bp.idle_bytes > limit) pool_trim(limit / 2);
  return MG_OK;
}

int mg_host_alloc(void **hptr, size_t nbytes) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!hptr) return fail(MG_ERR_BAD_ARG, "hptr is null");
  *hptr = nullptr;
  if (nbytes == 0) nbytes = 64;
  BlockPool &bp = host_pool();
  if (pool().off) {
    MG_HIP(hipHostMalloc(hptr, nbytes, hipHostMallocDefault));
    return MG_OK;
  }
  const size_t want = pool_round(nbytes);
  auto fit = bp.idle.lower_bound(want);
  if (fit != bp.idle.end() && fit->first <= want + want / 4) {
    *hptr = fit->second;
    bp.idle_bytes -= fit->first;
    bp.idle.erase(fit);
    return MG_OK;
  }
  hipError_t err = hipHostMalloc(hptr, want, hipHostMallocDefault);
  if (err != hipSuccess && bp.idle_bytes > 0) {
    (void)hipGetLastError();
    pool_trim(0, bp);
    err = hipHostMalloc(hptr, want, hipHostMallocDefault);
  }
  if (err != hipSuccess) {
    *hptr = nullptr;
    return hip_fail(err, "hipHostMalloc", __FILE__, __LINE__);
  }
  bp.size_of[*hptr] = want;
  return MG_OK;
}

int mg_host_free(void *hptr) {
  MG_LOCK();
  if (!hptr) return MG_OK;
  BlockPool &bp = host_pool();
  auto known = bp.size_of.find(hptr);
  if (!runtime().ready) {  // a pinned block that outlived mg_shutdown
    if (known != bp.size_of.end()) bp.size_of.erase(known);
    MG_HIP(hipHostFree(hptr));
    return MG_OK;
  }
  if (known == bp.size_of.end()) {
    MG_HIP(hipHostFree(hptr));
    return MG_OK;
  }
  // copies into and out of pinned blocks return only when they are done, so nothing is in flight
  bp.idle.emplace(known->second, hptr);
  bp.idle_bytes += known->second;
  const size_t limit = size_t(8) << 30;  // at most 8 GiB of pinned memory kept idle
  if (bp.idle_bytes > limit) pool_trim(limit / 2, bp);
  return MG_OK;
}

int mg_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (nbytes == 0) return MG_OK;
  if (!dst_dev || !src_host) return fail(MG_ERR_BAD_ARG, "null pointer in mg_memcpy_h2d");
  Runtime &rt = runtime();
  MG_HIP(hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, rt.stream));
  // The source may be pageable and may be reused by the caller right away.
  MG_HIP(hipStreamSynchronize(rt.stream));
  return MG_OK;
}

int mg_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (nbytes == 0) return MG_OK;
  if (!dst_host || !src_dev) return fail(MG_ERR_BAD_ARG, "null pointer in mg_memcpy_d2h");
  Runtime &rt = runtime();
  MG_HIP(hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, rt.stream));
  MG_HIP(hipStreamSynchronize(rt.stream));
  return MG_OK;
}

int mg_memcpy_d2d(void *dst_dev, const void *src_dev, size_t nbytes) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (nbytes == 0) return MG_OK;
  if (!dst_dev || !src_dev) return fail(MG_ERR_BAD_ARG, "null pointer in mg_memcpy_d2d");
  Runtime &rt = runtime();
  const bool aligned = ((reinterpret_cast<uintptr_t>(dst_dev) | reinterpret_cast<uintptr_t>(src_dev) | nbytes) & 15u) == 0;
  if (!aligned) {
    MG_HIP(hipMemcpyAsync(dst_dev, src_dev, nbytes, hipMemcpyDeviceToDevice, rt.stream));
    return MG_OK;
  }
  const size_t n16 = nbytes / 16;
  size_t blocks = (n16 + 255) / 256;
  const size_t cap = size_t(rt.props.multiProcessorCount) * 16;
  if (blocks > cap) blocks = cap;
  ScopedTiming timed(TAG_COPY);
  hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, rt.stream, static_cast<const uint4 *>(src_dev),
                     static_cast<uint4 *>(dst_dev), n16);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_memset_zero(void *dst_dev, size_t nbytes) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (nbytes == 0) return MG_OK;
  if (!dst_dev) return fail(MG_ERR_BAD_ARG, "null pointer in mg_memset_zero");
  Runtime &rt = runtime();
  const size_t nwords = nbytes / 4, tail = nbytes % 4;
  if ((reinterpret_cast<uintptr_t>(dst_dev) & 3u) != 0)
    return fail(MG_ERR_BAD_ARG, "mg_memset_zero needs a 4-byte aligned pointer");
  if (nwords) {
    size_t blocks = (nwords + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, rt.stream,
                       static_cast<uint32_t *>(dst_dev), nwords);
  }
  if (tail)
    hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(1), dim3(64), 0, rt.stream,
                       static_cast<uint8_t *>(dst_dev) + nwords * 4, tail);
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_sync(void) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  MG_HIP(hipStreamSynchronize(runtime().stream));
  return MG_OK;
}

int mg_timing_enable(int on) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  MG_HIP(hipStreamSynchronize(runtime().stream));
  timing_reset();
  g_timing.on = on != 0;
  g_timing.paused = false;
  return MG_OK;
}

int mg_timing_pause(int paused) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  g_timing.paused = paused != 0;
  g_timing.chain = false;  // whatever is enqueued while paused lies between the last event and the next
  return MG_OK;
}

int mg_timing_read(int32_t *tags, float *ms, int capacity, int *count) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!count || (capacity > 0 && (!tags || !ms))) return fail(MG_ERR_BAD_ARG, "null argument in mg_timing_read");
  MG_HIP(hipStreamSynchronize(runtime().stream));
  const int n = (int)g_timing.used;
  *count = n;
  for (int i = 0; i < n && i < capacity; ++i) {
    tags[i] = g_timing.records[i].tag;
    MG_HIP(hipEventElapsedTime(&ms[i], g_timing.events[g_timing.records[i].start], g_timing.events[g_timing.records[i].stop]));
  }
  timing_reset();
  return MG_OK;
}

int mg_probe_stream(void *big_dev, void *small_dev, size_t big_bytes, int share, int store_big, float *ms) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!big_dev || !small_dev || !ms) return fail(MG_ERR_BAD_ARG, "null argument in mg_probe_stream");
  if (big_bytes < 16 || big_bytes % 16 != 0) return fail(MG_ERR_BAD_ARG, "mg_probe_stream: %zu bytes (a multiple of 16 wanted)", big_bytes);
  if (share < 0) return fail(MG_ERR_BAD_ARG, "mg_probe_stream: share %d (0: no second stream)", share);
  if ((reinterpret_cast<uintptr_t>(big_dev) | reinterpret_cast<uintptr_t>(small_dev)) & 15u)
    return fail(MG_ERR_BAD_ARG, "mg_probe_stream needs 16-byte aligned buffers");
  const long long pieces = (long long)(big_bytes / 16);
  const long long blocks = (pieces + 255) / 256;
  if (blocks > 0x7fffffffll) return fail(MG_ERR_UNSUPPORTED, "mg_probe_stream: %zu bytes are more than one launch covers", big_bytes);
  hipStream_t s = runtime().stream;
  struct EventPair {  // destroyed on every way out
    hipEvent_t t0 = nullptr, t1 = nullptr;
    ~EventPair() {
      if (t0) (void)hipEventDestroy(t0);
      if (t1) (void)hipEventDestroy(t1);
    }
  } ev;
  MG_HIP(hipEventCreate(&ev.t0));
  MG_HIP(hipEventCreate(&ev.t1));
  MG_HIP(hipEventRecord(ev.t0, s));
  if (store_big)
    hipLaunchKernelGGL(stream_store_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (float4 *)big_dev, (const float4 *)small_dev, pieces, share);
  else
    hipLaunchKernelGGL(stream_load_kernel, dim3((unsigned)blocks), dim3(256), 0, s, (const float4 *)big_dev, (float4 *)small_dev, pieces, share);
  MG_HIP(hipEventRecord(ev.t1, s));
  MG_HIP(hipEventSynchronize(ev.t1));
  MG_HIP(hipEventElapsedTime(ms, ev.t0, ev.t1));
  MG_HIP(hipGetLastError());
  return MG_OK;
}

int mg_probe_mfma(int kind, int waves_per_simd, double *tflops) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!tflops) return fail(MG_ERR_BAD_ARG, "tflops is null");
  if (kind < 0 || kind > 2) return fail(MG_ERR_BAD_ARG, "mfma probe kind %d (0..2)", kind);
  if (waves_per_simd < 1 || waves_per_simd > 8) return fail(MG_ERR_BAD_ARG, "waves_per_simd %d (1..8)", waves_per_simd);
  const int cus = runtime().props.multiProcessorCount;
  const int blocks = cus * waves_per_simd;  // 256 threads = one wave on each of a unit's 4 SIMDs
  const int iters = 4000;
  void *sink = nullptr;
  if (int rc = workspace((size_t)blocks * 256 * sizeof(double), &sink)) return rc;
  hipStream_t s = runtime().stream;
  struct EventPair {  // destroyed on every way out
    hipEvent_t t0 = nullptr, t1 = nullptr;
    ~EventPair() {
      if (t0) (void)hipEventDestroy(t0);
      if (t1) (void)hipEventDestroy(t1);
    }
  } ev;
  MG_HIP(hipEventCreate(&ev.t0));
  MG_HIP(hipEventCreate(&ev.t1));
  float best = 0;
  for (int rep = 0; rep < 4; ++rep) {  // the first repetition warms the clocks up
    MG_HIP(hipEventRecord(ev.t0, s));
    if (kind == 0)
      hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(blocks), dim3(256), 0, s, (double *)sink, iters);
    else if (kind == 1)
      hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(blocks), dim3(256), 0, s, (double *)sink, iters);
    else
      hipLaunchKernelGGL(mfma_probe_kernel<2>, dim3(blocks), dim3(256), 0, s, (double *)sink, iters);
    MG_HIP(hipEventRecord(ev.t1, s));
    MG_HIP(hipEventSynchronize(ev.t1));
    float ms = 0;
    MG_HIP(hipEventElapsedTime(&ms, ev.t0, ev.t1));
    if (rep > 0 && ms > 0 && (best == 0 || ms < best)) best = ms;
  }
  if (!(best > 0)) return fail(MG_ERR_HIP, "mfma probe: every timed repetition reported 0 ms");
  const double per_wave = kind == 0 ? 16 * 2048.0 : kind == 1 ? 8 * 2048.0 : 16 * 512.0;  // flops per loop trip
  *tflops = (double)blocks * 4 * iters * per_wave / (best * 1e-3) * 1e-12;
  return MG_OK;
}

int mg_event_create(void **event) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!event) return fail(MG_ERR_BAD_ARG, "event is null");
  hipEvent_t ev;
  MG_HIP(hipEventCreate(&ev));
  *event = ev;
  return MG_OK;
}

int mg_event_record(void *event) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!event) return fail(MG_ERR_BAD_ARG, "event is null");
  MG_HIP(hipEventRecord(static_cast<hipEvent_t>(event), runtime().stream));
  return MG_OK;
}

int mg_event_elapsed_ms(void *start, void *stop, float *ms) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!start || !stop || !ms) return fail(MG_ERR_BAD_ARG, "null argument in mg_event_elapsed_ms");
  MG_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  MG_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return MG_OK;
}

int mg_event_destroy(void *event) {
  MG_LOCK();
  MG_REQUIRE_INIT();
  if (!event) return MG_OK;
  MG_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return MG_OK;
}

}  // extern "C"
