// Internal declarations shared by the translation units of libmygrad_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>

#include "mygrad_hip.h"

namespace mg {

// One global lock: the library is single-stream and not re-entrant.
std::recursive_mutex &api_mutex();

// Records the message that mg_last_error() returns and passes `code` through.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Maps a hipError_t to an mg_status, recording file:line and the HIP message.
int hip_fail(hipError_t err, const char *what, const char *file, int line);

struct Runtime {
  bool ready = false;
  int device = -1;
  hipStream_t stream = nullptr;
  hipDeviceProp_t props{};
  // Grow-only device scratch used by the convolution entry points (packed
  // filters, split-K partial sums).  Never handed to callers.
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
};

Runtime &runtime();

// Returns a device scratch area of at least `nbytes` (256-byte aligned), growing
// the allocation when needed.  Stream-ordered users may rely on its contents only
// until the next call that asks for workspace.
int workspace(size_t nbytes, void **ptr);

// Optional per-launch timing with HIP events on the library stream (off by
// default).  A launch site brackets its kernel with timing_begin/timing_end.
enum KernelTag {
  TAG_CONV_FWD = 1,
  TAG_CONV_DGRAD = 2,
  TAG_CONV_WGRAD = 3,
  TAG_WGRAD_REDUCE = 4,
  TAG_PACK_FILTERS = 5,
  TAG_POOL_FWD = 6,
  TAG_POOL_BWD = 7,
  TAG_COPY = 8,
  TAG_ELEMENTWISE = 9,
  TAG_REDUCE_ALL = 10,
  TAG_BN_STATS = 11,
  TAG_BN_APPLY = 12,
  TAG_BN_BWD_SUMS = 13,
  TAG_BN_BWD_APPLY = 14,
  TAG_REPEAT_FWD = 15,
  TAG_REPEAT_BWD = 16,
  TAG_WINDOW_GATHER = 17,
  TAG_SUM_OVER = 18,
  TAG_PERMUTE = 19,
  TAG_BATCHED_PRODUCT = 20,
};
void timing_begin(int tag);
void timing_end();

struct ScopedTiming {
  explicit ScopedTiming(int tag) { timing_begin(tag); }
  ~ScopedTiming() { timing_end(); }
};

// Remembers which kernel family (and tile) the entry point that is running chose: what
// mg_last_plan() returns.  `text` must outlive the next call (a literal, or a cached plan's note).
void note_plan(const char *text);

// Drops every cached convolution plan (device tables); called by mg_shutdown.
void release_conv_plans();

// Looks up the address of the file-scope device array behind mg_sum_all_static on `device`,
// which must be the current device; called once per device by mg_init.
int resolve_static_scratch(int device);

#define MG_HIP(expr)                                                   \
  do {                                                                 \
    hipError_t mg_err_ = (expr);                                       \
    if (mg_err_ != hipSuccess) return ::mg::hip_fail(mg_err_, #expr, __FILE__, __LINE__); \
  } while (0)

#define MG_REQUIRE_INIT()                                              \
  do {                                                                 \
    if (!::mg::runtime().ready)                                        \
      return ::mg::fail(MG_ERR_NOT_INIT, "mg_init() has not been called (or failed)"); \
  } while (0)

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace mg
