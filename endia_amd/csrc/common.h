// Shared host-side helpers for libendia_hip.so (context, error reporting, launch checks).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/endia_hip.h"

namespace endia {

struct Context {
  bool ready = false;
  bool capturing = false;  // between endia_hip_graph_begin and endia_hip_graph_end
  int device = -1;
  hipStream_t stream = nullptr;
  int cu_count = 0;
  int clock_mhz = 0;
  // Arrival counters of kernels whose work-groups meet in memory (the last one to arrive finishes the job).
  // All zero between launches: the group that arrives last puts its counter back to zero.
  unsigned* tickets = nullptr;
};

constexpr int kTicketCount = 4096;

Context& ctx();
int32_t fail(int32_t code, const char* fmt, ...);

// Scratch memory owned by the library (split-K partials, reduction partials). Grows on demand,
// never shrinks; all users run on the one stream, so consecutive users never overlap.
int32_t workspace(int64_t bytes, void** out);

// Resolves, once per device, the address of the static scratch array of the entry point that allocates nothing
// (reduce.hip). Called by endia_hip_init with `device` current.
int32_t static_scratch_init(int device);

}  // namespace endia

#define ENDIA_REQUIRE_INIT()                                                         \
  do {                                                                               \
    if (!endia::ctx().ready)                                                         \
      return endia::fail(ENDIA_HIP_ERR_NOT_INIT, "%s: endia_hip_init has not run", __func__); \
  } while (0)

#define ENDIA_CHECK_ARG(cond, ...)                                     \
  do {                                                                 \
    if (!(cond)) return endia::fail(ENDIA_HIP_ERR_INVALID, __VA_ARGS__); \
  } while (0)

#define ENDIA_HIP_CALL(expr)                                                              \
  do {                                                                                    \
    hipError_t e_ = (expr);                                                               \
    if (e_ != hipSuccess)                                                                 \
      return endia::fail(e_ == hipErrorOutOfMemory ? ENDIA_HIP_ERR_NOMEM : ENDIA_HIP_ERR_RUNTIME, \
                         "%s: %s failed: %s", __func__, #expr, hipGetErrorString(e_));    \
  } while (0)

#define ENDIA_LAUNCH_CHECK()                                                           \
  do {                                                                                 \
    hipError_t e_ = hipGetLastError();                                                 \
    if (e_ != hipSuccess)                                                              \
      return endia::fail(ENDIA_HIP_ERR_RUNTIME, "%s: kernel launch failed: %s", __func__, \
                         hipGetErrorString(e_));                                       \
  } while (0)

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
