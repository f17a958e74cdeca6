// Work-groups of one launch that meet in memory: each leaves its partial result, takes a ticket, and the one that
// draws the last ticket finishes the job (adds the partial results in a fixed order, so the outcome does not depend
// on which group that is). No group ever waits for another.
//
// The partial results travel as device-scope stores and loads, which are written through to, and read from, the
// level all XCDs share. Device-scope fences would do as well but write back and invalidate a whole L2 per use, which
// costs more than the work being split. A wave's stores have completed when its count of outstanding memory
// operations is zero; arrive_last() waits for that ahead of the barrier that precedes the ticket.
#pragma once
#include <hip/hip_runtime.h>

namespace endia {

__device__ __forceinline__ void store_shared(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float load_shared(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by every thread of the group after its store_shared() calls. True, in all threads, for the group that is
// the `expected`-th to arrive at `ticket`; that group also puts the ticket back to zero for the next launch.
// `flag` is one int of LDS that nobody else uses until the call returns.
__device__ __forceinline__ bool arrive_last(unsigned* ticket, unsigned expected, int* flag) {
  // (compiler-only fences: the relaxed accesses around this call keep their program order in the generated code; the
  // hardware side is the wait below)
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned before = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = before + 1u == expected;
    if (last) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last;
  }
  __syncthreads();
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  return *flag != 0;
}

}  // namespace endia
