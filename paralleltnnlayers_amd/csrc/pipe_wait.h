// Bounded waits between the waves of one workgroup, shared by the producer / consumer
// kernels: a wave spins on an LDS word that another wave of the same workgroup
// advances; a wait that runs out is recorded for the host and ends its wave.
#ifndef CP4_PIPE_WAIT_H
#define CP4_PIPE_WAIT_H

#include <hip/hip_runtime.h>

namespace cp4 {
namespace {

// What a wait needs besides its word: the bound on its polls, the workgroup's
// abort word in LDS, the device's sticky fault record and who is asking.
struct WaitCtx {
  int limit;       // polls before a wait gives up
  int* abort;      // LDS: set by the first wave of the workgroup that gives up
  int* fault;      // global, 4 ints: code, workgroup, wave, wait site (null: not recorded)
  int wg, wave;
};

// Wait until *word >= want and return the value seen.  The writer is another
// wave of this workgroup; the spin is bounded so that a logic error cannot hang
// the device.  With `backoff` the naps between polls grow (64, 256, then 1024
// cycles): fewer polls between the producers' LDS traffic on long strips; on
// the shortest strips the wake-up latency of a long nap would cost more.
// A wait that runs out never lets its wave go on with unfinished data: the wave
// records the fault for the host (first one wins; cp4_device_status reports it),
// raises the workgroup's abort word, which ends the other waves' waits early, and
// ends there - none of its later stores happen.  No barrier follows the
// prologue, so a wave may end on its own.
__device__ __forceinline__ int wait_ge(int* word, int want, bool backoff, const WaitCtx& cx,
                                       int site) {
  int v = 0;
  for (int it = 0; it < cx.limit; ++it) {
    v = __hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (v >= want) return v;
    if (!backoff || it < 6) __builtin_amdgcn_s_sleep(1);
    else if (it < 12) __builtin_amdgcn_s_sleep(4);
    else __builtin_amdgcn_s_sleep(16);
    if ((it & 63) == 63 &&
        __hip_atomic_load(cx.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP))
      break;
  }
  if ((threadIdx.x & 63) == 0) {
    __hip_atomic_store(cx.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (cx.fault && atomicCAS(cx.fault, 0, 1) == 0) {
      cx.fault[1] = cx.wg;
      cx.fault[2] = cx.wave;
      cx.fault[3] = site;
    }
  }
  __builtin_amdgcn_endpgm();
}

}  // namespace
}  // namespace cp4
#endif  // CP4_PIPE_WAIT_H
