// Shared helpers of libantares_amd.so: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string>

#include "../../include/antares_amd.h"

namespace art {

std::string& last_error();
int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

struct Workspace {
  void* base = nullptr;      // device memory
  size_t bytes = 0;
};
// Workspace of (current device, stream).  Launches on one stream are ordered, so they can share partial-result
// memory; launches on different streams are not, so every stream gets a workspace of its own, allocated and zeroed
// the first time the stream is seen (up to kMaxStreamsPerDevice streams per device; that first use must not happen
// while the stream is being captured into a graph, because it allocates).  Returns nullptr with the error set.
Workspace* workspace(hipStream_t stream);
int release_stream(hipStream_t stream);
constexpr int kMaxStreamsPerDevice = 40;      // torch hands out 32 pooled streams per device besides the default one

// Looks up, for the current device, the address of the scratch array built into the code object (used by
// art_gemv_w4a16_noalloc).  Called once per device by art_init.
int gemv_noalloc_setup(int device);

// Compute units of the current device (queried once per device).
int compute_units();

// Blocks per head the split decode attention may use, shared by its producer (art_llm.hip) and the projection that
// merges the per-part records (art_gemv_w4.hip).
constexpr int kMaxAttnParts = 8;

// True when the byte ranges [a, a + an) and [b, b + bn) overlap.
inline bool overlaps(const void* a, size_t an, const void* b, size_t bn) {
  const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
  return a0 < b0 + bn && b0 < a0 + an;
}

// Workspace layout.  The exchange words and the accumulators keep their meaning between launches,
// so they never share bytes with scratch data.
constexpr size_t kExchangeOffset = 0;                    // launch tag + one word per block of the phase-chain probe (tagged, never zeroed again)
constexpr size_t kExchangeBytes = 64 * 1024;
constexpr size_t kSlotOffset = 64 * 1024;                // 64-bit split-K accumulators (zero between launches)
constexpr size_t kScratchOffset = 4 * 1024 * 1024;       // partial sums, tile counts (any content)

}  // namespace art

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load of the wave (vmcnt(0)), which drains register prefetches at each barrier; this one
// leaves them in flight.  Use it only where the data exchanged through the barrier lives in LDS.
__device__ __forceinline__ void art_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#define ART_HIP(expr)                                                                   \
  do {                                                                                  \
    hipError_t _e = (expr);                                                             \
    if (_e != hipSuccess)                                                               \
      return art::fail("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
  } while (0)

#define ART_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) return art::fail(__VA_ARGS__); \
  } while (0)

#define ART_LAUNCH_CHECK()                                                                \
  do {                                                                                    \
    hipError_t _e = hipGetLastError();                                                    \
    if (_e != hipSuccess)                                                                 \
      return art::fail("kernel launch failed: %s (%s:%d)", hipGetErrorString(_e), __FILE__, __LINE__); \
  } while (0)
