// TEST INFRASTRUCTURE ONLY — CPU oracle runtime.  Only tests/, smoke() and the
// cpu_baseline leg of bench.py load this library; the GPU path never does.
//
// Restates the execution model of the reference's multi-thread CPU backend
// (backends/c-mcpu/include/backend.hpp:99-223): a kernel is a function
// `void f(int rank, void** args)`; a launch runs rank = i, i+T, i+2T, ... on
// worker i of a pool of T pinned threads and waits for all of them
// (backend.hpp:192-211); T comes from CPU_THREADS or the hardware concurrency
// (backend.hpp:117-124).  Also restates the evaluator's deterministic input
// fill and output digest (graph_evaluator/run_graph.cpp:125-149,189-208).
#include <pthread.h>
#include <sched.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <vector>
#include "ref_half.h"

typedef void (*kernel_fn)(int, void**);

namespace {

struct Pool {
  std::vector<std::thread> workers;
  std::mutex mu;
  std::condition_variable cv_start, cv_done;
  uint64_t generation = 0;
  int pending = 0;
  bool stop = false;
  kernel_fn fn = nullptr;
  void** args = nullptr;
  int nranks = 0;

  explicit Pool(int threads) {
    int ncpu = (int)std::thread::hardware_concurrency();
    for (int i = 0; i < threads; ++i) {
      workers.emplace_back([this, i, threads] { loop(i, threads); });
      cpu_set_t set;
      CPU_ZERO(&set);
      CPU_SET(ncpu > 0 ? i % ncpu : i, &set);
      pthread_setaffinity_np(workers[i].native_handle(), sizeof(set), &set);  // best effort
    }
  }

  void loop(int id, int threads) {
    uint64_t seen = 0;
    for (;;) {
      kernel_fn f; void** a; int n;
      {
        std::unique_lock<std::mutex> lock(mu);
        cv_start.wait(lock, [&] { return stop || generation != seen; });
        if (stop) return;
        seen = generation; f = fn; a = args; n = nranks;
      }
      for (int r = id; r < n; r += threads) f(r, a);
      {
        std::unique_lock<std::mutex> lock(mu);
        if (--pending == 0) cv_done.notify_all();
      }
    }
  }

  void run(kernel_fn f, int n, void** a) {
    std::unique_lock<std::mutex> lock(mu);
    fn = f; args = a; nranks = n; pending = (int)workers.size(); ++generation;
    cv_start.notify_all();
    cv_done.wait(lock, [&] { return pending == 0; });
  }

  ~Pool() {
    { std::unique_lock<std::mutex> lock(mu); stop = true; }
    cv_start.notify_all();
    for (auto& w : workers) w.join();
  }
};

Pool* g_pool = nullptr;
int g_threads = 0;

}  // namespace

// The harness's own half conversions (graph_evaluator/execute_module.hpp:46-55): bit moves without
// rounding, subnormal or zero handling.  They are part of what fill and digest produce - a float 0.0
// becomes the half 0x4000 (2.0), and the half 0x0000 reads back as 2^-14 - so they are restated as they are.
static inline float harness_h2f(uint16_t in) {
  const uint32_t f = ((uint32_t)(in & 0x8000) << 16) | ((((uint32_t)(in & 0x7c00)) + 0x1C000u) << 13) | ((uint32_t)(in & 0x03FF) << 13);
  float out;
  memcpy(&out, &f, sizeof(out));
  return out;
}
static inline uint16_t harness_f2h(float in) {
  uint32_t x;
  memcpy(&x, &in, sizeof(x));
  return (uint16_t)(((x >> 16) & 0x8000) | ((((x & 0x7f800000u) - 0x38000000u) >> 13) & 0x7c00) | ((x >> 13) & 0x03ff));
}

extern "C" {

// Number of worker threads a launch will use (CPU_THREADS env, else all cores).
int ref_threads(void) {
  if (g_threads) return g_threads;
  const char* env = getenv("CPU_THREADS");
  int t = (env && *env) ? atoi(env) : (int)std::thread::hardware_concurrency();
  g_threads = t > 0 ? t : 1;
  return g_threads;
}

// Resize the pool (0 = back to the default).  Not thread safe, like the reference.
void ref_set_threads(int t) {
  delete g_pool; g_pool = nullptr;
  g_threads = t > 0 ? t : 0;
}

// Run `fn(rank, args)` for rank in [0, nranks) with the reference's striding.
int ref_run(void* fn, int nranks, void** args) {
  if (!fn || nranks < 0) return 1;
  if (!g_pool) g_pool = new Pool(ref_threads());
  g_pool->run((kernel_fn)fn, nranks, args);
  return 0;
}

// Deterministic fill of input number `arg_index` (run_graph.cpp:125-149):
// floats get (x + i + 1) % 71, integer tensors get 0.
int ref_fill(void* data, long long count, const char* dtype, int arg_index) {
  const int i = arg_index;
  if (!strcmp(dtype, "int32")) { for (long long x = 0; x < count; ++x) ((int*)data)[x] = 0; }
  else if (!strcmp(dtype, "int16")) { for (long long x = 0; x < count; ++x) ((short*)data)[x] = 0; }
  else if (!strcmp(dtype, "int64")) { for (long long x = 0; x < count; ++x) ((long long*)data)[x] = 0; }
  else if (!strcmp(dtype, "float16")) { for (long long x = 0; x < count; ++x) ((uint16_t*)data)[x] = harness_f2h((float)((x + i + 1) % 71)); }
  else if (!strcmp(dtype, "float32")) { for (long long x = 0; x < count; ++x) ((float*)data)[x] = (float)((x + i + 1) % 71); }
  else if (!strcmp(dtype, "float64")) { for (long long x = 0; x < count; ++x) ((double*)data)[x] = (double)((x + i + 1) % 71); }
  else if (!strcmp(dtype, "int8") || !strcmp(dtype, "uint8")) {
    // other types: filled as 32-bit words of (x + i + 1) % 71, tail bytes 1
    long long bytes = count, words = bytes / 4;
    for (long long x = 0; x < words; ++x) ((int*)data)[x] = (int)((x + i + 1) % 71);
    for (long long x = bytes - bytes % 4; x < bytes; ++x) ((char*)data)[x] = 1;
  } else return 1;
  return 0;
}

// Output digest (run_graph.cpp:189-208): sum over x of ((x + 1) % 83) * out[x], in double.
int ref_digest(const void* data, long long count, const char* dtype, double* out) {
  double d = 0.0;
  if (!strcmp(dtype, "int32")) { for (long long x = 0; x < count; ++x) d += (double)((x + 1) % 83) * ((const int*)data)[x]; }
  else if (!strcmp(dtype, "int64")) { for (long long x = 0; x < count; ++x) d += (double)((x + 1) % 83) * ((const long long*)data)[x]; }
  else if (!strcmp(dtype, "float16")) { for (long long x = 0; x < count; ++x) d += (double)((x + 1) % 83) * harness_h2f(((const uint16_t*)data)[x]); }
  else if (!strcmp(dtype, "float32")) { for (long long x = 0; x < count; ++x) d += (double)((x + 1) % 83) * ((const float*)data)[x]; }
  else if (!strcmp(dtype, "float64")) { for (long long x = 0; x < count; ++x) d += (double)((x + 1) % 83) * ((const double*)data)[x]; }
  else if (!strcmp(dtype, "int8") || !strcmp(dtype, "uint8") || !strcmp(dtype, "int16")) {
    long long bytes = count * (!strcmp(dtype, "int16") ? 2 : 1);
    for (long long x = 0; x < bytes; ++x) d += (double)((x + 1) % 83) * ((const unsigned char*)data)[x];
  } else return 1;
  *out = d;
  return 0;
}

}  // extern "C"
