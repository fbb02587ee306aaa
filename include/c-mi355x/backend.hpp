// namespace ab for the reference's evaluator and plugins, forwarded to libantares_amd.so.
//
// Drop this directory in as backends/c-mi355x/include: graph_evaluator/execute_module.hpp and
// graph_evaluator/run_graph.cpp compile against it unchanged (they include "backend.hpp" and call the
// thirteen functions below; the originals are backends/c-rocm/include/backend.hpp:46-253).
// Everything device-specific lives behind the C ABI of include/antares_amd.h; this header needs no HIP headers.
//
//; eval_flags(c-mi355x): -lantares_amd
#pragma once
#include <stdio.h>
#include <stdlib.h>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "antares_amd.h"

#if !defined(CHECK_OK)
#define CHECK_OK(x) ((x) ? 1 : (fprintf(stderr, "[CheckFail] %s:%d\n", __FILE__, __LINE__), exit(1), 0))
#endif
#define ART_OK(call) ((0 == (call)) ? 1 : (fprintf(stderr, "[CheckFail] %s:%d: %s\n", __FILE__, __LINE__, art_last_error()), exit(1), 0))

namespace ab {

  static std::unordered_map<size_t, std::vector<void*>> _cached_memory;

  inline void init(int dev) {                                            // backend.hpp:51
    static bool ready = false;
    if (dev < 0 && ready) return;
    if (0 != art_init(dev < 0 ? 0 : dev)) throw std::runtime_error(std::string("GPU device is not found: ") + art_last_error());
    ready = true;
  }

  inline void finalize() {}                                              // backend.hpp:75

  inline size_t compute_slotsize(size_t value) {                          // power-of-two buckets, backend.hpp:78-90
    if (value >= (1ULL << 30)) return value;
    size_t slot = 1;
    while (slot < value) slot <<= 1;
    return slot;
  }

  inline void* alloc(size_t byteSize, const std::vector<size_t>&, const std::string&, const std::string&) {   // backend.hpp:92
    init(-1);
    byteSize = compute_slotsize(byteSize);
    auto& bucket = _cached_memory[byteSize];
    if (!bucket.empty()) {
      void* p = bucket.back();
      bucket.pop_back();
      return p;
    }
    void* p = (void*)1LU;
    if (byteSize) ART_OK(art_alloc(byteSize, &p));
    return p;
  }

  inline void release(void* dptr, size_t byteSize) {                     // backend.hpp:110
    _cached_memory[compute_slotsize(byteSize)].push_back(dptr);
  }

  inline std::string moduleCompile(const std::string& source) {          // backend.hpp:116 (in-process instead of hipcc --genco)
    void* blob = nullptr;
    size_t size = 0;
    if (0 != art_module_compile(source.c_str(), "gfx950", &blob, &size)) {
      fprintf(stderr, "%s\n%s\n", art_last_error(), art_compile_log());
      exit(1);
    }
    std::string out((const char*)blob, size);
    art_blob_free(blob);
    return out;
  }

  inline void* moduleLoad(const std::string& binary) {                   // backend.hpp:161
    init(-1);
    std::string compiled;
    const std::string* image = &binary;
    if (binary.size() > 2 && binary[0] == '/' && binary[1] == '/' && binary[2] == ' ') compiled = moduleCompile(binary), image = &compiled;
    art_module* m = nullptr;
    ART_OK(art_module_load(image->data(), image->size(), &m));
    return m;
  }

  // What the evaluator keeps per kernel is opaque to it (it only hands the vector back to launchKernel), so the
  // launch description is one record behind the first element.
  struct KernelLaunch {
    art_func* fn = nullptr;
    unsigned grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
    int first_sizing_arg = 0;                    // `$`: position of the first integer argument that sizes the grid (0: fixed grid)
    long grid_factor = 1;                        // `$$`
    std::vector<long> elements_per_block;        // `$0`, `$1`, ...: negative = that argument does not count
  };

  inline std::vector<void*> moduleGetFunction(const void* hModule, const std::string& fname,
                                              const std::unordered_map<std::string, int>& threads) {   // backend.hpp:172
    auto extent = [&threads](const std::string& key, long fallback) {
      const auto it = threads.find(key);
      return it == threads.end() ? fallback : (long)it->second;
    };
    KernelLaunch* k = new KernelLaunch;          // lives as long as the module: the reference never unloads either
    ART_OK(art_get_function((art_module*)hModule, fname.c_str(), &k->fn));
    static const char* const axes[3] = {"x", "y", "z"};
    for (int a = 0; a < 3; ++a) {
      k->grid[a] = (unsigned)extent(std::string("blockIdx.") + axes[a], 1);
      k->block[a] = (unsigned)extent(std::string("threadIdx.") + axes[a], 1);
    }
    k->first_sizing_arg = (int)extent("$", 0);
    if (k->first_sizing_arg) {                   // grid.x = $$ * prod(ceil(argument_i / $i)), worked out at launch
      k->grid_factor = extent("$$", 1);
      for (long per; (per = extent("$" + std::to_string(k->elements_per_block.size()), 0)) != 0;) k->elements_per_block.push_back(per);
    }
    return {k};
  }

  inline void launchKernel(std::vector<void*>& hFunc, const std::vector<void*>& krnl_args, void* stream) {   // backend.hpp:199
    const KernelLaunch& k = *(const KernelLaunch*)hFunc[0];
    unsigned grid_x = k.grid[0];
    if (k.first_sizing_arg) {
      long blocks = k.grid_factor;
      for (size_t i = 0; i < k.elements_per_block.size(); ++i) {
        const long per = k.elements_per_block[i];
        if (per > 0) blocks *= ((long)(int)(long)krnl_args[k.first_sizing_arg + i] + per - 1) / per;
      }
      if (blocks == 0) return;                   // nothing to do at these sizes
      grid_x = (unsigned)blocks;
    }
    // one 64-bit slot per argument, exactly what the evaluator hands over (execute_module.hpp:340-352)
    ART_OK(art_launch(k.fn, grid_x, k.grid[1], k.grid[2], k.block[0], k.block[1], k.block[2], 0, stream,
                      (const uint64_t*)krnl_args.data(), (int)krnl_args.size()));
  }

  inline void memcpyHtoD(void* dptr, void* hptr, size_t byteSize, void* stream) { ART_OK(art_memcpy_htod(dptr, hptr, byteSize, stream)); }   // :221
  inline void memcpyDtoD(void* dptr, void* dptr0, size_t byteSize, void* stream) { ART_OK(art_memcpy_dtod(dptr, dptr0, byteSize, stream)); }  // :225
  inline void memcpyDtoH(void* hptr, void* dptr, size_t byteSize, void* stream) { ART_OK(art_memcpy_dtoh(hptr, dptr, byteSize, stream)); }   // :229
  inline void synchronize(void* stream) { ART_OK(art_stream_synchronize(stream)); }                                                           // :233

  inline void* recordTime(void* stream) {                                // backend.hpp:237
    void* e = nullptr;
    ART_OK(art_event_create(&e));
    ART_OK(art_event_record(e, stream));
    return e;
  }

  inline double convertToElapsedTime(void* hStart, void* hStop) {        // backend.hpp:244
    float ms = 0.f;
    ART_OK(art_event_elapsed_ms(hStart, hStop, &ms));
    art_event_destroy(hStart);
    art_event_destroy(hStop);
    return ms * 1e-3;
  }
}
