// Stable even-first partition of int32 values on gfx950.
//
// Replaces the reference's three-step pipeline of samples/01_sort_even_first.py:9-27
// (classify scatter into a [2,N] flag plane, torch cumsum over 2N flags, bucket
// scatter; about 64 bytes of traffic per element) by two launches that move
// 12 bytes per element:
//
//   count    reads the input once, leaves the number of even values of every
//            4096-element tile in the workspace; the block that draws the last
//            ticket turns the counts into exclusive prefixes and the total.
//   scatter  reads the input again, ranks the even values of a tile with
//            wavefront ballots + popcounts and a 4-wave prefix through LDS,
//            compacts evens and odds of the tile into LDS and writes each run
//            with fully coalesced stores:
//              even -> out[prefix[t] + rank]
//              odd  -> out[total_even + (t*4096 - prefix[t]) + rank]
//
// The order inside both halves is the input order, and the result is
// bit-identical to the reference pipeline for non-negative inputs (for negative
// odd values the reference's `data % 2` is -1 and indexes out of bounds; here
// parity is the low bit).
#include "art_common.h"

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kVecPerThread = 4;
constexpr int kTile = kThreads * kVecPerThread * 4;   // 4096 elements

__device__ __forceinline__ int even_count4(i32x4 v) {
  return 4 - ((v.x & 1) + (v.y & 1) + (v.z & 1) + (v.w & 1));
}

// Loads vector `j` of this thread (elements 4*(j*256+tid) .. +3 of the tile); elements past n read as odd (1).
__device__ __forceinline__ i32x4 load_vec(const int* __restrict__ in, long long base, int j, long long n) {
  const long long e0 = base + 4LL * (j * kThreads + threadIdx.x);
  if (e0 + 3 < n) return *reinterpret_cast<const i32x4*>(in + e0);
  i32x4 v = {1, 1, 1, 1};
  if (e0 + 0 < n) v.x = in[e0 + 0];
  if (e0 + 1 < n) v.y = in[e0 + 1];
  if (e0 + 2 < n) v.z = in[e0 + 2];
  return v;
}

__global__ __launch_bounds__(kThreads) void partition_count_kernel(const int* __restrict__ in, long long n, int tiles,
                                                                    unsigned int* __restrict__ counts,   // [tiles + 1]
                                                                    unsigned int* __restrict__ ticket) {
  __shared__ unsigned int s_wave[4];
  __shared__ unsigned int s_last;
  const int tid = threadIdx.x;
  for (int t = blockIdx.x; t < tiles; t += gridDim.x) {
    const long long base = (long long)t * kTile;
    unsigned int c = 0;
#pragma unroll
    for (int j = 0; j < kVecPerThread; ++j) c += even_count4(load_vec(in, base, j, n));
    // wavefront sum: xor butterfly
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) c += __shfl_xor(c, m, 64);
    if ((tid & 63) == 0) s_wave[tid >> 6] = c;
    __syncthreads();
    if (tid == 0)
      __hip_atomic_store(&counts[t], s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
  }
  __threadfence();
  if (tid == 0) s_last = (atomicAdd(ticket, 1u) == gridDim.x - 1) ? 1u : 0u;
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  // exclusive scan of counts[0..tiles) in place; counts[tiles] = total.  One block, chunks of 256.
  __shared__ unsigned int s_scan[kThreads];
  unsigned int carry = 0;
  for (int c0 = 0; c0 < tiles; c0 += kThreads) {
    const int i = c0 + tid;
    const unsigned int v = (i < tiles) ? __hip_atomic_load(&counts[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
    s_scan[tid] = v;
    __syncthreads();
    // Hillis-Steele inclusive scan over 256 entries
    for (int off = 1; off < kThreads; off <<= 1) {
      const unsigned int add = (tid >= off) ? s_scan[tid - off] : 0u;
      __syncthreads();
      s_scan[tid] += add;
      __syncthreads();
    }
    if (i < tiles) counts[i] = carry + s_scan[tid] - v;
    carry += s_scan[kThreads - 1];
    __syncthreads();
  }
  if (tid == 0) {
    counts[tiles] = carry;
    *ticket = 0u;
  }
}

__global__ __launch_bounds__(kThreads) void partition_scatter_kernel(const int* __restrict__ in, int* __restrict__ out,
                                                                      long long n, const unsigned int* __restrict__ prefix,
                                                                      int tiles) {
  __shared__ int s_items[kTile];
  __shared__ unsigned int s_wave[4][kVecPerThread];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t = blockIdx.x;
  const long long base = (long long)t * kTile;
  const long long valid = (n - base < kTile) ? (n - base) : kTile;      // elements of this tile that exist
  const unsigned int tile_prefix = prefix[t];
  const unsigned int total_even = prefix[tiles];

  i32x4 v[kVecPerThread];
  unsigned int cnt[kVecPerThread], incl[kVecPerThread];
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    v[j] = load_vec(in, base, j, n);
    cnt[j] = even_count4(v[j]);
  }
  // inclusive prefix of cnt[j] over the lanes of the wavefront
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    unsigned int s = cnt[j];
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned int up = __shfl_up(s, off, 64);
      if (lane >= off) s += up;
    }
    incl[j] = s;
    if (lane == 63) s_wave[wave][j] = s;
  }
  __syncthreads();
  // evens before (j, wave, lane) in tile order (j outermost, then thread id)
  unsigned int tile_even = 0, before[kVecPerThread];
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    unsigned int b = tile_even;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) b += s_wave[w][j];
      tile_even += s_wave[w][j];
    }
    before[j] = b + incl[j] - cnt[j];
  }
  // compact into LDS: evens to [0, tile_even), odds to [tile_even, kTile)
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) {
    const unsigned int p0 = 4u * (j * kThreads + tid);      // tile-order index of v[j].x
    unsigned int ev = before[j];
    const int items[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool is_even = (items[e] & 1) == 0;
      const unsigned int dst = is_even ? ev : (tile_even + (p0 + e - ev));
      s_items[dst] = items[e];
      ev += is_even ? 1u : 0u;
    }
  }
  __syncthreads();
  const long long odd_base = (long long)total_even + (base - tile_prefix);
  const unsigned int tile_odd = (unsigned int)valid - tile_even;     // padded elements were counted as odd and sit last
  for (unsigned int i = tid; i < tile_even; i += kThreads) out[tile_prefix + i] = s_items[i];
  for (unsigned int i = tid; i < tile_odd; i += kThreads) out[odd_base + i] = s_items[tile_even + i];
}

}  // namespace

extern "C" int art_partition_even_first_i32(const void* in_dev, void* out_dev, long long n, void* stream) {
  ART_REQUIRE(n >= 0, "art_partition_even_first_i32: negative length");
  if (n == 0) return 0;
  ART_REQUIRE(in_dev && out_dev && in_dev != out_dev, "art_partition_even_first_i32: null or aliased pointers");
  ART_REQUIRE(((uintptr_t)in_dev % 16) == 0, "art_partition_even_first_i32: input must be 16-byte aligned");
  art::Workspace& ws = art::workspace();
  ART_REQUIRE(ws.base != nullptr, "art_partition_even_first_i32: call art_init first");
  const long long tiles_ll = (n + kTile - 1) / kTile;
  ART_REQUIRE(art::kScratchOffset + (size_t)(tiles_ll + 1) * 4 <= ws.bytes, "art_partition_even_first_i32: n too large (%lld)", n);
  const int tiles = (int)tiles_ll;
  unsigned int* ticket = reinterpret_cast<unsigned int*>(reinterpret_cast<char*>(ws.base) + art::kScanTicketOffset);
  unsigned int* counts = reinterpret_cast<unsigned int*>(reinterpret_cast<char*>(ws.base) + art::kScratchOffset);
  hipStream_t st = (hipStream_t)stream;
  const int count_blocks = tiles < 2048 ? tiles : 2048;
  partition_count_kernel<<<dim3(count_blocks), dim3(kThreads), 0, st>>>((const int*)in_dev, n, tiles, counts, ticket);
  ART_LAUNCH_CHECK();
  partition_scatter_kernel<<<dim3(tiles), dim3(kThreads), 0, st>>>((const int*)in_dev, (int*)out_dev, n, counts, tiles);
  ART_LAUNCH_CHECK();
  return 0;
}
