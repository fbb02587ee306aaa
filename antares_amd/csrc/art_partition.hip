// Stable even-first partition of int32 values on gfx950.
//
// Replaces the reference's three-step pipeline of samples/01_sort_even_first.py:9-27
// (classify scatter into a [2,N] flag plane, torch cumsum over 2N flags, bucket
// scatter; about 64 bytes of traffic per element) by two launches that move
// 12 bytes per element and need no atomics, fences or zeroed state (the barriers
// inside the scatter kernel order LDS only, so the next tile's loads stay in flight):
//
//   count    block b reads its span of the input (a whole number of
//            4096-element tiles) and stores the number of even values in
//            counts[b].
//   scatter  block b adds up counts[0..b) and counts[b..B) (B = 1024 words unless
//            the caller chooses otherwise, served by L2) to get the number of
//            evens before its span and the total; then, tile by tile, it ranks
//            the even values with wavefront ballots (v_mbcnt for the lanes below,
//            a population count for the total) + a 4-wave prefix through LDS, compacts evens
//            and odds of the tile in LDS and writes both runs with fully
//            coalesced 16-byte non-temporal stores:
//              even -> out[evens_before + rank]
//              odd  -> out[total_even + odds_before + rank]
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
template <bool LAST_USE = false>
__device__ __forceinline__ i32x4 load_vec(const int* __restrict__ in, long long base, int j, long long n) {
  const long long e0 = base + 4LL * (j * kThreads + threadIdx.x);
  if (e0 + 3 < n) {
    if (LAST_USE) return __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(in + e0));   // the scatter pass is the last reader
    return *reinterpret_cast<const i32x4*>(in + e0);
  }
  i32x4 v = {1, 1, 1, 1};
  if (e0 + 0 < n) v.x = in[e0 + 0];
  if (e0 + 1 < n) v.y = in[e0 + 1];
  if (e0 + 2 < n) v.z = in[e0 + 2];
  return v;
}

__global__ __launch_bounds__(kThreads) void partition_count_kernel(const int* __restrict__ in, long long n, int tiles_per_block,
                                                                    unsigned int* __restrict__ counts) {
  __shared__ unsigned int s_wave[4];
  const int tid = threadIdx.x;
  unsigned int c = 0;
  const long long first = (long long)blockIdx.x * tiles_per_block * kTile;
  for (int s = 0; s < tiles_per_block; s += 2) {       // two tiles (eight 16-byte loads per thread) in flight at a time
    i32x4 a[kVecPerThread], b2[kVecPerThread];
    const long long base = first + (long long)s * kTile;
#pragma unroll
    for (int j = 0; j < kVecPerThread; ++j) a[j] = load_vec(in, base, j, n);                 // past n: reads as odd, counts 0
#pragma unroll
    for (int j = 0; j < kVecPerThread; ++j) b2[j] = (s + 1 < tiles_per_block) ? load_vec(in, base + kTile, j, n) : i32x4{1, 1, 1, 1};
#pragma unroll
    for (int j = 0; j < kVecPerThread; ++j) c += even_count4(a[j]) + even_count4(b2[j]);
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) c += __shfl_xor(c, m, 64);
  if ((tid & 63) == 0) s_wave[tid >> 6] = c;
  __syncthreads();
  if (tid == 0) counts[blockIdx.x] = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
}

__global__ __launch_bounds__(kThreads) void partition_scatter_kernel(const int* __restrict__ in, int* __restrict__ out,
                                                                      long long n, const unsigned int* __restrict__ counts,
                                                                      int tiles_per_block) {
  __shared__ int s_items[kTile];
  __shared__ unsigned int s_wave[4][kVecPerThread];
  __shared__ unsigned long long s_sum[4][2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x, nblocks = gridDim.x;

  // first tile's loads go out before the prefix work
  const long long span_base = (long long)b * tiles_per_block * kTile;
  i32x4 v[kVecPerThread];
#pragma unroll
  for (int j = 0; j < kVecPerThread; ++j) v[j] = load_vec<true>(in, span_base, j, n);

  // evens before this block and in total (64-bit: n may exceed 2^31 / 2)
  unsigned long long before_sum = 0, total_sum = 0;
  for (int i = tid; i < nblocks; i += kThreads) {
    const unsigned int c = counts[i];
    total_sum += c;
    if (i < b) before_sum += c;
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    before_sum += __shfl_xor(before_sum, m, 64);
    total_sum += __shfl_xor(total_sum, m, 64);
  }
  if (lane == 0) { s_sum[wave][0] = before_sum; s_sum[wave][1] = total_sum; }
  art_lds_barrier();
  long long even_before = (long long)(s_sum[0][0] + s_sum[1][0] + s_sum[2][0] + s_sum[3][0]);
  const long long total_even = (long long)(s_sum[0][1] + s_sum[1][1] + s_sum[2][1] + s_sum[3][1]);

  for (int s = 0; s < tiles_per_block; ++s) {
    const long long base = span_base + (long long)s * kTile;
    if (base >= n) break;
    // the next tile's loads go out before this tile is ranked and written
    i32x4 vn[kVecPerThread];
    const bool more = (s + 1 < tiles_per_block) && (base + kTile < n);
    if (more) {
#pragma unroll
      for (int j = 0; j < kVecPerThread; ++j) vn[j] = load_vec<true>(in, base + kTile, j, n);
    }
    const long long valid = (n - base < kTile) ? (n - base) : kTile;      // elements of this tile that exist
    // Evens of vector j in the lanes below this one, and in the whole wavefront: one ballot per element slot, the
    // lanes below counted with v_mbcnt, the wavefront total with a scalar population count.
    unsigned int excl[kVecPerThread];
#pragma unroll
    for (int j = 0; j < kVecPerThread; ++j) {
      const int items[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
      unsigned int below = 0, total = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned long long m = __ballot((items[e] & 1) == 0);
        below = __builtin_amdgcn_mbcnt_hi((unsigned int)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned int)m, below));
        total += (unsigned int)__popcll(m);
      }
      excl[j] = below;
      if (lane == 0) s_wave[wave][j] = total;
    }
    art_lds_barrier();
    // evens before (j, wave, lane) in tile order (j outermost, then thread id)
    unsigned int tile_even = 0, before[kVecPerThread];
#pragma unroll
    for (int j = 0; j < kVecPerThread; ++j) {
      unsigned int acc = tile_even;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (w < wave) acc += s_wave[w][j];
        tile_even += s_wave[w][j];
      }
      before[j] = acc + excl[j];
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
    art_lds_barrier();
    const long long odd_base = total_even + (base - even_before);
    const unsigned int tile_odd = (unsigned int)valid - tile_even;     // padding was counted as odd and sits last
    // Both runs leave as 16-byte non-temporal stores (written once, read by nobody here): up to three elements
    // bring the destination to a 16-byte boundary, whole vectors follow, up to three elements finish the run.
    auto flush_run = [&](long long dst0, unsigned int src0, unsigned int count) {
      const unsigned int to_boundary = (4u - (unsigned int)((reinterpret_cast<uintptr_t>(out + dst0) >> 2) & 3)) & 3u;
      const unsigned int head = to_boundary < count ? to_boundary : count;
      const unsigned int vecs = (count - head) >> 2, tail = (count - head) & 3;
      if (tid < head) __builtin_nontemporal_store(s_items[src0 + tid], &out[dst0 + tid]);
      for (unsigned int q = tid; q < vecs; q += kThreads) {
        const unsigned int s = src0 + head + 4 * q;
        const i32x4 pack = {s_items[s], s_items[s + 1], s_items[s + 2], s_items[s + 3]};
        __builtin_nontemporal_store(pack, reinterpret_cast<i32x4*>(out + dst0 + head + 4 * (long long)q));
      }
      if (tid < tail) __builtin_nontemporal_store(s_items[src0 + head + 4 * vecs + tid], &out[dst0 + head + 4 * (long long)vecs + tid]);
    };
    flush_run(even_before, 0, tile_even);
    flush_run(odd_base, tile_even, tile_odd);
    even_before += tile_even;
    if (more) {
#pragma unroll
      for (int j = 0; j < kVecPerThread; ++j) v[j] = vn[j];
    }
    art_lds_barrier();                                            // s_items / s_wave are reused by the next tile
  }
}

}  // namespace

extern "C" int art_partition_even_first_i32(const void* in_dev, void* out_dev, long long n, void* stream) {
  return art_partition_even_first_i32_tuned(in_dev, out_dev, n, 0, stream);
}

extern "C" int art_partition_even_first_i32_tuned(const void* in_dev, void* out_dev, long long n, int max_blocks, void* stream) {
  ART_REQUIRE(max_blocks == 0 || (max_blocks >= 64 && max_blocks <= 16384),
              "art_partition_even_first_i32: max_blocks must be 0 (library's choice) or in 64..16384 (got %d)", max_blocks);
  ART_REQUIRE(n >= 0, "art_partition_even_first_i32: negative length");
  if (n == 0) return 0;
  ART_REQUIRE(in_dev && out_dev && in_dev != out_dev, "art_partition_even_first_i32: null or aliased pointers");
  ART_REQUIRE(((uintptr_t)in_dev % 16) == 0, "art_partition_even_first_i32: input must be 16-byte aligned");
  ART_REQUIRE(((uintptr_t)out_dev % 4) == 0, "art_partition_even_first_i32: output must be 4-byte aligned");
  art::Workspace* wsp = art::workspace((hipStream_t)stream);
  if (!wsp) return 1;
  art::Workspace& ws = *wsp;
  const long long tiles = (n + kTile - 1) / kTile;
  const long long kMaxBlocks = max_blocks ? max_blocks : 1024;  // bounds the counts every block adds up (4 KiB from L2 at 1024)
  const int tiles_per_block = (int)((tiles + kMaxBlocks - 1) / kMaxBlocks);
  const int blocks = (int)((tiles + tiles_per_block - 1) / tiles_per_block);
  unsigned int* counts = reinterpret_cast<unsigned int*>(reinterpret_cast<char*>(ws.base) + art::kScratchOffset);
  hipStream_t st = (hipStream_t)stream;
  partition_count_kernel<<<dim3(blocks), dim3(kThreads), 0, st>>>((const int*)in_dev, n, tiles_per_block, counts);
  ART_LAUNCH_CHECK();
  partition_scatter_kernel<<<dim3(blocks), dim3(kThreads), 0, st>>>((const int*)in_dev, (int*)out_dev, n, counts, tiles_per_block);
  ART_LAUNCH_CHECK();
  return 0;
}
