// fp16 GEMM on the gfx950 matrix cores:  C[M,N] = A[M,K] @ B[K,N], fp32 accumulate, fp16 out,
// all three row-major.
//
// Replaces the kernel the reference generates for `C[N,M] +=! A[N,K] * B[K,M]`
// (AntaresIR.md:115) with its tiled schedule (backends/c-rocm/schedule/standard/algo_tiling.py:35-98:
// scalar loads through LDS, one FMA per element, no matrix instructions).
//
// Design for MI355X:
//   * block tile 256 x 256 x 32, 256 threads = 2 x 2 wavefronts, each wavefront owns 128 x 128 of C as
//     4 x 4 accumulator tiles of v_mfma_f32_32x32x16_f16 (256 accumulator registers per lane, one
//     wavefront per SIMD); 16 MFMAs (512 matrix-core cycles) per 8 KiB of LDS reads.  The same tile can be worked
//     by 512 threads = 2 x 4 wavefronts of 128 x 64 (two wavefronts per SIMD): a launch parameter for tuning runs,
//     not the default - measured side by side it is 3 % slower at 4096^3 and 8 % slower at 8192^3;
//   * A tile in LDS as [m][k] (k contiguous, rows padded by 16 bytes): one ds_read_b128 gives a lane
//     its 8 consecutive k of one row;
//   * B tile in LDS exactly as it lies in memory, [k][n] (n contiguous, rows padded by 64 bytes); the
//     MFMA wants 8 consecutive k per lane for ONE column, which is the transpose: ds_read_b64_tr_b16
//     (new in gfx950) reads a 4(k) x 16(n) patch with 16 lanes and hands lane L the four k of column L.
//     Two such reads make one B operand; the row padding puts the four k rows on disjoint banks;
//   * global -> registers -> LDS with two register stages (indexed statically) and two LDS buffers;
//     the one barrier per tile waits for LDS only, so global loads stay in flight across it;
//   * one wavefront per SIMD means nothing else hides a stall, so every LDS read, LDS write and global
//     load is issued between two MFMAs of the other k-step (sched_group_barrier pins the order);
//   * block -> tile mapping is XCD aware: the 32 blocks that run on one XCD at a time cover a 4 x 8
//     super-tile, so they share 4 A panels and 8 B panels through that XCD's L2;
//   * C goes through LDS once more so that it leaves as 128-bit row-contiguous stores.
#include "art_common.h"

#include <type_traits>

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int A_LD = BK + 8;             // halves per A row in LDS (80 bytes)
constexpr int B_LD = BN + 32;            // halves per B row in LDS (576 bytes = 16 banks past a multiple of 64)
constexpr int A_TILE = BM * A_LD;        // halves
constexpr int B_TILE = BK * B_LD;
constexpr int C_LD = BN + 8;             // halves per C row while staging the output
constexpr size_t kOperandBytes = (size_t)(2 * A_TILE + 2 * B_TILE) * 2;
constexpr size_t kOutputBytes = (size_t)BM * C_LD * 2;
constexpr size_t kLdsBytes = kOperandBytes > kOutputBytes ? kOperandBytes : kOutputBytes;

__device__ __forceinline__ int xcd_tile(int b, int nb) {
  const int q = nb >> 3, r = nb & 7, xcd = b & 7, idx = b >> 3;
  return xcd < r ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
}

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

template <int WN>      // wavefronts along n: 2 (256 threads, 128 x 128 per wavefront) or 4 (512 threads, 128 x 64)
__global__ __launch_bounds__(128 * WN) void gemm_f16_kernel(const _Float16* __restrict__ A, const _Float16* __restrict__ B,
                                                           _Float16* __restrict__ C, int M, int N, int K) {
  constexpr int NT_ = 128 * WN;            // threads
  constexpr int CH = 1024 / NT_;           // 16-byte chunks per thread, operand and stage
  constexpr int NJ = 8 / WN;               // 32-column accumulator tiles per wavefront
  constexpr int WCOLS = 256 / WN;          // columns per wavefront
  extern __shared__ __align__(16) _Float16 smem[];
  _Float16* As = smem;                    // [2][BM][A_LD]
  _Float16* Bs = smem + 2 * A_TILE;       // [2][BK][B_LD]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int MT = (M + BM - 1) / BM, NT = (N + BN - 1) / BN;      // edge tiles are clamped on the way in and cut on the way out
  int tile = xcd_tile(blockIdx.x, gridDim.x), tm, tn;
  if ((MT % 4 == 0) && (NT % 8 == 0)) {   // 4 x 8 super-tiles, row-major inside and outside
    const int super = tile >> 5, in = tile & 31, sn_count = NT >> 3;
    tm = (super / sn_count) * 4 + (in >> 3);
    tn = (super % sn_count) * 8 + (in & 7);
  } else {
    tm = tile / NT;
    tn = tile % NT;
  }

  // global -> register staging: 4 chunks of 16 bytes per thread for each operand and stage.  The
  // per-thread part of every address is computed once; a tile only adds a wave-uniform offset.
  u32x4 ga[2][CH], gb[2][CH];
  const _Float16* pa[CH];
  const _Float16* pb[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    const int c = tid + NT_ * i;
    // rows past M and columns past N repeat the last valid ones: their products are never stored
    const int arow = tm * BM + (c >> 2), bcol = tn * BN + (c & 31) * 8;
    pa[i] = A + (size_t)(arow < M ? arow : M - 1) * K + (c & 3) * 8;
    pb[i] = B + (size_t)(c >> 5) * N + (bcol < N ? bcol : N - 8);
  }
  const size_t b_step = (size_t)BK * N;
  auto load_tiles = [&](int kt, auto tag) {
    constexpr int S = decltype(tag)::value;
    const size_t oa = (size_t)kt * BK, ob = (size_t)kt * b_step;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      ga[S][i] = *reinterpret_cast<const u32x4*>(pa[i] + oa);
      gb[S][i] = *reinterpret_cast<const u32x4*>(pb[i] + ob);
    }
  };
  auto store_tiles = [&](int buf, auto tag) {
    constexpr int S = decltype(tag)::value;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c = tid + NT_ * i;
      *reinterpret_cast<u32x4*>(As + buf * A_TILE + (c >> 2) * A_LD + (c & 3) * 8) = ga[S][i];
      *reinterpret_cast<u32x4*>(Bs + buf * B_TILE + (c >> 5) * B_LD + (c & 31) * 8) = gb[S][i];
    }
  };

  f16v acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // per-lane constants of the operand reads
  const int a_row = wm * 128 + (lane & 31);                 // + i*32
  const int a_k = (lane >> 5) * 8;                          // + kk*16
  const int s = lane & 15;
  const int b_k = (lane >> 5) * 8 + (s >> 2);               // + kk*16 + r*4
  const int b_n = wn * WCOLS + ((lane & 31) >> 4) * 16 + (s & 3) * 4;   // + j*32

  auto load_frags = [&](h8 (&af)[4], h8 (&bf)[NJ], const _Float16* as, const _Float16* bs, int kk) {
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const h8*>(as + (a_row + i * 32) * A_LD + kk * 16 + a_k);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const _Float16* p = bs + (kk * 16 + b_k) * B_LD + b_n + j * 32;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * B_LD));
      const h4 l4 = __builtin_bit_cast(h4, lo), h4v = __builtin_bit_cast(h4, hi);
      bf[j] = h8{l4[0], l4[1], l4[2], l4[3], h4v[0], h4v[1], h4v[2], h4v[3]};
    }
  };
  auto mfma_all = [&](const h8 (&af)[4], const h8 (&bf)[NJ]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
  };

  const int T = K / BK;
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  load_tiles(0, S0{});
  load_tiles(1, S1{});                     // K >= 64: there are at least two tiles
  store_tiles(0, S0{});
  load_tiles(T > 2 ? 2 : T - 1, S0{});
  art_lds_barrier();
  h8 af0[4], bf0[NJ], af1[4], bf1[NJ];
  load_frags(af0, bf0, As, Bs, 0);
  // One tile = two k-steps of 16 MFMAs.  Tile t sits in LDS buffer t & 1.  Register stage `nxt` holds
  // tile t + 1 (requested a tile and a half ago); once it is written to LDS it is refilled with tile
  // t + 3, while stage `cur` keeps tile t + 2 in flight.  Every LDS and global
  // instruction is issued between two MFMAs of the other k-step, so the single wavefront of a SIMD
  // never leaves the matrix core idle while it waits for operands:
  //   first half:   MFMAs of k-step 0  |  operand reads of k-step 1, tile t+1 written to the other buffer
  //   barrier (LDS only)
  //   second half:  MFMAs of k-step 1  |  operand reads of k-step 0 of tile t+1, global loads of tile t+3
  // The sched_group_barrier sequences pin that interleaving (0x008 MFMA, 0x080 LDS, 0x020 global load); sched_barrier(0) closes each half.
  auto k_tile = [&](int t, auto cur, auto nxt, auto last_tag) {
    constexpr bool LAST = decltype(last_tag)::value;
    const int buf = t & 1;
    const _Float16* as = As + buf * A_TILE;
    const _Float16* bs = Bs + buf * B_TILE;
    load_frags(af1, bf1, as, bs, 1);
    if (!LAST) store_tiles(buf ^ 1, nxt);
    mfma_all(af0, bf0);
#pragma unroll
    for (int i = 0; i < 4 * NJ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x080, 1, 0);                   // 12 reads + 8 writes (8 + 4 with 512 threads)
      if (i < 4) __builtin_amdgcn_sched_group_barrier(0x080, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    art_lds_barrier();
    if (!LAST) {
      load_frags(af0, bf0, As + (buf ^ 1) * A_TILE, Bs + (buf ^ 1) * B_TILE, 0);
      load_tiles(t + 3 < T ? t + 3 : T - 1, nxt);      // past the end: a harmless repeat of the last tile
    }
    mfma_all(af1, bf1);
#pragma unroll
    for (int i = 0; i < 4 * NJ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (NJ == 2 || i < 12) __builtin_amdgcn_sched_group_barrier(0x080, 1, 0);      // 12 reads (8 with 512 threads)
      if (NJ == 4 ? (i >= 4 && i < 12) : (i >= 2 && i < 6)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using No = std::false_type;
  // K is a multiple of 64, so T is even.  The last tile stores and reads a repeat of itself: harmless,
  // and it keeps the loop body free of branches, which the instruction interleaving needs.
  for (int t = 0; t < T; t += 2) {
    k_tile(t, S0{}, S1{}, No{});
    k_tile(t + 1, S1{}, S0{}, No{});
  }
  __syncthreads();          // every wavefront is done with the operand buffers before they are reused for C

  // ---- output: registers -> LDS (fp16, [256][C_LD]) -> 128-bit stores
  _Float16* cs = smem;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * 128 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        const int col = wn * WCOLS + j * 32 + (lane & 31);
        cs[row * C_LD + col] = (_Float16)acc[i][j][r];
      }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8192 / NT_; ++i) {
    const int c = tid + NT_ * i;               // 256 rows x 32 chunks of 8 halves
    const int row = c >> 5, ch = c & 31;
    const int grow = tm * BM + row, gcol = tn * BN + ch * 8;
    if (grow < M && gcol < N)
      *reinterpret_cast<u32x4*>(C + (size_t)grow * N + gcol) = *reinterpret_cast<const u32x4*>(cs + row * C_LD + ch * 8);
  }
}

}  // namespace

extern "C" int art_gemm_f16(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, void* stream) {
  return art_gemm_f16_tuned(a_dev, b_dev, c_dev, M, N, K, 0, stream);
}

extern "C" int art_gemm_f16_tuned(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, int threads, void* stream) {
  ART_REQUIRE(a_dev && b_dev && c_dev, "art_gemm_f16: null pointer");
  ART_REQUIRE(M > 0 && N > 0 && K > 0 && N % 8 == 0 && K % 64 == 0,
              "art_gemm_f16: N must be a multiple of 8 and K of 64 (M=%d N=%d K=%d)", M, N, K);
  ART_REQUIRE(((uintptr_t)a_dev % 16) == 0 && ((uintptr_t)b_dev % 16) == 0 && ((uintptr_t)c_dev % 16) == 0,
              "art_gemm_f16: operands must be 16-byte aligned");
  ART_REQUIRE(threads == 0 || threads == 256 || threads == 512, "art_gemm_f16: threads must be 0 (the library's choice), 256 or 512 (got %d)", threads);
  static bool configured = false;
  if (!configured) {
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_f16_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kLdsBytes));
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_f16_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kLdsBytes));
    configured = true;
  }
  const int blocks = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  if (threads == 0) threads = 256;       // one wavefront per SIMD measured faster at every benchmark size
  if (threads == 512)
    gemm_f16_kernel<4><<<dim3(blocks), dim3(512), kLdsBytes, (hipStream_t)stream>>>((const _Float16*)a_dev, (const _Float16*)b_dev,
                                                                                    (_Float16*)c_dev, M, N, K);
  else
    gemm_f16_kernel<2><<<dim3(blocks), dim3(256), kLdsBytes, (hipStream_t)stream>>>((const _Float16*)a_dev, (const _Float16*)b_dev,
                                                                                    (_Float16*)c_dev, M, N, K);
  ART_LAUNCH_CHECK();
  return 0;
}
