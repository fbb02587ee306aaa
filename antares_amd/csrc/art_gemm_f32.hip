// fp32 GEMM on the gfx950 matrix cores:  C[M,N] = A[M,K] @ B[K,N], all fp32, row-major.
//
// Replaces the kernel the reference generates for `output0[N, M] +=! input0[N, K] * input1[K, M]`
// (AntaresIR.md:115; the `gemm_f32` operator its README tunes, README.md:128-150) with its tiled schedule
// (backends/c-rocm/schedule/standard/algo_tiling.py:35-98: one FMA per element, no matrix instructions).
//
// Design for MI355X:
//   * v_mfma_f32_32x32x2_f32: a lane supplies ONE value of each operand per instruction (row or column lane % 32,
//     k = lane / 32), so the matrix pipe is fed from very little LDS traffic: per 8 values of k a lane reads one
//     16-byte vector per 32-row tile of A and one per 32-column tile of B and issues four instructions per tile pair.
//     Instruction m of such a group multiplies k = m (lanes 0-31) and k = 4 + m (lanes 32-63): any assignment of
//     k to instructions is right as long as both operands use the same one, and this one makes a lane's four values
//     contiguous;
//   * block tile 128 x 128 x 32, 256 threads = 2 x 2 wavefronts of 64 x 64 (2 x 2 accumulator tiles, 64 registers);
//     rows of 32 k are full 128-byte lines of A, kept in LDS as [m][k] (row pitch 36 floats: 16-byte aligned and the
//     eight rows of a quarter wavefront on distinct banks); B stays as it lies in memory, [k][n] (512 contiguous bytes
//     per wavefront on the way in, 16-byte LDS stores), and a lane picks its four values of k with four 4-byte reads
//     that 32 lanes spread over 32 banks - transposing B on the way into LDS costs 16-way bank conflicts instead;
//   * global -> registers -> LDS with one tile in flight in registers while the previous one is multiplied, two LDS
//     buffers, one barrier per tile;
//   * C leaves straight from the accumulators: 32 lanes write 128 contiguous bytes of a row.
#include "art_common.h"

namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 128, BN = 128, BK = 32, LD = BK + 4, LDB = BN + 4;
constexpr int kThreads = 256;
constexpr int TILE = BM * LD, TILE_B = BK * LDB;    // floats per operand tile in LDS
constexpr size_t kLdsBytes = (size_t)2 * (TILE + TILE_B) * sizeof(float);     // A and B, two buffers each: 70656

__global__ __launch_bounds__(kThreads) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                             float* __restrict__ C, int M, int N, int K, int tiles_n) {
  extern __shared__ __align__(16) float smem32[];
  float* As = smem32;                               // [2][BM][LD]
  float* Bs = smem32 + 2 * TILE;                    // [2][BK][LDB]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;

  // global -> registers: four 16-byte chunks of each operand per thread and tile.  Rows past M and columns past N
  // repeat the last valid ones; their products are never stored.
  const float* pa[4];
  const float* pb[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int arow = tm * BM + (tid >> 3) + 32 * i;                  // 8 chunks per row of 32 k
    pa[i] = A + (size_t)(arow < M ? arow : M - 1) * K + (tid & 7) * 4;
    const int bcol = tn * BN + (tid & 31) * 4;                       // 32 chunks per row of 128 n
    pb[i] = B + (size_t)((tid >> 5) + 8 * i) * N + (bcol < N ? bcol : N - 4);
  }
  f32x4 ga[4], gb[4];
  auto load_tiles = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ga[i] = *reinterpret_cast<const f32x4*>(pa[i] + (size_t)kt * BK);
      gb[i] = *reinterpret_cast<const f32x4*>(pb[i] + (size_t)kt * BK * N);
    }
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<f32x4*>(As + buf * TILE + ((tid >> 3) + 32 * i) * LD + (tid & 7) * 4) = ga[i];
      *reinterpret_cast<f32x4*>(Bs + buf * TILE_B + ((tid >> 5) + 8 * i) * LDB + (tid & 31) * 4) = gb[i];
    }
  };

  f16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int row_a = wm * 64 + (lane & 31), col_b = wn * 64 + (lane & 31), k_half = (lane >> 5) * 4;
  const int T = K / BK;
  load_tiles(0);
  store_tiles(0);
  __syncthreads();
  for (int t = 0; t < T; ++t) {
    const int buf = t & 1;
    if (t + 1 < T) load_tiles(t + 1);               // in flight while this tile is multiplied
    const float* as = As + buf * TILE;
    const float* bs = Bs + buf * TILE_B;
#pragma unroll
    for (int g = 0; g < BK / 8; ++g) {
      f32x4 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i] = *reinterpret_cast<const f32x4*>(as + (row_a + 32 * i) * LD + g * 8 + k_half);
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int m = 0; m < 4; ++m) b[j][m] = bs[(g * 8 + k_half + m) * LDB + col_b + 32 * j];
#pragma unroll
      for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][m], b[j][m], acc[i][j], 0, 0, 0);
    }
    if (t + 1 < T) store_tiles(buf ^ 1);            // the other buffer: everybody left it at the last barrier
    __syncthreads();
  }

  // accumulator element r of tile (i, j): row i*32 + (r/4)*8 + (lane/32)*4 + r%4, column j*32 + lane%32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = tn * BN + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = tm * BM + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (row < M && col < N) C[(size_t)row * N + col] = acc[i][j][r];
      }
    }
}

}  // namespace

extern "C" int art_gemm_f32(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, void* stream) {
  ART_REQUIRE(a_dev && b_dev && c_dev, "art_gemm_f32: null pointer");
  ART_REQUIRE(M > 0 && N >= 4 && K > 0 && N % 4 == 0 && K % 32 == 0,
              "art_gemm_f32: N must be a multiple of 4 and K of 32 (M=%d N=%d K=%d)", M, N, K);
  ART_REQUIRE(((uintptr_t)a_dev % 16) == 0 && ((uintptr_t)b_dev % 16) == 0 && ((uintptr_t)c_dev % 4) == 0,
              "art_gemm_f32: A and B must be 16-byte aligned");
  ART_REQUIRE(!art::overlaps(a_dev, (size_t)M * K * 4, c_dev, (size_t)M * N * 4) && !art::overlaps(b_dev, (size_t)K * N * 4, c_dev, (size_t)M * N * 4),
              "art_gemm_f32: C must not overlap A or B");
  static bool configured = false;
  if (!configured) {
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_f32_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBytes));
    configured = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  ART_REQUIRE((long long)tiles_m * tiles_n <= 0x7fffffffLL, "art_gemm_f32: too many tiles");
  gemm_f32_kernel<<<dim3((unsigned)(tiles_m * tiles_n)), dim3(kThreads), kLdsBytes, (hipStream_t)stream>>>(
      (const float*)a_dev, (const float*)b_dev, (float*)c_dev, M, N, K, tiles_n);
  ART_LAUNCH_CHECK();
  return 0;
}
