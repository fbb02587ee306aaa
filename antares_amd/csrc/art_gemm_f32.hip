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
//     that the two halves of a wavefront (rows 4 k apart, row pitch 136 floats) spread over all 64 banks -
//     transposing B on the way into LDS costs 16-way bank conflicts instead;
//   * global -> registers -> LDS with one tile in flight in registers while the previous one is multiplied, two LDS
//     buffers, one barrier per tile; inside a tile the issue order is pinned (sched_group_barrier): the LDS reads of
//     the next 8 values of k, the 16-byte global reads and the LDS writes each go out one at a time between matrix
//     instructions - issued in bursts they fill the LDS queues and the matrix pipe waits (measured at 4096^3:
//     126 -> 141 TFLOP/s);
//   * block -> tile mapping is XCD aware (a contiguous run of tiles per XCD, walked in 4 x 8 super-tiles);
//   * C leaves straight from the accumulators: 32 lanes write 128 contiguous bytes of a row;
//   * the kernel is a template over the layouts of A ([M][K] or [K][M]) and B ([K][N] or [N][K]): an operand is
//     staged in LDS as it lies in memory and read with a 16-byte vector where k is its contiguous axis, with four
//     4-byte reads where it is not.
#include "art_common.h"

namespace {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 128, BN = 128, BK = 32, LD = BK + 4, LDB = BN + 8;
constexpr int kThreads = 256;
// An operand tile in LDS: 128 rows (m or n) of 32 k when k is the contiguous axis in memory ([x][k], pitch LD), 32 rows
// of 128 m or n when it is not ([k][x], pitch LDB) - either way as it lies in memory.
constexpr int TILE_XK = BM * LD, TILE_KX = BK * LDB;
constexpr int kMaxTile = TILE_XK > TILE_KX ? TILE_XK : TILE_KX;
template <bool TA, bool TB> constexpr size_t lds_bytes() {
  return (size_t)2 * ((TA ? TILE_KX : TILE_XK) + (TB ? TILE_XK : TILE_KX)) * sizeof(float);
}

// TA: A is stored [K][M] (the product is A^T B); TB: B is stored [N][K] (A B^T).
template <bool TA, bool TB>
__global__ __launch_bounds__(kThreads) void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                             float* __restrict__ C, int M, int N, int K, int tiles_n) {
  extern __shared__ __align__(16) float smem32[];
  constexpr int TILE = TA ? TILE_KX : TILE_XK, TILE_B = TB ? TILE_XK : TILE_KX;
  float* As = smem32;                               // [2][BM][LD], or [2][BK][LDB] when TA
  float* Bs = smem32 + 2 * TILE;                    // [2][BK][LDB], or [2][BN][LD] when TB
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  A += (size_t)blockIdx.y * M * K;                  // one product of the batch per grid row
  B += (size_t)blockIdx.y * K * N;
  C += (size_t)blockIdx.y * M * N;
  // block -> tile, XCD aware: workgroups go to the eight XCDs round robin, so the blocks of one XCD get a contiguous
  // run of tiles, and a run is walked in 4 x 8 super-tiles (4 A panels and 8 B panels shared through that XCD's L2)
  int tm, tn;
  {
    const int nb = (int)gridDim.x, b = (int)blockIdx.x;
    const int q = nb >> 3, r = nb & 7, xcd = b & 7, idx = b >> 3;
    const int tile = xcd < r ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
    const int tiles_m = nb / tiles_n;
    if ((tiles_m % 4 == 0) && (tiles_n % 8 == 0)) {
      const int super = tile >> 5, in = tile & 31, sn = tiles_n >> 3;
      tm = (super / sn) * 4 + (in >> 3);
      tn = (super % sn) * 8 + (in & 7);
    } else {
      tm = tile / tiles_n;
      tn = tile % tiles_n;
    }
  }

  // global -> registers: four 16-byte chunks of each operand per thread and tile.  Rows past M and columns past N
  // repeat the last valid ones; their products are never stored.
  const float* pa[4];
  const float* pb[4];
  size_t step_a, step_b;                            // floats from one k tile to the next
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (!TA) {                                      // [M][K]: 8 chunks per row of 32 k
      const int arow = tm * BM + (tid >> 3) + 32 * i;
      pa[i] = A + (size_t)(arow < M ? arow : M - 1) * K + (tid & 7) * 4;
    } else {                                        // [K][M]: 32 chunks per row of 128 m
      const int acol = tm * BM + (tid & 31) * 4;
      pa[i] = A + (size_t)((tid >> 5) + 8 * i) * M + (acol < M ? acol : M - 4);
    }
    if (!TB) {                                      // [K][N]: 32 chunks per row of 128 n
      const int bcol = tn * BN + (tid & 31) * 4;
      pb[i] = B + (size_t)((tid >> 5) + 8 * i) * N + (bcol < N ? bcol : N - 4);
    } else {                                        // [N][K]: 8 chunks per row of 32 k
      const int brow = tn * BN + (tid >> 3) + 32 * i;
      pb[i] = B + (size_t)(brow < N ? brow : N - 1) * K + (tid & 7) * 4;
    }
  }
  step_a = TA ? (size_t)BK * M : (size_t)BK;
  step_b = TB ? (size_t)BK : (size_t)BK * N;
  f32x4 ga[4], gb[4];
  auto load_tiles = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ga[i] = *reinterpret_cast<const f32x4*>(pa[i] + (size_t)kt * step_a);
      gb[i] = *reinterpret_cast<const f32x4*>(pb[i] + (size_t)kt * step_b);
    }
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float* da = TA ? As + buf * TILE + ((tid >> 5) + 8 * i) * LDB + (tid & 31) * 4 : As + buf * TILE + ((tid >> 3) + 32 * i) * LD + (tid & 7) * 4;
      float* db = TB ? Bs + buf * TILE_B + ((tid >> 3) + 32 * i) * LD + (tid & 7) * 4 : Bs + buf * TILE_B + ((tid >> 5) + 8 * i) * LDB + (tid & 31) * 4;
      *reinterpret_cast<f32x4*>(da) = ga[i];
      *reinterpret_cast<f32x4*>(db) = gb[i];
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
  // Tile t is multiplied out of LDS buffer t % 2 while tile t + 1 travels global memory -> registers -> the other
  // buffer (past the last tile the last one is loaded and stored again, which nobody reads: no branch splits the
  // tile's scheduling region).  The loop is rotated by one group of 8 k: the last group of a tile is multiplied after
  // the barrier, out of registers, while the first group of the next tile is read - the wait at the barrier and the
  // first LDS reads behind it cost the matrix pipe nothing.  Before the first tile that group is all zeros.
  f32x4 a[2][2], b[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int m = 0; m < 4; ++m) a[1][i][m] = b[1][i][m] = 0.f;
  auto multiply = [&](int s) {
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s][i][m], b[s][j][m], acc[i][j], 0, 0, 0);
  };
  for (int t = 0; t < T; ++t) {
    const int buf = t & 1;
    const float* as = As + buf * TILE;
    const float* bs = Bs + buf * TILE_B;
    auto load_group = [&](int g, int s) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (!TA) a[s][i] = *reinterpret_cast<const f32x4*>(as + (row_a + 32 * i) * LD + g * 8 + k_half);
        else
#pragma unroll
          for (int m = 0; m < 4; ++m) a[s][i][m] = as[(g * 8 + k_half + m) * LDB + row_a + 32 * i];
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if (TB) b[s][j] = *reinterpret_cast<const f32x4*>(bs + (col_b + 32 * j) * LD + g * 8 + k_half);
        else
#pragma unroll
          for (int m = 0; m < 4; ++m) b[s][j][m] = bs[(g * 8 + k_half + m) * LDB + col_b + 32 * j];
      }
    };
    multiply(1);                                    // group 3 of the previous tile
    load_group(0, 0);
    load_tiles(t + 1 < T ? t + 1 : T - 1);
    load_group(1, 1);
    multiply(0);
    load_group(2, 0);
    multiply(1);
    load_group(3, 1);
    store_tiles(buf ^ 1);                           // the other buffer: everybody left it at the last barrier
    multiply(0);
    // Issue order of the tile (one scheduling region): memory instructions are spread between the matrix
    // instructions one at a time, so that neither the LDS queues nor the matrix pipe run dry or full.
    // masks: 0x008 matrix, 0x020 global read, 0x100 LDS read, 0x200 LDS write
    constexpr int NDS = (TA ? 4 : 2) + (TB ? 2 : 4);                         // LDS reads per group: a 16-byte read per tile when k is contiguous, else four 4-byte reads in two instructions
#pragma unroll
    for (int n = 0; n < NDS; ++n) {                                          // previous group 3 multiplies, group 0 is read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int n = 0; n < 8; ++n) {                                            // ... and the next tile is asked for
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    if constexpr (8 - NDS > 0) __builtin_amdgcn_sched_group_barrier(0x008, 8 - NDS, 0);
#pragma unroll
    for (int h = 0; h < 2; ++h) {                                            // groups 0 and 1 multiply, 1 and 2 are read
#pragma unroll
      for (int n = 0; n < NDS; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 16 - NDS, 0);
    }
#pragma unroll
    for (int n = 0; n < NDS; ++n) {                                          // group 2 multiplies, group 3 is read
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#pragma unroll
    for (int n = 0; n < 8; ++n) {                                            // ... and the next tile goes to LDS
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
    }
    if constexpr (8 - NDS > 0) __builtin_amdgcn_sched_group_barrier(0x008, 8 - NDS, 0);
    __syncthreads();
  }
  multiply(1);                                      // group 3 of the last tile

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

namespace {

template <bool TA, bool TB>
int launch_gemm_f32(const float* a, const float* b, float* c, int batch, int M, int N, int K, hipStream_t stream) {
  static bool configured = false;
  if (!configured) {
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_f32_kernel<TA, TB>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes<TA, TB>()));
    configured = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  ART_REQUIRE((long long)tiles_m * tiles_n <= 0x7fffffffLL, "art_gemm_f32: too many tiles");
  gemm_f32_kernel<TA, TB><<<dim3((unsigned)(tiles_m * tiles_n), (unsigned)batch), dim3(kThreads), lds_bytes<TA, TB>(), stream>>>(a, b, c, M, N, K, tiles_n);
  ART_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" int art_gemm_f32_ex(const void* a_dev, const void* b_dev, void* c_dev, int batch, int M, int N, int K, int trans_a,
                               int trans_b, void* stream) {
  ART_REQUIRE(a_dev && b_dev && c_dev, "art_gemm_f32: null pointer");
  ART_REQUIRE(batch > 0 && batch <= 65535, "art_gemm_f32: batch must be 1..65535 (got %d)", batch);
  ART_REQUIRE(M > 0 && N > 0 && K > 0 && K % 32 == 0, "art_gemm_f32: K must be a multiple of 32 (M=%d N=%d K=%d)", M, N, K);
  // an operand whose rows run along m or n is fetched in 16-byte pieces of those rows
  ART_REQUIRE(trans_b || (N % 4 == 0 && N >= 4), "art_gemm_f32: N must be a multiple of 4 when B is stored [K][N] (N=%d)", N);
  ART_REQUIRE(!trans_a || (M % 4 == 0 && M >= 4), "art_gemm_f32: M must be a multiple of 4 when A is stored [K][M] (M=%d)", M);
  ART_REQUIRE(((uintptr_t)a_dev % 16) == 0 && ((uintptr_t)b_dev % 16) == 0 && ((uintptr_t)c_dev % 4) == 0,
              "art_gemm_f32: A and B must be 16-byte aligned");
  const size_t nb = (size_t)batch;
  ART_REQUIRE(!art::overlaps(a_dev, nb * M * K * 4, c_dev, nb * M * N * 4) && !art::overlaps(b_dev, nb * K * N * 4, c_dev, nb * M * N * 4),
              "art_gemm_f32: C must not overlap A or B");
  const float* a = (const float*)a_dev;
  const float* b = (const float*)b_dev;
  float* c = (float*)c_dev;
  hipStream_t st = (hipStream_t)stream;
  if (trans_a) return trans_b ? launch_gemm_f32<true, true>(a, b, c, batch, M, N, K, st) : launch_gemm_f32<true, false>(a, b, c, batch, M, N, K, st);
  return trans_b ? launch_gemm_f32<false, true>(a, b, c, batch, M, N, K, st) : launch_gemm_f32<false, false>(a, b, c, batch, M, N, K, st);
}

extern "C" int art_gemm_f32_batched(const void* a_dev, const void* b_dev, void* c_dev, int batch, int M, int N, int K, void* stream) {
  return art_gemm_f32_ex(a_dev, b_dev, c_dev, batch, M, N, K, 0, 0, stream);
}

extern "C" int art_gemm_f32(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, void* stream) {
  return art_gemm_f32_ex(a_dev, b_dev, c_dev, 1, M, N, K, 0, 0, stream);
}
