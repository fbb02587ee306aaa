// fp16 GEMM on the gfx950 matrix cores:  C[M,N] = A[M,K] @ B[K,N], fp32 accumulate, fp16 out,
// all three row-major.
//
// Replaces the kernel the reference generates for `C[N,M] +=! A[N,K] * B[K,M]`
// (AntaresIR.md:115) with its tiled schedule (backends/c-rocm/schedule/standard/algo_tiling.py:35-98:
// scalar loads through LDS, one FMA per element, no matrix instructions).
//
// Design for MI355X:
//   * block tile 256 x 256 x 64, 256 threads = 2 x 2 wavefronts, each wavefront owns 128 x 128 of C as
//     4 x 4 accumulator tiles of v_mfma_f32_32x32x16_f16 (256 accumulator registers per lane, one
//     wavefront per SIMD); 16 MFMAs (512 matrix-core cycles) per 8 KiB of LDS reads;
//   * A tile in LDS as [m][k] (k contiguous, rows padded by 16 bytes): one ds_read_b128 gives a lane
//     its 8 consecutive k of one row;
//   * B tile in LDS exactly as it lies in memory, [k][n] (n contiguous, rows padded by 32 bytes); the
//     MFMA wants 8 consecutive k per lane for ONE column, which is the transpose: ds_read_b64_tr_b16
//     (new in gfx950) reads a 4(k) x 16(n) patch with 16 lanes and hands lane L the four k of column L.
//     Two such reads make one B operand; the 32-byte row padding spreads the four k rows over all banks;
//   * global -> registers -> LDS, double buffered: the loads of tile t+1 are issued before the MFMAs of
//     tile t and stored to the other LDS buffer after them; one barrier per 64 k;
//   * block -> tile mapping is XCD aware: the 32 blocks that run on one XCD at a time cover a 4 x 8
//     super-tile, so they share 4 A panels and 8 B panels through that XCD's L2;
//   * C goes through LDS once more so that it leaves as 128-bit row-contiguous stores.
#include "art_common.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int A_LD = BK + 8;             // halves per A row in LDS (144 bytes)
constexpr int B_LD = BN + 16;            // halves per B row in LDS (544 bytes)
constexpr int A_TILE = BM * A_LD;        // halves
constexpr int B_TILE = BK * B_LD;
constexpr int C_LD = BN + 8;             // halves per C row while staging the output
constexpr size_t kLdsBytes = (size_t)(2 * A_TILE + 2 * B_TILE) * 2;
static_assert((size_t)BM * C_LD * 2 <= kLdsBytes, "output staging must fit in the operand buffers");

__device__ __forceinline__ int xcd_tile(int b, int nb) {
  const int q = nb >> 3, r = nb & 7, xcd = b & 7, idx = b >> 3;
  return xcd < r ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
}

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

__global__ __launch_bounds__(256) void gemm_f16_kernel(const _Float16* __restrict__ A, const _Float16* __restrict__ B,
                                                        _Float16* __restrict__ C, int M, int N, int K) {
  extern __shared__ __align__(16) _Float16 smem[];
  _Float16* As = smem;                    // [2][BM][A_LD]
  _Float16* Bs = smem + 2 * A_TILE;       // [2][BK][B_LD]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int MT = M / BM, NT = N / BN;
  int tile = xcd_tile(blockIdx.x, gridDim.x), tm, tn;
  if ((MT % 4 == 0) && (NT % 8 == 0)) {   // 4 x 8 super-tiles, row-major inside and outside
    const int super = tile >> 5, in = tile & 31, sn_count = NT >> 3;
    tm = (super / sn_count) * 4 + (in >> 3);
    tn = (super % sn_count) * 8 + (in & 7);
  } else {
    tm = tile / NT;
    tn = tile % NT;
  }
  const _Float16* Ag = A + (size_t)tm * BM * K;
  const _Float16* Bg = B + (size_t)tn * BN;

  // global -> register staging: 8 chunks of 16 bytes per thread for each operand
  u32x4 ga[8], gb[8];
  auto load_tiles = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = tid + 256 * i;
      ga[i] = *reinterpret_cast<const u32x4*>(Ag + (size_t)(c >> 3) * K + (size_t)kt * BK + (c & 7) * 8);
      gb[i] = *reinterpret_cast<const u32x4*>(Bg + ((size_t)kt * BK + (c >> 5)) * N + (c & 31) * 8);
    }
  };
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = tid + 256 * i;
      *reinterpret_cast<u32x4*>(As + buf * A_TILE + (c >> 3) * A_LD + (c & 7) * 8) = ga[i];
      *reinterpret_cast<u32x4*>(Bs + buf * B_TILE + (c >> 5) * B_LD + (c & 31) * 8) = gb[i];
    }
  };

  f16v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // per-lane constants of the operand reads
  const int a_row = wm * 128 + (lane & 31);                 // + i*32
  const int a_k = (lane >> 5) * 8;                          // + kk*16
  const int s = lane & 15;
  const int b_k = (lane >> 5) * 8 + (s >> 2);               // + kk*16 + r*4
  const int b_n = wn * 128 + ((lane & 31) >> 4) * 16 + (s & 3) * 4;   // + j*32

  auto load_frags = [&](h8 (&af)[4], h8 (&bf)[4], const _Float16* as, const _Float16* bs, int kk) {
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const h8*>(as + (a_row + i * 32) * A_LD + kk * 16 + a_k);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const _Float16* p = bs + (kk * 16 + b_k) * B_LD + b_n + j * 32;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * B_LD));
      const h4 l4 = __builtin_bit_cast(h4, lo), h4v = __builtin_bit_cast(h4, hi);
      bf[j] = h8{l4[0], l4[1], l4[2], l4[3], h4v[0], h4v[1], h4v[2], h4v[3]};
    }
  };
  auto mfma_all = [&](const h8 (&af)[4], const h8 (&bf)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
  };

  const int T = K / BK;
  load_tiles(0);
  store_tiles(0);
  __syncthreads();
  h8 af0[4], bf0[4], af1[4], bf1[4];
  for (int t = 0; t < T; ++t) {
    const int buf = t & 1;
    const _Float16* as = As + buf * A_TILE;
    const _Float16* bs = Bs + buf * B_TILE;
    // The scheduler is told not to move anything across these fences: without them it sinks every
    // operand read next to its first use and the matrix cores wait for LDS sixteen times per tile.
#define ART_FENCE() __builtin_amdgcn_sched_barrier(0)
    load_frags(af0, bf0, as, bs, 0);
    ART_FENCE();
    if (t + 1 < T) load_tiles(t + 1);
    ART_FENCE();
    load_frags(af1, bf1, as, bs, 1);     // operands of k-step kk+1 are requested before the MFMAs of k-step kk
    ART_FENCE();
    mfma_all(af0, bf0);
    ART_FENCE();
    load_frags(af0, bf0, as, bs, 2);
    ART_FENCE();
    mfma_all(af1, bf1);
    ART_FENCE();
    load_frags(af1, bf1, as, bs, 3);
    ART_FENCE();
    mfma_all(af0, bf0);
    ART_FENCE();
    mfma_all(af1, bf1);
    ART_FENCE();
#undef ART_FENCE
    if (t + 1 < T) store_tiles(buf ^ 1);
    __syncthreads();
  }

  // ---- output: registers -> LDS (fp16, [256][C_LD]) -> 128-bit stores
  _Float16* cs = smem;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = wm * 128 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        const int col = wn * 128 + j * 32 + (lane & 31);
        cs[row * C_LD + col] = (_Float16)acc[i][j][r];
      }
  __syncthreads();
  _Float16* Cg = C + (size_t)tm * BM * N + (size_t)tn * BN;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int c = tid + 256 * i;               // 256 rows x 32 chunks of 8 halves
    const int row = c >> 5, ch = c & 31;
    *reinterpret_cast<u32x4*>(Cg + (size_t)row * N + ch * 8) = *reinterpret_cast<const u32x4*>(cs + row * C_LD + ch * 8);
  }
}

}  // namespace

extern "C" int art_gemm_f16(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, void* stream) {
  ART_REQUIRE(a_dev && b_dev && c_dev, "art_gemm_f16: null pointer");
  ART_REQUIRE(M > 0 && N > 0 && K > 0 && M % BM == 0 && N % BN == 0 && K % BK == 0,
              "art_gemm_f16: M and N must be multiples of 256 and K of 64 (M=%d N=%d K=%d)", M, N, K);
  ART_REQUIRE(((uintptr_t)a_dev % 16) == 0 && ((uintptr_t)b_dev % 16) == 0 && ((uintptr_t)c_dev % 16) == 0,
              "art_gemm_f16: operands must be 16-byte aligned");
  static bool configured = false;
  if (!configured) {
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_f16_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kLdsBytes));
    configured = true;
  }
  const int blocks = (M / BM) * (N / BN);
  gemm_f16_kernel<<<dim3(blocks), dim3(256), kLdsBytes, (hipStream_t)stream>>>((const _Float16*)a_dev, (const _Float16*)b_dev,
                                                                                (_Float16*)c_dev, M, N, K);
  ART_LAUNCH_CHECK();
  return 0;
}
