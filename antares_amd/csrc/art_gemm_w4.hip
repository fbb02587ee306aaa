// Weight-only int4 GEMM for a batch of rows (prefill, M > 8): the same arithmetic as the GEMV of
// art_gemv_w4.hip,
//     y[m,n] = sum_g s[g,n] * sum_{k in group g} x[m,k] * (q[k,n] - z[g,n]),      group = 128 k,
// with the inner sums on the matrix cores.  Replaces the kernel the reference generates when the
// dequant + matmul program of samples/05_llama2_7b_int4.py:135-144 is exported with a batch axis.
//
// Design for MI355X:
//   * the weights are read from HBM exactly once; a work item owns 128 columns (one full 128-byte line
//     of every packed row) and a contiguous range of k groups, and streams them two groups ahead;
//   * unpacking is fused into the LDS staging: 16 bytes (16 columns x 2 k) become two rows of fp16
//     (q - z) values - exact small integers - with one shift, four and-or and four packed subtractions
//     per word.  The columns of every group of four land in LDS in the order 0,2,1,3, which costs nothing:
//     the column an accumulator lane owns is permuted the same way and undone in the epilogue;
//   * v_mfma_f32_32x32x16_f16 per wave: 32 columns x 64 rows, B operand through ds_read_b64_tr_b16;
//     the group sum is scaled by s[g,n] in fp32 afterwards (one scalar per lane, since an accumulator
//     lane owns one column), so no scale is rounded to fp16;
//   * a block is two independent work items of four waves each that alternate phases: while one half
//     unpacks its next group on the vector units, the other half multiplies its current group on the
//     matrix cores.  One wave of each half sits on every SIMD, so both pipes stay busy;
//   * split-K without atomics (5.6 M float atomics cost 75 us on this chip): each K-split writes its
//     fp32 tile to the library workspace and a second small kernel adds the splits in a fixed order
//     and rounds once to fp16 - results do not depend on timing.
#include "art_common.h"

#include <type_traits>

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int BM = 64, BN = 128, GK = 128;     // rows, columns and k per staged tile
constexpr int W_LD = BN + 32;                  // halves per weight row in LDS: 320 bytes, so the four k rows
                                               // a transposing read touches fall on disjoint banks
constexpr int X_LD = GK + 8;                   // halves per x row in LDS (272 bytes)
constexpr int HALF_LDS = GK * W_LD + BM * X_LD;                 // halves of LDS per work item
constexpr size_t kLdsBytes = (size_t)2 * HALF_LDS * sizeof(_Float16);

struct Magic {
  unsigned int mask_lo, mask_hi, bias_lo, bias_hi;   // 0x000F000F 0x00F000F0 0x64006400 0x54005400
};

__device__ __forceinline__ h2 as_h2(unsigned int v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ unsigned int as_u32(h2 v) { return __builtin_bit_cast(unsigned int, v); }

// (w & mask) | bias in one v_bitop3_b32 (truth table 0xEA = (a & b) | c).
__device__ __forceinline__ unsigned int and_or(unsigned int w, unsigned int mask, unsigned int bias) {
  return __builtin_amdgcn_bitop3_b32(w, mask, bias, 0xEA);
}

// Position p of a staged column <-> column of the matrix: bits 0 and 1 swapped.
__device__ __forceinline__ int unpermute(int p) { return (p & ~3) | ((p & 1) << 1) | ((p >> 1) & 1); }

template <int MT>   // MT accumulator tiles of 32 rows: 1 for M <= 32, 2 for M <= 64
__global__ __launch_bounds__(512) void gemm_w4a16_kernel(const _Float16* __restrict__ x, const unsigned char* __restrict__ qweight,
                                                          const _Float16* __restrict__ scales,
                                                          const unsigned char* __restrict__ qzeros, _Float16* __restrict__ y,
                                                          float* __restrict__ partial, int M, int K, int N, int splits,
                                                          int col_tiles, Magic mg) {
  extern __shared__ __align__(16) _Float16 smem[];
  const int half = threadIdx.x >> 8;             // which of the block's two work items this wave serves
  const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
  _Float16* Ws = smem + half * HALF_LDS;         // [GK][W_LD]
  _Float16* Xs = Ws + GK * W_LD;                 // [BM][X_LD]

  // work item -> (column tile, K split); the two halves of a block take neighbouring column tiles
  const int G = K / GK, items = col_tiles * splits;
  auto group_range = [&](int item, int& begin, int& end) {
    const int split = item / col_tiles;
    begin = item < items ? (int)((long long)G * split / splits) : 0;
    end = item < items ? (int)((long long)G * (split + 1) / splits) : 0;
  };
  const int item = blockIdx.x * 2 + half;
  int g_begin, g_end, o_begin, o_end;
  group_range(item, g_begin, g_end);
  group_range(blockIdx.x * 2 + (1 - half), o_begin, o_end);
  const int steps = g_end - g_begin;
  const int T = steps > o_end - o_begin ? steps : o_end - o_begin;      // both halves pass the same barriers
  const int split = item / col_tiles;
  const int n0 = (item % col_tiles) * BN;

  // ---- global -> register staging
  // weights: 64 packed rows x 128 bytes per group = 512 chunks of 16 bytes, two per thread
  const int cc = tid & 7;                       // 16-column chunk
  const int pr = tid >> 3;                      // packed row (+32 for the second chunk)
  const bool col_ok = n0 + cc * 16 < N;         // N % 16 == 0: a chunk is inside or outside as a whole
  const int wcol = col_ok ? n0 + cc * 16 : 0;
  const unsigned char* wp = qweight + (size_t)pr * N + wcol;
  // x: MT*32 rows x 128 k = MT*512 chunks of 16 bytes, 2*MT per thread; rows past M repeat row M-1
  const _Float16* xp[2 * MT];
  int xs_off[2 * MT];
#pragma unroll
  for (int i = 0; i < 2 * MT; ++i) {
    const int c = tid + 256 * i, row = c >> 4, kc = c & 15;
    xp[i] = x + (size_t)(row < M ? row : M - 1) * K + kc * 8;
    xs_off[i] = row * X_LD + kc * 8;
  }

  // per-lane constants of the operand reads
  const int a_row = lane & 31, a_k = (lane >> 5) * 8;
  const int s16 = lane & 15;
  const int b_k = (lane >> 5) * 8 + (s16 >> 2);
  const int b_n = wave * 32 + ((lane & 31) >> 4) * 16 + (s16 & 3) * 4;
  const int my_col = n0 + unpermute(wave * 32 + (lane & 31));       // the column this lane accumulates
  const bool my_ok = my_col < N;
  const int sc_col = my_ok ? my_col : 0;

  // Two register stages: the loads of group g + 2 are issued while group g is unpacked.
  // Stages are indexed statically (a run-time index would put the arrays in scratch memory).
  u32x4 wq[2][2];      // [stage][chunk]
  u32x4 xr[2][2 * MT];
  u32x2 zq[2];
  _Float16 sc16[2];
  auto load_stage = [&](int g, auto tag) {
    constexpr int S = decltype(tag)::value;
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) xr[S][i] = *reinterpret_cast<const u32x4*>(xp[i] + (size_t)g * GK);
    const unsigned char* p = wp + (size_t)g * (GK / 2) * N;
    wq[S][0] = *reinterpret_cast<const u32x4*>(p);
    wq[S][1] = *reinterpret_cast<const u32x4*>(p + (size_t)32 * N);
    zq[S] = *reinterpret_cast<const u32x2*>(qzeros + (size_t)g * (N / 2) + (wcol >> 1));
    sc16[S] = scales[(size_t)g * N + sc_col];
  };

  f16v total[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) total[i][r] = 0.f;
  float sc_staged = 0.f;     // scale of the group that currently sits in LDS

  // Phase D: unpack step i of this work item into LDS and refill its register stage.
  auto unpack = [&](int i, auto tag) {
    constexpr int S = decltype(tag)::value;
    if (i >= steps) return;
    sc_staged = my_ok ? (float)sc16[S] : 0.f;
    // zero points of this thread's 16 columns, paired (c0,c2) and (c1,c3), on both nibble biases
    h2 z_lo[8], z_hi[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned int zw = (zq[S][j >> 1] >> ((j & 1) * 16)) & 0xffffu;   // z0 | z1<<4 | z2<<8 | z3<<12
      const unsigned int e = zw | (zw << 8);              // z0 at bits 0-3, z2 at bits 16-19
      const unsigned int o = (zw >> 4) | (zw << 4);       // z1 at bits 0-3, z3 at bits 16-19
      z_lo[2 * j] = as_h2(and_or(e, mg.mask_lo, mg.bias_lo));
      z_lo[2 * j + 1] = as_h2(and_or(o, mg.mask_lo, mg.bias_lo));
      z_hi[2 * j] = as_h2(and_or(e << 4, mg.mask_hi, mg.bias_hi));
      z_hi[2 * j + 1] = as_h2(and_or(o << 4, mg.mask_hi, mg.bias_hi));
    }
    // chunk c holds packed row pr + 32c = k rows 2*(pr+32c) and 2*(pr+32c)+1
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      u32x4 even[2], odd[2];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const unsigned int w = wq[S][c][j], w8 = w >> 8;    // columns past N hold finite garbage and are never stored
        const h2 e02 = as_h2(and_or(w, mg.mask_lo, mg.bias_lo)) - z_lo[2 * j];
        const h2 e13 = as_h2(and_or(w8, mg.mask_lo, mg.bias_lo)) - z_lo[2 * j + 1];
        const h2 o02 = as_h2(and_or(w, mg.mask_hi, mg.bias_hi)) - z_hi[2 * j];
        const h2 o13 = as_h2(and_or(w8, mg.mask_hi, mg.bias_hi)) - z_hi[2 * j + 1];
        even[j >> 1][(j & 1) * 2] = as_u32(e02);
        even[j >> 1][(j & 1) * 2 + 1] = as_u32(e13);
        odd[j >> 1][(j & 1) * 2] = as_u32(o02);
        odd[j >> 1][(j & 1) * 2 + 1] = as_u32(o13);
      }
      _Float16* row = Ws + (2 * (pr + 32 * c)) * W_LD + cc * 16;
      *reinterpret_cast<u32x4*>(row) = even[0];
      *reinterpret_cast<u32x4*>(row + 8) = even[1];
      *reinterpret_cast<u32x4*>(row + W_LD) = odd[0];
      *reinterpret_cast<u32x4*>(row + W_LD + 8) = odd[1];
    }
#pragma unroll
    for (int j = 0; j < 2 * MT; ++j) *reinterpret_cast<u32x4*>(Xs + xs_off[j]) = xr[S][j];
    if (i + 2 < steps) load_stage(g_begin + i + 2, tag);     // refill the stage just consumed
  };

  // Phase M: multiply the group that sits in LDS (step i) and add it, scaled, to the totals.
  auto multiply = [&](int i) {
    if (i < 0 || i >= steps) return;
    f16v grp[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) grp[t][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < GK / 16; ++kk) {
      const _Float16* p = Ws + (kk * 16 + b_k) * W_LD + b_n;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * W_LD));
      const h4 l4 = __builtin_bit_cast(h4, lo), h4v = __builtin_bit_cast(h4, hi);
      const h8 bf = h8{l4[0], l4[1], l4[2], l4[3], h4v[0], h4v[1], h4v[2], h4v[3]};
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const h8 af = *reinterpret_cast<const h8*>(Xs + (a_row + t * 32) * X_LD + kk * 16 + a_k);
        grp[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, grp[t], 0, 0, 0);
      }
    }
    const float sc = sc_staged;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) total[t][r] += grp[t][r] * sc;
  };

  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  if (steps > 0) load_stage(g_begin, S0{});
  if (steps > 1) load_stage(g_begin + 1, S1{});
  // Time slots, one barrier after each:   half 0:  D(0) M(0) D(1) M(1) ...
  //                                        half 1:   -   D(0) M(0) D(1) ...  M(T-1)
  auto iteration = [&](int i, auto tag) {
    if (half == 0) unpack(i, tag);
    else multiply(i - 1);
    art_lds_barrier();
    if (half == 0) multiply(i);
    else unpack(i, tag);
    art_lds_barrier();
  };
  for (int i = 0; i < T; i += 2) {
    iteration(i, S0{});
    if (i + 1 < T) iteration(i + 1, S1{});
  }
  if (half == 1) multiply(T - 1);

  // ---- epilogue: accumulator element r of tile t is row t*32 + (r/4)*8 + (lane/32)*4 + r%4, column my_col
  if (!my_ok || steps == 0) return;
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
      if (row < M) {
        if (splits == 1) y[(size_t)row * N + my_col] = (_Float16)total[t][r];
        else partial[((size_t)split * M + row) * N + my_col] = total[t][r];
      }
    }
}

// y[m,n] = fp16(sum over splits, in split order); four columns per thread (N % 4 == 0).
__global__ __launch_bounds__(256) void gemm_w4a16_combine_kernel(const float* __restrict__ partial, _Float16* __restrict__ y,
                                                                  long long count4, long long split_stride, int splits) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= count4) return;
  f32x4 t = *reinterpret_cast<const f32x4*>(partial + i * 4);
  for (int s = 1; s < splits; ++s) t += *reinterpret_cast<const f32x4*>(partial + s * split_stride + i * 4);
  const h4 out = h4{(_Float16)t[0], (_Float16)t[1], (_Float16)t[2], (_Float16)t[3]};
  *reinterpret_cast<h4*>(y + i * 4) = out;
}

// Number of K-splits: as many work items as fit the chip in one round (two per compute unit), but at
// least four groups per item, and no more than the scratch space for the partial tiles allows.
// Measured on MI355X at M = 64: N=4096 K=4096 -> 8, N=11008 -> 5, N=4096 K=11008 -> 16, N=32000 -> 2.
int choose_splits(int rows, int N, int G, size_t scratch_bytes, int compute_units) {
  const int col_tiles = (N + BN - 1) / BN;
  int s = 2 * compute_units / col_tiles;
  if (s > G / 4) s = G / 4;
  const size_t per_split = (size_t)rows * N * sizeof(float);
  const int cap = (int)(scratch_bytes / per_split);
  if (s > cap) s = cap;
  return s < 1 ? 1 : s;
}

}  // namespace

extern "C" int art_gemm_w4a16(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                              void* y_dev, int M, int K, int N, void* stream) {
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemm_w4a16: null pointer");
  ART_REQUIRE(M >= 1, "art_gemm_w4a16: M must be positive (got %d)", M);
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemm_w4a16: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 16) == 0 && ((uintptr_t)qzeros_dev % 8) == 0 &&
                  ((uintptr_t)y_dev % 8) == 0,
              "art_gemm_w4a16: x and qweight must be 16-byte aligned, qzeros and y 8-byte aligned");
  art::Workspace& ws = art::workspace();
  ART_REQUIRE(ws.base != nullptr, "art_gemm_w4a16: art_init has not been called on this device");
  float* scratch = reinterpret_cast<float*>((char*)ws.base + art::kScratchOffset);
  const size_t scratch_bytes = ws.bytes - art::kScratchOffset;
  static int compute_units = 0;
  if (compute_units == 0) {
    int dev = 0;
    ART_HIP(hipGetDevice(&dev));
    ART_HIP(hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, dev));
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_w4a16_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kLdsBytes));
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_w4a16_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)kLdsBytes));
  }
  const Magic mg{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  hipStream_t st = (hipStream_t)stream;
  const int G = K / GK, col_tiles = (N + BN - 1) / BN;
  for (int m0 = 0; m0 < M; m0 += BM) {      // 64 rows of x per pass over the weights
    const int rows = M - m0 < BM ? M - m0 : BM;
    const int splits = choose_splits(rows, N, G, scratch_bytes, compute_units);
    const _Float16* xs = (const _Float16*)x_dev + (size_t)m0 * K;
    _Float16* ys = (_Float16*)y_dev + (size_t)m0 * N;
    const dim3 grid((col_tiles * splits + 1) / 2);
    if (rows <= 32)
      gemm_w4a16_kernel<1><<<grid, 512, kLdsBytes, st>>>(xs, (const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                         (const unsigned char*)qzeros_dev, ys, scratch, rows, K, N, splits,
                                                         col_tiles, mg);
    else
      gemm_w4a16_kernel<2><<<grid, 512, kLdsBytes, st>>>(xs, (const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                         (const unsigned char*)qzeros_dev, ys, scratch, rows, K, N, splits,
                                                         col_tiles, mg);
    ART_LAUNCH_CHECK();
    if (splits > 1) {
      const long long count4 = (long long)rows * N / 4;
      gemm_w4a16_combine_kernel<<<dim3((unsigned)((count4 + 255) / 256)), 256, 0, st>>>(scratch, ys, count4, (long long)rows * N,
                                                                                        splits);
      ART_LAUNCH_CHECK();
    }
  }
  return 0;
}
