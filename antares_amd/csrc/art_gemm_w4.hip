// Weight-only int4 GEMM for a batch of rows (prefill, 9 <= M): the same arithmetic as the GEMV of
// art_gemv_w4.hip,
//     y[m,n] = sum_g s[g,n] * sum_{k in group g} x[m,k] * (q[k,n] - z[g,n]),      group = 128 k,
// with the inner sums on the matrix cores.  Replaces the kernel the reference generates when the
// dequant + matmul program of samples/05_llama2_7b_int4.py:135-144 is exported with a batch axis.
//
// Design for MI355X:
//   * the weights are read from HBM exactly once; a block owns 128 columns (one full 128-byte line of
//     every packed row) and a contiguous range of k groups, and streams them two groups ahead;
//   * unpacking is fused into the LDS staging: 16 bytes (16 columns x 2 k) become two rows of fp16
//     (q - z) values - exact small integers - with one shift, four and-or and four packed subtractions
//     per word.  The columns of every group of four land in LDS in the order 0,2,1,3, which costs nothing:
//     the column an accumulator lane owns is permuted the same way and undone in the epilogue;
//   * v_mfma_f32_32x32x16_f16 per wave: 32 columns x 64 rows, B operand through ds_read_b64_tr_b16;
//     the group sum is scaled by s[g,n] in fp32 afterwards (one scalar per lane, since an accumulator
//     lane owns one column), so no scale is rounded to fp16;
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
constexpr int W_LD = BN + 16;                  // halves per weight row in LDS (288 bytes)
constexpr int X_LD = GK + 8;                   // halves per x row in LDS (272 bytes)

struct Magic {
  unsigned int mask_lo, mask_hi, bias_lo, bias_hi;   // 0x000F000F 0x00F000F0 0x64006400 0x54005400
};

__device__ __forceinline__ h2 as_h2(unsigned int v) { return __builtin_bit_cast(h2, v); }
__device__ __forceinline__ unsigned int as_u32(h2 v) { return __builtin_bit_cast(unsigned int, v); }

// (w & mask) | bias for disjoint mask and bias.
__device__ __forceinline__ unsigned int and_or(unsigned int w, unsigned int mask, unsigned int bias) {
  return (w & mask) | (~mask & bias);
}

// Position p of a staged column <-> column of the matrix: bits 0 and 1 swapped.
__device__ __forceinline__ int unpermute(int p) { return (p & ~3) | ((p & 1) << 1) | ((p >> 1) & 1); }

template <int MT>   // MT accumulator tiles of 32 rows: 1 for M <= 32, 2 for M <= 64
__global__ __launch_bounds__(256) void gemm_w4a16_kernel(const _Float16* __restrict__ x, const unsigned char* __restrict__ qweight,
                                                          const _Float16* __restrict__ scales,
                                                          const unsigned char* __restrict__ qzeros, _Float16* __restrict__ y,
                                                          float* __restrict__ partial, int M, int K, int N, int splits,
                                                          Magic mg) {
  __shared__ __align__(16) _Float16 Ws[GK * W_LD];
  __shared__ __align__(16) _Float16 Xs[MT * 32 * X_LD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * BN;
  const int G = K / GK;
  const int g_begin = (int)((long long)G * blockIdx.y / splits), g_end = (int)((long long)G * (blockIdx.y + 1) / splits);

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

  // Two register stages: the loads of group g + 2 are issued while group g is unpacked and multiplied.
  // Stages are indexed statically (a run-time index would put the arrays in scratch memory).
  u32x4 wq[2][2];      // [stage][chunk]
  u32x4 xr[2][2 * MT];
  u32x2 zq[2];
  _Float16 sc16[2];
  const int sc_col = my_ok ? my_col : 0;
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

  f16v total[MT], grp[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) total[i][r] = 0.f;

  auto step = [&](int g, auto tag) {
    constexpr int S = decltype(tag)::value;
    // zero points of this thread's 16 columns, paired (c0,c2) and (c1,c3), on both nibble biases
    const float sc = my_ok ? (float)sc16[S] : 0.f;
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
    // unpack: chunk c holds packed row pr + 32c = k rows 2*(pr+32c) and 2*(pr+32c)+1
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      u32x4 even[2], odd[2];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const unsigned int w = col_ok ? wq[S][c][j] : 0u, w8 = w >> 8;
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
    for (int i = 0; i < 2 * MT; ++i) *reinterpret_cast<u32x4*>(Xs + xs_off[i]) = xr[S][i];
    if (g + 2 < g_end) load_stage(g + 2, tag);     // refill the stage just consumed
    __syncthreads();

#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) grp[i][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < GK / 16; ++kk) {
      const _Float16* p = Ws + (kk * 16 + b_k) * W_LD + b_n;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * W_LD));
      const h4 l4 = __builtin_bit_cast(h4, lo), h4v = __builtin_bit_cast(h4, hi);
      const h8 bf = h8{l4[0], l4[1], l4[2], l4[3], h4v[0], h4v[1], h4v[2], h4v[3]};
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const h8 af = *reinterpret_cast<const h8*>(Xs + (a_row + i * 32) * X_LD + kk * 16 + a_k);
        grp[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, grp[i], 0, 0, 0);
      }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) total[i][r] += grp[i][r] * sc;
    __syncthreads();
  };

  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  if (g_begin < g_end) load_stage(g_begin, S0{});
  if (g_begin + 1 < g_end) load_stage(g_begin + 1, S1{});
  for (int g = g_begin; g < g_end; g += 2) {
    step(g, S0{});
    if (g + 1 < g_end) step(g + 1, S1{});
  }

  // ---- epilogue: accumulator element r of tile i is row i*32 + (r/4)*8 + (lane/32)*4 + r%4, column my_col
  if (!my_ok) return;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
      if (row < M) {
        if (splits == 1) y[(size_t)row * N + my_col] = (_Float16)total[i][r];
        else partial[((size_t)blockIdx.y * M + row) * N + my_col] = total[i][r];
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

// Number of K-splits: enough blocks to occupy every compute unit about twice, bounded by the
// number of groups and by the scratch space the partial tiles need.
int choose_splits(int rows, int N, int G, size_t scratch_bytes) {
  const int col_tiles = (N + BN - 1) / BN;
  int s = (512 + col_tiles - 1) / col_tiles;
  const size_t per_split = (size_t)rows * N * sizeof(float);
  const int cap = (int)(scratch_bytes / per_split);
  if (s > cap) s = cap;
  if (s > G) s = G;
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
  const Magic mg{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  hipStream_t st = (hipStream_t)stream;
  const int G = K / GK;
  for (int m0 = 0; m0 < M; m0 += BM) {      // 64 rows of x per pass over the weights
    const int rows = M - m0 < BM ? M - m0 : BM;
    const int splits = choose_splits(rows, N, G, scratch_bytes);
    const _Float16* xs = (const _Float16*)x_dev + (size_t)m0 * K;
    _Float16* ys = (_Float16*)y_dev + (size_t)m0 * N;
    const dim3 grid((N + BN - 1) / BN, splits);
    if (rows <= 32)
      gemm_w4a16_kernel<1><<<grid, 256, 0, st>>>(xs, (const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                 (const unsigned char*)qzeros_dev, ys, scratch, rows, K, N, splits, mg);
    else
      gemm_w4a16_kernel<2><<<grid, 256, 0, st>>>(xs, (const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                 (const unsigned char*)qzeros_dev, ys, scratch, rows, K, N, splits, mg);
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
