// Weight-only int4 GEMM for a batch of rows (prefill, four rows and more): the same arithmetic as the GEMV of
// art_gemv_w4.hip,
//     y[m,n] = sum_g s[g,n] * sum_{k in group g} x[m,k] * (q[k,n] - z[g,n]),      group = 128 k,
// with the inner sums on the matrix cores.  Replaces the kernel the reference generates when the
// dequant + matmul program of samples/05_llama2_7b_int4.py:135-144 is exported with a batch axis.
//
// Design for MI355X:
//   * the weights are read from HBM exactly once; a block of eight waves owns 256 columns (two full
//     128-byte lines of every packed row, and as many bytes of weights as of x per step) and a contiguous
//     range of k groups;
//   * unpacking is fused into the LDS staging: 16 bytes (16 columns x 2 k) become two rows of fp16
//     (q - z) values - exact small integers - with one shift, four v_bitop3_b32 and four packed
//     subtractions per word.  The columns of every group of four land in LDS in the order 0,2,1,3,
//     which costs nothing: the column an accumulator lane owns is permuted the same way and undone
//     in the epilogue;
//   * v_mfma_f32_32x32x16_f16 per wave: 32 columns x 64 rows, B operand through ds_read_b64_tr_b16;
//     the group sum is scaled by s[g,n] in fp32 afterwards (one scalar per lane, since an accumulator
//     lane owns one column), so no scale is rounded to fp16;
//   * a step is 64 k.  LDS holds two steps: while the matrix cores work on step t, the same waves
//     unpack step t+1 into the other buffer; one barrier per step, and it waits for LDS only, so the
//     register stages (a whole group = two steps each, two of them) keep their global loads in flight
//     across it.  92 KiB of LDS and < 256 registers: one block = two waves per SIMD on every compute unit;
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

constexpr int kThreads = 512;                  // 8 waves: 32 columns each
constexpr int BM = 64, BN = kThreads / 2, GK = 128;   // rows and columns of a block, k of a quantisation group
constexpr int SK = 64;                         // k of a step (half a group)
constexpr int W_LD = BN + 32;                  // halves per weight row in LDS: 320 bytes, so the four k rows
                                               // a transposing read touches fall on disjoint banks
constexpr int X_LD = SK + 8;                   // halves per x row in LDS (144 bytes)
constexpr int W_TILE = SK * W_LD, X_TILE = BM * X_LD;
constexpr size_t kLdsBytes = (size_t)2 * (W_TILE + X_TILE) * sizeof(_Float16);

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
__global__ __launch_bounds__(kThreads, 512 / kThreads) void gemm_w4a16_kernel(const _Float16* __restrict__ x, const unsigned char* __restrict__ qweight,
                                                             const _Float16* __restrict__ scales,
                                                             const unsigned char* __restrict__ qzeros, _Float16* __restrict__ y,
                                                             float* __restrict__ partial, int M_total, int K, int N, int splits,
                                                             int col_tiles, int m_blocks, Magic mg,
                                                             const _Float16* __restrict__ residual) {
  extern __shared__ __align__(16) _Float16 smem[];
  _Float16* Ws = smem;                           // [2][SK][W_LD]
  _Float16* Xs = smem + 2 * W_TILE;              // [2][BM][X_LD]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // block -> (column tile, K split, block of 64 rows).  The row blocks of one (tile, split) stream the same weights:
  // they get block ids that are 8 apart, which the dispatcher places on the same XCD at the same time, so that the
  // weights come from HBM once and from that XCD's L2 for the others.
  const int G = K / GK;
  const int unit = (int)(blockIdx.x / (8 * m_blocks)) * 8 + (int)(blockIdx.x % 8);      // (tile, split) pair
  const int m_block = (int)(blockIdx.x % (8 * m_blocks)) / 8;
  if (unit >= col_tiles * splits) return;
  const int split = unit / col_tiles;
  const int n0 = (unit % col_tiles) * BN;
  const int m0 = m_block * BM;
  const int M = M_total - m0 < BM ? M_total - m0 : BM;          // rows of this block
  x += (size_t)m0 * K;
  y += (size_t)m0 * N;
  if (residual) residual += (size_t)m0 * N;
  const int g_begin = (int)((long long)G * split / splits), g_end = (int)((long long)G * (split + 1) / splits);
  const int groups = g_end - g_begin;

  // ---- global -> register staging, one quantisation group (two steps) per stage
  // weights of a step: 32 packed rows x BN bytes = kThreads chunks of 16 bytes, one per thread
  constexpr int kChunks = BN / 16;              // 16-column chunks per packed row
  const int cc = tid % kChunks;                 // 16-column chunk
  const int pr = tid / kChunks;                 // packed row of the step (kThreads / kChunks = 32 of them)
  const bool col_ok = n0 + cc * 16 < N;         // N % 16 == 0: a chunk is inside or outside as a whole
  const int wcol = col_ok ? n0 + cc * 16 : 0;   // columns past N: load valid memory, results are never stored
  const unsigned char* wp = qweight + (size_t)pr * N + wcol;
  // x of a step: MT*32 rows x 64 k = MT*256 chunks of 16 bytes, XC per thread; rows past M repeat row M-1
  constexpr int XC = (MT * 256 + kThreads - 1) / kThreads;     // chunks of x per thread and step
  const _Float16* xp[XC];
  int xs_off[XC];
#pragma unroll
  for (int i = 0; i < XC; ++i) {
    const int c = tid + kThreads * i, row = c >> 3, kc = c & 7;
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

  // Stages are indexed statically (a run-time index would put the arrays in scratch memory).
  u32x4 wq[2][2];      // [stage][step of the group]
  u32x4 xr[2][2][XC];
  u32x2 zq[2];
  _Float16 sc16[2];
  auto load_group = [&](int g, auto tag) {
    constexpr int S = decltype(tag)::value;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < XC; ++i) xr[S][h][i] = *reinterpret_cast<const u32x4*>(xp[i] + (size_t)g * GK + h * SK);
      wq[S][h] = *reinterpret_cast<const u32x4*>(wp + ((size_t)g * (GK / 2) + h * (SK / 2)) * N);
    }
    zq[S] = *reinterpret_cast<const u32x2*>(qzeros + (size_t)g * (N / 2) + (wcol >> 1));
    sc16[S] = scales[(size_t)g * N + sc_col];
  };

  f16v total[MT], grp[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) total[i][r] = 0.f;

  h2 z_lo[8], z_hi[8];   // zero points of this thread's 16 columns, paired (c0,c2) and (c1,c3), on both nibble biases
  auto prepare_zeros = [&](auto tag) {
    constexpr int S = decltype(tag)::value;
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
  };
  // Unpack one step (half H of the group in stage S) into LDS buffer `buf`.
  auto unpack = [&](int buf, auto tag, auto half_tag) {
    constexpr int S = decltype(tag)::value, H = decltype(half_tag)::value;
    u32x4 even[2], odd[2];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const unsigned int w = wq[S][H][j], w8 = w >> 8;
      const h2 e02 = as_h2(and_or(w, mg.mask_lo, mg.bias_lo)) - z_lo[2 * j];
      const h2 e13 = as_h2(and_or(w8, mg.mask_lo, mg.bias_lo)) - z_lo[2 * j + 1];
      const h2 o02 = as_h2(and_or(w, mg.mask_hi, mg.bias_hi)) - z_hi[2 * j];
      const h2 o13 = as_h2(and_or(w8, mg.mask_hi, mg.bias_hi)) - z_hi[2 * j + 1];
      even[j >> 1][(j & 1) * 2] = as_u32(e02);
      even[j >> 1][(j & 1) * 2 + 1] = as_u32(e13);
      odd[j >> 1][(j & 1) * 2] = as_u32(o02);
      odd[j >> 1][(j & 1) * 2 + 1] = as_u32(o13);
    }
    _Float16* row = Ws + buf * W_TILE + (2 * pr) * W_LD + cc * 16;       // packed row pr = k rows 2*pr, 2*pr+1 of the step
    *reinterpret_cast<u32x4*>(row) = even[0];
    *reinterpret_cast<u32x4*>(row + 8) = even[1];
    *reinterpret_cast<u32x4*>(row + W_LD) = odd[0];
    *reinterpret_cast<u32x4*>(row + W_LD + 8) = odd[1];
#pragma unroll
    for (int i = 0; i < XC; ++i) *reinterpret_cast<u32x4*>(Xs + buf * X_TILE + xs_off[i]) = xr[S][H][i];
  };
  // Operand fragments of two k-steps of 16 (kk0, kk0 + 1) of the step in LDS buffer `buf`.
  auto read_frags = [&](h8 (&fa)[2][MT], h8 (&fb)[2], int buf, int kk0) {
    const _Float16* ws = Ws + buf * W_TILE;
    const _Float16* xs = Xs + buf * X_TILE;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const _Float16* p = ws + ((kk0 + k) * 16 + b_k) * W_LD + b_n;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * W_LD));
      const h4 l4 = __builtin_bit_cast(h4, lo), h4v = __builtin_bit_cast(h4, hi);
      fb[k] = h8{l4[0], l4[1], l4[2], l4[3], h4v[0], h4v[1], h4v[2], h4v[3]};
#pragma unroll
      for (int t = 0; t < MT; ++t) fa[k][t] = *reinterpret_cast<const h8*>(xs + (a_row + t * 32) * X_LD + (kk0 + k) * 16 + a_k);
    }
  };
  auto mfma2 = [&](const h8 (&fa)[2][MT], const h8 (&fb)[2]) {
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
      for (int t = 0; t < MT; ++t) grp[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[k][t], fb[k], grp[t], 0, 0, 0);
  };
  // Scheduling masks of sched_group_barrier: 0x008 MFMA, 0x002 VALU, 0x100 LDS read, 0x200 LDS write, 0x020 global load.
  // First half of a step: the MFMAs of k-steps 0,1 with, between them, the operand reads of k-steps 2,3 and the
  // unpacking of the next step into the other buffer.
#define ART_FIRST_HALF()                                        \
  do {                                                          \
    __builtin_amdgcn_sched_group_barrier(0x100, 4 + 2 * MT, 0); \
    for (int m_ = 0; m_ < 2 * MT; ++m_) {                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        \
      __builtin_amdgcn_sched_group_barrier(0x002, 24, 0);       \
    }                                                           \
    __builtin_amdgcn_sched_group_barrier(0x200, 4 + XC, 0);     \
    __builtin_amdgcn_sched_barrier(0);                          \
  } while (0)
  // Second half: the MFMAs of k-steps 2,3 with the first operand reads of the next step (and the global loads) between them.
#define ART_SECOND_HALF()                                       \
  do {                                                          \
    __builtin_amdgcn_sched_group_barrier(0x100, 4 + 2 * MT, 0); \
    for (int m_ = 0; m_ < 2 * MT; ++m_) {                       \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        \
      __builtin_amdgcn_sched_group_barrier(0x020, 3, 0);        \
    }                                                           \
    __builtin_amdgcn_sched_barrier(0);                          \
  } while (0)

  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  using H0 = std::integral_constant<int, 0>;
  using H1 = std::integral_constant<int, 1>;
  const int last = groups - 1;
  if (groups > 0) {
    load_group(g_begin, S0{});
    load_group(g_begin + (groups > 1 ? 1 : 0), S1{});
    prepare_zeros(S0{});
    unpack(0, S0{}, H0{});
  }
  art_lds_barrier();
  h8 fa01[2][MT], fb01[2], fa23[2][MT], fb23[2];
  if (groups > 0) read_frags(fa01, fb01, 0, 0);
  // Group i (stage S): its first step sits in LDS buffer 0 and the operands of its k-steps 0,1 in registers.
  // The body has no branches (the scheduling directives work inside one basic block): past the last group it
  // reloads and unpacks the last group again, which nobody multiplies.
  auto group_body = [&](int i, auto tag, auto next_tag) {
    constexpr int S = decltype(tag)::value;
    const float sc = my_ok ? (float)sc16[S] : 0.f;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) grp[t][r] = 0.f;
    // step 0 of the group (buffer 0); step 1 is unpacked into buffer 1
    read_frags(fa23, fb23, 0, 2);
    unpack(1, tag, H1{});
    mfma2(fa01, fb01);
    ART_FIRST_HALF();
    art_lds_barrier();
    read_frags(fa01, fb01, 1, 0);
    load_group(g_begin + (i + 2 < groups ? i + 2 : last), tag);          // stage S is consumed: refill it
    mfma2(fa23, fb23);
    ART_SECOND_HALF();
    // step 1 of the group (buffer 1); step 0 of the next group is unpacked into buffer 0
    read_frags(fa23, fb23, 1, 2);
    prepare_zeros(next_tag);
    unpack(0, next_tag, H0{});
    mfma2(fa01, fb01);
    ART_FIRST_HALF();
    art_lds_barrier();
    read_frags(fa01, fb01, 0, 0);
    mfma2(fa23, fb23);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) total[t][r] += grp[t][r] * sc;
  };
  for (int i = 0; i < groups; i += 2) {
    group_body(i, S0{}, S1{});
    if (i + 1 < groups) group_body(i + 1, S1{}, S0{});
  }
#undef ART_FIRST_HALF
#undef ART_SECOND_HALF

  // ---- epilogue: accumulator element r of tile t is row t*32 + (r/4)*8 + (lane/32)*4 + r%4, column my_col
  if (!my_ok || groups == 0) return;
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = t * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
      if (row < M) {
        if (splits == 1) {
          _Float16 o = (_Float16)total[t][r];
          if (residual) o = (_Float16)((float)o + (float)residual[(size_t)row * N + my_col]);      // may alias y: same element
          y[(size_t)row * N + my_col] = o;
        }
        else partial[((size_t)split * M_total + m0 + row) * N + my_col] = total[t][r];
      }
    }
}

// y[m,n] = fp16(sum over splits, in split order); four columns per thread (N % 4 == 0).
__global__ __launch_bounds__(256) void gemm_w4a16_combine_kernel(const float* __restrict__ partial, _Float16* y,
                                                                  long long count4, long long split_stride, int splits,
                                                                  const _Float16* residual) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= count4) return;
  f32x4 t = *reinterpret_cast<const f32x4*>(partial + i * 4);
  for (int s = 1; s < splits; ++s) t += *reinterpret_cast<const f32x4*>(partial + s * split_stride + i * 4);
  h4 out = h4{(_Float16)t[0], (_Float16)t[1], (_Float16)t[2], (_Float16)t[3]};
  if (residual) {                    // y = fp16(fp16(product) + residual); residual may be y itself
    const h4 res = *reinterpret_cast<const h4*>(residual + i * 4);
    out = h4{(_Float16)((float)out[0] + (float)res[0]), (_Float16)((float)out[1] + (float)res[1]),
             (_Float16)((float)out[2] + (float)res[2]), (_Float16)((float)out[3] + (float)res[3])};
  }
  *reinterpret_cast<h4*>(y + i * 4) = out;
}

// Number of K-splits: as many blocks as the chip holds at once (one per compute unit), but at least
// two groups per block, no more partial-tile bytes than weight bytes (every split adds an fp32 copy of
// the output to the traffic), and no more than the scratch space allows.  The rule lands on the measured
// optimum at M = 64 on MI355X: 8 splits for 4096x4096, 5 for 4096x11008, 16 for 11008x4096, 2 for 4096x32000.
int choose_splits(int rows, int N, int K, size_t scratch_bytes, int compute_units) {
  const int col_tiles = (N + BN - 1) / BN, G = K / GK;
  int s = (512 / kThreads) * compute_units / col_tiles;      // blocks that are resident at once
  if (s > G / 2) s = G / 2;
  const size_t per_split = (size_t)rows * N * sizeof(float);
  const size_t weight_bytes = (size_t)K * N / 2;
  if ((size_t)s * per_split > weight_bytes) s = (int)(weight_bytes / per_split);
  const int cap = (int)(scratch_bytes / per_split);
  if (s > cap) s = cap;
  return s < 1 ? 1 : s;
}

}  // namespace

extern "C" int art_gemm_w4a16(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                              void* y_dev, int M, int K, int N, void* stream) {
  return art_gemm_w4a16_tuned(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, M, K, N, 0, stream);
}

extern "C" int art_gemm_w4a16_tuned(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                    void* y_dev, int M, int K, int N, int k_splits, void* stream) {
  return art_gemm_w4a16_residual(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, nullptr, M, K, N, k_splits, stream);
}

extern "C" int art_gemm_w4a16_residual(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                       void* y_dev, const void* residual_dev, int M, int K, int N, int k_splits, void* stream) {
  ART_REQUIRE(((uintptr_t)residual_dev % 8) == 0, "art_gemm_w4a16: the residual must be 8-byte aligned");
  ART_REQUIRE(!art::overlaps(x_dev, (size_t)M * K * 2, y_dev, (size_t)M * N * 2), "art_gemm_w4a16: y must not overlap x");
  ART_REQUIRE(k_splits >= 0, "art_gemm_w4a16: k_splits must be 0 (library's choice) or positive (got %d)", k_splits);
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemm_w4a16: null pointer");
  ART_REQUIRE(M >= 1, "art_gemm_w4a16: M must be positive (got %d)", M);
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemm_w4a16: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 16) == 0 && ((uintptr_t)qzeros_dev % 8) == 0 &&
                  ((uintptr_t)y_dev % 8) == 0,
              "art_gemm_w4a16: x and qweight must be 16-byte aligned, qzeros and y 8-byte aligned");
  art::Workspace* wsp = art::workspace((hipStream_t)stream);
  if (!wsp) return 1;
  art::Workspace& ws = *wsp;
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
  // Up to kMaxRowBlocks blocks of 64 rows go into one launch (they share the weight stream through L2, and the K-splits
  // are combined once); longer batches take several passes over the weights.
  constexpr int kMaxRowBlocks = 8;
  for (int m0 = 0; m0 < M; m0 += BM * kMaxRowBlocks) {
    const int rows = M - m0 < BM * kMaxRowBlocks ? M - m0 : BM * kMaxRowBlocks;
    const int m_blocks = (rows + BM - 1) / BM;
    int splits = choose_splits(rows, N, K, scratch_bytes, compute_units / m_blocks);
    if (k_splits > 0) {           // the caller's choice, within what the kernel and the scratch space take
      const int cap = (int)(scratch_bytes / ((size_t)rows * N * sizeof(float)));
      splits = k_splits > G ? G : k_splits;
      if (splits > cap) splits = cap < 1 ? 1 : cap;
    }
    const _Float16* xs = (const _Float16*)x_dev + (size_t)m0 * K;
    _Float16* ys = (_Float16*)y_dev + (size_t)m0 * N;
    const _Float16* rs = residual_dev ? (const _Float16*)residual_dev + (size_t)m0 * N : nullptr;
    const dim3 grid((unsigned)((col_tiles * splits + 7) / 8 * 8 * m_blocks));
    if (rows <= 32)
      gemm_w4a16_kernel<1><<<grid, kThreads, kLdsBytes, st>>>(xs, (const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                         (const unsigned char*)qzeros_dev, ys, scratch, rows, K, N, splits,
                                                         col_tiles, m_blocks, mg, rs);
    else
      gemm_w4a16_kernel<2><<<grid, kThreads, kLdsBytes, st>>>(xs, (const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                         (const unsigned char*)qzeros_dev, ys, scratch, rows, K, N, splits,
                                                         col_tiles, m_blocks, mg, rs);
    ART_LAUNCH_CHECK();
    if (splits > 1) {
      const long long count4 = (long long)rows * N / 4;
      gemm_w4a16_combine_kernel<<<dim3((unsigned)((count4 + 255) / 256)), 256, 0, st>>>(scratch, ys, count4, (long long)rows * N,
                                                                                        splits, rs);
      ART_LAUNCH_CHECK();
    }
  }
  return 0;
}
