// Weight-only int4 (group 128) GEMV / skinny GEMM for decode on gfx950.
//
//   y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/128,n]) * s[k/128,n]         (fp32 accumulate)
//
// Replaces the kernel the reference generates from the three-statement
// dequant + GEMV program of samples/05_llama2_7b_int4.py:135-139 (tiled or
// reduce schedule of backends/c-rocm/schedule/standard/, one nibble shifted,
// masked and converted per FMA).
//
// The kernel is bound by HBM: K*N/2 weight bytes are read exactly once and
// everything else is noise.  Design for MI355X:
//   * a lane owns 16 adjacent columns and R consecutive packed rows (2R values
//     of k), so every weight load is one 128-bit load and all R loads of a
//     lane are in flight before the first one is consumed;
//   * a 256-thread block is CL column lanes x (256/CL) k lanes; the grid is
//     (N / 16CL column tiles) x (K-splits), which gives >= 1 block per CU for
//     every Llama-2-7B shape;
//   * nibbles become fp16 without a convert: (w & 0x000F000F) | 0x64006400 is
//     the pair (1024+q, 1024+q') and (w & 0x00F000F0) | 0x54005400 the pair
//     (64+q, 64+q'); a v_perm puts two k values of one column into such a
//     pair, v_dot2_f32_f16 multiplies it with the matching pair of x and adds
//     into fp32.  The constants 1024 / 64 are removed once per lane from the
//     sums of x, together with the zero point;
//   * partial sums of the k lanes meet in LDS; the thread that owns a column
//     applies scale and zero point once per (group, column);
//   * K-splits meet in a workspace; the block that takes the last ticket of a
//     column tile adds them in a fixed order, so results are deterministic.
#include <hip/hip_fp16.h>

#include "art_common.h"

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kGroupRows = 64;         // packed rows per quantisation group (128 values of k)

__device__ __forceinline__ half2_t as_h2(unsigned int v) { return __builtin_bit_cast(half2_t, v); }

// One pair of packed words (rows i and i+1 of the same four columns) times the
// matching four values of x.  acc[0..3] are the four columns.
__device__ __forceinline__ void mac_word_pair(unsigned int a, unsigned int b, half2_t xe, half2_t xo, float* acc) {
  // p01 = [a.b0 a.b1 b.b0 b.b1], p23 = [a.b2 a.b3 b.b2 b.b3]
  const unsigned int p01 = __builtin_amdgcn_perm(b, a, 0x05040100u);
  const unsigned int p23 = __builtin_amdgcn_perm(b, a, 0x07060302u);
  const unsigned int p01s = p01 >> 8, p23s = p23 >> 8;
  acc[0] = __builtin_amdgcn_fdot2(as_h2((p01 & 0x000F000Fu) | 0x64006400u), xe, acc[0], false);
  acc[0] = __builtin_amdgcn_fdot2(as_h2((p01 & 0x00F000F0u) | 0x54005400u), xo, acc[0], false);
  acc[1] = __builtin_amdgcn_fdot2(as_h2((p01s & 0x000F000Fu) | 0x64006400u), xe, acc[1], false);
  acc[1] = __builtin_amdgcn_fdot2(as_h2((p01s & 0x00F000F0u) | 0x54005400u), xo, acc[1], false);
  acc[2] = __builtin_amdgcn_fdot2(as_h2((p23 & 0x000F000Fu) | 0x64006400u), xe, acc[2], false);
  acc[2] = __builtin_amdgcn_fdot2(as_h2((p23 & 0x00F000F0u) | 0x54005400u), xo, acc[2], false);
  acc[3] = __builtin_amdgcn_fdot2(as_h2((p23s & 0x000F000Fu) | 0x64006400u), xe, acc[3], false);
  acc[3] = __builtin_amdgcn_fdot2(as_h2((p23s & 0x00F000F0u) | 0x54005400u), xo, acc[3], false);
}

// R: packed rows per lane (4, 8, 16 or 32; a divisor of 64).  M: rows of x.  CL: column lanes per block.
template <int R, int M, int CL>
__global__ __launch_bounds__(kThreads) void gemv_w4a16_kernel(
    const _Float16* __restrict__ x, const unsigned char* __restrict__ qweight, const _Float16* __restrict__ scales,
    const unsigned char* __restrict__ qzeros, _Float16* __restrict__ y, int K, int N, int splits,
    float* __restrict__ partial, unsigned int* __restrict__ tickets) {
  constexpr int KL = kThreads / CL;          // k lanes per block
  constexpr int CT = 16 * CL;                // columns per block
  constexpr int KLG = kGroupRows / R;        // k lanes that share one quantisation group
  constexpr int GB = KL / KLG;               // groups per block
  static_assert(kGroupRows % R == 0 && KL % KLG == 0, "bad tiling");

  extern __shared__ __align__(16) unsigned char smem_raw[];
  float* red = reinterpret_cast<float*>(smem_raw);          // [M][KL][CT]
  float* aux = red + M * KL * CT;                           // [M][KL][2] : (corr, xsum)
  __shared__ unsigned int s_ticket;

  const int tid = threadIdx.x;
  const int cl = tid % CL, kl = tid / CL;
  const int tile = blockIdx.x, split = blockIdx.y;
  const int n0 = tile * CT + cl * 16;
  const int rows = K >> 1;
  const int r0 = (split * KL + kl) * R;                     // first packed row of this lane
  const bool active = (n0 < N) && (r0 < rows);

  // ---- issue every global load of this lane up front
  u32x4 w[R];
  if (active) {
    const unsigned char* wp = qweight + (size_t)r0 * N + n0;
#pragma unroll
    for (int i = 0; i < R; ++i) w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + (size_t)i * N));
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) w[i] = u32x4{0, 0, 0, 0};
  }
  // x: 2R consecutive halves = R dwords per row of x
  unsigned int xw[M][R];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const unsigned int* xp = reinterpret_cast<const unsigned int*>(x + (size_t)m * K + 2 * r0);
#pragma unroll
    for (int i = 0; i < R; ++i) xw[m][i] = (r0 < rows) ? xp[i] : 0u;
  }
  // column owners fetch scale / zero of their column for every group of the block
  const int col = tile * CT + tid;                          // owner of column `tid` of the tile (tid < CT)
  const int g0 = (split * KL * R) / kGroupRows;
  const int groups = K / 128;
  _Float16 sc[GB];
  unsigned char zb[GB];
  const bool owner = (tid < CT) && (col < N);
  if (CT <= kThreads) {
#pragma unroll
    for (int g = 0; g < GB; ++g) {
      const bool ok = owner && (g0 + g < groups);
      sc[g] = ok ? scales[(size_t)(g0 + g) * N + col] : (_Float16)0;
      zb[g] = ok ? qzeros[(size_t)(g0 + g) * (N >> 1) + (col >> 1)] : (unsigned char)0;
    }
  }

  // ---- multiply-accumulate
  float acc[M][16];
  float se[M], so[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    se[m] = 0.f; so[m] = 0.f;
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[m][c] = 0.f;
  }
  const half2_t ones = {(_Float16)1, (_Float16)1};
#pragma unroll
  for (int i = 0; i < R; i += 2) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      // rows i, i+1 hold k = 2i, 2i+1 | 2i+2, 2i+3 ; x words: (x[2i],x[2i+1]) , (x[2i+2],x[2i+3])
      const half2_t xe = as_h2(__builtin_amdgcn_perm(xw[m][i + 1], xw[m][i], 0x05040100u));   // even k pair
      const half2_t xo = as_h2(__builtin_amdgcn_perm(xw[m][i + 1], xw[m][i], 0x07060302u));   // odd k pair
      se[m] = __builtin_amdgcn_fdot2(xe, ones, se[m], false);
      so[m] = __builtin_amdgcn_fdot2(xo, ones, so[m], false);
#pragma unroll
      for (int j = 0; j < 4; ++j) mac_word_pair(w[i][j], w[i + 1][j], xe, xo, &acc[m][4 * j]);
    }
  }

  // ---- meet in LDS
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float* dst = red + ((size_t)m * KL + kl) * CT + cl * 16;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<f32x4*>(dst + 4 * j) = f32x4{acc[m][4 * j], acc[m][4 * j + 1], acc[m][4 * j + 2], acc[m][4 * j + 3]};
    if (cl == 0) {
      aux[(m * KL + kl) * 2 + 0] = 1024.f * se[m] + 64.f * so[m];
      aux[(m * KL + kl) * 2 + 1] = se[m] + so[m];
    }
  }
  __syncthreads();

  float res[M];
  if (tid < CT) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float r = 0.f;
#pragma unroll
      for (int g = 0; g < GB; ++g) {
        float a = 0.f, corr = 0.f, xs = 0.f;
#pragma unroll
        for (int q = 0; q < KLG; ++q) {
          const int k = g * KLG + q;
          a += red[((size_t)m * KL + k) * CT + tid];
          corr += aux[(m * KL + k) * 2 + 0];
          xs += aux[(m * KL + k) * 2 + 1];
        }
        const float z = (float)((col & 1) ? (zb[g] >> 4) : (zb[g] & 15));
        r += (float)sc[g] * (a - corr - z * xs);
      }
      res[m] = r;
    }
  }

  if (splits == 1) {
    if (owner) {
#pragma unroll
      for (int m = 0; m < M; ++m) y[(size_t)m * N + col] = (_Float16)res[m];
    }
    return;
  }

  // ---- K-splits: park the partial sums, the last block of the tile adds them up
  if (owner) {
#pragma unroll
    for (int m = 0; m < M; ++m)
      __hip_atomic_store(&partial[((size_t)split * M + m) * N + col], res[m], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __threadfence();
  __syncthreads();
  if (tid == 0) s_ticket = atomicAdd(&tickets[tile], 1u);
  __syncthreads();
  if (s_ticket != (unsigned int)(splits - 1)) return;
  __threadfence();
  if (owner) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float r = 0.f;
      for (int s = 0; s < splits; ++s)
        r += __hip_atomic_load(&partial[((size_t)s * M + m) * N + col], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      y[(size_t)m * N + col] = (_Float16)r;
    }
  }
  if (tid == 0) tickets[tile] = 0u;      // ready for the next launch (stream order makes this visible)
}

template <int R, int M, int CL>
int launch(const void* x, const void* qw, const void* sc, const void* qz, void* y, int K, int N, hipStream_t stream) {
  constexpr int KL = kThreads / CL, CT = 16 * CL;
  const int rows = K / 2;
  const int tiles = (N + CT - 1) / CT;
  const int splits = (rows + KL * R - 1) / (KL * R);
  art::Workspace& ws = art::workspace();
  ART_REQUIRE(ws.base != nullptr, "art_gemv_w4a16: call art_init first");
  const size_t ticket_bytes = art::kGemvTicketBytes;
  ART_REQUIRE((size_t)tiles * 4 <= ticket_bytes, "art_gemv_w4a16: N too large (%d)", N);
  const size_t need = art::kScratchOffset + (size_t)splits * M * N * sizeof(float);
  ART_REQUIRE(splits == 1 || need <= ws.bytes, "art_gemv_w4a16: workspace too small for K=%d N=%d", K, N);
  unsigned int* tickets = reinterpret_cast<unsigned int*>(ws.base);
  float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(ws.base) + art::kScratchOffset);
  const size_t lds = (size_t)M * KL * CT * sizeof(float) + (size_t)M * KL * 2 * sizeof(float);
  auto kernel = gemv_w4a16_kernel<R, M, CL>;
  if (lds > 48 * 1024) {
    ART_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  }
  kernel<<<dim3(tiles, splits), dim3(kThreads), lds, stream>>>(
      (const _Float16*)x, (const unsigned char*)qw, (const _Float16*)sc, (const unsigned char*)qz, (_Float16*)y, K, N,
      splits, partial, tickets);
  ART_LAUNCH_CHECK();
  return 0;
}

// Rows per lane: enough blocks to cover 256 CUs, otherwise as many rows as possible.
template <int M>
int dispatch_rows(const void* x, const void* qw, const void* sc, const void* qz, void* y, int K, int N, hipStream_t st) {
  constexpr int CL = 8;
  const int tiles = (N + 16 * CL - 1) / (16 * CL);
  const int rows = K / 2;
  auto blocks = [&](int R) { return tiles * ((rows + (kThreads / CL) * R - 1) / ((kThreads / CL) * R)); };
  const char* force = getenv("ART_GEMV_ROWS");
  int R = force ? atoi(force) : 0;
  if (!R) R = blocks(16) >= 256 ? 16 : (blocks(8) >= 256 ? 8 : 4);
  switch (R) {
    case 16: return launch<16, M, CL>(x, qw, sc, qz, y, K, N, st);
    case 8: return launch<8, M, CL>(x, qw, sc, qz, y, K, N, st);
    case 4: return launch<4, M, CL>(x, qw, sc, qz, y, K, N, st);
    default: return art::fail("art_gemv_w4a16: unsupported rows-per-lane %d", R);
  }
}

}  // namespace

extern "C" int art_gemv_w4a16(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                              void* y_dev, int M, int K, int N, void* stream) {
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemv_w4a16: null pointer");
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemv_w4a16: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 4) == 0, "art_gemv_w4a16: qweight must be 16-byte and x 4-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  switch (M) {
    case 1: return dispatch_rows<1>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st);
    case 2: return dispatch_rows<2>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st);
    case 4: return dispatch_rows<4>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st);
    default: break;
  }
  ART_REQUIRE(M >= 1 && M <= 8, "art_gemv_w4a16: M must be in 1..8 (got %d); use art_gemm_w4a16 for prefill", M);
  // other row counts: run rows one / two / four at a time
  int m = 0;
  while (m < M) {
    const int step = (M - m >= 4) ? 4 : ((M - m >= 2) ? 2 : 1);
    const _Float16* xs = (const _Float16*)x_dev + (size_t)m * K;
    _Float16* ys = (_Float16*)y_dev + (size_t)m * N;
    int rc = art_gemv_w4a16(xs, qweight_dev, scales_dev, qzeros_dev, ys, step, K, N, stream);
    if (rc) return rc;
    m += step;
  }
  return 0;
}
