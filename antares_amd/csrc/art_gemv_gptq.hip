// int4 GEMV in the reference's own weight format
// (samples/05_llama2_7b_int4.py:135-139):
//
//   y[n] = sum_k x[k] * ( scales[k/128, n] * ( ((qweight[k/8, n] >> (k%8*4)) & 15) - 8 ) )
//
// qweight is int32 [K/8, N] (eight nibbles of one column per word, least
// significant first), scales fp32 or fp16 [K/128, N], x and y fp32 or fp16.
// All arithmetic is fp32: nibble -> float through v_cvt_f32_ubyte after one
// mask, one FMA per weight.  A lane owns 4 adjacent columns (one 128-bit load
// per word row) and R word rows; k lanes meet in LDS, the column owner applies
// scale and the fixed zero point 8 once per (group, column); K-splits are
// added in a fixed order by the block that draws the last ticket.
#include "art_common.h"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int CL = 16;                 // column lanes  -> 64 columns per block
constexpr int KL = kThreads / CL;      // 16 k lanes
constexpr int CT = 4 * CL;
constexpr int R = 4;                   // word rows per lane (32 values of k)
constexpr int kGroupWordRows = 16;     // 128 / 8
constexpr int KLG = kGroupWordRows / R;
constexpr int GB = KL / KLG;           // groups per block

template <class T> __device__ __forceinline__ float ldf(const T* p, size_t i) { return (float)p[i]; }

template <class XT, class ST>
__global__ __launch_bounds__(kThreads) void gemv_gptq_kernel(const XT* __restrict__ x, const unsigned int* __restrict__ qweight,
                                                             const ST* __restrict__ scales, XT* __restrict__ y, int K, int N,
                                                             int splits, float* __restrict__ partial,
                                                             unsigned int* __restrict__ tickets) {
  __shared__ float red[KL][CT];
  __shared__ float xsum[KL];
  __shared__ unsigned int s_ticket;
  const int tid = threadIdx.x, cl = tid % CL, kl = tid / CL;
  const int tile = blockIdx.x, split = blockIdx.y;
  const int n0 = tile * CT + cl * 4;
  const int wrows = K >> 3;
  const int r0 = (split * KL + kl) * R;
  const bool active = (n0 < N) && (r0 < wrows);

  u32x4 w[R];
#pragma unroll
  for (int i = 0; i < R; ++i)
    w[i] = (active && r0 + i < wrows)
               ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(qweight + (size_t)(r0 + i) * N + n0))
               : u32x4{0, 0, 0, 0};
  float xv[R][8];
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) xv[i][j] = (r0 + i < wrows) ? ldf(x, (size_t)(r0 + i) * 8 + j) : 0.f;

  const int col = tile * CT + tid;
  const bool owner = (tid < CT) && (col < N);
  const int g0 = (split * KL * R) / kGroupWordRows, groups = K / 128;
  float sc[GB];
#pragma unroll
  for (int g = 0; g < GB; ++g) sc[g] = (owner && g0 + g < groups) ? ldf(scales, (size_t)(g0 + g) * N + col) : 0.f;

  float acc[4] = {0.f, 0.f, 0.f, 0.f}, xs = 0.f;
#pragma unroll
  for (int i = 0; i < R; ++i) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      xs += xv[i][j];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = fmaf(xv[i][j], (float)((w[i][c] >> (4 * j)) & 15u), acc[c]);
    }
  }
  *reinterpret_cast<f32x4*>(&red[kl][cl * 4]) = f32x4{acc[0], acc[1], acc[2], acc[3]};
  if (cl == 0) xsum[kl] = xs;
  __syncthreads();

  float res = 0.f;
  if (tid < CT) {
#pragma unroll
    for (int g = 0; g < GB; ++g) {
      float a = 0.f, s = 0.f;
#pragma unroll
      for (int q = 0; q < KLG; ++q) {
        a += red[g * KLG + q][tid];
        s += xsum[g * KLG + q];
      }
      res += sc[g] * (a - 8.f * s);
    }
  }
  if (splits == 1) {
    if (owner) y[col] = (XT)res;
    return;
  }
  if (owner) __hip_atomic_store(&partial[(size_t)split * N + col], res, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // The partial sums were written through to device-coherent memory; wait until
  // they have landed (vmcnt(0)) before this block's ticket can be seen.  A device-scope
  // release fence would do the same but writes back the whole L2 of the XCD.
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  if (tid == 0) s_ticket = __hip_atomic_fetch_add(&tickets[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (s_ticket != (unsigned int)(splits - 1)) return;
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  if (owner) {
    float r = 0.f;
    for (int s = 0; s < splits; ++s)
      r += __hip_atomic_load(&partial[(size_t)s * N + col], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    y[col] = (XT)r;
  }
  if (tid == 0) tickets[tile] = 0u;
}

template <class XT, class ST>
int launch(const void* x, const void* qw, const void* sc, void* y, int K, int N, hipStream_t stream) {
  const int wrows = K / 8;
  const int tiles = (N + CT - 1) / CT;
  const int splits = (wrows + KL * R - 1) / (KL * R);
  art::Workspace& ws = art::workspace();
  ART_REQUIRE(ws.base != nullptr, "art_gemv_gptq: call art_init first");
  const size_t ticket_bytes = art::kGemvTicketBytes;
  ART_REQUIRE((size_t)tiles * 4 <= ticket_bytes, "art_gemv_gptq: N too large (%d)", N);
  ART_REQUIRE(splits == 1 || art::kScratchOffset + (size_t)splits * N * 4 <= ws.bytes, "art_gemv_gptq: workspace too small");
  unsigned int* tickets = reinterpret_cast<unsigned int*>(ws.base);
  float* partial = reinterpret_cast<float*>(reinterpret_cast<char*>(ws.base) + art::kScratchOffset);
  gemv_gptq_kernel<XT, ST><<<dim3(tiles, splits), dim3(kThreads), 0, stream>>>(
      (const XT*)x, (const unsigned int*)qw, (const ST*)sc, (XT*)y, K, N, splits, partial, tickets);
  ART_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" int art_gemv_gptq(const void* x_dev, const void* qweight_dev, const void* scales_dev, void* y_dev, int K, int N,
                             int x_f16, int scales_f16, void* stream) {
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && y_dev, "art_gemv_gptq: null pointer");
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 4 == 0, "art_gemv_gptq: need K %% 128 == 0 and N %% 4 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0, "art_gemv_gptq: qweight must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (x_f16) {
    return scales_f16 ? launch<_Float16, _Float16>(x_dev, qweight_dev, scales_dev, y_dev, K, N, st)
                      : launch<_Float16, float>(x_dev, qweight_dev, scales_dev, y_dev, K, N, st);
  }
  return scales_f16 ? launch<float, _Float16>(x_dev, qweight_dev, scales_dev, y_dev, K, N, st)
                    : launch<float, float>(x_dev, qweight_dev, scales_dev, y_dev, K, N, st);
}
