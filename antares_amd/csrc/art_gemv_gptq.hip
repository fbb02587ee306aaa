// int4 GEMV in the reference's own weight format
// (samples/05_llama2_7b_int4.py:135-139):
//
//   y[n] = sum_k x[k] * ( scales[k/128, n] * ( ((qweight[k/8, n] >> (k%8*4)) & 15) - 8 ) )
//
// qweight is int32 [K/8, N] (eight nibbles of one column per word, least
// significant first), scales fp32 or fp16 [K/128, N], x and y fp32 or fp16.
// The sample runs it in fp32, so all arithmetic here is fp32 and exact per product:
//   * a lane owns 4 adjacent columns (one 128-bit load per word row) and 8 word rows (64 values of k);
//     16 column lanes x 16 k lanes make a block of 64 columns x 1024 k = 32 KiB of weights, all eight loads
//     of a lane in flight before the first is used; the grid is (N/64) x (K/1024): 688 blocks for 4096 x 11008;
//   * the block's 1024 values of x go through LDS once (one 16-byte load per thread, an LDS-only barrier so
//     the weight loads stay in flight) and are read back as broadcasts;
//   * (w & 0x0F0F0F0F) and ((w >> 4) & 0x0F0F0F0F) put the even and the odd nibbles of a word into bytes;
//     v_cvt_f32_ubyte0..3 turns each byte into a float, one FMA per weight: 2.4 VALU operations per weight;
//   * the k lanes of a block meet in LDS; the owner of a column applies scale and the fixed zero point 8 once
//     per (group, column): s * (acc - 8 * sum(x));
//   * the K-splits of a column meet in returning 64-bit atomics: a fixed-point partial sum with an arrival count in
//     the top byte and a count of non-finite partial sums in the bottom one.  Integer addition is associative, so
//     the result does not depend on the arrival order; the block that sees count == splits - 1 holds the total,
//     writes y and clears the slot.  One slot (steps of 2^-22) is all an fp16 result needs.  An fp32 result gets a
//     second slot for what the first one rounds away (first slot in steps of 2^-8 up to 2^39 / splits, second in steps of 2^-58): both atomics of a block are issued together,
//     and the block that completes the first slot usually completes the second as well (else it re-reads it until
//     the adds that are still in flight have landed), so the sum of the partial sums is exact wherever fp32 is.
#include "art_common.h"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int CL = 16;                 // column lanes  -> 64 columns per block
constexpr int KL = kThreads / CL;      // 16 k lanes
constexpr int CT = 4 * CL;             // columns per block
constexpr int R = 8;                   // word rows per lane (64 values of k)
constexpr int kBlockK = KL * R * 8;    // 1024 values of k per block
constexpr int GB = kBlockK / 128;      // 8 quantisation groups per block, two k lanes each
constexpr float kFix = 1073741824.f;   // 2^30

// A partial sum on its way through the 64-bit slot: a multiple of 256 in units of 2^-30 (so 2^-22 is the step), which
// leaves the low byte free to count the partial sums that are not finite or too large for the field (2^24 / splits
// keeps the sum of all of them below 2^55, clear of the arrival count above it).  Such a partial sum contributes 1:
// it can neither run into the count - which would leave the slot dirty for every later launch - nor get lost: a
// total with a non-zero low byte is written out as NaN.
__device__ __forceinline__ long long to_fixed(float r, int splits) {
  const float limit = 16777216.f / (float)splits;
  return fabsf(r) < limit ? __float2ll_rn(r * (kFix / 256.f)) * 256 : 1LL;     // NaN fails the comparison too
}
__device__ __forceinline__ float from_fixed(long long total) {
  return (total & 255) ? __builtin_nanf("") : (float)total * (1.f / kFix);
}

// fp32 results take two slots.  First slot: multiples of 256 in units of 2^-16 (steps of 2^-8, low byte = count of
// rejected partial sums as above), |r| < 2^39 / splits.  Second slot: what the first rounds away, in units of 2^-58
// (|r * 2^8| below 2^23 has a fraction, anything larger is an integer already).  Together: every partial sum with
// 2^-34 <= |r| < 2^39 / splits travels exactly, smaller ones to within 2^-59.
__device__ __forceinline__ long long to_fixed_wide(float r, int splits) {
  const float limit = 549755813888.f / (float)splits;
  return fabsf(r) < limit ? __float2ll_rn(r * 256.f) * 256 : 1LL;
}
__device__ __forceinline__ long long to_fixed_rest(float r, int splits) {
  const float limit = 549755813888.f / (float)splits;
  if (!(fabsf(r) < limit)) return 0LL;
  const float t = r * 256.f;                                  // exact
  return __float2ll_rn((t - rintf(t)) * 1125899906842624.f);  // (t - rint t) is exact, |.| <= 0.5; times 2^50
}
constexpr int kMaxSpin = 1 << 22;

template <class T> __device__ __forceinline__ float ldf(const T* p, size_t i) { return (float)p[i]; }

__device__ __forceinline__ float ubyte(unsigned int w, int b) {       // byte b of w as a float (v_cvt_f32_ubyte<b>)
  return (float)((w >> (8 * b)) & 0xffu);
}

template <class XT, class ST>
__global__ __launch_bounds__(kThreads) void gemv_gptq_kernel(const XT* __restrict__ x, const unsigned int* __restrict__ qweight,
                                                             const ST* __restrict__ scales, XT* __restrict__ y, int K, int N,
                                                             int splits, unsigned long long* __restrict__ slots) {
  __shared__ __align__(16) float s_x[kBlockK];
  __shared__ __align__(16) float red[KL][CT];
  __shared__ float xsum[KL];
  const int tid = threadIdx.x, cl = tid % CL, kl = tid / CL;
  const int tile = blockIdx.x, split = blockIdx.y;
  const int n0 = tile * CT + cl * 4;
  const int wrows = K >> 3;
  const int r0 = (split * KL + kl) * R;                   // first word row of this lane
  // lanes past an edge read a valid patch instead of branching; their x is zero / their columns are never written
  const int n0c = n0 < N ? n0 : 0;

  // x of the block first: it is small, comes from L2, and nothing can be multiplied without it
  const int k0 = split * kBlockK + 4 * tid;
#pragma unroll
  for (int j = 0; j < 4; ++j) s_x[4 * tid + j] = (k0 + j < K) ? ldf(x, (size_t)k0 + j) : 0.f;

  u32x4 w[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int r = r0 + i < wrows ? r0 + i : wrows - 1;    // past the end: any valid row, x is zero there
    w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(qweight + (size_t)r * N + n0c));   // streamed once
  }
  // column owners fetch the scales of their column for the eight groups of the block
  const int col = tile * CT + tid;
  const bool owner = (tid < CT) && (col < N);
  const int g0 = split * GB, groups = K >> 7;
  float sc[GB];
#pragma unroll
  for (int g = 0; g < GB; ++g) sc[g] = (owner && g0 + g < groups) ? ldf(scales, (size_t)(g0 + g) * N + col) : 0.f;

  art_lds_barrier();                                     // LDS only: the weight loads stay in flight
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, xs = 0.f;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const f32x4 xa = *reinterpret_cast<const f32x4*>(&s_x[(kl * R + i) * 8]);
    const f32x4 xb = *reinterpret_cast<const f32x4*>(&s_x[(kl * R + i) * 8 + 4]);
    xs += ((xa[0] + xa[1]) + (xa[2] + xa[3])) + ((xb[0] + xb[1]) + (xb[2] + xb[3]));
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const unsigned int even = w[i][c] & 0x0F0F0F0Fu, odd = (w[i][c] >> 4) & 0x0F0F0F0Fu;   // nibbles 0,2,4,6 | 1,3,5,7
      float a = acc[c];
      a = fmaf(xa[0], ubyte(even, 0), a);
      a = fmaf(xa[1], ubyte(odd, 0), a);
      a = fmaf(xa[2], ubyte(even, 1), a);
      a = fmaf(xa[3], ubyte(odd, 1), a);
      a = fmaf(xb[0], ubyte(even, 2), a);
      a = fmaf(xb[1], ubyte(odd, 2), a);
      a = fmaf(xb[2], ubyte(even, 3), a);
      a = fmaf(xb[3], ubyte(odd, 3), a);
      acc[c] = a;
    }
  }
  *reinterpret_cast<f32x4*>(&red[kl][cl * 4]) = f32x4{acc[0], acc[1], acc[2], acc[3]};
  if (cl == 0) xsum[kl] = xs;
  __syncthreads();
  if (!owner) return;

  float res = 0.f;
#pragma unroll
  for (int g = 0; g < GB; ++g) {                         // a group is two k lanes
    const float a = red[2 * g][tid] + red[2 * g + 1][tid];
    const float s = xsum[2 * g] + xsum[2 * g + 1];
    res += sc[g] * (a - 8.f * s);
  }
  if (splits == 1) {
    y[col] = (XT)res;
    return;
  }
  // returning atomics: [arrival count : 8][fixed-point sum : 56]
  constexpr bool exact = sizeof(XT) == 4;              // fp32 result: second slot for the rounded-away part
  unsigned long long* slot = slots + col;
  unsigned long long* slot_lo = slots + N + col;
  const long long mine = (1LL << 56) + (exact ? to_fixed_wide(res, splits) : to_fixed(res, splits));
  const long long mine_lo = (1LL << 56) + to_fixed_rest(res, splits);
  long long old_lo = 0;
  if (exact) old_lo = (long long)__hip_atomic_fetch_add(slot_lo, (unsigned long long)mine_lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const long long old = (long long)__hip_atomic_fetch_add(slot, (unsigned long long)mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (((old + (1LL << 55)) >> 56) == (long long)(splits - 1)) {
    const long long total = old + mine - ((long long)splits << 56);
    if (!exact) {
      y[col] = (XT)from_fixed(total);
    } else {
      // every other block issued its add to the second slot before (or with) the one this block has just seen
      // land in the first: the count there reaches `splits` within a memory round trip.  The wait is bounded.
      long long lo = old_lo + mine_lo;
      for (int spin = 0; ((lo + (1LL << 55)) >> 56) != (long long)splits && spin < kMaxSpin; ++spin)
        lo = (long long)__hip_atomic_load(slot_lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool complete = ((lo + (1LL << 55)) >> 56) == (long long)splits;
      lo -= (long long)splits << 56;
      const double v = (double)(total >> 8) * (1.0 / 256.0) + (double)lo * (1.0 / 288230376151711744.0);     // 2^-8, 2^-58
      y[col] = (XT)(((total & 255) || !complete) ? __builtin_nanf("") : (float)v);
      *slot_lo = 0ull;
    }
    *slot = 0ull;                       // ready for the next launch (stream order makes this visible)
  }
}

template <class XT, class ST>
int launch(const void* x, const void* qw, const void* sc, void* y, int K, int N, hipStream_t stream) {
  const int tiles = (N + CT - 1) / CT;
  const int splits = (K + kBlockK - 1) / kBlockK;
  ART_REQUIRE(splits <= 127, "art_gemv_gptq: K too large (%d)", K);
  art::Workspace* wsp = art::workspace(stream);
  if (!wsp) return 1;
  art::Workspace& ws = *wsp;
  ART_REQUIRE(art::kSlotOffset + (size_t)N * 16 <= art::kScratchOffset, "art_gemv_gptq: N too large (%d)", N);
  unsigned long long* slots = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(ws.base) + art::kSlotOffset);
  gemv_gptq_kernel<XT, ST><<<dim3(tiles, splits), dim3(kThreads), 0, stream>>>(
      (const XT*)x, (const unsigned int*)qw, (const ST*)sc, (XT*)y, K, N, splits, slots);
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
