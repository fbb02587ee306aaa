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
// everything else is noise.  What the hardware rewards (measured on MI355X with
// read-only kernels of the same access pattern): many small blocks on all 256
// CUs, 128 contiguous bytes per row per request, every load of a lane in flight
// before the first is consumed, and no second memory round trip after the
// stream.  Hence:
//   * a lane owns 16 adjacent columns and 8 consecutive packed rows (16 values
//     of k): eight 128-bit loads issued back to back; 8 adjacent lanes read a
//     whole 128-byte line of each row;
//   * a 256-thread block is 8 column lanes x 32 k lanes = a 128-column x 512-k
//     patch; each of its four wavefronts covers exactly one quantisation group.
//     The grid is (N/128 tiles) x (K/512 splits): 688 blocks for 4096x11008;
//   * nibbles become fp16 without a convert: (w & 0x000F000F) | 0x64006400 is
//     the pair (1024+q, 1024+q') and (w & 0x00F000F0) | 0x54005400 the pair
//     (64+q, 64+q'); a v_perm puts two k values of one column into such a
//     pair, v_dot2_f32_f16 multiplies it with the matching pair of x and adds
//     into fp32.  The constants 1024 / 64 leave together with the zero point,
//     once per (group, column): s * (acc - 1024*sum(x_even) - 64*sum(x_odd) - z*sum(x));
//   * the eight k lanes of a wavefront meet by a reduce-scatter over lane bits 5, 4, 3 (v_permlane32_swap,
//     v_permlane16_swap, row_ror:8 DPP): 16 -> 8 -> 4 -> 2 columns per lane, 30 vector operations; a wavefront is
//     one quantisation group, so each lane applies scale and zero point to its two columns right there, and the
//     four wavefronts of the block meet in 2 KiB of LDS;
//   * the K-splits of a column meet in ONE returning 64-bit atomic per block:
//     the partial sum travels as a fixed-point integer (steps of 2^-22) with an
//     arrival count in the top byte and a count of non-finite partial sums in the
//     bottom one.  Integer addition is associative, so the result
//     does not depend on arrival order (deterministic), and the block whose
//     atomic returns count == splits-1 holds the complete sum in registers: it
//     writes y and resets the slot.  One round trip, no fence, no re-read.
#include "art_common.h"

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ half2_t as_h2(unsigned int v) { return __builtin_bit_cast(half2_t, v); }

// Nibble -> fp16 constants.  They reach the kernel as arguments, not literals:
// with run-time values (w & m) | (~m & g) selects to one v_bfi_b32, with
// literals the compiler emits v_and_b32 + v_or_b32 (gfx9 VOP3 takes no literal).
struct Magic {
  unsigned int mask_lo, mask_hi, bias_lo, bias_hi;   // 0x000F000F 0x00F000F0 0x64006400 0x54005400
};

__device__ __forceinline__ half2_t nib(unsigned int w, unsigned int mask, unsigned int bias) {
  return as_h2((w & mask) | (~mask & bias));
}

// One pair of packed words (rows i and i+1 of the same four columns) times the
// matching four values of x.  acc[0..3] are the four columns.
__device__ __forceinline__ void mac_word_pair(unsigned int a, unsigned int b, half2_t xe, half2_t xo, float* acc, const Magic& k) {
  // p01 = [a.b0 a.b1 b.b0 b.b1], p23 = [a.b2 a.b3 b.b2 b.b3]
  const unsigned int p01 = __builtin_amdgcn_perm(b, a, 0x05040100u);
  const unsigned int p23 = __builtin_amdgcn_perm(b, a, 0x07060302u);
  const unsigned int p01s = p01 >> 8, p23s = p23 >> 8;
  acc[0] = __builtin_amdgcn_fdot2(nib(p01, k.mask_lo, k.bias_lo), xe, acc[0], false);
  acc[0] = __builtin_amdgcn_fdot2(nib(p01, k.mask_hi, k.bias_hi), xo, acc[0], false);
  acc[1] = __builtin_amdgcn_fdot2(nib(p01s, k.mask_lo, k.bias_lo), xe, acc[1], false);
  acc[1] = __builtin_amdgcn_fdot2(nib(p01s, k.mask_hi, k.bias_hi), xo, acc[1], false);
  acc[2] = __builtin_amdgcn_fdot2(nib(p23, k.mask_lo, k.bias_lo), xe, acc[2], false);
  acc[2] = __builtin_amdgcn_fdot2(nib(p23, k.mask_hi, k.bias_hi), xo, acc[2], false);
  acc[3] = __builtin_amdgcn_fdot2(nib(p23s, k.mask_lo, k.bias_lo), xe, acc[3], false);
  acc[3] = __builtin_amdgcn_fdot2(nib(p23s, k.mask_hi, k.bias_hi), xo, acc[3], false);
}

constexpr int CL = 8;                  // column lanes per block (8 k lanes per wavefront)
constexpr int CT = 16 * CL;            // 128 columns per block
// Wavefronts per block, W, is the other launch parameter (template): 4 (256 threads) or 8 (512 threads).  Eight
// double the k range of a block, so a column receives half as many returning atomics; a tuning run may pick it.
// Packed rows per lane, R, is a launch parameter (template): 8 rows make a block 128 columns x 512 k with each
// wavefront on exactly one quantisation group of 128 k; 4 rows make it 128 x 256 with two wavefronts per group -
// twice the blocks (and twice the returning atomics), which pays when 8 rows leave compute units without a block.
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

__device__ __forceinline__ float dpp_ror8(float v) {      // the value of lane ^ 8 (row_ror:8)
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
}
// One step of a reduce-scatter between lanes l and l ^ 32 (l ^ 16): the lower lane of the pair keeps `a`, the upper
// one keeps `b`; returns the pair's sum of what this lane keeps.  The swap exchanges the upper lanes' `a` with the
// lower lanes' `b`, so both operands of the addition are the kept quantity afterwards.
__device__ __forceinline__ float swap32_add(float a, float b) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b), false, false);
  return __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
}
__device__ __forceinline__ float swap16_add(float a, float b) {
  auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b), false, false);
  return __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
}

// Sum over the 8 k lanes of a wavefront (lanes that share lane % 8); all lanes get the sum.
__device__ __forceinline__ float sum_k_lanes_of_wave(float v) {
  v += dpp_ror8(v);
  {
    const unsigned int u = __builtin_bit_cast(unsigned int, v);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
  }
  {
    const unsigned int u = __builtin_bit_cast(unsigned int, v);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    v = __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
  }
  return v;
}

// sum over the 64 lanes of a wavefront; every lane gets the result
__device__ __forceinline__ float wave_sum_all(float v) {
#define ART_DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false))
  ART_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
  ART_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
  ART_DPP_ADD(0x141);   // row_half_mirror
  ART_DPP_ADD(0x140);   // row_mirror
#undef ART_DPP_ADD
  const int b = __builtin_bit_cast(int, v);
  return (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
}

// Optional work fused around the product (decode, M = 1):
//   norm_w   != NULL : x is replaced by RMSNorm(x) = fp16(x * rsqrt(sum(x^2) * inv_n + eps) * norm_w) before the product;
//   residual != NULL : y = fp16(fp16(product) + residual), i.e. the residual add that follows the projection.
//   gate_up  != NULL : x is not read; x[k] = fp16(silu(gate_up[k]) * gate_up[K + k]) (SwiGLU, line :171 of the sample).
struct Fused {
  const _Float16* norm_w;
  const _Float16* residual;
  const _Float16* gate_up;
  float inv_n, eps;
  const float* att_partial;   // != NULL: x is merged from the per-part records of a split decode attention (see MODE 3)
  int att_parts;
  // sum(y^2) handed from the projection that writes a residual stream to the projection that normalises it (M = 1):
  //   sumsq_out   != NULL : every block adds the squares of the outputs it finishes (after the residual add, as rounded
  //                         to fp16) to word [column tile] of it, as fixed point in units of 2^-30;
  //   sumsq_clear != NULL : its kSumsqWords words are set to zero (the buffer the NEXT projection adds into);
  //   sumsq_in    != NULL : with norm_w, the sum of squares of x is the sum of words [0, K/128) of it, x is not re-read.
  unsigned long long* sumsq_out;
  unsigned long long* sumsq_clear;
  const unsigned long long* sumsq_in;
};
constexpr int kSumsqWords = 256;                     // words of a sum-of-squares buffer: projections of up to 32768 columns
constexpr float kSumsqUnit = 1073741824.f;           // 2^30
// One square on its way into a word: exact below 2^25 (|y| < 5792), capped there above and for NaN, so that the 128
// squares of a column tile can never wrap the word.
__device__ __forceinline__ unsigned long long sumsq_fixed(float y) {
  const float t = y * y;
  return t < 33554432.f ? (unsigned long long)(t * kSumsqUnit) : (1ull << 55);
}
// sum over the 64 lanes of a wavefront of a value below 2^22; every lane gets the result
__device__ __forceinline__ unsigned int wave_sum_all_u32(unsigned int v) {
#define ART_DPP_ADD(ctrl) v += (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, ctrl, 0xf, 0xf, false)
  ART_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
  ART_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
  ART_DPP_ADD(0x141);   // row_half_mirror
  ART_DPP_ADD(0x140);   // row_mirror
#undef ART_DPP_ADD
  return ((unsigned int)__builtin_amdgcn_readlane((int)v, 0) + (unsigned int)__builtin_amdgcn_readlane((int)v, 16)) +
         ((unsigned int)__builtin_amdgcn_readlane((int)v, 32) + (unsigned int)__builtin_amdgcn_readlane((int)v, 48));
}

// The register allocator is told that four wavefronts per SIMD are plenty (a launch has three): with the default
// target of eight it postpones two of the eight weight loads until registers free up, a second memory round trip.
template <int M, int MODE, int R, int W>   // MODE 0: plain product, 1: RMSNorm of x fused, 2: x = SwiGLU(gate | up) fused, 3: x = merged split attention,
                                           // 4: RMSNorm of x fused, its sum of squares handed in (sumsq_in)
__global__ __launch_bounds__(64 * W) __attribute__((amdgpu_waves_per_eu(1, 4))) void gemv_w4a16_kernel(
    const _Float16* __restrict__ x, const unsigned char* __restrict__ qweight, const _Float16* __restrict__ scales,
    const unsigned char* __restrict__ qzeros, _Float16* __restrict__ y, int K, int N, int splits,
    unsigned long long* __restrict__ slots, Magic magic, Fused fused) {
  static_assert(R == 8 || (R == 4 && MODE == 0), "the fused prologues are written for 8 rows per lane");
  static_assert(MODE != 4 || W == 4, "the handed-in sum of squares comes with four wavefronts");
  static_assert(W == 4 || W == 8, "four or eight wavefronts per block");
  constexpr int kThreads = 64 * W, KL = kThreads / CL;  // k lanes per block: 32 or 64
  constexpr int kRowsPerBlock = KL * R;                 // packed rows per block: 256 (512 values of k) at R = 8, W = 4
  __shared__ __align__(16) float part[M][W][CT];        // per wavefront: scaled sums of the tile's columns
  __shared__ float s_ss[W];
  __shared__ __align__(16) unsigned int s_x[KL][CL];    // SwiGLU input, one fp16 pair per lane

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cl = tid % CL, kl = tid / CL;
  const int tile = blockIdx.x, split = blockIdx.y;
  const int n0 = tile * CT + cl * 16;
  const int rows = K >> 1;
  const int r0 = split * kRowsPerBlock + kl * R;          // first packed row of this lane
  const bool k_ok = r0 < rows;                            // rows % 64 == 0, so a lane is all in or all out
  // Lanes past the edge (last K-split when K % 512 != 0, last tile when N % 128 != 0) read a valid
  // patch instead of branching; their x is zeroed / their columns are never written.
  const int r0c = k_ok ? r0 : 0;
  const int n0c = (n0 < N) ? n0 : 0;

  // ---- fused RMSNorm, part 1: the loads for the sum of squares go out BEFORE the weight loads.  Loads
  // return in order, so these can be consumed (and the block-wide reduction done) while the weights are
  // still in flight; issued after the weights they would wait for the whole stream.
  constexpr bool norm = (M == 1) && (MODE == 1 || MODE == 4);      // x is normalised
  constexpr bool norm_own = (M == 1) && (MODE == 1);                // ... with a sum of squares computed here
  constexpr int kSq = 512 / kThreads;                     // 16-byte chunks of x per thread that cover K = 4096
  u32x4 sq[kSq];
  unsigned long long ss_word = 0;
  if constexpr (MODE == 4) {                              // one word per lane: K / 128 <= 64
    if (lane < (K >> 7)) ss_word = fused.sumsq_in[lane];
  }
  if (M == 1 && fused.sumsq_clear != nullptr && blockIdx.x == 0 && blockIdx.y == 0 && tid < kSumsqWords) fused.sumsq_clear[tid] = 0ull;
  if constexpr (norm_own) {
#pragma unroll
    for (int i = 0; i < kSq; ++i) {
      const int c = tid + i * kThreads;
      sq[i] = (c < (K >> 3)) ? reinterpret_cast<const u32x4*>(x)[c] : u32x4{0, 0, 0, 0};
    }
  }

  // ---- fused SwiGLU, part 1: the column lanes of a k lane share the same 16 values of x, so each
  // computes one pair; its two loads also go out ahead of the weight stream.
  constexpr bool swiglu = (M == 1) && (MODE == 2);
  unsigned int gpair = 0, upair = 0;
  if constexpr (swiglu) {
    const int k = 2 * r0c + 2 * cl;
    gpair = *reinterpret_cast<const unsigned int*>(fused.gate_up + k);
    upair = *reinterpret_cast<const unsigned int*>(fused.gate_up + K + k);
  }

  // ---- fused attention merge, part 1: x is the output of a decode attention that ran as `att_parts` blocks per
  // head and left, per (head, part), 128 unnormalised sums, the running maximum and the running sum of
  // exp.  As with SwiGLU each column lane produces one pair of the k lane's 16 values.
  constexpr bool attn = (M == 1) && (MODE == 3);
  constexpr int kMaxParts = art::kMaxAttnParts, kPartStride = 132;         // record layout of the attention kernel
  f32x2 pacc[kMaxParts], pml[kMaxParts];
  if constexpr (attn) {
    const int k = 2 * r0c + 2 * cl, head = k >> 7, d = k & 127;
    const float* rec = fused.att_partial + (size_t)head * fused.att_parts * kPartStride;
#pragma unroll
    for (int p = 0; p < kMaxParts; ++p) {
      const int pc = p < fused.att_parts ? p : 0;         // unused parts re-read part 0 and get weight 0 below
      pacc[p] = *reinterpret_cast<const f32x2*>(rec + pc * kPartStride + d);
      pml[p] = *reinterpret_cast<const f32x2*>(rec + pc * kPartStride + 128);
    }
  }

  // ---- every other global load of this lane: x first (small, returns first), then the whole weight patch, then the
  // scale and zero point of the two columns this lane holds after the reduce-scatter
  u32x4 xv[M][R / 4];                                     // 2 R halves of x per row of x
#pragma unroll
  for (int m = 0; m < M; ++m) {
    if (swiglu || attn) continue;
    const u32x4* xp = reinterpret_cast<const u32x4*>(x + (size_t)m * K + 2 * r0c);
#pragma unroll
    for (int i = 0; i < R / 4; ++i) xv[m][i] = xp[i];
  }
  // fused residual add: the first wavefront finishes the tile's columns, two per lane; their residual values are
  // fetched now, not behind the returning atomics at the very end of the block, where the round trip would be exposed.
  // (y may be the residual itself: only the block that arrives last at a column writes it, after every block of the
  // tile has issued its atomics, i.e. after every one of these loads has completed.)
  half2_t res2 = {(_Float16)0, (_Float16)0};
  if (M == 1 && fused.residual != nullptr && tid < 64) {
    const int rc = tile * CT + 2 * tid;
    if (rc < N) res2 = *reinterpret_cast<const half2_t*>(fused.residual + rc);
  }
  // fused RMSNorm: the norm weights of this lane's slice of x go out ahead of the weight stream too - loads return in
  // order, so behind it they would hold the first multiply-accumulate back until the whole patch has arrived
  u32x4 n0v = {0, 0, 0, 0}, n1v = {0, 0, 0, 0};
  if constexpr (norm) {
    const u32x4* np = reinterpret_cast<const u32x4*>(fused.norm_w + 2 * r0c);
    n0v = np[0];
    n1v = np[1];
  }
  u32x4 w[R];
  {
    const unsigned char* wp = qweight + (size_t)r0c * N + n0c;
#pragma unroll
    // streamed once, never reused: the non-temporal hint measured 1-3 % faster on all four benchmark shapes
    for (int i = 0; i < R; ++i) w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + (size_t)i * N));
  }
  const int pc = cl * 16 + 2 * (lane >> 3);               // column pair of this lane inside the tile (even)
  const int pcol = tile * CT + pc;
  const int pcolc = pcol < N ? pcol : 0;
  const int groups = K >> 7;
  const int g = (split * kRowsPerBlock * 2 + wave * 16 * R) >> 7;      // the wavefront's quantisation group
  const int gc = g < groups ? g : groups - 1;             // a group past the edge has x = 0: it contributes 0 * scale
  const unsigned int sc2 = *reinterpret_cast<const unsigned int*>(scales + (size_t)gc * N + pcolc);
  const unsigned char zb = qzeros[(size_t)gc * (N >> 1) + (pcolc >> 1)];
  __builtin_amdgcn_sched_barrier(0);                      // nothing below may move above the loads, no load below them
  if constexpr (swiglu || attn) {       // part 2: pair -> LDS -> all 16 values of the k lane (same wavefront: no block barrier needed)
    half2_t o;
    if (swiglu) {
      const half2_t gt = as_h2(gpair), u = as_h2(upair);
      const float g0f = (float)gt.x, g1f = (float)gt.y;
      o = half2_t{(_Float16)(g0f / (1.0f + expf(0.0f - g0f)) * (float)u.x), (_Float16)(g1f / (1.0f + expf(0.0f - g1f)) * (float)u.y)};
    } else {                  // softmax merge: out = sum_p e^(m_p - M) acc_p / sum_p e^(m_p - M) l_p, rounded once to fp16
      float mm = -INFINITY;
#pragma unroll
      for (int p = 0; p < kMaxParts; ++p)
        if (p < fused.att_parts) mm = fmaxf(mm, pml[p][0]);
      float n0f = 0.f, n1f = 0.f, den = 0.f;
#pragma unroll
      for (int p = 0; p < kMaxParts; ++p) {
        const float wgt = (p < fused.att_parts && pml[p][0] != -INFINITY) ? __expf(pml[p][0] - mm) : 0.f;
        n0f = fmaf(pacc[p][0], wgt, n0f);
        n1f = fmaf(pacc[p][1], wgt, n1f);
        den = fmaf(pml[p][1], wgt, den);
      }
      o = half2_t{(_Float16)(n0f / den), (_Float16)(n1f / den)};
    }
    s_x[kl][cl] = __builtin_bit_cast(unsigned int, o);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    xv[0][0] = *reinterpret_cast<const u32x4*>(&s_x[kl][0]);
    xv[0][1] = *reinterpret_cast<const u32x4*>(&s_x[kl][4]);
  }
  if (!k_ok) {
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int i = 0; i < R / 4; ++i) xv[m][i] = u32x4{0, 0, 0, 0};
  }

  // ---- fused RMSNorm, part 2 (while the weight loads are in flight): sum of squares over all of x.
  // Every block recomputes it from the 2*K bytes of x (served by L2) rather than waiting for another kernel.
  if constexpr (norm) {
    float ss_all;
    if constexpr (MODE == 4) {
      // words below 2^62 each: split at 2^32 so that both parts convert exactly enough (24 bits each) and sum in a fixed order
      ss_all = wave_sum_all((float)(unsigned int)(ss_word >> 32) * 4294967296.f + (float)(unsigned int)ss_word) * (1.f / kSumsqUnit);
    } else {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kSq; ++i) {
      const unsigned int wds[4] = {sq[i][0], sq[i][1], sq[i][2], sq[i][3]};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half2_t h = as_h2(wds[j]);
        ss = fmaf((float)h.x, (float)h.x, ss);
        ss = fmaf((float)h.y, (float)h.y, ss);
      }
    }
    for (int c = tid + kSq * kThreads; c < (K >> 3); c += kThreads) {      // K > 4096
      const u32x4 v = reinterpret_cast<const u32x4*>(x)[c];
      const unsigned int wds[4] = {v[0], v[1], v[2], v[3]};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half2_t h = as_h2(wds[j]);
        ss = fmaf((float)h.x, (float)h.x, ss);
        ss = fmaf((float)h.y, (float)h.y, ss);
      }
    }
    ss = wave_sum_all(ss);
    if (lane == 0) s_ss[wave] = ss;
    art_lds_barrier();      // LDS only: the weight loads issued above stay in flight
    ss_all = (s_ss[0] + s_ss[1]) + (s_ss[2] + s_ss[3]);
    if constexpr (W == 8) ss_all += (s_ss[4] + s_ss[5]) + (s_ss[6] + s_ss[7]);
    }
    const float r = 1.0f / sqrtf(ss_all * fused.inv_n + fused.eps);
    const unsigned int nw[8] = {n0v[0], n0v[1], n0v[2], n0v[3], n1v[0], n1v[1], n1v[2], n1v[3]};
    const unsigned int xw[8] = {xv[0][0][0], xv[0][0][1], xv[0][0][2], xv[0][0][3], xv[0][1][0], xv[0][1][1], xv[0][1][2], xv[0][1][3]};
    unsigned int out[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const half2_t xh = as_h2(xw[i]), wh = as_h2(nw[i]);
      const half2_t o = {(_Float16)((float)xh.x * r * (float)wh.x), (_Float16)((float)xh.y * r * (float)wh.y)};
      out[i] = __builtin_bit_cast(unsigned int, o);
    }
    xv[0][0] = u32x4{out[0], out[1], out[2], out[3]};
    xv[0][1] = u32x4{out[4], out[5], out[6], out[7]};
  }

  // ---- multiply-accumulate
  float acc[M][16], se[M], so[M];
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
      // rows i, i+1 hold k = 2i, 2i+1 | 2i+2, 2i+3; x words (x[2i],x[2i+1]) and (x[2i+2],x[2i+3])
      const unsigned int x0 = xv[m][i / 4][i % 4], x1 = xv[m][i / 4][i % 4 + 1];
      const half2_t xe = as_h2(__builtin_amdgcn_perm(x1, x0, 0x05040100u));   // (x[2i],   x[2i+2])
      const half2_t xo = as_h2(__builtin_amdgcn_perm(x1, x0, 0x07060302u));   // (x[2i+1], x[2i+3])
      se[m] = __builtin_amdgcn_fdot2(xe, ones, se[m], false);
      so[m] = __builtin_amdgcn_fdot2(xo, ones, so[m], false);
#pragma unroll
      for (int j = 0; j < 4; ++j) mac_word_pair(w[i][j], w[i + 1][j], xe, xo, &acc[m][4 * j], magic);
    }
  }

  // ---- the 8 k lanes of the wavefront meet by reduce-scatter (lane bits 5, 4, 3): afterwards this lane holds the
  // group's sums of columns pc and pc + 1; the x-only terms of a group are the same for every column
  const half2_t s2 = as_h2(sc2);
  const float z0 = (float)(zb & 15), z1 = (float)(zb >> 4);
  const bool upper8 = (lane & 8) != 0;
#pragma unroll
  for (int m = 0; m < M; ++m) {
    float v8[8], v4[4], v2[2];
#pragma unroll
    for (int j = 0; j < 8; ++j) v8[j] = swap32_add(acc[m][j], acc[m][8 + j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) v4[j] = swap16_add(v8[j], v8[4 + j]);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const float send = upper8 ? v4[j] : v4[2 + j], keep = upper8 ? v4[2 + j] : v4[j];
      v2[j] = keep + dpp_ror8(send);
    }
    const float se_g = sum_k_lanes_of_wave(se[m]), so_g = sum_k_lanes_of_wave(so[m]);
    const float a0 = 1024.f * se_g + 64.f * so_g, a1 = se_g + so_g;
    *reinterpret_cast<f32x2*>(&part[m][wave][pc]) = f32x2{(float)s2.x * (v2[0] - a0 - z0 * a1), (float)s2.y * (v2[1] - a0 - z1 * a1)};
  }
  __syncthreads();
  if (tid >= 64) return;
  const int c2 = 2 * tid, col = tile * CT + c2;           // the first wavefront finishes two columns per lane
  const bool hand_on = (M == 1) && fused.sumsq_out != nullptr;      // the whole wavefront stays for the sum of squares
  if (col >= N && !hand_on) return;
  unsigned long long sq_mine = 0;                         // squares of the outputs this lane has finished

  float r[M][2];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const f32x2 p0 = *reinterpret_cast<const f32x2*>(&part[m][0][c2]), p1 = *reinterpret_cast<const f32x2*>(&part[m][1][c2]);
    const f32x2 p2 = *reinterpret_cast<const f32x2*>(&part[m][2][c2]), p3 = *reinterpret_cast<const f32x2*>(&part[m][3][c2]);
    r[m][0] = (p0[0] + p1[0]) + (p2[0] + p3[0]);
    r[m][1] = (p0[1] + p1[1]) + (p2[1] + p3[1]);
    if constexpr (W == 8) {
      const f32x2 p4 = *reinterpret_cast<const f32x2*>(&part[m][4][c2]), p5 = *reinterpret_cast<const f32x2*>(&part[m][5][c2]);
      const f32x2 p6 = *reinterpret_cast<const f32x2*>(&part[m][6][c2]), p7 = *reinterpret_cast<const f32x2*>(&part[m][7][c2]);
      r[m][0] += (p4[0] + p5[0]) + (p6[0] + p7[0]);
      r[m][1] += (p4[1] + p5[1]) + (p6[1] + p7[1]);
    }
  }
  if (col < N) {
    if (splits == 1) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        half2_t o = {(_Float16)r[m][0], (_Float16)r[m][1]};
        if (M == 1 && fused.residual != nullptr) o = half2_t{(_Float16)((float)o.x + (float)res2.x), (_Float16)((float)o.y + (float)res2.y)};
        *reinterpret_cast<half2_t*>(y + (size_t)m * N + col) = o;
        if (hand_on) sq_mine = sumsq_fixed((float)o.x) + sumsq_fixed((float)o.y);
      }
    } else {
      // returning atomics, one per (row, column): [arrival count : 8][fixed-point sum : 56].  All of them go out
      // before the first result is looked at, so the lane pays one round trip.
      long long mine[M][2], old[M][2];
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < 2; ++j) mine[m][j] = (1LL << 56) + to_fixed(r[m][j], splits);
      // (pinned: left alone, the scheduler moves the first use of one atomic's result - and with it the wait for
      // that result - in front of the next atomic, and the lane pays one round trip per atomic)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          old[m][j] = (long long)__hip_atomic_fetch_add(slots + (size_t)m * N + col + j, (unsigned long long)mine[m][j], __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (((old[m][j] + (1LL << 55)) >> 56) == (long long)(splits - 1)) {
            const long long total = old[m][j] + mine[m][j] - ((long long)splits << 56);
            _Float16 o = (_Float16)from_fixed(total);
            if (M == 1 && fused.residual != nullptr) o = (_Float16)((float)o + (float)(j == 0 ? res2.x : res2.y));
            y[(size_t)m * N + col + j] = o;
            slots[(size_t)m * N + col + j] = 0ull;            // ready for the next launch (stream order makes this visible)
            if (hand_on) sq_mine += sumsq_fixed((float)o);
          }
        }
    }
  }
  if (hand_on) {
    // Which block finishes a column depends on timing, the sum of the integers does not.  Three 21-bit limbs, each
    // summed over the wavefront (two squares per lane: below 2^28), one atomic per block that finished anything.
    const unsigned int l0 = wave_sum_all_u32((unsigned int)sq_mine & 0x1fffffu);
    const unsigned int l1 = wave_sum_all_u32((unsigned int)(sq_mine >> 21) & 0x1fffffu);
    const unsigned int l2 = wave_sum_all_u32((unsigned int)(sq_mine >> 42));
    const unsigned long long total = (unsigned long long)l0 + ((unsigned long long)l1 << 21) + ((unsigned long long)l2 << 42);
    if (tid == 0 && total != 0ull)
      __hip_atomic_fetch_add(fused.sumsq_out + tile, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Split-K accumulators of the entry point that allocates nothing (art_gemv_w4a16_noalloc): 64-bit slots, one per
// (row of x, column), in device memory that belongs to the code object itself.  Zero when the code object is loaded;
// every launch leaves the slots it used at zero again.  Each GPU has its own copy at its own address.
constexpr int kNoAllocSlots = 131072;                   // 1 MiB per GPU: M * N <= 131072
static __device__ __align__(256) unsigned long long scratch[kNoAllocSlots];
constexpr int kMaxDevices = 16;
unsigned long long* g_scratch_ptr[kMaxDevices];          // device address of `scratch` on each GPU (set by art_init)

template <int M>
int launch(const void* x, const void* qw, const void* sc, const void* qz, void* y, int K, int N, hipStream_t stream,
           Fused fused = Fused{nullptr, nullptr, nullptr, 0.f, 0.f, nullptr, 0, nullptr, nullptr, nullptr}, unsigned long long* slots = nullptr,
           int rows_per_lane = 8, int waves = 0) {
  const int rows = K / 2;
  const int tiles = (N + CT - 1) / CT;
  // Four wavefronts unless the caller asks for eight: halving the atomics did not pay on any shape of the decode
  // step (4096 x 22016: 13.5 -> 13.9 us, 4096 x 32000: 17.0 -> 17.6 us), the blocks' larger k range costs more.
  if (waves == 0) waves = 4;
  const int rows_per_block = 8 * waves * rows_per_lane;
  const int splits = (rows + rows_per_block - 1) / rows_per_block;
  ART_REQUIRE(splits <= 127, "art_gemv_w4a16: K too large (%d) for %d rows per lane", K, rows_per_lane);
  if (slots == nullptr) {         // the library's own workspace for this stream
    art::Workspace* wsp = art::workspace(stream);
    if (!wsp) return 1;
    ART_REQUIRE(art::kSlotOffset + (size_t)M * N * 8 <= art::kScratchOffset, "art_gemv_w4a16: N too large (%d)", N);
    slots = reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(wsp->base) + art::kSlotOffset);
  }
  const Magic magic{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  const dim3 grid(tiles, splits), block(64 * waves);
#define ART_GEMV_LAUNCH(MODE, R, W)                                                                                          \
  gemv_w4a16_kernel<M, MODE, R, W><<<grid, block, 0, stream>>>((const _Float16*)x, (const unsigned char*)qw, (const _Float16*)sc, \
                                                               (const unsigned char*)qz, (_Float16*)y, K, N, splits, slots, magic, fused)
  // the plain product is its own instantiation: it carries none of the fused prologues; rows of x beyond the first
  // and four rows per lane come with four wavefronts only
  if constexpr (M == 1) {
    if (waves == 8) {
      if (fused.norm_w != nullptr) ART_GEMV_LAUNCH(1, 8, 8);
      else if (fused.gate_up != nullptr) ART_GEMV_LAUNCH(2, 8, 8);
      else if (fused.att_partial != nullptr) ART_GEMV_LAUNCH(3, 8, 8);
      else if (rows_per_lane == 4) ART_GEMV_LAUNCH(0, 4, 8);
      else ART_GEMV_LAUNCH(0, 8, 8);
    } else {
      if (fused.norm_w != nullptr && fused.sumsq_in != nullptr) ART_GEMV_LAUNCH(4, 8, 4);
      else if (fused.norm_w != nullptr) ART_GEMV_LAUNCH(1, 8, 4);
      else if (fused.gate_up != nullptr) ART_GEMV_LAUNCH(2, 8, 4);
      else if (fused.att_partial != nullptr) ART_GEMV_LAUNCH(3, 8, 4);
      else if (rows_per_lane == 4) ART_GEMV_LAUNCH(0, 4, 4);
      else ART_GEMV_LAUNCH(0, 8, 4);
    }
  } else {
    if (rows_per_lane == 4) ART_GEMV_LAUNCH(0, 4, 4);
    else ART_GEMV_LAUNCH(0, 8, 4);
  }
#undef ART_GEMV_LAUNCH
  ART_LAUNCH_CHECK();
  return 0;
}

}  // namespace

extern "C" int art_gemv_w4a16(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                              void* y_dev, int M, int K, int N, void* stream) {
  return art_gemv_w4a16_tuned(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, M, K, N, 0, stream);
}

extern "C" int art_gemv_w4a16_tuned(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                    void* y_dev, int M, int K, int N, int k_per_block, void* stream) {
  ART_REQUIRE(k_per_block == 0 || k_per_block == 256 || k_per_block == 512 || k_per_block == 1024,
              "art_gemv_w4a16: k_per_block must be 0 (library's choice), 256, 512 or 1024 (got %d)", k_per_block);
  // 256: four rows per lane, four wavefronts; 512: eight rows, four wavefronts; 1024: eight rows, eight wavefronts
  const int rpl = k_per_block == 0 ? 0 : (k_per_block == 256 ? 4 : 8), waves = k_per_block == 0 ? 0 : (k_per_block == 1024 ? 8 : 4);
  return art_gemv_w4a16_knobs(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, M, K, N, rpl, waves, stream);
}

extern "C" int art_gemv_w4a16_knobs(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                    void* y_dev, int M, int K, int N, int rows_per_lane, int waves_per_block, void* stream) {
  ART_REQUIRE(rows_per_lane == 0 || rows_per_lane == 4 || rows_per_lane == 8, "art_gemv_w4a16: rows_per_lane must be 0 (library's choice), 4 or 8 (got %d)",
              rows_per_lane);
  ART_REQUIRE(waves_per_block == 0 || waves_per_block == 4 || waves_per_block == 8,
              "art_gemv_w4a16: waves_per_block must be 0 (library's choice), 4 or 8 (got %d)", waves_per_block);
  ART_REQUIRE(waves_per_block != 8 || M == 1, "art_gemv_w4a16: eight wavefronts per block are for M = 1 (got M = %d)", M);
  // The library's choice: eight rows per lane, except where that many-row blocks need more than one and a half rounds
  // of the chip (four blocks per compute unit at a time) - there blocks of half the rows fill the rounds better
  // (M = 1, 4096 x 32000: 16.2 us against 16.9 on MI355X; the narrower benchmark shapes lose 0.1 - 1 us with them).
  int rpl = rows_per_lane == 0 ? 8 : rows_per_lane;
  if (rows_per_lane == 0 && M == 1) {
    const long long blocks = (long long)((N + 127) / 128) * ((K + 511) / 512);
    if (blocks > 6LL * art::compute_units()) rpl = 4;
  }
  const int waves = waves_per_block;
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemv_w4a16: null pointer");
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemv_w4a16: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 16) == 0,
              "art_gemv_w4a16: x and qweight must be 16-byte aligned");
  ART_REQUIRE(((uintptr_t)y_dev % 4) == 0 && ((uintptr_t)scales_dev % 4) == 0, "art_gemv_w4a16: y and scales must be 4-byte aligned");
  ART_REQUIRE(M >= 1 && M <= 8, "art_gemv_w4a16: M must be in 1..8 (got %d); larger batches go through art_gemm_w4a16", M);
  // blocks of one column tile write y while blocks of other tiles still read x
  ART_REQUIRE(!art::overlaps(x_dev, (size_t)M * K * 2, y_dev, (size_t)M * N * 2), "art_gemv_w4a16: y must not overlap x");
  hipStream_t st = (hipStream_t)stream;
  int m = 0;
  while (m < M) {       // rows of x are handled up to four at a time
    const int step = (M - m >= 4) ? 4 : (M - m);
    const _Float16* xs = (const _Float16*)x_dev + (size_t)m * K;
    _Float16* ys = (_Float16*)y_dev + (size_t)m * N;
    const Fused none{nullptr, nullptr, nullptr, 0.f, 0.f, nullptr, 0, nullptr, nullptr, nullptr};
    int rc = step == 4 ? launch<4>(xs, qweight_dev, scales_dev, qzeros_dev, ys, K, N, st, none, nullptr, rpl, 4)
           : step == 3 ? launch<3>(xs, qweight_dev, scales_dev, qzeros_dev, ys, K, N, st, none, nullptr, rpl, 4)
           : step == 2 ? launch<2>(xs, qweight_dev, scales_dev, qzeros_dev, ys, K, N, st, none, nullptr, rpl, 4)
                       : launch<1>(xs, qweight_dev, scales_dev, qzeros_dev, ys, K, N, st, none, nullptr, rpl, waves);
    if (rc) return rc;
    m += step;
  }
  return 0;
}

// Called by art_init with `device` current: finds where this GPU keeps `scratch`.
int art::gemv_noalloc_setup(int device) {
  ART_REQUIRE(device >= 0 && device < kMaxDevices, "gemv_noalloc_setup: bad device %d", device);
  if (g_scratch_ptr[device] != nullptr) return 0;
  unsigned long long* ptr = nullptr;
  ART_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
  ART_REQUIRE(ptr != nullptr, "gemv_noalloc_setup: no device address for the scratch array");
  g_scratch_ptr[device] = ptr;
  return 0;
}

extern "C" int art_gemv_w4a16_noalloc(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                      void* y_dev, int M, int K, int N, void* stream) {
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemv_w4a16_noalloc: null pointer");
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemv_w4a16_noalloc: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 16) == 0,
              "art_gemv_w4a16_noalloc: x and qweight must be 16-byte aligned");
  ART_REQUIRE(((uintptr_t)y_dev % 4) == 0 && ((uintptr_t)scales_dev % 4) == 0, "art_gemv_w4a16_noalloc: y and scales must be 4-byte aligned");
  ART_REQUIRE(M >= 1 && M <= 4, "art_gemv_w4a16_noalloc: M must be in 1..4 (got %d)", M);
  ART_REQUIRE((long long)M * N <= kNoAllocSlots, "art_gemv_w4a16_noalloc: M * N = %lld exceeds the %d accumulators of the built-in scratch array",
              (long long)M * N, kNoAllocSlots);
  ART_REQUIRE(!art::overlaps(x_dev, (size_t)M * K * 2, y_dev, (size_t)M * N * 2), "art_gemv_w4a16_noalloc: y must not overlap x");
  int dev = 0;
  ART_HIP(hipGetDevice(&dev));
  ART_REQUIRE(dev >= 0 && dev < kMaxDevices && g_scratch_ptr[dev] != nullptr, "art_gemv_w4a16_noalloc: call art_init(%d) first", dev);
  unsigned long long* slots = g_scratch_ptr[dev];
  const Fused none{nullptr, nullptr, nullptr, 0.f, 0.f, nullptr, 0, nullptr, nullptr, nullptr};
  hipStream_t st = (hipStream_t)stream;
  return M == 4 ? launch<4>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st, none, slots)
       : M == 3 ? launch<3>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st, none, slots)
       : M == 2 ? launch<2>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st, none, slots)
                : launch<1>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, st, none, slots);
}

extern "C" int art_gemv_w4a16_fused(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                    void* y_dev, int K, int N, const void* norm_weight_dev, float eps, const void* residual_dev,
                                    int swiglu_input, void* stream) {
  return art_gemv_w4a16_fused_sumsq(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, norm_weight_dev, eps, residual_dev,
                                    swiglu_input, nullptr, nullptr, nullptr, stream);
}

namespace {
// the checks the two entry points with sum-of-squares buffers share
int check_sumsq(const char* who, const void* in, const void* out, const void* clear, int K, int N, const void* norm_w) {
  ART_REQUIRE(((uintptr_t)in % 8) == 0 && ((uintptr_t)out % 8) == 0 && ((uintptr_t)clear % 8) == 0,
              "%s: the sum-of-squares buffers must be 8-byte aligned", who);
  ART_REQUIRE(in == nullptr || (norm_w != nullptr && K <= 64 * 128),
              "%s: a handed-in sum of squares needs a norm weight and K <= 8192 (K=%d)", who, K);
  ART_REQUIRE(out == nullptr || N <= kSumsqWords * CT, "%s: a sum-of-squares buffer covers %d columns (N=%d)", who, kSumsqWords * CT, N);
  ART_REQUIRE(out == nullptr || out != clear, "%s: the buffer that is cleared cannot be the one that is added to", who);
  ART_REQUIRE(in == nullptr || (in != clear && in != out), "%s: the buffer that is read cannot be cleared or added to by the same call", who);
  return 0;
}
}  // namespace

extern "C" int art_gemv_w4a16_fused_sumsq(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                                          void* y_dev, int K, int N, const void* norm_weight_dev, float eps,
                                          const void* residual_dev, int swiglu_input, const void* sumsq_in_dev,
                                          void* sumsq_out_dev, void* sumsq_clear_dev, void* stream) {
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemv_w4a16_fused: null pointer");
  ART_REQUIRE(!(swiglu_input && norm_weight_dev), "art_gemv_w4a16_fused: SwiGLU input and RMSNorm cannot be combined");
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemv_w4a16_fused: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 16) == 0 && ((uintptr_t)norm_weight_dev % 16) == 0,
              "art_gemv_w4a16_fused: x, qweight and the norm weight must be 16-byte aligned");
  ART_REQUIRE(((uintptr_t)y_dev % 4) == 0 && ((uintptr_t)scales_dev % 4) == 0 && ((uintptr_t)residual_dev % 4) == 0,
              "art_gemv_w4a16_fused: y, scales and the residual must be 4-byte aligned");
  // blocks of one column tile write y while blocks of other tiles still read x: only the residual may alias y
  ART_REQUIRE(!art::overlaps(x_dev, (size_t)(swiglu_input ? 2 : 1) * K * 2, y_dev, (size_t)N * 2),
              "art_gemv_w4a16_fused: y must not overlap x (it may alias the residual)");
  if (check_sumsq("art_gemv_w4a16_fused_sumsq", sumsq_in_dev, sumsq_out_dev, sumsq_clear_dev, K, N, norm_weight_dev)) return 1;
  Fused f{(const _Float16*)norm_weight_dev, (const _Float16*)residual_dev, swiglu_input ? (const _Float16*)x_dev : nullptr,
          1.0f / (float)K, eps, nullptr, 0, (unsigned long long*)sumsq_out_dev, (unsigned long long*)sumsq_clear_dev,
          (const unsigned long long*)sumsq_in_dev};
  return launch<1>(x_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, (hipStream_t)stream, f);
}

extern "C" int art_gemv_w4a16_attn(const void* partial_dev, int parts, const void* qweight_dev, const void* scales_dev,
                                   const void* qzeros_dev, void* y_dev, int K, int N, const void* residual_dev, void* stream) {
  return art_gemv_w4a16_attn_sumsq(partial_dev, parts, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, residual_dev, nullptr, nullptr,
                                   stream);
}

extern "C" int art_gemv_w4a16_attn_sumsq(const void* partial_dev, int parts, const void* qweight_dev, const void* scales_dev,
                                         const void* qzeros_dev, void* y_dev, int K, int N, const void* residual_dev,
                                         void* sumsq_out_dev, void* sumsq_clear_dev, void* stream) {
  ART_REQUIRE(partial_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemv_w4a16_attn: null pointer");
  ART_REQUIRE(parts >= 2 && parts <= art::kMaxAttnParts, "art_gemv_w4a16_attn: parts must be in 2..%d (got %d)", art::kMaxAttnParts, parts);
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemv_w4a16_attn: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)partial_dev % 16) == 0,
              "art_gemv_w4a16_attn: partial records and qweight must be 16-byte aligned");
  ART_REQUIRE(((uintptr_t)y_dev % 4) == 0 && ((uintptr_t)scales_dev % 4) == 0 && ((uintptr_t)residual_dev % 4) == 0,
              "art_gemv_w4a16_attn: y, scales and the residual must be 4-byte aligned");
  ART_REQUIRE(!art::overlaps(partial_dev, (size_t)(K / 128) * parts * 132 * 4, y_dev, (size_t)N * 2),
              "art_gemv_w4a16_attn: y must not overlap the partial records");
  if (check_sumsq("art_gemv_w4a16_attn_sumsq", nullptr, sumsq_out_dev, sumsq_clear_dev, K, N, nullptr)) return 1;
  Fused f{nullptr, (const _Float16*)residual_dev, nullptr, 0.f, 0.f, (const float*)partial_dev, parts,
          (unsigned long long*)sumsq_out_dev, (unsigned long long*)sumsq_clear_dev, nullptr};
  return launch<1>(partial_dev, qweight_dev, scales_dev, qzeros_dev, y_dev, K, N, (hipStream_t)stream, f);
}
