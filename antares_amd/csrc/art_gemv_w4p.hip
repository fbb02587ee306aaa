// Weight-only int4 (group 128) GEMV for decode over a one-time repacked weight layout, gfx950.
//
//   y[n] = sum_k x[k] * (q[k,n] - z[k/128,n]) * s[k/128,n]         (fp32 accumulate, M = 1)
//
// The kernel of art_gemv_w4.hip reads the benchmark layout ([K/2, N] bytes): a 128-byte line of a row is 128
// columns wide, so the chip can only be filled by cutting K into slices, and the slices of a column have to meet
// through memory (one returning atomic per block and column).  The reference repacks its weights once when it loads
// them (samples/05_llama2_7b_int4.py:34-66); the same step here (art_w4_prepack) stores a tile of 16 columns x all
// of K contiguously, so that ONE block owns its columns over the whole of K: no K-splits, no atomics, no
// accumulators in memory, y stored directly.
//
// Packed form: N/16 tiles, each `chunks` = ceil(K/1024) records of kChunkBytes:
//   [0, 8192)     weights of 1024 values of k x 16 columns, in the order the wavefront that owns the record reads
//                 them: load i (0..7) of lane l is the 16 bytes at i*1024 + l*16, so every load instruction of a
//                 wavefront is one contiguous KiB.  Lane l works on quantisation group l % 8 of the record and on
//                 the 16 values of k from (l / 8) * 16 of that group; load i holds columns 2i and 2i+1 as four
//                 32-bit words (column 2i: k 0..7, k 8..15; column 2i+1 likewise).  Inside a word the nibbles lie
//                 in the order k0 k2 k4 k6 k1 k3 k5 k7, so that (w & 0x000F000F), (w & 0x00F000F0) and the same of
//                 w >> 8 are the pairs (k0,k1) (k2,k3) (k4,k5) (k6,k7): four v_bfi + four v_dot2 per word, no
//                 permutes, and x is used as it lies in memory;
//   [8192, 8448)  fp16 scales [8 groups][16 columns];
//   [8448, 8512)  zero points [8 groups][8 bytes], low nibble = even column;
//   [8512, 8576)  padding to whole 128-byte lines.
// Records past the end of K (K % 1024 != 0) hold zeros.
//
// A block is one wavefront per record (4 for K = 4096, 11 for K = 11008).  The 8 lanes of a group meet by the
// reduce-scatter of art_gemv_w4.hip (lane bits 5, 4, 3; afterwards a lane holds two columns of its group), apply
// scale and zero point, the 8 groups of the wavefront meet by three DPP steps and the wavefronts of the block in LDS.
// (For K of 2049 .. 4096 a second form further down lets a wavefront own four columns over all of K.)
// One tile per block: the kernel needs about 60 registers per lane, so up to eight blocks of a compute unit have their
// loads in flight while others multiply (blocks that walk several tiles with a second register set measured 10-25 %
// slower on every decode shape).
#include "art_common.h"

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kTileCols = 16;
constexpr int kChunkK = 1024;
constexpr int kScaleOff = 8192, kZeroOff = 8448, kChunkBytes = 8576;
constexpr int kMaxWaves = 16;                      // K <= 16384

__device__ __forceinline__ half2_t as_h2(unsigned int v) { return __builtin_bit_cast(half2_t, v); }

// Nibble -> fp16 constants as kernel arguments: with run-time values (w & m) | (~m & g) selects to one v_bfi_b32.
struct Magic {
  unsigned int mask_lo, mask_hi, bias_lo, bias_hi;   // 0x000F000F 0x00F000F0 0x64006400 0x54005400
};
__device__ __forceinline__ half2_t nib(unsigned int w, unsigned int mask, unsigned int bias) {
  return as_h2((w & mask) | (~mask & bias));
}

// One packed word (8 values of k of one column) times the matching four pairs of x.
__device__ __forceinline__ float mac_word(unsigned int w, const unsigned int* xw, float acc, const Magic& k) {
  const unsigned int ws = w >> 8;
  acc = __builtin_amdgcn_fdot2(nib(w, k.mask_lo, k.bias_lo), as_h2(xw[0]), acc, false);
  acc = __builtin_amdgcn_fdot2(nib(w, k.mask_hi, k.bias_hi), as_h2(xw[1]), acc, false);
  acc = __builtin_amdgcn_fdot2(nib(ws, k.mask_lo, k.bias_lo), as_h2(xw[2]), acc, false);
  acc = __builtin_amdgcn_fdot2(nib(ws, k.mask_hi, k.bias_hi), as_h2(xw[3]), acc, false);
  return acc;
}

#define ART_DPP_F(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xf, 0xf, false))

__device__ __forceinline__ float swap32_add(float a, float b) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b), false, false);
  return __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
}
__device__ __forceinline__ float swap16_add(float a, float b) {
  auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b), false, false);
  return __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
}
// Sum over the 8 lanes that share lane % 8 (lane bits 3, 4, 5); all of them get the sum.
__device__ __forceinline__ float sum_over_lane_bits_345(float v) {
  v += ART_DPP_F(v, 0x128);                      // row_ror:8 = lane ^ 8
  v = swap16_add(v, v);
  v = swap32_add(v, v);
  return v;
}
// Sum over the 8 lanes that share lane / 8 (lane bits 0, 1, 2); all of them get the sum.
__device__ __forceinline__ float sum_over_lane_bits_012(float v) {
  v += ART_DPP_F(v, 0xB1);                       // quad_perm [1,0,3,2]
  v += ART_DPP_F(v, 0x4E);                       // quad_perm [2,3,0,1]
  v += ART_DPP_F(v, 0x141);                      // row_half_mirror
  return v;
}
// Sum over the 64 lanes of a wavefront; every lane gets the result.
__device__ __forceinline__ float wave_sum_all(float v) {
  v = sum_over_lane_bits_012(v);
  v += ART_DPP_F(v, 0x140);                      // row_mirror
  const int b = __builtin_bit_cast(int, v);
  return (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
}

struct Args {
  const _Float16* x;
  const unsigned char* packed;
  _Float16* y;
  const _Float16* norm_w;        // NORM: x is replaced by fp16(x * rsqrt(sum(x^2) * inv_n + eps) * norm_w)
  const _Float16* residual;      // EPI 1: y = fp16(fp16(product) + residual)
  float inv_n, eps;
  int K, N, tiles;
  unsigned int tile_stride;      // bytes between tiles
};

// EPI 0: y[n] = fp16(product);  1: + residual;  2: columns 0..7 of a tile are a gate, 8..15 the matching up
// projection: y[tile * 8 + j] = fp16(silu(fp16(gate_j)) * fp16(up_j)) (line :171 of the sample; N/2 outputs).
template <bool NORM, int EPI>
__global__ __launch_bounds__(64 * kMaxWaves) void gemv_w4p_kernel(Args a, Magic magic) {
  __shared__ __align__(16) float part[kMaxWaves][kTileCols];     // per wavefront: scaled sums of the tile's columns
  __shared__ float s_ss[kMaxWaves];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
  const int gi = lane & 7, sb = lane >> 3;
  const int g = wave * 8 + gi;                              // quantisation group of this lane
  const bool k_ok = g < (a.K >> 7);                         // groups past the end of K: x = 0 (their weights are zeros too)
  const int kbase = (k_ok ? g : 0) * 128 + sb * 16;

  // ---- loads that do not depend on the tile: x and the norm weights of this lane's 16 values of k
  const u32x4* xp = reinterpret_cast<const u32x4*>(a.x + kbase);
  u32x4 xv0 = xp[0], xv1 = xp[1];
  u32x4 n0v = {0, 0, 0, 0}, n1v = {0, 0, 0, 0};
  if constexpr (NORM) {
    const u32x4* np = reinterpret_cast<const u32x4*>(a.norm_w + kbase);
    n0v = np[0];
    n1v = np[1];
  }

  const unsigned char* lane_base = a.packed + (size_t)wave * kChunkBytes;
  auto issue = [&](int tile, u32x4 (&w)[8], unsigned int& sc2, unsigned int& zb, _Float16& res) {
    const unsigned char* wp = lane_base + (size_t)tile * a.tile_stride;
    if constexpr (EPI == 1) res = a.residual[tile * kTileCols + (tid & 15)];      // fetched with the tile, not behind its reduction (by every lane: no divergent branch around a load)
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + i * 1024 + lane * 16));
    sc2 = __builtin_nontemporal_load(reinterpret_cast<const unsigned int*>(wp + kScaleOff + (gi * 16 + 2 * sb) * 2));
    zb = __builtin_nontemporal_load(wp + kZeroOff + gi * 8 + sb);
  };

  u32x4 wa[8];
  unsigned int sca, za;
  _Float16 resa = (_Float16)0;
  int tile = blockIdx.x;
  issue(tile, wa, sca, za, resa);
  __builtin_amdgcn_sched_barrier(0);                        // nothing below moves above the loads

  // ---- x of this lane, normalised if asked (while the weights are in flight)
  if (!k_ok) { xv0 = u32x4{0, 0, 0, 0}; xv1 = u32x4{0, 0, 0, 0}; }
  unsigned int xw[8] = {xv0[0], xv0[1], xv0[2], xv0[3], xv1[0], xv1[1], xv1[2], xv1[3]};
  if constexpr (NORM) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half2_t h = as_h2(xw[j]);
      ss = fmaf((float)h.x, (float)h.x, ss);
      ss = fmaf((float)h.y, (float)h.y, ss);
    }
    ss = wave_sum_all(ss);
    if (lane == 0) s_ss[wave] = ss;
    art_lds_barrier();                                      // LDS only: the weight loads stay in flight
    // the wavefronts' sums, one per lane of a row of 16, summed without a loop (a loop of run-time length between
    // the loads and their use makes the compiler wait for every load in flight)
    float ss_all = s_ss[lane & 15];
    ss_all = (lane & 15) < waves ? ss_all : 0.f;
    ss_all = sum_over_lane_bits_012(ss_all);
    ss_all += ART_DPP_F(ss_all, 0x140);                     // row_mirror: all 16 lanes of the row
    const float r = __builtin_amdgcn_rsqf(ss_all * a.inv_n + a.eps);       // v_rsq_f32: within 1 ulp of 1 / sqrt
    const unsigned int nw[8] = {n0v[0], n0v[1], n0v[2], n0v[3], n1v[0], n1v[1], n1v[2], n1v[3]};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half2_t xh = as_h2(xw[j]), wh = as_h2(nw[j]);
      // (x * r) * w in fp32, rounded once to fp16; written as fused multiply-adds with a zero addend so that each
      // product is one v_fma_mix instruction that reads the fp16 halves directly
      const half2_t o = {(_Float16)fmaf(fmaf((float)xh.x, r, 0.f), (float)wh.x, 0.f), (_Float16)fmaf(fmaf((float)xh.y, r, 0.f), (float)wh.y, 0.f)};
      xw[j] = __builtin_bit_cast(unsigned int, o);
    }
  }
  // the terms that leave with the zero point: 1024 * (x of the low-nibble pairs) + 64 * (x of the high-nibble pairs),
  // and sum(x), each over the 128 values of the group
  float a0, a1;
  {
    const half2_t ones = {(_Float16)1, (_Float16)1};
    float se = 0.f, so = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      se = __builtin_amdgcn_fdot2(as_h2(xw[j]), ones, se, false);
      so = __builtin_amdgcn_fdot2(as_h2(xw[j + 1]), ones, so, false);
    }
    const float se_g = sum_over_lane_bits_345(se), so_g = sum_over_lane_bits_345(so);
    a0 = 1024.f * se_g + 64.f * so_g;
    a1 = se_g + so_g;
  }
  const bool upper8 = (lane & 8) != 0;
  const int pc = 2 * sb;                                    // column pair this lane holds after the reduce-scatter

  auto finish = [&](int t, const u32x4 (&w)[8], unsigned int sc2, unsigned int zb, _Float16 res) {
    float acc[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[2 * i] = mac_word(w[i][1], xw + 4, mac_word(w[i][0], xw, 0.f, magic), magic);
      acc[2 * i + 1] = mac_word(w[i][3], xw + 4, mac_word(w[i][2], xw, 0.f, magic), magic);
    }
    float v8[8], v4[4], v2[2];
#pragma unroll
    for (int j = 0; j < 8; ++j) v8[j] = swap32_add(acc[j], acc[8 + j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) v4[j] = swap16_add(v8[j], v8[4 + j]);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const float send = upper8 ? v4[j] : v4[2 + j], keep = upper8 ? v4[2 + j] : v4[j];
      v2[j] = keep + ART_DPP_F(send, 0x128);
    }
    const half2_t s2 = as_h2(sc2);
    const float z0 = (float)(zb & 15), z1 = (float)(zb >> 4);
    float r0 = (float)s2.x * (v2[0] - a0 - z0 * a1), r1 = (float)s2.y * (v2[1] - a0 - z1 * a1);
    r0 = sum_over_lane_bits_012(r0);                        // the 8 groups of the wavefront
    r1 = sum_over_lane_bits_012(r1);
    if (gi == 0) *reinterpret_cast<f32x2*>(&part[wave][pc]) = f32x2{r0, r1};
    art_lds_barrier();
    if (EPI == 2 ? tid < 8 : tid < kTileCols) {
      float s = 0.f, u = 0.f;
#pragma unroll
      for (int w = 0; w < kMaxWaves; ++w) {                 // fixed length, unused wavefronts' slots read and dropped
        const float sv = part[w][tid], uv = EPI == 2 ? part[w][tid + 8] : 0.f;
        s += w < waves ? sv : 0.f;
        if (EPI == 2) u += w < waves ? uv : 0.f;
      }
      if constexpr (EPI == 2) {
        const float gf = (float)(_Float16)s, uf = (float)(_Float16)u;
        a.y[t * 8 + tid] = (_Float16)(gf / (1.0f + expf(0.0f - gf)) * uf);
      } else {
        const int n = t * kTileCols + tid;
        _Float16 o = (_Float16)s;
        if constexpr (EPI == 1) o = (_Float16)((float)o + (float)res);
        a.y[n] = o;
      }
    }
  };

  finish(tile, wa, sca, za, resa);
}

// Repack: one block per (tile, record); thread -> 32-bit words of the record.
__global__ __launch_bounds__(256) void w4_prepack_kernel(const unsigned char* __restrict__ qweight, const _Float16* __restrict__ scales,
                                                          const unsigned char* __restrict__ qzeros, unsigned char* __restrict__ packed,
                                                          int K, int N, unsigned int tile_stride) {
  const int tile = blockIdx.x, chunk = blockIdx.y, tid = threadIdx.x;
  const int groups = K >> 7;
  unsigned char* rec = packed + (size_t)tile * tile_stride + (size_t)chunk * kChunkBytes;
  for (int wi = tid; wi < 2048; wi += 256) {
    const int i = wi >> 8, l = (wi >> 2) & 63, j = wi & 3;
    const int col = 2 * i + (j >> 1), kh = j & 1;
    const int g = chunk * 8 + (l & 7);
    unsigned int word = 0;
    if (g < groups) {
      const int kb = g * 128 + (l >> 3) * 16 + kh * 8;       // first of the word's 8 values of k
      const unsigned char* src = qweight + (size_t)(kb >> 1) * N + tile * kTileCols + col;
      const unsigned int b0 = src[0], b1 = src[(size_t)N], b2 = src[(size_t)2 * N], b3 = src[(size_t)3 * N];
      word = (b0 & 15u) | ((b1 & 15u) << 4) | ((b2 & 15u) << 8) | ((b3 & 15u) << 12) |
             ((b0 >> 4) << 16) | ((b1 >> 4) << 20) | ((b2 >> 4) << 24) | ((b3 >> 4) << 28);
    }
    reinterpret_cast<unsigned int*>(rec)[wi] = word;        // i * 1024 + l * 16 + j * 4 == wi * 4
  }
  if (tid < 128) {                                          // 8 groups x 16 columns of scales
    const int g = chunk * 8 + (tid >> 4), c = tid & 15;
    reinterpret_cast<_Float16*>(rec + kScaleOff)[tid] = g < groups ? scales[(size_t)g * N + tile * kTileCols + c] : (_Float16)0;
  } else if (tid < 192) {                                   // 8 groups x 8 bytes of zero points
    const int t = tid - 128, g = chunk * 8 + (t >> 3), c = t & 7;
    rec[kZeroOff + t] = g < groups ? qzeros[(size_t)g * (N >> 1) + tile * (kTileCols / 2) + c] : (unsigned char)0;
  } else {
    rec[kZeroOff + 64 + (tid - 192)] = 0;                   // padding
  }
  // bytes between the last record of the tile and the next tile (the stride is rounded up to 256) are never read;
  // they are cleared so that the whole buffer is defined
  if (chunk == 0) {
    const unsigned int used = gridDim.y * kChunkBytes;
    for (unsigned int o = used + tid; o < tile_stride; o += 256) packed[(size_t)tile * tile_stride + o] = 0;
  }
}


// ---------------------------------------------------------------------------------------------------------------
// K of 2049 .. 4096 (the hidden size of the decode step): a wavefront owns FOUR columns over all of K, so the four
// wavefronts of a block never meet - no LDS meeting, no barrier behind the stream, every wavefront stores its own
// four results - and a block is launched with 256 threads whatever K is.  ("Column quads"; the general form above
// keeps 16 columns per wavefront and 1024 values of k.)
//
// Packed form: N/16 tiles of four records (wavefront w: columns 2w, 2w+1, 8+2w, 8+2w+1 of the tile - two from each
// half, so that with gate | up interleaved in blocks of 8 a wavefront holds matching gate and up columns):
//   [0, 8192)     lane l owns the 64 values of k from 64 l (quantisation group l / 2); load i (0..7) is the 16 bytes at
//                 i*1024 + l*16: the 8 values of k from 8i of those, one 32-bit word per column, nibbles in the order
//                 k0 k2 k4 k6 k1 k3 k5 k7 as above;
//   [8192, 8448)  fp16 scales, lane l: group l / 2, the wavefront's columns 2 (l % 2) and 2 (l % 2) + 1 - the two a lane
//                 holds once the two lanes of a group have met;
//   [8448, 8512)  zero points of the same two columns, one byte per lane;  [8512, 8576) padding.
// x goes through LDS once (thread t prepares x[16t .. 16t+15], normalised if asked, and the four threads of a lane's 64
// values leave the two sums that go with the 1024 / 64 offsets and the zero point); a lane reads its x from there
// while its weights are in flight.
constexpr int kQuadMaxK = 4096, kQuadRecords = 4, kXChunkBytes = 144;   // 64 values of x + 16 bytes: neighbouring chunks lie on different banks

__device__ __forceinline__ int quad_column(int wave, int c) { return (c >> 1) * 8 + 2 * wave + (c & 1); }

template <bool NORM, int EPI>
__global__ __launch_bounds__(256) void gemv_w4q_kernel(Args a, Magic magic) {
  __shared__ __align__(16) unsigned char xs[64 * kXChunkBytes];
  __shared__ __align__(8) float corr[64][2];                // per 64 values of k: 1024 * sum(low positions) + 64 * sum(high positions), sum(x)
  __shared__ float s_ss[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- x: thread t prepares x[16t .. 16t+15]; past the end of K it is zero (the weights there are zeros too)
  const bool k_ok = 16 * tid < a.K;
  const int k0 = k_ok ? 16 * tid : 0;
  const u32x4* xp = reinterpret_cast<const u32x4*>(a.x + k0);
  u32x4 xv0 = xp[0], xv1 = xp[1];
  u32x4 n0v = {0, 0, 0, 0}, n1v = {0, 0, 0, 0};
  if constexpr (NORM) {
    const u32x4* np = reinterpret_cast<const u32x4*>(a.norm_w + k0);
    n0v = np[0];
    n1v = np[1];
  }
  const int tile = blockIdx.x;
  const unsigned char* wp = a.packed + (size_t)tile * a.tile_stride + (size_t)wave * kChunkBytes;
  u32x4 w[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + i * 1024 + lane * 16));
  const unsigned int sc2 = __builtin_nontemporal_load(reinterpret_cast<const unsigned int*>(wp + kScaleOff + lane * 4));
  const unsigned int zb = __builtin_nontemporal_load(wp + kZeroOff + lane);
  // after the reductions lane l < 4 holds the wavefront's column 2 (l % 2) + (l / 2): its residual comes with the tile
  const int out_col = quad_column(wave, 2 * (lane & 1) + ((lane >> 1) & 1));
  // (every lane loads it - the column repeats every four lanes: a load inside a divergent branch makes the compiler
  // wait there for every load in flight)
  _Float16 res = (_Float16)0;
  if constexpr (EPI == 1) res = a.residual[tile * kTileCols + out_col];
  __builtin_amdgcn_sched_barrier(0);                        // nothing below moves above the loads

  if (!k_ok) { xv0 = u32x4{0, 0, 0, 0}; xv1 = u32x4{0, 0, 0, 0}; }
  unsigned int xw[8] = {xv0[0], xv0[1], xv0[2], xv0[3], xv1[0], xv1[1], xv1[2], xv1[3]};
  if constexpr (NORM) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half2_t h = as_h2(xw[j]);
      ss = fmaf((float)h.x, (float)h.x, ss);
      ss = fmaf((float)h.y, (float)h.y, ss);
    }
    ss = wave_sum_all(ss);
    if (lane == 0) s_ss[wave] = ss;
    art_lds_barrier();                                      // LDS only: the weight loads stay in flight
    const float r = __builtin_amdgcn_rsqf(((s_ss[0] + s_ss[1]) + (s_ss[2] + s_ss[3])) * a.inv_n + a.eps);
    const unsigned int nw[8] = {n0v[0], n0v[1], n0v[2], n0v[3], n1v[0], n1v[1], n1v[2], n1v[3]};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const half2_t xh = as_h2(xw[j]), wh = as_h2(nw[j]);
      const half2_t o = {(_Float16)fmaf(fmaf((float)xh.x, r, 0.f), (float)wh.x, 0.f), (_Float16)fmaf(fmaf((float)xh.y, r, 0.f), (float)wh.y, 0.f)};
      xw[j] = __builtin_bit_cast(unsigned int, o);
    }
  }
  {
    const half2_t ones = {(_Float16)1, (_Float16)1};
    float se = 0.f, so = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      se = __builtin_amdgcn_fdot2(as_h2(xw[j]), ones, se, false);
      so = __builtin_amdgcn_fdot2(as_h2(xw[j + 1]), ones, so, false);
    }
    se += ART_DPP_F(se, 0xB1); se += ART_DPP_F(se, 0x4E);  // the four threads of 64 values of k are a quad
    so += ART_DPP_F(so, 0xB1); so += ART_DPP_F(so, 0x4E);
    if ((tid & 3) == 0) *reinterpret_cast<f32x2*>(&corr[tid >> 2][0]) = f32x2{1024.f * se + 64.f * so, se + so};
    unsigned char* dst = xs + (tid >> 2) * kXChunkBytes + (tid & 3) * 32;
    *reinterpret_cast<u32x4*>(dst) = u32x4{xw[0], xw[1], xw[2], xw[3]};
    *reinterpret_cast<u32x4*>(dst + 16) = u32x4{xw[4], xw[5], xw[6], xw[7]};
  }
  art_lds_barrier();

  // ---- multiply: the lane's 64 values of k, 8 at a time as the loads arrive, against its x from LDS
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const unsigned char* xsrc = xs + lane * kXChunkBytes;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const u32x4 xq = *reinterpret_cast<const u32x4*>(xsrc + 16 * i);
    const unsigned int xo[4] = {xq[0], xq[1], xq[2], xq[3]};
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = mac_word(w[i][c], xo, acc[c], magic);
  }
  // ---- the two lanes of a group meet (lane bit 0): the even lane keeps columns 0, 1, the odd one 2, 3; so do their sums of x
  // (the two sums are copied out of the loaded register pair before they go through DPP: with the pair's second
  // half as a DPP source the compiler's DPP combiner picks the first half)
  float c0 = corr[lane][0], c1 = corr[lane][1];
  asm volatile("" : "+v"(c0), "+v"(c1));
  const bool odd = (lane & 1) != 0;
  const float v0 = (odd ? acc[2] : acc[0]) + ART_DPP_F(odd ? acc[0] : acc[2], 0xB1);
  const float v1 = (odd ? acc[3] : acc[1]) + ART_DPP_F(odd ? acc[1] : acc[3], 0xB1);
  const float a0 = c0 + ART_DPP_F(c0, 0xB1), a1 = c1 + ART_DPP_F(c1, 0xB1);
  const half2_t s2 = as_h2(sc2);
  const float z0 = (float)(zb & 15), z1 = (float)(zb >> 4);
  const float r0 = (float)s2.x * (v0 - a0 - z0 * a1), r1 = (float)s2.y * (v1 - a0 - z1 * a1);
  // ---- the 32 groups meet: lane bit 1 splits the two columns, bits 2..5 are summed (rotations inside a row of 16
  // lanes, swaps between rows); lane l < 4 then holds column 2 (l % 2) + (l / 2) of the wavefront
  const bool b1 = (lane & 2) != 0;
  float r = (b1 ? r1 : r0) + ART_DPP_F(b1 ? r0 : r1, 0x4E);
  r += ART_DPP_F(r, 0x124);                                 // row_ror:4
  r += ART_DPP_F(r, 0x128);                                 // row_ror:8
  r = swap16_add(r, r);
  r = swap32_add(r, r);
  if constexpr (EPI == 2) {
    // the wavefront's columns are gate 2w, gate 2w+1, up 2w, up 2w+1 of the tile: the up value sits in the neighbouring lane
    const float up = ART_DPP_F(r, 0xB1);
    if (lane < 4 && !odd) {
      const float gf = (float)(_Float16)r, uf = (float)(_Float16)up;
      a.y[tile * 8 + 2 * wave + (lane >> 1)] = (_Float16)(gf / (1.0f + expf(0.0f - gf)) * uf);
    }
  } else if (lane < 4) {
    _Float16 o = (_Float16)r;
    if constexpr (EPI == 1) o = (_Float16)((float)o + (float)res);
    a.y[tile * kTileCols + out_col] = o;
  }
}

// Repack for the column-quad form: one block per (tile, wavefront record).
__global__ __launch_bounds__(256) void w4_prepack_quad_kernel(const unsigned char* __restrict__ qweight, const _Float16* __restrict__ scales,
                                                               const unsigned char* __restrict__ qzeros, unsigned char* __restrict__ packed,
                                                               int K, int N, unsigned int tile_stride) {
  const int tile = blockIdx.x, wave = blockIdx.y, tid = threadIdx.x;
  const int groups = K >> 7;
  unsigned char* rec = packed + (size_t)tile * tile_stride + (size_t)wave * kChunkBytes;
  for (int wi = tid; wi < 2048; wi += 256) {
    const int i = wi >> 8, l = (wi >> 2) & 63, c = wi & 3;
    const int kb = 64 * l + 8 * i;                          // first of the word's 8 values of k
    unsigned int word = 0;
    if ((kb >> 7) < groups) {
      const unsigned char* src = qweight + (size_t)(kb >> 1) * N + tile * kTileCols + quad_column(wave, c);
      const unsigned int b0 = src[0], b1 = src[(size_t)N], b2 = src[(size_t)2 * N], b3 = src[(size_t)3 * N];
      word = (b0 & 15u) | ((b1 & 15u) << 4) | ((b2 & 15u) << 8) | ((b3 & 15u) << 12) |
             ((b0 >> 4) << 16) | ((b1 >> 4) << 20) | ((b2 >> 4) << 24) | ((b3 >> 4) << 28);
    }
    reinterpret_cast<unsigned int*>(rec)[wi] = word;
  }
  if (tid < 64) {                                           // lane tid: group tid / 2, the two columns it keeps
    const int g = tid >> 1;
    _Float16 s0 = (_Float16)0, s1 = (_Float16)0;
    unsigned int z = 0;
    if (g < groups) {
      const int c0 = tile * kTileCols + quad_column(wave, 2 * (tid & 1)), c1 = c0 + 1;
      s0 = scales[(size_t)g * N + c0];
      s1 = scales[(size_t)g * N + c1];
      const unsigned int zbyte = qzeros[(size_t)g * (N >> 1) + (c0 >> 1)];      // c0 is even: both columns in one byte
      z = zbyte;
    }
    reinterpret_cast<_Float16*>(rec + kScaleOff)[2 * tid] = s0;
    reinterpret_cast<_Float16*>(rec + kScaleOff)[2 * tid + 1] = s1;
    rec[kZeroOff + tid] = (unsigned char)z;
  } else if (tid < 128) {
    rec[kZeroOff + tid] = 0;                                // padding
  }
  if (wave == 0) {
    const unsigned int used = kQuadRecords * kChunkBytes;
    for (unsigned int o = used + tid; o < tile_stride; o += 256) packed[(size_t)tile * tile_stride + o] = 0;
  }
}

inline bool quad_form(int K) { return K > kQuadMaxK / 2 && K <= kQuadMaxK; }
inline int chunks_of(int K) { return (K + kChunkK - 1) / kChunkK; }
inline int records_of(int K) { return quad_form(K) ? kQuadRecords : chunks_of(K); }
inline size_t tile_stride_of(int K) { return (((size_t)records_of(K) * kChunkBytes) + 255) & ~(size_t)255; }

int check_shape(const char* who, int K, int N) {
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "%s: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", who, K, N);
  ART_REQUIRE(K <= kMaxWaves * kChunkK, "%s: K = %d exceeds %d", who, K, kMaxWaves * kChunkK);
  ART_REQUIRE((size_t)(N / kTileCols) * tile_stride_of(K) < ((size_t)1 << 32) * 64, "%s: matrix too large", who);
  return 0;
}

}  // namespace

extern "C" size_t art_w4_prepack_bytes(int K, int N) {
  if (K <= 0 || N <= 0 || K % 128 != 0 || N % 16 != 0 || K > kMaxWaves * kChunkK) return 0;
  return (size_t)(N / kTileCols) * tile_stride_of(K);
}

extern "C" int art_w4_prepack(const void* qweight_dev, const void* scales_dev, const void* qzeros_dev, void* packed_dev, int K, int N,
                              void* stream) {
  ART_REQUIRE(qweight_dev && scales_dev && qzeros_dev && packed_dev, "art_w4_prepack: null pointer");
  if (check_shape("art_w4_prepack", K, N)) return 1;
  ART_REQUIRE(((uintptr_t)packed_dev % 256) == 0, "art_w4_prepack: the packed buffer must be 256-byte aligned");
  ART_REQUIRE(((uintptr_t)scales_dev % 2) == 0, "art_w4_prepack: scales must be 2-byte aligned");
  const size_t stride = tile_stride_of(K);
  const size_t bytes = (size_t)(N / kTileCols) * stride;
  ART_REQUIRE(!art::overlaps(packed_dev, bytes, qweight_dev, (size_t)(K / 2) * N) && !art::overlaps(packed_dev, bytes, scales_dev, (size_t)(K / 128) * N * 2) &&
                  !art::overlaps(packed_dev, bytes, qzeros_dev, (size_t)(K / 128) * (N / 2)),
              "art_w4_prepack: the packed buffer must not overlap the inputs");
  ART_REQUIRE(stride <= 0xffffffffu, "art_w4_prepack: K too large");
  const dim3 grid(N / kTileCols, records_of(K));
  if (quad_form(K))
    w4_prepack_quad_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                                 (const unsigned char*)qzeros_dev, (unsigned char*)packed_dev, K, N, (unsigned int)stride);
  else
  w4_prepack_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const unsigned char*)qweight_dev, (const _Float16*)scales_dev,
                                                          (const unsigned char*)qzeros_dev, (unsigned char*)packed_dev, K, N, (unsigned int)stride);
  ART_LAUNCH_CHECK();
  return 0;
}

extern "C" int art_gemv_w4p(const void* x_dev, const void* packed_dev, void* y_dev, int K, int N, const void* norm_weight_dev, float eps,
                            const void* residual_dev, int swiglu_out, void* stream) {
  ART_REQUIRE(x_dev && packed_dev && y_dev, "art_gemv_w4p: null pointer");
  if (check_shape("art_gemv_w4p", K, N)) return 1;
  ART_REQUIRE(!(swiglu_out && residual_dev), "art_gemv_w4p: the SwiGLU output and a residual cannot be combined");
  ART_REQUIRE(((uintptr_t)packed_dev % 256) == 0, "art_gemv_w4p: the packed weights must be 256-byte aligned");
  ART_REQUIRE(((uintptr_t)x_dev % 16) == 0 && ((uintptr_t)norm_weight_dev % 16) == 0, "art_gemv_w4p: x and the norm weight must be 16-byte aligned");
  ART_REQUIRE(((uintptr_t)y_dev % 2) == 0 && ((uintptr_t)residual_dev % 2) == 0, "art_gemv_w4p: y and the residual must be 2-byte aligned");
  const size_t y_bytes = (size_t)(swiglu_out ? N / 2 : N) * 2;
  // blocks of one tile write y while blocks of other tiles still read x: only the residual may alias y
  ART_REQUIRE(!art::overlaps(x_dev, (size_t)K * 2, y_dev, y_bytes), "art_gemv_w4p: y must not overlap x (it may alias the residual)");
  const int tiles = N / kTileCols, waves = chunks_of(K);
  const int blocks = tiles;
  Args a{(const _Float16*)x_dev, (const unsigned char*)packed_dev, (_Float16*)y_dev, (const _Float16*)norm_weight_dev,
         (const _Float16*)residual_dev, 1.0f / (float)K, eps, K, N, tiles, (unsigned int)tile_stride_of(K)};
  const Magic magic{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  const dim3 grid(blocks), block(64 * waves);
  hipStream_t st = (hipStream_t)stream;
#define ART_W4P_LAUNCH(NORM, EPI)                                                          \
  do {                                                                                    \
    if (quad_form(K)) gemv_w4q_kernel<NORM, EPI><<<grid, dim3(256), 0, st>>>(a, magic);    \
    else gemv_w4p_kernel<NORM, EPI><<<grid, block, 0, st>>>(a, magic);                     \
  } while (0)
  if (norm_weight_dev != nullptr) {
    if (swiglu_out) ART_W4P_LAUNCH(true, 2);
    else if (residual_dev != nullptr) ART_W4P_LAUNCH(true, 1);
    else ART_W4P_LAUNCH(true, 0);
  } else {
    if (swiglu_out) ART_W4P_LAUNCH(false, 2);
    else if (residual_dev != nullptr) ART_W4P_LAUNCH(false, 1);
    else ART_W4P_LAUNCH(false, 0);
  }
#undef ART_W4P_LAUNCH
  ART_LAUNCH_CHECK();
  return 0;
}
