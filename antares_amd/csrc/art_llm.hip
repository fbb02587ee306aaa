// Llama decode operators for gfx950: RMSNorm, rotary position embedding
// (rotate-half and interleaved), single-query attention with softmax.
//
// These are the built-in operators the reference's samples call as
// autort.ops.rmsnorm_f32/_f16, rotary_f32/_f16, rotate_f32, attention_f32/_f16
// (samples/05_llama2_7b_int4.py:128-131,157-158,165;
//  samples/04_llama2_7b_fp16.py:83,96-97,103; samples/03_llama_tiny.py:66-70).
// Their source is not part of the reference tree; the semantics implemented
// here are stated at each entry point and are the ones the call sites imply
// (samples/03_llama_tiny.py:94-99 spells the attention in torch).
//
// All three are bound by memory latency / bandwidth, not arithmetic: one pass
// over the data, 128-bit loads, fp32 math, wavefront reductions through DPP.
#include <hip/hip_fp16.h>

#include <type_traits>

#include "art_common.h"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <class T> __device__ __forceinline__ float ld(const T* p, size_t i) { return (float)p[i]; }
template <class T> __device__ __forceinline__ void st(T* p, size_t i, float v) { p[i] = (T)v; }

// sum over the 64 lanes of a wavefront; every lane gets the result (fixed order)
__device__ __forceinline__ float wave_sum(float v) {
#define ART_DPP_ADD(ctrl) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false))
  ART_DPP_ADD(0xB1);    // quad_perm [1,0,3,2]
  ART_DPP_ADD(0x4E);    // quad_perm [2,3,0,1]
  ART_DPP_ADD(0x141);   // row_half_mirror
  ART_DPP_ADD(0x140);   // row_mirror
#undef ART_DPP_ADD
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

// ------------------------------------------------------------------ RMSNorm
// out[i] = x[i] * rsqrt(vsum * inv_n + eps) * w[i];  vsum = sum x^2 (given by the caller or computed here)
template <class XT, class WT, class OT>
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const XT* __restrict__ x, const float* __restrict__ vsum,
                                                        const WT* __restrict__ w, OT* __restrict__ out, int n, float inv_n,
                                                        float eps) {
  __shared__ float s_part[16];
  const int tid = threadIdx.x;
  const XT* xr = x + (size_t)blockIdx.x * n;
  OT* orow = out + (size_t)blockIdx.x * n;
  float ss;
  if (vsum != nullptr) {
    ss = vsum[blockIdx.x];
  } else {
    float a = 0.f;
    for (int i = tid; i < n; i += 1024) {
      const float v = ld(xr, i);
      a = fmaf(v, v, a);
    }
    a = wave_sum(a);
    if ((tid & 63) == 0) s_part[tid >> 6] = a;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) ss += s_part[k];
  }
  const float r = 1.0f / sqrtf(ss * inv_n + eps);
  for (int i = tid; i < n; i += 1024) st(orow, i, ld(xr, i) * r * ld(w, i));
}

// ------------------------------------------------------------------ rotary
// rotate-half (HF Llama): x viewed as [H, 2, D/2]; theta_j = pos * inv_freq[j]
//   out[h,0,j] = x[h,0,j] cos - x[h,1,j] sin ;  out[h,1,j] = x[h,1,j] cos + x[h,0,j] sin
// interleaved (llama2.c): pairs (2j, 2j+1) of a flat vector, theta_j = pos * coef[j]
template <class XT, class FT, class OT, bool INTERLEAVED>
__global__ __launch_bounds__(256) void rotary_kernel(const XT* __restrict__ x, const FT* __restrict__ freq, OT* __restrict__ out,
                                                      int heads, int half, const int* __restrict__ pos_dev, int pos_host,
                                                      long long out_row_stride, int out_rows) {
  const int pos = pos_dev ? *pos_dev : pos_host;
  // out is a [out_rows, heads*head_dim] cache when the stride is set; a position past its end writes nothing
  // (a recorded graph replayed too often must not run off the cache)
  if (out_row_stride > 0 && (pos < 0 || pos >= out_rows)) return;
  out += (size_t)pos * out_row_stride;
  const int i = blockIdx.x * 256 + threadIdx.x;       // pair index over heads * half
  if (i >= heads * half) return;
  const int h = i / half, j = i % half;
  float s, c;
  if (INTERLEAVED) {
    sincosf((float)pos * ld(freq, i), &s, &c);        // coef has one entry per pair of the whole vector
    const size_t a = 2 * (size_t)i, b = a + 1;
    const float xa = ld(x, a), xb = ld(x, b);
    st(out, a, xa * c - xb * s);
    st(out, b, xa * s + xb * c);
  } else {
    sincosf((float)pos * ld(freq, j), &s, &c);
    const size_t a = (size_t)h * 2 * half + j, b = a + half;
    const float xa = ld(x, a), xb = ld(x, b);
    st(out, a, xa * c - xb * s);
    st(out, b, xb * c + xa * s);
  }
}

// ------------------------------------------------------------------ attention (one query)
// att[h,s] = (sum_m q[h,m] k[s,h,m]) * att_f ; p = softmax_s(att) ; out[h,m] = sum_s p[h,s] v[s,h,m]
// One block of 512 threads per head.  Eight lanes share a position (16 dims = 32 bytes of fp16 each), so
// a wavefront reads eight 256-byte rows per step; every 8-lane group keeps an online-softmax state (max,
// sum, 16 partial outputs) for the positions it visits and has four fp16 (two fp32) positions in flight,
// 128 KiB per block - a compute unit needs that much outstanding to stream at its full rate.  The
// eight groups of a wavefront are merged with lane exchanges, the eight wavefronts through LDS.

// 16 consecutive elements of a cache row, kept as loaded (fp16 rows stay packed: half the registers of a
// converted copy, which is what lets four positions per group be in flight without spilling) and converted where
// they are used.
template <class T> struct Row16;
template <> struct Row16<_Float16> {
  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  struct Raw { h8 lo, hi; };
  static __device__ __forceinline__ void load(const _Float16* p, Raw& r) {
    r.lo = *reinterpret_cast<const h8*>(p);
    r.hi = *reinterpret_cast<const h8*>(p + 8);
  }
  static __device__ __forceinline__ float at(const Raw& r, int i) { return i < 8 ? (float)r.lo[i] : (float)r.hi[i - 8]; }
};
template <> struct Row16<float> {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  struct Raw { f32x4 q[4]; };
  static __device__ __forceinline__ void load(const float* p, Raw& r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) r.q[i] = *reinterpret_cast<const f32x4*>(p + 4 * i);
  }
  static __device__ __forceinline__ float at(const Raw& r, int i) { return r.q[i >> 2][i & 3]; }
};

constexpr int kAttThreads = 512;
constexpr int kAttGroups = kAttThreads / 8;   // 64 position groups per block
constexpr int kAttWaves = kAttThreads / 64;
constexpr int kAttPartialStride = 132;        // floats per (head, part) record: acc[128], max, sum, 2 of padding (16-byte rows)

// Lane exchanges between the eight position groups of a wavefront (lanes that differ in bits 3, 4, 5).
__device__ __forceinline__ float att_ror8(float v) {      // the value of lane ^ 8 (row_ror:8)
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
}
// One step of a reduce-scatter between lanes l and l ^ 16 (l ^ 32): the lower lane of a pair keeps `a`, the upper one
// keeps `b`; the swap exchanges the upper lanes' `a` with the lower lanes' `b`, so both results are the kept quantity.
template <class F> __device__ __forceinline__ float att_swap16(float a, float b, F op) {
  auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b), false, false);
  return op(__builtin_bit_cast(float, (unsigned int)r[0]), __builtin_bit_cast(float, (unsigned int)r[1]));
}
template <class F> __device__ __forceinline__ float att_swap32(float a, float b, F op) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b), false, false);
  return op(__builtin_bit_cast(float, (unsigned int)r[0]), __builtin_bit_cast(float, (unsigned int)r[1]));
}
// `op` over the eight groups; every lane gets the result.
template <class F> __device__ __forceinline__ float att_over_groups(float v, F op) {
  v = op(v, att_ror8(v));
  v = att_swap16(v, v, op);
  return att_swap32(v, v, op);
}

// ROPE = true: the block first rotates its head's q and k (rotate-half form) from the token's q|k|v vector,
// writes k and v into cache row `pos` and attends over rows 0..pos; q_or_qkv then points at q|k|v.
template <class QT, class KT, class OT, bool ROPE>
__global__ __launch_bounds__(kAttThreads) void attention_kernel(const QT* __restrict__ q_or_qkv, KT* __restrict__ k, KT* __restrict__ v,
                                                                 const float* __restrict__ att_f, OT* __restrict__ out, int heads,
                                                                 const int* __restrict__ len_dev, int len_host,
                                                                 const _Float16* __restrict__ inv_freq,
                                                                 float* __restrict__ partial, int parts) {
  // parts > 1: `parts` blocks share a head, each attends over a contiguous range of the cached positions and
  // leaves its unnormalised state in partial[head][part][kAttPartialStride] = { acc[128], max, sum, -, - };
  // whoever consumes the result merges them (the o-projection does it while it loads x).
  constexpr int D = 128, U = 8 / sizeof(KT);              // len_host: the length, or the rows of the cache when len_dev is given
  __shared__ float s_m[kAttWaves], s_l[kAttWaves];
  __shared__ float s_acc[kAttWaves][D];
  __shared__ float s_q[D];
  __shared__ float s_k[D], s_v[D];
  const int h = blockIdx.x / parts, part = blockIdx.x % parts, tid = threadIdx.x;
  const int sub = tid & 7, group = tid >> 3, wave = tid >> 6, lane = tid & 63;
  const size_t row = (size_t)heads * D;
  // From here to the first use of a cache row the code is one straight line for every lane: all loads are issued
  // unconditionally (lanes without work re-read a valid address) and kept as loaded.  A load inside a divergent branch,
  // or a branch join between a load and its use, makes the compiler wait for every outstanding load on the spot, which
  // would put the trips to memory for the position, the token's vector and the cache rows one after another.
  QT xa = (QT)0.f, xb = (QT)0.f, xv = (QT)0.f;
  _Float16 freq = (_Float16)0.f;
  if constexpr (ROPE) {                                   // wavefront 0 rotates q, wavefront 1 rotates k, 2 and 3 carry v
    const int dim = heads * D;
    const QT* src = q_or_qkv + (wave == 1 ? dim : 0) + (size_t)h * D;
    xa = src[lane];
    xb = src[lane + 64];
    xv = q_or_qkv[2 * (size_t)dim + (size_t)h * D + (tid & 127)];
    freq = inv_freq[lane];
  }
  const float scale = att_f[0];
  int S;                                                  // device form carries the position, length = pos + 1
  if constexpr (ROPE) S = *len_dev + 1; else S = len_dev ? (*len_dev + 1) : len_host;
  if (len_dev && (S < 1 || S > len_host)) {
    // The position read on the device is past the end of the cache (len_host rows): touch no cache row and
    // hand on NaN, which every consumer propagates, instead of running off the allocation.
    if (tid < D) {
      const float nan = __builtin_nanf("");
      if (parts == 1) {
        st(out, (size_t)h * D + tid, nan);
      } else {
        float* dst = partial + ((size_t)h * parts + part) * kAttPartialStride;
        dst[tid] = nan;
        if (tid == 0) { dst[D] = 0.f; dst[D + 1] = nan; }
      }
    }
    return;
  }
  // With ROPE the newest position is served from LDS: the block does not wait for its own cache write.
  const int cached = ROPE ? S - 1 : S;                    // positions read from the cache
  const int span = (cached + parts - 1) / parts;          // ... of which this block takes [s_first, Sc)
  const int s_first = part * span < cached ? part * span : cached;
  const int Sc = s_first + span < cached ? s_first + span : cached;
  const int s_safe = Sc > 0 ? Sc - 1 : 0;                 // a row that exists, for lanes past the end (weight 0 below)
  const bool newest_here = ROPE && part == 0;             // one block of the head writes the cache row and attends to it
  const int s_start = s_first + group;

  float m = -INFINITY, l = 0.f, acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  auto group_sum = [](float d) {   // sum over the 8 lanes of a group (xor 1, xor 2 inside a quad, then the neighbouring quad)
    d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0xB1, 0xf, 0xf, false));
    d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x4E, 0xf, 0xf, false));
    d += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, d), 0x141, 0xf, 0xf, false));
    return d;
  };
  auto absorb = [&](float d, auto value) {                // one position into this group's online softmax
    const float mn = fmaxf(m, d);
    const float corr = __expf(m - mn), p = __expf(d - mn);
    l = l * corr + p;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = fmaf(acc[i], corr, p * value(i));
    m = mn;
  };
  // The cached positions of this block, UU per group in flight: requested first, then the rotary phase (which does
  // not depend on them), then the online softmax.
  auto stream = [&](auto in_flight) {
    constexpr int UU = decltype(in_flight)::value;
    typename Row16<KT>::Raw kf[UU], vf[UU];
    auto request = [&](int s0) {
#pragma unroll
      for (int u = 0; u < UU; ++u) {
        const int s = s0 + u * kAttGroups;
        const int sc = s < Sc ? s : s_safe;
        Row16<KT>::load(k + (size_t)sc * row + (size_t)h * D + sub * 16, kf[u]);
        Row16<KT>::load(v + (size_t)sc * row + (size_t)h * D + sub * 16, vf[u]);
      }
    };
    request(s_start);
    float qf[16];
    if constexpr (ROPE) {
      const int pos = S - 1;
      if (tid < 128) {
        float sn, cs;
        sincosf((float)pos * (float)freq, &sn, &cs);
        const float fa = (float)xa, fb = (float)xb;
        const float ra = fa * cs - fb * sn, rb = fb * cs + fa * sn;
        if (wave == 1) {                                  // the cache gets the rounded value, and so does this step
          if (newest_here) {
            KT* dst = k + (size_t)pos * row + (size_t)h * D;
            st(dst, lane, ra);
            st(dst, lane + 64, rb);
            s_k[lane] = (float)(KT)ra;
            s_k[lane + 64] = (float)(KT)rb;
          }
        } else {                                          // q goes through the output dtype like the separate operator
          s_q[lane] = (float)(QT)ra;
          s_q[lane + 64] = (float)(QT)rb;
        }
      } else if (tid < 256 && newest_here) {
        const int e = tid - 128;
        v[(size_t)pos * row + (size_t)h * D + e] = (KT)(float)xv;
        s_v[e] = (float)(KT)(float)xv;
      }
      art_lds_barrier();
#pragma unroll
      for (int i = 0; i < 16; ++i) qf[i] = s_q[sub * 16 + i] * scale;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) qf[i] = ld(q_or_qkv, (size_t)h * D + sub * 16 + i) * scale;
    }
    for (int s0 = s_start; s0 < Sc; s0 += kAttGroups * UU) {
      if (s0 != s_start) request(s0);
#pragma unroll
      for (int u = 0; u < UU; ++u) {
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) d = fmaf(qf[i], Row16<KT>::at(kf[u], i), d);
        d = group_sum(d);
        if (s0 + u * kAttGroups < Sc) absorb(d, [&](int i) { return Row16<KT>::at(vf[u], i); });
      }
    }
    if (newest_here) {                                    // the newest position, from LDS, joins group 0
      float kn[16], vn[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        kn[i] = s_k[sub * 16 + i];
        vn[i] = s_v[sub * 16 + i];
      }
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) d = fmaf(qf[i], kn[i], d);
      d = group_sum(d);
      if (group == 0) absorb(d, [&](int i) { return vn[i]; });
    }
  };
  // A block with at most one position per group (the usual case when several blocks share a head) keeps one row per
  // group in flight: every further one would be a second copy of the same row, and a wavefront's 16-byte load
  // occupies the compute unit's load path for 16 cycles whether it hits or not.
  if (Sc - s_first <= kAttGroups) stream(std::integral_constant<int, 1>()); else stream(std::integral_constant<int, U>());
  // The eight groups of a wavefront become one state: a common maximum, then the weighted sums.  The 16 outputs per
  // lane are summed over the groups by a reduce-scatter over lane bits 3, 4, 5 (16 -> 8 -> 4 -> 2 dims per lane, 14
  // exchanges instead of one per output and level), which leaves every lane with two dims of the wavefront's total.
  {
    const auto vmax = [](float a, float b) { return fmaxf(a, b); };
    const auto vadd = [](float a, float b) { return a + b; };
    const float mw = att_over_groups(m, vmax);
    const float wgt = (m == -INFINITY) ? 0.f : __expf(m - mw);
    const float lw = att_over_groups(l * wgt, vadd);
    const bool up = lane & 8;
    float r8[8], r4[4], r2[2];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float lo = acc[i] * wgt, hi = acc[8 + i] * wgt;
      r8[i] = (up ? hi : lo) + att_ror8(up ? lo : hi);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) r4[i] = att_swap16(r8[i], r8[i + 4], vadd);
#pragma unroll
    for (int i = 0; i < 2; ++i) r2[i] = att_swap32(r4[i], r4[i + 2], vadd);
    const int dim0 = sub * 16 + (lane & 8) + ((lane & 16) >> 2) + ((lane & 32) >> 4);
    s_acc[wave][dim0] = r2[0];
    s_acc[wave][dim0 + 1] = r2[1];
    if (lane == 0) { s_m[wave] = mw; s_l[wave] = lw; }
  }
  art_lds_barrier();                  // LDS only: the cache-row stores above need not have landed
  if (tid < D) {
    float mm = -INFINITY;
#pragma unroll
    for (int g = 0; g < kAttWaves; ++g) mm = fmaxf(mm, s_m[g]);
    float ll = 0.f, o = 0.f;
#pragma unroll
    for (int g = 0; g < kAttWaves; ++g) {
      const float wgt = (s_m[g] == -INFINITY) ? 0.f : __expf(s_m[g] - mm);
      ll = fmaf(s_l[g], wgt, ll);
      o = fmaf(s_acc[g][tid], wgt, o);
    }
    if (parts == 1) {
      st(out, (size_t)h * D + tid, o / ll);
    } else {                                  // an empty range leaves max = -inf, sum = 0: weight 0 in the merge
      float* dst = partial + ((size_t)h * parts + part) * kAttPartialStride;
      dst[tid] = o;
      if (tid == 0) { dst[D] = mm; dst[D + 1] = ll; }
    }
  }
}

}  // namespace

namespace {

// q | k | v of one token (3 * heads * head_dim values) -> rotated q, rotated k into its cache row, v into its cache row.
// One launch instead of two rotary launches and a row copy; the position comes from the device.
template <class T, class FT>
__global__ __launch_bounds__(256) void rope_qkv_store_kernel(const T* __restrict__ qkv, const FT* __restrict__ freq, T* __restrict__ q_out,
                                                              T* __restrict__ key_cache, T* __restrict__ val_cache, int heads, int half,
                                                              const int* __restrict__ pos_dev, int max_positions) {
  const int pos = *pos_dev;
  if (pos < 0 || pos >= max_positions) return;        // past the end of the caches: write nothing
  const int dim = heads * half * 2;
  const int pairs = heads * half;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < 2 * pairs) {                       // q pairs, then k pairs
    const bool is_k = i >= pairs;
    const int p = is_k ? i - pairs : i;
    const int h = p / half, j = p % half;
    const T* src = qkv + (is_k ? dim : 0);
    T* dst = is_k ? key_cache + (size_t)pos * dim : q_out;
    float s, c;
    sincosf((float)pos * ld(freq, j), &s, &c);
    const size_t a = (size_t)h * 2 * half + j, b = a + half;
    const float xa = ld(src, a), xb = ld(src, b);
    st(dst, a, xa * c - xb * s);
    st(dst, b, xb * c + xa * s);
  } else if (i < 2 * pairs + dim) {          // v row copy
    const int e = i - 2 * pairs;
    val_cache[(size_t)pos * dim + e] = qkv[2 * (size_t)dim + e];
  }
}

// The same for the T tokens of a prompt (row t of qkv at position first_pos + t): rotated q to q_out[t], rotated k and
// v into cache rows first_pos + t.  grid.y = t; the threads of a block walk the row's pairs with j fastest, so loads and
// stores of a wavefront are 128 contiguous bytes.
__global__ __launch_bounds__(256) void rope_qkv_store_rows_kernel(const _Float16* __restrict__ qkv, const _Float16* __restrict__ freq,
                                                                   _Float16* __restrict__ q_out, _Float16* __restrict__ key_cache,
                                                                   _Float16* __restrict__ val_cache, int heads, int half,
                                                                   int first_pos) {
  const int t = blockIdx.y, pos = first_pos + t;
  const int dim = heads * half * 2, pairs = heads * half;
  const _Float16* row = qkv + (size_t)t * 3 * dim;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < 2 * pairs) {                       // q pairs, then k pairs
    const bool is_k = i >= pairs;
    const int p = is_k ? i - pairs : i;
    const int h = p / half, j = p % half;
    const _Float16* src = row + (is_k ? dim : 0);
    _Float16* dst = is_k ? key_cache + (size_t)pos * dim : q_out + (size_t)t * dim;
    float s, c;
    sincosf((float)pos * (float)freq[j], &s, &c);
    const size_t a = (size_t)h * 2 * half + j, b = a + half;
    const float xa = (float)src[a], xb = (float)src[b];
    dst[a] = (_Float16)(xa * c - xb * s);
    dst[b] = (_Float16)(xb * c + xa * s);
  } else if (i < 2 * pairs + dim) {          // v row copy
    const int e = i - 2 * pairs;
    val_cache[(size_t)pos * dim + e] = row[2 * (size_t)dim + e];
  }
}

}  // namespace

// dtype codes: 0 = float32, 1 = float16
#define ART_DT_OK(d) ((d) == 0 || (d) == 1)

extern "C" int art_rmsnorm(const void* x_dev, const void* vsum_dev, const void* w_dev, void* out_dev, int rows, int n,
                           float inv_n, float eps, int x_dtype, int w_dtype, int out_dtype, void* stream) {
  ART_REQUIRE(x_dev && w_dev && out_dev && rows >= 1 && n >= 1, "art_rmsnorm: bad arguments");
  ART_REQUIRE(ART_DT_OK(x_dtype) && ART_DT_OK(w_dtype) && ART_DT_OK(out_dtype), "art_rmsnorm: dtype codes are 0 (f32) / 1 (f16)");
  hipStream_t st = (hipStream_t)stream;
  const float* vs = (const float*)vsum_dev;
#define ART_RMS(XT, WT, OT) rmsnorm_kernel<XT, WT, OT><<<dim3(rows), dim3(1024), 0, st>>>((const XT*)x_dev, vs, (const WT*)w_dev, (OT*)out_dev, n, inv_n, eps)
  const int key = x_dtype * 4 + w_dtype * 2 + out_dtype;
  switch (key) {
    case 0: ART_RMS(float, float, float); break;
    case 1: ART_RMS(float, float, _Float16); break;
    case 2: ART_RMS(float, _Float16, float); break;
    case 3: ART_RMS(float, _Float16, _Float16); break;
    case 4: ART_RMS(_Float16, float, float); break;
    case 5: ART_RMS(_Float16, float, _Float16); break;
    case 6: ART_RMS(_Float16, _Float16, float); break;
    default: ART_RMS(_Float16, _Float16, _Float16); break;
  }
#undef ART_RMS
  ART_LAUNCH_CHECK();
  return 0;
}

extern "C" int art_rotary(const void* x_dev, const void* freq_dev, void* out_dev, int heads, int head_dim, int interleaved,
                          const void* pos_dev, int pos, long long out_row_stride, int out_rows, int x_dtype, int freq_dtype,
                          int out_dtype, void* stream) {
  ART_REQUIRE(x_dev && freq_dev && out_dev && heads >= 1 && head_dim >= 2 && head_dim % 2 == 0, "art_rotary: bad arguments");
  ART_REQUIRE(ART_DT_OK(x_dtype) && ART_DT_OK(freq_dtype) && ART_DT_OK(out_dtype), "art_rotary: dtype codes are 0 (f32) / 1 (f16)");
  ART_REQUIRE(x_dtype == out_dtype, "art_rotary: input and output must have the same dtype");
  ART_REQUIRE(out_row_stride >= 0 && (out_row_stride == 0 || out_rows >= 1), "art_rotary: a cache output needs its row stride and row count");
  hipStream_t st = (hipStream_t)stream;
  const int half = head_dim / 2, pairs = heads * half;
  const dim3 grid((pairs + 255) / 256), block(256);
  const int* pd = (const int*)pos_dev;
#define ART_ROT(XT, FT, IL) rotary_kernel<XT, FT, XT, IL><<<grid, block, 0, st>>>((const XT*)x_dev, (const FT*)freq_dev, (XT*)out_dev, heads, half, pd, pos, out_row_stride, out_rows)
  if (interleaved) {
    if (x_dtype == 0) { if (freq_dtype == 0) ART_ROT(float, float, true); else ART_ROT(float, _Float16, true); }
    else { if (freq_dtype == 0) ART_ROT(_Float16, float, true); else ART_ROT(_Float16, _Float16, true); }
  } else {
    if (x_dtype == 0) { if (freq_dtype == 0) ART_ROT(float, float, false); else ART_ROT(float, _Float16, false); }
    else { if (freq_dtype == 0) ART_ROT(_Float16, float, false); else ART_ROT(_Float16, _Float16, false); }
  }
#undef ART_ROT
  ART_LAUNCH_CHECK();
  return 0;
}

extern "C" int art_decode_attention(const void* q_dev, const void* k_dev, const void* v_dev, const void* att_f_dev, void* out_dev,
                                    int seq_len, int heads, int head_dim, const void* pos_dev, int q_dtype, int kv_dtype,
                                    int out_dtype, void* stream) {
  ART_REQUIRE(q_dev && k_dev && v_dev && att_f_dev && out_dev, "art_decode_attention: null pointer");
  ART_REQUIRE(head_dim == 128, "art_decode_attention: head_dim must be 128 (got %d)", head_dim);
  ART_REQUIRE(heads >= 1 && seq_len >= 1, "art_decode_attention: bad shape (seq_len is the length, or the rows of the cache when the position is read on the device)");
  ART_REQUIRE(ART_DT_OK(q_dtype) && ART_DT_OK(kv_dtype) && ART_DT_OK(out_dtype), "art_decode_attention: dtype codes are 0 (f32) / 1 (f16)");
  ART_REQUIRE(q_dtype == out_dtype, "art_decode_attention: q and out must have the same dtype");
  ART_REQUIRE(((uintptr_t)k_dev % 16) == 0 && ((uintptr_t)v_dev % 16) == 0, "art_decode_attention: k and v must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int* pd = (const int*)pos_dev;
  const float* af = (const float*)att_f_dev;
#define ART_ATT(QT, KT) attention_kernel<QT, KT, QT, false><<<dim3(heads), dim3(kAttThreads), 0, st>>>((const QT*)q_dev, (KT*)k_dev, (KT*)v_dev, af, (QT*)out_dev, heads, pd, seq_len, nullptr, nullptr, 1)
  if (q_dtype == 0) { if (kv_dtype == 0) ART_ATT(float, float); else ART_ATT(float, _Float16); }
  else { if (kv_dtype == 0) ART_ATT(_Float16, float); else ART_ATT(_Float16, _Float16); }
#undef ART_ATT
  ART_LAUNCH_CHECK();
  return 0;
}

extern "C" int art_rope_qkv_store(const void* qkv_dev, const void* freq_dev, void* q_out_dev, void* key_cache_dev, void* val_cache_dev,
                                  int heads, int head_dim, const void* pos_dev, int max_positions, int dtype, int freq_dtype,
                                  void* stream) {
  ART_REQUIRE(qkv_dev && freq_dev && q_out_dev && key_cache_dev && val_cache_dev && pos_dev, "art_rope_qkv_store: null pointer");
  ART_REQUIRE(max_positions >= 1, "art_rope_qkv_store: the caches have no rows");
  ART_REQUIRE(heads >= 1 && head_dim >= 2 && head_dim % 2 == 0, "art_rope_qkv_store: bad shape");
  ART_REQUIRE(ART_DT_OK(dtype) && ART_DT_OK(freq_dtype), "art_rope_qkv_store: dtype codes are 0 (f32) / 1 (f16)");
  const int half = head_dim / 2, dim = heads * head_dim;
  const dim3 grid((2 * heads * half + dim + 255) / 256), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int* pd = (const int*)pos_dev;
#define ART_RQS(T, FT) rope_qkv_store_kernel<T, FT><<<grid, block, 0, st>>>((const T*)qkv_dev, (const FT*)freq_dev, (T*)q_out_dev, (T*)key_cache_dev, (T*)val_cache_dev, heads, half, pd, max_positions)
  if (dtype == 0) { if (freq_dtype == 0) ART_RQS(float, float); else ART_RQS(float, _Float16); }
  else { if (freq_dtype == 0) ART_RQS(_Float16, float); else ART_RQS(_Float16, _Float16); }
#undef ART_RQS
  ART_LAUNCH_CHECK();
  return 0;
}

extern "C" int art_rope_qkv_store_rows(const void* qkv_dev, const void* freq_dev, void* q_out_dev, void* key_cache_dev,
                                       void* val_cache_dev, int rows, int heads, int head_dim, int first_pos, int max_positions,
                                       void* stream) {
  ART_REQUIRE(qkv_dev && freq_dev && q_out_dev && key_cache_dev && val_cache_dev, "art_rope_qkv_store_rows: null pointer");
  ART_REQUIRE(heads >= 1 && head_dim >= 2 && head_dim % 2 == 0, "art_rope_qkv_store_rows: bad shape");
  ART_REQUIRE(rows >= 1 && rows <= 65535 && first_pos >= 0 && first_pos + rows <= max_positions,
              "art_rope_qkv_store_rows: positions %d..%d do not fit caches of %d rows", first_pos, first_pos + rows - 1, max_positions);
  const int half = head_dim / 2, dim = heads * head_dim;
  const dim3 grid((2 * heads * half + dim + 255) / 256, rows), block(256);
  rope_qkv_store_rows_kernel<<<grid, block, 0, (hipStream_t)stream>>>((const _Float16*)qkv_dev, (const _Float16*)freq_dev,
                                                                      (_Float16*)q_out_dev, (_Float16*)key_cache_dev,
                                                                      (_Float16*)val_cache_dev, heads, half, first_pos);
  ART_LAUNCH_CHECK();
  return 0;
}

extern "C" int art_decode_attention_rope(const void* qkv_dev, const void* inv_freq_dev, void* key_cache_dev, void* val_cache_dev,
                                         const void* att_f_dev, void* out_dev, int heads, int head_dim, const void* pos_dev,
                                         int max_positions, void* stream) {
  return art_decode_attention_rope_split(qkv_dev, inv_freq_dev, key_cache_dev, val_cache_dev, att_f_dev, out_dev, heads, head_dim,
                                         pos_dev, max_positions, 1, stream);
}

extern "C" int art_decode_attention_rope_split(const void* qkv_dev, const void* inv_freq_dev, void* key_cache_dev,
                                               void* val_cache_dev, const void* att_f_dev, void* out_dev, int heads, int head_dim,
                                               const void* pos_dev, int max_positions, int parts, void* stream) {
  ART_REQUIRE(qkv_dev && inv_freq_dev && key_cache_dev && val_cache_dev && att_f_dev && out_dev && pos_dev,
              "art_decode_attention_rope: null pointer");
  ART_REQUIRE(head_dim == 128 && heads >= 1, "art_decode_attention_rope: head_dim must be 128 (got %d)", head_dim);
  ART_REQUIRE(parts >= 1 && parts <= art::kMaxAttnParts, "art_decode_attention_rope_split: parts must be in 1..%d (got %d)",
              art::kMaxAttnParts, parts);
  ART_REQUIRE(max_positions >= 1, "art_decode_attention_rope: the caches have no rows");
  ART_REQUIRE(((uintptr_t)key_cache_dev % 16) == 0 && ((uintptr_t)val_cache_dev % 16) == 0 && ((uintptr_t)out_dev % 16) == 0,
              "art_decode_attention_rope: caches and output must be 16-byte aligned");
  attention_kernel<_Float16, _Float16, _Float16, true><<<dim3(heads * parts), dim3(kAttThreads), 0, (hipStream_t)stream>>>(
      (const _Float16*)qkv_dev, (_Float16*)key_cache_dev, (_Float16*)val_cache_dev, (const float*)att_f_dev,
      parts == 1 ? (_Float16*)out_dev : nullptr, heads, (const int*)pos_dev, max_positions, (const _Float16*)inv_freq_dev,
      parts == 1 ? nullptr : (float*)out_dev, parts);
  ART_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ greedy step bookkeeping
// The tail of one decode step of samples/05_llama2_7b_int4.py:196-201 in a single block:
//   pos <- pos + 1;  token <- prompt[pos] while the prompt lasts, else argmax(logits);  x <- embedding[token].
// Replaces an argmax, five elementwise launches and the embedding gather of the next step.
namespace {

constexpr int kGreedyThreads = 1024;

__global__ __launch_bounds__(kGreedyThreads) void greedy_next_kernel(const _Float16* __restrict__ logits, int vocab,
                                                                      const int* __restrict__ prompt, int prompt_len,
                                                                      int* __restrict__ token, int* __restrict__ pos,
                                                                      const _Float16* __restrict__ embed, int dim,
                                                                      _Float16* __restrict__ x_out) {
  __shared__ float s_val[kGreedyThreads / 64];
  __shared__ int s_idx[kGreedyThreads / 64];
  __shared__ int s_token;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int next_pos = *pos + 1;
  // largest logit, smallest index among equals (what torch.argmax returns)
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  // 16-byte chunks, four of them requested before the first is looked at (one round trip for 32768 logits)
  const int chunks = vocab >> 3;
  for (int c0 = tid; c0 < chunks; c0 += 4 * kGreedyThreads) {
    u32x4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = c0 + j * kGreedyThreads;
      v[j] = *reinterpret_cast<const u32x4*>(logits + 8 * (size_t)(c < chunks ? c : c0));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = c0 + j * kGreedyThreads;
      if (c >= chunks) break;
      const unsigned int wds[4] = {v[j][0], v[j][1], v[j][2], v[j][3]};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 pair = __builtin_bit_cast(h2, wds[e >> 1]);
        const float f = (float)((e & 1) ? pair.y : pair.x);
        if (f > best) { best = f; best_i = 8 * c + e; }      // indices grow: the first maximum of this thread stays
      }
    }
  }
  for (int i = (chunks << 3) + tid; i < vocab; i += kGreedyThreads) {      // vocab % 8 leftovers
    const float f = (float)logits[i];
    if (f > best || (f == best && i < best_i)) { best = f; best_i = i; }
  }
#pragma unroll
  for (int m = 1; m < 64; m <<= 1) {
    const float ov = __shfl_xor(best, m, 64);
    const int oi = __shfl_xor(best_i, m, 64);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  if (lane == 0) { s_val[wave] = best; s_idx[wave] = best_i; }
  __syncthreads();
  if (tid == 0) {
    float b = s_val[0];
    int bi = s_idx[0];
    for (int w = 1; w < kGreedyThreads / 64; ++w)
      if (s_val[w] > b || (s_val[w] == b && s_idx[w] < bi)) { b = s_val[w]; bi = s_idx[w]; }
    if (bi == 0x7fffffff) bi = 0;                 // every logit was NaN or -inf
    int t = (next_pos < prompt_len) ? prompt[next_pos] : bi;
    t = t < 0 ? 0 : (t >= vocab ? vocab - 1 : t);            // a prompt id outside the vocabulary must not index past the table
    s_token = t;
    *token = t;
    *pos = next_pos;
  }
  __syncthreads();
  const _Float16* row = embed + (size_t)s_token * dim;
  for (int i = tid * 8; i < dim; i += kGreedyThreads * 8)
    *reinterpret_cast<u32x4*>(x_out + i) = *reinterpret_cast<const u32x4*>(row + i);
}

}  // namespace

extern "C" int art_greedy_next(const void* logits_dev, int vocab, const void* prompt_dev, int prompt_len, void* token_dev,
                               void* pos_dev, const void* embed_dev, int dim, void* x_out_dev, void* stream) {
  ART_REQUIRE(logits_dev && token_dev && pos_dev && embed_dev && x_out_dev, "art_greedy_next: null pointer");
  ART_REQUIRE(vocab >= 1 && dim >= 8 && dim % 8 == 0, "art_greedy_next: need vocab >= 1 and dim %% 8 == 0 (vocab=%d dim=%d)", vocab, dim);
  ART_REQUIRE(prompt_len == 0 || prompt_dev != nullptr, "art_greedy_next: prompt_len > 0 needs a prompt");
  ART_REQUIRE(((uintptr_t)embed_dev % 16) == 0 && ((uintptr_t)x_out_dev % 16) == 0 && ((uintptr_t)logits_dev % 16) == 0,
              "art_greedy_next: logits, embedding and x must be 16-byte aligned");
  greedy_next_kernel<<<dim3(1), dim3(kGreedyThreads), 0, (hipStream_t)stream>>>((const _Float16*)logits_dev, vocab, (const int*)prompt_dev,
                                                                                prompt_len, (int*)token_dev, (int*)pos_dev,
                                                                                (const _Float16*)embed_dev, dim, (_Float16*)x_out_dev);
  ART_LAUNCH_CHECK();
  return 0;
}
