// Causal attention over a whole prompt on the gfx950 matrix cores (fp16 in, fp32 accumulation, fp16 out):
//
//   a[t,h,s] = att_f * sum_m q[t,h,m] k[s,h,m]   for s <= t;   p = softmax_s(a);   out[t,h,m] = sum_s p[t,h,s] v[s,h,m]
//
// i.e. the attention of samples/03_llama_tiny.py:94-99 / samples/05_llama2_7b_int4.py:161-165 for T query positions at
// once, position t attending to cache rows 0..t.  It replaces the two generated contraction kernels (scores, then
// softmax times V) that the reference's tiled schedule would produce for a prompt
// (backends/c-rocm/schedule/standard/algo_tiling.py:35-98).
//
// One wavefront per (head, tile of 32 queries); it walks the key tiles 0..its own, so nothing is computed above the
// diagonal and no block barrier exists.  Everything is kept transposed so that a lane owns ONE query:
//   * S^T = K Q^T on v_mfma_f32_32x32x16_f16: A = a K tile as it lies in the cache (32 rows of 128 dims, staged in LDS
//     with coalesced 16-byte loads, read back as 16-byte rows), B = the lane's query row from registers.  The 32 x 32
//     result has query lane % 32 in every lane, 16 keys per lane: the running maximum and sum of the online softmax
//     are per-lane scalars, completed with one exchange between lanes l and l ^ 32.
//   * O^T += V^T P^T: the probabilities go from the accumulator layout straight into the B operand (the order of
//     the summed index is free as long as both operands agree), V^T comes out of the row-major V tile through the
//     transposing LDS read ds_read_b64_tr_b16, with the row quadruples chosen to match that order.
//   * the rescaling by e^(m_old - m_new) is one multiplication per accumulator register.
#include "art_common.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int D = 128;                 // head dimension
constexpr int QT = 32, KT = 32;        // queries per wavefront, keys per step
constexpr int K_LD = D + 8;            // halves per K row in LDS (272 bytes)
constexpr int V_LD = D + 32;           // halves per V row in LDS (320 bytes: the four rows of a transposing read fall on disjoint banks)

__device__ __forceinline__ float max_with_lane_xor_32(float v) {
  const unsigned int u = __builtin_bit_cast(unsigned int, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (unsigned int)r[0]), __builtin_bit_cast(float, (unsigned int)r[1]));
}
__device__ __forceinline__ float sum_with_lane_xor_32(float v) {
  const unsigned int u = __builtin_bit_cast(unsigned int, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (unsigned int)r[0]) + __builtin_bit_cast(float, (unsigned int)r[1]);
}

// q: [T, heads, 128]; k, v: rows of kv_stride halves, row s holding [heads, 128]; out: [T, heads, 128]
__global__ __launch_bounds__(64) void prefill_attention_kernel(const _Float16* __restrict__ q, const _Float16* __restrict__ k,
                                                                const _Float16* __restrict__ v, _Float16* __restrict__ out, int T,
                                                                int heads, long long kv_stride, const float* __restrict__ att_f,
                                                                int q_tiles) {
  __shared__ __align__(16) _Float16 Ks[KT * K_LD];
  __shared__ __align__(16) _Float16 Vs[KT * V_LD];
  const int lane = threadIdx.x, half = lane >> 5, qi = lane & 31;
  // the longest walks (last query tiles) are handed out first
  const int qt = q_tiles - 1 - (int)(blockIdx.x % q_tiles), h = blockIdx.x / q_tiles;
  const int query = qt * QT + qi;
  const int qrow = query < T ? query : T - 1;                    // rows past T repeat the last one and are never stored
  const float scale = att_f[0];

  // B operand of S^T = K Q^T: query lane % 32, dims 16 s + 8 half .. + 8 of step s
  h8 bq[D / 16];
  {
    const _Float16* qp = q + ((size_t)qrow * heads + h) * D + 8 * half;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) bq[s] = *reinterpret_cast<const h8*>(qp + 16 * s);
  }
  // staging of a K / V tile: 32 rows x 16 chunks of 16 bytes = 8 chunks per lane and matrix
  const int st_row = lane >> 4, st_col = (lane & 15) * 8;      // + 4 rows per i
  u32x4 kreg[8], vreg[8];
  auto load_tile = [&](int kt) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int key = kt * KT + st_row + 4 * i;
      const size_t off = (size_t)(key < T ? key : T - 1) * kv_stride + (size_t)h * D + st_col;
      kreg[i] = *reinterpret_cast<const u32x4*>(k + off);
      vreg[i] = *reinterpret_cast<const u32x4*>(v + off);
    }
  };
  load_tile(0);

  float m_run = -INFINITY, l_run = 0.f;
  f16v o[D / 32];
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;

  // per-lane constants of the transposing read of V^T: 16 lanes cover 4 rows x 16 columns
  const int s16 = lane & 15;
  const int tr_row = s16 >> 2, tr_col = ((lane & 31) >> 4) * 16 + (s16 & 3) * 4;

  for (int kt = 0; kt <= qt; ++kt) {
    // registers -> LDS (a wavefront's LDS operations execute in order: the reads of the previous tile are done)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      *reinterpret_cast<u32x4*>(&Ks[(st_row + 4 * i) * K_LD + st_col]) = kreg[i];
      *reinterpret_cast<u32x4*>(&Vs[(st_row + 4 * i) * V_LD + st_col]) = vreg[i];
    }
    if (kt < qt) load_tile(kt + 1);                              // next tile's loads fly during this tile's arithmetic
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- S^T tile: rows = keys of the tile, columns = queries
    f16v st;
#pragma unroll
    for (int r = 0; r < 16; ++r) st[r] = 0.f;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      const h8 a = *reinterpret_cast<const h8*>(&Ks[qi * K_LD + 16 * s + 8 * half]);      // key row lane % 32
      st = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bq[s], st, 0, 0, 0);
    }
    // element r of the accumulator: key (r / 4) * 8 + 4 * half + r % 4 of the tile, query lane % 32
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = kt * KT + (r >> 2) * 8 + 4 * half + (r & 3);
      st[r] = key <= query ? st[r] * scale : -INFINITY;
      mx = fmaxf(mx, st[r]);
    }
    mx = max_with_lane_xor_32(mx);
    // key kt * 32 <= query for every query of this wavefront's tile, so the maximum is finite from the first tile on
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __expf(m_run - m_new);                   // first tile: e^(-inf) = 0
    float lsum = 0.f;
    float p[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      p[r] = __expf(st[r] - m_new);                              // masked: e^(-inf) = 0
      lsum += p[r];
    }
    lsum = sum_with_lane_xor_32(lsum);
    l_run = l_run * alpha + lsum;
    m_run = m_new;
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][r] *= alpha;

    // ---- O^T += V^T P^T.  Step j sums over 16 keys; lane half `half` supplies, as elements 0..7, the keys
    // (2j) * 8 + 4 half + 0..3 and (2j + 1) * 8 + 4 half + 0..3 - exactly p[8j .. 8j + 7] - and V^T is read with the same
    // two row quadruples.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const h8 bp = {(_Float16)p[8 * j], (_Float16)p[8 * j + 1], (_Float16)p[8 * j + 2], (_Float16)p[8 * j + 3],
                     (_Float16)p[8 * j + 4], (_Float16)p[8 * j + 5], (_Float16)p[8 * j + 6], (_Float16)p[8 * j + 7]};
      const int row_lo = 16 * j + 4 * half + tr_row, row_hi = row_lo + 8;
#pragma unroll
      for (int t = 0; t < D / 32; ++t) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(&Vs[row_lo * V_LD + t * 32 + tr_col]));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(&Vs[row_hi * V_LD + t * 32 + tr_col]));
        const h4 l4 = __builtin_bit_cast(h4, lo), h4v = __builtin_bit_cast(h4, hi);
        const h8 a = {l4[0], l4[1], l4[2], l4[3], h4v[0], h4v[1], h4v[2], h4v[3]};      // dim t * 32 + lane % 32, eight keys
        o[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bp, o[t], 0, 0, 0);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");      // the LDS reads above precede the next tile's writes
    __builtin_amdgcn_wave_barrier();
  }

  if (query >= T) return;
  const float inv = 1.0f / l_run;
  _Float16* op = out + ((size_t)query * heads + h) * D;
  // element r of tile t: dim t * 32 + (r / 4) * 8 + 4 * half + r % 4
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const h4 w = {(_Float16)(o[t][4 * g] * inv), (_Float16)(o[t][4 * g + 1] * inv), (_Float16)(o[t][4 * g + 2] * inv),
                    (_Float16)(o[t][4 * g + 3] * inv)};
      *reinterpret_cast<h4*>(op + t * 32 + g * 8 + 4 * half) = w;
    }
}

}  // namespace

extern "C" int art_prefill_attention(const void* q_dev, const void* k_dev, const void* v_dev, const void* att_f_dev, void* out_dev,
                                     int T, int heads, int head_dim, long long kv_row_stride, void* stream) {
  ART_REQUIRE(q_dev && k_dev && v_dev && att_f_dev && out_dev, "art_prefill_attention: null pointer");
  ART_REQUIRE(head_dim == D, "art_prefill_attention: head_dim must be 128 (got %d)", head_dim);
  ART_REQUIRE(T >= 1 && heads >= 1 && kv_row_stride >= (long long)heads * D, "art_prefill_attention: bad sizes (T=%d heads=%d stride=%lld)",
              T, heads, kv_row_stride);
  ART_REQUIRE(((uintptr_t)q_dev % 16) == 0 && ((uintptr_t)k_dev % 16) == 0 && ((uintptr_t)v_dev % 16) == 0 && ((uintptr_t)out_dev % 8) == 0 &&
                  kv_row_stride % 8 == 0,
              "art_prefill_attention: q, k, v must be 16-byte aligned (row stride a multiple of 8 halves), out 8-byte aligned");
  const int q_tiles = (T + QT - 1) / QT;
  const long long blocks = (long long)q_tiles * heads;
  ART_REQUIRE(blocks <= 0x7fffffffLL, "art_prefill_attention: too many blocks");
  prefill_attention_kernel<<<dim3((unsigned)blocks), dim3(64), 0, (hipStream_t)stream>>>(
      (const _Float16*)q_dev, (const _Float16*)k_dev, (const _Float16*)v_dev, (_Float16*)out_dev, T, heads, kv_row_stride,
      (const float*)att_f_dev, q_tiles);
  ART_LAUNCH_CHECK();
  return 0;
}
