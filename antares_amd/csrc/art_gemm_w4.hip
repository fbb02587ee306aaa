// Weight-only int4 GEMM for a batch of rows (prefill, four rows and more): the same arithmetic as the GEMV of
// art_gemv_w4.hip,
//     y[m,n] = sum_k x[m,k] * w[k,n],   w[k,n] = fp16(s[g,n] * fp16(q[k,n] - z[g,n])),   group g = k / 128,
// on the matrix cores with fp32 accumulation; w is rounded exactly as the reference's dequant + matmul program
// does (samples/05_llama2_7b_int4.py:135-144 exported with a batch axis).
//
// Design for MI355X:
//   * a block of eight wavefronts owns 256 columns, up to 64 rows and a contiguous range of quantisation groups; it
//     works one group (128 k) per loop iteration;
//   * everything a group needs - 16 KiB of packed weights, 16 KiB of x, 512 B of scales, 128 B of zero points - goes
//     from global memory straight into LDS (global_load_lds_dwordx4 / _dword: no registers hold data in flight), into
//     a ring of four stages, so three groups (100 KiB per compute unit) are on their way while one is multiplied.
//     Register staging two groups ahead held a compute unit to about 45 GB/s; this ring sustains over 100 GB/s;
//   * each lane chooses which 16-byte chunk it fetches, and LDS position (row r, chunk c) holds chunk c ^ (r & 7) of
//     the weights (c ^ (r & 15) of x): the reads below then touch every bank once although rows are 256 bytes apart;
//   * the packed bytes stay packed in LDS.  ds_read_b64_tr_b8 hands a lane the 8 bytes = 16 values of k of ONE column,
//     i.e. the B operand of two v_mfma_f32_32x32x16_f16; a lane unpacks only the columns it multiplies (one shift,
//     four v_bitop3_b32, four packed subtractions of the zero point, four packed multiplications by the scale per
//     word).  The nibble extraction leaves k in the order 0 4 1 5 2 6 3 7; the A operand is permuted the same way
//     (four v_perm_b32 per 16 bytes of x);
//   * wavefront (c, h) multiplies 64 columns (c = 0..3) by the k half h of every group: per group 16 bytes of x and
//     of packed weights per lane and MFMA, 112 KiB of LDS traffic per group instead of 280 KiB with fp16 weights in
//     LDS; the two k halves meet in LDS once, after the loop;
//   * the loop is rolled (one group per iteration, one barrier): the whole kernel is 7 KiB of code.  A launch fetches
//     its code cold - straight-line code costs about 0.3 us per KiB executed - so unrolled stages are not free;
//   * split-K without atomics (5.6 M float atomics cost 75 us on this chip): each K-split writes its fp32 tile to the
//     library workspace and a second small kernel adds the splits in a fixed order and rounds once to fp16 - results
//     do not depend on timing.
#include "art_common.h"

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;

constexpr int kThreads = 512;                       // 8 wavefronts: 4 column quarters x 2 k halves
constexpr int BM = 64, BN = 256, GK = 128;          // rows and columns of a block, k of a quantisation group
constexpr int NS = 4;                               // stages of the LDS ring, one quantisation group each
constexpr int W_BYTES = (GK / 2) * BN;              // packed weights of a group: 64 byte-rows x 256 columns
constexpr int X_BYTES = BM * GK * 2;                // x of a group: 64 rows x 128 k, fp16
constexpr int Q_BYTES = 2048;                       // scales (512 B) at 0, zero points (128 B) at 512; the rest takes the idle lanes
constexpr int STAGE = W_BYTES + X_BYTES + Q_BYTES;
constexpr int RLD = BN + 4;                         // floats per row of a result tile in LDS
constexpr size_t kLdsBytes = (size_t)NS * STAGE;    // 139264; the two result tiles of the epilogue (133120) reuse it
static_assert(2 * BM * RLD * sizeof(float) <= kLdsBytes, "the result tiles fit the ring");

struct Magic {
  unsigned int mask_lo, mask_hi, bias_lo, bias_hi;   // 0x000F000F 0x00F000F0 0x64006400 0x54005400
};

__device__ __forceinline__ h2 as_h2(unsigned int v) { return __builtin_bit_cast(h2, v); }

// (w & mask) | bias in one v_bitop3_b32 (truth table 0xEA = (a & b) | c).
__device__ __forceinline__ unsigned int and_or(unsigned int w, unsigned int mask, unsigned int bias) {
  return __builtin_amdgcn_bitop3_b32(w, mask, bias, 0xEA);
}

// 8 halves of x in the k order the nibble extraction leaves in a B operand: k0 k4 k1 k5 k2 k6 k3 k7.
__device__ __forceinline__ h8 permute_k(u32x4 v) {
  u32x4 o;
  o[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
  o[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
  o[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
  o[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
  return __builtin_bit_cast(h8, o);
}

// 64 lanes x 16 (4) bytes from global memory straight into LDS: lane l's bytes land at lds_dst + 16 l (4 l); the lane
// chooses its global address freely.  The instruction takes the LDS address from m0, which is put back afterwards.
// Counted by vmcnt like any load; the compiler does not see these loads, so every wait for them below is written by
// hand (the compiler's own builtin for this instruction makes it wait for vmcnt(0) before every LDS read).
__device__ __forceinline__ void load_lds_x4(const void* g, unsigned int lds_dst) {
  unsigned int keep;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
               : "=&s"(keep) : "v"(g), "s"(lds_dst) : "memory");
}
__device__ __forceinline__ void load_lds_x1(const void* g, unsigned int lds_dst) {
  unsigned int keep;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %1, off\n\ts_mov_b32 m0, %0"
               : "=&s"(keep) : "v"(g), "s"(lds_dst) : "memory");
}

template <int MT>   // MT accumulator tiles of 32 rows: a block owns 32 MT rows
__global__ __launch_bounds__(kThreads) void gemm_w4a16_kernel(const _Float16* __restrict__ x, const unsigned char* __restrict__ qweight,
                                                              const _Float16* __restrict__ scales,
                                                              const unsigned char* __restrict__ qzeros, _Float16* y,
                                                              float* __restrict__ partial, int M_total, int K, int N, int splits,
                                                              int col_tiles, int m_blocks, Magic mg,
                                                              const _Float16* residual) {       // residual may be y itself
  extern __shared__ __align__(1024) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cw = wave & 3, kh = wave >> 2;          // 64-column quarter of the tile, k half of every group

  // block -> (column tile, K split, block of 64 rows).  The row blocks of one (tile, split) stream the same weights:
  // they get block ids that are 8 apart, which the dispatcher places on the same XCD at the same time, so that the
  // weights come from HBM once and from that XCD's L2 for the others.
  const int G = K / GK;
  const int unit = (int)(blockIdx.x / (8 * m_blocks)) * 8 + (int)(blockIdx.x % 8);      // (tile, split) pair
  const int m_block = (int)(blockIdx.x % (8 * m_blocks)) / 8;
  if (unit >= col_tiles * splits) return;
  const int split = unit / col_tiles;
  const int n0 = (unit % col_tiles) * BN;
  constexpr int RB = 32 * MT;                       // rows of a block
  constexpr int kLoadsPerGroup = 3 + MT;            // LDS-direct loads per wavefront and group: 2 weights, MT x, 1 scales / zero points
  const int m0 = m_block * RB;
  const int M = M_total - m0 < RB ? M_total - m0 : RB;          // rows of this block
  x += (size_t)m0 * K;
  y += (size_t)m0 * N;
  if (residual) residual += (size_t)m0 * N;
  const int g_begin = (int)((long long)G * split / splits), g_end = (int)((long long)G * (split + 1) / splits);
  const int groups = g_end - g_begin;
  const unsigned int lds0 = (unsigned int)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;

  // ---- what this lane fetches per group: two 16-byte chunks of packed weights, two of x, one dword of scales or
  // zero points.  Wavefront w fills LDS bytes [1024 j, 1024 j + 1024), j = w and w + 8, of the weight and the x area:
  // rows 4 j .. 4 j + 3 of 256 bytes.  Columns past N and rows past M re-read valid memory; nothing of them is stored.
  const unsigned char* wsrc[2];
  const _Float16* xsrc[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int r = 4 * (wave + 8 * u) + (lane >> 4);
    const int col = n0 + ((lane & 15) ^ (r & 7)) * 16;            // N % 16 == 0: a chunk is inside or outside as a whole
    wsrc[u] = qweight + ((size_t)g_begin * (GK / 2) + r) * N + (col < N ? col : 0);
    xsrc[u] = x + (size_t)(r < M ? r : M - 1) * K + (size_t)g_begin * GK + ((lane & 15) ^ (r & 15)) * 8;
  }
  const unsigned char* qsrc;
  int qstep;                                        // bytes from one group to the next
  {
    const int d = wave * 64 + lane;                 // dword of the 2 KiB area
    if (d < 128) {                                  // scales of columns 2 d, 2 d + 1
      const int col = n0 + 2 * d;
      qsrc = reinterpret_cast<const unsigned char*>(scales + (size_t)g_begin * N + (col < N ? col : 0));
      qstep = 2 * N;
    } else if (d < 160) {                           // zero points of columns 8 (d - 128) .. + 7
      const int col = n0 + 8 * (d - 128);
      qsrc = qzeros + (size_t)g_begin * (N / 2) + ((col < N ? col : 0) >> 1);
      qstep = N / 2;
    } else {                                        // idle lanes re-read the first scales into the padding
      qsrc = reinterpret_cast<const unsigned char*>(scales + (size_t)g_begin * N);
      qstep = 2 * N;
    }
  }
  // batch b (group g_begin + b) goes to stage b % NS: kLoadsPerGroup loads per wavefront
  auto issue = [&](int b) {
    const unsigned int st = lds0 + (unsigned int)(b % NS) * STAGE;
#pragma unroll
    for (int u = 0; u < 2; ++u) load_lds_x4(wsrc[u] + (size_t)b * (GK / 2) * N, st + (wave + 8 * u) * 1024);
#pragma unroll
    for (int u = 0; u < MT; ++u) load_lds_x4(xsrc[u] + (size_t)b * GK, st + W_BYTES + (wave + 8 * u) * 1024);    // 32 rows each
    load_lds_x1(qsrc + (size_t)b * qstep, st + W_BYTES + X_BYTES + wave * 256);
  };

  // ---- operand roles.  A transposing read takes 8 byte-rows x 16 columns per 16 lanes: lane s16 supplies the
  // 8-byte piece (row s16 / 2, half s16 % 2) and receives the 8 bytes of column s16.  Lanes 16-31 of a column tile
  // take the chunk 8 further on, so that the 32 lanes of a pass touch 16 different chunk positions.
  const int s16 = lane & 15, hi16 = (lane >> 4) & 1, h = lane >> 5;
  int b_off[2], colpos[2];
#pragma unroll
  for (int ct = 0; ct < 2; ++ct) {
    const int chunk = cw * 2 + ct + 8 * hi16;       // this lane's 16-column chunk of column tile ct
    b_off[ct] = (kh * 32 + h * 16 + (s16 >> 1)) * 256 + ((chunk ^ (s16 >> 1)) * 16) + (s16 & 1) * 8;
    colpos[ct] = chunk * 16 + s16;                  // the column (within the tile) this lane accumulates
  }
  int a_off[4];                                     // x chunk kh * 8 + h * 4 + e of row lane % 32 (+ 32 per accumulator tile)
#pragma unroll
  for (int e = 0; e < 4; ++e) a_off[e] = W_BYTES + (lane & 31) * 256 + (((kh * 8 + h * 4 + e) ^ s16) * 16);

  f16v acc[MT][2];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][c][r] = 0.f;

  for (int b = 0; b < NS - 1; ++b)
    if (b < groups) issue(b);
#pragma unroll 1
  for (int i = 0; i < groups; ++i) {
    // loads return in order: batch i is complete when at most the batches issued after it are outstanding
    const int later = groups - 1 - i;
    if (later >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoadsPerGroup) : "memory");
    else if (later == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerGroup) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();                   // batch i is in LDS for everybody; everybody has left stage (i - 1) % NS
    asm volatile("" ::: "memory");
    if (i + NS - 1 < groups) issue(i + NS - 1);     // ... which the batch three groups ahead overwrites
    const unsigned char* st = smem + (size_t)(i % NS) * STAGE;
    h2 s2[2], zlo[2], zhi[2];                       // scale, zero point on the two nibble biases, of this lane's two columns
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const _Float16 sc = *reinterpret_cast<const _Float16*>(st + W_BYTES + X_BYTES + colpos[ct] * 2);
      const unsigned int zb = st[W_BYTES + X_BYTES + 512 + (colpos[ct] >> 1)];
      const _Float16 s = (n0 + colpos[ct] < N) ? sc : (_Float16)0.f;
      s2[ct] = h2{s, s};
      const unsigned int z = (zb >> ((colpos[ct] & 1) * 4)) & 15u;
      const unsigned int zz = z | (z << 16);
      zlo[ct] = as_h2(zz | mg.bias_lo);             // 1024 + z
      zhi[ct] = as_h2((zz << 4) | mg.bias_hi);      // 64 + z
    }
    // every LDS operand of the group goes to registers first: 4 transposing reads (q x column tile), 4 MT reads of x
    i32x2 pk[2][2];
    u32x4 ax[4][MT];
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) pk[q][ct] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(st + b_off[ct] + q * 2048));
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int t = 0; t < MT; ++t) ax[e][t] = *reinterpret_cast<const u32x4*>(st + a_off[e] + t * 32 * 256);
    // round e = (q, dword of the 8 bytes): 16 values of k for each lane half; its operands are built while the
    // MFMAs of round e - 1 run
    h8 fa[2][MT], fb[2][2];
    auto build = [&](int e, int slot) {
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) {
        const unsigned int w = (unsigned int)pk[e >> 1][ct][e & 1], w8 = w >> 8;
        const h2 p0 = (as_h2(and_or(w, mg.mask_lo, mg.bias_lo)) - zlo[ct]) * s2[ct];      // k0 k4
        const h2 p1 = (as_h2(and_or(w, mg.mask_hi, mg.bias_hi)) - zhi[ct]) * s2[ct];      // k1 k5
        const h2 p2 = (as_h2(and_or(w8, mg.mask_lo, mg.bias_lo)) - zlo[ct]) * s2[ct];     // k2 k6
        const h2 p3 = (as_h2(and_or(w8, mg.mask_hi, mg.bias_hi)) - zhi[ct]) * s2[ct];     // k3 k7
        fb[slot][ct] = h8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) fa[slot][t] = permute_k(ax[e][t]);
    };
    auto multiply = [&](int slot) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          acc[t][ct] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[slot][t], fb[slot][ct], acc[t][ct], 0, 0, 0);
    };
    build(0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int e = 0; e < 3; ++e) {
      multiply(e & 1);
      build(e + 1, (e + 1) & 1);
      // one MFMA (mask 0x008), then a share of the vector work (mask 0x002) of the next round: 26 + 4 MT instructions
#pragma unroll
      for (int m = 0; m < 2 * MT; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, (26 + 4 * MT + 2 * MT - 1) / (2 * MT), 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    multiply(1);
  }

  // ---- the two k halves meet in LDS as [k half][row][column]; then every thread owns four neighbouring columns.
  // Accumulator element r of tile t is row t*32 + (r/4)*8 + (lane/32)*4 + r%4.
  __syncthreads();
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = t * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
        red[((size_t)kh * BM + row) * RLD + colpos[ct]] = acc[t][ct][r];
      }
  __syncthreads();
  if (groups == 0) return;
#pragma unroll 1
  for (int e = tid; e < MT * 32 * (BN / 4); e += kThreads) {
    const int row = e >> 6, c4 = (e & 63) * 4;
    if (row >= M || n0 + c4 >= N) continue;         // N % 4 == 0: four columns are inside or outside as a whole
    const f32x4 v = *reinterpret_cast<const f32x4*>(red + (size_t)row * RLD + c4) +
                    *reinterpret_cast<const f32x4*>(red + ((size_t)BM + row) * RLD + c4);
    if (splits == 1) {
      h4 o = h4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
      if (residual) {                               // y = fp16(fp16(product) + residual); may alias y: same elements
        const h4 res = *reinterpret_cast<const h4*>(residual + (size_t)row * N + n0 + c4);
        o = h4{(_Float16)((float)o[0] + (float)res[0]), (_Float16)((float)o[1] + (float)res[1]),
               (_Float16)((float)o[2] + (float)res[2]), (_Float16)((float)o[3] + (float)res[3])};
      }
      *reinterpret_cast<h4*>(y + (size_t)row * N + n0 + c4) = o;
    } else {
      *reinterpret_cast<f32x4*>(partial + ((size_t)split * M_total + m0 + row) * N + n0 + c4) = v;
    }
  }
}

// y[m,n] = fp16(sum over splits, in split order); four columns per thread (N % 4 == 0).
__global__ __launch_bounds__(256) void gemm_w4a16_combine_kernel(const float* __restrict__ partial, _Float16* y,
                                                                  long long count4, long long split_stride, int splits,
                                                                  const _Float16* residual) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= count4) return;
  // eight splits at a time: all eight loads are issued before the first is added (a loop of load-then-add runs one
  // memory round trip per split); the additions keep the split order.  Past the last split a load repeats split 0
  // and is not added.
  f32x4 t = *reinterpret_cast<const f32x4*>(partial + i * 4);
  for (int s0 = 1; s0 < splits; s0 += 8) {
    f32x4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int s = s0 + j < splits ? s0 + j : 0;
      v[j] = *reinterpret_cast<const f32x4*>(partial + s * split_stride + i * 4);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (s0 + j < splits) t += v[j];
  }
  h4 out = h4{(_Float16)t[0], (_Float16)t[1], (_Float16)t[2], (_Float16)t[3]};
  if (residual) {                    // y = fp16(fp16(product) + residual); residual may be y itself
    const h4 res = *reinterpret_cast<const h4*>(residual + i * 4);
    out = h4{(_Float16)((float)out[0] + (float)res[0]), (_Float16)((float)out[1] + (float)res[1]),
             (_Float16)((float)out[2] + (float)res[2]), (_Float16)((float)out[3] + (float)res[3])};
  }
  *reinterpret_cast<h4*>(y + i * 4) = out;
}

// Number of K-splits: as many blocks as the chip holds at once (one per compute unit), but at least
// two groups per block, no more partial-tile bytes than twice the weight bytes (every split adds an fp32 copy of
// the output to the traffic; 256 rows over 4096 x 4096: 4 splits 23.1 us, the 2 that the weight bytes allow 28.3),
// and no more than the scratch space allows.  The rule lands on the measured
// optimum at M = 64 on MI355X: 8 splits for 4096x4096 and 11008x4096 (two 32-row blocks each), 5 for 4096x11008,
// 2 for 4096x32000.
int choose_splits(int rows, int N, int K, size_t scratch_bytes, int compute_units) {
  const int col_tiles = (N + BN - 1) / BN, G = K / GK;
  int s = (512 / kThreads) * compute_units / col_tiles;      // blocks that are resident at once
  if (s > G / 2) s = G / 2;
  const size_t per_split = (size_t)rows * N * sizeof(float);
  const size_t weight_bytes = (size_t)K * N / 2;
  if ((size_t)s * per_split > 2 * weight_bytes) s = (int)(2 * weight_bytes / per_split);
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
  ART_REQUIRE(k_splits >= 0 && k_splits < 0x300, "art_gemm_w4a16: k_splits must be 0 (library's choice) or 1..255, plus 256 x the rows-per-block code (got %d)", k_splits);
  ART_REQUIRE(((uintptr_t)residual_dev % 8) == 0, "art_gemm_w4a16: the residual must be 8-byte aligned");
  ART_REQUIRE(!art::overlaps(x_dev, (size_t)M * K * 2, y_dev, (size_t)M * N * 2), "art_gemm_w4a16: y must not overlap x");
  ART_REQUIRE(x_dev && qweight_dev && scales_dev && qzeros_dev && y_dev, "art_gemm_w4a16: null pointer");
  ART_REQUIRE(M >= 1, "art_gemm_w4a16: M must be positive (got %d)", M);
  ART_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 16 == 0, "art_gemm_w4a16: need K %% 128 == 0 and N %% 16 == 0 (K=%d N=%d)", K, N);
  ART_REQUIRE(((uintptr_t)qweight_dev % 16) == 0 && ((uintptr_t)x_dev % 16) == 0 && ((uintptr_t)qzeros_dev % 8) == 0 &&
                  ((uintptr_t)y_dev % 8) == 0 && ((uintptr_t)scales_dev % 4) == 0,
              "art_gemm_w4a16: x and qweight must be 16-byte aligned, qzeros and y 8-byte aligned, scales 4-byte aligned");
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
  // Up to kMaxRowBlocks row blocks go into one launch (they share the weight stream through L2, and the K-splits
  // are combined once); longer batches take several passes over the weights.
  // Rows per block: 64, or 32 where twice the blocks fill the chip better than twice the K-splits do - a block of 32
  // rows unpacks the same weights for half the matrix instructions, but every K-split it saves is an fp32 copy of
  // the output less to write and read back.  The caller's choice arrives in the upper bits of k_splits.
  constexpr int kMaxRowBlocks = 8;
  const int want_rows = k_splits >> 8;              // 0: library's choice, 1: 32-row blocks, 2: 64-row blocks
  k_splits &= 0xff;
  ART_REQUIRE(want_rows <= 2, "art_gemm_w4a16: rows-per-block code must be 0, 1 or 2 (got %d)", want_rows);
  int block_rows = BM;
  if (want_rows == 1 || M <= 32) block_rows = 32;
  else if (want_rows == 0 && (M <= 64 || (M <= 128 && K <= 8192))) {
    // measured at M = 64 and 128 on MI355X: 32-row blocks win where one block per compute unit then covers at least
    // four K-splits' worth of (column tile, row block) pairs (M = 64: up to 8192 columns, M = 128: 4096), and lose
    // where they would need a second round of blocks; beyond 64 rows also where the loop over K is long (128 rows
    // over 11008 x 4096: 27.2 us against 25.8 with 64-row blocks; over 4096 x 4096: 17.3 against 19.7)
    if (col_tiles * ((M + 31) / 32) * 4 <= compute_units) block_rows = 32;
  }
  for (int m0 = 0; m0 < M; m0 += block_rows * kMaxRowBlocks) {
    const int rows = M - m0 < block_rows * kMaxRowBlocks ? M - m0 : block_rows * kMaxRowBlocks;
    const int m_blocks = (rows + block_rows - 1) / block_rows;
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
    if (block_rows == 32)
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
