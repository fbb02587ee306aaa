/* TEST INFRASTRUCTURE ONLY — CPU oracle.  Only tests/, __graft_entry__.smoke()
 * and the cpu_baseline leg of bench.py load this library; the GPU path never
 * does.
 *
 * Plain-C restatements of the hot operators, written directly from the
 * reference's sample programs as the loop nests AntaresIR.md:6-67 prescribes.
 * They are independent of this repository's IR parser, so they also check the
 * generic loop-nest emitter (cpu_emit.py) on the same programs.
 *
 * Pinned by (see tests/test_oracle.py): README known answers for sigmoid and
 * the even-first sort; one-hot / all-equal special cases and a float64 numpy
 * recomputation for the int4 products; the closed forms stated at each
 * function for rmsnorm / rotary / attention.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "ref_half.h"

/* sigmoid_f32[N] = 1 - 1 / (1 + exp(data[N]))          (README.md:66) */
void ref_sigmoid_f32(const float* data, float* out, long long n) {
  for (long long i = 0; i < n; ++i) out[i] = 1.0f - 1.0f / (1.0f + expf(data[i]));
}

/* samples/01_sort_even_first.py:9-27, step by step:
 *   space[data[n] % 2, n] = 1                                  (classify, space zeroed)
 *   ids = cumsum(space.flat, int32) * space.flat               (host glue at :24)
 *   output[ids[n] - 1] = val[n % M]   when ids[n] > 0          (bucket, n over 2M) */
int ref_sort_even_first_i32(const int32_t* data, int32_t* output, long long m) {
  int32_t* space = (int32_t*)calloc((size_t)(2 * m), sizeof(int32_t));
  int32_t* ids = (int32_t*)malloc((size_t)(2 * m) * sizeof(int32_t));
  if (!space || !ids) { free(space); free(ids); return 1; }
  for (long long n = 0; n < m; ++n) space[(long long)(data[n] % 2) * m + n] = 1;
  int32_t run = 0;
  for (long long n = 0; n < 2 * m; ++n) { run += space[n]; ids[n] = run * space[n]; }
  for (long long n = 0; n < m; ++n) output[n] = 0;
  for (long long n = 0; n < 2 * m; ++n)
    if (ids[n] > 0) output[ids[n] - 1] = data[n % m];
  free(space); free(ids);
  return 0;
}

/* int4 g128 GEMV / GEMM with per-group zero points (the packed format of the
 * benchmark configuration):
 *   q[k,n]  = (qweight[k/2, n] >> (k%2*4)) & 15          uint8 [K/2,N], low nibble = even k
 *   z[g,n]  = (qzeros[g, n/2] >> (n%2*4)) & 15           uint8 [K/128,N/2], low nibble = even n
 *   w[k,n]  = fp16( scales[k/128,n] * fp16(q - z) )      the dequantised weight is a half, as in
 *                                                        samples/05_llama2_7b_int4.py:138 (.to(x.dtype))
 *   y[m,n]  = fp16( sum_k float(x[m,k]) * float(w[k,n]) )   fp32 accumulate in k order */
void ref_gemm_w4a16(const uint16_t* x, const uint8_t* qweight, const uint16_t* scales, const uint8_t* qzeros,
                    uint16_t* y, int M, int K, int N) {
  /* The column of dequantised weights and the rows of x are widened once; every y[m,n] is still the
   * k-ordered fp32 sum written above. */
  float* w = (float*)malloc((size_t)K * sizeof(float));
  float* xf = (float*)malloc((size_t)M * K * sizeof(float));
  for (size_t i = 0; i < (size_t)M * K; ++i) xf[i] = ref_h2f(x[i]);
  for (int n = 0; n < N; ++n) {
    for (int k = 0; k < K; ++k) {
      const int q = (qweight[(size_t)(k / 2) * N + n] >> (k % 2 * 4)) & 15;
      const int z = (qzeros[(size_t)(k / 128) * (N / 2) + n / 2] >> (n % 2 * 4)) & 15;
      const float s = ref_h2f(scales[(size_t)(k / 128) * N + n]);
      w[k] = ref_h2f(ref_f2h(s * ref_h2f(ref_f2h((float)(q - z)))));
    }
    for (int m = 0; m < M; ++m) {
      const float* xr = xf + (size_t)m * K;
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) acc += xr[k] * w[k];
      y[(size_t)m * N + n] = ref_f2h(acc);
    }
  }
  free(w);
  free(xf);
}

/* The sample's own program (samples/05_llama2_7b_int4.py:135-139), fp32 x:
 *   input1[s,n] = float((qweight[s/8, n] >> (s%8*4)) & 15)
 *   w[s,n]      = float(scales[s/128, n]) * (input1[s,n] - 8)
 *   y[n]       += x[s] * w[s,n]
 * scales_f16 selects half scales (promoted to float before the multiply). */
void ref_gemv_gptq_f32(const float* x, const int32_t* qweight, const void* scales, int scales_f16, float* y, int K, int N) {
  for (int n = 0; n < N; ++n) {
    float acc = 0.0f;
    for (int s = 0; s < K; ++s) {
      const float q = (float)((qweight[(size_t)(s / 8) * N + n] >> (s % 8 * 4)) & 15);
      const float sc = scales_f16 ? ref_h2f(((const uint16_t*)scales)[(size_t)(s / 128) * N + n])
                                  : ((const float*)scales)[(size_t)(s / 128) * N + n];
      acc += x[s] * (sc * (q - 8.0f));
    }
    y[n] = acc;
  }
}

/* RMSNorm as the samples call it (samples/05_llama2_7b_int4.py:128-131): the caller passes
 * vsum = sum x^2 and 1/N; out[i] = x[i] * rsqrt(vsum/N + eps) * w[i].  vsum == NULL: computed here.
 * Closed form used to pin it: sum_i (out[i]/w[i])^2 = N / (1 + eps*N/sum x^2). */
void ref_rmsnorm_f32(const float* x, const float* vsum, const float* w, float* out, int n, float inv_n, float eps) {
  float ss = 0.0f;
  if (vsum) ss = vsum[0];
  else for (int i = 0; i < n; ++i) ss += x[i] * x[i];
  const float r = 1.0f / sqrtf(ss * inv_n + eps);
  for (int i = 0; i < n; ++i) out[i] = x[i] * r * w[i];
}

/* Rotate-half RoPE on x viewed as [heads, 2, half] (the view the sample passes,
 * samples/05_llama2_7b_int4.py:157): theta_j = pos * inv_freq[j];
 * out[h,0,j] = x[h,0,j] cos - x[h,1,j] sin ; out[h,1,j] = x[h,1,j] cos + x[h,0,j] sin.
 * Pinned by: pos = 0 is the identity; every (j, j+half) pair keeps its norm; equals
 * x*cos + rotate_half(x)*sin of the HF Llama formulation. */
void ref_rotary_f32(const float* x, const float* inv_freq, float* out, int heads, int head_dim, int pos) {
  const int half = head_dim / 2;
  for (int h = 0; h < heads; ++h)
    for (int j = 0; j < half; ++j) {
      const float t = (float)pos * inv_freq[j], c = cosf(t), s = sinf(t);
      const float a = x[(size_t)h * head_dim + j], b = x[(size_t)h * head_dim + half + j];
      out[(size_t)h * head_dim + j] = a * c - b * s;
      out[(size_t)h * head_dim + half + j] = b * c + a * s;
    }
}

/* Interleaved-pair rotation (samples/03_llama_tiny.py:60,68-70): pair (2j, 2j+1) of a flat
 * vector is rotated by pos * coef[j]; coef has dim/2 entries. */
void ref_rotate_f32(const float* coef, const float* data, float* out, int dim, int pos) {
  for (int j = 0; j < dim / 2; ++j) {
    const float t = (float)pos * coef[j], c = cosf(t), s = sinf(t);
    const float a = data[2 * j], b = data[2 * j + 1];
    out[2 * j] = a * c - b * s;
    out[2 * j + 1] = a * s + b * c;
  }
}

/* Single-query attention, the torch spelling of samples/03_llama_tiny.py:94-99:
 * att[h,s] = (sum_m q[h,m] k[s,h,m]) * att_f ; softmax over s ; out[h,m] = sum_s att[h,s] v[s,h,m]. */
void ref_attention_f32(const float* q, const float* k, const float* v, float att_f, float* out, int S, int H, int D) {
  float* att = (float*)malloc((size_t)S * sizeof(float));
  for (int h = 0; h < H; ++h) {
    float mx = -INFINITY;
    for (int s = 0; s < S; ++s) {
      float d = 0.0f;
      for (int m = 0; m < D; ++m) d += q[(size_t)h * D + m] * k[((size_t)s * H + h) * D + m];
      att[s] = d * att_f;
      if (att[s] > mx) mx = att[s];
    }
    float sum = 0.0f;
    for (int s = 0; s < S; ++s) { att[s] = expf(att[s] - mx); sum += att[s]; }
    for (int m = 0; m < D; ++m) {
      float o = 0.0f;
      for (int s = 0; s < S; ++s) o += (att[s] / sum) * v[((size_t)s * H + h) * D + m];
      out[(size_t)h * D + m] = o;
    }
  }
  free(att);
}
