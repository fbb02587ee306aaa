/*
 * antares_amd.h — flat C ABI of libantares_amd.so, the MI355X (gfx950) runtime
 * and kernel library behind the AutoRT / Antares operator surface.
 *
 * Every function returns 0 on success and non-zero on failure; the message of
 * the last failure on the calling thread is available from art_last_error().
 * Nothing here calls exit().  All pointers named *_dev are raw device
 * addresses (e.g. torch `tensor.data_ptr()`); `stream` is a hipStream_t passed
 * as void* (NULL = the default stream).  The caller owns all tensor memory;
 * the library owns loaded modules for the life of the process and internal
 * workspaces (64 MiB each) that it never frees.
 *
 * The kernels that split K or work in two passes (art_gemv_w4a16*, art_gemv_gptq,
 * art_gemm_w4a16, art_partition_even_first_i32) keep their partial results in
 * a workspace.  Launches on one stream are ordered and share one; every stream
 * gets a workspace of its own the first time such a kernel is launched on it
 * (art_init allocates the default stream's), so launches on different streams
 * do not disturb each other.  At most 40 streams per device may do so, and a
 * stream's first such launch must happen outside graph capture (it allocates).
 * Host calls may come from several threads (the reference allows one: static
 * state, no locks, frameworks/pytorch/main_ops.cc:14-15).  Launches leave
 * the workspace clean, also when their inputs hold NaN or infinities.
 *
 * The first group replaces the reference's header-only `namespace ab` device
 * runtime and its ExecutionModule; the second group are typed entry points for
 * the hand-written kernels that replace generated code on the hot path; the
 * last group (calibration launches) is measurement tooling, not part of the
 * drop-in surface.
 */
#ifndef ANTARES_AMD_H_
#define ANTARES_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------- runtime */

typedef struct art_module art_module;   /* a loaded code object            */
typedef struct art_func art_func;       /* one kernel inside a module      */

typedef struct art_props {
  char name[256];
  char arch[64];              /* e.g. "gfx950" */
  int compute_units;
  int wavefront_size;
  int max_threads_per_block;
  int lds_bytes_per_block;
  int clock_khz;
  int memory_clock_khz;
  int memory_bus_width_bits;
  int l2_bytes;
  size_t total_memory_bytes;
} art_props;

/* Bind the calling process to `device` and allocate the library workspace.
 * Idempotent.  Replaces ab::init (backends/c-rocm/include/backend.hpp:51). */
int art_init(int device);

/* Message of the last error on this thread ("" if none). */
const char* art_last_error(void);

/* Device properties; replaces the device-property probe used to fill
 * hardware configs (engine/cuda_properties.cc:35-52). */
int art_device_props(art_props* out);

/* Compile HIP source text for `arch` (NULL = "gfx950") into a code object.
 * Works without a GPU.  `*blob` is owned by the library until art_blob_free.
 * Replaces ab::moduleCompile (backends/c-rocm/include/backend.hpp:116-158),
 * which forks `hipcc --genco`; this one compiles in-process. */
int art_module_compile(const char* hip_source, const char* arch, void** blob, size_t* size);
void art_blob_free(void* blob);
/* Text of the compiler log of the last art_module_compile on this thread. */
const char* art_compile_log(void);

/* Load a code object; replaces ab::moduleLoad (backend.hpp:161-170). */
int art_module_load(const void* image, size_t size, art_module** out);
/* The same from a code-object file (what `hipcc --genco` or art_module_compile wrote). */
int art_module_load_file(const char* path, art_module** out);
int art_module_unload(art_module* module);

/* Look a kernel up by name; replaces ab::moduleGetFunction (backend.hpp:172-197). */
int art_get_function(art_module* module, const char* name, art_func** out);

/* Launch with `nargs` kernel arguments, each held in one 64-bit slot of
 * `args` (device pointers as they are, integers widened) — the slot convention
 * of the reference's launch path (graph_evaluator/execute_module.hpp:340-352).
 * Replaces ab::launchKernel (backend.hpp:199-219). */
int art_launch(art_func* func, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz,
               unsigned lds_bytes, void* stream, const uint64_t* args, int nargs);

/* Timing and synchronisation; replace ab::recordTime / convertToElapsedTime /
 * synchronize (backend.hpp:233-252). */
int art_event_create(void** event);
int art_event_record(void* event, void* stream);
int art_event_elapsed_ms(void* start, void* stop, float* ms);   /* synchronises on `stop` */
int art_event_destroy(void* event);
int art_stream_synchronize(void* stream);

/* Device memory and host<->device copies for callers that bring no allocator of their own (the
 * reference's evaluator).  Replace ab::alloc / release / memcpyHtoD / memcpyDtoH (backend.hpp:92-114,
 * 221-232); the power-of-two bucket cache of ab::alloc stays on the caller's side (include/c-mi355x/backend.hpp).
 * The copies are asynchronous on `stream`; pair them with art_stream_synchronize. */
int art_alloc(size_t bytes, void** out_dev);
int art_free(void* dev);
int art_memcpy_htod(void* dst_dev, const void* src_host, size_t bytes, void* stream);
int art_memcpy_dtoh(void* dst_host, const void* src_dev, size_t bytes, void* stream);
/* Device to device, asynchronous on `stream`; replaces ab::memcpyDtoD (backend.hpp:225-227). */
int art_memcpy_dtod(void* dst_dev, const void* src_dev, size_t bytes, void* stream);

/* ---------------------------------------------------- hand-written kernels */

/* Weight-only int4 GEMV / skinny GEMM, group size 128 along K:
 *     y[m,n] = sum_k x[m,k] * (q[k,n] - z[k/128,n]) * s[k/128,n]
 * x: fp16 [M,K]; qweight: uint8 [K/2,N], low nibble = even k; scales: fp16
 * [K/128,N]; qzeros: uint8 [K/128,N/2], low nibble = even n; y: fp16 [M,N].
 * fp32 accumulation.  M <= 8 here (decode); K % 128 == 0, N % 16 == 0.
 * The sums over the K/512 slices of k meet as fixed-point numbers (steps of
 * 2^-22): a slice whose sum is NaN, infinite or beyond 2^24 / (K/512) in
 * magnitude turns y[m,n] into NaN (its exact value would be far outside fp16).
 * Replaces the kernel the reference generates from the dequant+GEMV program
 * of samples/05_llama2_7b_int4.py:135-144 (antares/default_codegen.py:13). */
int art_gemv_w4a16(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                   void* y_dev, int M, int K, int N, void* stream);

/* The same three operators with the launch parameter a tuning run may vary (the knobs that
 * `config="tune:N"` searches, as the reference's tuner searches the knobs of its schedules:
 * tuner/OpEvo/main.py:467-616, antares/common.py:81-118).  0 always means the library's own choice, and results do
 * not depend on the parameter beyond fp32 re-association.
 *   k_per_block:   256, 512 or 1024 values of k per block of the int4 GEMV (4 or 8 packed rows per lane in four
 *                  wavefronts, or 8 rows in eight wavefronts; 1024 needs M = 1): fewer k per block = more blocks and
 *                  more returning atomics per column;
 *   k_splits:      number of K-splits of the int4 GEMM, 1..255 (clamped to K/128 and to what the workspace holds),
 *                  plus 256 for blocks of 32 rows or 512 for blocks of 64 rows (neither: the library picks; batches of
 *                  up to 32 rows always take 32-row blocks): 32-row blocks are twice as many and need fewer K-splits,
 *                  i.e. fewer fp32 copies of the output written and read back, but unpack every weight twice;
 *   max_blocks:    cap on the blocks of the partition, 64..16384 (each walks its span tile by tile). */
int art_gemv_w4a16_tuned(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                         void* y_dev, int M, int K, int N, int k_per_block, void* stream);
/* The two factors behind k_per_block as independent knobs: rows_per_lane 4 or 8 (packed rows a lane loads before it
 * multiplies: 8 or 16 values of k), waves_per_block 4 or 8 (a block's k range is 16 x rows_per_lane x waves_per_block:
 * 256 .. 1024); 0 = the library's choice for either.  Eight wavefronts need M = 1. */
int art_gemv_w4a16_knobs(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                         void* y_dev, int M, int K, int N, int rows_per_lane, int waves_per_block, void* stream);
int art_gemm_w4a16_tuned(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                         void* y_dev, int M, int K, int N, int k_splits, void* stream);
int art_partition_even_first_i32_tuned(const void* in_dev, void* out_dev, long long n, int max_blocks, void* stream);
/* art_gemm_w4a16_tuned with the residual add that follows a projection (samples/05_llama2_7b_int4.py:168,173) folded
 * into the last pass: y = fp16(fp16(product) + residual).  residual_dev: fp16 [M,N], may be y itself, may be NULL. */
int art_gemm_w4a16_residual(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                            void* y_dev, const void* residual_dev, int M, int K, int N, int k_splits, void* stream);

/* art_gemv_w4a16 for callers that cannot allocate device memory or let a library do it (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * operands, constraints and results (bit for bit) as art_gemv_w4a16, with M in 1..4 and M * N <= 131072: the
 * split-K accumulators live in a 1 MiB array that is part of the library's code object on every GPU, so the call
 * allocates nothing, on any stream, first call included (art_init(device) must have run once on that device).  Larger
 * sizes are refused with an error.  All calls on one GPU share that array: calls that overlap in time on one GPU
 * (two streams) race; order them on one stream or with events. */
int art_gemv_w4a16_noalloc(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                           void* y_dev, int M, int K, int N, void* stream);

/* The same product for any M >= 1 on the matrix cores (prefill batches; the samples' decode loop uses
 * M = 1): operands, layouts and constraints as for art_gemv_w4a16, plus qzeros and y 8-byte aligned.
 * Rows are processed 64 at a time; each pass reads the weights once.  K-splits are combined through the
 * library workspace in a fixed order, so results do not depend on timing. */
int art_gemm_w4a16(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                   void* y_dev, int M, int K, int N, void* stream);

/* The same GEMV (M = 1) with the operators that surround a projection in the
 * decode step of samples/05_llama2_7b_int4.py:146-177 folded in:
 *   norm_weight_dev != NULL: x is first replaced by
 *       fp16(x * rsqrt(sum(x^2)/K + eps) * norm_weight)                     (lines :128-131,:150,:169)
 *   residual_dev != NULL:    y = fp16(fp16(product) + residual)             (lines :168,:173)
 *   swiglu_input != 0:       x_dev holds gate | up (2*K values) and the product is taken with
 *       fp16(silu(gate[k]) * up[k])                                         (line :171)
 * y may alias residual and nothing else (x and y must not overlap in any of the three entry points).
 * Same roundings as the separate operators. */
int art_gemv_w4a16_fused(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                         void* y_dev, int K, int N, const void* norm_weight_dev, float eps, const void* residual_dev,
                         int swiglu_input, void* stream);

/* art_gemv_w4a16_fused with the sum of squares of a residual stream handed from the projection that writes the
 * stream to the projection that normalises it, so that the RMSNorm of lines :128-131 of the sample does not re-read
 * its input in every block.  A sum-of-squares buffer is 256 64-bit words of device memory, zero before its first use:
 *   sumsq_out_dev   != NULL: word [n / 128] receives, added up over the call, the squares of the y[n] written (as
 *                            rounded to fp16, after the residual add) in units of 2^-30; a square of 2^25 or more
 *                            (|y| >= 5793) or of a NaN counts as 2^25.  Integer sums: independent of timing.
 *   sumsq_clear_dev != NULL: that buffer is set to zero (the one the NEXT writer of a stream adds into).
 *   sumsq_in_dev    != NULL: needs norm_weight_dev and K <= 8192; sum(x^2) is taken as the sum of words
 *                            [0, K/128) of it instead of being computed from x.
 * The three must be different buffers.  With all three NULL this is art_gemv_w4a16_fused.  No counterpart in the
 * reference, which normalises in a separate operator. */
int art_gemv_w4a16_fused_sumsq(const void* x_dev, const void* qweight_dev, const void* scales_dev, const void* qzeros_dev,
                               void* y_dev, int K, int N, const void* norm_weight_dev, float eps, const void* residual_dev,
                               int swiglu_input, const void* sumsq_in_dev, void* sumsq_out_dev, void* sumsq_clear_dev,
                               void* stream);

/* The int4 GEMV (M = 1) over weights repacked once, when they are loaded - as the reference repacks its checkpoint
 * when it loads it (samples/05_llama2_7b_int4.py:34-66).  The packed form stores a tile of 16 columns over all of K
 * contiguously (records of 1024 values of k: weights in the order a wavefront reads them, then the scales and zero
 * points of the record's 8 groups), so one block owns its columns over the whole of K: no K-splits, no atomics,
 * no workspace.  Same arithmetic as art_gemv_w4a16 (fp32 accumulation in another order).  K % 128 == 0, K <= 16384,
 * N % 16 == 0.
 *   art_w4_prepack_bytes: size of the packed form (0 for a shape that is not supported).
 *   art_w4_prepack:       qweight / scales / qzeros as for art_gemv_w4a16 -> packed_dev (256-byte aligned).
 *   art_gemv_w4p:         y = x @ dequant(W), with the operators around a projection folded in as in
 *                         art_gemv_w4a16_fused: norm_weight_dev != NULL normalises x first (RMSNorm, lines :128-131),
 *                         residual_dev != NULL adds it to the rounded product (lines :168,:173; may alias y), and
 *                         swiglu_out != 0 takes columns 16t..16t+7 of the matrix as gate columns and 16t+8..16t+15
 *                         as the matching up columns and writes y[8t + j] = fp16(silu(gate) * up) (line :171; N/2
 *                         outputs; the caller interleaves the two matrices in blocks of 8 columns before packing).
 * Replaces the kernel the reference generates from samples/05_llama2_7b_int4.py:135-144. */
size_t art_w4_prepack_bytes(int K, int N);
int art_w4_prepack(const void* qweight_dev, const void* scales_dev, const void* qzeros_dev, void* packed_dev, int K, int N,
                   void* stream);
int art_gemv_w4p(const void* x_dev, const void* packed_dev, void* y_dev, int K, int N, const void* norm_weight_dev, float eps,
                 const void* residual_dev, int swiglu_out, void* stream);

/* The reference's own weight format (samples/05_llama2_7b_int4.py:135-139):
 * qweight int32 [K/8,N], eight nibbles per word along K (least significant
 * first), zero point fixed at 8, scales fp32 or fp16 [K/128,N], x and y fp32
 * or fp16 (x_f16 / scales_f16 select).  M = 1.  The sums over the K/1024
 * slices of k meet as fixed-point numbers, so y does not depend on the order in
 * which they arrive.  fp16 y: steps of 2^-22; a slice whose sum is NaN, infinite
 * or beyond 2^24 / (K/1024) in magnitude turns y[n] into NaN.  fp32 y: two
 * fixed-point words per column, exact for slice sums between 2^-34 and
 * 2^39 / (K/1024) in magnitude (smaller ones to within 2^-59, larger ones or
 * non-finite ones turn y[n] into NaN). */
int art_gemv_gptq(const void* x_dev, const void* qweight_dev, const void* scales_dev, void* y_dev,
                  int K, int N, int x_f16, int scales_f16, void* stream);

/* fp16 GEMM on the matrix cores: C[M,N] = A[M,K] @ B[K,N], all row-major, fp32
 * accumulation, fp16 output.  Any M; N % 8 == 0, K % 64 == 0 (tiles of 256 x 256; edge tiles are clamped).
 * Replaces the kernel the reference generates for `C[N,M] +=! A[N,K] * B[K,M]`
 * (AntaresIR.md:115; tiled schedule backends/c-rocm/schedule/standard/algo_tiling.py:35-98). */
int art_gemm_f16(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, void* stream);
/* The same with the block shape a tuning run may vary: threads = 256 (2 x 2 wavefronts of 128 x 128 outputs, one per
 * SIMD) or 512 (2 x 4 wavefronts of 128 x 64, two per SIMD), 0 = the library's choice (256). */
int art_gemm_f16_tuned(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, int threads, void* stream);

/* fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32): C[M,N] = A[M,K] @ B[K,N], all fp32, row-major; any M,
 * N % 4 == 0, K % 32 == 0; A and B 16-byte aligned, C must not overlap them.
 * Replaces the kernel the reference generates for `output0[N, M] +=! input0[N, K] * input1[K, M]` in float32
 * (AntaresIR.md:115), the `gemm_f32` operator its README tunes (README.md:128-150; tiled schedule
 * backends/c-rocm/schedule/standard/algo_tiling.py:35-98). */
int art_gemm_f32(const void* a_dev, const void* b_dev, void* c_dev, int M, int N, int K, void* stream);
/* `batch` such products in one launch, operands and results stored one after the other: C[b] = A[b] @ B[b].
 * Replaces the kernel the reference generates for `output0[B, N, M] +=! input0[B, N, K] * input1[B, K, M]`
 * (AntaresIR.md:121). */
int art_gemm_f32_batched(const void* a_dev, const void* b_dev, void* c_dev, int batch, int M, int N, int K, void* stream);
/* The same with either operand stored the other way round: trans_a != 0 means A is [K][M] (C = A^T B, M % 4 == 0),
 * trans_b != 0 means B is [N][K] (C = A B^T, the layout of a linear layer's weight; N need not be a multiple of 4 then).
 * Replaces the kernels the reference generates for `out[M, N] +=! a[K, M] * b[K, N]`, `... a[M, K] * b[N, K]` and
 * `... a[K, M] * b[N, K]` (the same tiled schedule, backends/c-rocm/schedule/standard/algo_tiling.py:35-98). */
int art_gemm_f32_ex(const void* a_dev, const void* b_dev, void* c_dev, int batch, int M, int N, int K, int trans_a, int trans_b,
                    void* stream);

/* Stable even-first partition of int32 values: all even values in input order,
 * then all odd values in input order.  Two launches (count, then rank + scatter),
 * 12 bytes of traffic per element, no atomics; at most 1024 blocks, each walking its span tile by tile
 * with the next tile's loads in flight.
 * Replaces the classify -> cumsum -> bucket pipeline of
 * samples/01_sort_even_first.py:9-27. */
int art_partition_even_first_i32(const void* in_dev, void* out_dev, long long n, void* stream);

/* Llama decode operators.  dtype codes: 0 = float32, 1 = float16.  They replace
 * the built-in operators the reference's samples call by name and whose source
 * is not in the reference tree (call sites: samples/05_llama2_7b_int4.py:128-131,
 * 157-158,165; samples/04_llama2_7b_fp16.py:83,96-97,103; samples/03_llama_tiny.py:66-70).
 *
 * art_rmsnorm: out[r,i] = x[r,i] * rsqrt(vsum[r] * inv_n + eps) * w[i], r < rows, i < n.
 *   vsum (fp32, one per row) is the caller's sum of squares as in the samples, or
 *   NULL to have the kernel compute it.
 * art_rotary: rotate-half form, x viewed as [heads, 2, head_dim/2]:
 *     out[h,0,j] = x[h,0,j] cos(t) - x[h,1,j] sin(t);  out[h,1,j] = x[h,1,j] cos(t) + x[h,0,j] sin(t)
 *   with t = pos * freq[j]; or, with interleaved != 0, the pairwise form over a
 *   flat vector: (x[2j], x[2j+1]) rotated by pos * freq[j], freq having one entry
 *   per pair of the whole vector.  pos is read from pos_dev (int32 on the device)
 *   when pos_dev != NULL, else taken from `pos`.  With out_row_stride > 0 the result
 *   is written at out + pos * out_row_stride elements (a row of a key cache of out_rows rows;
 *   a position outside 0..out_rows-1 writes nothing).
 * art_decode_attention: one query per head against a cache of seq_len positions:
 *     a[h,s] = att_f[0] * sum_m q[h,m] k[s,h,m];  p = softmax_s(a);  out[h,m] = sum_s p[h,s] v[s,h,m]
 *   q, out: [heads, 128]; k, v: [seq_len, heads, 128] (dense).  When pos_dev != NULL
 *   the length is *pos_dev + 1 and seq_len is the number of rows k and v have: a length
 *   beyond it reads nothing and returns NaN. */
int art_rmsnorm(const void* x_dev, const void* vsum_dev, const void* w_dev, void* out_dev, int rows, int n, float inv_n,
                float eps, int x_dtype, int w_dtype, int out_dtype, void* stream);
int art_rotary(const void* x_dev, const void* freq_dev, void* out_dev, int heads, int head_dim, int interleaved,
               const void* pos_dev, int pos, long long out_row_stride, int out_rows, int x_dtype, int freq_dtype,
               int out_dtype, void* stream);
/* One token's q | k | v (3 * heads * head_dim values): q rotated into q_out, k rotated into row
 * *pos_dev of key_cache, v copied into row *pos_dev of val_cache (caches: [max_positions, heads*head_dim];
 * a position outside 0..max_positions-1 writes nothing).  One launch for lines :155-158 and the v part of :151-152 of samples/05_llama2_7b_int4.py. */
int art_rope_qkv_store(const void* qkv_dev, const void* freq_dev, void* q_out_dev, void* key_cache_dev, void* val_cache_dev,
                       int heads, int head_dim, const void* pos_dev, int max_positions, int dtype, int freq_dtype,
                       void* stream);
/* art_rope_qkv_store for the `rows` tokens of a prompt (fp16; qkv [rows, 3 * heads * head_dim], row t at position
 * first_pos + t): rotated q into q_out [rows, heads, head_dim], rotated k and v into cache rows first_pos + t.  The
 * positions are host values here; they must fit the caches (max_positions rows). */
int art_rope_qkv_store_rows(const void* qkv_dev, const void* freq_dev, void* q_out_dev, void* key_cache_dev, void* val_cache_dev,
                            int rows, int heads, int head_dim, int first_pos, int max_positions, void* stream);
/* art_rope_qkv_store and art_decode_attention in one launch (fp16): block h rotates its head's q and k,
 * writes k and v into cache row *pos_dev and attends over rows 0..*pos_dev.  The caches have max_positions rows:
 * a position outside 0..max_positions-1 (a recorded graph replayed once too often) touches no cache row and
 * returns NaN. */
int art_decode_attention_rope(const void* qkv_dev, const void* inv_freq_dev, void* key_cache_dev, void* val_cache_dev,
                              const void* att_f_dev, void* out_dev, int heads, int head_dim, const void* pos_dev,
                              int max_positions, void* stream);
/* art_decode_attention_rope spread over `parts` blocks per head (1..8), each attending over a contiguous share of
 * the cached positions.  With parts == 1 out_dev receives the fp16 result as above.  With parts > 1 out_dev is a
 * float buffer [heads][parts][132] that receives, per (head, part), 128 unnormalised sums, the running maximum and
 * the running sum of exponentials (2 floats of padding); the merge
 *     out[h,m] = sum_p e^(max_p - max) acc_p[m] / sum_p e^(max_p - max) sum_p
 * is left to the consumer - art_gemv_w4a16_attn does it while it loads x, so the projection that follows the
 * attention (samples/05_llama2_7b_int4.py:165-168) needs no extra launch. */
int art_decode_attention_rope_split(const void* qkv_dev, const void* inv_freq_dev, void* key_cache_dev, void* val_cache_dev,
                                    const void* att_f_dev, void* out_dev, int heads, int head_dim, const void* pos_dev,
                                    int max_positions, int parts, void* stream);
/* y = fp16(product of the merged attention output with the int4 matrix) [+ residual]; partial_dev as written by
 * art_decode_attention_rope_split with the same `parts` (2..8), K = heads * 128. */
int art_gemv_w4a16_attn(const void* partial_dev, int parts, const void* qweight_dev, const void* scales_dev,
                        const void* qzeros_dev, void* y_dev, int K, int N, const void* residual_dev, void* stream);
/* art_gemv_w4a16_attn that also adds the squares of its outputs to sumsq_out_dev and clears sumsq_clear_dev (see
 * art_gemv_w4a16_fused_sumsq; either may be NULL). */
int art_gemv_w4a16_attn_sumsq(const void* partial_dev, int parts, const void* qweight_dev, const void* scales_dev,
                              const void* qzeros_dev, void* y_dev, int K, int N, const void* residual_dev,
                              void* sumsq_out_dev, void* sumsq_clear_dev, void* stream);
int art_decode_attention(const void* q_dev, const void* k_dev, const void* v_dev, const void* att_f_dev, void* out_dev,
                         int seq_len, int heads, int head_dim, const void* pos_dev, int q_dtype, int kv_dtype, int out_dtype,
                         void* stream);

/* Causal attention over a whole prompt (fp16, fp32 accumulation, matrix cores): query position t (row t of q,
 * [T, heads, 128]) attends to rows 0..t of k and v (row s at k_dev + s * kv_row_stride halves, holding [heads, 128]:
 * the rows of a key / value cache), out[t] = softmax_s(att_f[0] * q[t] . k[s]) v, [T, heads, 128].  The same
 * arithmetic as art_decode_attention applied to T positions at once (torch spelling: samples/03_llama_tiny.py:94-99);
 * replaces the two generated contraction kernels of a whole-prompt pass. */
int art_prefill_attention(const void* q_dev, const void* k_dev, const void* v_dev, const void* att_f_dev, void* out_dev,
                          int T, int heads, int head_dim, long long kv_row_stride, void* stream);

/* The bookkeeping between two decode steps of samples/05_llama2_7b_int4.py:196-201, one launch, all on the
 * device:  *pos += 1;  *token = (*pos < prompt_len) ? prompt[*pos] : argmax(logits[0..vocab));
 * x_out[0..dim) = embed[*token][0..dim).  logits, embed, x_out fp16; prompt, token, pos int32.  Ties of the
 * argmax go to the smallest index.  prompt_dev may be NULL when prompt_len == 0. */
int art_greedy_next(const void* logits_dev, int vocab, const void* prompt_dev, int prompt_len, void* token_dev,
                    void* pos_dev, const void* embed_dev, int dim, void* x_out_dev, void* stream);

/* Bytes of one library workspace (one per stream that launches split-K / two-pass kernels). */
size_t art_workspace_bytes(void);

/* Hands back the workspace the library allocated for `stream` on the current device (waits for the stream's work
 * first), so that a process that creates and destroys streams does not run out of the 40 slots: call it before
 * destroying a stream that launched a split-K / two-pass kernel.  A stream that has none is no error; the default
 * stream keeps its workspace.  A HIP graph recorded on a stream has that stream's workspace baked into its kernel
 * arguments: replay it on the stream it was recorded on (or order it there), and do not release that stream while
 * the graph is alive.  The reference frees nothing either way (its allocation cache never shrinks,
 * backends/c-rocm/include/backend.hpp:78-114). */
int art_release_stream(void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * Calibration launches - NOT part of the drop-in surface.  Nothing in the operator path calls them and a binding
 * of the reference needs none of them; they exist so that the figures under profiles/ can be reproduced with
 * committed code (`bench.py --calibrate-copy / --read-floor / --stream-floors / --phase-chain`): a copy of known size
 * to scale memory-traffic counters, and the floors of one launch that only reads, only writes, or meets inside
 * itself.  They have no counterpart in the reference.
 * ------------------------------------------------------------------------------------------------------------ */

/* Plain device copy kernel (dst, src: 16-byte aligned, bytes % 16 == 0); used
 * as the calibration workload for memory-traffic counters. */
int art_copy_bytes(void* dst_dev, const void* src_dev, size_t bytes, void* stream);

/* Read-only counterpart: one launch that fetches `bytes` (a multiple of 32768, at most 128 MiB; 16-byte aligned)
 * with the access pattern of the int4 GEMV's weight stream (blocks of 256 threads x eight 16-byte loads, rows of
 * 11008 bytes when bytes is a multiple of 11008 * 256, else of 128 bytes) and computes nothing.  Its duration is the
 * floor of any single launch that has to bring these bytes on chip.  sink_dev: 4096 words of scratch (never
 * written in practice). */
int art_read_bytes(const void* src_dev, size_t bytes, void* sink_dev, void* stream);

/* Store-only counterpart: one launch that writes `bytes` (a multiple of 16, 16-byte aligned) of the 32-bit `value`
 * with non-temporal 16-byte stores and reads nothing: the floor of a launch that has to write these bytes. */
int art_fill_bytes(void* dst_dev, size_t bytes, unsigned int value, void* stream);

/* Measurement only, no counterpart in the reference: what a grid-wide meeting inside ONE launch costs on this part,
 * i.e. what a persistent whole-token kernel would pay instead of a dependent launch.  256 resident blocks run `phases`
 * phases over src_dev (phases * phase_bytes bytes, at most src_bytes; phase_bytes a multiple of 32768, at most
 * 24 MiB); in every phase a block fetches its share with the access pattern of art_read_bytes, then all blocks meet
 * through one word per block in the stream's workspace (agent-scope stores and loads, no atomics, no fences, every
 * wait bounded).  mode 0: no loads; 1: a phase's loads follow the previous meeting; 2: the next phase's loads are
 * issued before the meeting.  status_dev: one 32-bit word, zero before the call, 1 afterwards if a block gave up
 * waiting (the chip was not free to hold all 256 blocks).  sink_dev: 256 words of scratch. */
int art_phase_chain_probe(const void* src_dev, size_t src_bytes, size_t phase_bytes, int phases, int mode, void* sink_dev,
                          void* status_dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* ANTARES_AMD_H_ */
