"""Device check-up programs of the AutoRT package, run as modules (README.md:43-55, 128-150):

    python -m autort.utils.memtest          device memory bandwidth of a plain copy
    python -m autort.utils.fp32test         fp32 multiply-add rate of the vector units
    python -m autort.utils.mmtest           `gemm_f32` (C[M,N] +=! A[M,K] * B[K,N]) through autort.export
    python -m autort.utils.export -s 20     tunes `gemm_f32` and writes its module file for later sessions

Their source is not in the reference tree (they ship in its wheel); what they print follows the README."""

GEMM_F32_IR = 'output0[M, N] +=! input0[M, K] * input1[K, N]'
GEMM_F32_INPUTS = ['input0=float32[M:4096, K:4096]', 'input1=float32[K:4096, N:4096]']
