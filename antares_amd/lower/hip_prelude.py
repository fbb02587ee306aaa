"""Device-side helpers pasted in front of every generated HIP kernel.

Hand-written for gfx950 (64-wide wavefronts): DPP butterflies inside a 16-lane
row, v_readlane across the four rows, LDS across the wavefronts of a block.
These replace the macro block the reference prepends to its generated kernels
(backends/c-rocm/config.py:50-77).
"""

PRELUDE = r'''
// (the in-process compiler pre-includes the HIP device runtime)
typedef _Float16 half_t;
#define ART_DEV static __device__ __forceinline__
#define ART_MEM __device__ __forceinline__

template <class T, class U> ART_DEV T art_max(T a, U b) { return a < (T)b ? (T)b : a; }
template <class T, class U> ART_DEV T art_min(T a, U b) { return (T)b < a ? (T)b : a; }
template <class T> ART_DEV T art_abs(T a) { return a < (T)0 ? (T)(-a) : a; }
template <class T, class U> ART_DEV T bitwise_and(T a, U b) { return (T)(a & (T)b); }
template <class T, class U> ART_DEV T bitwise_or(T a, U b) { return (T)(a | (T)b); }
template <class T, class U> ART_DEV T bitwise_xor(T a, U b) { return (T)(a ^ (T)b); }
ART_DEV float art_rsqrt(float x) { return 1.0f / sqrtf(x); }
ART_DEV double art_rsqrt(double x) { return 1.0 / sqrt(x); }
ART_DEV float art_normcdf(float x) { return normcdff(x); }
ART_DEV double art_normcdf(double x) { return normcdf(x); }
ART_DEV half_t fp16_exp(half_t x) { return (half_t)expf((float)x); }
ART_DEV half_t fp16_log(half_t x) { return (half_t)logf((float)x); }
ART_DEV half_t fp16_sqrt(half_t x) { return (half_t)sqrtf((float)x); }
ART_DEV half_t fp16_rsqrt(half_t x) { return (half_t)(1.0f / sqrtf((float)x)); }
ART_DEV half_t fp16_sin(half_t x) { return (half_t)sinf((float)x); }
ART_DEV half_t fp16_cos(half_t x) { return (half_t)cosf((float)x); }
ART_DEV half_t fp16_floor(half_t x) { return (half_t)floorf((float)x); }
ART_DEV half_t fp16_ceil(half_t x) { return (half_t)ceilf((float)x); }
ART_DEV half_t fp16_max(half_t a, half_t b) { return a < b ? b : a; }
ART_DEV half_t fp16_min(half_t a, half_t b) { return b < a ? b : a; }

// ---- reduce operators
struct OpAdd { template <class T> ART_MEM T operator()(T a, T b) const { return (T)(a + b); } };
struct OpMul { template <class T> ART_MEM T operator()(T a, T b) const { return (T)(a * b); } };
struct OpMax { template <class T> ART_MEM T operator()(T a, T b) const { return a < b ? b : a; } };
struct OpMin { template <class T> ART_MEM T operator()(T a, T b) const { return b < a ? b : a; } };
struct OpAny { template <class T> ART_MEM T operator()(T a, T b) const { return (T)((a != (T)0) || (b != (T)0)); } };
struct OpAll { template <class T> ART_MEM T operator()(T a, T b) const { return (T)((a != (T)0) && (b != (T)0)); } };

// ---- wavefront reduction
// 32-bit payloads move through DPP inside each 16-lane row (xor 1, xor 2,
// half-mirror, mirror), then the four row results are read with v_readlane and
// combined in a fixed order, so every lane ends with the same, run-to-run
// identical value.
template <int CTRL> ART_DEV int art_dpp(int v) { return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false); }

template <class T> struct art_carrier { typedef T type; };
template <> struct art_carrier<half_t> { typedef float type; };
template <> struct art_carrier<signed char> { typedef int type; };
template <> struct art_carrier<unsigned char> { typedef int type; };
template <> struct art_carrier<short> { typedef int type; };

template <class T, class Op> ART_DEV T art_row_step(T v, Op op, int which) {
  int bits = __builtin_bit_cast(int, v), other;
  switch (which) {
    case 0: other = art_dpp<0xB1>(bits); break;    // quad_perm [1,0,3,2]
    case 1: other = art_dpp<0x4E>(bits); break;    // quad_perm [2,3,0,1]
    case 2: other = art_dpp<0x141>(bits); break;   // row_half_mirror
    default: other = art_dpp<0x140>(bits); break;  // row_mirror
  }
  return op(v, __builtin_bit_cast(T, other));
}

template <class T, class Op> ART_DEV T art_wave_reduce32(T v, Op op) {
  v = art_row_step(v, op, 0);
  v = art_row_step(v, op, 1);
  v = art_row_step(v, op, 2);
  v = art_row_step(v, op, 3);
  const int bits = __builtin_bit_cast(int, v);
  const T r0 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(bits, 0));
  const T r1 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(bits, 16));
  const T r2 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(bits, 32));
  const T r3 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(bits, 48));
  return op(op(r0, r1), op(r2, r3));
}

template <class T, class Op> ART_DEV T art_wave_reduce64(T v, Op op) {
  #pragma unroll
  for (int m = 1; m < 64; m <<= 1) v = op(v, __shfl_xor(v, m, 64));
  return v;
}

template <class T, class Op> ART_DEV T art_wave_reduce(T v, Op op) {
  typedef typename art_carrier<T>::type C;
  if constexpr (sizeof(C) == 4) {
    // the operator is applied in T after every exchange, so narrow types keep their own rounding
    struct Wrapped { Op op; ART_MEM C operator()(C a, C b) const { return (C)op((T)a, (T)b); } };
    return (T)art_wave_reduce32<C>((C)v, Wrapped{op});
  } else {
    return art_wave_reduce64<T>(v, op);
  }
}

// A compile-time integer as a function argument (selects a register set without run-time indexing).
template <int V> struct art_ic { static constexpr int value = V; };

// Reduction over a block of 256 threads (4 wavefronts); `smem` holds 4 values.
template <class T, class Op> ART_DEV T art_block_reduce(T v, Op op, T* smem) {
  v = art_wave_reduce(v, op);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) smem[wave] = v;
  __syncthreads();
  T r = op(op(smem[0], smem[1]), op(smem[2], smem[3]));
  __syncthreads();
  return r;
}
'''
