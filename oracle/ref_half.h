// TEST INFRASTRUCTURE ONLY — part of the CPU oracle; never linked into or
// called from the shipped GPU path.
//
// IEEE binary16 storage type for CPU kernels.  Arithmetic is carried out in
// float and rounded to nearest-even after every operation, which is what a
// storage-only half type (`__fp16`, used by the reference's CPU backends:
// backends/c-scpu/config.py:49) does and what native fp16 hardware does for
// + - * / (float has enough bits that the double rounding is exact).
#pragma once
#include <stdint.h>
#include <string.h>
#include <math.h>

static inline float ref_h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, f;
  if (exp == 0) {
    if (man == 0) {
      f = sign;
    } else {  // subnormal: normalise
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      f = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    f = sign | 0x7f800000u | (man << 13);
  } else {
    f = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float out; memcpy(&out, &f, 4); return out;
}

static inline uint16_t ref_f2h(float x) {
  uint32_t f; memcpy(&f, &x, 4);
  uint32_t sign = (f >> 16) & 0x8000u;
  uint32_t a = f & 0x7fffffffu;
  if (a >= 0x7f800000u)  // inf / nan
    return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0));
  if (a >= 0x477ff000u)  // rounds to >= 65520 -> inf
    return (uint16_t)(sign | 0x7c00u);
  if (a < 0x33000001u)   // < 2^-25 (or exactly 2^-25 which ties to even 0)
    return (uint16_t)sign;
  int e = (int)(a >> 23) - 127;
  uint32_t man = (a & 0x7fffffu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;  // bits dropped
  uint32_t halfbit = 1u << (shift - 1);
  uint32_t rest = man & ((1u << shift) - 1);
  uint32_t q = man >> shift;
  if (rest > halfbit || (rest == halfbit && (q & 1))) ++q;
  uint32_t out;
  if (e < -14) out = q;                       // subnormal (q may carry into exponent 1: fine)
  else out = ((uint32_t)(e + 15) << 10) + (q - 0x400u);  // carry from q propagates into the exponent
  return (uint16_t)(sign | out);
}

#ifdef __cplusplus
struct half {
  uint16_t bits;
  half() : bits(0) {}
  half(float f) : bits(ref_f2h(f)) {}
  half(double f) : bits(ref_f2h((float)f)) {}
  half(int i) : bits(ref_f2h((float)i)) {}
  half(long long i) : bits(ref_f2h((float)i)) {}
  operator float() const { return ref_h2f(bits); }
};
static inline half operator+(half a, half b) { return half((float)a + (float)b); }
static inline half operator-(half a, half b) { return half((float)a - (float)b); }
static inline half operator*(half a, half b) { return half((float)a * (float)b); }
static inline half operator/(half a, half b) { return half((float)a / (float)b); }
static inline half operator-(half a) { half r; r.bits = a.bits ^ 0x8000u; return r; }
static inline bool operator<(half a, half b) { return (float)a < (float)b; }
static inline bool operator<=(half a, half b) { return (float)a <= (float)b; }
static inline bool operator==(half a, half b) { return (float)a == (float)b; }
static inline bool operator!=(half a, half b) { return (float)a != (float)b; }
#endif
