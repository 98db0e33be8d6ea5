// Shared device/host helpers of the samfast HIP kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "samfast.h"

namespace samfast {

// ---- error reporting (host) -------------------------------------------------
void set_error(const char* fmt, ...);
#define SF_FAIL(code, ...)              \
  do {                                  \
    ::samfast::set_error(__VA_ARGS__);  \
    return (code);                      \
  } while (0)
#define SF_REQUIRE(cond, ...)                              \
  do {                                                     \
    if (!(cond)) SF_FAIL(SAMFAST_E_INVALID, __VA_ARGS__);  \
  } while (0)

int check_launch(const char* what);

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- vector types -------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define SF_DEVICE __device__ __forceinline__

// bf16 <-> fp32 on raw bits
SF_DEVICE float bf16_lo_to_f32(unsigned int w) { return __uint_as_float(w << 16); }
SF_DEVICE float bf16_hi_to_f32(unsigned int w) { return __uint_as_float(w & 0xffff0000u); }
SF_DEVICE float bf16_bits_to_f32(unsigned short h) { return __uint_as_float(((unsigned int)h) << 16); }

// round-to-nearest-even fp32 -> bf16 bits (finite inputs; NaN kept quiet)
SF_DEVICE unsigned int f32_to_bf16_bits(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
// two fp32 -> packed bf16 pair, round to nearest even, one v_cvt_pk_bf16_f32
SF_DEVICE unsigned int pack_bf16x2(float lo, float hi) {
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2));
}

SF_DEVICE float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// value held by lane (lane ^ 32) of the same wavefront
SF_DEVICE float xor32(float v) { return __shfl_xor(v, 32, 64); }

// GELU(x) = x * Phi(x) with 1 - Phi(|x|) = 0.5 * erfc(|x| / sqrt 2) from the
// Abramowitz-Stegun 7.1.26 polynomial (|error| < 1.5e-7), written so that the negative
// side keeps its relative accuracy:  gelu(x) = max(x, 0) - |x| * h,
//   h = 0.5 * poly(t) * exp(-x^2 / 2),  t = 1 / (1 + p |x| / sqrt 2).
SF_DEVICE float gelu_erf(float x) {
#pragma clang fp contract(fast)  // an approximation anyway: let the polynomial use FMAs
  const float ax = fabsf(x);
  const float t = __builtin_amdgcn_rcpf(fmaf(ax, 0.3275911f * 0.70710678118654752f, 1.0f));
  const float w = ax * 0.84932180028801904f;  // sqrt(log2(e) / 2): exp(-x^2/2) = exp2(-w^2)
  const float e = __builtin_amdgcn_exp2f(-(w * w));
  float poly = 0.5f * 1.061405429f;            // the 0.5 of h is folded into the coefficients
  poly = fmaf(poly, t, 0.5f * -1.453152027f);
  poly = fmaf(poly, t, 0.5f * 1.421413741f);
  poly = fmaf(poly, t, 0.5f * -0.284496736f);
  poly = fmaf(poly, t, 0.5f * 0.254829592f);
  const float h = poly * t * e;
  return fmaf(-ax, h, fmaxf(x, 0.f));
}

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2.  Map the hardware id to a logical id so that every XCD walks one
// contiguous range of logical ids (neighbours then share an L2).
SF_DEVICE unsigned int xcd_contiguous_id(unsigned int hw_id, unsigned int total) {
  const unsigned int per = (total + 7u) >> 3;
  return (hw_id & 7u) * per + (hw_id >> 3);
}

}  // namespace samfast
