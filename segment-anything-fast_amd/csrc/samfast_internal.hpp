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

// Tuning knobs: each is an environment variable read ONCE (at the first query of any knob), after
// which samfast_bench_set_knob (include/samfast_bench.h) is the only way to change it.
enum Knob {
  KNOB_GEMM_TM,           // SAMFAST_GEMM_TM: 4 = 256 x 256 tiles in the two-per-CU kernel
  KNOB_GEMM_WG3,          // SAMFAST_GEMM_WG3: 0 = two workgroups per CU instead of three
  KNOB_GEMM_TILE,         // SAMFAST_GEMM_TILE: 64 / 128 forces the small / large tile of the three-per-CU kernel
  KNOB_GEMM_SMALL_BELOW,  // SAMFAST_GEMM_SMALL_BELOW: tile count below which the small tile is taken
  KNOB_GEMM_PERSIST,      // SAMFAST_GEMM_PERSIST: 0 off, 1 where it pays, 2 wherever it is built
  KNOB_GEMM_PERSIST_SKEW, // SAMFAST_GEMM_PERSIST_SKEW: start delay of every second resident workgroup, 64 cycles per k tile
  KNOB_GEMM_PERSIST_PRIO, // SAMFAST_GEMM_PERSIST_PRIO: 0 = no wave priority changes in the persistent kernel
  KNOB_GEMM_SPLITK,       // SAMFAST_GEMM_SPLITK: 0 off, 1 where it pays (launches that leave the GPU half empty)
  KNOB_ATTN_WAVES,        // SAMFAST_ATTN_WAVES: 4 / 8 wavefronts per global-attention workgroup
  KNOB_ATTN_WINDOW_ROWS,  // SAMFAST_ATTN_WINDOW_ROWS: 1 = window keys as grid rows padded to 16 (attn_window_rows_kernel) where built
  KNOB_SPARSE_PERSIST,    // SAMFAST_SPARSE_PERSIST: 2:4 GEMM, 0 = one workgroup per tile (default), 1 = resident workgroups from two tiles each on, 2 wherever built
  KNOB_COUNT
};
constexpr int kKnobUnset = INT32_MIN;
int knob(Knob k);                      // kKnobUnset when neither the environment nor a setter gave a value
static inline int knob_or(Knob k, int dflt) {
  const int v = knob(k);
  return v == kKnobUnset ? dflt : v;
}

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

// GELU(x) = x * Phi(x), written so that the negative side keeps its relative accuracy:
//   gelu(x) = max(x, 0) - |x| * h,   h = Phi(-|x|) = 2^P(|x|),
// P = degree-7 least-squares fit (Chebyshev nodes) of log2 Phi(-z) on [0, 6]: |P - log2 Phi|
// < 7e-6, i.e. h to 5e-6 relative in fp32 Horner form - a result that differs from the
// correctly rounded bf16 value in about one of a thousand cases, by one step.  Beyond |x| = 6
// h is held at Phi(-6) = 1e-9.  One transcendental and ten other instructions per value: the two
// clamps are median-of-three instructions (|x| as a source modifier), which unlike fminf / fmaxf
// need no separate instruction to quiet a signalling NaN first.
SF_DEVICE float gelu_erf(float x) {
#pragma clang fp contract(fast)  // an approximation anyway: let the polynomial use FMAs
  const float ax = fabsf(x);
  const float z = __builtin_amdgcn_fmed3f(ax, 0.0f, 6.0f);
  float p = -1.88962623e-06f;
  p = fmaf(p, z, 6.26814010e-05f);
  p = fmaf(p, z, -9.38867933e-04f);
  p = fmaf(p, z, 8.53946133e-03f);
  p = fmaf(p, z, -5.40206871e-02f);
  p = fmaf(p, z, -4.58409777e-01f);
  p = fmaf(p, z, -1.15126915e+00f);
  p = fmaf(p, z, -9.99994340e-01f);
  const float h = __builtin_amdgcn_exp2f(p);
  return fmaf(-ax, h, __builtin_amdgcn_fmed3f(x, 0.0f, 3.4028234664e38f));
}

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2.  Map the hardware id to a logical id so that every XCD walks one
// contiguous range of logical ids (neighbours then share an L2).
SF_DEVICE unsigned int xcd_contiguous_id(unsigned int hw_id, unsigned int total) {
  const unsigned int per = (total + 7u) >> 3;
  return (hw_id & 7u) * per + (hw_id >> 3);
}

}  // namespace samfast
