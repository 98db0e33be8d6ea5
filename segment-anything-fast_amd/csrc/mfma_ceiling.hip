// Measurement aid: what the gfx950 matrix pipe sustains with no data movement at all.
//
// Every wavefront runs `iters` rounds of eight independent MFMAs (eight accumulator sets, so no
// instruction waits for another's result) on operands that sit in registers for the whole kernel:
// no global loads, no LDS, no barriers.  The operands are read once from a caller-filled buffer,
// four different (A, B) pairs per lane that rotate over the accumulator sets, so the caller decides
// what the multipliers see: zeros / small constants, or random data like a real GEMM's.  The
// rate of this loop is the ceiling any kernel built from the same instruction can approach on
// the same data; on this part it depends on the data (the power limit lowers the clock when the
// operands toggle), which is why the buffer is an argument.
//
// The accumulators are folded into one word that is stored only if it equals a fixed pattern -
// a condition on the data that the compiler cannot decide, so the arithmetic stays, and that in
// practice never holds, so the kernel writes nothing.
#include "samfast_internal.hpp"
#include "samfast_bench.h"

namespace samfast {

constexpr int kCeilSets = 8;   // independent accumulator sets per wavefront
constexpr int kCeilPairs = 4;  // distinct (A, B) operand pairs per lane

// operands: (kCeilPairs, 2, 256) 16-byte vectors, indexed [pair][a|b][thread of the workgroup]
template <bool INT8>
__global__ __launch_bounds__(256, 2) void mfma_ceiling_kernel(const u32x4* __restrict__ operands,
                                                               int iters, int* out) {
  const int tid = threadIdx.x;
  u32x4 av[kCeilPairs], bv[kCeilPairs];
#pragma unroll
  for (int p = 0; p < kCeilPairs; ++p) {
    av[p] = operands[(2 * p) * 256 + tid];
    bv[p] = operands[(2 * p + 1) * 256 + tid];
  }
  int check = 0;
  if constexpr (INT8) {
    i32x16 acc[kCeilSets];
#pragma unroll
    for (int j = 0; j < kCeilSets; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < kCeilSets; ++j)
        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, av[j % kCeilPairs]),
                                                       __builtin_bit_cast(i32x4, bv[(j + j / kCeilPairs) % kCeilPairs]),
                                                       acc[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < kCeilSets; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) check ^= acc[j][r];
  } else {
    f32x16 acc[kCeilSets];
#pragma unroll
    for (int j = 0; j < kCeilSets; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < kCeilSets; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av[j % kCeilPairs]),
                                                         __builtin_bit_cast(bf16x8, bv[(j + j / kCeilPairs) % kCeilPairs]),
                                                         acc[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < kCeilSets; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) check ^= __float_as_int(acc[j][r]);
  }
  if (check == 0x5a17c0de) out[tid] = check;
}

// Second question: how much vector work runs in the shadow of another wavefront's MFMAs on the same
// SIMD?  512-thread workgroups, one per CU: wavefronts 0-3 run `mfma_rounds` rounds of eight
// independent v_mfma_f32_32x32x16_bf16, wavefronts 4-7 - their SIMD partners - run `vector_rounds`
// rounds of 64 independent vector instructions (v_fma_f32, or v_exp_f32 followed by a v_mul_f32
// that keeps the value in range).  Either count may be 0; timing the kernel with one side, the
// other side and both gives the overlap.
template <bool EXP>
__global__ __launch_bounds__(512, 1) void mfma_valu_overlap_kernel(const u32x4* __restrict__ operands,
                                                                   int mfma_rounds, int vector_rounds, int* out) {
  const int tid = threadIdx.x;
  int check = 0;
  if ((tid >> 6) < 4) {  // uniform per wavefront
    if (mfma_rounds <= 0) return;
    const bf16x8 a = __builtin_bit_cast(bf16x8, operands[tid]);
    const bf16x8 b = __builtin_bit_cast(bf16x8, operands[256 + tid]);
    f32x16 acc[kCeilSets];
#pragma unroll
    for (int j = 0; j < kCeilSets; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    for (int it = 0; it < mfma_rounds; ++it) {
#pragma unroll
      for (int j = 0; j < kCeilSets; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < kCeilSets; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) check ^= __float_as_int(acc[j][r]);
  } else {
    if (vector_rounds <= 0) return;
    const u32x4 o = operands[tid & 255];
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = __uint_as_float((o[i & 3] & 0x007fffffu) | 0x3f000000u) + 0.01f * i;  // [0.5, 1.2)
    const float c0 = __uint_as_float((o[0] & 0x007fffffu) | 0x3a000000u), c1 = 0.999f;  // data the compiler cannot fold
    for (int it = 0; it < vector_rounds; ++it) {
#pragma unroll
      for (int rep = 0; rep < (EXP ? 2 : 4); ++rep)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          x[i] = EXP ? __builtin_amdgcn_exp2f(x[i]) * 0.5f : fmaf(x[i], c1, c0);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) check ^= __float_as_int(x[i]);
  }
  if (check == 0x5a17c0de) out[tid] = check;
}

}  // namespace samfast

extern "C" int samfast_bench_mfma_valu_overlap(int vector_kind, const void* operands, int workgroups,
                                               int mfma_rounds, int vector_rounds, void* scratch_out, void* stream) {
  using namespace samfast;
  SF_REQUIRE(vector_kind == 0 || vector_kind == 1, "bench_mfma_valu_overlap: vector_kind must be 0 (fma) or 1 (exp + mul)");
  SF_REQUIRE(operands && scratch_out && aligned16(operands), "bench_mfma_valu_overlap: null or unaligned buffer");
  SF_REQUIRE(workgroups > 0 && workgroups <= (1 << 20) && mfma_rounds >= 0 && mfma_rounds <= (1 << 24) &&
                 vector_rounds >= 0 && vector_rounds <= (1 << 24),
             "bench_mfma_valu_overlap: bad workgroup or round count");
  // a launch stays below about a second of GPU time
  SF_REQUIRE((int64_t)workgroups * ((int64_t)mfma_rounds + vector_rounds) <= (1ll << 27),
             "bench_mfma_valu_overlap: workgroups * rounds must not exceed 2^27");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const u32x4* ops = reinterpret_cast<const u32x4*>(operands);
  if (vector_kind == 0)
    hipLaunchKernelGGL((mfma_valu_overlap_kernel<false>), dim3(workgroups), dim3(512), 0, s, ops, mfma_rounds,
                       vector_rounds, (int*)scratch_out);
  else
    hipLaunchKernelGGL((mfma_valu_overlap_kernel<true>), dim3(workgroups), dim3(512), 0, s, ops, mfma_rounds,
                       vector_rounds, (int*)scratch_out);
  return check_launch("mfma_valu_overlap_kernel");
}

extern "C" int samfast_bench_mfma_ceiling(int instruction, const void* operands, int workgroups,
                                          int iters, int64_t* host_ops_out, void* scratch_out, void* stream) {
  using namespace samfast;
  SF_REQUIRE(instruction == 0 || instruction == 1, "bench_mfma_ceiling: instruction must be 0 (int8) or 1 (bf16)");
  SF_REQUIRE(operands && scratch_out && aligned16(operands), "bench_mfma_ceiling: null or unaligned buffer");
  SF_REQUIRE(workgroups > 0 && workgroups <= (1 << 20) && iters > 0 && iters <= (1 << 24),
             "bench_mfma_ceiling: bad workgroup or iteration count");
  // a launch stays below about a second of GPU time
  SF_REQUIRE((int64_t)workgroups * iters <= (1ll << 27), "bench_mfma_ceiling: workgroups * iters must not exceed 2^27");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const u32x4* ops = reinterpret_cast<const u32x4*>(operands);
  if (instruction == 0)
    hipLaunchKernelGGL((mfma_ceiling_kernel<true>), dim3(workgroups), dim3(256), 0, s, ops, iters, (int*)scratch_out);
  else
    hipLaunchKernelGGL((mfma_ceiling_kernel<false>), dim3(workgroups), dim3(256), 0, s, ops, iters, (int*)scratch_out);
  // arithmetic operations the launch executes: 2 * 32 * 32 * k per MFMA, k = 32 (int8) or 16 (bf16)
  if (host_ops_out)
    *host_ops_out = (int64_t)workgroups * 4 * iters * kCeilSets * 2 * 32 * 32 * (instruction == 0 ? 32 : 16);
  return check_launch("mfma_ceiling_kernel");
}
