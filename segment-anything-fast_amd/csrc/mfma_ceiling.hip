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

}  // namespace samfast

extern "C" int samfast_bench_mfma_ceiling(int instruction, const void* operands, int workgroups,
                                          int iters, int64_t* host_ops_out, void* scratch_out, void* stream) {
  using namespace samfast;
  SF_REQUIRE(instruction == 0 || instruction == 1, "bench_mfma_ceiling: instruction must be 0 (int8) or 1 (bf16)");
  SF_REQUIRE(operands && scratch_out && aligned16(operands), "bench_mfma_ceiling: null or unaligned buffer");
  SF_REQUIRE(workgroups > 0 && workgroups <= (1 << 20) && iters > 0 && iters <= (1 << 24),
             "bench_mfma_ceiling: bad workgroup or iteration count");
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
