// Per-row symmetric int8 quantiser (bf16 -> int8 + fp32 scale), HBM-bound.
//
// One wavefront owns one row: the row is read once with 16-byte loads into
// registers, reduced to its absmax across the 64 lanes, then divided, rounded
// half-to-even and written back as 8-byte packs of int8.  Algorithmic traffic is
// 2 bytes read + 1 byte written per element plus 4 bytes of scale per row.
#include "samfast_internal.hpp"

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

constexpr int kQuantWavesPerBlock = 4;

template <int NCH>  // 16-byte chunks per lane: covers K <= NCH * 512
__global__ __launch_bounds__(64 * kQuantWavesPerBlock) void quant_rowwise_bf16_kernel(
    const unsigned short* __restrict__ x, int64_t ldx, int8_t* __restrict__ xq,
    float* __restrict__ sx, int64_t M, int K) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kQuantWavesPerBlock + (threadIdx.x >> 6);
  if (row >= M) return;  // whole wavefront leaves together
  const int nchunk = K >> 3;
  const u32x4* src = reinterpret_cast<const u32x4*>(x + row * ldx);

  u32x4 buf[NCH];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    u32x4 w = {0u, 0u, 0u, 0u};
    if (c < nchunk) w = src[c];
    buf[i] = w;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      amax = fmaxf(amax, fabsf(bf16_lo_to_f32(w[j])));
      amax = fmaxf(amax, fabsf(bf16_hi_to_f32(w[j])));
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));

  const float scale = fmaxf(amax, 1e-5f) / 127.0f;
  if (lane == 0) sx[row] = scale;

  u32x2* dst = reinterpret_cast<u32x2*>(xq + row * (int64_t)K);
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunk) {
      unsigned int packed[2] = {0u, 0u};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float lo = bf16_lo_to_f32(buf[i][j]);
        const float hi = bf16_hi_to_f32(buf[i][j]);
        // IEEE division, then round half to even, then clamp
        const int qlo = (int)fminf(fmaxf(rintf(lo / scale), -127.f), 127.f);
        const int qhi = (int)fminf(fmaxf(rintf(hi / scale), -127.f), 127.f);
        const int e = 2 * j;  // element index inside the chunk
        packed[e >> 2] |= ((unsigned int)(qlo & 0xff)) << (8 * (e & 3));
        packed[(e + 1) >> 2] |= ((unsigned int)(qhi & 0xff)) << (8 * ((e + 1) & 3));
      }
      u32x2 o = {packed[0], packed[1]};
      dst[c] = o;
    }
  }
}

template <int NCH>
static int launch_quant(const void* x, int64_t ldx, int8_t* xq, float* sx, int64_t M, int K,
                        hipStream_t stream) {
  const int64_t blocks = (M + kQuantWavesPerBlock - 1) / kQuantWavesPerBlock;
  hipLaunchKernelGGL(quant_rowwise_bf16_kernel<NCH>, dim3((unsigned int)blocks),
                     dim3(64 * kQuantWavesPerBlock), 0, stream,
                     reinterpret_cast<const unsigned short*>(x), ldx, xq, sx, M, K);
  return check_launch("quant_rowwise_bf16_kernel");
}

}  // namespace samfast

extern "C" int samfast_quant_rowwise_i8(const void* x, int64_t ldx, int8_t* xq, float* sx,
                                        int64_t M, int K, int dtype, void* stream) {
  using namespace samfast;
  SF_REQUIRE(x && xq && sx, "quant_rowwise: null pointer");
  SF_REQUIRE(M >= 0 && K > 0, "quant_rowwise: bad shape M=%lld K=%d", (long long)M, K);
  if (dtype != SAMFAST_BF16) SF_FAIL(SAMFAST_E_UNSUPPORTED, "quant_rowwise: only bf16 input");
  SF_REQUIRE(K % 8 == 0 && K <= 8192, "quant_rowwise: K=%d must be a multiple of 8, <= 8192", K);
  SF_REQUIRE(ldx >= K && ldx % 8 == 0, "quant_rowwise: ldx=%lld must be >= K and a multiple of 8",
             (long long)ldx);
  SF_REQUIRE(aligned16(x) && (reinterpret_cast<uintptr_t>(xq) & 7u) == 0,
             "quant_rowwise: x must be 16-byte and xq 8-byte aligned");
  SF_REQUIRE((M + 3) / 4 < (1ll << 31), "quant_rowwise: M too large");
  if (M == 0) return SAMFAST_OK;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int need = (K / 8 + 63) / 64;
  if (need <= 2) return launch_quant<2>(x, ldx, xq, sx, M, K, s);
  if (need <= 3) return launch_quant<3>(x, ldx, xq, sx, M, K, s);
  if (need <= 4) return launch_quant<4>(x, ldx, xq, sx, M, K, s);
  if (need <= 6) return launch_quant<6>(x, ldx, xq, sx, M, K, s);
  if (need <= 8) return launch_quant<8>(x, ldx, xq, sx, M, K, s);
  if (need <= 10) return launch_quant<10>(x, ldx, xq, sx, M, K, s);
  if (need <= 12) return launch_quant<12>(x, ldx, xq, sx, M, K, s);
  return launch_quant<16>(x, ldx, xq, sx, M, K, s);
}
