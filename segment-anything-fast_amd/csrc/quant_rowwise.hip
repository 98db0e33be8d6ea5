// Per-row symmetric int8 quantiser (bf16 -> int8 + fp32 scale), optionally preceded
// by LayerNorm over the row and a row gather (window partition).  HBM-bound.
//
// One wavefront owns one output row: the source row is read once with 16-byte loads
// into registers, (normalised,) reduced to its absmax across the 64 lanes, then
// scaled, rounded half-to-even and written back as 8-byte packs of int8.
// Algorithmic traffic: 2 bytes read + 1 byte written per element + 4 bytes of scale.
//
// q = rint(x / s) must equal the IEEE division bit for bit.  Most elements take a
// cheap route: r = x * (1/s) differs from x / s by a few ulp, so rint(r) can only
// differ when r lies within 1e-4 of a half-integer; only those elements (and their
// 8-element chunk) are redone with the true division.  |x| <= absmax makes
// |x / s| <= 127 by construction, so no clamp is needed.
#include "samfast_internal.hpp"

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

constexpr int kQuantWavesPerBlock = 4;

struct QuantArgs {
  const unsigned short* x;
  int64_t ldx;
  const unsigned short* gamma;  // LN only
  const unsigned short* beta;   // LN only
  const int32_t* src_row;       // LN only: source row per output row, -1 = all-zero row; may be null
  int8_t* xq;
  float* sx;
  int64_t M;
  int K;
  float eps;
  int kb64;  // 1: write xq K-block major, (K/64, M, 64)
};

SF_DEVICE float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
SF_DEVICE float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// 8 values -> 8 int8 codes packed in 8 bytes.
// Rounding: adding 1.5 * 2^23 to r (|r| <= 127) leaves rint(r) - half to even - in the low
// mantissa bits, so the low byte of the sum's bit pattern is the int8 code; subtracting the
// constant again gives rint(r) as a float for the near-tie test.
SF_DEVICE u32x2 quantize8(const float (&v)[8], float scale, float inv_scale) {
  constexpr float kMagic = 12582912.0f;  // 1.5 * 2^23
  float m[8];
  bool near_tie = false;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float r = v[e] * inv_scale;
    m[e] = r + kMagic;
    const float d = r - (m[e] - kMagic);  // r - rint(r), exact
    near_tie |= fabsf(d) > 0.5f - 1e-4f;
  }
  if (near_tie) {
#pragma unroll
    for (int e = 0; e < 8; ++e) m[e] = v[e] / scale + kMagic;  // IEEE division
  }
  unsigned int b[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) b[e] = __builtin_bit_cast(unsigned int, m[e]);
  // byte 0 of each of four words -> one word (v_perm_b32: selector bytes pick from {hi, lo})
  auto pack4 = [](unsigned int w0, unsigned int w1, unsigned int w2, unsigned int w3) {
    const unsigned int lo = __builtin_amdgcn_perm(w1, w0, 0x0c0c0400u);  // [w0.b0, w1.b0, 0, 0]
    const unsigned int hi = __builtin_amdgcn_perm(w3, w2, 0x04000c0cu);  // [0, 0, w2.b0, w3.b0]
    return lo | hi;
  };
  const u32x2 o = {pack4(b[0], b[1], b[2], b[3]), pack4(b[4], b[5], b[6], b[7])};
  return o;
}

template <int NCH, bool LN>  // 16-byte chunks per lane: covers K <= NCH * 512
__global__ __launch_bounds__(64 * kQuantWavesPerBlock) void quant_rowwise_bf16_kernel(QuantArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * kQuantWavesPerBlock + (threadIdx.x >> 6);
  if (row >= a.M) return;  // whole wavefront leaves together
  const int nchunk = a.K >> 3;
  // 8-byte chunk c of the row: row-major at row*K + 8c; K-block major at ((c/8)*M + row)*64 + (c%8)*8
  auto dst_of = [&](int c) {
    const int64_t off = a.kb64 ? ((int64_t)(c >> 3) * a.M + row) * 64 + (c & 7) * 8
                               : row * (int64_t)a.K + (int64_t)c * 8;
    return reinterpret_cast<u32x2*>(a.xq + off);
  };

  int64_t srow = row;
  if (LN && a.src_row) {
    srow = a.src_row[row];
    if (srow < 0) {  // a padding token: LayerNorm output replaced by zeros
      const u32x2 z = {0u, 0u};
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = lane + i * 64;
        if (c < nchunk) *dst_of(c) = z;
      }
      if (lane == 0) a.sx[row] = 1e-5f / 127.0f;
      return;
    }
  }
  const u32x4* src = reinterpret_cast<const u32x4*>(a.x + srow * a.ldx);

  // the row as floats, unpacked once: lane holds chunks lane, lane + 64, ... of 8 elements
  float f[NCH][8];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    u32x4 w = {0u, 0u, 0u, 0u};
    if (c < nchunk) w = src[c];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[i][2 * j] = bf16_lo_to_f32(w[j]);
      f[i][2 * j + 1] = bf16_hi_to_f32(w[j]);
    }
  }

  if (LN) {
    // two-pass mean / biased variance over the K real elements, fp32
    float s1 = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) s1 += f[i][2 * j] + f[i][2 * j + 1];
    const float mean = wave_sum(s1) / (float)a.K;
    float s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (lane + i * 64 < nchunk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float d0 = f[i][2 * j] - mean, d1 = f[i][2 * j + 1] - mean;
          f[i][2 * j] = d0;
          f[i][2 * j + 1] = d1;
          s2 += d0 * d0 + d1 * d1;
        }
      }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(s2) / (float)a.K + a.eps);
    const u32x4* g4 = reinterpret_cast<const u32x4*>(a.gamma);
    const u32x4* b4 = reinterpret_cast<const u32x4*>(a.beta);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        const u32x4 g = g4[c], b = b4[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float y0 = f[i][2 * j] * rstd * bf16_lo_to_f32(g[j]) + bf16_lo_to_f32(b[j]);
          const float y1 = f[i][2 * j + 1] * rstd * bf16_hi_to_f32(g[j]) + bf16_hi_to_f32(b[j]);
          const unsigned int y = pack_bf16x2(y0, y1);  // the bf16 values a separate LayerNorm would have stored
          f[i][2 * j] = bf16_lo_to_f32(y);
          f[i][2 * j + 1] = bf16_hi_to_f32(y);
        }
      }
    }
  }

  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(f[i][e]));
  amax = wave_max(amax);

  const float scale = fmaxf(amax, 1e-5f) / 127.0f;
  const float inv_scale = 1.0f / scale;
  if (lane == 0) a.sx[row] = scale;

#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = lane + i * 64;
    if (c < nchunk) *dst_of(c) = quantize8(f[i], scale, inv_scale);
  }
}

template <int NCH, bool LN>
static int launch_quant(const QuantArgs& a, hipStream_t stream) {
  const int64_t blocks = (a.M + kQuantWavesPerBlock - 1) / kQuantWavesPerBlock;
  hipLaunchKernelGGL((quant_rowwise_bf16_kernel<NCH, LN>), dim3((unsigned int)blocks),
                     dim3(64 * kQuantWavesPerBlock), 0, stream, a);
  return check_launch("quant_rowwise_bf16_kernel");
}

template <bool LN>
static int dispatch_quant(const QuantArgs& a, hipStream_t s) {
  const int need = (a.K / 8 + 63) / 64;
  if (need <= 2) return launch_quant<2, LN>(a, s);
  if (need <= 3) return launch_quant<3, LN>(a, s);
  if (need <= 4) return launch_quant<4, LN>(a, s);
  if (need <= 6) return launch_quant<6, LN>(a, s);
  if (need <= 8) return launch_quant<8, LN>(a, s);
  if (need <= 10) return launch_quant<10, LN>(a, s);
  if (need <= 12) return launch_quant<12, LN>(a, s);
  return launch_quant<16, LN>(a, s);
}

static int check_common(const char* who, const void* x, int64_t ldx, const int8_t* xq, const float* sx,
                        int64_t M, int K, int dtype, int layout) {
  SF_REQUIRE(layout == SAMFAST_LAYOUT_ROWMAJOR || (layout == SAMFAST_LAYOUT_KB64 && K % 64 == 0),
             "%s: layout must be row-major, or K-block major with K %% 64 == 0", who);
  SF_REQUIRE(x && xq && sx, "%s: null pointer", who);
  SF_REQUIRE(M >= 0 && K > 0, "%s: bad shape M=%lld K=%d", who, (long long)M, K);
  if (dtype != SAMFAST_BF16) SF_FAIL(SAMFAST_E_UNSUPPORTED, "%s: only bf16 input", who);
  SF_REQUIRE(K % 8 == 0 && K <= 8192, "%s: K=%d must be a multiple of 8, <= 8192", who, K);
  SF_REQUIRE(ldx >= K && ldx % 8 == 0, "%s: ldx=%lld must be >= K and a multiple of 8", who,
             (long long)ldx);
  SF_REQUIRE(aligned16(x) && (reinterpret_cast<uintptr_t>(xq) & 7u) == 0,
             "%s: x must be 16-byte and xq 8-byte aligned", who);
  SF_REQUIRE((M + 3) / 4 < (1ll << 31), "%s: M too large", who);
  return SAMFAST_OK;
}

}  // namespace samfast

extern "C" int samfast_quant_rowwise_i8(const void* x, int64_t ldx, int8_t* xq, float* sx,
                                        int64_t M, int K, int dtype, int layout, void* stream) {
  using namespace samfast;
  const int rc = check_common("quant_rowwise", x, ldx, xq, sx, M, K, dtype, layout);
  if (rc != SAMFAST_OK) return rc;
  if (M == 0) return SAMFAST_OK;
  QuantArgs a = {};
  a.x = reinterpret_cast<const unsigned short*>(x);
  a.ldx = ldx; a.xq = xq; a.sx = sx; a.M = M; a.K = K;
  a.kb64 = layout == SAMFAST_LAYOUT_KB64;
  return dispatch_quant<false>(a, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_layernorm_quant_i8(const void* x, int64_t ldx, const void* gamma,
                                          const void* beta, float eps, const int32_t* src_row,
                                          int8_t* xq, float* sx, int64_t M, int K, int dtype,
                                          int layout, void* stream) {
  using namespace samfast;
  const int rc = check_common("layernorm_quant", x, ldx, xq, sx, M, K, dtype, layout);
  if (rc != SAMFAST_OK) return rc;
  SF_REQUIRE(gamma && beta && aligned16(gamma) && aligned16(beta),
             "layernorm_quant: gamma / beta must be non-null and 16-byte aligned");
  SF_REQUIRE(eps > 0.f, "layernorm_quant: eps must be positive");
  if (M == 0) return SAMFAST_OK;
  QuantArgs a = {};
  a.x = reinterpret_cast<const unsigned short*>(x);
  a.ldx = ldx; a.xq = xq; a.sx = sx; a.M = M; a.K = K;
  a.gamma = reinterpret_cast<const unsigned short*>(gamma);
  a.beta = reinterpret_cast<const unsigned short*>(beta);
  a.src_row = src_row; a.eps = eps;
  a.kb64 = layout == SAMFAST_LAYOUT_KB64;
  return dispatch_quant<true>(a, reinterpret_cast<hipStream_t>(stream));
}
