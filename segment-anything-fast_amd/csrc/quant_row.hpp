// The per-row int8 quantiser (optionally behind a LayerNorm) as device code shared by the
// stand-alone kernels (quant_rowwise.hip) and by the int8 GEMM, whose last workgroup of a row
// tile quantises the rows the tile's workgroups have just written (gemm_i8.hip).  One
// wavefront owns one row; both users run exactly this code, so their codes and scales agree
// bit for bit.
#pragma once

#include "samfast_internal.hpp"

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

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
  float inv_K;  // 1 / K for the LayerNorm statistics
  int kb64;  // 1: write xq K-block major, (K/64, M, 64)
};

// Wavefront-wide reductions without LDS traffic: four DPP steps combine the 16 lanes of a row
// (lane ^ 1, lane ^ 2, then the mirrored half row and the mirrored row, which by then hold the
// other quad's / other half's partial result), two lane-swap steps combine the four rows.
template <int CTRL>
SF_DEVICE float dpp_f32(float v) {
  return __uint_as_float((unsigned int)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
template <typename Op>
SF_DEVICE float wave_reduce(float v, Op op) {
  v = op(v, dpp_f32<0xB1>(v));   // quad_perm [1, 0, 3, 2]
  v = op(v, dpp_f32<0x4E>(v));   // quad_perm [2, 3, 0, 1]
  v = op(v, dpp_f32<0x141>(v));  // row_half_mirror
  v = op(v, dpp_f32<0x140>(v));  // row_mirror
  typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
  unsigned int b = __float_as_uint(v);
  u32x2_t r = __builtin_amdgcn_permlane16_swap(b, b, false, false);  // rows 0<->1, 2<->3
  v = op(__uint_as_float(r[0]), __uint_as_float(r[1]));
  b = __float_as_uint(v);
  r = __builtin_amdgcn_permlane32_swap(b, b, false, false);          // halves of the wavefront
  return op(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
SF_DEVICE float wave_sum(float v) {
  return wave_reduce(v, [](float x, float y) { return x + y; });
}
// for values >= 0 (absolute maxima): the bit patterns order like the values, and the unsigned
// maximum needs no canonicalisation of its operands
SF_DEVICE float wave_max_nonneg(float v) {
  return wave_reduce(v, [](float x, float y) {
    return __uint_as_float(max(__float_as_uint(x), __float_as_uint(y)));
  });
}

// EPC (4 or 8) values -> EPC int8 codes packed in EPC bytes.
// The code wanted is rint(fl(v / scale)) with the correctly rounded IEEE quotient.  The cheap
// route works on p = v * inv_scale (inv_scale = fl(1 / scale)), taken exactly inside fused
// multiply-adds: m = fl(p + 1.5 * 2^23) holds rint(p) - half to even - in its low mantissa bits
// (|p| <= 127 (1 + 2^-23)), so the low byte of m's bit pattern is the int8 code of p, and
// d = fl(p - (m - 1.5 * 2^23)) is p - rint(p) to 3e-8.  p differs from v / scale by at most
// 127 * 2^-24 (the rounding of inv_scale) and fl(v / scale) from v / scale by as much: 1.6e-5
// together.  Unless p lies within that distance of a half-integer, rint(p) is the wanted code;
// chunks with a |d| above 0.5 - 2.5e-5 are redone with the true division.
// Returns true when the chunk holds a NaN: the comparison that finds near-ties is written so
// that a NaN product also takes the slow path, where the chunk's values are looked at once more;
// the common path pays nothing for it.
template <int EPC>
SF_DEVICE bool quantize_chunk(const float (&v)[EPC], float scale, float inv_scale, unsigned int (&out)[EPC / 4]) {
  constexpr float kMagic = 12582912.0f;  // 1.5 * 2^23
  float m[EPC];
  bool near_tie = false, saw_nan = false;
#pragma unroll
  for (int e = 0; e < EPC; ++e) {
    m[e] = fmaf(v[e], inv_scale, kMagic);
    const float d = fmaf(v[e], inv_scale, kMagic - m[e]);  // kMagic - m[e] = -rint(p), exact
    near_tie |= !(fabsf(d) <= 0.5f - 2.5e-5f);  // also true for a NaN
  }
  if (near_tie) {
#pragma unroll
    for (int e = 0; e < EPC; ++e) {
      m[e] = v[e] / scale + kMagic;  // IEEE division
      saw_nan |= v[e] != v[e];
    }
  }
#pragma unroll
  for (int g = 0; g < EPC / 4; ++g) {
    const unsigned int w0 = __builtin_bit_cast(unsigned int, m[4 * g]), w1 = __builtin_bit_cast(unsigned int, m[4 * g + 1]);
    const unsigned int w2 = __builtin_bit_cast(unsigned int, m[4 * g + 2]), w3 = __builtin_bit_cast(unsigned int, m[4 * g + 3]);
    // byte 0 of each of four words -> one word (v_perm_b32: selector bytes pick from {hi, lo})
    const unsigned int lo = __builtin_amdgcn_perm(w1, w0, 0x0c0c0400u);  // [w0.b0, w1.b0, 0, 0]
    const unsigned int hi = __builtin_amdgcn_perm(w3, w2, 0x04000c0cu);  // [0, 0, w2.b0, w3.b0]
    out[g] = lo | hi;
  }
  return saw_nan;
}

// A lane holds chunks lane, lane + 64, ... of EPC elements (NCH of them: K <= NCH * 64 * EPC).
// EPC = 8 (16-byte loads) is the general case; EPC = 4 (8-byte loads) is taken when it divides the
// row among the lanes without a remainder and EPC = 8 does not (K = 1280: five chunks of 4 per
// lane instead of three chunks of 8 of which the third is half empty).
template <int NCH, int EPC, bool LN>
struct RowQuantizer {
  static_assert(EPC == 4 || EPC == 8, "chunk width");
  static constexpr int W = EPC / 2;  // 32-bit words per input chunk
  typedef unsigned int in_t __attribute__((ext_vector_type(W)));

  // Requests the lane's chunks of one source row; nothing here waits for the data.
  // STREAM: the row is read once and never again (the 671 MB lin1 output at ViT-H batch 16).
  template <bool STREAM>
  static SF_DEVICE void load_row(const unsigned short* row_ptr, int nchunk, int lane, in_t (&xw)[NCH]) {
    const in_t* src = reinterpret_cast<const in_t*>(row_ptr);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = lane + i * 64;
      const in_t z = {};
      xw[i] = z;
      if (c < nchunk) xw[i] = STREAM ? __builtin_nontemporal_load(src + c) : src[c];
    }
  }
  // the lane's slices of gamma and beta (LN): independent of the row
  static SF_DEVICE void load_affine(const unsigned short* gamma, const unsigned short* beta, int nchunk,
                                    int lane, in_t (&gw)[NCH], in_t (&bw)[NCH]) {
    const in_t* g4 = reinterpret_cast<const in_t*>(gamma);
    const in_t* b4 = reinterpret_cast<const in_t*>(beta);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = min(lane + i * 64, nchunk - 1);
      gw[i] = g4[c];
      bw[i] = b4[c];
    }
  }

  // chunk c of output row `row`: row-major at row*K + EPC*c; K-block major at
  // ((c*EPC/64)*M + row)*64 + (c*EPC)%64.  Written as a uniform base (the row is the same for the
  // whole wavefront) plus an unsigned 32-bit lane offset - M*K < 2^31 is checked on the host - so
  // that the stores take the scalar-base form and no 64-bit arithmetic runs per lane.
  static SF_DEVICE void store_chunk(const QuantArgs& a, int64_t row, int c, const unsigned int (&codes)[EPC / 4]) {
    const unsigned int k = (unsigned int)c * EPC;
    int8_t* base;
    unsigned int off;
    if (a.kb64) {
      base = a.xq + row * 64;
      off = (k >> 6) * ((unsigned int)a.M * 64u) + (k & 63u);
    } else {
      base = a.xq + row * (int64_t)a.K;
      off = k;
    }
    unsigned int* dst = reinterpret_cast<unsigned int*>(base + off);
    if (EPC == 8) {
      const u32x2 o = {codes[0], codes[EPC / 4 - 1]};
      *reinterpret_cast<u32x2*>(dst) = o;
    } else {
      *dst = codes[0];
    }
  }

  // an all-zero output row (a padding token): codes 0, scale at its floor
  static SF_DEVICE void zero_row(const QuantArgs& a, int64_t row, int nchunk, int lane) {
    const unsigned int z[EPC / 4] = {};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) store_chunk(a, row, c, z);
    }
    if (lane == 0) a.sx[row] = 1e-5f / 127.0f;
  }

  // Everything after the loads: (LayerNorm,) absmax, scale, codes of output row `row`.
  static SF_DEVICE void finish_row(const QuantArgs& a, int64_t row, int nchunk, int lane,
                                   const in_t (&xw)[NCH], const in_t (&gw)[NCH], const in_t (&bw)[NCH]) {
    // the row as floats, unpacked once
    float f[NCH][EPC];
#pragma unroll
    for (int i = 0; i < NCH; ++i)
#pragma unroll
      for (int j = 0; j < W; ++j) {
        f[i][2 * j] = bf16_lo_to_f32(xw[i][j]);
        f[i][2 * j + 1] = bf16_hi_to_f32(xw[i][j]);
      }

    if (LN) {
      // two-pass mean / biased variance over the K real elements, fp32
      float s1 = 0.f;
#pragma unroll
      for (int i = 0; i < NCH; ++i)
#pragma unroll
        for (int j = 0; j < W; ++j) s1 += f[i][2 * j] + f[i][2 * j + 1];
      // statistics: multiplication by 1/K and a hardware reciprocal square root (1 ulp each; the
      // LayerNorm result is compared with the reference to one code step, not bit for bit)
      const float mean = wave_sum(s1) * a.inv_K;
      float s2 = 0.f;
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        if (lane + i * 64 < nchunk) {
#pragma unroll
          for (int j = 0; j < W; ++j) {
            const float d0 = f[i][2 * j] - mean, d1 = f[i][2 * j + 1] - mean;
            f[i][2 * j] = d0;
            f[i][2 * j + 1] = d1;
            s2 = fmaf(d1, d1, fmaf(d0, d0, s2));
          }
        }
      }
      const float rstd = __builtin_amdgcn_rsqf(fmaf(wave_sum(s2), a.inv_K, a.eps));
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = lane + i * 64;
        if (c < nchunk) {
          const in_t g = gw[i], b = bw[i];
#pragma unroll
          for (int j = 0; j < W; ++j) {
            // (x - mean) * rstd, then one fused multiply-add with gamma and beta
            const float y0 = fmaf(f[i][2 * j] * rstd, bf16_lo_to_f32(g[j]), bf16_lo_to_f32(b[j]));
            const float y1 = fmaf(f[i][2 * j + 1] * rstd, bf16_hi_to_f32(g[j]), bf16_hi_to_f32(b[j]));
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
      for (int e = 0; e < EPC; ++e) amax = fmaxf(amax, fabsf(f[i][e]));
    amax = wave_max_nonneg(amax);

    const float scale = fmaxf(amax, 1e-5f) / 127.0f;
    const float inv_scale = 1.0f / scale;

    bool saw_nan = false;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = lane + i * 64;
      if (c < nchunk) {
        unsigned int codes[EPC / 4];
        saw_nan |= quantize_chunk<EPC>(f[i], scale, inv_scale, codes);
        store_chunk(a, row, c, codes);
      }
    }
    // the maximum above drops NaNs (fmaxf returns its other operand); a row that holds one gets a
    // NaN scale, so that the Linear reading it returns NaN for this row as a float Linear would
    const bool row_nan = __any(saw_nan);
    if (lane == 0) a.sx[row] = row_nan ? __uint_as_float(0x7fc00000u) : scale;
  }
};

// (NCH, EPC) the stand-alone kernels and the GEMM tail use for a row of K elements: 4-element
// chunks where they divide the row among the 64 lanes exactly and 8-element chunks do not
constexpr int quant_epc_for(int K) { return (K == 768 || K == 1280) ? 4 : 8; }
constexpr int quant_nch_for(int K) {
  if (K == 768) return 3;
  if (K == 1280) return 5;
  const int need = (K / 8 + 63) / 64;
  return need <= 2 ? 2 : need <= 3 ? 3 : need <= 4 ? 4 : need <= 6 ? 6 : need <= 8 ? 8
       : need <= 10 ? 10 : need <= 12 ? 12 : 16;
}

}  // namespace samfast
