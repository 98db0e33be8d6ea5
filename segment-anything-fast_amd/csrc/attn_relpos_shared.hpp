// Definitions shared by the attention kernels (attn_relpos.hip, attn_window_rows.hip).
#pragma once

#include "samfast_internal.hpp"
#include <type_traits>

namespace samfast {

struct AttnArgs {
  const unsigned short* q;
  const unsigned short* k;
  const unsigned short* v;
  const unsigned short* rh;  // FUSED: rel_pos_h table (2gh-1, hd); else rel_h (B,nH,N,gh)
  const unsigned short* rw;  // FUSED: rel_pos_w table (2gw-1, hd); else rel_w (B,nH,N,gw)
  unsigned short* out;
  int64_t q_sb, q_sh, q_sn;
  int64_t k_sb, k_sh, k_sn;
  int64_t v_sb, v_sh, v_sn;
  int64_t o_sb, o_sh, o_sn;
  int64_t rh_sb, rh_sh, rh_sn;
  int64_t rw_sb, rw_sh, rw_sn;
  int B, nH, gh, gw, N;
  float c;          // sm_scale * log2(e)
  float inv_scale;  // 1 / sm_scale
  // window kernel on image-ordered tokens (ws > 0): B counts images of img_h x img_w tokens,
  // a workgroup's window (iy, ix) covers tokens (iy*ws + y, ix*ws + x); positions outside the
  // image are padding tokens whose K / V rows are pad_k / pad_v (nH * hd values each)
  int img_h, img_w, ws, wins_x, wins_y;
  const unsigned short* pad_k;
  const unsigned short* pad_v;
};

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLazyLog2 = 8.0f;  // softmax reference lags the running maximum by at most 2^8

// The two 16-bit element types of q / k / v / out (and of the bias factors): what differs between
// them is the matrix instruction, the conversions and three bit patterns.  Eight elements travel
// as four 32-bit words (u32x4) everywhere outside these functions.
struct ElemBf16 {
  static constexpr unsigned int kOne = 0x3F80u;   // 1.0
  static constexpr unsigned int kMask = 0xF149u;  // -1e30: added to a score (before the scale), it removes the key
  static SF_DEVICE f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static SF_DEVICE unsigned int pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
  static SF_DEVICE float lo(unsigned int w) { return bf16_lo_to_f32(w); }
  static SF_DEVICE float hi(unsigned int w) { return bf16_hi_to_f32(w); }
  static SF_DEVICE float from_bits(unsigned short h) { return bf16_bits_to_f32(h); }
};
struct ElemF16 {
  typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  static constexpr unsigned int kOne = 0x3C00u;   // 1.0
  static constexpr unsigned int kMask = 0xFB53u;  // -60000 (fp16 ends at 65504): times scale*log2(e) still below -2^12
  static SF_DEVICE f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static SF_DEVICE unsigned int pack2(float lo, float hi) {  // round to nearest even
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, f16x2));
  }
  static SF_DEVICE float from_bits(unsigned short h) { return (float)__builtin_bit_cast(_Float16, h); }
  static SF_DEVICE float lo(unsigned int w) { return from_bits((unsigned short)(w & 0xffffu)); }
  static SF_DEVICE float hi(unsigned int w) { return from_bits((unsigned short)(w >> 16)); }
};

SF_DEVICE u32x4 load_x8_global(const unsigned short* p) { return *reinterpret_cast<const u32x4*>(p); }

template <typename T>
SF_DEVICE u32x4 cvt_x8(const f32x16& s, int base) {
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = T::pack2(s[base + 2 * i], s[base + 2 * i + 1]);
  return w;
}

// max(v, v of lane ^ 32) without an LDS round trip: v_permlane32_swap exchanges the upper half
// of its first operand with the lower half of its second, after which every lane holds its own
// value in one of the two and its partner's in the other
SF_DEVICE float max_with_lane_xor32(float v) {
  typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
  const unsigned int b = __float_as_uint(v);
  const u32x2_t r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// all LDS operations this wavefront has issued are complete and ordered
SF_DEVICE void wave_lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// one-hot vector of eight 16-bit elements: element e is 1.0 iff slot == 8*lh + e
template <typename T>
SF_DEVICE u32x4 onehot_x8(int slot, int lh) {
  const int e = slot - 8 * lh;  // may be outside [0, 8)
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    unsigned int v = 0u;
    if ((e >> 1) == i) v = (e & 1) ? (T::kOne << 16) : T::kOne;
    w[i] = v;
  }
  return w;
}

// Window kernel with the keys laid out as grid rows padded to 16 (attn_window_rows.hip): whether it
// covers the call (gw <= 16, gh <= 14) and its launch.
bool attn_window_rows_covers(const AttnArgs& a);
int attn_window_rows_launch(const AttnArgs& a, int hd, int dtype, bool fused, hipStream_t stream);

}  // namespace samfast
