// int8 GEMM with a 2:4-sparse weight operand on the gfx950 sparse matrix cores
// (v_smfmac_i32_32x32x64_i8): acc[m,n] = sum_k X[m,k] W[n,k] where every aligned group of
// 4 consecutive k of a W row holds at most 2 non-zeros.  Only the 2 kept values of a
// group are stored (plus a 4-bit position code), so the instruction does 64 k of dense
// work in the time of 32 and the W operand costs 0.5625 bytes per dense element.
//
// Operand semantics of v_smfmac_i32_32x32x64_i8 D = A_sparse * B (measured on hardware):
//   A  16 stored bytes per lane: lane (i = lane%32, h = lane/32) holds row i, bytes 2g, 2g+1
//      = the kept values of dense group g (g = 0..7); group g covers dense
//      k = 32*(g/4) + 16*h + 4*(g%4) + {0,1,2,3}.
//   idx  32 bits per lane: nibble g = p0 | p1 << 2, the positions (0..3) inside group g of
//      stored byte 2g and stored byte 2g+1; a lane's index word applies to its own row.
//   B  32 bytes per lane: lane (j = lane%32, h) holds column j, dense k = 32*h + 0..31.
//   D  32x32, register r of lane (j, h) = D[8*(r/4) + 4*h + r%4][j].
// The sparse operand must be A, so W supplies the MFMA rows and X the columns: a lane ends
// up with one token m and groups of 4 consecutive output channels n.
//
// Packed weight format (written by samfast_prune24_pack_i8), K-block major so that the
// operand tile of one k-step is contiguous memory:
//   wc   (K/64, N, 32) int8   byte 16*h + 2*g + e of row n, block kb = W[n, 64*kb + k(g,h) + p_e]
//   widx (K/64, N, 2)  int32  word h of row n, block kb = the eight position nibbles
//
// Tiling: a 256-thread workgroup owns 256 W rows x 128 X rows; its four wavefronts sit
// 2x2, each holding 128 x 64 as 4x2 MFMA tiles (128 accumulators), two workgroups per CU.
// One k-step of 64 dense k per tile; tiles travel global memory -> LDS directly
// (global_load_lds) through NST stages with vmcnt-tracked arrival, the operand fragments
// of the next k-step are read from LDS while the current MFMAs execute.
//
// W rows are placed in LDS in a permuted order so that a lane's 4x4 accumulator groups are
// 16 consecutive output channels: slot (tile ta, MFMA row 8g + 4h + e) of a wave's 128 rows
// holds W row 32g + 16*(ta/2) + 8h + 4*(ta%2) + e; the lane then writes 8 adjacent bf16 per
// 16-byte store.
#include "gemm_i8_sparse24_shared.hpp"
#include <type_traits>

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

constexpr int S_NST = 4;                       // LDS stages (73 728 B: two workgroups per CU)

template <int EPI>
SF_DEVICE void sp24_epilogue(const SparseArgs& a, i32x16 (&acc)[4][2], int x0, int w0, int wa,
                             int wb, int lr, int lh) {
  int m[2];
  float sxs[2];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    m[tb] = x0 + wb * 64 + tb * 32 + lr;
    sxs[tb] = (EPI == SEPI_I32) ? 0.f : a.sx[min(m[tb], a.M - 1)];
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      // 8 consecutive channels: acc[2j][tb][4g + 0..3], acc[2j+1][tb][4g + 0..3]
      const int n = w0 + wa * 128 + 32 * g + 16 * j + 8 * lh;
      if (n >= a.N) continue;  // N % 8 == 0
      if (EPI == SEPI_I32) {
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
          if (m[tb] < a.M) {
            int32_t* dst = reinterpret_cast<int32_t*>(a.out) + (int64_t)m[tb] * a.ldo + n;
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              const i32x4 o = {acc[2 * j + t][tb][4 * g], acc[2 * j + t][tb][4 * g + 1],
                               acc[2 * j + t][tb][4 * g + 2], acc[2 * j + t][tb][4 * g + 3]};
              *reinterpret_cast<i32x4*>(dst + 4 * t) = o;
            }
          }
        }
        continue;
      }
      f32x4 swv[2], bv[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        swv[t] = *reinterpret_cast<const f32x4*>(a.sw + n + 4 * t);
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        bv[t] = a.bias ? *reinterpret_cast<const f32x4*>(a.bias + n + 4 * t) : z;
      }
      u32x4 res[2];
      if (EPI == SEPI_RESIDUAL) {
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
          const u32x4 z = {0u, 0u, 0u, 0u};
          res[tb] = z;
          if (m[tb] < a.M)
            res[tb] = *reinterpret_cast<const u32x4*>(a.residual + (int64_t)m[tb] * a.ld_res + n);
        }
      }
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) {
        if (m[tb] >= a.M) continue;
        u32x4 o;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          float y[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // three separately rounded fp32 operations (no fused multiply-add)
            float v = (float)acc[2 * j + t][tb][4 * g + e] * sxs[tb];
            v = v * swv[t][e];
            y[e] = v + bv[t][e];
          }
          o[2 * t] = pack_bf16x2(y[0], y[1]);
          o[2 * t + 1] = pack_bf16x2(y[2], y[3]);
        }
        if (EPI == SEPI_GELU) {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            o[c] = pack_bf16x2(gelu_erf(bf16_lo_to_f32(o[c])), gelu_erf(bf16_hi_to_f32(o[c])));
        }
        if (EPI == SEPI_RESIDUAL) {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            o[c] = pack_bf16x2(bf16_lo_to_f32(o[c]) + bf16_lo_to_f32(res[tb][c]),
                               bf16_hi_to_f32(o[c]) + bf16_hi_to_f32(res[tb][c]));
        }
        *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned short*>(a.out) + (int64_t)m[tb] * a.ldo + n) = o;
      }
    }
  }
}

// Staged epilogue (bf16 outputs), same scheme as the dense kernel: scales and bias of the tile
// were fetched by global->LDS loads at kernel start; phase 1 scales the accumulators and writes
// a row-major 128 (tokens) x 256 (channels) bf16 tile into the LDS that held the operand
// stages; phase 2 walks it 8 rows at a time with 16 bytes per lane, so every store and
// residual load instruction covers two whole 512-byte row segments.
constexpr int SEP_STRIDE = 544;                     // tile row pitch in bytes

template <int EPI>
SF_DEVICE void sp24_epilogue_staged(const SparseArgs& a, i32x16 (&acc)[4][2], unsigned char* lds,
                                    const unsigned char* sc, int x0, int w0, int wa, int wb,
                                    int lr, int lh, int tid) {
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt 0, lgkmcnt 0
  __builtin_amdgcn_s_barrier();        // nobody reads operand stages any more
  __builtin_amdgcn_sched_barrier(0);

  const int chunk = tid & 31, rsub = tid >> 5;
  const int n = w0 + chunk * 8;
  const bool col_ok = n < a.N;  // N % 8 == 0
  auto out_row = [&](int p) {
    const int m = x0 + 8 * p + rsub;
    return (m < a.M && col_ok) ? m : -1;
  };
  u32x4 res[16];
  if (EPI == SEPI_RESIDUAL) {  // requested before the conversion work, waited for once
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      res[p] = z;
      const int dr = out_row(p);
      if (dr >= 0) res[p] = *reinterpret_cast<const u32x4*>(a.residual + (int64_t)dr * a.ld_res + n);
    }
  }
  {
    float sxs[2];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) sxs[tb] = *reinterpret_cast<const float*>(sc + (wb * 64 + tb * 32 + lr) * 4);
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // 8 consecutive channels: acc[2j][tb][4g + 0..3], acc[2j+1][tb][4g + 0..3]
        const int nl = wa * 128 + 32 * g + 16 * j + 8 * lh;
        f32x4 swv[2], bv[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          swv[t] = *reinterpret_cast<const f32x4*>(sc + 512 + (nl + 4 * t) * 4);
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
          bv[t] = a.bias ? *reinterpret_cast<const f32x4*>(sc + 1536 + (nl + 4 * t) * 4) : z;
        }
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
          u32x4 o;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            float y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              // three separately rounded fp32 operations (no fused multiply-add)
              float v = (float)acc[2 * j + t][tb][4 * g + e] * sxs[tb];
              v = v * swv[t][e];
              y[e] = v + bv[t][e];
            }
            o[2 * t] = pack_bf16x2(y[0], y[1]);
            o[2 * t + 1] = pack_bf16x2(y[2], y[3]);
          }
          if (EPI == SEPI_GELU) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
              o[c] = pack_bf16x2(gelu_erf(bf16_lo_to_f32(o[c])), gelu_erf(bf16_hi_to_f32(o[c])));
          }
          *reinterpret_cast<u32x4*>(lds + (wb * 64 + tb * 32 + lr) * SEP_STRIDE + nl * 2) = o;
        }
      }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // LDS writes done, residual values arrived
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);

  unsigned short* outp = reinterpret_cast<unsigned short*>(a.out);
#pragma unroll
  for (int p = 0; p < 16; ++p) {
    const int dr = out_row(p);
    u32x4 val = *reinterpret_cast<const u32x4*>(lds + (8 * p + rsub) * SEP_STRIDE + chunk * 16);
    if (EPI == SEPI_RESIDUAL) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        val[c] = pack_bf16x2(bf16_lo_to_f32(val[c]) + bf16_lo_to_f32(res[p][c]),
                             bf16_hi_to_f32(val[c]) + bf16_hi_to_f32(res[p][c]));
    }
    if (dr >= 0) *reinterpret_cast<u32x4*>(outp + (int64_t)dr * a.ldo + n) = val;
  }
}

template <int EPI>
__global__ __launch_bounds__(256, 2) void gemm_i8_sp24_kernel(SparseArgs a) {
  constexpr int NST = S_NST;
  constexpr bool STAGED = EPI != SEPI_I32;  // epilogue through LDS
  static_assert(128 * SEP_STRIDE <= NST * S_STAGE, "output tile must fit in the operand stages");
  __shared__ __attribute__((aligned(16))) unsigned char lds[NST * S_STAGE + (STAGED ? SEP_SCALE_BYTES : 0)];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wa = wave >> 1, wb = wave & 1;  // position along W rows / X rows
  const int lr = lane & 31, lh = lane >> 5;

  const unsigned int total = (unsigned int)a.tiles_x * (unsigned int)a.tiles_w;
  const unsigned int pid = xcd_contiguous_id(blockIdx.x, total);
  if (pid >= total) return;  // uniform over the workgroup
  const unsigned int GROUP_X = (unsigned int)a.group_x;  // X panels per scheduling group
  const unsigned int per_group = GROUP_X * a.tiles_w;
  const unsigned int first_x = (pid / per_group) * GROUP_X;
  const unsigned int gsz = min((unsigned int)a.tiles_x - first_x, GROUP_X);
  const unsigned int in_group = pid % per_group;
  const int x0 = (int)(first_x + in_group % gsz) * SBX;
  const int w0 = (int)(in_group / gsz) * SBW;

  // ---- global -> LDS: per tile and wave 2 x (X, 16 B) + 2 x (Wc, 16 B) + 2 x (index, 4 B) ----
  constexpr int NLD = 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  unsigned int off_x[2], off_w[2], off_i[2];  // unsigned lane offsets: scalar-base load form
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int blk = wave_u + 4 * i;  // 1 KB block of the X / Wc tile, 256 B block of the index tile
    const int xr = 16 * blk + (lane >> 2);
    off_x[i] = (unsigned int)(min(x0 + xr, a.M - 1) * a.x_row_pitch + (((lane & 3) ^ sp_swizzle_x(xr)) * 16));
    const int slot = 32 * blk + (lane >> 1);
    const int gn = min(w0 + sp_slot_to_row(slot), a.N - 1);
    off_w[i] = (unsigned int)(gn * 32 + (((lane & 1) ^ sp_swizzle_w(slot)) * 16));
    off_i[i] = (unsigned int)(gn * 8 + (lane & 1) * 4);
  }
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  auto dma_issue = [&](int kt, int stage_off) {
    const int8_t* xb = a.x + kt * a.x_kstep;
    const int8_t* wb_ = a.wc + (int64_t)kt * a.N * 32;
    const int8_t* ib = reinterpret_cast<const int8_t*>(a.widx) + (int64_t)kt * a.N * 8;
    // tile bases stay in scalar registers and the lane offsets 32-bit at the point of use, so the
    // loads take the scalar-base form (the 64-bit per-lane address form costs the MFMA stream
    // several times more per load)
    asm volatile("" : "+s"(xb), "+s"(wb_), "+s"(ib));
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int blk = wave_u + 4 * i;
      unsigned int ox = off_x[i], ow = off_w[i], oi = off_i[i];
      asm volatile("" : "+v"(ox), "+v"(ow), "+v"(oi));
      __builtin_amdgcn_global_load_lds((gptr_t)(xb + ox), (lptr_t)(lds + stage_off + blk * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)(wb_ + ow),
                                       (lptr_t)(lds + stage_off + S_OFF_W + blk * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)(ib + oi),
                                       (lptr_t)(lds + stage_off + S_OFF_I + blk * 256), 4, 0, 0);
    }
  };

  // ---- operand fragments ----
  const int fa_off = S_OFF_W + (wa * 128 + lr) * 32 + ((lh ^ sp_swizzle_w(lr)) * 16);
  const int fi_off = S_OFF_I + (wa * 128 + lr) * 8 + lh * 4;
  const int fb_row = (wb * 64 + lr) * SBK;
  const int fb_c0 = ((2 * lh) ^ sp_swizzle_x(lr)) * 16, fb_c1 = ((2 * lh + 1) ^ sp_swizzle_x(lr)) * 16;
  i32x4 fa[2][4];
  int fi[2][4];
  i32x8 fb[2][2];
  auto frags_at = [&](int stage_off, i32x4 (&av)[4], int (&iv)[4], i32x8 (&bv)[2]) {
    const unsigned char* src = lds + stage_off;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      av[t] = *reinterpret_cast<const i32x4*>(src + fa_off + t * 32 * 32);
      iv[t] = *reinterpret_cast<const int*>(src + fi_off + t * 32 * 8);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const i32x4 lo = *reinterpret_cast<const i32x4*>(src + fb_row + t * 32 * SBK + fb_c0);
      const i32x4 hi = *reinterpret_cast<const i32x4*>(src + fb_row + t * 32 * SBK + fb_c1);
      const i32x8 b = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      bv[t] = b;
    }
  };

  i32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  auto mma = [&](const i32x4 (&av)[4], const int (&iv)[4], const i32x8 (&bv)[2]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_smfmac_i32_32x32x64_i8(av[i], bv[j], acc[i][j], iv[i], 0, 0);
  };

  // s_waitcnt immediate: vmcnt in bits 3:0 and 15:14 ("at most n loads still in flight"),
  // expcnt 6:4 = 7 (no wait), lgkmcnt 11:8 = 0 (all of this wave's LDS reads done)
  auto wait_imm = [](int n) constexpr { return 0x0070 | (n & 15) | ((n >> 4) << 14); };
  static_assert((NST - 1) * NLD <= 63, "vmcnt immediate");

  if constexpr (STAGED) {
    // row scales, column scales and bias of this tile, 4 bytes per lane, straight into LDS; they
    // are the oldest loads in flight, so every later vmcnt wait covers them
    unsigned char* sc = lds + NST * S_STAGE;
    const int mm = min(x0 + (wave_u & 1) * 64 + lane, a.M - 1);
    const int nn = min(w0 + wave_u * 64 + lane, a.N - 1);
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sx + mm), (lptr_t)(sc + (wave_u & 1) * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sw + nn), (lptr_t)(sc + 512 + wave_u * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)((a.bias ? a.bias : a.sw) + nn),
                                     (lptr_t)(sc + 1536 + wave_u * 256), 4, 0, 0);
  }
  const int nk = a.K / SBK;  // even and >= NST (checked by the host)
  int st[NST];  // st[j] = LDS offset of the stage holding tile kt + j (uniform, rotated)
#pragma unroll
  for (int j = 0; j < NST; ++j) {
    st[j] = j * S_STAGE;
    dma_issue(j, st[j]);
  }
  __builtin_amdgcn_s_waitcnt(wait_imm((NST - 1) * NLD));
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  frags_at(st[0], fa[0], fi[0], fb[0]);

  // Iteration kt (the fragments of tile kt were read into register set P one iteration ago):
  //   wait until those reads are done and the own share of tile kt+1 has landed (in-order
  //   completion: at most KEEP later tiles may still be in flight); barrier - tile kt+1 is
  //   complete and nobody reads the stage of tile kt any more; fetch tile kt+NST into that
  //   stage, read the fragments of tile kt+1 into set 1-P, and run the 8 MFMAs of tile kt
  //   meanwhile.  (sched_group_barrier masks: 0x008 MFMA, 0x100 LDS read, 0x020 global read)
  auto iteration = [&](int kt, auto p_c, auto issue_c, auto next_c, auto keep_c) {
    constexpr int P = decltype(p_c)::value;
    constexpr bool ISSUE = decltype(issue_c)::value != 0;
    constexpr bool NEXT = decltype(next_c)::value != 0;
    constexpr int KEEP = decltype(keep_c)::value;
    __builtin_amdgcn_s_waitcnt(wait_imm(KEEP * NLD));
    if constexpr (NEXT) {
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (ISSUE) dma_issue(kt + NST, st[0]);
      frags_at(st[1], fa[1 - P], fi[1 - P], fb[1 - P]);
    }
    mma(fa[P], fi[P], fb[P]);
    // 12 LDS reads and 6 global->LDS loads spread over the 8 MFMAs
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (NEXT) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      if constexpr (ISSUE) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr (NEXT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      if constexpr (ISSUE)
        if (g < 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    const int t = st[0];
#pragma unroll
    for (int j = 0; j + 1 < NST; ++j) st[j] = st[j + 1];
    st[NST - 1] = t;
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  using C2 = std::integral_constant<int, 2>;
  static_assert(NST == 4, "pairing and tail below are written for four stages");
  int kt = 0;
  for (; kt + NST < nk; kt += 2) {  // fetching iterations come in pairs: nk and NST are even
    iteration(kt, C0{}, C1{}, C1{}, C2{});
    iteration(kt + 1, C1{}, C1{}, C1{}, C2{});
  }
  // the last NST iterations fetch nothing; fewer and fewer tiles remain in flight
  iteration(kt, C0{}, C0{}, C1{}, C2{});
  iteration(kt + 1, C1{}, C0{}, C1{}, C1{});
  iteration(kt + 2, C0{}, C0{}, C1{}, C0{});
  iteration(kt + 3, C1{}, C0{}, C0{}, C0{});

  if constexpr (STAGED)
    sp24_epilogue_staged<EPI>(a, acc, lds, lds + NST * S_STAGE, x0, w0, wa, wb, lr, lh, tid);
  else
    sp24_epilogue<EPI>(a, acc, x0, w0, wa, wb, lr, lh);
}

// ---- 2:4 pruning + packing --------------------------------------------------------
// One thread per (k block, row, half): two 16-byte pieces of the dense row (groups 0-3 and
// 4-7 of this half), keeps the two largest magnitudes of every group (ties: lowest
// position), writes 16 stored bytes and one index word.
__global__ __launch_bounds__(256) void prune24_pack_kernel(const int8_t* __restrict__ w,
                                                           int8_t* __restrict__ wc,
                                                           int32_t* __restrict__ widx, int N, int K) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t units = (int64_t)(K / 64) * N * 2;
  if (t >= units) return;
  const int h = (int)(t & 1);
  const int64_t rn = t >> 1;
  const int n = (int)(rn % N);
  const int kb = (int)(rn / N);
  const int8_t* src = w + (int64_t)n * K + kb * 64 + 16 * h;
  const u32x4 d0 = *reinterpret_cast<const u32x4*>(src);
  const u32x4 d1 = *reinterpret_cast<const u32x4*>(src + 32);
  unsigned int outw[4] = {0u, 0u, 0u, 0u};
  unsigned int idx = 0u;
#pragma unroll
  for (int g = 0; g < 8; ++g) {
    const unsigned int word = g < 4 ? d0[g & 3] : d1[g & 3];
    int v[4], mag[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      v[p] = (int)(signed char)((word >> (8 * p)) & 0xffu);
      mag[p] = v[p] < 0 ? -v[p] : v[p];
    }
    // rank of position p = number of positions that beat it (larger magnitude, or equal and lower position)
    int kept[2] = {0, 0}, nk = 0;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      int beat = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) beat += (mag[q] > mag[p]) || (mag[q] == mag[p] && q < p);
      if (beat < 2) {
        if (nk == 0) kept[0] = p; else kept[1] = p;
        ++nk;
      }
    }
    const unsigned int b0 = (unsigned int)(v[kept[0]] & 0xff), b1 = (unsigned int)(v[kept[1]] & 0xff);
    outw[g >> 1] |= (b0 | (b1 << 8)) << (16 * (g & 1));
    idx |= (unsigned int)(kept[0] | (kept[1] << 2)) << (4 * g);
  }
  const u32x4 o = {outw[0], outw[1], outw[2], outw[3]};
  *reinterpret_cast<u32x4*>(wc + ((int64_t)kb * N + n) * 32 + 16 * h) = o;
  widx[((int64_t)kb * N + n) * 2 + h] = (int32_t)idx;
}

static int sparse_common(int epi, const int8_t* xq, const float* sx, const int8_t* wc,
                         const int32_t* widx, const float* sw, const float* bias, void* out,
                         int64_t ldo, int64_t M, int N, int K, hipStream_t stream,
                         const void* residual = nullptr, int64_t ld_res = 0,
                         int layout = SAMFAST_LAYOUT_ROWMAJOR) {
  // no rows: nothing to do, and the row operands of an empty call may be null
  SF_REQUIRE(wc && widx && (M == 0 || (xq && out)), "gemm_i8_sparse24: null pointer");
  SF_REQUIRE(layout == SAMFAST_LAYOUT_ROWMAJOR || layout == SAMFAST_LAYOUT_KB64,
             "gemm_i8_sparse24: unknown layout %d", layout);
  SF_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_i8_sparse24: bad shape M=%lld N=%d K=%d", (long long)M, N, K);
  SF_REQUIRE(M < (1ll << 31) - 256, "gemm_i8_sparse24: M=%lld too large", (long long)M);
  SF_REQUIRE(M * K < (1ll << 31) && (int64_t)N * 32 < (1ll << 31),
             "gemm_i8_sparse24: operands of 2 GiB or more are not supported");
  SF_REQUIRE(N % 8 == 0, "gemm_i8_sparse24: N=%d must be a multiple of 8", N);
  if (K % 128 != 0 || K / SBK < S_NST)
    SF_FAIL(SAMFAST_E_UNSUPPORTED, "gemm_i8_sparse24: K=%d must be a multiple of 128, >= %d", K,
            S_NST * SBK);
  SF_REQUIRE(ldo >= N && ldo % 8 == 0, "gemm_i8_sparse24: output row stride %lld must be >= N and a multiple of 8",
             (long long)ldo);
  SF_REQUIRE(aligned16(xq) && aligned16(wc) && aligned16(widx) && aligned16(out),
             "gemm_i8_sparse24: operands and output must be 16-byte aligned");
  if (epi != SEPI_I32) {
    SF_REQUIRE(sw && (M == 0 || sx), "gemm_i8_sparse24: null scale pointer");
    SF_REQUIRE(aligned16(sw) && (!bias || aligned16(bias)), "gemm_i8_sparse24: sw / bias must be 16-byte aligned");
  }
  if (epi == SEPI_RESIDUAL)
    SF_REQUIRE((residual || M == 0) && aligned16(residual) && ld_res >= N && ld_res % 8 == 0,
               "gemm_i8_sparse24: residual must be non-null with 16-byte aligned rows");
  if (M == 0) return SAMFAST_OK;
  SparseArgs a;
  a.x = xq; a.wc = wc; a.widx = widx; a.out = out; a.sx = sx; a.sw = sw; a.bias = bias;
  a.ldo = ldo; a.M = (int)M; a.N = N; a.K = K;
  a.x_row_pitch = layout == SAMFAST_LAYOUT_KB64 ? SBK : K;
  a.x_kstep = layout == SAMFAST_LAYOUT_KB64 ? M * SBK : SBK;
  a.residual = reinterpret_cast<const unsigned short*>(residual);
  a.ld_res = ld_res;
  a.tiles_x = (int)((M + SBX - 1) / SBX);
  a.tiles_w = (N + SBW - 1) / SBW;
  // few column tiles (lin2: 5): the column tiles of one X panel run next to each other, the panel is
  // fetched through the fabric once (2.0 instead of 3.6 GB per launch at 131072 x 1280 x 5120, -2 %);
  // many column tiles (lin1: 20): groups of 8 X panels (1024 rows) whose panels stay in the XCD's L2
  a.group_x = a.tiles_w <= 6 ? 1 : 8;
  const int64_t total = (int64_t)a.tiles_x * a.tiles_w;
  SF_REQUIRE(total < (1ll << 30), "gemm_i8_sparse24: too many tiles");
  if (gemm_i8_sp24_persist_covers(epi, a)) return gemm_i8_sp24_persist_launch(epi, a, stream);
  const unsigned int grid = (unsigned int)(((total + 7) / 8) * 8);
  switch (epi) {
    case SEPI_I32:
      hipLaunchKernelGGL((gemm_i8_sp24_kernel<SEPI_I32>), dim3(grid), dim3(256), 0, stream, a); break;
    case SEPI_SCALE_BIAS:
      hipLaunchKernelGGL((gemm_i8_sp24_kernel<SEPI_SCALE_BIAS>), dim3(grid), dim3(256), 0, stream, a); break;
    case SEPI_GELU:
      hipLaunchKernelGGL((gemm_i8_sp24_kernel<SEPI_GELU>), dim3(grid), dim3(256), 0, stream, a); break;
    default:
      hipLaunchKernelGGL((gemm_i8_sp24_kernel<SEPI_RESIDUAL>), dim3(grid), dim3(256), 0, stream, a); break;
  }
  return check_launch("gemm_i8_sp24_kernel");
}

}  // namespace samfast

extern "C" int samfast_prune24_pack_i8(const int8_t* wq, int8_t* wc, int32_t* widx, int N, int K,
                                       void* stream) {
  using namespace samfast;
  SF_REQUIRE(wq && wc && widx, "prune24_pack: null pointer");
  SF_REQUIRE(N > 0 && K > 0 && K % 64 == 0, "prune24_pack: bad shape N=%d K=%d (K must be a multiple of 64)", N, K);
  SF_REQUIRE(aligned16(wq) && aligned16(wc) && aligned16(widx), "prune24_pack: pointers must be 16-byte aligned");
  const int64_t units = (int64_t)(K / 64) * N * 2;
  SF_REQUIRE((units + 255) / 256 < (1ll << 31), "prune24_pack: matrix too large");
  hipLaunchKernelGGL(prune24_pack_kernel, dim3((unsigned int)((units + 255) / 256)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), wq, wc, widx, N, K);
  return check_launch("prune24_pack_kernel");
}

extern "C" int samfast_gemm_i8_sparse24_i32(const int8_t* xq, const int8_t* wc, const int32_t* widx,
                                            int32_t* acc, int64_t M, int N, int K, void* stream) {
  return samfast::sparse_common(samfast::SEPI_I32, xq, nullptr, wc, widx, nullptr, nullptr, acc, N, M,
                                N, K, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_gemm_i8_sparse24_fused(const int8_t* xq, const float* sx, const int8_t* wc,
                                              const int32_t* widx, const float* sw, const float* bias,
                                              void* y, int64_t ldy, int64_t M, int N, int K, int dtype,
                                              int epilogue, const void* residual, int64_t ld_res,
                                              int layout, void* stream) {
  using namespace samfast;
  if (dtype != SAMFAST_BF16) {
    set_error("gemm_i8_sparse24_fused: only bf16 output");
    return SAMFAST_E_UNSUPPORTED;
  }
  int epi;
  switch (epilogue) {
    case SAMFAST_EPILOGUE_NONE: epi = SEPI_SCALE_BIAS; break;
    case SAMFAST_EPILOGUE_GELU: epi = SEPI_GELU; break;
    case SAMFAST_EPILOGUE_RESIDUAL: epi = SEPI_RESIDUAL; break;
    default:
      set_error("gemm_i8_sparse24_fused: unknown epilogue %d", epilogue);
      return SAMFAST_E_INVALID;
  }
  return sparse_common(epi, xq, sx, wc, widx, sw, bias, y, ldy, M, N, K,
                       reinterpret_cast<hipStream_t>(stream), residual, ld_res, layout);
}
