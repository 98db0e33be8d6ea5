// Resident-workgroup form of the 2:4-sparse int8 GEMM (gemm_i8_sparse24.hip): two workgroups per
// CU stay for the whole launch and walk a list of 256 (W rows) x 128 (X rows) output tiles each.
//
// What it changes against one workgroup per tile:
//   * the K loop is one pipeline across tiles: the last three k-steps of a tile request the first
//     three k tiles (and the scales) of the next one, so only a workgroup's very first tile waits
//     for memory with nothing to do;
//   * the output of tile t is produced at the top of tile t+1's first k-step, wavefront by
//     wavefront, without a workgroup barrier and without borrowing the operand stages: a lane
//     (one token, runs of 8 channels) scales a 32-token x 64-channel piece of its wavefront's
//     64 x 128 share, writes it into 4 KB of LDS owned by the wavefront, reads it back with 8 lanes
//     per token and stores whole 128-byte lines (16 B per lane); four such pieces per tile.  The
//     new tile's first matrix instructions start from zero as soon as the accumulators of their
//     token half are converted, and the other resident workgroup has the matrix pipe meanwhile;
//   * the stores are never waited for at a barrier: vector memory operations complete in issue
//     order, so "k tile kt+1 has landed" stays a vmcnt threshold that counts the younger loads and
//     stores exactly.
// Residual epilogue: the residual values are fetched with the store pattern (whole lines, the same
// lane reads and later writes a location, so output and residual may be one buffer) and added
// after the trip through LDS; each piece's values are requested one piece ahead, the first
// piece's in the tile's last k-step ahead of that step's tile loads.
//
// Covered: scale + bias, GELU and residual epilogues on full tiles (M % 128 == 0, N % 256 == 0,
// K % 128 == 0, K >= 512).  Arithmetic, operand layouts in LDS and the tile -> XCD mapping are those
// of gemm_i8_sp24_kernel, and the results are bit-equal.
#include "gemm_i8_sparse24_shared.hpp"

#include <type_traits>

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

constexpr int QNST = 3;            // LDS operand stages
constexpr int QNLD = 6;            // global->LDS wave instructions per k tile and wavefront
constexpr int QSC_LOADS = 3;       // scale loads per wavefront and tile
constexpr int Q_STAGING = 4096;    // output staging per wavefront: 32 tokens x 128 B
constexpr int Q_OFF_SC = QNST * S_STAGE;
constexpr int Q_OFF_STG = Q_OFF_SC + 2 * SEP_SCALE_BYTES;
constexpr int Q_LDS = Q_OFF_STG + 4 * Q_STAGING;  // 76 800 B: two workgroups per CU
constexpr int Q_STORES = 16;       // store instructions per wavefront and tile

template <int V>
using QC = std::integral_constant<int, V>;

// compile-time shape of one k-step of gemm_i8_sp24_persist_kernel (see `step` there)
template <int P_, bool ZERO_, bool CONV_, bool RFIRST_, bool SC_, bool ISSUE_, bool NEXT_, int THRESH_>
struct SpStep {
  static constexpr int P = P_, THRESH = THRESH_;
  static constexpr bool ZERO = ZERO_, CONV = CONV_, RFIRST = RFIRST_, SC = SC_, ISSUE = ISSUE_, NEXT = NEXT_;
};

template <int EPI>
__global__ __launch_bounds__(256, 2) void gemm_i8_sp24_persist_kernel(SparseArgs a) {
  static_assert(EPI == SEPI_SCALE_BIAS || EPI == SEPI_GELU || EPI == SEPI_RESIDUAL, "epilogues built");
  constexpr bool RES = EPI == SEPI_RESIDUAL;
  __shared__ __attribute__((aligned(16))) unsigned char lds[Q_LDS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave_u >> 1, wb = wave_u & 1;  // position along W rows / X rows
  const int lr = lane & 31, lh = lane >> 5;

  // ---- the tiles of this workgroup ------------------------------------------------------------
  // Hardware workgroup ids are dealt round-robin to the 8 XCDs.  XCD x owns the contiguous range
  // [x * chunk, (x + 1) * chunk) of logical tile ids; its workgroups walk it side by side, so the
  // tiles in flight on an XCD are neighbours and share operand panels in that XCD's L2.
  const unsigned int total = (unsigned int)a.tiles_x * (unsigned int)a.tiles_w;
  const unsigned int xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_x = gridDim.x >> 3;
  const unsigned int chunk = (total + 7u) >> 3;
  const unsigned int first = xcd * chunk + slot;
  const unsigned int last = min(total, (xcd + 1u) * chunk);
  if (slot >= chunk || first >= last) return;  // uniform over the workgroup
  const int nt = (int)((last - first + per_x - 1u) / per_x);

  auto tile_origin = [&](unsigned int pid, int& x0, int& w0) __attribute__((always_inline)) {
    const unsigned int GROUP_X = (unsigned int)a.group_x;  // X panels per scheduling group
    const unsigned int per_group = GROUP_X * a.tiles_w;
    const unsigned int first_x = (pid / per_group) * GROUP_X;
    const unsigned int gsz = min((unsigned int)a.tiles_x - first_x, GROUP_X);
    const unsigned int in_group = pid % per_group;
    x0 = (int)(first_x + in_group % gsz) * SBX;
    w0 = (int)(in_group / gsz) * SBW;
  };

  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;

  // ---- global -> LDS: per k tile and wave 2 x (X, 16 B) + 2 x (Wc, 16 B) + 2 x (index, 4 B) ----
  // Lane offsets inside a tile (they do not depend on the tile); the tile origin goes into the
  // scalar bases below.
  unsigned int off_x[2], off_w[2], off_i[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int blk = wave_u + 4 * i;  // 1 KB block of the X / Wc tile, 256 B block of the index tile
    const int xr = 16 * blk + (lane >> 2);
    off_x[i] = (unsigned int)(xr * a.x_row_pitch + (((lane & 3) ^ sp_swizzle_x(xr)) * 16));
    const int sl = 32 * blk + (lane >> 1);
    const int wrow = sp_slot_to_row(sl);
    off_w[i] = (unsigned int)(wrow * 32 + (((lane & 1) ^ sp_swizzle_w(sl)) * 16));
    off_i[i] = (unsigned int)(wrow * 8 + (lane & 1) * 4);
  }
  // operand bases of the tile whose k tiles are being requested
  const int8_t* ld_x = nullptr;
  const int8_t* ld_w = nullptr;
  const int8_t* ld_i = nullptr;
  auto set_dma = [&](int x0, int w0) __attribute__((always_inline)) {
    ld_x = a.x + (int64_t)x0 * a.x_row_pitch;
    ld_w = a.wc + (int64_t)w0 * 32;
    ld_i = reinterpret_cast<const int8_t*>(a.widx) + (int64_t)w0 * 8;
  };
  auto dma_issue = [&](int kt, int stage_off) __attribute__((always_inline)) {
    const int8_t* xb = ld_x + kt * a.x_kstep;
    const int8_t* wb_ = ld_w + (int64_t)kt * a.N * 32;
    const int8_t* ib = ld_i + (int64_t)kt * a.N * 8;
    // tile bases stay in scalar registers and the lane offsets 32-bit at the point of use, so the
    // loads take the scalar-base form
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
  // row scales, column scales and bias of a tile, 4 bytes per lane, straight into scale buffer `buf`
  auto scales_issue = [&](int x0, int w0, int buf) __attribute__((always_inline)) {
    unsigned char* sc = lds + Q_OFF_SC + buf * SEP_SCALE_BYTES;
    const int mm = x0 + (wave_u & 1) * 64 + lane;
    const int nn = w0 + wave_u * 64 + lane;
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sx + mm), (lptr_t)(sc + (wave_u & 1) * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sw + nn), (lptr_t)(sc + 512 + wave_u * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)((a.bias ? a.bias : a.sw) + nn),
                                     (lptr_t)(sc + 1536 + wave_u * 256), 4, 0, 0);
  };

  // ---- operand fragments ----
  const int fa_off = S_OFF_W + (wa * 128 + lr) * 32 + ((lh ^ sp_swizzle_w(lr)) * 16);
  const int fi_off = S_OFF_I + (wa * 128 + lr) * 8 + lh * 4;
  const int fb_row = (wb * 64 + lr) * SBK;
  const int fb_c0 = ((2 * lh) ^ sp_swizzle_x(lr)) * 16, fb_c1 = ((2 * lh + 1) ^ sp_swizzle_x(lr)) * 16;
  i32x4 fa[2][4];
  int fi[2][4];
  i32x8 fb[2][2];
  auto frags_at = [&](int stage_off, i32x4 (&av)[4], int (&iv)[4], i32x8 (&bv)[2]) __attribute__((always_inline)) {
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
  auto mma = [&](const i32x4 (&av)[4], const int (&iv)[4], const i32x8 (&bv)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_smfmac_i32_32x32x64_i8(av[i], bv[j], acc[i][j], iv[i], 0, 0);
  };
  // first matrix instructions of a tile for token half j: the accumulators start from zero
  auto mma_zero_half = [&](int j, const i32x4 (&av)[4], const int (&iv)[4], const i32x8 (&bv)[2]) __attribute__((always_inline)) {
    const i32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc[i][j] = __builtin_amdgcn_smfmac_i32_32x32x64_i8(av[i], bv[j], z, iv[i], 0, 0);
  };

  // ---- output of the previous tile --------------------------------------------------------------
  // Piece (tb, gp) = tokens tb*32 .. +31 of the wavefront's 64, channels gp*64 .. +63 of its 128.
  // Conversion side: lane (lr, lh) holds token lr and, for g = 2*gp + gg and j, the 8 channels
  // 32*g + 16*j + 8*lh + 0..7 = acc[2j][tb][4g + 0..3], acc[2j+1][tb][4g + 0..3]: chunk
  // 4*gg + 2*j + lh of the token's 128-byte row.  Store side: lane l holds chunk l % 8 of token
  // 8*q + l / 8.  Chunk c of token row r sits at position c ^ (r % 8) ^ (r / 8 % 2): the writes (8 or
  // 16 consecutive tokens, one chunk each) and the reads (1 or 2 tokens, 8 chunks each) then touch
  // every bank once, whether the LDS cycles through 128 or 256 bytes.
  unsigned char* stg = lds + Q_OFF_STG + wave_u * Q_STAGING;
  const int stg_wr = lr * 128;                      // + ((chunk ^ wr_swz) * 16)
  const int wr_swz = (lr & 7) ^ ((lr >> 3) & 1);
  const int stg_rd = (lane >> 3) * 128;             // + q * 1024 + ((l%8 ^ rd_swz(q)) * 16)
  const unsigned short* prev_out = nullptr;         // out + x0 * ldo + w0 of the tile whose output is due
  const unsigned short* prev_res = nullptr;         // residual + x0 * ld_res + w0 of that tile
  const unsigned int voff = (unsigned int)(((wb * 64 + (lane >> 3)) * a.ldo + wa * 128 + (lane & 7) * 8) * 2);
  const unsigned int voff_res =
      RES ? (unsigned int)(((wb * 64 + (lane >> 3)) * a.ld_res + wa * 128 + (lane & 7) * 8) * 2) : 0u;
  typedef __attribute__((address_space(1))) unsigned char* gbytes_t;
  u32x4 res[2][4];  // residual values of the piece being converted and of the next one

  // (the row pitch is made opaque at every use: as a loop invariant the 16 row offsets of a tile
  // would be kept in scalar registers for the whole kernel)
  auto residual_request = [&](int p, u32x4 (&dst)[4]) __attribute__((always_inline)) {
    const int tb = p >> 1, gp = p & 1;
    unsigned int pitch = (unsigned int)a.ld_res * 2u;
    asm volatile("" : "+s"(pitch));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned char* rowp = reinterpret_cast<const unsigned char*>(prev_res) +
                                  (unsigned int)(tb * 32 + 8 * q) * pitch + gp * 128;
      asm volatile("" : "+s"(rowp));
      unsigned int off = voff_res;
      asm volatile("" : "+v"(off));
      typedef __attribute__((address_space(1))) const u32x4* gsrc_t;
      dst[q] = *(gsrc_t)((gbytes_t)(uintptr_t)rowp + off);
    }
  };

  // Converts piece p from the accumulators, takes it through the wavefront's LDS and stores it.
  //   REQ_NEXT  residual epilogue: piece p+1's residual values are requested once this piece's
  //             conversion registers are free;
  //   RES_WAIT  residual epilogue: operations issued after this piece's residual request and before
  //             its use (what may stay in flight when the values are needed).
  auto convert_piece = [&](auto p_c, const unsigned char* sc, auto req_next_c, auto res_wait_c) __attribute__((always_inline)) {
    constexpr int p = decltype(p_c)::value;
    constexpr int tb = p >> 1, gp = p & 1;
    constexpr bool REQ_NEXT = decltype(req_next_c)::value != 0;
    constexpr int RES_WAIT = decltype(res_wait_c)::value;
    const float sxs = *reinterpret_cast<const float*>(sc + (wb * 64 + tb * 32 + lr) * 4);
#pragma unroll
    for (int gg = 0; gg < 2; ++gg)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int g = 2 * gp + gg;
        const int nl = wa * 128 + 32 * g + 16 * j + 8 * lh;
        f32x4 swv[2], bv[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          swv[t] = *reinterpret_cast<const f32x4*>(sc + 512 + (nl + 4 * t) * 4);
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
          bv[t] = a.bias ? *reinterpret_cast<const f32x4*>(sc + 1536 + (nl + 4 * t) * 4) : z;
        }
        u32x4 o;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          float y[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // three separately rounded fp32 operations (no fused multiply-add)
            float v = (float)acc[2 * j + t][tb][4 * g + e] * sxs;
            v = v * swv[t][e];
            y[e] = v + bv[t][e];
          }
          o[2 * t] = pack_bf16x2(y[0], y[1]);
          o[2 * t + 1] = pack_bf16x2(y[2], y[3]);
        }
        if (EPI == SEPI_GELU) {
          // activation of the bf16-rounded Linear output, as a separate GELU would see it
#pragma unroll
          for (int c = 0; c < 4; ++c)
            o[c] = pack_bf16x2(gelu_erf(bf16_lo_to_f32(o[c])), gelu_erf(bf16_hi_to_f32(o[c])));
        }
        *reinterpret_cast<u32x4*>(stg + stg_wr + (((4 * gg + 2 * j + lh) ^ wr_swz) * 16)) = o;
        // keep the conversion narrow (one run of 8 channels at a time)
        __builtin_amdgcn_sched_barrier(0);
      }
    if constexpr (RES && REQ_NEXT) residual_request(p + 1, res[(p + 1) & 1]);
    // LDS operations of one wavefront execute in order: the reads below see the writes above
    u32x4 val[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      // token row r = 8q + l/8: r % 8 = l / 8, r / 8 % 2 = q % 2
      const int rd_swz = (lane >> 3) ^ (q & 1);
      val[q] = *reinterpret_cast<const u32x4*>(stg + stg_rd + q * 1024 + (((lane & 7) ^ rd_swz) * 16));
    }
    if constexpr (RES) {
      __builtin_amdgcn_s_waitcnt(0x0070 | (RES_WAIT & 15) | ((RES_WAIT >> 4) << 14));  // and the LDS reads
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int c = 0; c < 4; ++c)
          // bf16 add of the bf16-rounded Linear output and the residual stream
          val[q][c] = pack_bf16x2(bf16_lo_to_f32(val[q][c]) + bf16_lo_to_f32(res[p & 1][q][c]),
                                  bf16_hi_to_f32(val[q][c]) + bf16_hi_to_f32(res[p & 1][q][c]));
    }
    unsigned int pitch = (unsigned int)a.ldo * 2u;
    asm volatile("" : "+s"(pitch));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const unsigned char* rowp = reinterpret_cast<const unsigned char*>(prev_out) +
                                  (unsigned int)(tb * 32 + 8 * q) * pitch + gp * 128;
      asm volatile("" : "+s"(rowp));  // uniform row base in scalar registers, 32-bit lane offset
      unsigned int off = voff;
      asm volatile("" : "+v"(off));
      typedef __attribute__((address_space(1))) u32x4* gdst_t;
      *(gdst_t)((gbytes_t)(uintptr_t)rowp + off) = val[q];
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // s_waitcnt immediate: vmcnt in bits 3:0 and 15:14 ("at most n operations still in flight"),
  // expcnt 6:4 = 7 (no wait), lgkmcnt 11:8 = 0 (all of this wave's LDS reads done)
  auto wait_imm = [](int n) constexpr { return 0x0070 | (n & 15) | ((n >> 4) << 14); };

  int st[QNST];  // st[j] = LDS offset of the stage holding k tile (current + j); uniform, rotated
  const unsigned char* conv_sc = lds + Q_OFF_SC;  // scale buffer of the tile whose output is due

  // One k-step (the fragments of its k tile were read into register set P one step ago):
  //   wait until those reads are done and the own share of the next k tile has landed; barrier -
  //   that k tile is complete and nobody reads the current stage any more; request a k tile into
  //   the current stage; read the next fragments into set 1-P; 8 matrix instructions on set P.
  // F carries the step's compile-time shape:
  //   ZERO    first k-step of a tile, accumulators start at zero;
  //   CONV    the previous tile's output is produced first (implies ZERO);
  //   RFIRST  residual epilogue: the first piece's residual values are requested, ahead of the tile
  //           loads (the tile's last k-step);
  //   SC      the next tile's scales are requested (into scale buffer sc_buf) before the tile loads;
  //   ISSUE   k tile ld_kt (of the tile set_dma named last) is requested;
  //   NEXT    a following k tile exists (of this tile or the next);
  //   THRESH  operations younger than the loads of the k tile needed next.
  auto step = [&](int ld_kt, int sc_x0, int sc_w0, int sc_buf, auto f) __attribute__((always_inline)) {
    using F = decltype(f);
    constexpr int P = F::P, THRESH = F::THRESH;
    constexpr bool ZERO = F::ZERO, CONV = F::CONV, RFIRST = F::RFIRST, SC = F::SC, ISSUE = F::ISSUE, NEXT = F::NEXT;
    __builtin_amdgcn_s_waitcnt(wait_imm(THRESH));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (RES && RFIRST) residual_request(0, res[0]);
    if constexpr (SC) scales_issue(sc_x0, sc_w0, sc_buf);
    if constexpr (ISSUE) dma_issue(ld_kt, st[0]);
    if constexpr (CONV) {
      // the K loop runs at raised wave priority, the conversion at base priority: the SIMD partner's
      // matrix instructions issue as soon as they are ready (lin1 840 -> 798 us)
      __builtin_amdgcn_s_setprio(0);
      // (the fences keep the zero-initialised matrix instructions of a token half behind the
      // conversion of that half: hoisted above it, old and new accumulators would be live together)
      __builtin_amdgcn_sched_barrier(0);
      // residual waits: piece 0 - the last step's and this step's tile loads and piece 1's request;
      // pieces 1, 2 - the stores of the piece before and the next request; piece 3 - piece 2's stores
      convert_piece(QC<0>{}, conv_sc, QC<1>{}, QC<2 * QNLD + 4>{});
      convert_piece(QC<1>{}, conv_sc, QC<1>{}, QC<8>{});
      mma_zero_half(0, fa[P], fi[P], fb[P]);
      __builtin_amdgcn_sched_barrier(0);
      convert_piece(QC<2>{}, conv_sc, QC<1>{}, QC<8>{});
      convert_piece(QC<3>{}, conv_sc, QC<0>{}, QC<4>{});
      mma_zero_half(1, fa[P], fi[P], fb[P]);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(1);
      if constexpr (NEXT) frags_at(st[1], fa[1 - P], fi[1 - P], fb[1 - P]);
    } else {
      if constexpr (NEXT) frags_at(st[1], fa[1 - P], fi[1 - P], fb[1 - P]);
      if constexpr (ZERO) {
        mma_zero_half(0, fa[P], fi[P], fb[P]);
        mma_zero_half(1, fa[P], fi[P], fb[P]);
      } else {
        mma(fa[P], fi[P], fb[P]);
      }
      // 12 LDS reads and up to 9 global->LDS loads spread over the 8 matrix instructions
      // (sched_group_barrier masks: 0x008 MFMA, 0x100 LDS read, 0x020 global read)
      if constexpr (!(RES && RFIRST)) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if constexpr (NEXT) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
          if constexpr (SC) { if (g < QSC_LOADS) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); }
          if constexpr (ISSUE) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if constexpr (NEXT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if constexpr (ISSUE)
            if (g < 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      }
    }
    // The matrix instructions are pure values to the compiler: nothing but their operands ties them
    // to this step.  Passing the accumulators through an empty asm statement pins every chain
    // between two steps (their fragments would otherwise be free to pile up across barriers).
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) asm volatile("" : "+v"(acc[i][j]));
    __builtin_amdgcn_sched_barrier(0);
    const int t = st[0];
#pragma unroll
    for (int j = 0; j + 1 < QNST; ++j) st[j] = st[j + 1];
    st[QNST - 1] = t;
  };
  // plain k-steps: tile loads only, one k tile in flight across the barrier
  using Plain0 = SpStep<0, false, false, false, false, true, true, QNLD>;
  using Plain1 = SpStep<1, false, false, false, false, true, true, QNLD>;

  __builtin_amdgcn_s_setprio(1);
  // ---- prologue: the first tile's scales and first three k tiles --------------------------------
  const int nk = a.K / SBK;  // even and >= 8 (checked by the host)
  int x0, w0;
  tile_origin(first, x0, w0);
  set_dma(x0, w0);
  scales_issue(x0, w0, 0);
#pragma unroll
  for (int j = 0; j < QNST; ++j) {
    st[j] = j * S_STAGE;
    dma_issue(j, st[j]);
  }
  __builtin_amdgcn_s_waitcnt(wait_imm((QNST - 1) * QNLD));
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  frags_at(st[0], fa[0], fi[0], fb[0]);

  // k-steps 3 .. nk-1 of a tile.  The last three request the next tile's scales and first three k
  // tiles; the last tile of the list requests its own again (nobody reads them): every tile then
  // runs the same code with the same operation counts in flight.
  auto tile_rest = [&](int ti) __attribute__((always_inline)) {
    step(6, 0, 0, 0, Plain1{});  // k-step 3
    for (int kt = 4; kt < nk - 4; kt += 2) {
      step(kt + 3, 0, 0, 0, Plain0{});
      step(kt + 4, 0, 0, 0, Plain1{});
    }
    step(nk - 1, 0, 0, 0, Plain0{});  // k-step nk-4
    // the output of this tile is produced at the top of the next one (or after the loop)
    prev_out = reinterpret_cast<const unsigned short*>(a.out) + (int64_t)x0 * a.ldo + w0;
    if (RES) prev_res = a.residual + (int64_t)x0 * a.ld_res + w0;
    conv_sc = lds + Q_OFF_SC + (ti & 1) * SEP_SCALE_BYTES;
    const unsigned int nxt = ti + 1 < nt ? (unsigned int)(ti + 1) : (unsigned int)ti;
    tile_origin(first + nxt * per_x, x0, w0);
    set_dma(x0, w0);
    step(0, x0, w0, (ti + 1) & 1, SpStep<1, false, false, false, true, true, true, QNLD>{});
    step(1, 0, 0, 0, SpStep<0, false, false, false, false, true, true, QNLD + QSC_LOADS>{});
    step(2, 0, 0, 0, SpStep<1, false, false, true, false, true, true, QNLD>{});
  };

  // ---- first tile: nothing to convert or store yet ----------------------------------------------
  step(3, 0, 0, 0, SpStep<0, true, false, false, false, true, true, QNLD>{});
  step(4, 0, 0, 0, Plain1{});
  step(5, 0, 0, 0, Plain0{});
  tile_rest(0);

  constexpr int NR0 = RES ? 4 : 0;  // the first piece's residual request sits between two k tiles' loads
  for (int ti = 1; ti < nt; ++ti) {
    // k-step 0 produces the previous tile's output; its 16 stores follow this step's tile loads, so
    // they are younger than the k tiles the next two steps wait for
    step(3, 0, 0, 0, SpStep<0, true, true, false, false, true, true, QNLD + NR0>{});
    step(4, 0, 0, 0, SpStep<1, false, false, false, false, true, true, QNLD + Q_STORES>{});
    step(5, 0, 0, 0, SpStep<0, false, false, false, false, true, true, QNLD + Q_STORES>{});
    tile_rest(ti);
  }

  // ---- the last tile's output ---------------------------------------------------------------------
  // (no tile loads were requested after the first piece's residual values this time)
  __builtin_amdgcn_sched_barrier(0);
  convert_piece(QC<0>{}, conv_sc, QC<1>{}, QC<QNLD + 4>{});
  convert_piece(QC<1>{}, conv_sc, QC<1>{}, QC<8>{});
  convert_piece(QC<2>{}, conv_sc, QC<1>{}, QC<8>{});
  convert_piece(QC<3>{}, conv_sc, QC<0>{}, QC<4>{});
  __builtin_amdgcn_s_waitcnt(0x0070);  // the unused loads of the last tile's tail land before the LDS is given back
}

static int sp_persist_grid() {
  static const int grid = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return (2 * cus) / 8 * 8;
  }();
  return grid;
}

bool gemm_i8_sp24_persist_covers(int epi, const SparseArgs& a) {
  // 0 (default): one workgroup per tile always - this form measures level with it (lin1 / lin2 of
  // ViT-H at 131072 rows inside the encoder: 798 against 805 us, 608 against 591 us); 1: from two
  // tiles per resident workgroup on; 2: wherever this form is built
  const int mode = knob_or(KNOB_SPARSE_PERSIST, 0);
  if (mode <= 0) return false;
  if (epi != SEPI_SCALE_BIAS && epi != SEPI_GELU && epi != SEPI_RESIDUAL) return false;
  if (a.M % SBX != 0 || a.N % SBW != 0 || a.K % (2 * SBK) != 0 || a.K / SBK < 8) return false;
  // 32-bit lane offsets inside a tile
  if (a.ldo >= (1ll << 23) || (epi == SEPI_RESIDUAL && a.ld_res >= (1ll << 23))) return false;
  return mode >= 2 || (int64_t)a.tiles_x * a.tiles_w >= 2ll * sp_persist_grid();
}

int gemm_i8_sp24_persist_launch(int epi, const SparseArgs& a, hipStream_t stream) {
  const int64_t total = (int64_t)a.tiles_x * a.tiles_w;
  const unsigned int grid = (unsigned int)min((int64_t)sp_persist_grid(), ((total + 7) / 8) * 8);
  if (epi == SEPI_GELU)
    hipLaunchKernelGGL((gemm_i8_sp24_persist_kernel<SEPI_GELU>), dim3(grid), dim3(256), 0, stream, a);
  else if (epi == SEPI_RESIDUAL)
    hipLaunchKernelGGL((gemm_i8_sp24_persist_kernel<SEPI_RESIDUAL>), dim3(grid), dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL((gemm_i8_sp24_persist_kernel<SEPI_SCALE_BIAS>), dim3(grid), dim3(256), 0, stream, a);
  return check_launch("gemm_i8_sp24_persist_kernel");
}

}  // namespace samfast
