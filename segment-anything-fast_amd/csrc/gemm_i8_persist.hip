// Persistent form of the 128 x 256 int8 GEMM: two workgroups per CU stay resident for the whole
// launch and walk a list of output tiles each.
//
// What it changes against one workgroup per tile (gemm_i8.hip):
//   * the K loop is one pipeline across tiles: the last three iterations of a tile request the
//     first three k tiles (and the scales) of the next one, so only the very first tile of a
//     workgroup waits for memory with nothing to do;
//   * the output of tile t does not leave in a burst between two loops.  At the top of tile t+1
//     every lane scales its accumulators and keeps the bf16 results packed in 64 registers (the
//     accumulators are free again at once: tile t+1 starts on zero-initialised matrix
//     instructions); the 32 store instructions of a wavefront's 64 x 128 share then go out a few per
//     k iteration of tile t+1, between its matrix instructions, and the operand stages in LDS are
//     never borrowed for the output;
//   * no barrier, LDS round trip or idle loader belongs to the epilogue any more.
// The k iterations that carry stores are unrolled (register indices are static); vector memory
// operations complete in issue order, so "tile kt+1 has landed" stays a vmcnt threshold that
// counts the younger loads and stores exactly.
//
// Residual epilogue: the residual values of the rows that leave with the conversion (and of the first
// held stores) are requested in the tile's last iteration, ahead of that iteration's tile loads, so a
// vmcnt wait that still leaves those tile loads in flight covers them; every later held store gets
// its residual one iteration ahead, again requested before the stores and tile loads it must not wait
// for.  Output and residual may be the same buffer: a lane reads a location before it writes it.
//
// Covered: scale + bias, GELU and residual (no row scatter) epilogues on full tiles (M % 128 == 0,
// N % 256 == 0, K >= 768).
// Arithmetic, operand layouts in LDS and the tile -> XCD mapping are those of gemm_i8_kernel, and
// the results are bit-equal.
#include "gemm_i8_shared.hpp"

#include <stdlib.h>
#include <type_traits>

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

#ifndef PERSIST_MIN_WG
#define PERSIST_MIN_WG 2
#endif
constexpr int PBM = 128, PBN = 256;
constexpr int PNST = 3;                           // LDS operand stages
constexpr int PSTAGE = (PBM + PBN) * GLD;         // 24 KB
constexpr int PNLD = (PBM + PBN) / 64;            // global->LDS wave instructions per k tile and wavefront
constexpr int PSC_BYTES = 512 + 1024 + 1024;      // sx[128], sw[256], bias[256] as fp32
constexpr int PSC_LOADS = 3;                      // scale loads per wavefront and tile

template <int V>
using IC = std::integral_constant<int, V>;

// compile-time shape of one k iteration of gemm_i8_persist_kernel (see `iteration` there)
template <bool ZERO_, bool CONV_, int S0_, int NSTORE_, int D_, bool RFIRST_, bool SC_, bool ISSUE_, bool NEXT_, int THRESH_>
struct PersistIter {
  static constexpr bool ZERO = ZERO_, CONV = CONV_, RFIRST = RFIRST_, SC = SC_, ISSUE = ISSUE_, NEXT = NEXT_;
  static constexpr int S0 = S0_, NSTORE = NSTORE_, D = D_, THRESH = THRESH_;
};

template <int EPI, int DI, int IMM, bool NT, bool PRIO = true>
__global__ __launch_bounds__(256, PERSIST_MIN_WG) void gemm_i8_persist_kernel(GemmArgs a) {
  static_assert(EPI == EPI_SCALE_BIAS_BF16 || EPI == EPI_GELU_BF16 || EPI == EPI_RESIDUAL_BF16, "epilogues built");
  constexpr bool RES = EPI == EPI_RESIDUAL_BF16;
  static_assert((32 - IMM) % DI == 0, "the held stores of a wavefront are spread evenly over DI iterations");
  constexpr int NS = (32 - IMM) / DI;  // stores per drain iteration
  __shared__ __attribute__((aligned(16))) unsigned char lds[PNST * PSTAGE + 2 * PSC_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave_u >> 1, wn = wave_u & 1;
  const int lr = lane & 31, lh = lane >> 5;

  // ---- the tiles of this workgroup ------------------------------------------------------------
  // Hardware workgroup ids are dealt round-robin to the 8 XCDs.  XCD x owns the contiguous range
  // [x * chunk, (x + 1) * chunk) of logical tile ids; its workgroups walk it side by side, so at any
  // time the tiles in flight on an XCD are neighbours and share operand panels in that XCD's L2.
  const unsigned int total = (unsigned int)a.tiles_m * (unsigned int)a.tiles_n;
  const unsigned int xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per_x = gridDim.x >> 3;
  const unsigned int chunk = (total + 7u) >> 3;
  const unsigned int first = xcd * chunk + slot;
  const unsigned int last = min(total, (xcd + 1u) * chunk);
  if (slot >= chunk || first >= last) return;  // uniform over the workgroup
  const int nt = (int)((last - first + per_x - 1u) / per_x);

  auto tile_origin = [&](unsigned int pid, int& m0, int& n0) __attribute__((always_inline)) {
    const unsigned int per_group = (unsigned int)a.group_m * a.tiles_n;
    const unsigned int first_m = (pid / per_group) * a.group_m;
    const unsigned int gsz = min((unsigned int)a.tiles_m - first_m, (unsigned int)a.group_m);
    const unsigned int in_group = pid % per_group;
    m0 = (int)(first_m + in_group % gsz) * PBM;
    n0 = (int)(in_group / gsz) * PBN;
  };

  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;

  // lane offsets of the tile loads (see gemm_i8_kernel: the XOR swizzle is applied to the global
  // address; slot s of a wavefront's 128 columns holds W row (s % 32) * 4 + s / 32)
  unsigned int dma_off[PNLD];
  auto set_dma = [&](int m0, int n0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < PNLD; ++i) {
      const int rho = 16 * (wave_u + 4 * i) + (lane >> 2);
      const int chunk16 = ((lane & 3) ^ lds_swizzle(rho)) * 16;
      if (i < PBM / 64) {
        dma_off[i] = (unsigned int)((m0 + rho) * a.row_pitch + chunk16);
      } else {
        const int sl = rho - PBM;
        const int wrow = (sl & 128) + (sl & 31) * 4 + ((sl & 127) >> 5);
        dma_off[i] = (unsigned int)((n0 + wrow) * a.row_pitch + chunk16);
      }
      asm volatile("" : "+v"(dma_off[i]));  // a 32-bit value from here on (not a widened 64-bit product)
    }
  };
  auto dma_issue = [&](int kt, int stage_off) __attribute__((always_inline)) {
    const int8_t* xb = a.x + kt * a.x_kstep;
    const int8_t* wb = a.w + kt * a.w_kstep;
    asm volatile("" : "+s"(xb), "+s"(wb));  // tile bases stay scalar: scalar-base load form
#pragma unroll
    for (int i = 0; i < PNLD; ++i) {
      unsigned int off = dma_off[i];
      asm volatile("" : "+v"(off));
      const int8_t* src = (i < PBM / 64 ? xb : wb) + off;
      unsigned char* dst = lds + stage_off + (wave_u + 4 * i) * 1024;
      __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
    }
  };
  // row scales, column scales and bias of a tile, 4 bytes per lane, straight into scale buffer `buf`
  auto scales_issue = [&](int m0, int n0, int buf) __attribute__((always_inline)) {
    unsigned char* sc = lds + PNST * PSTAGE + buf * PSC_BYTES;
    const int mm = m0 + (wave_u & 1) * 64 + lane;
    const int nn = n0 + wave_u * 64 + lane;
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sx + mm), (lptr_t)(sc + (wave_u & 1) * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sw + nn), (lptr_t)(sc + 512 + wave_u * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)((a.bias ? a.bias : a.sw) + nn), (lptr_t)(sc + 1536 + wave_u * 256), 4, 0, 0);
  };

  const int frag_chunk = (lh ^ lds_swizzle(lr)) * 16;
  const int a_off = (wm * 64 + lr) * GLD + frag_chunk;
  const int b_off = PBM * GLD + (wn * 128 + lr) * GLD + frag_chunk;
  auto frags_at = [&](int stage_off, int step, i32x4 (&av)[2], i32x4 (&bv)[4]) __attribute__((always_inline)) {
    const unsigned char* src = lds + stage_off;
    const int flip = step * 32;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < 2) av[i] = *reinterpret_cast<const i32x4*>(src + ((a_off + i * 32 * GLD) ^ flip));
      bv[i] = *reinterpret_cast<const i32x4*>(src + ((b_off + i * 32 * GLD) ^ flip));
    }
  };

  i32x16 acc[2][4];
  i32x4 fa0[2], fb0[4], fa1[2], fb1[4];
  auto mma = [&](const i32x4 (&av)[2], const i32x4 (&bv)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], acc[i][j], 0, 0, 0);
  };
  // first matrix instructions of a tile: the accumulators start from zero
  auto mma_zero_row = [&](int i, const i32x4 (&av)[2], const i32x4 (&bv)[4]) __attribute__((always_inline)) {
    const i32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], z, 0, 0, 0);
  };

  // ---- output of the previous tile --------------------------------------------------------------
  // The lane owns 4 adjacent output columns of each of its 32 rows (MFMA tile i, register r -> row
  // i*32 + 8*(r/4) + 4*lh + r%4); held[i][r] keeps them as two packed bf16 pairs.
  u32x2 held[2][16];
  f32x4 swv, bv4;
  // residual epilogue: values of the IMM rows that leave with the conversion plus the first NS held
  // stores (requested in the tile's last iteration), and of the held stores of the iterations
  // d (slot d & 1), each requested one iteration ahead
  u32x2 res_first[RES ? IMM + NS : 1];
  u32x2 res_ring[2][RES ? NS : 1];
  auto add_residual = [&](u32x2& val, const u32x2& r) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < 2; ++c)
      // bf16 add of the bf16-rounded Linear output and the residual stream
      val[c] = pack_bf16x2(bf16_lo_to_f32(val[c]) + bf16_lo_to_f32(r[c]),
                           bf16_hi_to_f32(val[c]) + bf16_hi_to_f32(r[c]));
  };
  auto convert_begin = [&](const unsigned char* sc) __attribute__((always_inline)) {
    swv = *reinterpret_cast<const f32x4*>(sc + 512 + (wn * 128 + 4 * lr) * 4);
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    bv4 = a.bias ? *reinterpret_cast<const f32x4*>(sc + 1536 + (wn * 128 + 4 * lr) * 4) : z;
  };
  // byte offset of the lane's first element inside an output tile; rows are added as uniform offsets
  const unsigned int voff = (unsigned int)(((wm * 64 + 4 * lh) * a.ldo + wn * 128 + 4 * lr) * 2);
  const unsigned short* prev_base = nullptr;  // out + m0 * ldo + n0 of the tile whose output is held
  typedef __attribute__((address_space(1))) unsigned char* gstore_t;
  auto store_piece = [&](int s) __attribute__((always_inline)) {
    const int i = s >> 4, r = s & 15;
    // (the row pitch is made opaque at every use: as a loop invariant the 32 row offsets would be
    // kept in 64 scalar registers for the whole kernel)
    unsigned int pitch = (unsigned int)a.ldo * 2u;
    asm volatile("" : "+s"(pitch));
    const unsigned char* p = reinterpret_cast<const unsigned char*>(prev_base) +
                             (unsigned int)(i * 32 + 8 * (r >> 2) + (r & 3)) * pitch;
    asm volatile("" : "+s"(p));  // uniform row base in scalar registers, 32-bit lane offset
    unsigned int off = voff;
    asm volatile("" : "+v"(off));
    typedef __attribute__((address_space(1))) u32x2* gdst_t;
    gdst_t dst = (gdst_t)((gstore_t)(uintptr_t)p + off);
    // an output larger than the last-level cache that is read once (qkv, lin1) is streamed out
    if (NT) __builtin_nontemporal_store(held[i][r], dst);
    else *dst = held[i][r];
  };

  auto convert_half = [&](int i, const unsigned char* sc, bool store_now) __attribute__((always_inline)) {
    f32x4 sxv[4];
#pragma unroll
    for (int g = 0; g < 4; ++g)
      sxv[g] = *reinterpret_cast<const f32x4*>(sc + (wm * 64 + i * 32 + 8 * g + 4 * lh) * 4);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float s = sxv[r >> 2][r & 3];
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // three separately rounded fp32 operations (no fused multiply-add)
        float t = (float)acc[i][j][r] * s;
        t = t * swv[j];
        y[j] = t + bv4[j];
      }
      u32x2 o = {pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3])};
      if (EPI == EPI_GELU_BF16) {
        // activation of the bf16-rounded Linear output, as a separate GELU would see it
        o[0] = pack_bf16x2(gelu_erf(bf16_lo_to_f32(o[0])), gelu_erf(bf16_hi_to_f32(o[0])));
        o[1] = pack_bf16x2(gelu_erf(bf16_lo_to_f32(o[1])), gelu_erf(bf16_hi_to_f32(o[1])));
      }
      if (RES && i == 0) add_residual(o, res_first[r]);  // these rows leave at once, residual included
      held[i][r] = o;
      if (store_now && i * 16 + r < IMM) store_piece(i * 16 + r);  // (its registers are free again at once)
      // keep the conversion narrow (four rows at a time): scheduled for parallelism it would hold
      // all 64 values of a half as floats at once
      if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0);
    }
  };
  // residual values of store piece s of the tile whose output is converted next
  const unsigned int voff_res = (unsigned int)(((wm * 64 + 4 * lh) * a.ld_res + wn * 128 + 4 * lr) * 2);
  const unsigned short* prev_res = nullptr;  // residual + m0 * ld_res + n0 of that tile
  auto residual_piece = [&](int s) __attribute__((always_inline)) {
    const int i = s >> 4, r = s & 15;
    unsigned int pitch = (unsigned int)a.ld_res * 2u;
    asm volatile("" : "+s"(pitch));
    const unsigned char* p = reinterpret_cast<const unsigned char*>(prev_res) +
                             (unsigned int)(i * 32 + 8 * (r >> 2) + (r & 3)) * pitch;
    asm volatile("" : "+s"(p));
    unsigned int off = voff_res;
    asm volatile("" : "+v"(off));
    typedef __attribute__((address_space(1))) const u32x2* gsrc_t;
    return *(gsrc_t)((gstore_t)(uintptr_t)p + off);
  };

  // s_waitcnt immediate: vmcnt in bits 3:0 and 15:14 ("at most n operations still in flight"),
  // expcnt 6:4 = 7 (no wait), lgkmcnt 11:8 = 0 (all of this wave's LDS reads done)
  auto wait_imm = [](int n) constexpr { return 0x0070 | (n & 15) | ((n >> 4) << 14); };

  int st[PNST];  // st[j] = LDS offset of the stage holding k tile (current + j); uniform, rotated
  const unsigned char* conv_sc = lds + PNST * PSTAGE;  // scale buffer of the tile whose output is converted next

  // One k iteration; F carries its compile-time shape:
  //   ZERO    first iteration of a tile, accumulators start at zero;
  //   CONV    the previous tile's accumulators are converted first (implies ZERO), IMM stores leave;
  //   S0, NSTORE  held stores S0 .. S0+NSTORE-1 go out after the barrier, ahead of the tile loads;
  //   D       index of a drain iteration (residual epilogue: which residual ring slot it uses);
  //   RFIRST  residual epilogue: the residual values the next conversion needs are requested, ahead of
  //           the tile loads (the tile's last iteration);
  //   SC      the next tile's scales are requested (into scale buffer sc_buf) before the tile loads;
  //   ISSUE   k tile ld_kt is requested into the stage freed at the barrier;
  //   NEXT    a following k tile exists (of this tile or the next);
  //   THRESH  operations younger than the loads of the k tile needed next, i.e. what may stay in
  //           flight across the barrier.
  auto iteration = [&](int ld_kt, int sc_m0, int sc_n0, int sc_buf, auto f) __attribute__((always_inline)) {
    using F = decltype(f);
    constexpr bool ZERO = F::ZERO, CONV = F::CONV, SC = F::SC, ISSUE = F::ISSUE, NEXT = F::NEXT, RFIRST = F::RFIRST;
    constexpr int S0 = F::S0, NSTORE = F::NSTORE, THRESH = F::THRESH, D = F::D;
    if constexpr (CONV) {
      if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
      // residual epilogue: the values requested in the last iteration have landed (its tile loads, the
      // youngest operations in flight, need not have)
      if constexpr (RES) __builtin_amdgcn_s_waitcnt(0x0F70 | PNLD);  // vmcnt <= PNLD, nothing else waited for
      // (the fences keep the zero-initialised matrix instructions of a row half behind the conversion
      // of that half: hoisted above it, old and new accumulators would be live together)
      convert_begin(conv_sc);
      convert_half(0, conv_sc, true);  // the first IMM pieces leave as they are converted; the rest is held
      __builtin_amdgcn_sched_barrier(0);
      // residual epilogue: the first fragments of this tile are read here rather than in the previous
      // iteration (whose barrier made the k tile visible), so that they and the residual values the
      // conversion consumes are not live together
      if constexpr (RES) frags_at(st[0], 0, fa0, fb0);
      mma_zero_row(0, fa0, fb0);
      convert_half(1, conv_sc, true);
      __builtin_amdgcn_sched_barrier(0);
      mma_zero_row(1, fa0, fb0);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
      frags_at(st[0], 1, fa1, fb1);
    } else {
      frags_at(st[0], 1, fa1, fb1);
      if constexpr (ZERO) {
        mma_zero_row(0, fa0, fb0);
        mma_zero_row(1, fa0, fb0);
      } else {
        mma(fa0, fb0);
      }
#pragma unroll
      for (int g = 0; g < 6; ++g) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // own LDS reads of this stage done; own share of the next k tile landed; then all waves meet
    __builtin_amdgcn_s_waitcnt(wait_imm(THRESH));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (RES && NSTORE > 0) {
      // the next drain iteration's residual values first, then this iteration's stores: the wait for
      // this iteration's values (requested an iteration ago, or with the conversion's) then covers
      // nothing younger than them
      constexpr bool MORE = S0 + 2 * NSTORE <= 32;  // another drain iteration follows
      if constexpr (MORE) {
#pragma unroll
        for (int s = 0; s < NSTORE; ++s) res_ring[(D + 1) & 1][s] = residual_piece(S0 + NSTORE + s);
      }
      if constexpr (D > 0) {
        constexpr int younger = NSTORE + PNLD + (MORE ? NSTORE : 0);
        __builtin_amdgcn_s_waitcnt(0x0F70 | (younger & 15) | ((younger >> 4) << 14));
      }
#pragma unroll
      for (int s = 0; s < NSTORE; ++s) {
        const int piece = S0 + s;
        add_residual(held[piece >> 4][piece & 15], D == 0 ? res_first[IMM + s] : res_ring[D & 1][s]);
      }
    }
#pragma unroll
    for (int s = 0; s < NSTORE; ++s) store_piece(S0 + s);
    if constexpr (RES && RFIRST) {
#pragma unroll
      for (int s = 0; s < IMM + NS; ++s) res_first[s] = residual_piece(s);
    }
    if constexpr (SC) scales_issue(sc_m0, sc_n0, sc_buf);
    if constexpr (ISSUE) dma_issue(ld_kt, st[0]);
    if constexpr (NEXT) frags_at(st[1], 0, fa0, fb0);
    mma(fa1, fb1);
    if constexpr (!(RES && (NSTORE > 0 || RFIRST))) {
#pragma unroll
      for (int g = 0; g < 6; ++g) {
        if constexpr (NEXT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (g < NSTORE) __builtin_amdgcn_sched_group_barrier(0x040, 1, 0);
        if constexpr (SC) { if (g < PSC_LOADS) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0); }
        if constexpr (ISSUE) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }
    // The matrix instructions are pure values to the compiler: nothing but their operands ties them
    // to this iteration, and instruction selection has been seen to sink three iterations' worth of
    // them below the following barriers (their fragments then all live at once).  Passing the
    // accumulators through an empty asm statement here pins every chain between two iterations.
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(acc[i][j]));
    __builtin_amdgcn_sched_barrier(0);
    const int t = st[0];
#pragma unroll
    for (int j = 0; j + 1 < PNST; ++j) st[j] = st[j + 1];
    st[PNST - 1] = t;
  };
  // plain iteration: tile loads only, one k tile in flight across the barrier
  using Plain = PersistIter<false, false, 0, 0, 0, false, false, true, true, PNLD>;

  // A wavefront in its K loop runs at raised priority and drops to the base priority while it converts
  // the previous tile's accumulators (PRIO): when its SIMD partner - the other resident workgroup's
  // wavefront - is in its loop at that time, the partner's matrix instructions issue as soon as they
  // are ready and the conversion's vector work fills the slots between them (lin1 + GELU -3 %).
  //
  // Two resident workgroups that start in the same cycle run the same code on the same CU and tend
  // to stay in step: both in their LDS reads, both at their barriers, both converting.  The
  // workgroup whose first wavefront sits in an odd wave slot of its SIMD starts a.skew * 64 cycles late.
  if (a.skew > 0) {
    const unsigned int hw_id = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (3 << 11));  // HW_ID, WAVE_ID bits 3:0
    int* flag = reinterpret_cast<int*>(lds + PNST * PSTAGE);
    if (tid == 0) *flag = (int)(hw_id & 1u);
    __syncthreads();
    const int odd = __builtin_amdgcn_readfirstlane(*flag);
    __syncthreads();
    if (odd)
      for (int i = 0; i < a.skew; ++i) __builtin_amdgcn_s_sleep(1);
  }

  if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
  // ---- prologue: the first tile's scales and first three k tiles --------------------------------
  const int nk = a.K / GBK;
  int m0, n0;
  tile_origin(first, m0, n0);
  set_dma(m0, n0);
  scales_issue(m0, n0, 0);
#pragma unroll
  for (int j = 0; j < PNST; ++j) {
    st[j] = j * PSTAGE;
    dma_issue(j, st[j]);
  }
  __builtin_amdgcn_s_waitcnt(wait_imm((PNST - 1) * PNLD));
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  frags_at(st[0], 0, fa0, fb0);

  // The last three iterations of a tile request the next tile's scales and first three k tiles.  The
  // last tile of the list requests its own again (nobody reads them): every tile then runs the same
  // code with the same operation counts in flight.
  auto tile_tail = [&](int ti) __attribute__((always_inline)) {
    // the output of this tile is converted at the top of the next one (or after the loop)
    prev_base = reinterpret_cast<const unsigned short*>(a.out) + (int64_t)m0 * a.ldo + n0;
    if (RES) prev_res = a.residual + (int64_t)m0 * a.ld_res + n0;
    conv_sc = lds + PNST * PSTAGE + (ti & 1) * PSC_BYTES;
    const unsigned int nxt = ti + 1 < nt ? (unsigned int)(ti + 1) : (unsigned int)ti;
    tile_origin(first + nxt * per_x, m0, n0);
    set_dma(m0, n0);
    iteration(0, m0, n0, (ti + 1) & 1, PersistIter<false, false, 0, 0, 0, false, true, true, true, PNLD>{});
    iteration(1, 0, 0, 0, PersistIter<false, false, 0, 0, 0, false, false, true, true, PNLD + PSC_LOADS>{});
    iteration(2, 0, 0, 0, PersistIter<false, false, 0, 0, 0, true, false, true, !RES, PNLD>{});
  };

  // ---- first tile: nothing to convert or store yet ----------------------------------------------
  iteration(3, 0, 0, 0, PersistIter<true, false, 0, 0, 0, false, false, true, true, PNLD>{});
  for (int kt = 1; kt < nk - 3; ++kt) iteration(kt + 3, 0, 0, 0, Plain{});
  tile_tail(0);

  // residual values requested per drain iteration (they sit between the stores and tile loads that a
  // threshold counts)
  constexpr int NR = RES ? NS : 0;
  for (int ti = 1; ti < nt; ++ti) {
    // Iterations 0 .. DI-1 carry the previous tile's held stores, each ahead of its tile loads.
    // Younger than the k tile needed next: in iteration 0 one k tile and the IMM stores issued with
    // the conversion; in iteration 1 those stores, iteration 0's (and the residual values requested
    // with them) and one k tile; from then on the stores (and residual requests) of the iteration
    // before and one k tile.
    iteration(3, 0, 0, 0, PersistIter<true, true, IMM, NS, 0, false, false, true, true, PNLD + IMM>{});
    iteration(4, 0, 0, 0, PersistIter<false, false, IMM + NS, NS, 1, false, false, true, true, PNLD + IMM + NS + NR>{});
    auto drain = [&](auto self, auto d) __attribute__((always_inline)) {
      constexpr int D = decltype(d)::value;
      if constexpr (D < DI) {
        iteration(D + 3, 0, 0, 0, PersistIter<false, false, IMM + D * NS, NS, D, false, false, true, true, PNLD + NS + NR>{});
        self(self, IC<D + 1>{});
      }
    };
    drain(drain, IC<2>{});
    iteration(DI + 3, 0, 0, 0, PersistIter<false, false, 0, 0, 0, false, false, true, true, PNLD + NS>{});
    for (int kt = DI + 1; kt < nk - 3; ++kt) iteration(kt + 3, 0, 0, 0, Plain{});
    tile_tail(ti);
  }

  // ---- the last tile's output ---------------------------------------------------------------------
  if constexpr (RES) __builtin_amdgcn_s_waitcnt(0x0F70 | PNLD);  // the residual values requested in the last iteration
  convert_begin(conv_sc);
  convert_half(0, conv_sc, false);
#pragma unroll
  for (int s = 0; s < 16; ++s) store_piece(s);
  if constexpr (RES) {
    // the second half's residual values (only the first NS of them were requested ahead)
    u32x2 res_late[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) res_late[r] = residual_piece(16 + r);
    convert_half(1, conv_sc, false);
#pragma unroll
    for (int r = 0; r < 16; ++r) add_residual(held[1][r], res_late[r]);
  } else {
    convert_half(1, conv_sc, false);
  }
#pragma unroll
  for (int s = 16; s < 32; ++s) store_piece(s);
  __builtin_amdgcn_s_waitcnt(0x0070);  // the unused loads of the last tail land before the LDS is given back
}

static int persist_grid() {
  static const int grid = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return (2 * cus) / 8 * 8;
  }();
  return grid;
}

bool gemm_i8_persist_covers(int epi, const GemmArgs& a) {
  // 0: off; 1 (default): the scale + bias and GELU epilogues, where it measures faster than one
  // workgroup per tile (qkv -20 %, lin1 -5 % at 65536 rows), from two tiles per workgroup on; 2: also the
  // residual epilogue (measured 4-10 % slower than three workgroups per CU) and any tile count
  const int mode = knob_or(KNOB_GEMM_PERSIST, 1);
  if (mode <= 0) return false;
  if (mode == 1 && epi == EPI_RESIDUAL_BF16) return false;
  if (epi != EPI_SCALE_BIAS_BF16 && epi != EPI_GELU_BF16 && epi != EPI_RESIDUAL_BF16) return false;
  if (epi == EPI_RESIDUAL_BF16 && a.ld_res >= (1ll << 23)) return false;
  if (a.M % PBM != 0 || a.N % PBN != 0 || a.K / GBK < 12) return false;
  if (a.dst_row || a.tile_counters || a.ldo >= (1ll << 23)) return false;  // 32-bit row offsets inside a tile
  // worth it from two tiles per workgroup on (mode 2: wherever it is built)
  return mode >= 2 || (int64_t)(a.M / PBM) * (a.N / PBN) >= 2ll * persist_grid();
}

int gemm_i8_persist_launch(int epi, const GemmArgs& a0, hipStream_t stream) {
  GemmArgs a = a0;
  // start delay of every second workgroup: knob x 64 cycles per k tile of a tile's K loop
  a.skew = min(max(knob_or(KNOB_GEMM_PERSIST_SKEW, 22), 0) * (a.K / GBK), 1 << 16);
  a.prio = knob_or(KNOB_GEMM_PERSIST_PRIO, 1) != 0;
  a.tiles_m = a.M / PBM;
  a.tiles_n = a.N / PBN;
  a.group_m = a.tiles_n <= 6 ? 1 : 1024 / PBM;
  const int64_t total = (int64_t)a.tiles_m * a.tiles_n;
  const unsigned int grid = (unsigned int)min((int64_t)persist_grid(), ((total + 7) / 8) * 8);
  const bool di16 = a.K / GBK >= 20;
#define SF_PERSIST_P(E, P)                                                                                       \
  do {                                                                                                           \
    if (di16 && a.stream_out) hipLaunchKernelGGL((gemm_i8_persist_kernel<E, 16, 16, true, P>), dim3(grid), dim3(256), 0, stream, a);  \
    else if (di16) hipLaunchKernelGGL((gemm_i8_persist_kernel<E, 16, 16, false, P>), dim3(grid), dim3(256), 0, stream, a);           \
    else if (a.stream_out) hipLaunchKernelGGL((gemm_i8_persist_kernel<E, 8, 16, true, P>), dim3(grid), dim3(256), 0, stream, a);     \
    else hipLaunchKernelGGL((gemm_i8_persist_kernel<E, 8, 16, false, P>), dim3(grid), dim3(256), 0, stream, a);                      \
  } while (0)
#define SF_PERSIST(E) do { if (a.prio) SF_PERSIST_P(E, true); else SF_PERSIST_P(E, false); } while (0)
  if (epi == EPI_GELU_BF16) SF_PERSIST(EPI_GELU_BF16);
  else if (epi == EPI_RESIDUAL_BF16) SF_PERSIST(EPI_RESIDUAL_BF16);
  else SF_PERSIST(EPI_SCALE_BIAS_BF16);
#undef SF_PERSIST
#undef SF_PERSIST_P
  return check_launch("gemm_i8_persist_kernel");
}

}  // namespace samfast
