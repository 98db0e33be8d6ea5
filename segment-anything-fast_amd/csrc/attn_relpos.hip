// Attention with decomposed relative-position bias for gfx950 (bf16 MFMA).
//
//   out = softmax(q k^T * sm_scale + rel_h[q, kh] + rel_w[q, kw]) v,   key n = kh*gw + kw
//
// Both kernels compute the TRANSPOSED score tile S^T = K Q^T with
// v_mfma_f32_32x32x16_bf16 (A = 32 keys x 16 channels from LDS, B = Q^T held in
// registers for the whole kernel).  In the MFMA result layout a lane then owns
// ONE query (column lane%32) and 16 keys per tile (rows 8*(r/4) + 4*(lane/32) +
// r%4), so the softmax row statistics are per-lane scalars: the row maximum and
// sum are reduced in registers plus one exchange with lane^32.  The same
// registers, converted to bf16, are directly the B operand (P^T) of the second
// product O^T = V^T P^T.  K and V tiles travel global memory -> LDS directly
// (global_load_lds_dwordx4), row-major; the V^T operand is formed by transposing
// LDS reads (ds_read_b64_tr_b16) that follow the key order of the P registers.
// The exponent offset of the online softmax follows the running maximum lazily
// (only in steps of more than 2^8), so the output accumulators are rescaled a
// few times per row of keys instead of once per key tile.
//
// Everything runs in the base-2 domain with the exact scale folded into the
// exponent argument: p = exp2(fma(s, c, -m)), c = sm_scale*log2(e), so q is
// never re-rounded.
//
// global kernel (gw == 64): one key tile is exactly one key grid row, so
//   rel_w is identical for every key tile -> kept in registers as the INITIAL
//   accumulator of the score MFMA (pre-divided by sm_scale), and rel_h is one
//   scalar per (query, key tile) -> folded into the running-max bookkeeping.
//   With FUSED the two factors are produced in the prologue by MFMA from the
//   (2S-1, hd) tables: rel_h^T = Rh[qh+gh-1-kh] Q^T directly, rel_w through the
//   full product T = Rw Q^T followed by the per-query diagonal gather
//   rel_w[q, kw] = T[qw - kw + 63, q] staged through LDS.
//
// window kernel (N <= 208, e.g. 14x14): all keys of one (window, head) fit in
//   LDS; eight wavefronts stage them, each then owns one 32-query tile and walks
//   the key tiles with an online softmax (under 128 registers per lane, so four
//   wavefronts per SIMD are resident).  The bias is added BY THE MFMA: the
//   channel axis is extended by 32 slots, B carries [rel_h[q, 0..15] | rel_w[q,
//   0..15]] / sm_scale in bf16 and A carries the 0/1 indicators [n/gw == j |
//   n%gw == j]; slot 15 of the rel_h half is the padding mask (B = -1e30, A = 1
//   for key rows >= N).
#include "attn_relpos_shared.hpp"

namespace samfast {

// =============================================================================
// global kernel: gw == 64, N % (32*WAVES*QT) == 0.  WAVES = 4: two workgroups per CU; WAVES = 8:
// one workgroup of 256 queries per CU, which stages every K / V tile once for twice the queries
// (the global->LDS loads are a fifth of the kernel's time), taken when the grid is large enough
// =============================================================================
template <int HD, int QT, int WAVES>
struct GlobalCfg {
  static constexpr int KS = HD / 16;          // score k-steps
  static constexpr int DT = (HD + 31) / 32;   // output channel tiles
  static constexpr int BM = 32 * WAVES * QT;  // queries per workgroup
  // K and V tiles travel global memory -> LDS directly (global_load_lds_dwordx4), row-major,
  // in 16-byte pieces: a staged row is HD/8 data pieces plus one spare piece that no load
  // writes (its lanes are masked), so rows are HD + 8 elements apart (bank spread) and 64 rows
  // are exactly PPR wave instructions of 64 pieces.
  static constexpr int PPR = HD / 8 + 1;      // pieces per staged row
  static constexpr int KSTR = PPR * 8;        // K row stride in LDS (elements)
  static constexpr int VSTR = PPR * 8;        // V row stride in LDS (elements)
  static constexpr int KBYTES = 64 * KSTR * 2;
  static constexpr int VBYTES = 64 * VSTR * 2;
  // when HD is not a multiple of 32 the last output tile has spare rows: the spare piece of
  // every V row is preset to (1, 0, ..., 0), i.e. channel HD of every key is one, and the P V
  // product delivers the softmax denominator for free
  static constexpr bool ONES_ROW = HD % 32 != 0;
  static constexpr int STAGE = KBYTES + VBYTES;
  static constexpr int RELH_OFF = 2 * STAGE;
  static constexpr int RELH_BYTES = 64 * BM * 4;
  static constexpr int LDS_BYTES = RELH_OFF + RELH_BYTES;
  static constexpr int XSTR = 65;             // gather scratch row stride (floats)
  static constexpr int X_BYTES = WAVES * 32 * XSTR * 4;
  static constexpr int NDMA = PPR;            // wave instructions per K (or V) tile
  static constexpr int DPW = (NDMA + WAVES - 1) / WAVES;  // of which each wave issues at most
  // the scratch is dead (barrier) before the stages and relhT are written
  static_assert(X_BYTES <= LDS_BYTES, "gather scratch must fit in the workgroup's LDS");
};

template <typename T, int HD, int QT, bool FUSED, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES == 4 ? 2 : 1) void attn_global_kernel(AttnArgs a) {
  using C = GlobalCfg<HD, QT, WAVES>;
  __shared__ __attribute__((aligned(16))) unsigned char lds[C::LDS_BYTES];
  float* relhT = reinterpret_cast<float*>(lds + C::RELH_OFF);  // [kh][BM]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 31, lh = lane >> 5;

  const unsigned int nqb = a.N / C::BM;
  const unsigned int total = (unsigned int)(a.B * a.nH) * nqb;
  const unsigned int pid = xcd_contiguous_id(blockIdx.x, total);
  if (pid >= total) return;
  const int bh = pid / nqb, qb = pid % nqb;
  const int b = bh / a.nH, h = bh % a.nH;
  const int q_wg = qb * C::BM;            // first query of the workgroup
  const int q_wave = wave * 32 * QT;      // first query of the wave inside the workgroup

  const unsigned short* kbase = a.k + b * a.k_sb + h * a.k_sh;
  const unsigned short* vbase = a.v + b * a.v_sb + h * a.v_sh;
  const unsigned short* qbase = a.q + b * a.q_sb + h * a.q_sh;

  // ---- K/V tiles: global memory -> LDS without staging registers ----------------
  // wave instruction n of a tile fills pieces 64n .. 64n+63 of the stage; piece P is row
  // P / PPR, 16-byte column P % PPR (the spare column stays unwritten: lane masked)
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  unsigned int koff[C::DPW], voff[C::DPW];  // unsigned lane offsets: scalar-base load form
  bool dma_ok[C::DPW];
#pragma unroll
  for (int m = 0; m < C::DPW; ++m) {
    const int P = 64 * (wave_u + WAVES * m) + lane;
    const int row = P / C::PPR, col = P % C::PPR;
    const bool ok = (wave_u + WAVES * m < C::NDMA) && col < HD / 8;
    dma_ok[m] = ok;
    koff[m] = ok ? (unsigned int)(row * (int)a.k_sn + col * 8) * 2u : 0u;  // bytes
    voff[m] = ok ? (unsigned int)(row * (int)a.v_sn + col * 8) * 2u : 0u;
  }
  auto stage_dma = [&](int kt, int buf) {
    const unsigned char* kb = reinterpret_cast<const unsigned char*>(kbase + (int64_t)kt * 64 * a.k_sn);
    const unsigned char* vb = reinterpret_cast<const unsigned char*>(vbase + (int64_t)kt * 64 * a.v_sn);
    // tile bases in scalar registers, 32-bit lane offsets at the point of use: the loads take the
    // scalar-base form, which disturbs the MFMA stream several times less than 64-bit lane addresses
    asm volatile("" : "+s"(kb), "+s"(vb));
    unsigned char* kl = lds + buf * C::STAGE + wave_u * 1024;
#pragma unroll
    for (int m = 0; m < C::DPW; ++m) {
      if (wave_u + WAVES * m < C::NDMA && dma_ok[m]) {
        unsigned int ok_ = koff[m], ov_ = voff[m];
        asm volatile("" : "+v"(ok_), "+v"(ov_));
        __builtin_amdgcn_global_load_lds((gptr_t)(kb + ok_), (lptr_t)(kl + m * WAVES * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(vb + ov_), (lptr_t)(kl + C::KBYTES + m * WAVES * 1024), 16, 0, 0);
      }
    }
  };
  // V^T operand of the P V product through transposing LDS reads (ds_read_b64_tr_b16): in
  // each group of 16 lanes, lane l receives as element j the l%4-th 16-bit value of the 8
  // bytes addressed by lane 4j + l/4 of the group.  Source lane 4j + i therefore points at
  // key j of the lane half's four keys, channels 4i .. 4i+3 of the group's 16 channels, and
  // lane l ends up with channel l of four consecutive keys: the MFMA A operand.
  int vrd[C::DT];
  {
    const int g = lane >> 4, sl = lane & 15;
    const int key = 4 * (g >> 1) + (sl >> 2);
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) {
      int d = 32 * dt + 16 * (g & 1) + 4 * (sl & 3);
      if (d >= HD + 8) d = HD + 4;  // past the spare piece (1, 0, .., 0): its zero half
      vrd[dt] = (key * C::VSTR + d) * 2;
    }
  }
  // The reads are issued as inline asm: the compiler would otherwise make each of them wait
  // for every global->LDS load in flight (the next tile), and their completion is awaited by
  // hand (LDS operations complete in order, so "all but the youngest n" is a counter value).
  const unsigned int lds_base = (unsigned int)(uintptr_t)((__attribute__((address_space(3))) unsigned char*)lds);
  auto vt_issue = [&](unsigned int stage_addr, auto jc, u32x2 (&f)[2 * C::DT]) {
    constexpr int j = decltype(jc)::value;
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) {
      const unsigned int addr = stage_addr + vrd[dt];
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f[2 * dt]) : "v"(addr), "n"(C::KBYTES + 16 * j * C::VSTR * 2) : "memory");
      asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(f[2 * dt + 1]) : "v"(addr), "n"(C::KBYTES + (16 * j + 8) * C::VSTR * 2) : "memory");
    }
  };
  // all LDS operations of this wave except the youngest KEEP are complete; f is valid after it
  auto vt_wait = [&](auto keepc, u32x2 (&f)[2 * C::DT]) {
    constexpr int KEEP = decltype(keepc)::value;
    if constexpr (C::DT == 3)
      asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]) : "n"(KEEP));
    else
      asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]) : "n"(KEEP));
  };

  // ---- Q^T operand: lane holds query lr of tile t, channels 16s + 8lh .. +7 ----
  u32x4 qf[QT][C::KS];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const unsigned short* qp = qbase + (int64_t)(q_wg + q_wave + 32 * t + lr) * a.q_sn + 8 * lh;
#pragma unroll
    for (int s = 0; s < C::KS; ++s) qf[t][s] = load_x8_global(qp + 16 * s);
  }

  // ---- bias prologue -----------------------------------------------------------
  // b1[t][nt][r]: rel_w / sm_scale for the lane's query and key column kw of the
  // score-tile layout.  relhT[kh][q]: rel_h * log2(e).
  f32x16 b1[QT][2];
  auto first_tile = [&]() {
    if (C::ONES_ROW && tid < 128) {  // spare piece of every V row of both stages: (1, 0, .., 0)
      const int buf = tid >> 6, row = tid & 63;
      const u32x4 one = {T::kOne, 0u, 0u, 0u};
      *reinterpret_cast<u32x4*>(lds + buf * C::STAGE + C::KBYTES + (row * C::VSTR + HD) * 2) = one;
    }
    stage_dma(0, 0);
  };
  auto relh_from_table = [&]() {
    const unsigned short* th = a.rh;
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      const int qh = (q_wg + q_wave + 32 * t) >> 6;  // one grid row per 32-query tile
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int kh_row = 32 * mt + lr;
        int trow = qh - kh_row + a.gh - 1;
        trow = max(0, min(trow, 2 * a.gh - 2));
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < C::KS; ++s) {
          const u32x4 av = load_x8_global(th + trow * HD + 16 * s + 8 * lh);
          acc = T::mfma(av, qf[t][s], acc);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kh = 32 * mt + 8 * (r >> 2) + 4 * lh + (r & 3);
          relhT[kh * C::BM + q_wave + 32 * t + lr] = acc[r] * kLog2e;
        }
      }
    }
  };
  if (FUSED) {
    const unsigned short* tw = a.rw;
    // rel_w: T[rel][q] for rel in [0,128) in two passes of 64 through LDS scratch
    float* X = reinterpret_cast<float*>(lds) + wave * 32 * C::XSTR;
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      const int qw = (q_wg + q_wave + 32 * t + lr) & 63;
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int mt = 2 * pass + half;
          const int trow = min(32 * mt + lr, 126);
          f32x16 acc;
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
          for (int s = 0; s < C::KS; ++s) {
            const u32x4 av = load_x8_global(tw + trow * HD + 16 * s + 8 * lh);
            acc = T::mfma(av, qf[t][s], acc);
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int rel_local = 32 * half + 8 * (r >> 2) + 4 * lh + (r & 3);
            X[lr * C::XSTR + rel_local] = acc[r];
          }
        }
        wave_lds_fence();
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int kw = 32 * nt + 8 * (r >> 2) + 4 * lh + (r & 3);
            const int rel = qw + 63 - kw;
            const float val = X[lr * C::XSTR + (rel & 63)] * a.inv_scale;  // always in range
            if (pass == 0) b1[t][nt][r] = val;
            else b1[t][nt][r] = (rel >= 64) ? val : b1[t][nt][r];
          }
        wave_lds_fence();
      }
    }
    __syncthreads();  // every wave is done with the scratch: the stages may be filled
    first_tile();     // in flight while rel_h is formed
    relh_from_table();
  } else {
    first_tile();
    const unsigned short* rhb = a.rh + b * a.rh_sb + h * a.rh_sh + (int64_t)q_wg * a.rh_sn;
    for (int idx = tid; idx < C::BM * a.gh; idx += 64 * WAVES) {
      const int ql = idx % C::BM, kh = idx / C::BM;
      relhT[kh * C::BM + ql] = T::from_bits(rhb[(int64_t)ql * a.rh_sn + kh]) * kLog2e;
    }
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      const unsigned short* rwp =
          a.rw + b * a.rw_sb + h * a.rw_sh + (int64_t)(q_wg + q_wave + 32 * t + lr) * a.rw_sn;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x2 w = *reinterpret_cast<const u32x2*>(rwp + 32 * nt + 8 * j + 4 * lh);
          b1[t][nt][4 * j + 0] = T::lo(w[0]) * a.inv_scale;
          b1[t][nt][4 * j + 1] = T::hi(w[0]) * a.inv_scale;
          b1[t][nt][4 * j + 2] = T::lo(w[1]) * a.inv_scale;
          b1[t][nt][4 * j + 3] = T::hi(w[1]) * a.inv_scale;
        }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of tile 0 has landed
  __syncthreads();                                   // tile 0 and relhT complete

  // ---- main loop over key grid rows ---------------------------------------------
  f32x16 oacc[QT][C::DT];
  float m_i[QT], l_i[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m_i[t] = -INFINITY;
    l_i[t] = 0.f;
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[t][dt][r] = 0.f;
  }

  const int nkt = a.N / 64;
  for (int kt = 0; kt < nkt; ++kt) {
    const unsigned int v_stage = lds_base + (kt & 1) * C::STAGE;
    if (kt + 1 < nkt) stage_dma(kt + 1, (kt + 1) & 1);  // that stage was last read before the barrier

    // S^T = K Q^T, accumulator initialised with rel_w / sm_scale
    const unsigned char* kl = lds + (kt & 1) * C::STAGE;
    f32x16 s[QT][2];
#pragma unroll
    for (int ks = 0; ks < C::KS; ++ks) {
      // the two key half-tiles are independent accumulator chains: alternate them
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        const u32x4 av = *reinterpret_cast<const u32x4*>(
            kl + ((32 * nt + lr) * C::KSTR + 16 * ks + 8 * lh) * 2);
#pragma unroll
        for (int t = 0; t < QT; ++t)  // the first step takes rel_w / sm_scale as its accumulator input
          s[t][nt] = T::mfma(av, qf[t][ks], ks == 0 ? b1[t][nt] : s[t][nt]);
      }
    }

    // the V^T fragments of the first two key steps travel under the softmax
    using std::integral_constant;
    constexpr int NF = 2 * C::DT;
    u32x2 vf[2][NF];
    vt_issue(v_stage, integral_constant<int, 0>{}, vf[0]);
    vt_issue(v_stage, integral_constant<int, 1>{}, vf[1]);

    // online softmax, one query per lane
    u32x4 pk[QT][4];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float mx = s[t][0][0];
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[t][0][r]);
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[t][1][r]);
      mx = max_with_lane_xor32(mx);
      const float b0 = relhT[kt * C::BM + q_wave + 32 * t + lr];
      // lazy reference: the exponent offset m_i follows the running maximum only when that has
      // grown by more than kLazyLog2 (p stays <= 2^kLazyLog2; the final division by the
      // denominator, accumulated with the same offsets, makes the result independent of it),
      // so the accumulators are rescaled a few times per row of keys instead of once per tile
      const float m_new = fmaxf(m_i[t], fmaf(mx, a.c, b0));
      float alpha = 1.0f;
      if (__any(m_new - m_i[t] > kLazyLog2)) {  // uniform; first tile: m_i = -inf
        alpha = fast_exp2(m_i[t] - m_new);
        m_i[t] = m_new;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[t][dt][r] *= alpha;
      }
      const float neg_mrow = b0 - m_i[t];
      float lsum = 0.f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fast_exp2(fmaf(s[t][nt][r], a.c, neg_mrow));
          s[t][nt][r] = p;
          if (!C::ONES_ROW) lsum += p;
        }
      if (!C::ONES_ROW) l_i[t] = l_i[t] * alpha + lsum;
#pragma unroll
      for (int j = 0; j < 4; ++j) pk[t][j] = cvt_x8<T>(s[t][j >> 1], 8 * (j & 1));
    }

    // O^T += V^T P^T, the V^T fragments of key step j+1 in flight under the MFMAs of step j
    {
      auto pv_step = [&](auto jc, u32x2 (&f)[2 * C::DT]) {
        constexpr int j = decltype(jc)::value;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
          const u32x4 w = {f[2 * dt][0], f[2 * dt][1], f[2 * dt + 1][0], f[2 * dt + 1][1]};
#pragma unroll
          for (int t = 0; t < QT; ++t)
            oacc[t][dt] = T::mfma(w, pk[t][j], oacc[t][dt]);
        }
      };
      vt_wait(integral_constant<int, NF>{}, vf[0]);
      pv_step(integral_constant<int, 0>{}, vf[0]);
      vt_issue(v_stage, integral_constant<int, 2>{}, vf[0]);
      vt_wait(integral_constant<int, NF>{}, vf[1]);
      pv_step(integral_constant<int, 1>{}, vf[1]);
      vt_issue(v_stage, integral_constant<int, 3>{}, vf[1]);
      vt_wait(integral_constant<int, NF>{}, vf[0]);
      pv_step(integral_constant<int, 2>{}, vf[0]);
      vt_wait(integral_constant<int, 0>{}, vf[1]);
      pv_step(integral_constant<int, 3>{}, vf[1]);
    }

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's share of tile kt+1 has landed
    __syncthreads();
  }

  // ---- epilogue: O = acc / l, 4 adjacent channels per store --------------------
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    float l;
    if (C::ONES_ROW) {
      // output row HD (the ones row) = tile DT-1, row HD % 32, held by the lh = (HD % 32) / 4 % 2 lanes
      constexpr int orow = HD % 32;
      constexpr int oreg = 4 * (orow / 8) + orow % 4, olh = (orow / 4) % 2;
      const float own = oacc[t][C::DT - 1][oreg];
      const float other = xor32(own);
      l = (lh == olh) ? own : other;
    } else {
      l = l_i[t] + xor32(l_i[t]);
    }
    const float inv = 1.0f / l;
    unsigned short* op = a.out + b * a.o_sb + h * a.o_sh + (int64_t)(q_wg + q_wave + 32 * t + lr) * a.o_sn;
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = 32 * dt + 8 * j + 4 * lh;
        if (d < HD) {
          const u32x2 o = {T::pack2(oacc[t][dt][4 * j] * inv, oacc[t][dt][4 * j + 1] * inv),
                           T::pack2(oacc[t][dt][4 * j + 2] * inv, oacc[t][dt][4 * j + 3] * inv)};
          *reinterpret_cast<u32x2*>(op + d) = o;
        }
      }
  }
}

// =============================================================================
// window kernel: gh <= 15, gw <= 16, N = gh*gw <= 208; one workgroup per (window, head)
// =============================================================================
// Eight wavefronts: all of them stage K / V, wavefront w then owns query tile w (32 queries;
// 7 tiles for 196 tokens).  Registers are kept under 128 per lane (online softmax over the
// key tiles instead of holding all scores) so that two workgroups = four wavefronts per SIMD
// are resident and fill each other's pipeline gaps.
template <int HD>
struct WindowCfg {
  static constexpr int KS = HD / 16;
  static constexpr int DT = (HD + 31) / 32;
  static constexpr int NMAX = 208;
  static constexpr int NT = 7;                 // key tiles of 32
  static constexpr int WAVES = 8;
  static constexpr int THREADS = 64 * WAVES;
  // K and V rows travel global memory -> LDS directly, row-major, in 16-byte pieces; a staged
  // row is HD/8 data pieces and one spare piece that no load writes (rows HD + 8 elements apart)
  static constexpr int PPR = HD / 8 + 1;
  static constexpr int KSTR = PPR * 8;
  static constexpr int VSTR = PPR * 8;
  static constexpr int KBYTES = NMAX * KSTR * 2;
  static constexpr int VBYTES = NMAX * VSTR * 2;
  static constexpr int NDMA = (NMAX * PPR + 63) / 64;        // wave instructions per K (or V) window
  static constexpr int DPW = (NDMA + WAVES - 1) / WAVES;     // of which each wavefront issues at most
  // when HD is not a multiple of 32 the last output tile has spare rows: the spare piece of
  // every V row is preset to (1, 0, ..., 0) and row HD of O^T is the softmax denominator
  static constexpr bool ONES_ROW = HD % 32 != 0;
  static constexpr int XSTR = 50;              // bf16 elements per scratch row: 32 products stored in reverse + read-ahead room; 25 words: odd, no bank conflicts
  static constexpr int XBYTES_WAVE = 32 * XSTR * 2;  // gather scratch, aliases the V area before V arrives
  // the 0/1 indicator operands of the bias MFMAs as a table behind V: entry e < 16 is the one-hot
  // vector of slot e (16 elements of 2 bytes), entry 16 all zeros; a lane reads its half by one
  // 16-byte LDS read instead of building it from compares
  static constexpr int HOT_ENTRIES = 17;
  static constexpr int HOT_BYTES = HOT_ENTRIES * 32;
  static constexpr int LDS_BYTES = KBYTES + VBYTES + HOT_BYTES;
  static_assert(WAVES * XBYTES_WAVE <= VBYTES, "gather scratch must fit in the V area");
  static_assert(NT <= WAVES, "one query tile per wavefront");
};

template <typename T, int HD, bool FUSED>
__global__ __launch_bounds__(WindowCfg<HD>::THREADS, 2) void attn_window_kernel(AttnArgs a) {
  using C = WindowCfg<HD>;
  __shared__ __attribute__((aligned(16))) unsigned char lds[C::LDS_BYTES];
  unsigned char* kl = lds;
  unsigned char* vl = lds + C::KBYTES;
  unsigned char* hot = lds + C::KBYTES + C::VBYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 31, lh = lane >> 5;
  const int N = a.N;
  // the indicator table (read only after the barrier that follows the arrival of K)
  if (tid < 2 * C::HOT_ENTRIES) *reinterpret_cast<u32x4*>(hot + tid * 16) = onehot_x8<T>(tid >> 1, tid & 1);
  // all heads of a window run on one XCD: their 2*HD-byte slices of a token share cache lines
  const unsigned int total = (unsigned int)((a.ws > 0 ? a.B * a.wins_x * a.wins_y : a.B) * a.nH);
  const int bh = (int)xcd_contiguous_id(blockIdx.x, total);
  if ((unsigned int)bh >= total) return;  // uniform over the workgroup
  const int bwin = bh / a.nH, h = bh % a.nH;
  // image-ordered mode: bwin = (image, window row, window column)
  int b = bwin, win_y0 = 0, win_x0 = 0;
  if (a.ws > 0) {
    const int per_img = a.wins_x * a.wins_y;
    b = bwin / per_img;
    const int wi = bwin - b * per_img;
    win_y0 = (wi / a.wins_x) * a.ws;
    win_x0 = (wi % a.wins_x) * a.ws;
  }
  // token n of the window -> row index inside the (b, head) slice, or -1 for a padding token
  // n / gw for 0 <= n < 256 and gw <= 16 by multiplication (exact in that range)
  // (24-bit multiplies: full-rate instructions, and every product here is below 2^24)
  const int gw_magic = 65536 / a.gw + 1;
  auto div_gw = [&](int n) { return (int)(__umul24((unsigned int)n, (unsigned int)gw_magic) >> 16); };
  auto times_gw = [&](int r) { return (int)__umul24((unsigned int)r, (unsigned int)a.gw); };
  auto tok_of = [&](int n) {
    if (a.ws <= 0) return n;
    const int ny = div_gw(n);
    const int y = win_y0 + ny, x = win_x0 + n - times_gw(ny);
    return (y < a.img_h && x < a.img_w) ? y * a.img_w + x : -1;
  };

  const unsigned short* kbase = a.k + b * a.k_sb + h * a.k_sh;
  const unsigned short* vbase = a.v + b * a.v_sb + h * a.v_sh;
  const unsigned short* qbase = a.q + b * a.q_sb + h * a.q_sh;
  const unsigned short* kpad = a.ws > 0 ? a.pad_k + h * HD : kbase;
  const unsigned short* vpad = a.ws > 0 ? a.pad_v + h * HD : vbase;

  const int ntq = (N + 31) / 32;
  const int nsteps = (N + 15) / 16;
  const bool has_tile = wave < ntq;  // uniform per wavefront
  const int qi = 32 * wave + lr;
  const int qc = min(qi, N - 1);

  // ---- requests first: this wavefront's query rows, then the K / V staging loads ----------
  u32x4 qf[C::KS];
  {
    const unsigned short* qp = qbase + (int64_t)max(tok_of(qc), 0) * a.q_sn + 8 * lh;  // padding queries: any row
#pragma unroll
    for (int s = 0; s < C::KS; ++s) qf[s] = load_x8_global(qp + 16 * s);
  }
  // the table rows both bias products need (row min(lr, 2g-2) of rel_pos_h and of rel_pos_w):
  // requested now, so that their latency runs under the K requests below
  u32x4 tfrag[FUSED ? 2 : 1][C::KS];
  if (FUSED && has_tile) {
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      const unsigned short* tab = which ? a.rw : a.rh;
      const int trow = min(lr, 2 * (which ? a.gw : a.gh) - 2);
#pragma unroll
      for (int s = 0; s < C::KS; ++s) tfrag[which][s] = load_x8_global(tab + trow * HD + 16 * s + 8 * lh);
    }
  }
  // wave instruction i of the window fills pieces 64i .. 64i+63: piece P is key P / PPR,
  // 16-byte column P % PPR (spare column and keys >= N: lane masked).  K goes first and travels
  // under the bias prologue; V follows once the scratch in its area is free.
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  // per issued instruction: the lane's token row (-1 padding token, -2 lane masked) and column
  int dma_tok[C::DPW], dma_col[C::DPW];
#pragma unroll
  for (int m = 0; m < C::DPW; ++m) {
    const int P = 64 * (wave_u + C::WAVES * m) + lane;
    const int row = P / C::PPR, col = P % C::PPR;
    dma_col[m] = col * 8;
    dma_tok[m] = (row < N && col < HD / 8) ? tok_of(row) : -2;
  }
  // Token rows and padding rows come from different allocations: one load per source, each with
  // a wave-uniform base and an unsigned 32-bit lane offset (the scalar-base form disturbs the
  // matrix pipe of the co-resident workgroup much less than 64-bit per-lane addresses); the two
  // loads of an instruction slot have complementary lane masks and the same LDS block.
  auto window_dma = [&](const unsigned short* base, int64_t sn, const unsigned short* pad, unsigned char* dst) {
    const unsigned char* tb = reinterpret_cast<const unsigned char*>(base);
    const unsigned char* pb = reinterpret_cast<const unsigned char*>(pad);
    asm volatile("" : "+s"(tb), "+s"(pb));
    const unsigned int sn_bytes = (unsigned int)sn * 2u;
#pragma unroll
    for (int m = 0; m < C::DPW; ++m) {
      const int inst = wave_u + C::WAVES * m;
      if (64 * inst < N * C::PPR) {  // uniform
        if (dma_tok[m] >= 0) {
          unsigned int off = (unsigned int)dma_tok[m] * sn_bytes + (unsigned int)dma_col[m] * 2u;
          asm volatile("" : "+v"(off));
          __builtin_amdgcn_global_load_lds((gptr_t)(tb + off), (lptr_t)(dst + inst * 1024), 16, 0, 0);
        }
        if (dma_tok[m] == -1) {
          unsigned int off = (unsigned int)dma_col[m] * 2u;
          asm volatile("" : "+v"(off));
          __builtin_amdgcn_global_load_lds((gptr_t)(pb + off), (lptr_t)(dst + inst * 1024), 16, 0, 0);
        }
      }
    }
  };
  window_dma(kbase, a.k_sn, kpad, kl);

  // ---- bias operands while the staging loads are in flight: lane (query, lh) element e <->
  //      slot 8*lh + e.  The gather scratch lives where K will be stored afterwards ----------
  u32x4 bias_hv, bias_wv;
  {
    const int qh = div_gw(qc), qw = qc - times_gw(qh);
    unsigned int bhw[4] = {0u, 0u, 0u, 0u}, bww[4] = {0u, 0u, 0u, 0u};
    if (FUSED) {
      unsigned short* X = reinterpret_cast<unsigned short*>(vl + wave * C::XBYTES_WAVE);
#pragma unroll
      for (int which = 0; which < 2; ++which) {
        // T[rel][q] = <table[rel], q> for rel in [0, 32): one MFMA row tile, staged through the
        // wave's scratch rows and read back at rel = qpos - slot + g - 1
        const int g = which ? a.gw : a.gh;
        const int qpos = which ? qw : qh;
        f32x16 tacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) tacc[r] = 0.f;
        if (has_tile) {
#pragma unroll
          for (int s = 0; s < C::KS; ++s) tacc = T::mfma(tfrag[which][s], qf[s], tacc);
        }
#pragma unroll
        // stored in reverse (position 31 - rel), so that the lane's eight slots 8lh .. 8lh+7, which
        // want rel = qpos + g - 1 - slot, are eight consecutive positions E0 .. E0+7
        for (int r = 0; r < 16; r += 2) {  // registers r, r+1 are adjacent rel: one packed 4-byte write
          const int rel = 8 * (r >> 2) + 4 * lh + (r & 3);
          *reinterpret_cast<unsigned int*>(X + lr * C::XSTR + 30 - rel) =
              T::pack2(tacc[r + 1] * a.inv_scale, tacc[r] * a.inv_scale);
        }
        wave_lds_fence();
        {
          const int e0 = 31 - (qpos + g - 1 - 8 * lh);  // 1 <= e0 <= 39 for 1 <= g <= 16
          const unsigned int* xw = reinterpret_cast<const unsigned int*>(X + lr * C::XSTR) + (e0 >> 1);
          unsigned int w[5];
#pragma unroll
          for (int i = 0; i < 5; ++i) w[i] = xw[i];
          const unsigned int sh = (e0 & 1) * 16;  // odd start: shift the pairs down by one element
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const unsigned int pair = __builtin_amdgcn_alignbit(w[i + 1], w[i], sh);
            const int slot = 8 * lh + 2 * i;  // positions past the table (slot >= g) hold no product: zero
            const unsigned int mask = (slot < g ? 0xffffu : 0u) | (slot + 1 < g ? 0xffff0000u : 0u);
            if (which) bww[i] = pair & mask; else bhw[i] = pair & mask;
          }
        }
        wave_lds_fence();
      }
    } else {
      const unsigned short* rhp = a.rh + b * a.rh_sb + h * a.rh_sh + (int64_t)qc * a.rh_sn;
      const unsigned short* rwp = a.rw + b * a.rw_sb + h * a.rw_sh + (int64_t)qc * a.rw_sn;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float fh[2] = {0.f, 0.f}, fw[2] = {0.f, 0.f};
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const int slot = 8 * lh + 2 * i + v;
          const float rh_raw = T::from_bits(rhp[min(slot, a.gh - 1)]) * a.inv_scale;
          const float rw_raw = T::from_bits(rwp[min(slot, a.gw - 1)]) * a.inv_scale;
          fh[v] = (slot < a.gh) ? rh_raw : 0.f;
          fw[v] = (slot < a.gw) ? rw_raw : 0.f;
        }
        bhw[i] = T::pack2(fh[0], fh[1]);
        bww[i] = T::pack2(fw[0], fw[1]);
      }
    }
    if (lh == 1) bhw[3] = (bhw[3] & 0xffffu) | (T::kMask << 16);  // slot 15: the masking value
    const u32x4 bhv = {bhw[0], bhw[1], bhw[2], bhw[3]};
    const u32x4 bwv = {bww[0], bww[1], bww[2], bww[3]};
    bias_hv = bhv;
    bias_wv = bwv;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's share of K has landed
  __syncthreads();  // K complete; every wavefront is done with the scratch: V may overwrite it
  window_dma(vbase, a.v_sn, vpad, vl);
  // V rows past the last key, up to the 16-key step boundary, are multiplied by P = 0: zeros
  for (int idx = tid; idx < (16 * nsteps - N) * (HD / 8); idx += C::THREADS) {
    const int row = N + idx / (HD / 8), col = idx % (HD / 8);
    const u32x4 z = {0u, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(vl + (row * C::VSTR + col * 8) * 2) = z;
  }
  if (C::ONES_ROW && tid < 16 * nsteps) {  // the ones channel (P = 0 beyond the last key anyway)
    const u32x4 one = {T::kOne, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(vl + (tid * C::VSTR + HD) * 2) = one;
  }
  if (!has_tile) {  // a wavefront without a query tile only helps with the staging and with the output
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // V complete (the barrier the others reach after their first score tile)
  }

  if (has_tile) {
    // V^T operand through transposing LDS reads (ds_read_b64_tr_b16): in each group of 16 lanes,
    // lane l receives as element j the l%4-th 16-bit value of the 8 bytes addressed by lane
    // 4j + l/4.  Source lane 4j + i points at key j of the lane half's four keys, channels
    // 4i .. 4i+3 of the group's 16 channels; lane l ends up with channel l of four keys.
    int vrd[C::DT];
    {
      const int g = lane >> 4, sl = lane & 15;
      const int key = 4 * (g >> 1) + (sl >> 2);
#pragma unroll
      for (int dt = 0; dt < C::DT; ++dt) {
        int d = 32 * dt + 16 * (g & 1) + 4 * (sl & 3);
        if (C::ONES_ROW) d = d >= HD + 8 ? HD + 4 : d;  // past the spare piece (1, 0, .., 0): its zero half
        else d = min(d, HD - 4);
        vrd[dt] = (key * C::VSTR + d) * 2;
      }
    }
    auto vt_frag = [&](int dt, int j) {
      typedef short s16x4 __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) s16x4* trptr_t;
      const unsigned char* p = vl + vrd[dt] + 16 * j * C::VSTR * 2;
      const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((trptr_t)p));
      const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((trptr_t)(p + 8 * C::VSTR * 2)));
      const u32x4 w = {lo[0], lo[1], hi[0], hi[1]};
      return w;
    };

    const u32x4 bh_op = bias_hv, bw_op = bias_wv;

    // ---- online softmax over the key tiles: S^T tile, running max, P, O^T += V^T P^T --------
    f32x16 oacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
    float m_run = -3.0e38f, l_run = 0.f;
#pragma unroll
    for (int nt = 0; nt < C::NT; ++nt) {
      if (32 * nt < N) {  // uniform
        const int n = 32 * nt + lr;
        // A key tile that lies inside the window whole (all but the last one: 6 of 7 at 196 keys)
        // needs neither the clamp of its K rows nor the selects of the padding mask; its K
        // addresses are then the lane's tile-0 address plus a constant.
        auto score_tile = [&](auto whole_c) {
          constexpr bool WHOLE = decltype(whole_c)::value;
          const int nc = WHOLE ? n : min(n, N - 1);
          f32x16 sacc;
#pragma unroll
          for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
          for (int ks = 0; ks < C::KS; ++ks) {
            const u32x4 av = *reinterpret_cast<const u32x4*>(kl + (nc * C::KSTR + 16 * ks + 8 * lh) * 2);
            sacc = T::mfma(av, qf[ks], sacc);
          }
          const int nh = div_gw(WHOLE ? n : min(n, 255));
          const bool real = WHOLE || n < N;
          // slot 15 of the row part is the padding mask; a padding key has no column
          const u32x4 ih = *reinterpret_cast<const u32x4*>(hot + (real ? nh : 15) * 32 + lh * 16);
          const u32x4 iw = *reinterpret_cast<const u32x4*>(hot + (real ? n - times_gw(nh) : 16) * 32 + lh * 16);
          sacc = T::mfma(ih, bh_op, sacc);
          return T::mfma(iw, bw_op, sacc);
        };
        f32x16 acc;
        if (32 * nt + 32 <= N) acc = score_tile(std::true_type{});  // uniform
        else acc = score_tile(std::false_type{});

        float mx = acc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(mx, acc[r]);
        mx = max_with_lane_xor32(mx);
        // lazy reference (see the global kernel): m_run follows the maximum in steps > 2^kLazyLog2
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.0f;
        const bool move = __any((m_new - m_run) * a.c > kLazyLog2);  // uniform; first tile: always
        if (move) {
          alpha = fast_exp2((m_run - m_new) * a.c);
          m_run = m_new;
        }
        const float neg_m = -m_run * a.c;
        float lsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fast_exp2(fmaf(acc[r], a.c, neg_m));
          acc[r] = p;
          if (!C::ONES_ROW) lsum += p;
        }
        if (!C::ONES_ROW) l_run = l_run * alpha + lsum;
        if (nt == 0) {  // V travelled under the first score tile; every wavefront's share has landed
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __syncthreads();
        } else if (move) {
#pragma unroll
          for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int j = 2 * nt + half;
          if (j < nsteps) {  // uniform
            const u32x4 pk = cvt_x8<T>(acc, 8 * half);
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt) {
              oacc[dt] = T::mfma(vt_frag(dt, j), pk, oacc[dt]);
            }
          }
        }
      }
    }
    float l;
    if (C::ONES_ROW) {
      // output row HD = tile DT-1, row HD % 32, held by the lh = (HD % 32) / 4 % 2 lanes
      constexpr int orow = HD % 32;
      constexpr int oreg = 4 * (orow / 8) + orow % 4, olh = (orow / 4) % 2;
      const float own = oacc[C::DT - 1][oreg];
      const float other = xor32(own);
      l = (lh == olh) ? own : other;
    } else {
      l = l_run + xor32(l_run);
    }
    const float inv = 1.0f / l;
    // ---- output: through LDS, so that a token's HD channels leave as one contiguous run ----------
    // Written straight from the accumulators a lane would store 8 bytes to each of 32 different
    // token rows per instruction; staged as (token, channel) rows in the K area - free once every
    // wavefront has left its key loop - the whole workgroup then writes 16 bytes per lane with the
    // HD/8 pieces of a token in neighbouring lanes.
    __syncthreads();
    if (qi < N) {
      unsigned char* orow_l = kl + qi * (C::KSTR * 2);
#pragma unroll
      for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int d = 32 * dt + 8 * j + 4 * lh;
          if (d < HD) {
            const u32x2 o = {T::pack2(oacc[dt][4 * j] * inv, oacc[dt][4 * j + 1] * inv),
                             T::pack2(oacc[dt][4 * j + 2] * inv, oacc[dt][4 * j + 3] * inv)};
            *reinterpret_cast<u32x2*>(orow_l + d * 2) = o;
          }
        }
    }
  } else {
    __syncthreads();  // the key loops are over: the K area becomes the output staging area
  }
  __syncthreads();    // the staged output is complete
  {
    constexpr int PPT = HD / 8;  // 16-byte pieces per token
    unsigned short* obase = a.out + b * a.o_sb + h * a.o_sh;
    for (int p = tid; p < N * PPT; p += C::THREADS) {
      const int n = (p * (65536 / PPT + 1)) >> 16;  // p / PPT, exact for p < 4096
      const int col = p - n * PPT;
      const int otok = tok_of(n);  // padding tokens produce no output
      if (otok >= 0) {
        const u32x4 o = *reinterpret_cast<const u32x4*>(kl + n * (C::KSTR * 2) + col * 16);
        *reinterpret_cast<u32x4*>(obase + (int64_t)otok * a.o_sn + col * 8) = o;
      }
    }
  }
}

// =============================================================================
// host side
// =============================================================================
template <typename T, int HD, bool FUSED>
static int launch_hd(const AttnArgs& a, bool global_path, hipStream_t stream) {
  if (global_path) {
    constexpr int QT = 1;
    auto launch = [&](auto wc) {
      constexpr int WAVES = decltype(wc)::value;
      using C = GlobalCfg<HD, QT, WAVES>;
      const int64_t total = (int64_t)a.B * a.nH * (a.N / C::BM);
      const unsigned int grid = (unsigned int)(((total + 7) / 8) * 8);
      hipLaunchKernelGGL((attn_global_kernel<T, HD, QT, FUSED, WAVES>), dim3(grid), dim3(64 * WAVES), 0, stream, a);
    };
    // 256 queries per workgroup when that still gives every CU several workgroups
    // (SAMFAST_ATTN_WAVES=4 / 8 overrides the choice where the shape allows it)
    const int64_t wg8 = (int64_t)a.B * a.nH * (a.N / 256);
    const int force = knob(KNOB_ATTN_WAVES);
    const bool want8 = force != kKnobUnset ? force == 8 : wg8 >= 1024;
    if (a.N % 256 == 0 && want8) launch(std::integral_constant<int, 8>{});
    else launch(std::integral_constant<int, 4>{});
    return check_launch("attn_global_kernel");
  }
  const int64_t wins = a.ws > 0 ? (int64_t)a.B * a.wins_x * a.wins_y : a.B;
  const unsigned int grid = (unsigned int)(((wins * a.nH + 7) / 8) * 8);
  hipLaunchKernelGGL((attn_window_kernel<T, HD, FUSED>), dim3(grid), dim3(WindowCfg<HD>::THREADS), 0, stream, a);
  return check_launch("attn_window_kernel");
}

static int attn_dispatch(bool fused, AttnArgs& a, int hd, int dtype, float sm_scale,
                         hipStream_t stream) {
  SF_REQUIRE(a.B >= 0 && a.nH > 0 && a.gh > 0 && a.gw > 0, "attn_relpos: bad shape");
  SF_REQUIRE(sm_scale > 0.f, "attn_relpos: sm_scale must be positive");
  // an empty batch is a valid call that does nothing (its buffers may be null)
  SF_REQUIRE(a.B == 0 || (a.q && a.k && a.v && a.out && a.rh && a.rw), "attn_relpos: null pointer");
  if (dtype != SAMFAST_BF16 && dtype != SAMFAST_F16)
    SF_FAIL(SAMFAST_E_UNSUPPORTED, "attn_relpos: element type %d is neither SAMFAST_BF16 nor SAMFAST_F16", dtype);
  if (hd != 64 && hd != 80)
    SF_FAIL(SAMFAST_E_UNSUPPORTED, "attn_relpos: head_dim %d not in {64, 80}", hd);
  SF_REQUIRE((int64_t)a.B * a.nH < (1ll << 24), "attn_relpos: B*nH too large");
  if (a.ws > 0) {
    SF_REQUIRE(fused && a.gh == a.ws && a.gw == a.ws && a.img_h > 0 && a.img_w > 0 && a.pad_k && a.pad_v &&
                   aligned16(a.pad_k) && aligned16(a.pad_v),
               "attn_relpos_windowed: bad window geometry or padding rows");
    a.wins_y = (a.img_h + a.ws - 1) / a.ws;
    a.wins_x = (a.img_w + a.ws - 1) / a.ws;
    SF_REQUIRE((int64_t)a.B * a.wins_x * a.wins_y * a.nH < (1ll << 30), "attn_relpos_windowed: too many windows");
  }
  a.N = a.gh * a.gw;
  const bool global_path = a.ws <= 0 && (a.gw == 64) && (a.N % 128 == 0) && (a.gh <= 64);
  const bool window_path = (a.gh <= 15) && (a.gw <= 16) && (a.N <= 208);
  if (!global_path && !window_path)
    SF_FAIL(SAMFAST_E_UNSUPPORTED,
            "attn_relpos: grid %dx%d is neither 64-wide (rows even, <= 64) nor a window of <= 15x16",
            a.gh, a.gw);
  // every row start 16-byte aligned: strides multiples of 8 elements
  const int64_t st[12] = {a.q_sb, a.q_sh, a.q_sn, a.k_sb, a.k_sh, a.k_sn,
                          a.v_sb, a.v_sh, a.v_sn, a.o_sb, a.o_sh, a.o_sn};
  for (int i = 0; i < 12; ++i)
    SF_REQUIRE(st[i] >= 0 && st[i] % 8 == 0, "attn_relpos: stride %d = %lld is not a multiple of 8",
               i, (long long)st[i]);
  SF_REQUIRE(aligned16(a.q) && aligned16(a.k) && aligned16(a.v) && aligned16(a.out),
             "attn_relpos: q/k/v/out must be 16-byte aligned");
  SF_REQUIRE(a.q_sn >= hd && a.k_sn >= hd && a.v_sn >= hd && a.o_sn >= hd,
             "attn_relpos: token stride smaller than head_dim");
  if (!global_path) {  // byte offsets of a token row inside its (batch, head) slice are kept in 32 bits
    const int64_t toks = a.ws > 0 ? (int64_t)a.img_h * a.img_w : a.N;
    SF_REQUIRE(toks * a.k_sn * 2 < (1ll << 32) && toks * a.v_sn * 2 < (1ll << 32),
               "attn_relpos: k / v token stride too large for %lld tokens", (long long)toks);
  }
  if (global_path)  // tile-relative element offsets are kept in 32 bits
    SF_REQUIRE(a.k_sn < (1 << 24) && a.v_sn < (1 << 24), "attn_relpos: k / v token stride too large");
  if (fused) {
    SF_REQUIRE(aligned16(a.rh) && aligned16(a.rw), "attn_relpos: tables must be 16-byte aligned");
  } else if (global_path) {
    SF_REQUIRE((reinterpret_cast<uintptr_t>(a.rw) & 7u) == 0 && a.rw_sb % 4 == 0 &&
                   a.rw_sh % 4 == 0 && a.rw_sn % 4 == 0,
               "attn_relpos: rel_w rows must be 8-byte aligned");
  }
  if (a.B == 0) return SAMFAST_OK;
  a.c = sm_scale * kLog2e;
  a.inv_scale = 1.0f / sm_scale;
  // windows whose rows fit the padded-row key layout take that kernel (attn_window_rows.hip)
  if (!global_path && attn_window_rows_covers(a)) return attn_window_rows_launch(a, hd, dtype, fused, stream);
  auto by_type = [&](auto elem) {
    using T = decltype(elem);
    if (hd == 64)
      return fused ? launch_hd<T, 64, true>(a, global_path, stream) : launch_hd<T, 64, false>(a, global_path, stream);
    return fused ? launch_hd<T, 80, true>(a, global_path, stream) : launch_hd<T, 80, false>(a, global_path, stream);
  };
  return dtype == SAMFAST_F16 ? by_type(ElemF16{}) : by_type(ElemBf16{});
}

}  // namespace samfast

extern "C" int samfast_attn_relpos_fwd(
    const void* q, const void* k, const void* v, const void* rel_pos_h, const void* rel_pos_w,
    void* out, int B, int nH, int gh, int gw, int hd,
    int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn,
    int64_t v_sb, int64_t v_sh, int64_t v_sn, int64_t o_sb, int64_t o_sh, int64_t o_sn,
    int dtype, float sm_scale, void* stream) {
  using us = unsigned short;
  samfast::AttnArgs a = {};
  a.q = (const us*)q; a.k = (const us*)k; a.v = (const us*)v;
  a.rh = (const us*)rel_pos_h; a.rw = (const us*)rel_pos_w; a.out = (us*)out;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn; a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.B = B; a.nH = nH; a.gh = gh; a.gw = gw;
  return samfast::attn_dispatch(true, a, hd, dtype, sm_scale, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_attn_relpos_bias_fwd(
    const void* q, const void* k, const void* v, const void* rel_h, const void* rel_w, void* out,
    int B, int nH, int gh, int gw, int hd,
    int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn,
    int64_t v_sb, int64_t v_sh, int64_t v_sn, int64_t o_sb, int64_t o_sh, int64_t o_sn,
    int64_t rh_sb, int64_t rh_sh, int64_t rh_sn, int64_t rw_sb, int64_t rw_sh, int64_t rw_sn,
    int dtype, float sm_scale, void* stream) {
  using us = unsigned short;
  samfast::AttnArgs a = {};
  a.q = (const us*)q; a.k = (const us*)k; a.v = (const us*)v;
  a.rh = (const us*)rel_h; a.rw = (const us*)rel_w; a.out = (us*)out;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn; a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.rh_sb = rh_sb; a.rh_sh = rh_sh; a.rh_sn = rh_sn;
  a.rw_sb = rw_sb; a.rw_sh = rw_sh; a.rw_sn = rw_sn;
  a.B = B; a.nH = nH; a.gh = gh; a.gw = gw;
  SF_REQUIRE(rh_sb >= 0 && rh_sh >= 0 && rh_sn >= 0 && rw_sb >= 0 && rw_sh >= 0 && rw_sn >= 0,
             "attn_relpos_bias: negative bias stride");
  return samfast::attn_dispatch(false, a, hd, dtype, sm_scale, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_attn_relpos_windowed_fwd(
    const void* q, const void* k, const void* v, const void* rel_pos_h, const void* rel_pos_w,
    const void* pad_k, const void* pad_v, void* out,
    int B, int nH, int img_h, int img_w, int ws, int hd,
    int64_t q_sb, int64_t q_sh, int64_t q_sn, int64_t k_sb, int64_t k_sh, int64_t k_sn,
    int64_t v_sb, int64_t v_sh, int64_t v_sn, int64_t o_sb, int64_t o_sh, int64_t o_sn,
    int dtype, float sm_scale, void* stream) {
  using us = unsigned short;
  samfast::AttnArgs a = {};
  if (ws <= 0) {
    samfast::set_error("attn_relpos_windowed: window size must be positive");
    return SAMFAST_E_INVALID;
  }
  a.q = (const us*)q; a.k = (const us*)k; a.v = (const us*)v;
  a.rh = (const us*)rel_pos_h; a.rw = (const us*)rel_pos_w; a.out = (us*)out;
  a.pad_k = (const us*)pad_k; a.pad_v = (const us*)pad_v;
  a.q_sb = q_sb; a.q_sh = q_sh; a.q_sn = q_sn; a.k_sb = k_sb; a.k_sh = k_sh; a.k_sn = k_sn;
  a.v_sb = v_sb; a.v_sh = v_sh; a.v_sn = v_sn; a.o_sb = o_sb; a.o_sh = o_sh; a.o_sn = o_sn;
  a.B = B; a.nH = nH; a.gh = ws; a.gw = ws; a.img_h = img_h; a.img_w = img_w; a.ws = ws;
  return samfast::attn_dispatch(true, a, hd, dtype, sm_scale, reinterpret_cast<hipStream_t>(stream));
}
