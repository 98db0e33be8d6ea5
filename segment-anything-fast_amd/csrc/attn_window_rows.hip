// Window attention with decomposed relative-position bias, keys laid out as grid rows padded to 16.
//
// One 512-thread workgroup per (window, head), K and V of the whole window in LDS, eight
// wavefronts of which wavefront w owns query tile w (32 queries), online softmax over key tiles of
// 32 - the structure of attn_window_kernel (attn_relpos.hip).  What differs is where a key sits:
// key (kh, kw) of the gh x gw window is LDS row 16*kh + kw, so a key tile of 32 rows is exactly two
// grid rows (columns gw .. 15 are padding rows: zeros in LDS, masked in the scores).  In the
// S^T = K Q^T accumulator a lane owns one query and, per tile, the same 8 key columns twice
// (registers 0-7: grid row 2t, registers 8-15: grid row 2t + 1).  Therefore
//   * rel_w[q, kw] is the same for every key tile: it enters through ONE extra k-step of the score
//     MFMA whose A operand - the one-hot vector of the row's column - is a constant of the lane (no
//     indicator table, no per-tile index arithmetic); its padding columns carry the mask value;
//   * rel_h[q, kh] is one scalar per (query, grid row): it goes into the exponent's addend, two
//     values per tile, kept as 16-bit pairs (tile t <-> pair t);
//   * every key tile is whole: no clamped rows, no tail variant, no per-key masks.
// Against the token-ordered kernel that is one matrix instruction and two 16-byte LDS reads fewer per
// key tile and about a fifth fewer vector instructions in the key loop; LDS grows from 208 to 224
// rows per operand (78 848 B at head_dim 80: still two workgroups per CU).
//
// Covers gw <= 16 and gh <= 14 (7 key tiles).  Selected by SAMFAST_ATTN_WINDOW_ROWS=1; the default
// is attn_window_kernel, which measures 3 % faster inside the encoder.
#include "attn_relpos_shared.hpp"

namespace samfast {

template <int HD>
struct RowsCfg {
  static constexpr int KS = HD / 16;
  static constexpr int DT = (HD + 31) / 32;
  static constexpr int NT = 7;                 // key tiles of two grid rows
  static constexpr int SLOTS = 32 * NT;        // LDS rows per operand
  static constexpr int WAVES = 8;
  static constexpr int THREADS = 64 * WAVES;
  static constexpr int PPR = HD / 8 + 1;       // 16-byte pieces per staged row: data + one spare
  static constexpr int KSTR = PPR * 8;
  static constexpr int VSTR = PPR * 8;
  static constexpr int KBYTES = SLOTS * KSTR * 2;
  static constexpr int VBYTES = SLOTS * VSTR * 2;
  static constexpr int NDMA = (SLOTS * PPR + 63) / 64;       // wave instructions per K (or V) window
  static constexpr int DPW = (NDMA + WAVES - 1) / WAVES;     // of which each wavefront issues at most
  static constexpr bool ONES_ROW = HD % 32 != 0;             // spare piece of V = (1, 0, ..): row HD of O^T is the denominator
  static constexpr int XSTR = 50;              // scratch row: 32 products stored in reverse + read-ahead room (25 words: odd)
  static constexpr int XBYTES_WAVE = 32 * XSTR * 2;
  static constexpr int LDS_BYTES = KBYTES + VBYTES;
  static_assert(WAVES * XBYTES_WAVE <= VBYTES, "gather scratch must fit in the V area");
  static_assert(LDS_BYTES <= 80 * 1024, "two workgroups per CU");
};

template <typename T, int HD, bool FUSED>
__global__ __launch_bounds__(RowsCfg<HD>::THREADS, 2) void attn_window_rows_kernel(AttnArgs a) {
  using C = RowsCfg<HD>;
  __shared__ __attribute__((aligned(16))) unsigned char lds[C::LDS_BYTES];
  unsigned char* kl = lds;
  unsigned char* vl = lds + C::KBYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 31, lh = lane >> 5;
  const int N = a.N;
  // all heads of a window run on one XCD: their 2*HD-byte slices of a token share cache lines
  const unsigned int total = (unsigned int)((a.ws > 0 ? a.B * a.wins_x * a.wins_y : a.B) * a.nH);
  const int bh = (int)xcd_contiguous_id(blockIdx.x, total);
  if ((unsigned int)bh >= total) return;  // uniform over the workgroup
  const int bwin = bh / a.nH, h = bh % a.nH;
  int b = bwin, win_y0 = 0, win_x0 = 0;
  if (a.ws > 0) {  // image-ordered mode: bwin = (image, window row, window column)
    const int per_img = a.wins_x * a.wins_y;
    b = bwin / per_img;
    const int wi = bwin - b * per_img;
    win_y0 = (wi / a.wins_x) * a.ws;
    win_x0 = (wi % a.wins_x) * a.ws;
  }
  // (24-bit multiplies: full-rate instructions, and every product here is below 2^24)
  const int gw_magic = 65536 / a.gw + 1;  // n / gw for 0 <= n < 256, gw <= 16, by multiplication
  auto div_gw = [&](int n) { return (int)(__umul24((unsigned int)n, (unsigned int)gw_magic) >> 16); };
  auto times_gw = [&](int r) { return (int)__umul24((unsigned int)r, (unsigned int)a.gw); };
  // window position (y, x) -> row index inside the (b, head) slice, or -1 for a padding token of the image border
  auto tok_at = [&](int y, int x) {
    if (a.ws <= 0) return times_gw(y) + x;
    const int iy = win_y0 + y, ix = win_x0 + x;
    return (iy < a.img_h && ix < a.img_w) ? iy * a.img_w + ix : -1;
  };

  const unsigned short* kbase = a.k + b * a.k_sb + h * a.k_sh;
  const unsigned short* vbase = a.v + b * a.v_sb + h * a.v_sh;
  const unsigned short* qbase = a.q + b * a.q_sb + h * a.q_sh;
  const unsigned short* kpad = a.ws > 0 ? a.pad_k + h * HD : kbase;
  const unsigned short* vpad = a.ws > 0 ? a.pad_v + h * HD : vbase;

  const int ntq = (N + 31) / 32;
  const int ntk = (a.gh + 1) >> 1;   // key tiles in use
  const bool has_tile = wave < ntq;  // uniform per wavefront
  const int qi = 32 * wave + lr;
  const int qc = min(qi, N - 1);
  const int qh = div_gw(qc), qw = qc - times_gw(qh);

  // ---- requests first: this wavefront's query rows, then the K / V staging loads ----------
  u32x4 qf[C::KS];
  {
    const unsigned short* qp = qbase + (int64_t)max(tok_at(qh, qw), 0) * a.q_sn + 8 * lh;  // padding queries: any row
#pragma unroll
    for (int s = 0; s < C::KS; ++s) qf[s] = load_x8_global(qp + 16 * s);
  }
  // the table rows both bias products need (row min(lr, 2g-2) of rel_pos_h and of rel_pos_w)
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
  // Wave instruction i of the window fills pieces 64i .. 64i+63: piece P is LDS row P / PPR, 16-byte
  // column P % PPR.  Per issued instruction the lane's source: a token row (>= 0), the padding
  // token's row (-1), nothing (-2: the spare column), or zeros to be written by the lane itself
  // (-3: a data piece of a padding row of the layout, kw >= gw or kh >= gh).
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  int dma_tok[C::DPW], dma_col[C::DPW];
#pragma unroll
  for (int m = 0; m < C::DPW; ++m) {
    const int P = 64 * (wave_u + C::WAVES * m) + lane;
    const int row = P / C::PPR, col = P % C::PPR;
    const int kh = row >> 4, kw = row & 15;
    dma_col[m] = col * 8;
    int src = -2;
    if (row < 32 * ntk && col < HD / 8) src = (kh < a.gh && kw < a.gw) ? tok_at(kh, kw) : -3;
    dma_tok[m] = src;
  }
  // Token rows and padding-token rows come from different allocations: one load per source, each
  // with a wave-uniform base and an unsigned 32-bit lane offset; the two loads of an instruction
  // slot have complementary lane masks and the same LDS block.  The layout's padding rows are
  // written as zeros by their lanes (their products must be finite: they are masked, not skipped).
  auto window_dma = [&](const unsigned short* base, int64_t sn, const unsigned short* pad, unsigned char* dst, int str) {
    const unsigned char* tb = reinterpret_cast<const unsigned char*>(base);
    const unsigned char* pb = reinterpret_cast<const unsigned char*>(pad);
    asm volatile("" : "+s"(tb), "+s"(pb));
    const unsigned int sn_bytes = (unsigned int)sn * 2u;
#pragma unroll
    for (int m = 0; m < C::DPW; ++m) {
      const int inst = wave_u + C::WAVES * m;
      if (64 * inst < 32 * ntk * C::PPR) {  // uniform
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
        if (dma_tok[m] == -3) {
          const int P = 64 * inst + lane;
          const u32x4 z = {0u, 0u, 0u, 0u};
          *reinterpret_cast<u32x4*>(dst + ((P / C::PPR) * str + dma_col[m]) * 2) = z;
        }
      }
    }
  };
  window_dma(kbase, a.k_sn, kpad, kl, C::KSTR);

  // ---- bias while the staging loads are in flight ---------------------------------------------
  // bw_op: B operand of the rel_w k-step: element e of the lane's half <-> column 8*lh + e, value
  //        rel_w[q, col] / sm_scale, the mask value for col >= gw.
  // relh_pk[t]: (rel_h[q, 2t], rel_h[q, 2t+1]) * log2(e) as a 16-bit pair; rows >= gh: the mask value.
  u32x4 bw_op;
  unsigned int relh_pk[8];
  {
    unsigned int bww[4] = {0u, 0u, 0u, 0u};
    if (FUSED) {
      unsigned short* X = reinterpret_cast<unsigned short*>(vl + wave * C::XBYTES_WAVE);
#pragma unroll
      for (int which = 0; which < 2; ++which) {
        // T[rel][q] = <table[rel], q> for rel in [0, 32): one MFMA row tile, staged through the
        // wave's scratch rows (in reverse: position 31 - rel) and read back at rel = qpos - slot + g - 1,
        // i.e. at consecutive positions E0 + slot
        const int g = which ? a.gw : a.gh;
        const int qpos = which ? qw : qh;
        const float factor = which ? a.inv_scale : kLog2e;
        f32x16 tacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) tacc[r] = 0.f;
        if (has_tile) {
#pragma unroll
          for (int s = 0; s < C::KS; ++s) tacc = T::mfma(tfrag[which][s], qf[s], tacc);
        }
#pragma unroll
        for (int r = 0; r < 16; r += 2) {  // registers r, r+1 are adjacent rel: one packed 4-byte write
          const int rel = 8 * (r >> 2) + 4 * lh + (r & 3);
          *reinterpret_cast<unsigned int*>(X + lr * C::XSTR + 30 - rel) = T::pack2(tacc[r + 1] * factor, tacc[r] * factor);
        }
        wave_lds_fence();
        if (which) {
          // the lane's eight columns 8*lh .. 8*lh + 7
          const int e0 = 31 - (qpos + g - 1 - 8 * lh);  // 1 <= e0 <= 39
          const unsigned int* xw = reinterpret_cast<const unsigned int*>(X + lr * C::XSTR) + (e0 >> 1);
          unsigned int w[5];
#pragma unroll
          for (int i = 0; i < 5; ++i) w[i] = xw[i];
          const unsigned int sh = (e0 & 1) * 16;  // odd start: shift the pairs down by one element
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const unsigned int pair = __builtin_amdgcn_alignbit(w[i + 1], w[i], sh);
            const int slot = 8 * lh + 2 * i;
            const unsigned int lo = slot < g ? (pair & 0xffffu) : T::kMask;
            const unsigned int hi = slot + 1 < g ? (pair & 0xffff0000u) : (T::kMask << 16);
            bww[i] = lo | hi;
          }
        } else {
          // all sixteen rows 0 .. 15 (both lane halves need every row)
          const int e0 = 31 - (qpos + g - 1);  // 1 <= e0 <= 31
          const unsigned int* xw = reinterpret_cast<const unsigned int*>(X + lr * C::XSTR) + (e0 >> 1);
          unsigned int w[9];
#pragma unroll
          for (int i = 0; i < 9; ++i) w[i] = xw[i];
          const unsigned int sh = (e0 & 1) * 16;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const unsigned int pair = __builtin_amdgcn_alignbit(w[i + 1], w[i], sh);
            const int slot = 2 * i;
            const unsigned int lo = slot < g ? (pair & 0xffffu) : T::kMask;
            const unsigned int hi = slot + 1 < g ? (pair & 0xffff0000u) : (T::kMask << 16);
            relh_pk[i] = lo | hi;
          }
        }
        wave_lds_fence();
      }
    } else {
      const unsigned short* rhp = a.rh + b * a.rh_sb + h * a.rh_sh + (int64_t)qc * a.rh_sn;
      const unsigned short* rwp = a.rw + b * a.rw_sb + h * a.rw_sh + (int64_t)qc * a.rw_sn;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        unsigned int pr[2];
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const int slot = 8 * lh + 2 * i + v;
          const float raw = T::from_bits(rwp[min(slot, a.gw - 1)]) * a.inv_scale;
          pr[v] = slot < a.gw ? (T::pack2(raw, 0.f) & 0xffffu) : T::kMask;
        }
        bww[i] = pr[0] | (pr[1] << 16);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        unsigned int pr[2];
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const int slot = 2 * i + v;
          const float raw = T::from_bits(rhp[min(slot, a.gh - 1)]) * kLog2e;
          pr[v] = slot < a.gh ? (T::pack2(raw, 0.f) & 0xffffu) : T::kMask;
        }
        relh_pk[i] = pr[0] | (pr[1] << 16);
      }
    }
    const u32x4 bwv = {bww[0], bww[1], bww[2], bww[3]};
    bw_op = bwv;
  }
  // A operand of the rel_w k-step: LDS row lr of every key tile is column lr % 16
  const u32x4 iw_op = onehot_x8<T>(lr & 15, lh);

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's share of K has landed
  __syncthreads();  // K complete; every wavefront is done with the scratch: V may overwrite it
  window_dma(vbase, a.v_sn, vpad, vl, C::VSTR);
  if (C::ONES_ROW && tid < 32 * ntk) {  // the ones channel of every row (padding rows are multiplied by P = 0)
    const u32x4 one = {T::kOne, 0u, 0u, 0u};
    *reinterpret_cast<u32x4*>(vl + (tid * C::VSTR + HD) * 2) = one;
  }
  if (!has_tile) {  // a wavefront without a query tile only helps with the staging and with the output
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();  // V complete (the barrier the others reach after their first score tile)
  }

  if (has_tile) {
    // V^T operand through transposing LDS reads (ds_read_b64_tr_b16), as in attn_window_kernel
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

    // ---- online softmax over the key tiles: S^T tile, running max, P, O^T += V^T P^T --------
    f32x16 oacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;
    float m_run = -3.0e38f, l_run = 0.f;  // m_run in exponent (log2) units
    const unsigned char* krow = kl + (lr * C::KSTR + 8 * lh) * 2;
#pragma unroll
    for (int nt = 0; nt < C::NT; ++nt) {
      if (nt < ntk) {  // uniform
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < C::KS; ++ks) {
          const u32x4 av = *reinterpret_cast<const u32x4*>(krow + (32 * nt * C::KSTR + 16 * ks) * 2);
          acc = T::mfma(av, qf[ks], acc);
        }
        acc = T::mfma(iw_op, bw_op, acc);  // + rel_w[q, column] / sm_scale (padding columns: the mask value)

        // the two grid rows of the tile: registers 0-7 and 8-15
        const float b0a = T::lo(relh_pk[nt]), b0b = T::hi(relh_pk[nt]);
        float mxa = acc[0], mxb = acc[8];
#pragma unroll
        for (int r = 1; r < 8; ++r) {
          mxa = fmaxf(mxa, acc[r]);
          mxb = fmaxf(mxb, acc[8 + r]);
        }
        const float mx = max_with_lane_xor32(fmaxf(fmaf(mxa, a.c, b0a), fmaf(mxb, a.c, b0b)));
        // lazy reference (see the global kernel): m_run follows the maximum in steps > 2^kLazyLog2
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.0f;
        const bool move = __any(m_new - m_run > kLazyLog2);  // uniform; first tile: always
        if (move) {
          alpha = fast_exp2(m_run - m_new);
          m_run = m_new;
        }
        const float na = b0a - m_run, nb = b0b - m_run;
        float lsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = fast_exp2(fmaf(acc[r], a.c, r < 8 ? na : nb));
          acc[r] = p;
          if (!C::ONES_ROW) lsum += p;
        }
        if (!C::ONES_ROW) l_run = l_run * alpha + lsum;
        if (nt == 0) {  // V travelled under the first score tile; every wavefront's share has landed
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          __syncthreads();
        } else if (move) {
#pragma unroll
          for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const u32x4 pk = cvt_x8<T>(acc, 8 * half);
#pragma unroll
          for (int dt = 0; dt < C::DT; ++dt) oacc[dt] = T::mfma(vt_frag(dt, 2 * nt + half), pk, oacc[dt]);
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
    // ---- output: staged as (token, channel) rows in the K area (free once every wavefront has left
    //      its key loop), then written by the whole workgroup 16 bytes per lane ------------------
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
      const int ny = div_gw(n);
      const int otok = tok_at(ny, n - times_gw(ny));  // padding tokens produce no output
      if (otok >= 0) {
        const u32x4 o = *reinterpret_cast<const u32x4*>(kl + n * (C::KSTR * 2) + col * 16);
        *reinterpret_cast<u32x4*>(obase + (int64_t)otok * a.o_sn + col * 8) = o;
      }
    }
  }
}

bool attn_window_rows_covers(const AttnArgs& a) {
  // measured inside the ViT-H batch-16 encoder: 215 us per launch against 209 for the token-ordered kernel
  // (fewer vector and matrix instructions, but 14 % more LDS rows to fill and one more P V step), so it
  // runs only when asked for
  return knob_or(KNOB_ATTN_WINDOW_ROWS, 0) != 0 && a.gw <= 16 && a.gh <= 2 * RowsCfg<80>::NT;
}

template <typename T, int HD, bool FUSED>
static int launch_rows(const AttnArgs& a, hipStream_t stream) {
  const int64_t wins = a.ws > 0 ? (int64_t)a.B * a.wins_x * a.wins_y : a.B;
  const unsigned int grid = (unsigned int)(((wins * a.nH + 7) / 8) * 8);
  hipLaunchKernelGGL((attn_window_rows_kernel<T, HD, FUSED>), dim3(grid), dim3(RowsCfg<HD>::THREADS), 0, stream, a);
  return check_launch("attn_window_rows_kernel");
}

int attn_window_rows_launch(const AttnArgs& a, int hd, int dtype, bool fused, hipStream_t stream) {
  auto by_type = [&](auto elem) {
    using T = decltype(elem);
    if (hd == 64) return fused ? launch_rows<T, 64, true>(a, stream) : launch_rows<T, 64, false>(a, stream);
    return fused ? launch_rows<T, 80, true>(a, stream) : launch_rows<T, 80, false>(a, stream);
  };
  return dtype == SAMFAST_F16 ? by_type(ElemF16{}) : by_type(ElemBf16{});
}

}  // namespace samfast
