// int8 x int8 -> int32 GEMM on the gfx950 matrix cores, acc[m,n] = sum_k X[m,k] W[n,k].
//
// Both operands are K-contiguous, which is exactly what v_mfma_i32_32x32x32_i8
// wants per lane (16 consecutive k bytes of one row / column).
//
// Tiling: a 256-thread workgroup owns a (64*TM)x256 output tile; its four
// wavefronts sit 2x2, each holding a (32*TM)x128 sub-tile as TMx4 MFMA tiles.
// TM = 2 (128x256, 128 accumulators) is the default: two workgroups share a CU, so
// the epilogue of one (a burst of HBM writes) runs under the MFMA loop of the other.
// TM = 4 (256x256, one workgroup per CU) has better operand reuse but no such overlap
// and measures slower at the encoder's shapes.
//
// K loop (main kernel, K >= 256): tiles of 64 bytes of K travel global memory -> LDS
// directly (global_load_lds_dwordx4: no staging registers, no LDS write instructions)
// through three (TM = 2) or four (TM = 4) LDS stages; in-order completion of vector
// memory loads lets "tile kt+1 has landed" be a vmcnt threshold that leaves later tiles
// in flight across the one barrier per iteration.  The MFMA operand fragments of the
// next 32-byte k-step - also across the iteration boundary - are read from LDS while
// the current MFMAs execute, and sched_group_barrier sequences slot every LDS / global
// instruction between MFMAs.  LDS rows are 64 bytes with their four 16-byte chunks
// XOR-swizzled by the row index: tile writes and operand reads are bank-conflict free
// (SQ_LDS_BANK_CONFLICT = 0).  A small register-staged variant of the same loop handles
// K < 256.
//
// W rows are stored in LDS in a permuted order (slot s of a wave's 128 columns holds
// row (s%32)*4 + s/32) so that MFMA tile j, lane-column c holds output column 4c+j:
// after the K loop every lane owns 4 adjacent columns of each of its rows and writes
// them with one 8-byte (bf16) or 16-byte (int32) store.
//
// The loads use a wave-uniform base and an unsigned 32-bit lane offset
// (global_load_lds_dwordx4 v_off, s[base:base+1]): each costs the MFMA stream ~15 cycles,
// against ~100 with a 64-bit address per lane, which is the form the compiler picks unless
// the base is pinned in scalar registers and the offset kept 32-bit at the point of use.
//
// Workgroup ids are first made contiguous per XCD, then walked in groups of row tiles x all
// column tiles so that the tiles resident on one XCD share operand panels in that XCD's L2:
// 1024 rows per group when there are many column tiles (W panels shared), one row tile per
// group when there are few (the column tiles of a row tile run side by side and share X).
// Outputs larger than the last-level cache that carry no residual (qkv, lin1: read once by
// the next kernel) are written with streaming stores.
//
// Quantiser of the output inside the GEMM (TAILN > 0).  The next Linear wants the rows this
// GEMM produces quantised per row, (LayerNorm first where one sits between them,) and a row's
// scale needs the whole row, which the tiles_n workgroups of a row tile produce between them.
// Nobody waits for anybody: a workgroup stores its tile, makes the stores visible to the whole
// device (release fence at agent scope) and adds one to the row tile's counter with a
// device-scope atomic; the workgroup that reads tiles_n - 1 knows every other tile of these 128
// rows is complete and visible, acquires, and runs the row quantiser (the code of
// quant_rowwise.hip, one wavefront per row, rows double-buffered) over them, then puts the
// counter back to zero for the next launch.  The other workgroup resident on the CU keeps the
// matrix pipe busy meanwhile.
#include "gemm_i8_shared.hpp"
#include "quant_row.hpp"
#include <pthread.h>
#include <stdlib.h>
#include <type_traits>

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

// Epilogue shared by the kernels: the lane owns 4 adjacent output columns of each of
// its 16*TM rows (MFMA tile i, register r -> row i*32 + 8*(r/4) + 4*lh + r%4).
template <int EPI, int TM>
SF_DEVICE void gemm_epilogue(const GemmArgs& a, i32x16 (&acc)[TM][4], int m0, int n0, int wm,
                             int wn, int lr, int lh) {
  const int nc = n0 + wn * 128 + 4 * lr;
  if (nc >= a.N) return;  // N % 8 == 0, so a lane's 4 columns are in or out together
  const int mrow0 = m0 + wm * 32 * TM + 4 * lh;  // + i*32 + 8*(r>>2) + (r&3)
  if (EPI == EPI_I32) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = mrow0 + i * 32 + 8 * (r >> 2) + (r & 3);
        if (m < a.M) {
          const i32x4 o = {acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
          *reinterpret_cast<i32x4*>(reinterpret_cast<int32_t*>(a.out) + (int64_t)m * a.ldo + nc) = o;
        }
      }
    return;
  }
  // all row scales of this lane first (16 groups of 4 consecutive rows), so that no
  // store has to wait behind a load
  f32x4 sxv[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int m = mrow0 + i * 32 + 8 * g;
      if (m + 3 < a.M) {
        sxv[i][g] = *reinterpret_cast<const f32x4*>(a.sx + m);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) sxv[i][g][e] = a.sx[min(m + e, a.M - 1)];
      }
    }
  const f32x4 swv = *reinterpret_cast<const f32x4*>(a.sw + nc);
  f32x4 bv4 = {0.f, 0.f, 0.f, 0.f};
  if (a.bias) bv4 = *reinterpret_cast<const f32x4*>(a.bias + nc);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    // EPI_RESIDUAL: output rows (possibly remapped) and the residual values of this
    // group of 16 rows are fetched before any of them is stored
    int drow[16];
    u32x2 res[16];
    if (EPI == EPI_RESIDUAL_BF16) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int m = mrow0 + i * 32 + 8 * g;
        if (a.dst_row) {
          if (m + 3 < a.M) {
            const i32x4 d = *reinterpret_cast<const i32x4*>(a.dst_row + m);
            drow[4 * g] = d[0]; drow[4 * g + 1] = d[1]; drow[4 * g + 2] = d[2]; drow[4 * g + 3] = d[3];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) drow[4 * g + e] = (m + e < a.M) ? a.dst_row[m + e] : -1;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) drow[4 * g + e] = (m + e < a.M) ? m + e : -1;
        }
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const u32x2 z = {0u, 0u};
        res[r] = z;
        if (drow[r] >= 0)
          res[r] = *reinterpret_cast<const u32x2*>(a.residual + (int64_t)drow[r] * a.ld_res + nc);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = mrow0 + i * 32 + 8 * (r >> 2) + (r & 3);
      const int orow = (EPI == EPI_RESIDUAL_BF16) ? drow[r] : (m < a.M ? m : -1);
      if (orow >= 0) {
        const float s = sxv[i][r >> 2][r & 3];
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
        if (EPI == EPI_RESIDUAL_BF16) {
          // bf16 add of the bf16-rounded Linear output and the residual stream
          o[0] = pack_bf16x2(bf16_lo_to_f32(o[0]) + bf16_lo_to_f32(res[r][0]),
                             bf16_hi_to_f32(o[0]) + bf16_hi_to_f32(res[r][0]));
          o[1] = pack_bf16x2(bf16_lo_to_f32(o[1]) + bf16_lo_to_f32(res[r][1]),
                             bf16_hi_to_f32(o[1]) + bf16_hi_to_f32(res[r][1]));
        }
        *reinterpret_cast<u32x2*>(reinterpret_cast<unsigned short*>(a.out) + (int64_t)orow * a.ldo + nc) = o;
      }
    }
  }
}

// Staged epilogue of the main kernel (TM = 2, bf16 outputs).  Phase 1: every lane scales
// its accumulators (row scales, column scales and bias come from a small LDS area that was
// filled by global->LDS loads at kernel start) and writes the bf16 results into the LDS
// that held the operand stages, as a row-major 128 x 256 tile.  Phase 2: the workgroup
// walks that tile 8 rows at a time, 16 bytes per lane, so that every global store (and
// residual load) instruction covers two whole 512-byte row segments.
constexpr int EP_STRIDE = 544;                 // tile row pitch in bytes: rows r and r+4 half a bank cycle apart
constexpr int EP_SCALE_BYTES = 512 + 1024 + 1024;  // sx[128], sw[256], bias[256] as fp32
constexpr int EP_ROWMAP_BYTES = 512;                // dst_row[128] (EPI_RESIDUAL)

template <int EPI>
SF_DEVICE void gemm_epilogue_staged(const GemmArgs& a, i32x16 (&acc)[2][4], unsigned char* lds,
                                    const unsigned char* sc, int m0, int n0, int wm, int wn,
                                    int lr, int lh, int tid) {
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt 0, lgkmcnt 0
  __builtin_amdgcn_s_barrier();        // nobody reads operand stages any more
  __builtin_amdgcn_sched_barrier(0);

  // phase-2 geometry: pass p (0..15) handles tile row 8p + rsub, 16-byte chunk `chunk`
  const int chunk = tid & 31, rsub = tid >> 5;
  const int n = n0 + chunk * 8;
  const bool col_ok = n < a.N;  // N % 8 == 0
  // a tile that lies inside the matrix and is not row-scattered takes straight-line code: no
  // predicates, so all residual loads and all tile reads of phase 2 are in flight together
  const bool full = m0 + 128 <= a.M && n0 + GBN <= a.N && !(EPI == EPI_RESIDUAL_BF16 && a.dst_row);
  auto out_row = [&](int p) {
    const int row = 8 * p + rsub;
    if (m0 + row >= a.M || !col_ok) return -1;
    if (EPI == EPI_RESIDUAL_BF16 && a.dst_row)  // the row map of this tile sits behind the scales
      return *reinterpret_cast<const int*>(sc + EP_SCALE_BYTES + row * 4);
    return m0 + row;
  };
  // EPI_RESIDUAL: the residual values are requested before the conversion work below, so
  // their latency is hidden behind it
  u32x4 res[16];
  if (EPI == EPI_RESIDUAL_BF16) {
    if (full) {
      const unsigned short* rp = a.residual + (int64_t)(m0 + rsub) * a.ld_res + n;
#pragma unroll
      for (int p = 0; p < 16; ++p) res[p] = *reinterpret_cast<const u32x4*>(rp + (int64_t)(8 * p) * a.ld_res);
    } else {
#pragma unroll
      for (int p = 0; p < 16; ++p) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        res[p] = z;
        const int dr = out_row(p);
        if (dr >= 0) res[p] = *reinterpret_cast<const u32x4*>(a.residual + (int64_t)dr * a.ld_res + n);
      }
    }
  }

  {
    const f32x4 swv = *reinterpret_cast<const f32x4*>(sc + 512 + (wn * 128 + 4 * lr) * 4);
    f32x4 bv4 = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) bv4 = *reinterpret_cast<const f32x4*>(sc + 1536 + (wn * 128 + 4 * lr) * 4);
    unsigned char* dst = lds + (wm * 64 + 4 * lh) * EP_STRIDE + (wn * 128 + 4 * lr) * 2;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
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
        *reinterpret_cast<u32x2*>(dst + (i * 32 + 8 * (r >> 2) + (r & 3)) * EP_STRIDE) = o;
      }
    }
  }
  // LDS writes done and, once for all of phase 2, the residual values have arrived: later
  // vmcnt waits would also wait for the stores issued in between
  __builtin_amdgcn_s_waitcnt(0x0070);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);

  unsigned short* outp = reinterpret_cast<unsigned short*>(a.out);
  const unsigned char* tile = lds + rsub * EP_STRIDE + chunk * 16;
  auto add_residual = [&](u32x4& val, const u32x4& r) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
      // bf16 add of the bf16-rounded Linear output and the residual stream
      val[c] = pack_bf16x2(bf16_lo_to_f32(val[c]) + bf16_lo_to_f32(r[c]),
                           bf16_hi_to_f32(val[c]) + bf16_hi_to_f32(r[c]));
  };
  if (full) {
    u32x4 val[16];
#pragma unroll
    for (int p = 0; p < 16; ++p) val[p] = *reinterpret_cast<const u32x4*>(tile + 8 * p * EP_STRIDE);
    unsigned short* op = outp + (int64_t)(m0 + rsub) * a.ldo + n;
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      if (EPI == EPI_RESIDUAL_BF16) add_residual(val[p], res[p]);
      // an output larger than the last-level cache that is read once (qkv, lin1) is streamed out
      if (a.stream_out) __builtin_nontemporal_store(val[p], reinterpret_cast<u32x4*>(op + (int64_t)(8 * p) * a.ldo));
      else *reinterpret_cast<u32x4*>(op + (int64_t)(8 * p) * a.ldo) = val[p];
    }
  } else {
#pragma unroll
    for (int p = 0; p < 16; ++p) {
      const int dr = out_row(p);
      u32x4 val = *reinterpret_cast<const u32x4*>(tile + 8 * p * EP_STRIDE);
      if (EPI == EPI_RESIDUAL_BF16) add_residual(val, res[p]);
      if (dr >= 0) *reinterpret_cast<u32x4*>(outp + (int64_t)dr * a.ldo + n) = val;
    }
  }
}

// The quantiser tail (see the file header).  Called by every thread of the workgroup after its
// last output store; `flag` is one LDS word nobody else uses any more.
template <int TAILN, bool TAILLN>
SF_DEVICE void gemm_quant_tail(const GemmArgs& a, int m0, int tile_m, int tid, int* flag) {
  constexpr int EPC = quant_epc_for(TAILN), NCH = quant_nch_for(TAILN);
  using RQ = RowQuantizer<NCH, EPC, TAILLN>;
  // every wavefront's stores have completed (vmcnt counts stores as well), then one thread
  // releases them - the fence is cumulative over what the barrier ordered before it
  __builtin_amdgcn_s_waitcnt(0x0070);
  __builtin_amdgcn_s_barrier();
  if (tid == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    *flag = __hip_atomic_fetch_add(a.tile_counters + tile_m, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (*flag != a.tiles_n - 1) return;  // uniform: somebody else will be the last
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");

  QuantArgs q;
  q.x = reinterpret_cast<const unsigned short*>(a.out);
  q.ldx = a.ldo;
  q.gamma = a.ln_gamma; q.beta = a.ln_beta; q.src_row = nullptr;
  q.xq = a.yq; q.sx = a.sy; q.M = a.M; q.K = TAILN;
  q.eps = a.ln_eps; q.inv_K = 1.0f / (float)TAILN; q.kb64 = a.yq_kb64;
  constexpr int nchunk = TAILN / EPC;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: rows and their addresses stay scalar
  typename RQ::in_t gw[NCH], bw[NCH];
  if (TAILLN) RQ::load_affine(q.gamma, q.beta, nchunk, lane, gw, bw);
  // wavefront w takes rows w, w + 4, ...; the loads of the next DEPTH - 1 rows are in flight while
  // one row is worked on (a lone wavefront per SIMD has nobody else to hide their latency)
  constexpr int DEPTH = NCH * RQ::W <= 12 ? 6 : 2;
  typename RQ::in_t buf[DEPTH][NCH];
  const int last = min(m0 + 128, a.M);
  const int row0 = m0 + wave;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (row0 + 4 * d < last) RQ::template load_row<false>(q.x + (int64_t)(row0 + 4 * d) * q.ldx, nchunk, lane, buf[d]);
  for (int base = row0; base < last; base += 4 * DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int row = base + 4 * d;
      if (row < last) {  // uniform over the wavefront
        RQ::finish_row(q, row, nchunk, lane, buf[d], gw, bw);
        const int next = row + 4 * DEPTH;
        if (next < last) RQ::template load_row<false>(q.x + (int64_t)next * q.ldx, nchunk, lane, buf[d]);
      }
    }
  }
  if (tid == 0) a.tile_counters[tile_m] = 0;  // the next launch finds the counter at zero
}

template <int EPI, int TM, bool GENERIC, int TAILN = 0, bool TAILLN = false>
__global__ __launch_bounds__(256, (TM == 4 ? 1 : 2)) void gemm_i8_kernel(GemmArgs a) {
  constexpr int GBM = 64 * TM;
  constexpr int GSTAGE = (GBM + GBN) * GLD;
  constexpr int NST = GENERIC ? 2 : (TM == 4 ? 4 : 3);  // LDS stages
  constexpr bool STAGED = !GENERIC && TM == 2 && EPI != EPI_I32;  // epilogue through LDS
  static_assert(!STAGED || 128 * EP_STRIDE <= NST * GSTAGE, "output tile must fit in the operand stages");
  static_assert(TAILN == 0 || STAGED, "the quantiser tail follows the staged epilogue");
  __shared__ __attribute__((aligned(16))) unsigned char lds[NST * GSTAGE + (STAGED ? EP_SCALE_BYTES + EP_ROWMAP_BYTES : 0)];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 31, lh = lane >> 5;

  const unsigned int total = (unsigned int)a.tiles_m * (unsigned int)a.tiles_n;
  const unsigned int pid = xcd_contiguous_id(blockIdx.x, total);
  if (pid >= total) return;  // uniform over the workgroup
  const unsigned int GGROUP_M = a.group_m;
  const unsigned int per_group = GGROUP_M * a.tiles_n;
  const unsigned int first_m = (pid / per_group) * GGROUP_M;
  const unsigned int gsz = min((unsigned int)a.tiles_m - first_m, (unsigned int)GGROUP_M);
  const unsigned int in_group = pid % per_group;
  const int m0 = (int)(first_m + in_group % gsz) * GBM;
  const int n0 = (int)(in_group / gsz) * GBN;

  // ---- global -> LDS staging: 16-byte chunks, TM per thread for X and 4 for W ----
  // (32-bit lane offsets from the uniform matrix bases; M*K and N*K fit in 31 bits)
  int ox[TM], ow[4];
  int lx[TM], lw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i;
    const int row = c >> 2, kc = c & 3;
    if (i < TM) {
      const int gm = min(m0 + row, a.M - 1);
      ox[i] = gm * a.row_pitch + kc * 16;
      lx[i] = row * GLD + ((kc ^ lds_swizzle(row)) * 16);
    }
    // W: consecutive chunk groups go to consecutive LDS slots (no write bank conflicts);
    // slot s of a 128-column half holds W row (s % 32) * 4 + s / 32 of that half
    const int slot = row & 127;
    const int wrow = (row & 128) + (slot & 31) * 4 + (slot >> 5);
    const int gn = min(n0 + wrow, a.N - 1);
    ow[i] = gn * a.row_pitch + kc * 16;
    lw[i] = GBM * GLD + row * GLD + ((kc ^ lds_swizzle(row)) * 16);
  }

  i32x16 acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // ---- software pipeline -------------------------------------------------------
  // Two LDS stages, the barrier in the MIDDLE of an iteration.  Iteration kt:
  //   A. read the fragments of k-step 1 of tile kt (stage kt&1) while the MFMAs of
  //      k-step 0 run;
  //   B. barrier: every wave now holds all of tile kt in registers, so stage kt&1 is
  //      free, and tile kt+1 (written in the previous iteration) is visible;
  //   C. read the fragments of k-step 0 of tile kt+1, write tile kt+2 (fetched from
  //      global memory into registers one iteration ago) into the freed stage, issue
  //      the global loads of tile kt+3 - all while the MFMAs of k-step 1 run.
  i32x4 stg_x[TM], stg_w[4];
  auto global_fetch = [&](int kt) {
    const int8_t* xb = a.x + kt * a.x_kstep;  // uniform
    const int8_t* wb = a.w + kt * a.w_kstep;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < TM) stg_x[i] = *reinterpret_cast<const i32x4*>(xb + ox[i]);
      stg_w[i] = *reinterpret_cast<const i32x4*>(wb + ow[i]);
    }
  };
  auto lds_store = [&](int stage) {
    unsigned char* dst = lds + stage * GSTAGE;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < TM) *reinterpret_cast<i32x4*>(dst + lx[i]) = stg_x[i];
      *reinterpret_cast<i32x4*>(dst + lw[i]) = stg_w[i];
    }
  };
  // fragment of k-step s: chunk 2s + lh of row (tile row base + lr); the swizzle only
  // depends on lr because every tile row base is a multiple of 32
  const int frag_chunk = (lh ^ lds_swizzle(lr)) * 16;
  const int a_off = (wm * 32 * TM + lr) * GLD + frag_chunk;
  const int b_off = GBM * GLD + (wn * 128 + lr) * GLD + frag_chunk;
  auto load_frags = [&](int stage, int step, i32x4 (&av)[TM], i32x4 (&bv)[4]) {
    const unsigned char* src = lds + stage * GSTAGE;
    const int flip = step * 32;  // (2*step + lh) ^ swz == ((lh ^ swz) ^ 2*step) as a chunk index
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (i < TM) av[i] = *reinterpret_cast<const i32x4*>(src + ((a_off + i * 32 * GLD) ^ flip));
      bv[i] = *reinterpret_cast<const i32x4*>(src + ((b_off + i * 32 * GLD) ^ flip));
    }
  };
  auto mma = [&](const i32x4 (&av)[TM], const i32x4 (&bv)[4]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], acc[i][j], 0, 0, 0);
  };

  const int nk = a.K / GBK;
  i32x4 fa0[TM], fb0[4], fa1[TM], fb1[4];
  int kt = 0;
  if constexpr (GENERIC) {
    global_fetch(0);
    lds_store(0);
    if (nk > 1) {
      global_fetch(1);
      lds_store(1);
    }
    if (nk > 2) global_fetch(2);
    __syncthreads();
    load_frags(0, 0, fa0, fb0);
    // any K: run-time conditions inside the loop
    auto iteration = [&](int kt, int stage) {
      load_frags(stage, 1, fa1, fb1);
      mma(fa0, fb0);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      if (kt + 1 < nk) load_frags(stage ^ 1, 0, fa0, fb0);
      if (kt + 2 < nk) {
        lds_store(stage);
        if (kt + 3 < nk) global_fetch(kt + 3);
      }
      mma(fa1, fb1);
    };
    for (; kt + 1 < nk; kt += 2) {
      iteration(kt, 0);
      iteration(kt + 1, 1);
    }
    if (kt < nk) iteration(kt, 0);
  } else {
    // nk >= 4.  Tiles travel global memory -> LDS directly (global_load_lds_dwordx4, no
    // staging registers, no LDS write instructions) through THREE stages, so a tile has
    // two full iterations to arrive.  One wave instruction fills 1 KB = 16 LDS rows; lane l
    // lands at chunk position l&3 of row l>>2 of that block, so the XOR swizzle is applied
    // to the GLOBAL address (the lane fetches the chunk that belongs at its position).
    // In-order completion lets "tile kt+1 has landed" be expressed as vmcnt <= (loads per
    // tile), leaving tile kt+2 in flight across the barrier.
    constexpr int NLD = (GBM + GBN) / 64;  // wave instructions per tile and wave: 6 / 8
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // unsigned 32-bit lane offsets from a wave-uniform base: the loads then take the
    // scalar-base form (global_load_lds_dwordx4 v_off, s[base]).  With 64-bit per-lane
    // addresses each of them costs the MFMA stream ~100 cycles instead of ~15 (measured).
    unsigned int dma_off[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int rho = 16 * (wave_u + 4 * i) + (lane >> 2);  // LDS row of this lane's chunk
      const int chunk = (lane & 3) ^ lds_swizzle(rho);
      if (i < GBM / 64) {  // X rows
        dma_off[i] = (unsigned int)(min(m0 + rho, a.M - 1) * a.row_pitch + chunk * 16);
      } else {             // W slots (slot s of a 128-column half holds W row (s%32)*4 + s/32)
        const int sl = rho - GBM;
        const int wrow = (sl & 128) + (sl & 31) * 4 + ((sl & 127) >> 5);
        dma_off[i] = (unsigned int)(min(n0 + wrow, a.N - 1) * a.row_pitch + chunk * 16);
      }
    }
    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto dma_issue = [&](int kt, int stage_off) {
      const int8_t* xb = a.x + kt * a.x_kstep;
      const int8_t* wb = a.w + kt * a.w_kstep;
      // keep the tile bases in scalar registers: folded into the lane offsets they would
      // turn the loads back into the 64-bit per-lane address form
      asm volatile("" : "+s"(xb), "+s"(wb));
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        unsigned int off = dma_off[i];
        asm volatile("" : "+v"(off));  // a 32-bit value at the point of use: no hoisted 64-bit copy
        const int8_t* src = (i < GBM / 64 ? xb : wb) + off;
        unsigned char* dst = lds + stage_off + (wave_u + 4 * i) * 1024;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
      }
    };
    auto frags_at = [&](int stage_off, int step, i32x4 (&av)[TM], i32x4 (&bv)[4]) {
      const unsigned char* src = lds + stage_off;
      const int flip = step * 32;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (i < TM) av[i] = *reinterpret_cast<const i32x4*>(src + ((a_off + i * 32 * GLD) ^ flip));
        bv[i] = *reinterpret_cast<const i32x4*>(src + ((b_off + i * 32 * GLD) ^ flip));
      }
    };
    // s_waitcnt immediate: vmcnt in bits 3:0 and 15:14 ("at most n loads still in flight"),
    // expcnt 6:4 = 7 (no wait), lgkmcnt 11:8 = 0 (all of this wave's LDS reads done)
    auto wait_imm = [](int n) constexpr { return 0x0070 | (n & 15) | ((n >> 4) << 14); };
    static_assert((NST - 1) * NLD <= 63, "vmcnt immediate");

    if constexpr (STAGED) {
      // row scales, column scales and bias of this tile, 4 bytes per lane, straight into LDS;
      // they are the oldest loads in flight, so every later vmcnt wait covers them
      unsigned char* sc = lds + NST * GSTAGE;
      const int mm = min(m0 + (wave_u & 1) * 64 + lane, a.M - 1);
      const int nn = min(n0 + wave_u * 64 + lane, a.N - 1);
      __builtin_amdgcn_global_load_lds((gptr_t)(a.sx + mm), (lptr_t)(sc + (wave_u & 1) * 256), 4, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)(a.sw + nn), (lptr_t)(sc + 512 + wave_u * 256), 4, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr_t)((a.bias ? a.bias : a.sw) + nn),
                                       (lptr_t)(sc + 1536 + wave_u * 256), 4, 0, 0);
      if (EPI == EPI_RESIDUAL_BF16 && a.dst_row)  // uniform: every wave issues it or none does
        __builtin_amdgcn_global_load_lds((gptr_t)(a.dst_row + mm),
                                         (lptr_t)(sc + EP_SCALE_BYTES + (wave_u & 1) * 256), 4, 0, 0);
    }
    int st[NST];  // st[j] = LDS offset of the stage holding tile kt + j (uniform, rotated)
#pragma unroll
    for (int j = 0; j < NST; ++j) {
      st[j] = j * GSTAGE;
      dma_issue(j, st[j]);  // nk >= NST is guaranteed by the host
    }
    __builtin_amdgcn_s_waitcnt(wait_imm((NST - 1) * NLD));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    frags_at(st[0], 0, fa0, fb0);

    // ISSUE: fetch tile kt+NST into the stage freed at the barrier; NEXT: a tile kt+1
    // exists; KEEP: tiles that may stay in flight across the barrier (after tile kt+1).
    // (sched_group_barrier masks: 0x008 MFMA, 0x100 LDS read, 0x020 global read)
    auto iteration = [&](int kt, auto issue_c, auto next_c, auto keep_c, auto extra_c) {
      constexpr bool ISSUE = decltype(issue_c)::value != 0;
      constexpr bool NEXT = decltype(next_c)::value != 0;
      constexpr int KEEP = decltype(keep_c)::value;
      constexpr int EXTRA = decltype(extra_c)::value;  // younger non-tile loads that may stay in flight
      frags_at(st[0], 1, fa1, fb1);
      mma(fa0, fb0);
#pragma unroll
      for (int g = 0; g < TM + 4; ++g) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, TM / 2, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // own LDS reads of this stage done; own share of tile kt+1 landed; then all waves meet
      __builtin_amdgcn_s_waitcnt(wait_imm(NEXT ? KEEP * NLD + EXTRA : 63));
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (ISSUE) dma_issue(kt + NST, st[0]);
      if constexpr (NEXT) frags_at(st[1], 0, fa0, fb0);
      mma(fa1, fb1);
#pragma unroll
      for (int g = 0; g < TM + 4; ++g) {
        if constexpr (NEXT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, TM / 2, 0);
        if constexpr (ISSUE) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      const int t = st[0];
#pragma unroll
      for (int j = 0; j + 1 < NST; ++j) st[j] = st[j + 1];
      st[NST - 1] = t;
    };
    using Yes = std::integral_constant<int, 1>;
    using No = std::integral_constant<int, 0>;
    for (; kt + NST < nk; ++kt) iteration(kt, Yes{}, Yes{}, std::integral_constant<int, NST - 2>{}, No{});
    // the last NST iterations fetch nothing; fewer and fewer tiles remain in flight
    if constexpr (NST == 4) iteration(kt++, No{}, Yes{}, std::integral_constant<int, 2>{}, No{});
    iteration(kt++, No{}, Yes{}, std::integral_constant<int, 1>{}, No{});
    iteration(kt++, No{}, Yes{}, No{}, No{});
    iteration(kt++, No{}, No{}, No{}, No{});
  }

  if constexpr (STAGED)
    gemm_epilogue_staged<EPI>(a, acc, lds, lds + NST * GSTAGE, m0, n0, wm, wn, lr, lh, tid);
  else
    gemm_epilogue<EPI, TM>(a, acc, m0, n0, wm, wn, lr, lh);
  if constexpr (TAILN > 0)
    gemm_quant_tail<TAILN, TAILLN>(a, m0, m0 / GBM, tid, reinterpret_cast<int*>(lds + NST * GSTAGE));
}


// =============================================================================================
// Three (or more) workgroups per CU.  Same LDS layout and arithmetic as gemm_i8_kernel<EPI, 2,
// false>; what changes is the budget: at most 168 registers per lane and 53 KB of LDS per
// workgroup, so that a third workgroup fits on the CU.  While one workgroup is in its epilogue
// (no matrix instructions for 7-16 K cycles), two others are in their loops.
//   * operand fragments are single-buffered: the other wavefronts of the SIMD cover a
//     wavefront's LDS read latency;
//   * two LDS stages: at the top of iteration kt every wavefront has finished tile kt-1
//     (barrier), so tile kt+1 is requested into the stage tile kt-1 used, and has the whole
//     iteration to land;
//   * the epilogue is staged through LDS 64 rows at a time (the full bf16 tile does not fit
//     next to nothing in 48 KB), residual values are fetched after the conversion work.
// The tile is BM x BN = 128 x 256 (waves 2 x 2, each 64 x 128: 2 x 4 MFMA tiles), or 64 x 128
// (each wave 32 x 64: 1 x 2 tiles, 32 accumulators, 27 KB of LDS) for launches whose large tiles
// would leave most of the GPU's workgroup slots empty (4096 rows of a single image): four times
// the workgroups, each a quarter of the work.
// KSPLIT = 2 (64 x 128 tiles only) puts eight wavefronts on a tile: wavefronts 0-3 take the even k
// tiles, wavefronts 4-7 the odd ones, each half with operand stages of its own, so the chain of
// dependent iterations a single small launch has to sit through is half as long (a 4096-row lin2 at
// K = 3072 is 384 workgroups of 48 iterations: one round, latency-bound).  The two partial sums are
// int32 and meet in LDS after the loop - integer addition is order-free, so the result has the
// same bits - and wavefronts 0-3 run the epilogue.
// =============================================================================================
template <int BM, int BN, int KSPLIT = 1>
struct Gemm3Cfg {
  static constexpr int TMW = BM / 64, TNW = BN / 64;  // MFMA tiles per wavefront: rows, columns
  static constexpr int NST = 2;
  static constexpr int GSTAGE = (BM + BN) * GLD;
  static constexpr int NLD = (BM + BN) / 64;          // global->LDS wave instructions per tile and wavefront
  static constexpr int EP_PITCH = BN * 2 + 32;        // staged output tile: row pitch in bytes
  static constexpr int SX_OFF = 0, SW_OFF = BM * 4, BIAS_OFF = SW_OFF + BN * 4, MAP_OFF = BIAS_OFF + BN * 4;
  static constexpr int SC_BYTES = MAP_OFF + BM * 4;
  static constexpr int LDS_BYTES = KSPLIT * NST * GSTAGE + SC_BYTES;
  static constexpr int THREADS = 256 * KSPLIT;
  static constexpr int CHUNKS = BN / 8;               // 16-byte pieces per output row
  static constexpr int ROWS_PER_PASS = 256 / CHUNKS;  // output rows the workgroup stores per pass
  static constexpr int PASSES = 64 / ROWS_PER_PASS;   // passes over a staged 64-row tile
  static constexpr int MIN_WG = BM == 128 ? 3 : (KSPLIT == 2 ? 2 : 4);
  static_assert(64 * EP_PITCH <= NST * GSTAGE, "a 64-row output tile must fit in the operand stages");
  static_assert((BM == 128 && BN == 256) || (BM == 64 && BN == 128), "tile shapes built");
  static_assert(KSPLIT == 1 || (KSPLIT == 2 && BM == 64), "the K split is built for the small tile");
  static_assert(KSPLIT == 1 || BM * BN * 4 <= KSPLIT * NST * GSTAGE, "the partial sums must fit in the operand stages");
};

template <int EPI, int BM, int BN, int KSPLIT = 1>
__global__ __launch_bounds__((Gemm3Cfg<BM, BN, KSPLIT>::THREADS), (Gemm3Cfg<BM, BN, KSPLIT>::MIN_WG)) void gemm_i8_kernel3(GemmArgs a) {
  static_assert(EPI != EPI_I32, "bf16 epilogues only");
  using C = Gemm3Cfg<BM, BN, KSPLIT>;
  constexpr int TMW = C::TMW, TNW = C::TNW, NLD = C::NLD, GSTAGE = C::GSTAGE;
  __shared__ __attribute__((aligned(16))) unsigned char lds_all[C::LDS_BYTES];
  unsigned char* sc = lds_all + KSPLIT * C::NST * GSTAGE;

  const int tid = threadIdx.x & 255;  // index inside the wavefront group (KSPLIT = 1: the workgroup)
  const int lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_u = wave_all & 3;    // wavefront inside its group of four
  const int grp = wave_all >> 2;      // K split: which k tiles this group takes
  unsigned char* lds = lds_all + grp * (C::NST * GSTAGE);  // the group's operand stages (and, group 0, the epilogue's tile)
  const int wm = wave_u >> 1, wn = wave_u & 1;
  const int lr = lane & 31, lh = lane >> 5;

  const unsigned int total = (unsigned int)a.tiles_m * (unsigned int)a.tiles_n;
  const unsigned int pid = xcd_contiguous_id(blockIdx.x, total);
  if (pid >= total) return;  // uniform over the workgroup
  const unsigned int per_group = (unsigned int)a.group_m * a.tiles_n;
  const unsigned int first_m = (pid / per_group) * a.group_m;
  const unsigned int gsz = min((unsigned int)a.tiles_m - first_m, (unsigned int)a.group_m);
  const unsigned int in_group = pid % per_group;
  const int m0 = (int)(first_m + in_group % gsz) * BM;
  const int n0 = (int)(in_group / gsz) * BN;

  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;

  // lane offsets of the tile loads (see gemm_i8_kernel: the XOR swizzle is applied to the global
  // address; W rows are permuted - slot s of a wavefront's BN/2 columns holds W row (s % 32) * TNW
  // + s / 32 - so that a lane ends with TNW adjacent output columns)
  unsigned int dma_off[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int rho = 16 * (wave_u + 4 * i) + (lane >> 2);
    const int chunk = (lane & 3) ^ lds_swizzle(rho);
    if (i < BM / 64) {
      dma_off[i] = (unsigned int)(min(m0 + rho, a.M - 1) * a.row_pitch + chunk * 16);
    } else {
      const int sl = rho - BM;                      // slot inside the W part of the stage
      const int half = sl / (BN / 2), sh = sl % (BN / 2);
      const int wrow = half * (BN / 2) + (sh & 31) * TNW + (sh >> 5);
      dma_off[i] = (unsigned int)(min(n0 + wrow, a.N - 1) * a.row_pitch + chunk * 16);
    }
  }
  auto dma_issue = [&](int kt, int stage_off) {
    const int8_t* xb = a.x + kt * a.x_kstep;
    const int8_t* wb = a.w + kt * a.w_kstep;
    asm volatile("" : "+s"(xb), "+s"(wb));  // tile bases stay scalar: scalar-base load form
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      unsigned int off = dma_off[i];
      asm volatile("" : "+v"(off));
      const int8_t* src = (i < BM / 64 ? xb : wb) + off;
      unsigned char* dst = lds + stage_off + (wave_u + 4 * i) * 1024;
      __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)dst, 16, 0, 0);
    }
  };

  {
    // row scales, column scales, bias (and row map) of this tile, 4 bytes per lane, straight into
    // LDS; wavefront w fetches 64-entry slice w % (count / 64) of each (duplicates are harmless)
    const int rs = wave_u % (BM / 64), cs = wave_u % (BN / 64);
    const int mm = min(m0 + rs * 64 + lane, a.M - 1);
    const int nn = min(n0 + cs * 64 + lane, a.N - 1);
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sx + mm), (lptr_t)(sc + C::SX_OFF + rs * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)(a.sw + nn), (lptr_t)(sc + C::SW_OFF + cs * 256), 4, 0, 0);
    __builtin_amdgcn_global_load_lds((gptr_t)((a.bias ? a.bias : a.sw) + nn),
                                     (lptr_t)(sc + C::BIAS_OFF + cs * 256), 4, 0, 0);
    if (EPI == EPI_RESIDUAL_BF16 && a.dst_row)
      __builtin_amdgcn_global_load_lds((gptr_t)(a.dst_row + mm), (lptr_t)(sc + C::MAP_OFF + rs * 256), 4, 0, 0);
  }

  i32x16 acc[TMW][TNW];
#pragma unroll
  for (int i = 0; i < TMW; ++i)
#pragma unroll
    for (int j = 0; j < TNW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  const int frag_chunk = (lh ^ lds_swizzle(lr)) * 16;
  const int a_off = (wm * (BM / 2) + lr) * GLD + frag_chunk;
  const int b_off = BM * GLD + (wn * (BN / 2) + lr) * GLD + frag_chunk;

  const int nk = a.K / GBK;
  dma_issue(grp, 0);
  for (int kt = grp, it = 0; kt < nk; kt += KSPLIT, ++it) {  // (K split: nk % KSPLIT == 0, both groups iterate alike)
    const int stage_off = (it & 1) * GSTAGE;
    // own share of tile kt has landed; after the barrier the whole tile is visible and every
    // wavefront has left tile kt-1, whose stage may be refilled
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (kt + KSPLIT < nk) dma_issue(kt + KSPLIT, stage_off ^ GSTAGE);
    const unsigned char* src = lds + stage_off;
#pragma unroll
    for (int step = 0; step < 2; ++step) {
      const int flip = step * 32;
      i32x4 av[TMW], bv[TNW];
#pragma unroll
      for (int i = 0; i < TMW; ++i) av[i] = *reinterpret_cast<const i32x4*>(src + ((a_off + i * 32 * GLD) ^ flip));
#pragma unroll
      for (int j = 0; j < TNW; ++j) bv[j] = *reinterpret_cast<const i32x4*>(src + ((b_off + j * 32 * GLD) ^ flip));
#pragma unroll
      for (int j = 0; j < TNW; ++j)
#pragma unroll
        for (int i = 0; i < TMW; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
  }

  bool active = true;  // whether this wavefront takes part in the epilogue's data movement
  if constexpr (KSPLIT == 2) {
    // the odd group's partial sums meet the even group's in LDS (the operand stages are free once
    // every wavefront has left the loop); conflict-free: consecutive lanes, consecutive words
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    int* red = reinterpret_cast<int*>(lds_all);
    if (grp == 1) {
#pragma unroll
      for (int i = 0; i < TMW; ++i)
#pragma unroll
        for (int j = 0; j < TNW; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) red[((wave_u * TMW * TNW + i * TNW + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();
    if (grp == 0) {
#pragma unroll
      for (int i = 0; i < TMW; ++i)
#pragma unroll
        for (int j = 0; j < TNW; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] += red[((wave_u * TMW * TNW + i * TNW + j) * 16 + r) * 64 + lane];
    }
    active = grp == 0;
  }

  // ---- epilogue, 64 rows at a time: pass h holds MFMA row tile h of both wavefront rows ----
  // LDS tile row t = wm*32 + rr stands for output row m0 + wm*(BM/2) + h*32 + rr
  const int chunk = tid % C::CHUNKS, rsub = tid / C::CHUNKS;
  const int n = n0 + chunk * 8;
  const bool col_ok = n < a.N;  // N % 8 == 0
  const bool full = m0 + BM <= a.M && n0 + BN <= a.N && !(EPI == EPI_RESIDUAL_BF16 && a.dst_row);
  unsigned short* outp = reinterpret_cast<unsigned short*>(a.out);
  float swv[TNW], bvv[TNW];
#pragma unroll
  for (int j = 0; j < TNW; ++j) bvv[j] = 0.f;
#pragma unroll
  for (int h = 0; h < TMW; ++h) {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's LDS reads are done (stores may stay in flight)
    __builtin_amdgcn_s_barrier();  // operand stages (h = 0) / the previous pass's tile are no longer read
    __builtin_amdgcn_sched_barrier(0);
    if (h == 0) {
#pragma unroll
      for (int j = 0; j < TNW; ++j) {
        swv[j] = *reinterpret_cast<const float*>(sc + C::SW_OFF + (wn * (BN / 2) + TNW * lr + j) * 4);
        if (a.bias) bvv[j] = *reinterpret_cast<const float*>(sc + C::BIAS_OFF + (wn * (BN / 2) + TNW * lr + j) * 4);
      }
    }
    if (active) {
      unsigned char* dst = lds + (wm * 32 + 4 * lh) * C::EP_PITCH + (wn * (BN / 2) + TNW * lr) * 2;
      f32x4 sxv[4];
#pragma unroll
      for (int g = 0; g < 4; ++g)
        sxv[g] = *reinterpret_cast<const f32x4*>(sc + C::SX_OFF + (wm * (BM / 2) + h * 32 + 8 * g + 4 * lh) * 4);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float sxr = sxv[r >> 2][r & 3];
        float y[TNW];
#pragma unroll
        for (int j = 0; j < TNW; ++j) {
          // three separately rounded fp32 operations (no fused multiply-add)
          float t = (float)acc[h][j][r] * sxr;
          t = t * swv[j];
          y[j] = t + bvv[j];
        }
        unsigned int o[TNW / 2];
#pragma unroll
        for (int j = 0; j < TNW / 2; ++j) {
          o[j] = pack_bf16x2(y[2 * j], y[2 * j + 1]);
          if (EPI == EPI_GELU_BF16)  // activation of the bf16-rounded Linear output, as a separate GELU would see it
            o[j] = pack_bf16x2(gelu_erf(bf16_lo_to_f32(o[j])), gelu_erf(bf16_hi_to_f32(o[j])));
        }
        unsigned char* d = dst + (8 * (r >> 2) + (r & 3)) * C::EP_PITCH;
        if (TNW == 4) {
          const u32x2 o2 = {o[0], o[TNW / 2 - 1]};
          *reinterpret_cast<u32x2*>(d) = o2;
        } else {
          *reinterpret_cast<unsigned int*>(d) = o[0];
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the tile writes have landed
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // the workgroup walks the 64-row tile ROWS_PER_PASS rows at a time, 16 bytes per lane
    const unsigned char* tile = lds + rsub * C::EP_PITCH + chunk * 16;
    auto add_residual = [&](u32x4& val, const u32x4& r) {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        // bf16 add of the bf16-rounded Linear output and the residual stream
        val[c] = pack_bf16x2(bf16_lo_to_f32(val[c]) + bf16_lo_to_f32(r[c]),
                             bf16_hi_to_f32(val[c]) + bf16_hi_to_f32(r[c]));
    };
    // pass p: tile row t = ROWS_PER_PASS * p + rsub -> row (t / 32) * (BM / 2) + h * 32 + t % 32 of the tile
    auto tile_row = [&](int p) {
      const int t = C::ROWS_PER_PASS * p + rsub;
      return (t >> 5) * (BM / 2) + h * 32 + (t & 31);
    };
    if (!active) {
      // (the odd group only keeps the barrier count)
    } else if (full) {
      u32x4 res[C::PASSES], val[C::PASSES];
      if (EPI == EPI_RESIDUAL_BF16) {
#pragma unroll
        for (int p = 0; p < C::PASSES; ++p)
          res[p] = *reinterpret_cast<const u32x4*>(a.residual + (int64_t)(m0 + tile_row(p)) * a.ld_res + n);
      }
#pragma unroll
      for (int p = 0; p < C::PASSES; ++p)
        val[p] = *reinterpret_cast<const u32x4*>(tile + C::ROWS_PER_PASS * p * C::EP_PITCH);
#pragma unroll
      for (int p = 0; p < C::PASSES; ++p) {
        if (EPI == EPI_RESIDUAL_BF16) add_residual(val[p], res[p]);
        u32x4* op = reinterpret_cast<u32x4*>(outp + (int64_t)(m0 + tile_row(p)) * a.ldo + n);
        // an output larger than the last-level cache that is read once (qkv, lin1) is streamed out
        if (a.stream_out) __builtin_nontemporal_store(val[p], op);
        else *op = val[p];
      }
    } else {
#pragma unroll
      for (int p = 0; p < C::PASSES; ++p) {
        const int row = tile_row(p);
        int dr = -1;
        if (m0 + row < a.M && col_ok) {
          dr = m0 + row;
          if (EPI == EPI_RESIDUAL_BF16 && a.dst_row) dr = *reinterpret_cast<const int*>(sc + C::MAP_OFF + row * 4);
        }
        u32x4 val = *reinterpret_cast<const u32x4*>(tile + C::ROWS_PER_PASS * p * C::EP_PITCH);
        if (dr >= 0) {
          if (EPI == EPI_RESIDUAL_BF16)
            add_residual(val, *reinterpret_cast<const u32x4*>(a.residual + (int64_t)dr * a.ld_res + n));
          *reinterpret_cast<u32x4*>(outp + (int64_t)dr * a.ldo + n) = val;
        }
      }
    }
  }
}

// the output quantiser a launch may carry (null = none)
struct GemmTail {
  int8_t* yq;
  float* sy;
  const void* gamma;  // non-null: LayerNorm before the quantiser
  const void* beta;
  float eps;
  int yq_layout;
  int32_t* counters;
};

// N for which the quantiser tail is built, per kind: plain after GELU (the MLP widths of
// ViT-B / L / H), LayerNorm after a residual epilogue (their embedding widths)
static bool tail_built(int epi, bool ln, int N) {
  if (epi == EPI_GELU_BF16 && !ln) return N == 3072 || N == 4096 || N == 5120;
  if (epi == EPI_RESIDUAL_BF16 && ln) return N == 768 || N == 1024 || N == 1280;
  return false;
}

// whether gemm_common would run `tail` inside the GEMM for this call
static bool tail_fusable(int epi, const GemmTail& t, int N, int K, const int32_t* dst_row) {
  return K / GBK >= 4 && knob(KNOB_GEMM_TM) != 4 && !dst_row && tail_built(epi, t.gamma != nullptr, N);
}

static int gemm_common(int epi, const int8_t* xq, const float* sx, const int8_t* wq,
                       const float* sw, const float* bias, void* out, int64_t ldo, int64_t M,
                       int N, int K, hipStream_t stream, const void* residual = nullptr,
                       int64_t ld_res = 0, const int32_t* dst_row = nullptr,
                       int layout = SAMFAST_LAYOUT_ROWMAJOR, const GemmTail* tail = nullptr) {
  // no rows: nothing to do, and the row operands of an empty call may be null
  SF_REQUIRE(wq && (M == 0 || (xq && out)), "gemm_i8: null pointer");
  SF_REQUIRE(layout == SAMFAST_LAYOUT_ROWMAJOR || layout == SAMFAST_LAYOUT_KB64, "gemm_i8: unknown layout %d", layout);
  SF_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_i8: bad shape M=%lld N=%d K=%d", (long long)M, N, K);
  SF_REQUIRE(M < (1ll << 31) - 256, "gemm_i8: M=%lld too large", (long long)M);
  SF_REQUIRE(M * K < (1ll << 31) && (int64_t)N * K < (1ll << 31),
             "gemm_i8: operands of 2 GiB or more are not supported");
  SF_REQUIRE(K % GBK == 0, "gemm_i8: K=%d must be a multiple of %d", K, GBK);
  SF_REQUIRE(N % 8 == 0, "gemm_i8: N=%d must be a multiple of 8", N);
  SF_REQUIRE(ldo >= N, "gemm_i8: output row stride %lld < N=%d", (long long)ldo, N);
  SF_REQUIRE(aligned16(xq) && aligned16(wq), "gemm_i8: operands must be 16-byte aligned");
  if (epi == EPI_I32) {
    SF_REQUIRE(aligned16(out) && ldo % 4 == 0, "gemm_i8: int32 output must be 16-byte aligned rows");
  } else {
    SF_REQUIRE(sw && (M == 0 || sx), "gemm_i8: null scale pointer");
    SF_REQUIRE(aligned16(out) && ldo % 8 == 0, "gemm_i8: bf16 output rows must be 16-byte aligned");
    SF_REQUIRE(aligned16(sw) && aligned16(sx) && (!bias || aligned16(bias)),
               "gemm_i8: sx / sw / bias must be 16-byte aligned");
  }
  if (epi == EPI_RESIDUAL_BF16) {
    SF_REQUIRE((residual || M == 0) && aligned16(residual) && ld_res >= N && ld_res % 8 == 0,
               "gemm_i8: residual must be non-null with 16-byte aligned rows");
    SF_REQUIRE(!dst_row || aligned16(dst_row), "gemm_i8: dst_row must be 16-byte aligned");
  }
  if (M == 0) return SAMFAST_OK;
  GemmArgs a;
  a.x = xq; a.w = wq; a.out = out; a.sx = sx; a.sw = sw; a.bias = bias;
  a.ldo = ldo; a.M = (int)M; a.N = N; a.K = K;
  if (layout == SAMFAST_LAYOUT_KB64) {
    a.row_pitch = GBK; a.x_kstep = M * GBK; a.w_kstep = (int64_t)N * GBK;
  } else {
    a.row_pitch = K; a.x_kstep = GBK; a.w_kstep = GBK;
  }
  a.residual = reinterpret_cast<const unsigned short*>(residual);
  a.ld_res = ld_res; a.dst_row = dst_row;
  const bool generic_k = K / GBK < 4;  // fewer k tiles than LDS stages
  const int tm = generic_k ? 2 : (knob(KNOB_GEMM_TM) == 4 ? 4 : 2);  // tuning aid: 2 or 4
  const int bm = 64 * tm;
  a.tiles_m = (int)((M + bm - 1) / bm);
  a.tiles_n = (N + GBN - 1) / GBN;
  // row tiles per scheduling group, from the fabric traffic measured per shape: with few column
  // tiles (proj, lin2: 5) the workgroups that share an X row tile should be adjacent (-23 % / -31 %
  // fetched bytes); with many (qkv 15, lin1 20) 1024 rows per group let W panels be shared
  a.group_m = a.tiles_n <= 6 ? 1 : 1024 / bm;
  // (an output the quantiser tail reads back right away is not streamed past the caches)
  a.stream_out = !tail && (epi == EPI_SCALE_BIAS_BF16 || epi == EPI_GELU_BF16) && M * (int64_t)N * 2 >= (256ll << 20);
  a.skew = 0;
  a.prio = 0;
  a.tile_counters = nullptr; a.yq = nullptr; a.sy = nullptr; a.ln_gamma = a.ln_beta = nullptr;
  a.ln_eps = 0.f; a.yq_kb64 = 0;
  if (tail) {
    a.tile_counters = tail->counters; a.yq = tail->yq; a.sy = tail->sy;
    a.ln_gamma = reinterpret_cast<const unsigned short*>(tail->gamma);
    a.ln_beta = reinterpret_cast<const unsigned short*>(tail->beta);
    a.ln_eps = tail->eps; a.yq_kb64 = tail->yq_layout == SAMFAST_LAYOUT_KB64;
  }
  const int64_t total = (int64_t)a.tiles_m * a.tiles_n;
  SF_REQUIRE(total < (1ll << 30), "gemm_i8: too many tiles");
  // resident workgroups that walk a list of tiles each (SAMFAST_GEMM_PERSIST=1), where built
  if (!tail && !generic_k && tm == 2 && gemm_i8_persist_covers(epi, a)) return gemm_i8_persist_launch(epi, a, stream);
  const unsigned int grid = (unsigned int)(((total + 7) / 8) * 8);
  const bool generic = generic_k;
  // the three-workgroups-per-CU form of the main kernel (SAMFAST_GEMM_WG3=0: two per CU)
  if (!tail && !generic && tm == 2 && epi != EPI_I32 && knob(KNOB_GEMM_WG3) != 0) {
    // 64 x 128 tiles when 128 x 256 ones would leave more than half of the 768 workgroup slots of
    // the GPU empty (SAMFAST_GEMM_TILE=64 / 128 forces either)
    const int ft = knob(KNOB_GEMM_TILE);
    const bool small = ft != kKnobUnset ? ft == 64 : total < knob_or(KNOB_GEMM_SMALL_BELOW, 385);
    if (small) {
      a.tiles_m = (int)((M + 63) / 64);
      a.tiles_n = (N + 127) / 128;
      a.group_m = a.tiles_n <= 6 ? 1 : 1024 / 64;
    }
    const int64_t total3 = (int64_t)a.tiles_m * a.tiles_n;
    // small tiles that do not even fill the GPU's slots once, on a long K loop: two wavefront groups
    // per tile, each on every second k tile (SAMFAST_GEMM_SPLITK=0 off, 2 wherever it is built)
    const int sk = knob_or(KNOB_GEMM_SPLITK, 1);
    const bool ksplit = small && (K / GBK) % 2 == 0 && (sk >= 2 || (sk == 1 && total3 <= 768 && K / GBK >= 12));
    const unsigned int grid3 = (unsigned int)(((total3 + 7) / 8) * 8);
#define SF_GEMM3(E)                                                                                          \
  do {                                                                                                       \
    if (small && ksplit) hipLaunchKernelGGL((gemm_i8_kernel3<E, 64, 128, 2>), dim3(grid3), dim3(512), 0, stream, a); \
    else if (small) hipLaunchKernelGGL((gemm_i8_kernel3<E, 64, 128>), dim3(grid3), dim3(256), 0, stream, a); \
    else hipLaunchKernelGGL((gemm_i8_kernel3<E, 128, 256>), dim3(grid3), dim3(256), 0, stream, a);           \
  } while (0)
    switch (epi) {
      case EPI_SCALE_BIAS_BF16: SF_GEMM3(EPI_SCALE_BIAS_BF16); break;
      case EPI_GELU_BF16: SF_GEMM3(EPI_GELU_BF16); break;
      default: SF_GEMM3(EPI_RESIDUAL_BF16); break;
    }
#undef SF_GEMM3
    return check_launch("gemm_i8_kernel3");
  }
  if (tail) {
    // the caller has checked tail_fusable(): main kernel, 128-row tiles
#define SF_GEMM_TAIL(E, NN, LN)                                                                              \
  case NN:                                                                                                   \
    hipLaunchKernelGGL((gemm_i8_kernel<E, 2, false, NN, LN>), dim3(grid), dim3(256), 0, stream, a);          \
    break
    if (epi == EPI_GELU_BF16) {
      switch (N) {
        SF_GEMM_TAIL(EPI_GELU_BF16, 3072, false);
        SF_GEMM_TAIL(EPI_GELU_BF16, 4096, false);
        SF_GEMM_TAIL(EPI_GELU_BF16, 5120, false);
      }
    } else {
      switch (N) {
        SF_GEMM_TAIL(EPI_RESIDUAL_BF16, 768, true);
        SF_GEMM_TAIL(EPI_RESIDUAL_BF16, 1024, true);
        SF_GEMM_TAIL(EPI_RESIDUAL_BF16, 1280, true);
      }
    }
#undef SF_GEMM_TAIL
    return check_launch("gemm_i8_kernel (quantiser tail)");
  }
#define SF_GEMM_LAUNCH(E)                                                                      \
  do {                                                                                         \
    if (generic)                                                                               \
      hipLaunchKernelGGL((gemm_i8_kernel<E, 2, true>), dim3(grid), dim3(256), 0, stream, a);   \
    else if (tm == 4)                                                                          \
      hipLaunchKernelGGL((gemm_i8_kernel<E, 4, false>), dim3(grid), dim3(256), 0, stream, a);  \
    else                                                                                       \
      hipLaunchKernelGGL((gemm_i8_kernel<E, 2, false>), dim3(grid), dim3(256), 0, stream, a);  \
  } while (0)
  switch (epi) {
    case EPI_I32: SF_GEMM_LAUNCH(EPI_I32); break;
    case EPI_SCALE_BIAS_BF16: SF_GEMM_LAUNCH(EPI_SCALE_BIAS_BF16); break;
    case EPI_GELU_BF16: SF_GEMM_LAUNCH(EPI_GELU_BF16); break;
    default: SF_GEMM_LAUNCH(EPI_RESIDUAL_BF16); break;
  }
#undef SF_GEMM_LAUNCH
  return check_launch("gemm_i8_kernel");
}

}  // namespace samfast

extern "C" int samfast_gemm_i8_i32(const int8_t* xq, const int8_t* wq, int32_t* acc, int64_t M,
                                   int N, int K, void* stream) {
  return samfast::gemm_common(samfast::EPI_I32, xq, nullptr, wq, nullptr, nullptr, acc, N, M, N, K,
                              reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_gemm_i8_scale_bias(const int8_t* xq, const float* sx, const int8_t* wq,
                                          const float* sw, const float* bias, void* y, int64_t ldy,
                                          int64_t M, int N, int K, int dtype, void* stream) {
  if (dtype != SAMFAST_BF16) {
    samfast::set_error("gemm_i8_scale_bias: only bf16 output");
    return SAMFAST_E_UNSUPPORTED;
  }
  return samfast::gemm_common(samfast::EPI_SCALE_BIAS_BF16, xq, sx, wq, sw, bias, y, ldy, M, N, K,
                              reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_gemm_i8_fused(const int8_t* xq, const float* sx, const int8_t* wq,
                                     const float* sw, const float* bias, void* y, int64_t ldy,
                                     int64_t M, int N, int K, int dtype, int epilogue,
                                     const void* residual, int64_t ld_res, const int32_t* dst_row,
                                     int layout, void* stream) {
  using namespace samfast;
  if (dtype != SAMFAST_BF16) {
    set_error("gemm_i8_fused: only bf16 output");
    return SAMFAST_E_UNSUPPORTED;
  }
  int epi;
  switch (epilogue) {
    case SAMFAST_EPILOGUE_NONE: epi = EPI_SCALE_BIAS_BF16; break;
    case SAMFAST_EPILOGUE_GELU: epi = EPI_GELU_BF16; break;
    case SAMFAST_EPILOGUE_RESIDUAL: epi = EPI_RESIDUAL_BF16; break;
    default:
      set_error("gemm_i8_fused: unknown epilogue %d", epilogue);
      return SAMFAST_E_INVALID;
  }
  return gemm_common(epi, xq, sx, wq, sw, bias, y, ldy, M, N, K,
                     reinterpret_cast<hipStream_t>(stream), residual, ld_res, dst_row, layout);
}

extern "C" int samfast_gemm_i8_fused_quant(const int8_t* xq, const float* sx, const int8_t* wq,
                                           const float* sw, const float* bias, void* y, int64_t ldy,
                                           int64_t M, int N, int K, int dtype, int epilogue,
                                           const void* residual, int64_t ld_res, int layout,
                                           const void* ln_gamma, const void* ln_beta, float ln_eps,
                                           int8_t* yq, float* sy, int yq_layout,
                                           int32_t* tile_counters, void* stream) {
  using namespace samfast;
  if (dtype != SAMFAST_BF16) {
    set_error("gemm_i8_fused_quant: only bf16 output");
    return SAMFAST_E_UNSUPPORTED;
  }
  int epi;
  switch (epilogue) {
    case SAMFAST_EPILOGUE_NONE: epi = EPI_SCALE_BIAS_BF16; break;
    case SAMFAST_EPILOGUE_GELU: epi = EPI_GELU_BF16; break;
    case SAMFAST_EPILOGUE_RESIDUAL: epi = EPI_RESIDUAL_BF16; break;
    default:
      set_error("gemm_i8_fused_quant: unknown epilogue %d", epilogue);
      return SAMFAST_E_INVALID;
  }
  // the quantiser addresses yq with 32-bit lane offsets (the two-launch form checks the same limit)
  SF_REQUIRE(M >= 0 && N > 0 && M * (int64_t)N < (1ll << 31),
             "gemm_i8_fused_quant: outputs of 2^31 elements or more are not supported (M=%lld N=%d)", (long long)M, N);
  SF_REQUIRE((ln_gamma == nullptr) == (ln_beta == nullptr), "gemm_i8_fused_quant: gamma and beta go together");
  SF_REQUIRE(M == 0 || (yq && sy && tile_counters), "gemm_i8_fused_quant: null output or counter pointer");
  SF_REQUIRE(yq_layout == SAMFAST_LAYOUT_ROWMAJOR || (yq_layout == SAMFAST_LAYOUT_KB64 && N % 64 == 0),
             "gemm_i8_fused_quant: yq layout must be row-major, or K-block major with N %% 64 == 0");
  SF_REQUIRE((reinterpret_cast<uintptr_t>(yq) & 7u) == 0 && (reinterpret_cast<uintptr_t>(tile_counters) & 3u) == 0,
             "gemm_i8_fused_quant: yq must be 8-byte aligned");
  SF_REQUIRE(!ln_gamma || (aligned16(ln_gamma) && aligned16(ln_beta) && ln_eps > 0.f),
             "gemm_i8_fused_quant: gamma / beta must be 16-byte aligned and eps positive");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  GemmTail t = {yq, sy, ln_gamma, ln_beta, ln_eps, yq_layout, tile_counters};
  if (tail_fusable(epi, t, N, K, nullptr))
    return gemm_common(epi, xq, sx, wq, sw, bias, y, ldy, M, N, K, s, residual, ld_res, nullptr, layout, &t);
  // shapes the in-kernel quantiser is not built for: the same result from two launches
  const int rc = gemm_common(epi, xq, sx, wq, sw, bias, y, ldy, M, N, K, s, residual, ld_res, nullptr, layout);
  if (rc != SAMFAST_OK) return rc;
  if (ln_gamma)
    return samfast_layernorm_quant_i8(y, ldy, ln_gamma, ln_beta, ln_eps, nullptr, yq, sy, M, N, dtype, yq_layout, stream);
  return samfast_quant_rowwise_i8(y, ldy, yq, sy, M, N, dtype, yq_layout, stream);
}

// ---- the same call for callers that cannot allocate ---------------------------------------
// The counter workspace of samfast_gemm_i8_fused_quant lives in a file-scope device array, one
// copy per GPU, held until the process ends.  Its address on a device is looked up once per
// device (the array's name is only a host-side handle, never a device address).
namespace samfast {

constexpr int kNoAllocMaxTiles = 32768;  // 128 KiB per GPU: up to 32768 * 128 = 4 194 304 rows
constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) int32_t scratch[kNoAllocMaxTiles];

static int32_t* g_scratch_ptr[kNoAllocMaxDevices];  // per device, null until looked up
static pthread_mutex_t g_scratch_lock = PTHREAD_MUTEX_INITIALIZER;

// address of `scratch` on the current device, looked up on the first call per device
static int scratch_of_current_device(int32_t** out) {
  int dev = -1;
  const hipError_t e0 = hipGetDevice(&dev);
  if (e0 != hipSuccess) SF_FAIL(SAMFAST_E_LAUNCH, "gemm_i8_fused_quant_noalloc: hipGetDevice: %s", hipGetErrorString(e0));
  SF_REQUIRE(dev >= 0 && dev < kNoAllocMaxDevices, "gemm_i8_fused_quant_noalloc: device index %d out of range", dev);
  pthread_mutex_lock(&g_scratch_lock);
  int32_t* p = g_scratch_ptr[dev];
  hipError_t e1 = hipSuccess;
  if (!p) {
    e1 = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
    if (e1 == hipSuccess) g_scratch_ptr[dev] = p;
  }
  pthread_mutex_unlock(&g_scratch_lock);
  if (e1 != hipSuccess || !p)
    SF_FAIL(SAMFAST_E_LAUNCH, "gemm_i8_fused_quant_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e1));
  *out = p;
  return SAMFAST_OK;
}

// the counters a launch is about to use start at zero whatever an earlier call left behind
// (a fill kernel rather than a memset node: the call may be recorded into a graph)
__global__ void clear_counters_kernel(int32_t* counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}

}  // namespace samfast

extern "C" int samfast_gemm_i8_fused_quant_noalloc(const int8_t* xq, const float* sx, const int8_t* wq,
                                                   const float* sw, const float* bias, void* y, int64_t ldy,
                                                   int64_t M, int N, int K, int dtype, int epilogue,
                                                   const void* residual, int64_t ld_res, int layout,
                                                   const void* ln_gamma, const void* ln_beta, float ln_eps,
                                                   int8_t* yq, float* sy, int yq_layout, void* stream) {
  using namespace samfast;
  SF_REQUIRE(M >= 0, "gemm_i8_fused_quant_noalloc: bad M=%lld", (long long)M);
  const int64_t tiles = (M + 127) / 128;
  SF_REQUIRE(tiles <= kNoAllocMaxTiles,
             "gemm_i8_fused_quant_noalloc: M=%lld needs %lld row-tile counters, the built-in workspace holds %d "
             "(at most %lld rows); use samfast_gemm_i8_fused_quant with a workspace of your own",
             (long long)M, (long long)tiles, kNoAllocMaxTiles, (long long)kNoAllocMaxTiles * 128);
  SF_REQUIRE(N > 0 && M * (int64_t)N < (1ll << 31),
             "gemm_i8_fused_quant_noalloc: outputs of 2^31 elements or more are not supported (M=%lld N=%d)",
             (long long)M, N);
  int32_t* counters = nullptr;
  const int rc = scratch_of_current_device(&counters);
  if (rc != SAMFAST_OK) return rc;
  if (tiles > 0) {
    hipLaunchKernelGGL(clear_counters_kernel, dim3((unsigned int)((tiles + 255) / 256)), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), counters, (int)tiles);
    const int rl = check_launch("clear_counters_kernel");
    if (rl != SAMFAST_OK) return rl;
  }
  return samfast_gemm_i8_fused_quant(xq, sx, wq, sw, bias, y, ldy, M, N, K, dtype, epilogue, residual, ld_res,
                                     layout, ln_gamma, ln_beta, ln_eps, yq, sy, yq_layout, counters, stream);
}
