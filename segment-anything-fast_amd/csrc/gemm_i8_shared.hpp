// Definitions shared by the int8 GEMM kernels (gemm_i8.hip, gemm_i8_persist.hip).
#pragma once

#include "samfast_internal.hpp"

namespace samfast {

constexpr int GBN = 256, GBK = 64;
constexpr int GLD = GBK;  // LDS row, bytes (unpadded; chunks are XOR-swizzled instead)

enum { EPI_I32 = 0, EPI_SCALE_BIAS_BF16 = 1, EPI_GELU_BF16 = 2, EPI_RESIDUAL_BF16 = 3 };

struct GemmArgs {
  const int8_t* x;
  const int8_t* w;
  void* out;
  const float* sx;
  const float* sw;
  const float* bias;
  int64_t ldo;
  int M, N, K;
  int tiles_m, tiles_n;
  int group_m;     // row tiles per scheduling group
  int stream_out;  // outputs without residual that exceed the 256 MB last-level cache
  int prio;        // persistent kernel: 1 = wavefronts in their K loop run at raised priority, converting ones at base priority
  int skew;        // persistent kernel: start delay of the workgroups in odd wave slots, units of 64 cycles
  int row_pitch;            // bytes between consecutive rows of X / W: K (row-major) or 64 (K-block major)
  int64_t x_kstep, w_kstep; // bytes between consecutive 64-byte k tiles: 64, or rows * 64
  const unsigned short* residual;  // EPI_RESIDUAL: (rows, N) bf16, row stride ld_res
  int64_t ld_res;
  const int32_t* dst_row;          // EPI_RESIDUAL: output row per GEMM row, -1 = drop; may be null
  // quantiser of the output rows (kernels with TAILN > 0)
  int32_t* tile_counters;          // one per row tile; zero before the launch and again after it
  int8_t* yq;                      // codes of the (LayerNorm of the) output rows, layout yq_kb64
  float* sy;                       // their scales
  const unsigned short* ln_gamma;  // TAILLN: LayerNorm weight / bias (N bf16 values each)
  const unsigned short* ln_beta;
  float ln_eps;
  int yq_kb64;
};

// 16-byte chunk c of LDS row r lives at chunk position c ^ lds_swizzle(r).  With it the
// operand reads (one chunk of 8 / 16 consecutive rows per LDS cycle) and the tile writes
// (4 chunks of 2 / 4 consecutive rows per cycle) both touch every bank once, whether the
// LDS cycles through 128 or 256 bytes.
SF_DEVICE int lds_swizzle(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }

// Persistent form of the 128 x 256 kernel (gemm_i8_persist.hip): whether it is built for this
// call, and its launch.  `a` is complete (tiles, layout, epilogue operands).
bool gemm_i8_persist_covers(int epi, const GemmArgs& a);
int gemm_i8_persist_launch(int epi, const GemmArgs& a, hipStream_t stream);

}  // namespace samfast
