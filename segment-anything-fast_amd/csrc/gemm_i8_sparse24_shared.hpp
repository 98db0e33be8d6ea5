// Definitions shared by the 2:4-sparse int8 GEMM kernels (gemm_i8_sparse24.hip,
// gemm_i8_sp24_persist.hip): tile shape, LDS stage layout, operand swizzles, launch arguments.
#pragma once

#include "samfast_internal.hpp"

namespace samfast {

typedef int i32x8 __attribute__((ext_vector_type(8)));

constexpr int SBW = 256;  // W rows per workgroup (sparse operand = MFMA rows)
constexpr int SBX = 128;  // X rows per workgroup (dense operand = MFMA columns)
constexpr int SBK = 64;   // dense k per tile = one sparse MFMA k-step
constexpr int S_OFF_W = SBX * SBK;             // X tile: 128 rows x 64 B
constexpr int S_OFF_I = S_OFF_W + SBW * 32;    // Wc tile: 256 rows x 32 B
constexpr int S_STAGE = S_OFF_I + SBW * 8;     // index tile: 256 rows x 8 B
constexpr int SEP_SCALE_BYTES = 512 + 1024 + 1024;  // sx[128], sw[256], bias[256] of a tile as fp32

enum { SEPI_I32 = 0, SEPI_SCALE_BIAS = 1, SEPI_GELU = 2, SEPI_RESIDUAL = 3 };

struct SparseArgs {
  const int8_t* x;
  const int8_t* wc;
  const int32_t* widx;
  void* out;
  const float* sx;
  const float* sw;
  const float* bias;
  int64_t ldo;
  int M, N, K;
  int tiles_x, tiles_w;
  int group_x;       // X panels (128 rows) per scheduling group
  int x_row_pitch;   // bytes between consecutive X rows: K (row-major) or 64 (K-block major)
  int64_t x_kstep;   // bytes between consecutive 64-byte k tiles of X: 64, or M * 64
  const unsigned short* residual;
  int64_t ld_res;
};

// X rows: 64 B, four 16-byte chunks XOR-swizzled (same function as the dense kernel)
SF_DEVICE int sp_swizzle_x(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }
// Wc rows: 32 B, two chunks; 8 / 16 consecutive rows read one chunk each without bank conflicts
SF_DEVICE int sp_swizzle_w(int row) { return ((row >> 2) ^ (row >> 3)) & 1; }
// LDS slot (0..255) of the W tile -> W row of the tile held there
SF_DEVICE int sp_slot_to_row(int slot) {
  const int ta = (slot >> 5) & 3, i = slot & 31;
  const int g = i >> 3, h = (i >> 2) & 1, e = i & 3;
  return (slot & 128) + 32 * g + 16 * (ta >> 1) + 8 * h + 4 * (ta & 1) + e;
}

// Resident-workgroup form (gemm_i8_sp24_persist.hip): whether it is built for this call, and its
// launch.  `a` is complete (tiles, layout, epilogue operands).
bool gemm_i8_sp24_persist_covers(int epi, const SparseArgs& a);
int gemm_i8_sp24_persist_launch(int epi, const SparseArgs& a, hipStream_t stream);

}  // namespace samfast
