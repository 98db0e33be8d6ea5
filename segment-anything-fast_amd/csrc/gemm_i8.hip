// int8 x int8 -> int32 GEMM on the gfx950 matrix cores, acc[m,n] = sum_k X[m,k] W[n,k].
//
// Both operands are K-contiguous, which is exactly what v_mfma_i32_32x32x32_i8
// wants per lane (16 consecutive k bytes of one row / column).
//
// Tiling: a 256-thread workgroup owns a 256x256 output tile; its four wavefronts
// sit 2x2, each holding a 128x128 sub-tile as 4x4 MFMA tiles (256 accumulator
// registers).  K advances 64 bytes per step through two LDS stages: the global
// loads of step t+1 are issued before the MFMAs of step t and written to the
// other stage afterwards, so one barrier per step is enough.  LDS rows are
// padded from 64 to 80 bytes so that the 16-byte operand reads of consecutive
// rows fall in distinct bank groups.
//
// W rows are stored in LDS in a permuted order (row n of a wave's 128 columns
// goes to slot (n%4)*32 + n/4) so that MFMA tile j, lane-column c holds output
// column 4c+j: after the K loop every lane owns 4 adjacent columns of each of its
// rows and writes them with one 8-byte (bf16) or 16-byte (int32) store.
//
// Workgroup ids are first made contiguous per XCD, then walked in groups of 8
// row-panels x all column tiles so that the tiles resident on one XCD share
// their X panels and the W matrix in that XCD's L2.
#include "samfast_internal.hpp"

// every fp32 step below is rounded on its own (no fused multiply-add), so results
// can be reproduced bit for bit on a CPU
#pragma clang fp contract(off)

namespace samfast {

constexpr int GBM = 256, GBN = 256, GBK = 64;
constexpr int GLD = GBK + 16;  // padded LDS row, bytes
constexpr int GSTAGE = (GBM + GBN) * GLD;
constexpr int GGROUP_M = 8;

enum { EPI_I32 = 0, EPI_SCALE_BIAS_BF16 = 1 };

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
};

template <int EPI>
__global__ __launch_bounds__(256) void gemm_i8_kernel(GemmArgs a) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * GSTAGE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 31, lh = lane >> 5;

  const unsigned int total = (unsigned int)a.tiles_m * (unsigned int)a.tiles_n;
  const unsigned int pid = xcd_contiguous_id(blockIdx.x, total);
  if (pid >= total) return;  // uniform over the workgroup
  const unsigned int per_group = GGROUP_M * a.tiles_n;
  const unsigned int first_m = (pid / per_group) * GGROUP_M;
  const unsigned int gsz = min((unsigned int)a.tiles_m - first_m, (unsigned int)GGROUP_M);
  const unsigned int in_group = pid % per_group;
  const int m0 = (int)(first_m + in_group % gsz) * GBM;
  const int n0 = (int)(in_group / gsz) * GBN;

  // ---- global -> LDS staging: 4 chunks of 16 bytes per thread and operand ----
  const int8_t* gx[4];
  const int8_t* gw[4];
  int lx[4], lw[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i;
    const int row = c >> 2, kc = c & 3;
    const int gm = min(m0 + row, a.M - 1);
    const int gn = min(n0 + row, a.N - 1);
    gx[i] = a.x + (int64_t)gm * a.K + kc * 16;
    gw[i] = a.w + (int64_t)gn * a.K + kc * 16;
    lx[i] = row * GLD + kc * 16;
    const int within = row & 127;
    const int slot = (row & 128) + (within & 3) * 32 + (within >> 2);
    lw[i] = GBM * GLD + slot * GLD + kc * 16;
  }

  i32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  i32x4 stg_x[4], stg_w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    stg_x[i] = *reinterpret_cast<const i32x4*>(gx[i]);
    stg_w[i] = *reinterpret_cast<const i32x4*>(gw[i]);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    *reinterpret_cast<i32x4*>(lds + lx[i]) = stg_x[i];
    *reinterpret_cast<i32x4*>(lds + lw[i]) = stg_w[i];
  }
  __syncthreads();

  const int a_off = (wm * 128 + lr) * GLD + lh * 16;
  const int b_off = GBM * GLD + (wn * 128 + lr) * GLD + lh * 16;
  const int nk = a.K / GBK;

  for (int kt = 0; kt < nk; ++kt) {
    const unsigned char* cur = lds + (kt & 1) * GSTAGE;
    const bool more = (kt + 1) < nk;
    if (more) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        stg_x[i] = *reinterpret_cast<const i32x4*>(gx[i] + (int64_t)(kt + 1) * GBK);
        stg_w[i] = *reinterpret_cast<const i32x4*>(gw[i] + (int64_t)(kt + 1) * GBK);
      }
    }
#pragma unroll
    for (int s = 0; s < GBK / 32; ++s) {
      i32x4 av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = *reinterpret_cast<const i32x4*>(cur + a_off + i * 32 * GLD + s * 32);
        bv[i] = *reinterpret_cast<const i32x4*>(cur + b_off + i * 32 * GLD + s * 32);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      unsigned char* nxt = lds + ((kt + 1) & 1) * GSTAGE;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<i32x4*>(nxt + lx[i]) = stg_x[i];
        *reinterpret_cast<i32x4*>(nxt + lw[i]) = stg_w[i];
      }
    }
    __syncthreads();
  }

  // ---- epilogue: lane owns columns nc..nc+3 of rows (i, r) -------------------
  const int nc = n0 + wn * 128 + 4 * lr;
  if (nc >= a.N) return;  // N % 8 == 0, so a lane's 4 columns are in or out together
  float swv[4] = {1.f, 1.f, 1.f, 1.f}, bv4[4] = {0.f, 0.f, 0.f, 0.f};
  if (EPI == EPI_SCALE_BIAS_BF16) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(a.sw + nc);
    swv[0] = t[0]; swv[1] = t[1]; swv[2] = t[2]; swv[3] = t[3];
    if (a.bias) {
      const f32x4 b = *reinterpret_cast<const f32x4*>(a.bias + nc);
      bv4[0] = b[0]; bv4[1] = b[1]; bv4[2] = b[2]; bv4[3] = b[3];
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
      if (m < a.M) {
        if (EPI == EPI_I32) {
          i32x4 o = {acc[i][0][r], acc[i][1][r], acc[i][2][r], acc[i][3][r]};
          *reinterpret_cast<i32x4*>(reinterpret_cast<int32_t*>(a.out) + (int64_t)m * a.ldo + nc) = o;
        } else {
          const float s = a.sx[m];
          float y[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // three separately rounded fp32 operations (no fused multiply-add)
            float t = (float)acc[i][j][r] * s;
            t = t * swv[j];
            y[j] = t + bv4[j];
          }
          u32x2 o = {pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3])};
          *reinterpret_cast<u32x2*>(reinterpret_cast<unsigned short*>(a.out) + (int64_t)m * a.ldo + nc) = o;
        }
      }
    }
  }
}

static int gemm_common(int epi, const int8_t* xq, const float* sx, const int8_t* wq,
                       const float* sw, const float* bias, void* out, int64_t ldo, int64_t M,
                       int N, int K, hipStream_t stream) {
  SF_REQUIRE(xq && wq && out, "gemm_i8: null pointer");
  SF_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_i8: bad shape M=%lld N=%d K=%d", (long long)M, N, K);
  SF_REQUIRE(M < (1ll << 31) - GBM, "gemm_i8: M=%lld too large", (long long)M);
  SF_REQUIRE(K % GBK == 0, "gemm_i8: K=%d must be a multiple of %d", K, GBK);
  SF_REQUIRE(N % 8 == 0, "gemm_i8: N=%d must be a multiple of 8", N);
  SF_REQUIRE(ldo >= N, "gemm_i8: output row stride %lld < N=%d", (long long)ldo, N);
  SF_REQUIRE(aligned16(xq) && aligned16(wq), "gemm_i8: operands must be 16-byte aligned");
  if (epi == EPI_I32) {
    SF_REQUIRE(aligned16(out) && ldo % 4 == 0, "gemm_i8: int32 output must be 16-byte aligned rows");
  } else {
    SF_REQUIRE(sx && sw, "gemm_i8: null scale pointer");
    SF_REQUIRE((reinterpret_cast<uintptr_t>(out) & 7u) == 0 && ldo % 4 == 0,
               "gemm_i8: bf16 output rows must be 8-byte aligned");
    SF_REQUIRE(aligned16(sw) && (!bias || aligned16(bias)),
               "gemm_i8: sw / bias must be 16-byte aligned");
  }
  if (M == 0) return SAMFAST_OK;
  GemmArgs a;
  a.x = xq; a.w = wq; a.out = out; a.sx = sx; a.sw = sw; a.bias = bias;
  a.ldo = ldo; a.M = (int)M; a.N = N; a.K = K;
  a.tiles_m = (int)((M + GBM - 1) / GBM);
  a.tiles_n = (N + GBN - 1) / GBN;
  const int64_t total = (int64_t)a.tiles_m * a.tiles_n;
  SF_REQUIRE(total < (1ll << 30), "gemm_i8: too many tiles");
  const unsigned int grid = (unsigned int)(((total + 7) / 8) * 8);
  if (epi == EPI_I32)
    hipLaunchKernelGGL(gemm_i8_kernel<EPI_I32>, dim3(grid), dim3(256), 0, stream, a);
  else
    hipLaunchKernelGGL(gemm_i8_kernel<EPI_SCALE_BIAS_BF16>, dim3(grid), dim3(256), 0, stream, a);
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
