// Per-row symmetric int8 quantiser (bf16 -> int8 + fp32 scale), optionally preceded
// by LayerNorm over the row and a row gather (window partition).  HBM-bound for long rows
// (K = 5120); for K = 1280, whose tensors sit in the last-level cache, the vector ALU is the
// limit (310 vector instructions per row plain, 530 with LayerNorm, by the hardware counters).
//
// One wavefront owns one output row: the source row is read once with 16- or 8-byte loads
// and unpacked to fp32 registers, (normalised,) reduced to its absmax across the 64 lanes
// (DPP within rows of 16 lanes, lane swaps between them: no LDS), then scaled, rounded
// half-to-even and written back as 8- or 4-byte packs of int8.
// Algorithmic traffic: 2 bytes read + 1 byte written per element + 4 bytes of scale.
//
// q = rint(x / s) must equal the IEEE division bit for bit.  Most elements take a
// cheap route: the exact product x * fl(1/s) differs from fl(x / s) by at most 1.6e-5, so
// its rint can only differ when it lies within that distance of a half-integer; only those
// elements (and their 8-element chunk) are redone with the true division (quant_row.hpp).
// |x| <= absmax makes |x / s| <= 127 by construction, so no clamp is needed.
#include "quant_row.hpp"

namespace samfast {

constexpr int kQuantWavesPerBlock = 4;

template <int NCH, int EPC, bool LN>
__global__ __launch_bounds__(64 * kQuantWavesPerBlock) void quant_rowwise_bf16_kernel(QuantArgs a) {
  using RQ = RowQuantizer<NCH, EPC, LN>;
  const int lane = threadIdx.x & 63;
  // the wavefront index is uniform: telling the compiler so keeps the row and everything derived from it
  // (row pointers, output offsets) in scalar registers instead of 64-bit arithmetic per lane
  const int64_t row = (int64_t)blockIdx.x * kQuantWavesPerBlock + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (row >= a.M) return;  // whole wavefront leaves together
  const int nchunk = a.K / EPC;

  int64_t srow = row;
  if (LN && a.src_row) {
    srow = a.src_row[row];
    if (srow < 0) {  // a padding token: LayerNorm output replaced by zeros
      RQ::zero_row(a, row, nchunk, lane);
      return;
    }
  }
  // all global loads first: the row, and (LN) the lane's slices of gamma and beta, which do not
  // depend on the statistics and would otherwise add a second memory latency to the chain
  typename RQ::in_t xw[NCH], gw[NCH], bw[NCH];
  // long rows (the 671 MB lin1 output at ViT-H batch 16) are read once and never again: streamed
  RQ::template load_row<(!LN && NCH >= 8)>(a.x + srow * a.ldx, nchunk, lane, xw);
  if (LN) RQ::load_affine(a.gamma, a.beta, nchunk, lane, gw, bw);
  RQ::finish_row(a, row, nchunk, lane, xw, gw, bw);
}

template <int NCH, int EPC, bool LN>
static int launch_quant(const QuantArgs& a, hipStream_t stream) {
  const int64_t blocks = (a.M + kQuantWavesPerBlock - 1) / kQuantWavesPerBlock;
  hipLaunchKernelGGL((quant_rowwise_bf16_kernel<NCH, EPC, LN>), dim3((unsigned int)blocks),
                     dim3(64 * kQuantWavesPerBlock), 0, stream, a);
  return check_launch("quant_rowwise_bf16_kernel");
}

template <bool LN>
static int dispatch_quant(const QuantArgs& a, hipStream_t s) {
  // rows that 4-element chunks divide among the 64 lanes exactly and 8-element chunks do not
  if (a.K == 768) return launch_quant<3, 4, LN>(a, s);
  if (a.K == 1280) return launch_quant<5, 4, LN>(a, s);
  const int need = (a.K / 8 + 63) / 64;
  if (need <= 2) return launch_quant<2, 8, LN>(a, s);
  if (need <= 3) return launch_quant<3, 8, LN>(a, s);
  if (need <= 4) return launch_quant<4, 8, LN>(a, s);
  if (need <= 6) return launch_quant<6, 8, LN>(a, s);
  if (need <= 8) return launch_quant<8, 8, LN>(a, s);
  if (need <= 10) return launch_quant<10, 8, LN>(a, s);
  if (need <= 12) return launch_quant<12, 8, LN>(a, s);
  return launch_quant<16, 8, LN>(a, s);
}

static int check_common(const char* who, const void* x, int64_t ldx, const int8_t* xq, const float* sx,
                        int64_t M, int K, int dtype, int layout) {
  SF_REQUIRE(layout == SAMFAST_LAYOUT_ROWMAJOR || (layout == SAMFAST_LAYOUT_KB64 && K % 64 == 0),
             "%s: layout must be row-major, or K-block major with K %% 64 == 0", who);
  SF_REQUIRE(M >= 0 && K > 0, "%s: bad shape M=%lld K=%d", who, (long long)M, K);
  SF_REQUIRE(M == 0 || (x && xq && sx), "%s: null pointer", who);  // no rows: the buffers may be null
  if (dtype != SAMFAST_BF16) SF_FAIL(SAMFAST_E_UNSUPPORTED, "%s: only bf16 input", who);
  SF_REQUIRE(K % 8 == 0 && K <= 8192, "%s: K=%d must be a multiple of 8, <= 8192", who, K);
  SF_REQUIRE(ldx >= K && ldx % 8 == 0, "%s: ldx=%lld must be >= K and a multiple of 8", who,
             (long long)ldx);
  SF_REQUIRE(aligned16(x) && (reinterpret_cast<uintptr_t>(xq) & 7u) == 0,
             "%s: x must be 16-byte and xq 8-byte aligned", who);
  SF_REQUIRE((M + 3) / 4 < (1ll << 31), "%s: M too large", who);
  SF_REQUIRE(M * (int64_t)K < (1ll << 31), "%s: outputs of 2 GiB or more are not supported (the GEMM cannot read them)", who);
  return SAMFAST_OK;
}

}  // namespace samfast

extern "C" int samfast_quant_rowwise_i8(const void* x, int64_t ldx, int8_t* xq, float* sx,
                                        int64_t M, int K, int dtype, int layout, void* stream) {
  using namespace samfast;
  const int rc = check_common("quant_rowwise", x, ldx, xq, sx, M, K, dtype, layout);
  if (rc != SAMFAST_OK) return rc;
  if (M == 0) return SAMFAST_OK;
  QuantArgs a = {};
  a.x = reinterpret_cast<const unsigned short*>(x);
  a.ldx = ldx; a.xq = xq; a.sx = sx; a.M = M; a.K = K;
  a.kb64 = layout == SAMFAST_LAYOUT_KB64;
  return dispatch_quant<false>(a, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int samfast_layernorm_quant_i8(const void* x, int64_t ldx, const void* gamma,
                                          const void* beta, float eps, const int32_t* src_row,
                                          int8_t* xq, float* sx, int64_t M, int K, int dtype,
                                          int layout, void* stream) {
  using namespace samfast;
  const int rc = check_common("layernorm_quant", x, ldx, xq, sx, M, K, dtype, layout);
  if (rc != SAMFAST_OK) return rc;
  SF_REQUIRE(gamma && beta && aligned16(gamma) && aligned16(beta),
             "layernorm_quant: gamma / beta must be non-null and 16-byte aligned");
  SF_REQUIRE(eps > 0.f, "layernorm_quant: eps must be positive");
  if (M == 0) return SAMFAST_OK;
  QuantArgs a = {};
  a.x = reinterpret_cast<const unsigned short*>(x);
  a.ldx = ldx; a.xq = xq; a.sx = sx; a.M = M; a.K = K;
  a.gamma = reinterpret_cast<const unsigned short*>(gamma);
  a.beta = reinterpret_cast<const unsigned short*>(beta);
  a.src_row = src_row; a.eps = eps; a.inv_K = 1.0f / (float)K;
  a.kb64 = layout == SAMFAST_LAYOUT_KB64;
  return dispatch_quant<true>(a, reinterpret_cast<hipStream_t>(stream));
}
