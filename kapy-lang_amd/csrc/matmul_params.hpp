// matmul_params.hpp — kernel argument block shared by the 16-bit and fp8 matmul paths.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kapy_hip.h"

namespace kapy {

struct GemmParams {
  const char *a, *b, *acc;
  char *d;
  const float *row_scale, *col_scale;  // optional fp32 scales applied to the accumulator (both or neither)
  // fused elementwise tail on the fp32 accumulator: d = act(acc * alpha + bias[n]) (mulf by a splat, addf of a
  // broadcast row, a unary op, then the cast to the result type)
  const char *bias;    // [N] values of bias_dtype, or null
  float alpha;         // 1.0f: no mulf
  int32_t bias_dtype;
  int32_t act;         // a unary kapy_ew_op, maximumf / minimumf against act_operand, or -1
  float act_operand;
  int64_t a_sm, a_sk;  // lhs element strides along M and K
  int64_t b_sn, b_sk;  // rhs element strides along N and K
  int64_t acc_sm, acc_sn, d_sm, d_sn;
  int32_t M, N, K;
  int32_t acc_dtype;  // -1: no accumulator input
  int32_t d_dtype;
  int32_t rz;         // final cast rounds toward zero
  int32_t tiles_m, tiles_n;
  // K split across split_k workgroups per output tile (blockIdx.y = the split): each leaves its fp32 partial tile in
  // `partial`, counts itself in counters[tile], and the workgroup that arrives last sums the partials in split order
  // (so the result does not depend on who was last), runs the epilogue and sets the counter back to zero.
  int32_t split_k;     // 1: no split
  float *partial;      // [tile][split][register quad][thread] float4, written whole before it is read
  uint32_t *counters;  // [tile], zero between calls
};

// Bytes of workspace in front of the partial sums that hold the per-tile arrival counters (room for 4096 tiles).
constexpr int64_t kSplitCounterBytes = 16384;
constexpr int kMaxSplitK = 8;

// Tiled LDS-direct MFMA kernel on fp8 operands (both K-contiguous, extents multiples of the tile).
// lhs_fmt / rhs_fmt: 0 = E4M3, 1 = E5M2.  Returns KAPY_ERR_UNSUPPORTED when no compiled tile fits,
// without having launched anything.
int matmul_f8_tiled(const GemmParams &p, int lhs_fmt, int rhs_fmt, int want_tile, hipStream_t s);

// Decides whether a 128 x 128 tiled kernel with K-tiles of tile_k splits K for this problem (kapy_matmul_cfg::split_k,
// workspace) and sets p.split_k / p.partial / p.counters; KAPY_OK, or the status of a split that was asked for and
// cannot be honoured.
int plan_split_k(GemmParams &p, const kapy_matmul_cfg &c, int tile_k);

// 256 x 256 x 64 tiles for a row-major lhs and a row-major rhs (matmul_nn256.hip): whether the kernel serves the problem
// (the strip epilogue's own conditions are the caller's to check), and its launch.
bool nn256_serves(const GemmParams &p);
int launch_nn256(GemmParams p, bool bf16, hipStream_t s);

}  // namespace kapy
