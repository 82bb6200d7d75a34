// batched.hip — many small copies, or many small matrix products, of ONE shape in one launch.
//
// The reference compiles a kapy.func to one kernel in which every program instance and warp executes an op at once
// (FuncOpToLLVM.cpp:72-88).  kapy_run_mlir reaches the same op for all instances in flight one after the other; when it
// repeats a run it has kept, the calls that differ only in where their operands lie - the same kapy.ld_matrix,
// kapy.cp_async_global_to_shared or kapy.matmul of every instance and warp - are made here as one launch over a table of
// base addresses in device memory (one row per call), with the arithmetic of the calls they stand for:
//   copy_table    dst[i, j] = src[i, j] over [d0 x d1] elements of 1, 2 or 4 bytes, any positive strides, nothing padded
//                 (kapy_copy without transpose whose source view covers the target's extent);
//   matmul_table  D = A . B (+ C) on f16 / bf16 operands as the library's kernel for a row-major lhs and a row-major rhs
//                 computes it (nn_kernel, matmul.hip): fp32 accumulators from zero, one v_mfma_f32_16x16x32 per 32 values of
//                 K in ascending order, K positions 8 * (lane / 16) .. + 7 of a slice in a lane, the positions past K fed
//                 zeros, then the accumulator input added in fp32 and one rounding to nearest even - so a product made here
//                 has the bits of the same product made by kapy_matmul.
#include "common.hpp"
#include "mfma.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

struct CopyTableParams {
  const uint64_t *table;  // [n][2]: source base, target base (addresses of element (0, 0) of the views)
  int32_t d0, d1, elem_bytes, vec16;
  int64_t ss0, ss1, ds0, ds1;  // element strides
};

// grid: (workgroups per view, views).  vec16: rows are contiguous on both sides and every base and pitch is a multiple of 16
// bytes, as is a row's length: 16 bytes per lane.
__global__ __launch_bounds__(256) void copy_table_kernel(CopyTableParams p) {
  const char *src = (const char *)p.table[2 * (size_t)blockIdx.y];
  char *dst = (char *)p.table[2 * (size_t)blockIdx.y + 1];
  const int64_t step = (int64_t)gridDim.x * 256, first = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (p.vec16) {
    const int32_t per_row = p.d1 * p.elem_bytes / 16;
    const int64_t pieces = (int64_t)p.d0 * per_row, spitch = p.ss0 * p.elem_bytes, dpitch = p.ds0 * p.elem_bytes;
    for (int64_t i = first; i < pieces; i += step) {
      const int64_t r = i / per_row, c = i % per_row;
      *(u32x4 *)(dst + r * dpitch + c * 16) = *(const u32x4 *)(src + r * spitch + c * 16);
    }
    return;
  }
  const int64_t n = (int64_t)p.d0 * p.d1;
  for (int64_t i = first; i < n; i += step) {
    const int64_t r = i / p.d1, c = i % p.d1;
    const int64_t so = r * p.ss0 + c * p.ss1, to = r * p.ds0 + c * p.ds1;
    switch (p.elem_bytes) {
    case 1: ((uint8_t *)dst)[to] = ((const uint8_t *)src)[so]; break;
    case 2: ((uint16_t *)dst)[to] = ((const uint16_t *)src)[so]; break;
    default: ((uint32_t *)dst)[to] = ((const uint32_t *)src)[so]; break;
    }
  }
}

struct MatmulTableParams {
  const uint64_t *table;  // [n][4]: lhs, rhs, accumulator input (0: none), result
  int32_t M, N, K, blocks_n, blocks;
  int32_t acc_dtype, d_dtype;
  int64_t a_sm, b_sk, acc_sm, acc_sn, d_sm, d_sn;  // (lhs rows and rhs k-rows are contiguous: a_sk = b_sn = 1)
};

// grid: (16 x 16 blocks of a result / 4, products); a wavefront per block.  The instruction is issued as the library's
// kernels issue it, the rhs fragment in the first slot: a lane's four registers are four consecutive columns of one row.
template <typename T>
__global__ __launch_bounds__(256) void matmul_table_kernel(MatmulTableParams p) {
  const int lane = threadIdx.x & 63;
  const int32_t block = (int32_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (block >= p.blocks) return;
  const uint64_t *row = p.table + 4 * (size_t)blockIdx.y;
  const uint16_t *a = (const uint16_t *)row[0], *b = (const uint16_t *)row[1];
  const char *acc_in = (const char *)row[2];
  char *d = (char *)row[3];
  const int32_t m0 = (block / p.blocks_n) * 16, n0 = (block % p.blocks_n) * 16;
  const OperandLane at = operand_lane(T::kShape, lane);  // row (lhs) / column (rhs) of the block, first of the lane's 8 K positions
  const int32_t m = m0 + at.row, n = n0 + at.row;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int32_t k0 = 0; k0 < p.K; k0 += 32) {
    const int32_t k = k0 + at.k0;
    u32x4 af = {0, 0, 0, 0}, bf = {0, 0, 0, 0};
    // (K is a multiple of 8 and the rows are 16-byte aligned: a lane's 8 positions are all there or all beyond K)
    if (k < p.K && m < p.M) af = *(const u32x4 *)(a + (int64_t)m * p.a_sm + k);
    if (k < p.K && n < p.N) {
      uint16_t e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = b[(int64_t)(k + i) * p.b_sk + n];
      bf = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16), (uint32_t)e[4] | ((uint32_t)e[5] << 16),
                 (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
    }
    acc = T::mfma(&bf, &af, acc);
  }
  const AccLane out = acc_lane(mfma_acc_exchanged(T::kShape), T::kShape, lane);
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int32_t r = m0 + out.row + v * out.drow, c = n0 + out.col + v * out.dcol;
    if (r >= p.M || c >= p.N) continue;
    float x = acc[v];
    if (acc_in) x += load_as_f32(acc_in, p.acc_dtype, (int64_t)r * p.acc_sm + (int64_t)c * p.acc_sn);
    const int64_t idx = (int64_t)r * p.d_sm + (int64_t)c * p.d_sn;
    switch (p.d_dtype) {
    case KAPY_F32: ((float *)d)[idx] = x; break;
    case KAPY_F16: ((uint16_t *)d)[idx] = f32_to_f16_rn(x); break;
    default: ((uint16_t *)d)[idx] = f32_to_bf16_rn(x); break;
    }
  }
}

}  // namespace

int copy_table_launch(const uint64_t *device_table, int32_t n, const CopyTableShape &sh, bool vec16, hipStream_t s) {
  if (n <= 0 || sh.d0 <= 0 || sh.d1 <= 0) return KAPY_OK;
  if (n > 65535) return fail(KAPY_ERR_INVALID, "copy table: %d views in one launch", n);
  CopyTableParams p;
  p.table = device_table;
  p.d0 = sh.d0; p.d1 = sh.d1; p.elem_bytes = sh.elem_bytes; p.vec16 = vec16 ? 1 : 0;
  p.ss0 = sh.ss0; p.ss1 = sh.ss1; p.ds0 = sh.ds0; p.ds1 = sh.ds1;
  const int64_t items = vec16 ? (int64_t)sh.d0 * sh.d1 * sh.elem_bytes / 16 : (int64_t)sh.d0 * sh.d1;
  const int64_t per_view = std::min<int64_t>(std::max<int64_t>((items + 255) / 256, 1), 64);
  copy_table_kernel<<<dim3((unsigned)per_view, (unsigned)n), 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int matmul_table_launch(const uint64_t *device_table, int32_t n, const MatmulTableShape &sh, hipStream_t s) {
  if (n <= 0 || sh.M <= 0 || sh.N <= 0) return KAPY_OK;
  if (n > 65535) return fail(KAPY_ERR_INVALID, "matmul table: %d products in one launch", n);
  MatmulTableParams p;
  p.table = device_table;
  p.M = sh.M; p.N = sh.N; p.K = sh.K;
  p.blocks_n = (sh.N + 15) / 16;
  p.blocks = ((sh.M + 15) / 16) * p.blocks_n;
  p.acc_dtype = sh.acc_dtype; p.d_dtype = sh.d_dtype;
  p.a_sm = sh.a_sm; p.b_sk = sh.b_sk; p.acc_sm = sh.acc_sm; p.acc_sn = sh.acc_sn; p.d_sm = sh.d_sm; p.d_sn = sh.d_sn;
  const dim3 grid((unsigned)((p.blocks + 3) / 4), (unsigned)n);
  if (sh.ab_dtype == KAPY_BF16) matmul_table_kernel<Bf16M16><<<grid, 256, 0, s>>>(p);
  else matmul_table_kernel<F16M16><<<grid, 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace kapy
