// matmul_f16acc.hip — kapy.matmul in the arithmetic of the reference's own f16-result instruction.
//
// For f16 operands and an f16 result the reference emits mma.sync ... .f16.f16.f16.f16 (MatmulOpToLLVM.cpp:270-291): the
// accumulator registers hold f16 values, and the K loop of MatmulOpToLLVM.cpp:207-262 hands every instruction's result to the
// next as its accumulator, so the running sum is rounded to f16 once per instruction (8 columns of the lhs for
// mma_m16n8k8_f16, 16 for mma_m16n8k16_f16).  The library's matmul kernels keep fp32 accumulators until the final cast, which
// is more accurate and a different result: a long sum of like-signed terms stalls in f16 (ones: at 32768 with 16 per step)
// where fp32 does not.  This file is the mode that reproduces the reference (kapy_matmul_cfg::accumulate =
// KAPY_ACCUMULATE_ELEMENT): one wavefront per 16 x 16 block of the result, v_mfma_f32_16x16x16_f16 per step with the f16
// accumulator widened on the way in and rounded to nearest even on the way out (for 8 columns per step the upper half of
// the instruction's K is fed zeros).  Inside a step the matrix unit adds in fp32.  Any strides; a mode for checking
// programs against the reference's numbers, not a fast path: operands come straight from global memory, element by element.
#include "common.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

struct F16AccParams {
  const uint16_t *a, *b, *acc;
  uint16_t *d;
  int64_t a_sm, a_sk, b_sk, b_sn, acc_sm, acc_sn, d_sm, d_sn;
  int32_t M, N, K, k_step, tiles_n;
};

// Operand lanes of v_mfma_f32_16x16x16_f16: lane l holds 4 consecutive k (4 * (l / 16) ..) of row (lhs) / column (rhs) l % 16;
// accumulator register v of lane l is element (4 * (l / 16) + v, l % 16) of the block.
__global__ __launch_bounds__(256) void matmul_f16acc_kernel(F16AccParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int32_t m0 = (int32_t)(tile / p.tiles_n) * 16, n0 = (int32_t)(tile % p.tiles_n) * 16;
  if (m0 >= p.M) return;
  const int r = lane & 15, kg = lane >> 4;
  const int32_t m = m0 + r, n = n0 + r;
  uint16_t held[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int32_t row = m0 + 4 * kg + v;
    held[v] = p.acc && row < p.M && n < p.N ? p.acc[row * p.acc_sm + n * p.acc_sn] : (uint16_t)0;
  }
  for (int32_t k0 = 0; k0 < p.K; k0 += p.k_step) {
    f16x4 a, b;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int32_t kk = 4 * kg + e, k = k0 + kk;
      const bool live = kk < p.k_step && k < p.K;
      const uint16_t av = live && m < p.M ? p.a[m * p.a_sm + k * p.a_sk] : (uint16_t)0;
      const uint16_t bv = live && n < p.N ? p.b[k * p.b_sk + n * p.b_sn] : (uint16_t)0;
      a[e] = __builtin_bit_cast(_Float16, av);
      b[e] = __builtin_bit_cast(_Float16, bv);
    }
    f32x4_t c;
#pragma unroll
    for (int v = 0; v < 4; ++v) c[v] = f16_to_f32(held[v]);
    c = __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
#pragma unroll
    for (int v = 0; v < 4; ++v) held[v] = f32_to_f16_rn(c[v]);
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int32_t row = m0 + 4 * kg + v;
    if (row < p.M && n < p.N) p.d[row * p.d_sm + n * p.d_sn] = held[v];
  }
}

}  // namespace

int run_matmul_f16acc(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result, int k_step, hipStream_t s) {
  if (lhs->dtype != KAPY_F16 || rhs->dtype != KAPY_F16 || result->dtype != KAPY_F16 || (acc && acc->dtype != KAPY_F16))
    return fail(KAPY_ERR_UNSUPPORTED, "matmul: accumulation on the element type exists for f16 operands with an f16 accumulator and result (the "
                                      "reference's .f16.f16.f16.f16 instruction); %s x %s -> %s is multiplied with fp32 accumulators only",
                dtype_name(lhs->dtype), dtype_name(rhs->dtype), dtype_name(result->dtype));
  F16AccParams p;
  p.a = (const uint16_t *)view_base(lhs);
  p.b = (const uint16_t *)view_base(rhs);
  p.acc = acc ? (const uint16_t *)view_base(acc) : nullptr;
  p.d = (uint16_t *)view_base(result);
  p.a_sm = lhs->stride0; p.a_sk = lhs->stride1;
  p.b_sk = rhs->stride0; p.b_sn = rhs->stride1;
  p.acc_sm = acc ? acc->stride0 : 0; p.acc_sn = acc ? acc->stride1 : 0;
  p.d_sm = result->stride0; p.d_sn = result->stride1;
  p.M = (int32_t)extent0(lhs); p.K = (int32_t)extent1(lhs); p.N = (int32_t)extent1(rhs);
  p.k_step = k_step;
  if (p.M == 0 || p.N == 0) return KAPY_OK;
  p.tiles_n = (p.N + 15) / 16;
  const int64_t tiles = (int64_t)((p.M + 15) / 16) * p.tiles_n;
  if ((tiles + 3) / 4 > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "matmul: result too large for one launch");
  matmul_f16acc_kernel<<<(unsigned)((tiles + 3) / 4), 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace kapy
