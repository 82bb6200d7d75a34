// matmul_f8.hip — kapy.matmul on OCP fp8 operands (E4M3FN / E5M2, mixable) with fp32 accumulate,
// and the W8A8 form with fp32 row/column scales applied in the epilogue.
//
// Reference: MatmulImplWay::MMA_M16N8K16_F8 (lib/Dialect/Kapy/IR/Kapy.cpp:545-564 verifier,
// MatmulOpToLLVM.cpp:269-311 mma.sync.m16n8k16 e4m3/e5m2 strings, operand layouts
// LayoutUtils.cpp:141-147) followed by mulf with broadcast scales and fptofp rn.
// gfx950: v_mfma_scale_f32_16x16x128_f8f6f4 with unit E8M0 block scales (2^0); the operand format
// selectors (cbsz / blgp: 0 = E4M3, 1 = E5M2) carry kapy's mixed-f8 rule.
//
//   skinny_kernel  few rows of lhs (decode shape): HBM-bound on the weight.  One workgroup per 16*NG
//                  output columns, its 8 wavefronts split K; every weight byte is read once,
//                  straight from global memory into the MFMA operand registers (each lane's 32
//                  K-contiguous bytes are exactly its operand), partial sums meet in LDS.
//   naive_kernel   any strides / ragged K: one output element per lane, software decode.
#include "common.hpp"
#include "layout.hpp"
#include "matmul_params.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct F8Params {
  const uint8_t *a, *b;
  const char *acc;
  char *d;
  const float *row_scale, *col_scale;
  int64_t a_sm, a_sk, b_sn, b_sk, acc_sm, acc_sn, d_sm, d_sn;
  int32_t M, N, K;
  int32_t a_dtype, b_dtype, acc_dtype, d_dtype, rz;
};

__device__ __forceinline__ void finish(const F8Params &p, int32_t m, int32_t n, float v) {
  if (m >= p.M || n >= p.N) return;
  if (p.row_scale) v *= __fmul_rn(p.row_scale[m], p.col_scale[n]);
  if (p.acc_dtype >= 0) v += load_as_f32(p.acc, p.acc_dtype, m * p.acc_sm + n * p.acc_sn);
  int64_t idx = m * p.d_sm + n * p.d_sn;
  switch (p.d_dtype) {
  case KAPY_F32: ((float *)p.d)[idx] = v; break;
  case KAPY_F16: ((uint16_t *)p.d)[idx] = p.rz ? f32_to_f16_rz(v) : f32_to_f16_rn(v); break;
  default: ((uint16_t *)p.d)[idx] = p.rz ? f32_to_bf16_rz(v) : f32_to_bf16_rn(v); break;
  }
}

__global__ __launch_bounds__(256) void naive_kernel(F8Params p) {
  int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= (int64_t)p.M * p.N) return;
  int32_t m = (int32_t)(t / p.N), n = (int32_t)(t - (int64_t)m * p.N);
  float s = 0.f;
  for (int32_t k = 0; k < p.K; ++k) {
    float x = load_as_f32(p.a, p.a_dtype, m * p.a_sm + k * p.a_sk);
    float y = load_as_f32(p.b, p.b_dtype, n * p.b_sn + k * p.b_sk);
    s = __fmaf_rn(x, y, s);
  }
  finish(p, m, n, s);
}

// 32 K-contiguous bytes of one row/column as the 8-dword MFMA operand; rows past the end read zero.
__device__ __forceinline__ i32x8 load_k32(const uint8_t *base, int64_t stride, int32_t row, int32_t rows, int32_t k) {
  i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
  if (row < rows) {
    const i32x4 *ptr = (const i32x4 *)(base + row * stride + k);
    i32x4 lo = ptr[0], hi = ptr[1];
    r = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }
  return r;
}

// Skinny kernel.  Workgroup = 8 wavefronts = 8 contiguous K ranges, NG groups of 16 output columns.
// A wave first requests everything it will multiply in a chunk of CH K-steps - the weight bytes of
// its NG column groups and the activation bytes they share - and only then starts the matrix
// instructions, so that a CU keeps >100 KiB of HBM reads in flight with only 8 resident waves.
#ifndef KAPY_SKINNY_NG
#define KAPY_SKINNY_NG 1
#endif
#ifndef KAPY_SKINNY_CH
#define KAPY_SKINNY_CH 8
#endif
constexpr int kSkinnyWaves = 8;
template <int A_FMT, int B_FMT, int NG, int CH>
__global__ __launch_bounds__(64 * kSkinnyWaves) void skinny_kernel(F8Params p) {
  __shared__ float partial[kSkinnyWaves][NG][16][16 + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int32_t n0 = blockIdx.x * 16 * NG, m0 = blockIdx.y * 16;
  const int32_t row = lane & 15, kq = (lane >> 4) * 32;  // this lane's row/column and its 32-byte K quarter
  const int32_t steps = p.K / 128, per_wave = (steps + kSkinnyWaves - 1) / kSkinnyWaves;
  const int32_t s_begin = wave * per_wave, s_end = min(steps, s_begin + per_wave);
  f32x4 acc[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int32_t s = s_begin; s < s_end; s += CH) {
    i32x8 bw[NG][CH], aw[CH];
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const bool live = s + u < s_end;
#pragma unroll
      for (int g = 0; g < NG; ++g) bw[g][u] = load_k32(p.b, p.b_sn, n0 + 16 * g + row, live ? p.N : 0, (s + u) * 128 + kq);
    }
#pragma unroll
    for (int u = 0; u < CH; ++u) aw[u] = load_k32(p.a, p.a_sm, m0 + row, s + u < s_end ? p.M : 0, (s + u) * 128 + kq);
#pragma unroll
    for (int u = 0; u < CH; ++u)
#pragma unroll
      for (int g = 0; g < NG; ++g)
        acc[g] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(aw[u], bw[g][u], acc[g], A_FMT, B_FMT, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  }
  // accumulator register v of lane l: row 4*(l/16) + v, column l%16
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int v = 0; v < 4; ++v) partial[wave][g][4 * (lane >> 4) + v][lane & 15] = acc[g][v];
  __syncthreads();
  for (int e = threadIdx.x; e < NG * 256; e += 64 * kSkinnyWaves) {
    const int g = e >> 8, m = (e >> 4) & 15, n = e & 15;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kSkinnyWaves; ++w) sum += partial[w][g][m][n];
    finish(p, m0 + m, n0 + 16 * g + n, sum);
  }
}

int fmt_of(int dtype) { return dtype == KAPY_F8E5M2 ? 1 : 0; }

}  // namespace

int matmul_f8(const kapy_global *a, const kapy_global *b, const float *row_scale, const float *col_scale, const kapy_global *acc,
              const kapy_global *result, const kapy_matmul_cfg *cfg, hipStream_t s) {
  F8Params p;
  p.a = (const uint8_t *)view_base(a);
  p.b = (const uint8_t *)view_base(b);
  p.acc = acc ? view_base(acc) : nullptr;
  p.d = (char *)view_base(result);
  p.row_scale = row_scale;
  p.col_scale = col_scale;
  p.a_sm = a->stride0; p.a_sk = a->stride1;
  p.b_sk = b->stride0; p.b_sn = b->stride1;
  p.acc_sm = acc ? acc->stride0 : 0; p.acc_sn = acc ? acc->stride1 : 0;
  p.d_sm = result->stride0; p.d_sn = result->stride1;
  p.M = (int32_t)extent0(a); p.K = (int32_t)extent1(a); p.N = (int32_t)extent1(b);
  p.a_dtype = a->dtype; p.b_dtype = b->dtype;
  p.acc_dtype = acc ? acc->dtype : -1;
  p.d_dtype = result->dtype;
  p.rz = cfg && cfg->rmode == KAPY_RZ;
  if (p.M == 0 || p.N == 0) return KAPY_OK;
  bool k_contig = p.a_sk == 1 && p.b_sk == 1 && vector_bytes(a, 1) == 16 && vector_bytes(b, 0) == 16 && p.K % 128 == 0 && p.K > 0;
  // Many rows: the tiled LDS-direct kernel (MFMA-bound).  Few rows: the skinny kernel (HBM-bound).
  if (k_contig && p.M >= 128 && !acc && (result->dtype == KAPY_BF16 || result->dtype == KAPY_F16 || result->dtype == KAPY_F32)) {
    GemmParams g;
    g.a = (const char *)p.a; g.b = (const char *)p.b; g.acc = nullptr; g.d = p.d;
    g.row_scale = row_scale; g.col_scale = col_scale;
    g.a_sm = p.a_sm; g.a_sk = 1; g.b_sn = p.b_sn; g.b_sk = 1;
    g.acc_sm = g.acc_sn = 0; g.d_sm = p.d_sm; g.d_sn = p.d_sn;
    g.M = p.M; g.N = p.N; g.K = p.K;
    g.acc_dtype = -1; g.d_dtype = p.d_dtype; g.rz = p.rz; g.tiles_m = g.tiles_n = 0;
    int rc = matmul_f8_tiled(g, fmt_of(a->dtype), fmt_of(b->dtype), s);
    if (rc != KAPY_ERR_UNSUPPORTED) return rc;
  }
  if (k_contig) {
    constexpr int NG = KAPY_SKINNY_NG, CH = KAPY_SKINNY_CH;
    dim3 grid((unsigned)((p.N + 16 * NG - 1) / (16 * NG)), (unsigned)((p.M + 15) / 16));
    if (grid.y <= 65535) {
      int fa = fmt_of(a->dtype), fb = fmt_of(b->dtype);
      if (fa == 0 && fb == 0) skinny_kernel<0, 0, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      else if (fa == 0) skinny_kernel<0, 1, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      else if (fb == 0) skinny_kernel<1, 0, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      else skinny_kernel<1, 1, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      KAPY_HIP_CHECK(hipGetLastError());
      return KAPY_OK;
    }
  }
  int64_t total = (int64_t)p.M * p.N;
  naive_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace kapy

using namespace kapy;

extern "C" int kapy_matmul_scaled_f8(const kapy_global *a8, const kapy_global *w8, const float *row_scale, const float *col_scale,
                                     const kapy_global *result, const kapy_matmul_cfg *cfg, void *stream) {
  int rc = check_global(a8, "matmul lhs");
  if (!rc) rc = check_global(w8, "matmul rhs");
  if (!rc) rc = check_global(result, "matmul result");
  if (rc) return rc;
  if (!row_scale || !col_scale) return fail(KAPY_ERR_INVALID, "matmul_scaled_f8: null scale array");
  if (!is_f8(a8->dtype) || !is_f8(w8->dtype))
    return fail(KAPY_ERR_VERIFY, "matmul: mma f8 operands must have f8E4M3 or f8E5M2 element type");
  if (extent1(a8) != extent0(w8))
    return fail(KAPY_ERR_VERIFY, "matmul: number of columns of lhs must be equal to number of rows of rhs");
  if (extent0(result) != extent0(a8))
    return fail(KAPY_ERR_VERIFY, "matmul: number of rows of acc must be equal to number of rows of lhs");
  if (extent1(result) != extent1(w8))
    return fail(KAPY_ERR_VERIFY, "matmul: number of columns of acc must be equal to number of columns of rhs");
  if (result->dtype != KAPY_F16 && result->dtype != KAPY_BF16 && result->dtype != KAPY_F32)
    return fail(KAPY_ERR_VERIFY, "matmul: result must have f16, bf16 or f32 element type");
  for (const kapy_global *g : {a8, w8, result})
    if (g->start0 < 0 || g->start1 < 0) return fail(KAPY_ERR_INVALID, "matmul: negative view start");
  if (cfg && cfg->rmode != KAPY_RN && cfg->rmode != KAPY_RZ) return fail(KAPY_ERR_INVALID, "matmul: unknown rounding mode %d", cfg->rmode);
  rc = ensure_device();
  if (rc) return rc;
  return matmul_f8(a8, w8, row_scale, col_scale, nullptr, result, cfg, (hipStream_t)stream);
}
