// elementwise_col.hip — softmax of every column of a 16-bit row-major matrix: kapy.reduce along axis 0 (ReduceOpToLLVM.cpp:51-172
// reduces either axis) fused with the elementwise ops around it, for the program
//     st( fptofp_rn( divf( E, reduce_sum0(E) ) ) ),  E = exp( subf( F, reduce_max0(F) ) ),  F = extf( ld x )
// A column does not fit on chip, so the matrix is read twice: one launch leaves every column's maximum M and the sum S of
// exp(x - M) (strips of 256 columns x chunks of rows; a lane keeps a running (m, s) per column and rescales s when m grows;
// the chunks' pairs meet in the library's workspace array and the strip's last workgroup to arrive merges them in chunk
// order), a second launch stores exp(x - M) / S.  Arithmetic in fp32, one rounding to the 16-bit type at the store.
#include <algorithm>

#include "common.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// exp(x) for x <= 0 up to a relative error of about |x| * 1e-7 (the rounding of x * log2 e): the differences from a column's
// maximum that matter are a few tens at most, so this stays some hundred times below the 16-bit rounding of the result.
constexpr float kLog2e = 1.44269504088896341f;
__device__ __forceinline__ float exp_f32(float x) { return __builtin_amdgcn_exp2f(x * kLog2e); }

template <bool BF16>
__device__ __forceinline__ void widen16(u32x4_t v, float (&f)[8]) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    if (BF16) {
      f[2 * w] = bits_f32(v[w] << 16);
      f[2 * w + 1] = bits_f32(v[w] & 0xFFFF0000u);
    } else {
      f[2 * w] = f16_to_f32((uint16_t)v[w]);
      f[2 * w + 1] = f16_to_f32((uint16_t)(v[w] >> 16));
    }
  }
}

struct ColSoftmax {
  const char *x;
  char *out;
  int64_t x_stride0, out_stride0;  // elements
  int32_t rows, cols;
  float *stats;        // [2][cols]: M, then S
  float *lines;        // [chunks][2][cols]
  uint32_t *counters;  // one per strip
};

// (m, s) <- (m, s) merged with (m2, s2): the sum rescaled to the larger maximum.  A pair with s == 0 holds no element.
__device__ __forceinline__ void merge(float &m, float &s, float m2, float s2) {
  if (s2 == 0.f) return;
  if (s == 0.f) { m = m2; s = s2; return; }
  const bool nan = m != m || m2 != m2;
  const float top = nan ? __builtin_nanf("") : fmaxf(m, m2);
  s = s * exp_f32(m - top) + s2 * exp_f32(m2 - top);
  m = top;
}

constexpr int kStrip = 256, kLanesPerRow = 32, kRowGroups = 8;

template <bool BF16>
__global__ __launch_bounds__(256) void col_softmax_stats_kernel(ColSoftmax p, int32_t per_chunk) {
  __shared__ float pm[kRowGroups][kStrip + 1], ps[kRowGroups][kStrip + 1];
  __shared__ uint32_t word;
  const int cl = threadIdx.x % kLanesPerRow, rg = threadIdx.x / kLanesPerRow;
  const int32_t col0 = blockIdx.x * kStrip + cl * 8;
  const int32_t r_begin = blockIdx.y * per_chunk, r_end = min(p.rows, r_begin + per_chunk);
  const int32_t chunks = gridDim.y;
  float m[8], s[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { m[e] = -__builtin_inff(); s[e] = 0.f; }
  if (col0 < p.cols) {
    const char *col = p.x + (int64_t)col0 * 2;
    constexpr int U = 8;
    int32_t r = r_begin + rg;
    for (; r + kRowGroups * (U - 1) < r_end; r += kRowGroups * U) {
      u32x4_t v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = *(const u32x4_t *)(col + (int64_t)(r + kRowGroups * u) * p.x_stride0 * 2);
      float f[U][8];
#pragma unroll
      for (int u = 0; u < U; ++u) widen16<BF16>(v[u], f[u]);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float top = m[e];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          top = fmaxf(top, f[u][e]);   // (a NaN element is skipped here; its exp below makes the sum NaN, which marks the column)
        }
        float acc = s[e] * exp_f32(m[e] - top);
        // (the difference first: folding top * log2 e into a fused multiply-add would put that product's own rounding - half
        // a unit in ITS last place, which for a top of 6e4 is 0.4 %, and another one per chunk - into every term)
#pragma unroll
        for (int u = 0; u < U; ++u) acc += exp_f32(f[u][e] - top);
        s[e] = acc;
        m[e] = top;
      }
    }
    for (; r < r_end; r += kRowGroups) {
      float f[8];
      widen16<BF16>(*(const u32x4_t *)(col + (int64_t)r * p.x_stride0 * 2), f);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float top = fmaxf(m[e], f[e]);
        s[e] = s[e] * exp_f32(m[e] - top) + exp_f32(f[e] - top);
        m[e] = top;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    pm[rg][cl * 8 + e] = m[e];
    ps[rg][cl * 8 + e] = s[e];
  }
  __syncthreads();
  const int32_t col = blockIdx.x * kStrip + threadIdx.x;
  float tm = -__builtin_inff(), ts = 0.f;
  if (col < p.cols) {
#pragma unroll
    for (int g = 0; g < kRowGroups; ++g) merge(tm, ts, pm[g][threadIdx.x], ps[g][threadIdx.x]);
    if (ts != ts) tm = __builtin_nanf("");   // a NaN element made its exp, hence the sum, NaN: the column's maximum is NaN as well
    if (chunks == 1) {
      p.stats[col] = tm;
      p.stats[p.cols + col] = ts;
    } else {
      float *line = p.lines + (int64_t)blockIdx.y * 2 * p.cols;
      __hip_atomic_store((uint32_t *)(line + col), f32_bits(tm), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store((uint32_t *)(line + p.cols + col), f32_bits(ts), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (chunks == 1) return;
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this lane's partial results have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) word = __hip_atomic_fetch_add(p.counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (word != (uint32_t)chunks - 1) return;
  // the strip's last workgroup: the chunks' pairs in chunk order, eight pairs in flight per lane
  if (col < p.cols) {
    tm = -__builtin_inff();
    ts = 0.f;
    for (int32_t c0 = 0; c0 < chunks; c0 += 8) {
      float lm[8], lsum[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float *line = p.lines + (int64_t)min(c0 + u, chunks - 1) * 2 * p.cols;
        lm[u] = bits_f32(__hip_atomic_load((const uint32_t *)(line + col), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        lsum[u] = bits_f32(__hip_atomic_load((const uint32_t *)(line + p.cols + col), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (c0 + u < chunks) merge(tm, ts, lm[u], lsum[u]);
    }
    if (ts != ts) tm = __builtin_nanf("");
    p.stats[col] = tm;
    p.stats[p.cols + col] = ts;
  }
  if (threadIdx.x == 0) __hip_atomic_store(p.counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// y = exp(x - M) / S: a lane owns 8 consecutive columns, keeps their M and 1 / S in registers and walks `rows_per_wg` rows,
// two in flight.  The quotient is e * (1 / S): within two fp32 ulps of e / S, far inside the 16-bit rounding that follows.
template <bool BF16>
__global__ __launch_bounds__(256) void col_softmax_apply_kernel(ColSoftmax p, int32_t rows_per_wg) {
  const int32_t col0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (col0 >= p.cols) return;
  float M[8], R[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    M[e] = p.stats[col0 + e];
    R[e] = __builtin_amdgcn_rcpf(p.stats[p.cols + col0 + e]);
  }
  const int32_t r_begin = blockIdx.y * rows_per_wg, r_end = min(p.rows, r_begin + rows_per_wg);
  const char *col = p.x + (int64_t)col0 * 2;
  char *dst = p.out + (int64_t)col0 * 2;
  for (int32_t r = r_begin; r < r_end; r += 2) {
    u32x4_t v[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
      if (r + u < r_end) v[u] = __builtin_nontemporal_load((const u32x4_t *)(col + (int64_t)(r + u) * p.x_stride0 * 2));
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (r + u >= r_end) break;
      float f[8];
      widen16<BF16>(v[u], f);
      u32x4_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        f[e] = exp_f32(f[e] - M[e]) * R[e];   // (S >= 1 and finite, or NaN, which 1 / S and the product hand on)
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) o[w] = BF16 ? pack2_bf16_rn(f[2 * w], f[2 * w + 1]) : pack2_f16_rn(f[2 * w], f[2 * w + 1]);
      __builtin_nontemporal_store(o, (u32x4_t *)(dst + (int64_t)(r + u) * p.out_stride0 * 2));
    }
  }
}

}  // namespace

int run_column_softmax(const kapy_global *x, const kapy_global *out, hipStream_t s) {
  const int64_t m = extent0(out), n = extent1(out);
  if ((x->dtype != KAPY_F16 && x->dtype != KAPY_BF16) || out->dtype != x->dtype) return 0;
  if (extent0(x) != m || extent1(x) != n || x->stride1 != 1 || out->stride1 != 1 || n % 8 != 0 || m < 64 || n < 8) return 0;
  if (vector_bytes(x, 1) != 16 || vector_bytes(out, 1) != 16) return 0;
  if (m >= (int64_t(1) << 31) || n >= (int64_t(1) << 30)) return 0;
  size_t bytes = 0;
  uint32_t *counters = nullptr;
  float *lines = reduce_scratch_lines(&bytes, &counters);
  if (!lines) return 0;
  // [M, S per column][chunks x (M, S) lines]
  const int64_t floats = (int64_t)(bytes / sizeof(float));
  const int64_t strips = (n + kStrip - 1) / kStrip, want = 4 * (int64_t)device_cus();
  if (strips > 4096 || 4 * n > floats) return 0;
  int64_t chunks = std::max<int64_t>(1, std::min<int64_t>({(want + strips - 1) / strips, m / 64, 256, floats / (2 * n) - 1}));
  const int32_t per_chunk = (int32_t)((m + chunks - 1) / chunks);
  chunks = (m + per_chunk - 1) / per_chunk;
  ColSoftmax p;
  p.x = view_base(x);
  p.out = (char *)view_base(out);
  p.x_stride0 = x->stride0;
  p.out_stride0 = out->stride0;
  p.rows = (int32_t)m;
  p.cols = (int32_t)n;
  p.stats = lines;
  p.lines = lines + 2 * n;
  p.counters = counters;
  const bool bf16 = x->dtype == KAPY_BF16;
  dim3 grid((unsigned)strips, (unsigned)chunks);
  if (bf16) col_softmax_stats_kernel<true><<<grid, 256, 0, s>>>(p, per_chunk);
  else col_softmax_stats_kernel<false><<<grid, 256, 0, s>>>(p, per_chunk);
  const int64_t col_blocks = (n / 8 + 255) / 256;
  int64_t row_blocks = std::max<int64_t>(1, std::min<int64_t>((8 * (int64_t)device_cus() + col_blocks - 1) / col_blocks, (m + 15) / 16));
  const int32_t rows_per_wg = (int32_t)((((m + row_blocks - 1) / row_blocks) + 1) / 2 * 2);
  row_blocks = (m + rows_per_wg - 1) / rows_per_wg;
  dim3 grid2((unsigned)col_blocks, (unsigned)row_blocks);
  if (bf16) col_softmax_apply_kernel<true><<<grid2, 256, 0, s>>>(p, rows_per_wg);
  else col_softmax_apply_kernel<false><<<grid2, 256, 0, s>>>(p, rows_per_wg);
  KAPY_HIP_CHECK(hipGetLastError());
  return 1;
}

}  // namespace kapy
