// elementwise_row.hip — the row machine: elementwise programs with a reduce along the rows (softmax,
// layer norm, RMS norm ...), one pass over HBM with each row resident on chip.  kapy.reduce with an addf /
// maximumf combiner (Ops.td:441-457, ReduceOpToLLVM.cpp:51-172) and the kapy.broadcast of its result
// (BroadcastOpToLLVM.cpp:25-52) fused with the elementwise ops around them.
//
// A workgroup owns one row.  Lane t holds CH chunks of 8 elements, chunk c at vector c*THREADS + t of the
// row.  Values come in two kinds: row values (one fp32 per element: up to NS stack slots of CH*8 registers)
// and per-row values (a reduce's result, a constant, a [m x 1] operand and whatever is computed from
// those: one register each on a second stack of four).  The host compiles the program's DAG into steps
// that name their slots statically, so no register is indexed at run time; a row value used again while
// it still sits lower on the stack is copied from there, one that has been overwritten in between is
// parked in LDS by its first evaluation and read back by the lane that wrote it.
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <functional>
#include <vector>

#include "ew_row_machine.hpp"

namespace kapy {

// the kernels that carry the general step (elementwise_row_narrow.hip, elementwise_row_any.hip)
int launch_row_narrow(const StackProgram &P, int ns, hipStream_t s);
int launch_row_any(const StackProgram &P, int ns, hipStream_t s);

namespace {

// ---------------------------------------------------------------------------------------------
// The two row programs that have names get kernels of their own (as act(x*s+bias) does among the plain elementwise
// programs): softmax and the layer / RMS norm family, on 16-bit operands with fp32 arithmetic, step for step what the
// row machine's light kernel would compute, without its decoding.
struct FusedRow {
  const char *x, *gamma, *beta;  // gamma / beta: [1 x n] rows or null
  char *out;
  int64_t x_stride0, out_stride0;
  int32_t rows, vec_per_row;
  int32_t centre;  // norm: subtract the mean first (layer norm) or not (RMS norm)
  float inv_n, eps;
};

template <int THREADS, bool MAX>
__device__ __forceinline__ float row_fold(float acc, float *red) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float other = __shfl_xor(acc, off, 64);
    acc = MAX ? max_nan(acc, other) : acc + other;
  }
  if (THREADS > 64) {
    constexpr int WAVES = THREADS / 64;
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    acc = red[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) acc = MAX ? max_nan(acc, red[w]) : acc + red[w];
  }
  return acc;
}

template <int CH, int THREADS, bool STREAM>
__device__ __forceinline__ void row_fetch(const char *base, int32_t vpr, u32x4 (&raw)[CH]) {
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int32_t jv = c * THREADS + threadIdx.x;
    raw[c] = u32x4{0, 0, 0, 0};
    if (jv < vpr) raw[c] = STREAM ? __builtin_nontemporal_load((const u32x4 *)(base + (int64_t)jv * 16)) : *(const u32x4 *)(base + (int64_t)jv * 16);
  }
}

// Both kernels walk rows blockIdx.x, blockIdx.x + gridDim.x, ... and ask for the next row's 16 bytes per chunk before they
// work on the current one, so that a workgroup always has a load in flight.  The two exchange areas of a row's two
// reduces are safe to reuse from row to row: a wave can write one again only after the barrier of the other, which every
// wave reaches after it has read the first.
// WALK = false: one row per workgroup and as many workgroups as rows (the host's choice for many rows of up to 8192
// elements: the dispatcher then keeps every CU full to the end and workgroups drift into different phases, which is worth
// more than the load in flight across rows - 1024 elements 49 -> 44 us, 8192 elements 47.7 -> 46.3 us for 128 MiB).
template <int CH, int THREADS, bool WALK>
__global__ __launch_bounds__(THREADS) void softmax_kernel(FusedRow p, int dtype) {
  __shared__ float red[2][16];
  u32x4 raw[CH];
  row_fetch<CH, THREADS, true>(p.x + (int64_t)blockIdx.x * p.x_stride0 * 2, p.vec_per_row, raw);
  for (int32_t i = blockIdx.x; i < p.rows; i += gridDim.x) {
    float f[CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) widen16x8(raw[c], dtype, f[c]);
    if (WALK && i + (int32_t)gridDim.x < p.rows) row_fetch<CH, THREADS, true>(p.x + (int64_t)(i + gridDim.x) * p.x_stride0 * 2, p.vec_per_row, raw);
    // (a NaN is skipped by the maximum; its exponential below is NaN, so is the row's sum, and with it every quotient of the
    // row - what a NaN maximum would have made of them)
    float m = -__builtin_inff();
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (c * THREADS + (int)threadIdx.x < p.vec_per_row) {
#pragma unroll
        for (int e = 0; e < 8; ++e) m = fmaxf(m, f[c][e]);
      }
    m = row_fold<THREADS, true>(m, red[0]);
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const bool active = c * THREADS + (int)threadIdx.x < p.vec_per_row;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // exp(x) = 2^hi * (1 + lo*ln2) with hi + lo = x*log2(e), lo the product's rounding error: about 1 ulp of fp32
        // for the x <= 0 that reach here.  A NaN passes through every step; x = -inf gives hi = -inf, 2^hi = 0, and
        // needs lo, which would be inf - inf, set aside.
        const float x = __fsub_rn(f[c][e], m);
        const float hi = x * 1.44269504088896341f;
        float lo = __builtin_fmaf(x, 1.44269504088896341f, -hi);
        lo = !(x <= -3e38f) ? lo : 0.f;
        const float pw = __builtin_amdgcn_exp2f(hi);
        f[c][e] = __builtin_fmaf(pw, lo * 0.693147180559945309f, pw);
      }
      if (active) sum += ((f[c][0] + f[c][1]) + (f[c][2] + f[c][3])) + ((f[c][4] + f[c][5]) + (f[c][6] + f[c][7]));
    }
    sum = row_fold<THREADS, false>(sum, red[1]);
    const float rcp = __builtin_amdgcn_rcpf(sum);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // e / sum as e*(1/sum) corrected by the remainder: the correctly rounded quotient (e <= 1 <= sum <= n here; a
        // NaN in either is a NaN in both forms)
        const float q = f[c][e] * rcp;
        const float rem = __builtin_fmaf(-q, sum, f[c][e]);
        f[c][e] = __builtin_fmaf(rem, rcp, q);
      }
      const int32_t jv = c * THREADS + threadIdx.x;
      if (jv < p.vec_per_row) store8<true>(p.out, dtype, (int64_t)i * p.out_stride0 + (int64_t)jv * 8, f[c]);
    }
    if (!WALK) break;
  }
}

template <int CH, int THREADS>
__global__ __launch_bounds__(THREADS) void norm_kernel(FusedRow p, int dtype) {
  __shared__ float red[2][16];
  // gamma and beta are the same for every row: each lane keeps its own 16-byte pieces of them in LDS (its private
  // corner of it: written once, read back by the same lane, no barrier) rather than in registers the row needs
  extern __shared__ u32x4 stash[];
  u32x4 raw[CH];
  row_fetch<CH, THREADS, true>(p.x + (int64_t)blockIdx.x * p.x_stride0 * 2, p.vec_per_row, raw);
  {
    u32x4 gb[CH];
    if (p.gamma) {
      row_fetch<CH, THREADS, false>(p.gamma, p.vec_per_row, gb);
#pragma unroll
      for (int c = 0; c < CH; ++c) stash[c * THREADS + threadIdx.x] = gb[c];
    }
    if (p.beta) {
      row_fetch<CH, THREADS, false>(p.beta, p.vec_per_row, gb);
#pragma unroll
      for (int c = 0; c < CH; ++c) stash[(CH + c) * THREADS + threadIdx.x] = gb[c];
    }
  }
  for (int32_t i = blockIdx.x; i < p.rows; i += gridDim.x) {
    float f[CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) widen16x8(raw[c], dtype, f[c]);
    if (i + (int32_t)gridDim.x < p.rows) row_fetch<CH, THREADS, true>(p.x + (int64_t)(i + gridDim.x) * p.x_stride0 * 2, p.vec_per_row, raw);
    if (p.centre) {
      float sum = -0.f;  // the identity of addition: a row of only -0 has mean -0
#pragma unroll
      for (int c = 0; c < CH; ++c)
        if (c * THREADS + (int)threadIdx.x < p.vec_per_row) sum += ((f[c][0] + f[c][1]) + (f[c][2] + f[c][3])) + ((f[c][4] + f[c][5]) + (f[c][6] + f[c][7]));
      const float mean = __fmul_rn(row_fold<THREADS, false>(sum, red[0]), p.inv_n);
#pragma unroll
      for (int c = 0; c < CH; ++c)
#pragma unroll
        for (int e = 0; e < 8; ++e) f[c][e] = __fsub_rn(f[c][e], mean);
    }
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (c * THREADS + (int)threadIdx.x < p.vec_per_row) {
        float s8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) s8[e] = __fmul_rn(f[c][e], f[c][e]);
        sq += ((s8[0] + s8[1]) + (s8[2] + s8[3])) + ((s8[4] + s8[5]) + (s8[6] + s8[7]));
      }
    const float var = __fmul_rn(row_fold<THREADS, false>(sq, red[1]), p.inv_n);
    const float rstd = __builtin_amdgcn_rsqf(__fadd_rn(var, p.eps));
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int32_t jv = c * THREADS + threadIdx.x;
      const bool active = jv < p.vec_per_row;
      float g[8], b[8];
      if (p.gamma) widen16x8(stash[c * THREADS + threadIdx.x], dtype, g);
      if (p.beta) widen16x8(stash[(CH + c) * THREADS + threadIdx.x], dtype, b);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float r = __fmul_rn(f[c][e], rstd);
        if (p.gamma) r = __fmul_rn(r, g[e]);
        if (p.beta) r = __fadd_rn(r, b[e]);
        f[c][e] = r;
      }
      if (active) store8<true>(p.out, dtype, (int64_t)i * p.out_stride0 + (int64_t)jv * 8, f[c]);
    }
  }
}

// Rows of up to 32 vectors (256 elements): a wave holds 64 / GROUP rows at a time, GROUP lanes each (GROUP = 8, 16, 32: the
// next power of two from the row's vectors), so that short rows do not leave most lanes of a wave idle (one wave per row of
// 64 elements: 8 lanes of 64 at work).  A row's reduces are butterflies inside its group of lanes; no LDS, no barrier.
template <int GROUP, bool MAX>
__device__ __forceinline__ float group_fold(float acc) {
#pragma unroll
  for (int off = GROUP / 2; off >= 1; off >>= 1) {
    const float other = __shfl_xor(acc, off, 64);
    acc = MAX ? max_nan(acc, other) : acc + other;
  }
  return acc;
}

template <int GROUP>
__global__ __launch_bounds__(256) void softmax_short_kernel(FusedRow p, int dtype) {
  const int64_t i = (int64_t)blockIdx.x * (256 / GROUP) + threadIdx.x / GROUP;
  const int32_t jv = threadIdx.x % GROUP;
  const bool active = i < p.rows && jv < p.vec_per_row;
  u32x4 raw = {0, 0, 0, 0};
  if (active) raw = __builtin_nontemporal_load((const u32x4 *)(p.x + (i * p.x_stride0 + (int64_t)jv * 8) * 2));
  float f[8];
  widen16x8(raw, dtype, f);
  float m = -__builtin_inff();
  bool any_nan = false;
  if (active) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      m = fmaxf(m, f[e]);
      any_nan |= f[e] != f[e];
    }
  }
  m = group_fold<GROUP, true>(any_nan ? __builtin_nanf("") : m);
#pragma unroll
  for (int e = 0; e < 8; ++e) {  // (the same steps as softmax_kernel, which explains them)
    const float x = __fsub_rn(f[e], m);
    const float hi = x * 1.44269504088896341f;
    float lo = __builtin_fmaf(x, 1.44269504088896341f, -hi);
    lo = !(x <= -3e38f) ? lo : 0.f;
    const float pw = __builtin_amdgcn_exp2f(hi);
    f[e] = __builtin_fmaf(pw, lo * 0.693147180559945309f, pw);
  }
  float sum = active ? ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7])) : 0.f;
  sum = group_fold<GROUP, false>(sum);
  const float rcp = __builtin_amdgcn_rcpf(sum);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float q = f[e] * rcp;
    const float rem = __builtin_fmaf(-q, sum, f[e]);
    f[e] = __builtin_fmaf(rem, rcp, q);
  }
  if (active) store8<true>(p.out, dtype, i * p.out_stride0 + (int64_t)jv * 8, f);
}

template <int GROUP>
__global__ __launch_bounds__(256) void norm_short_kernel(FusedRow p, int dtype) {
  const int64_t i = (int64_t)blockIdx.x * (256 / GROUP) + threadIdx.x / GROUP;
  const int32_t jv = threadIdx.x % GROUP;
  const bool active = i < p.rows && jv < p.vec_per_row;
  u32x4 raw = {0, 0, 0, 0}, graw = {0, 0, 0, 0}, braw = {0, 0, 0, 0};
  if (active) raw = __builtin_nontemporal_load((const u32x4 *)(p.x + (i * p.x_stride0 + (int64_t)jv * 8) * 2));
  if (active && p.gamma) graw = *(const u32x4 *)(p.gamma + (int64_t)jv * 16);
  if (active && p.beta) braw = *(const u32x4 *)(p.beta + (int64_t)jv * 16);
  float f[8];
  widen16x8(raw, dtype, f);
  if (p.centre) {
    float sum = active ? ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7])) : -0.f;
    const float mean = __fmul_rn(group_fold<GROUP, false>(sum), p.inv_n);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = __fsub_rn(f[e], mean);
  }
  float sq = 0.f;
  if (active) {
    float s8[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) s8[e] = __fmul_rn(f[e], f[e]);
    sq = ((s8[0] + s8[1]) + (s8[2] + s8[3])) + ((s8[4] + s8[5]) + (s8[6] + s8[7]));
  }
  const float var = __fmul_rn(group_fold<GROUP, false>(sq), p.inv_n);
  const float rstd = __builtin_amdgcn_rsqf(__fadd_rn(var, p.eps));
  float g[8], b[8];
  widen16x8(graw, dtype, g);
  widen16x8(braw, dtype, b);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float r = __fmul_rn(f[e], rstd);
    if (p.gamma) r = __fmul_rn(r, g[e]);
    if (p.beta) r = __fadd_rn(r, b[e]);
    f[e] = r;
  }
  if (active) store8<true>(p.out, dtype, i * p.out_stride0 + (int64_t)jv * 8, f);
}

template <int GROUP>
int launch_short_row(const FusedRow &p, int dtype, bool softmax, hipStream_t s) {
  const int64_t groups = ((int64_t)p.rows + 256 / GROUP - 1) / (256 / GROUP);
  if (softmax) softmax_short_kernel<GROUP><<<dim3((unsigned)groups), 256, 0, s>>>(p, dtype);
  else norm_short_kernel<GROUP><<<dim3((unsigned)groups), 256, 0, s>>>(p, dtype);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int launch_fused_row(const FusedRow &p, int dtype, bool softmax, hipStream_t s) {
  const int vpr = p.vec_per_row;
  if (vpr <= 32 && p.rows >= 64) return vpr <= 8 ? launch_short_row<8>(p, dtype, softmax, s) : vpr <= 16 ? launch_short_row<16>(p, dtype, softmax, s) : launch_short_row<32>(p, dtype, softmax, s);
  // one wave per row up to 256 vectors for softmax, up to 128 for the norms (whose 64-lane build with four chunks per lane
  // needs more registers than the occupancy it is meant to buy: 2048 elements 61 -> 50 us on 256 lanes)
  const int threads = vpr <= (softmax ? 256 : 128) ? 64 : vpr <= 1024 ? 256 : 1024;
  const int ch = (vpr + threads - 1) / threads;
  // as many workgroups as are resident at once; each walks its share of the rows
#define KAPY_FUSED(CH_, TH_)                                                           \
  do {                                                                                 \
    int per_cu = 1;                                                                    \
    const size_t lds = softmax ? 0 : (size_t)2 * CH_ * TH_ * 16;                       \
    if (lds > 48 * 1024) KAPY_HIP_CHECK(hipFuncSetAttribute((const void *)norm_kernel<CH_, TH_>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
    if (softmax) KAPY_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, softmax_kernel<CH_, TH_, true>, TH_, 0)); \
    else KAPY_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, norm_kernel<CH_, TH_>, TH_, lds)); \
    const int64_t resident = (int64_t)device_cus() * (per_cu > 0 ? per_cu : 1);        \
    dim3 grid((unsigned)(p.rows < resident ? p.rows : resident));                      \
    if (softmax && TH_ <= 256 && p.rows >= 4 * resident) softmax_kernel<CH_, TH_, false><<<dim3((unsigned)p.rows), TH_, 0, s>>>(p, dtype); \
    else if (softmax) softmax_kernel<CH_, TH_, true><<<grid, TH_, 0, s>>>(p, dtype);   \
    else norm_kernel<CH_, TH_><<<grid, TH_, lds, s>>>(p, dtype);                       \
  } while (0)
#define KAPY_FUSED_CH(TH_)                                                             \
  do {                                                                                 \
    if (ch == 1) KAPY_FUSED(1, TH_); else if (ch == 2) KAPY_FUSED(2, TH_); else KAPY_FUSED(4, TH_); \
  } while (0)
  if (threads == 64) KAPY_FUSED_CH(64);
  else if (threads == 256) KAPY_FUSED_CH(256);
  else KAPY_FUSED_CH(1024);
#undef KAPY_FUSED_CH
#undef KAPY_FUSED
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

// ---------------------------------------------------------------------------------------------
// Host: the program's DAG compiled into steps.
struct RowBuilder {
  struct N {
    int op, a = -1, b = -1, c = -1, dtype = -1, rmode = KAPY_RN, input = -1;
    float imm = 0.f;
  };
  std::vector<N> nodes;
  std::vector<char> uniform;  // one value per row?
  std::vector<int> uses, need;
  int stored = -1;
  StackProgram *P = nullptr;
  int out_dtype = 0;

  // per run
  bool full_first = false;  // a row operand before its per-row partner (keeps the row operand on the stack for the partner's own use of it)
  bool dry = true, ok = true;
  int count = 0, max_slot = 0, n_tmps = 0;
  int holder[3], holder_u[kUSlots];
  std::vector<int> tmp_of;
  std::vector<char> parked, read_back;

  void push(int op, int a, int dtype, int rmode, int slot, float imm, int flags = 0, int k = 0) {
    if (count >= kMaxPost || slot > 2 || k >= kUSlots) { ok = false; return; }
    max_slot = std::max(max_slot, slot);
    P->post[count++] = PostOp{(int16_t)op, (int16_t)a, (int16_t)dtype, (int16_t)rmode, slot | flags | (k << 8), imm};
  }
  static int reversed(int op) { return op == KAPY_EW_SUBF ? kRevSub : op == KAPY_EW_DIVF ? kRevDiv : op; }
  bool is_reduce(int id) const { return nodes[id].op == KAPY_EW_REDUCE_SUM || nodes[id].op == KAPY_EW_REDUCE_MAX; }

  // row slots an expression needs (a per-row expression needs them only while its reduces run)
  void compute_need() {
    need.assign(nodes.size(), 0);
    for (size_t id = 0; id < nodes.size(); ++id) {
      const N &n = nodes[id];
      auto nf = [&](int x) { return std::max(need[x], 1); };
      if (uniform[id]) {
        if (is_reduce((int)id)) need[id] = nf(n.a);
        else need[id] = std::max(n.a >= 0 ? need[n.a] : 0, std::max(n.b >= 0 ? need[n.b] : 0, n.c >= 0 ? need[n.c] : 0));
      } else if (n.op == KAPY_EW_LD_GLOBAL) need[id] = 1;
      else if (n.op == KAPY_EW_FMA) need[id] = std::max(nf(n.a), std::max(nf(n.b) + 1, nf(n.c) + 2));
      else if (n.b >= 0) {
        if (n.a == n.b) need[id] = nf(n.a);
        else if (uniform[n.a] || uniform[n.b]) {
          const int f = uniform[n.a] ? n.b : n.a, un = uniform[n.a] ? n.a : n.b;
          need[id] = std::max(nf(f), need[un]);  // the better of the two orders; the other needs need[un] + 1
        } else need[id] = std::min(std::max(nf(n.a), nf(n.b) + 1), std::max(nf(n.b), nf(n.a) + 1));
      } else need[id] = nf(n.a);
    }
  }

  // node id into per-row value k; row slots from d and per-row values above k are free
  void emit_uni(int id, int d, int k) {
    if (!ok) return;
    if (k >= kUSlots) { ok = false; return; }
    const N &n = nodes[id];
    if (uses[id] > 1 && n.op != KAPY_EW_SPLAT)
      for (int below = 0; below < k; ++below)
        if (holder_u[below] == id) {
          push(kPick, below, n.dtype, 0, 0, 0.f, kUniformResult, k);
          holder_u[k] = id;
          return;
        }
    switch (n.op) {
    case KAPY_EW_SPLAT: push(kPushImm, 0, n.dtype, 0, 0, n.imm, kUniformResult, k); break;
    case KAPY_EW_LD_GLOBAL: push(kPushIn, n.input, n.dtype, 0, 0, 0.f, kUniformResult, k); break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX: {
      int from = -1;
      for (int s = 0; s <= std::min(d, 2); ++s)
        if (holder[s] == n.a) from = s;  // the operand already sits on the stack: a reduce only reads it
      if (from < 0) {
        emit_full(n.a, d, k);
        from = d;
      }
      push(n.op, 0, n.dtype, 0, from, 0.f, 0, k);
      break;
    }
    case KAPY_EW_FPTOFP:
      emit_uni(n.a, d, k);
      if (n.dtype != KAPY_F32) push(kCast, 0, n.dtype, n.rmode, 0, 0.f, kUniformResult, k);  // values are fp32 images: widening changes nothing
      break;
    case KAPY_EW_FMA:
      emit_uni(n.a, d, k); emit_uni(n.b, d, k + 1); emit_uni(n.c, d, k + 2);
      push(KAPY_EW_FMA, 0, n.dtype, 0, 0, 0.f, kUniformResult, k);
      break;
    KAPY_EW_BINARY_CASES:
      emit_uni(n.a, d, k); emit_uni(n.b, d, k + 1);
      push(n.op, 0, n.dtype, 0, 0, 0.f, kUniformResult, k);
      break;
    default: emit_uni(n.a, d, k); push(n.op, 0, n.dtype, 0, 0, 0.f, kUniformResult, k);
    }
    for (int above = k + 1; above < kUSlots; ++above) holder_u[above] = -1;
    holder_u[k] = id;
  }

  // node id into row slot d; row slots above d and per-row values from k are free
  void emit_full(int id, int d, int k) {
    if (!ok) return;
    if (d > 2) { ok = false; return; }
    if (holder[d] == id) return;  // still there from an evaluation that only read it since
    const N &n = nodes[id];
    if (uniform[id]) {
      emit_uni(id, d, k);
      push(kPushU, 0, n.dtype, 0, d, 0.f, 0, k);
      holder[d] = id;
      return;
    }
    const bool shared_value = uses[id] > 1;
    if (shared_value) {
      for (int below = 0; below < d; ++below)
        if (holder[below] == id) {
          push(kPick, below, n.dtype, 0, d, 0.f);
          holder[d] = id;
          return;
        }
      if (parked[id]) {
        read_back[id] = 1;
        push(kPushTmp, dry ? 0 : tmp_of[id], n.dtype, 0, d, 0.f);
        holder[d] = id;
        return;
      }
    }
    switch (n.op) {
    case KAPY_EW_LD_GLOBAL: push(kPushIn, n.input, n.dtype, 0, d, 0.f); break;
    case KAPY_EW_FPTOFP:
      emit_full(n.a, d, k);
      // values are fp32 images, so widening changes nothing; and the store rounds to nearest itself
      if (n.dtype != KAPY_F32 && !(id == stored && n.dtype == out_dtype && n.rmode != KAPY_RZ && uses[id] == 1)) push(kCast, 0, n.dtype, n.rmode, d, 0.f);
      break;
    case KAPY_EW_FMA:
      emit_full(n.a, d, k); emit_full(n.b, d + 1, k); emit_full(n.c, d + 2, k);
      push(KAPY_EW_FMA, 0, n.dtype, 0, d, 0.f);
      break;
    KAPY_EW_BINARY_CASES:
      if (n.a == n.b) {
        emit_full(n.a, d, k);
        push(n.op, 0, n.dtype, 0, d, 0.f, kSameOperand);
      } else if (uniform[n.a] || uniform[n.b]) {
        const bool left_uniform = uniform[n.a] != 0;
        const int f = left_uniform ? n.b : n.a, un = left_uniform ? n.a : n.b;
        if (full_first && need[un] > 0) { emit_full(f, d, k); emit_uni(un, d + 1, k); }
        else { emit_uni(un, d, k); emit_full(f, d, k + 1); }
        push(left_uniform ? reversed(n.op) : n.op, 0, n.dtype, 0, d, 0.f, kUniformRight, k);
      } else {
        auto nf = [&](int x) { return std::max(need[x], 1); };
        const bool a_first = std::max(nf(n.a), nf(n.b) + 1) <= std::max(nf(n.b), nf(n.a) + 1);
        if (a_first) { emit_full(n.a, d, k); emit_full(n.b, d + 1, k); push(n.op, 0, n.dtype, 0, d, 0.f); }
        else { emit_full(n.b, d, k); emit_full(n.a, d + 1, k); push(reversed(n.op), 0, n.dtype, 0, d, 0.f); }
      }
      break;
    default: emit_full(n.a, d, k); push(n.op, 0, n.dtype, 0, d, 0.f);
    }
    for (int above = d + 1; above < 3; ++above) holder[above] = -1;
    holder[d] = id;
    if (shared_value) {
      parked[id] = 1;
      if (dry || tmp_of[id] >= 0) push(kSaveTmp, dry ? 0 : tmp_of[id], n.dtype, 0, d, 0.f);
    }
  }

  // one whole emission; returns false when the program does not fit
  bool run(bool full_first_, bool dry_) {
    full_first = full_first_;
    dry = dry_;
    ok = true;
    count = 0;
    max_slot = 0;
    for (int &h : holder) h = -1;
    for (int &h : holder_u) h = -1;
    parked.assign(nodes.size(), 0);
    emit_full(stored, 0, 0);
    push(kStore, 0, out_dtype, 0, 0, 0.f);
    return ok;
  }
  // cost of a strategy: parked values first (LDS traffic and footprint), then row slots, then steps
  bool build(bool full_first_, int *cost) {
    tmp_of.assign(nodes.size(), -1);
    read_back.assign(nodes.size(), 0);
    n_tmps = 0;
    if (!run(full_first_, true)) return false;
    for (size_t id = 0; id < nodes.size(); ++id)
      if (read_back[id]) tmp_of[id] = n_tmps++;
    if (!run(full_first_, false)) return false;
    *cost = n_tmps * 1000 + (max_slot + 1) * 100 + count;
    return true;
  }
};

// Structural match of the named row programs on the DAG.  Shared values must be shared nodes (the same register
// read twice), every intermediate fp32, operands and result the same 16-bit type.
bool match_fused_row(const RowBuilder &B, const StackProgram &SP, const kapy_global *out, FusedRow *p, bool *softmax) {
  const auto &nodes = B.nodes;
  const int T = out->dtype;
  if (T != KAPY_F16 && T != KAPY_BF16) return false;
  auto is = [&](int id, int op) { return id >= 0 && nodes[id].op == op && (op == KAPY_EW_LD_GLOBAL || nodes[id].dtype == KAPY_F32); };
  // cast32(ld input) of a given operand kind: the input's index, or -1
  auto loaded = [&](int id, int kind) {
    if (!is(id, KAPY_EW_FPTOFP)) return -1;
    const int ld = nodes[id].a;
    if (ld < 0 || nodes[ld].op != KAPY_EW_LD_GLOBAL) return -1;
    const int in = nodes[ld].input;
    return SP.in[in].kind == kind && SP.in[in].dtype == T ? in : -1;
  };
  // op(a, b) with operands in either order, `second` chosen by a predicate; returns the other operand or -1
  auto other_of = [&](int id, int op, const std::function<bool(int)> &second) {
    if (!is(id, op)) return -1;
    if (second(nodes[id].b)) return nodes[id].a;
    if (second(nodes[id].a)) return nodes[id].b;
    return -1;
  };
  const int st = B.stored;
  if (nodes[st].op != KAPY_EW_FPTOFP || nodes[st].dtype != T || nodes[st].rmode == KAPY_RZ) return false;
  int body = nodes[st].a;
  int x_in = -1;
  memset(p, 0, sizeof *p);
  // softmax: div(E, sum(E)), E = exp(sub(F, max(F)))
  if (is(body, KAPY_EW_DIVF)) {
    const int e = nodes[body].a, rs = nodes[body].b;
    if (!is(rs, KAPY_EW_REDUCE_SUM) || nodes[rs].a != e || !is(e, KAPY_EW_EXP)) return false;
    const int sub = nodes[e].a;
    if (!is(sub, KAPY_EW_SUBF)) return false;
    const int f = nodes[sub].a, rm = nodes[sub].b;
    if (!is(rm, KAPY_EW_REDUCE_MAX) || nodes[rm].a != f) return false;
    x_in = loaded(f, kInFull);
    if (x_in < 0) return false;
    *softmax = true;
  } else {
    // norm: [add(., beta)] [mul(., gamma)] mul(C, rsqrt(add(mul(sum(mul(C, C)), 1/n), eps))), C = F or sub(F, mul(sum(F), 1/n))
    int gamma = -1, beta = -1;
    auto row_operand = [&](int id) { return loaded(id, kInRow) >= 0; };
    int inner = other_of(body, KAPY_EW_ADDF, row_operand);
    if (inner >= 0) {
      beta = loaded(nodes[body].a == inner ? nodes[body].b : nodes[body].a, kInRow);
      body = inner;
    }
    inner = other_of(body, KAPY_EW_MULF, row_operand);
    if (inner >= 0) {
      gamma = loaded(nodes[body].a == inner ? nodes[body].b : nodes[body].a, kInRow);
      body = inner;
    }
    if (beta >= 0 && gamma < 0) return false;
    const int c = other_of(body, KAPY_EW_MULF, [&](int id) { return is(id, KAPY_EW_RSQRT); });
    if (c < 0) return false;
    const int rsq = nodes[body].a == c ? nodes[body].b : nodes[body].a;
    auto splat = [&](int id) { return is(id, KAPY_EW_SPLAT); };
    const int plus = nodes[rsq].a;
    const int scaled = other_of(plus, KAPY_EW_ADDF, splat);
    if (scaled < 0) return false;
    p->eps = nodes[nodes[plus].a == scaled ? nodes[plus].b : nodes[plus].a].imm;
    const int total = other_of(scaled, KAPY_EW_MULF, splat);
    if (total < 0 || !is(total, KAPY_EW_REDUCE_SUM)) return false;
    p->inv_n = nodes[nodes[scaled].a == total ? nodes[scaled].b : nodes[scaled].a].imm;
    const int sq = nodes[total].a;
    if (!is(sq, KAPY_EW_MULF) || nodes[sq].a != c || nodes[sq].b != c) return false;
    int f = c;
    if (is(c, KAPY_EW_SUBF)) {
      f = nodes[c].a;
      const int mean = nodes[c].b;
      const int fsum = other_of(mean, KAPY_EW_MULF, splat);
      if (fsum < 0 || !is(fsum, KAPY_EW_REDUCE_SUM) || nodes[fsum].a != f) return false;
      if (nodes[nodes[mean].a == fsum ? nodes[mean].b : nodes[mean].a].imm != p->inv_n) return false;
      p->centre = 1;
    }
    x_in = loaded(f, kInFull);
    if (x_in < 0) return false;
    p->gamma = gamma >= 0 ? SP.in[gamma].base : nullptr;
    p->beta = beta >= 0 ? SP.in[beta].base : nullptr;
    *softmax = false;
  }
  p->x = SP.in[x_in].base;
  p->x_stride0 = SP.in[x_in].stride0;
  p->out = (char *)view_base(out);
  p->out_stride0 = out->stride0;
  p->rows = (int32_t)extent0(out);
  p->vec_per_row = (int32_t)(extent1(out) / 8);
  return true;
}

}  // namespace

int run_row_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                    hipStream_t stream) {
  const char *why = "elementwise: a program with a reduce needs axis 1, contiguous rows of a multiple of 8 and at most 32768 elements, zero "
                    "padding, full / row / column / scalar operands of float type, one st_global and at most three row values in flight";
  RowBuilder B;
  int reg[kMaxRegs];
  for (int r = 0; r < kMaxRegs; ++r) reg[r] = -1;
  int n_store = 0;
  for (int k = 0; k < n_inst; ++k) {
    const kapy_ew_inst &I = prog[k];
    RowBuilder::N n;
    n.op = I.op;
    n.dtype = result_dtype[k];
    n.rmode = I.rmode;
    n.imm = I.imm;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL:
      n.input = I.a;
      if (I.c != KAPY_PAD_ZERO) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
      break;
    case KAPY_EW_SPLAT: break;
    case KAPY_EW_ST_GLOBAL: B.stored = reg[I.a]; ++n_store; continue;
    case KAPY_EW_FMA: n.a = reg[I.a]; n.b = reg[I.b]; n.c = reg[I.c]; break;
    KAPY_EW_BINARY_CASES:
      if (I.op == KAPY_EW_REMF) return fail(KAPY_ERR_UNSUPPORTED, "elementwise: remf in a program with a reduce along rows is served by a compiled kernel only");
      n.a = reg[I.a]; n.b = reg[I.b]; break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX:
      if (I.b != 1) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
      n.a = reg[I.a];
      break;
    default: n.a = reg[I.a];
    }
    B.nodes.push_back(n);
    reg[I.dst] = (int)B.nodes.size() - 1;
  }
  if (n_store != 1 || B.stored < 0) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  StackProgram SP;
  memset(&SP, 0, sizeof SP);
  const int64_t o0 = extent0(out), o1 = extent1(out);
  const int ob = dtype_bytes(out->dtype);
  if (!is_float(out->dtype) || out->stride1 != 1 || o1 % 8 != 0 || o1 / 8 > 4096 || ((uintptr_t)view_base(out) % (8 * ob)) || (out->stride0 * ob) % (8 * ob) ||
      o0 >= (int64_t(1) << 31) - 1)
    return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  for (int k = 0; k < n_ins; ++k) {
    const kapy_global *g = ins[k];
    StackIn &in = SP.in[k];
    in.base = view_base(g);
    in.stride0 = g->stride0;
    in.dtype = g->dtype;
    if (!is_float(g->dtype)) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
    const int64_t e0 = extent0(g), e1 = extent1(g);
    const int eb = dtype_bytes(g->dtype);
    const bool vec_ok = g->stride1 == 1 && ((uintptr_t)in.base % (8 * eb)) == 0 && (g->stride0 * eb) % (8 * eb) == 0;
    if (e0 == o0 && e1 == o1 && vec_ok) in.kind = kInFull;
    else if (e0 == 1 && e1 == o1 && vec_ok) in.kind = kInRow;
    else if (e1 == 1 && e0 == o0) in.kind = kInCol;
    else if (e0 == 1 && e1 == 1) in.kind = kInScalar;
    else return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  }
  const size_t nn = B.nodes.size();
  B.uniform.assign(nn, 0);
  for (size_t id = 0; id < nn; ++id) {
    const RowBuilder::N &n = B.nodes[id];
    if (B.is_reduce((int)id) || n.op == KAPY_EW_SPLAT) B.uniform[id] = 1;
    else if (n.op == KAPY_EW_LD_GLOBAL) B.uniform[id] = SP.in[n.input].kind == kInCol || SP.in[n.input].kind == kInScalar;
    else B.uniform[id] = (n.a < 0 || B.uniform[n.a]) && (n.b < 0 || B.uniform[n.b]) && (n.c < 0 || B.uniform[n.c]);
  }
  B.uses.assign(nn, 0);
  {
    std::vector<char> reached(nn, 0);
    std::function<void(int)> visit = [&](int id) {
      ++B.uses[id];
      if (reached[id]) return;
      reached[id] = 1;
      const RowBuilder::N &n = B.nodes[id];
      if (n.a >= 0) visit(n.a);
      if (n.b >= 0 && n.b != n.a) visit(n.b);
      if (n.c >= 0) visit(n.c);
    };
    visit(B.stored);
  }
  {
    FusedRow fr;
    bool softmax = false;
    // KAPY_ROW_FUSED=0 sends the named programs through the row machine as well (tests compare the two)
    const char *sw = getenv("KAPY_ROW_FUSED");
    if (!(sw && sw[0] == '0') && match_fused_row(B, SP, out, &fr, &softmax)) return launch_fused_row(fr, out->dtype, softmax, stream);
  }
  B.compute_need();
  B.out_dtype = out->dtype;
  // two evaluation orders for an op with one row operand and one per-row operand; the cheaper program wins
  StackProgram best;
  int best_cost = -1, best_ns = 0, best_tmps = 0;
  for (int order = 0; order < 2; ++order) {
    StackProgram cand = SP;
    B.P = &cand;
    int cost = 0;
    if (!B.build(order == 1, &cost)) continue;
    if (best_cost < 0 || cost < best_cost) {
      best = cand;
      best.n_post = B.count;
      best_cost = cost;
      best_ns = B.max_slot + 1;
      best_tmps = B.n_tmps;
    }
  }
  if (best_cost < 0) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  best.n_ins = n_ins;
  best.out = (char *)view_base(out);
  best.out_stride0 = out->stride0;
  best.out_dtype = out->dtype;
  best.rows = (int32_t)o0;
  best.vec_per_row = (int32_t)(o1 / 8);
  best.n_tmps = best_tmps;
  bool narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
  for (int k = 0; k < n_ins; ++k) narrow = narrow && (ins[k]->dtype == KAPY_F16 || ins[k]->dtype == KAPY_BF16);
  for (int k = 0; k < n_inst; ++k) narrow = narrow && !is_f8(result_dtype[k]);
  // the light kernel takes programs whose row steps all have cheap forms
  bool light = narrow;
  for (int k = 0; k < best.n_post && light; ++k) {
    const PostOp &I = best.post[k];
    if (I.slot & kUniformResult) continue;
    switch (I.op) {
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX: case kPick: case kPushU: case kSaveTmp: case kPushTmp: case kPushIn: case kPushImm: case kStore:
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case kRevSub: case KAPY_EW_MULF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF: case KAPY_EW_FMA:
    case KAPY_EW_NEGF: case KAPY_EW_ABSF: case KAPY_EW_RSQRT: case KAPY_EW_SQRT: case KAPY_EW_GELU_TANH:
      break;
    case KAPY_EW_EXP: light = I.dtype == KAPY_F32; break;
    case KAPY_EW_DIVF: light = (I.slot & kUniformRight) != 0; break;
    case kCast: light = I.dtype == KAPY_F32 || I.rmode != KAPY_RZ; break;
    default: light = false;
    }
  }
  if (light) return launch_row_kernel<kModeLight>(best, best_ns, stream);
  return narrow ? launch_row_narrow(best, best_ns, stream) : launch_row_any(best, best_ns, stream);
}

}  // namespace kapy
