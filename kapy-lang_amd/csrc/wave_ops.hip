// wave_ops.hip — cross-lane ops of one wavefront: kgpu.change (register re-layout by shuffles)
// and kapy.reduce (butterfly reduction).
//
// Reference: ChangeOpToLLVM.cpp:21-93 — result (lane, iv) takes the value of source
// (lane', iv') = srcMap3(dstMap2(lane, iv)); every source iv that some lane needs from another
// lane is shuffled with shfl.sync.idx and a select chain keeps the one whose iv' matches.
// ReduceOpToLLVM.cpp:51-172 — an in-lane tree over the loop ivs, then shfl.sync.bfly rounds over
// the lanes that share the reduced axis.  On gfx950 the shuffles are ds_bpermute_b32 over 64 lanes.
#include <algorithm>

#include "common.hpp"
#include "layout.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

constexpr int kMaxLoop = 64;

__global__ __launch_bounds__(64) void change_kernel(const uint32_t *in, uint32_t *out, Fragments src, Fragments dst, Idx2 shape,
                                                    int n_src, int n_dst) {
  const int lane = threadIdx.x;
  for (int iv = 0; iv < n_dst; ++iv) {
    Idx2 from = change_source(src, dst, shape, lane, iv);
    uint32_t result = 0;
    // one shuffle per source register; the select keeps the register this lane asked for
    for (int s = 0; s < n_src; ++s) {
      uint32_t mine = in[lane * n_src + s];
      uint32_t got = (uint32_t)__builtin_amdgcn_ds_bpermute((int)from.v0 << 2, (int)mine);
      if (from.v1 == s) result = got;
    }
    out[lane * n_dst + iv] = result;
  }
}

struct ReduceParams {
  const char *src;
  char *dst;
  int64_t s_keep, s_red;  // source strides along the kept and the reduced axis
  int64_t d_keep;         // result stride along the kept axis
  int32_t n_keep, n_red;
  int32_t src_dtype, dst_dtype, kind;  // kind: kapy_reduce_combiner
};

// What a fold starts from so that the elements themselves decide the result (ReduceOpToLLVM.cpp:60-101 folds the elements,
// no identity joins them): -0 for a sum (-0 + x = x for every x, -0 included, so a line of only -0 sums to -0), the
// infinities for maximumf / minimumf, NaN for maxnumf / minnumf (ignored unless every element is one), 1 for a product;
// for the integer combiners the usual neutral elements, as containers.
__device__ __forceinline__ float identity_of(int kind, int dtype) {
  switch (kind) {
  case KAPY_REDUCE_ADDF: return -0.f;
  case KAPY_REDUCE_MAXIMUMF: return -__builtin_inff();
  case KAPY_REDUCE_MINIMUMF: return __builtin_inff();
  case KAPY_REDUCE_MULF: return 1.f;
  case KAPY_REDUCE_MAXNUMF: case KAPY_REDUCE_MINNUMF: return __builtin_nanf("");
  case KAPY_REDUCE_MULI: return int_reg(int_canon(1, dtype));
  case KAPY_REDUCE_MAXSI: return int_reg(int_canon(dtype == KAPY_I8 ? -128 : dtype == KAPY_I16 ? -32768 : (int32_t)0x80000000u, dtype));
  case KAPY_REDUCE_MINSI: return int_reg(int_canon(dtype == KAPY_I8 ? 127 : dtype == KAPY_I16 ? 32767 : 0x7FFFFFFF, dtype));
  case KAPY_REDUCE_MINUI: case KAPY_REDUCE_ANDI: return int_reg(int_canon(-1, dtype));
  default: return int_reg(0);  // addi, maxui, ori, xori
  }
}
// float combiners on fp32 values; -0 orders below +0 for the four orderings (fmaxf / fminf do that on this device)
__device__ __forceinline__ float combine(float a, float b, int kind) {
  switch (kind) {
  case KAPY_REDUCE_ADDF: return a + b;
  case KAPY_REDUCE_MAXIMUMF: return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b);
  case KAPY_REDUCE_MINIMUMF: return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b);
  case KAPY_REDUCE_MULF: return a * b;
  case KAPY_REDUCE_MAXNUMF: return a != a ? b : b != b ? a : fmaxf(a, b);
  default: return a != a ? b : b != b ? a : fminf(a, b);
  }
}
// any combiner, integer ones on containers of element type dtype
__device__ __forceinline__ float combine_any(float a, float b, int kind, int dtype) {
  if (kind < KAPY_REDUCE_ADDI) return combine(a, b, kind);
  constexpr int op_of[] = {KAPY_EW_ADDI, KAPY_EW_MULI, KAPY_EW_MAXSI, KAPY_EW_MINSI, KAPY_EW_MAXUI, KAPY_EW_MINUI, KAPY_EW_ANDI, KAPY_EW_ORI, KAPY_EW_XORI};
  return int_reg(int_binary(op_of[kind - KAPY_REDUCE_ADDI], reg_int(a), reg_int(b), dtype));
}
// the vector kernels are built twice: KIND 0 adds, KIND 1 reads the (float) combiner from the parameters
template <int KIND>
__device__ __forceinline__ float combine_t(float a, float b, int kind) { return KIND == 0 ? a + b : combine(a, b, kind); }

// ---- sharing a reduced axis out over workgroups -----------------------------------------------------------------------
// Every workgroup that owns a chunk of a line leaves fp32 partial results in `lines` and counts itself at the line group's
// counter; the one that arrives last folds the partials in chunk order (the same bits every run) and stores the result,
// then sets the counter back to zero.  Nobody waits for anybody.  The partials cross XCDs, whose L2 caches are not coherent
// with each other: they are written and read with relaxed device-scope accesses (which go past the L2), every lane waits
// until its stores have been acknowledged before the workgroup counts itself, and the reader starts only after its count
// has come back.
constexpr int kCounterBytes = 16 << 10, kMaxGroups = kCounterBytes / 4;
constexpr size_t kScratchLineBytes = size_t(4) << 20;
struct Shared {
  float *lines = nullptr;
  uint32_t *counters = nullptr;
  int64_t floats = 0;
};
__device__ __forceinline__ void partial_store(float *at, float v) {
  __hip_atomic_store((uint32_t *)at, f32_bits(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float partial_load(const float *at) {
  return bits_f32(__hip_atomic_load((const uint32_t *)at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// true in the workgroup that arrived last of `parts` at `counter` (all lanes get the same answer); `word`: 4 bytes of LDS
__device__ __forceinline__ bool arrived_last(uint32_t *counter, uint32_t parts, uint32_t *word) {
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this lane's partial results have been acknowledged (lgkmcnt, expcnt: no wait)
  __syncthreads();
  if (threadIdx.x == 0) *word = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const bool last = *word == parts - 1;
  __syncthreads();
  return last;
}

// One wavefront per kept index: lanes stride over the reduced axis, then 6 butterfly rounds.  Any element type and strides.
__global__ __launch_bounds__(256) void reduce_wave_kernel(ReduceParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t keep = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (keep >= p.n_keep) return;
  float acc = identity_of(p.kind, p.src_dtype);
  int32_t r = lane;
  for (; r + 192 < p.n_red; r += 256) {  // four loads in flight
    float f[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) f[u] = load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)(r + 64 * u) * p.s_red);
#pragma unroll
    for (int u = 0; u < 4; ++u) acc = combine_any(acc, f[u], p.kind, p.src_dtype);
  }
  for (; r < p.n_red; r += 64) acc = combine_any(acc, load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)r * p.s_red), p.kind, p.src_dtype);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ off) << 2, (int)f32_bits(acc)));
    acc = combine_any(acc, other, p.kind, p.src_dtype);
  }
  if (lane == 0) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
}

// 16-bit elements, reduced axis contiguous, 16-byte aligned rows, n_red a multiple of 8: one wavefront
// per kept index, 128-bit non-temporal loads (a wave reads 1 KiB of the row per instruction, four in
// flight), the 8 values of a load combined in the lane first (the in-lane tree over loop ivs of
// ReduceOpToLLVM.cpp:76-101), then the six butterfly rounds (:104-119).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
// SRC: what a 128-bit load holds - 0: 8 x f16, 1: 8 x bf16, 2: 4 x f32.
template <int SRC>
constexpr int per_vec() { return SRC == 2 ? 4 : 8; }
template <int SRC>
__device__ __forceinline__ void widen(u32x4_t v, float (&f)[per_vec<SRC>()]) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t word = v[w];
    if constexpr (SRC == 2) f[w] = bits_f32(word);
    else if constexpr (SRC == 1) {
      f[2 * w] = bits_f32(word << 16);
      f[2 * w + 1] = bits_f32(word & 0xFFFF0000u);
    } else {
      f[2 * w] = f16_to_f32((uint16_t)word);
      f[2 * w + 1] = f16_to_f32((uint16_t)(word >> 16));
    }
  }
}
// the values of one load folded as a tree
template <int SRC, int KIND>
__device__ __forceinline__ float fold_vec(const float (&f)[per_vec<SRC>()], int kind) {
  if constexpr (SRC == 2) return combine_t<KIND>(combine_t<KIND>(f[0], f[1], kind), combine_t<KIND>(f[2], f[3], kind), kind);
  else return combine_t<KIND>(combine_t<KIND>(combine_t<KIND>(f[0], f[1], kind), combine_t<KIND>(f[2], f[3], kind), kind),
                              combine_t<KIND>(combine_t<KIND>(f[4], f[5], kind), combine_t<KIND>(f[6], f[7], kind), kind), kind);
}
// Four lines per workgroup, one wave each; gridDim.y > 1: a wave folds one chunk of its line, and the workgroup that is last
// to arrive for these four lines folds the chunks' partial results (lane c holds chunk c, c + 64, ..., then the butterfly).
template <int SRC, int KIND>
__global__ __launch_bounds__(256) void reduce_rows_vec_kernel(ReduceParams p, Shared sh, int32_t vecs_per_chunk) {
  __shared__ uint32_t word;
  const int lane = threadIdx.x & 63;
  const int64_t keep = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  constexpr int E = per_vec<SRC>();
  const int32_t chunks = gridDim.y;
  float acc = identity_of(p.kind, p.src_dtype);
  if (keep < p.n_keep) {
    const u32x4_t *row = (const u32x4_t *)(p.src + keep * p.s_keep * (16 / E));
    const int32_t vecs = min(p.n_red / E, (int32_t)(blockIdx.y + 1) * vecs_per_chunk);
    constexpr int U = 4;
    int32_t v = blockIdx.y * vecs_per_chunk + lane;
    for (; v + 64 * (U - 1) < vecs; v += 64 * U) {
      u32x4_t x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = __builtin_nontemporal_load(row + v + 64 * u);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float f[E];
        widen<SRC>(x[u], f);
        const float t = fold_vec<SRC, KIND>(f, p.kind);
        acc = combine_t<KIND>(acc, t, p.kind);
      }
    }
    for (; v < vecs; v += 64) {
      float f[E];
      widen<SRC>(__builtin_nontemporal_load(row + v), f);
#pragma unroll
      for (int e = 0; e < E; ++e) acc = combine_t<KIND>(acc, f[e], p.kind);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ off) << 2, (int)f32_bits(acc)));
      acc = combine_t<KIND>(acc, other, p.kind);
    }
  }
  if (chunks == 1) {
    if (lane == 0 && keep < p.n_keep) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
    return;
  }
  if (lane == 0 && keep < p.n_keep) partial_store(sh.lines + keep * chunks + blockIdx.y, acc);
  if (!arrived_last(sh.counters + blockIdx.x, (uint32_t)chunks, &word)) return;
  if (keep < p.n_keep) {
    float t = identity_of(p.kind, p.src_dtype);
    for (int32_t c = lane; c < chunks; c += 64) t = combine_t<KIND>(t, partial_load(sh.lines + keep * chunks + c), p.kind);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
      float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ off) << 2, (int)f32_bits(t)));
      t = combine_t<KIND>(t, other, p.kind);
    }
    if (lane == 0) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
  }
  if (threadIdx.x == 0) __hip_atomic_store(sh.counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The same for lines of up to 512 elements: a line takes GROUP lanes (8, 16, 32 or 64: the next power of two from its
// vectors), a wave 64 / GROUP lines at a time, each lane one 128-bit load; the butterfly stays inside the group.
template <int SRC, int KIND, int GROUP>
__global__ __launch_bounds__(256) void reduce_rows_short_kernel(ReduceParams p) {
  const int64_t keep = (int64_t)blockIdx.x * (256 / GROUP) + threadIdx.x / GROUP;
  const int32_t jv = threadIdx.x % GROUP;
  float acc = identity_of(p.kind, p.src_dtype);
  constexpr int E = per_vec<SRC>();
  if (keep < p.n_keep && jv < p.n_red / E) {
    float f[E];
    widen<SRC>(__builtin_nontemporal_load((const u32x4_t *)(p.src + keep * p.s_keep * (16 / E)) + jv), f);
    acc = fold_vec<SRC, KIND>(f, p.kind);
  }
#pragma unroll
  for (int off = GROUP / 2; off >= 1; off >>= 1) {
    float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute(((threadIdx.x & 63) ^ off) << 2, (int)f32_bits(acc)));
    acc = combine_t<KIND>(acc, other, p.kind);
  }
  if (jv == 0 && keep < p.n_keep) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
}

// The last-arrived workgroup's fold of `chunks` partial lines for COLS kept indices starting at keep0: the 256 lanes form
// 256 / COLS groups that take chunks g, g + groups, ... (sixteen loads in flight per lane), the groups meet in LDS and are
// folded in group order.  part: [256 / COLS][COLS + 1] floats.
template <int COLS, int KIND>
__device__ __forceinline__ void fold_partial_lines(const ReduceParams &p, const Shared &sh, int64_t keep0, int32_t chunks, float *part) {
  constexpr int GROUPS = 256 / COLS;
  const int cl = threadIdx.x % COLS, g = threadIdx.x / COLS;
  const int64_t keep = keep0 + cl;
  float t = identity_of(p.kind, p.src_dtype);
  if (keep < p.n_keep) {
    int32_t c = g;
    constexpr int U = 16;
    for (; c + GROUPS * (U - 1) < chunks; c += GROUPS * U) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = partial_load(sh.lines + (int64_t)(c + GROUPS * u) * p.n_keep + keep);
#pragma unroll
      for (int u = 0; u < U; ++u) t = combine_t<KIND>(t, x[u], p.kind);
    }
    for (; c < chunks; c += GROUPS) t = combine_t<KIND>(t, partial_load(sh.lines + (int64_t)c * p.n_keep + keep), p.kind);
  }
  if (GROUPS > 1) {
    part[g * (COLS + 1) + cl] = t;
    __syncthreads();
    if (g == 0) {
      t = part[cl];
#pragma unroll
      for (int k = 1; k < GROUPS; ++k) t = combine_t<KIND>(t, part[k * (COLS + 1) + cl], p.kind);
    }
  }
  if (g == 0 && keep < p.n_keep) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
}

// 16-bit or f32 elements, kept axis contiguous: a workgroup of 256 lanes owns a strip of E * LPR kept indices - LPR lanes x
// one 128-bit load per reduced index - and a chunk of the reduced axis, which its 256 / LPR groups of lanes walk with four
// loads in flight each; the groups' partial results meet in LDS.  With one chunk the strip's results go to the result;
// with more (few kept indices, many reduced ones: a tall matrix would otherwise keep a handful of CUs busy) every chunk
// leaves an fp32 partial line and the strip's last workgroup to arrive folds the lines in chunk order.
template <int SRC, int KIND, int LPR>
__global__ __launch_bounds__(256) void reduce_cols_strip_kernel(ReduceParams p, Shared sh, int32_t per_chunk) {
  constexpr int E = per_vec<SRC>(), EB = 16 / E, GROUPS = 256 / LPR, COLS = LPR * E;
  __shared__ float part[GROUPS][COLS + 1];
  __shared__ uint32_t word;
  const int cl = threadIdx.x % LPR, rg = threadIdx.x / LPR;
  const int64_t keep0 = (int64_t)blockIdx.x * COLS + cl * E;
  const int32_t r_begin = blockIdx.y * per_chunk, r_end = min(p.n_red, r_begin + per_chunk);
  const int32_t chunks = gridDim.y;
  float acc[E];
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = identity_of(p.kind, p.src_dtype);
  if (keep0 < p.n_keep) {  // (whole vectors: n_keep is a multiple of E)
    const char *col = p.src + keep0 * EB;
    constexpr int U = 4;
    int32_t r = r_begin + rg;
    for (; r + GROUPS * (U - 1) < r_end; r += GROUPS * U) {
      u32x4_t x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = __builtin_nontemporal_load((const u32x4_t *)(col + (int64_t)(r + GROUPS * u) * p.s_red * EB));
#pragma unroll
      for (int u = 0; u < U; ++u) {
        float f[E];
        widen<SRC>(x[u], f);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] = combine_t<KIND>(acc[e], f[e], p.kind);
      }
    }
    for (; r < r_end; r += GROUPS) {
      float f[E];
      widen<SRC>(__builtin_nontemporal_load((const u32x4_t *)(col + (int64_t)r * p.s_red * EB)), f);
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] = combine_t<KIND>(acc[e], f[e], p.kind);
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) part[rg][cl * E + e] = acc[e];
  __syncthreads();
  const int64_t keep = (int64_t)blockIdx.x * COLS + threadIdx.x;
  if (threadIdx.x < COLS && keep < p.n_keep) {
    float t = identity_of(p.kind, p.src_dtype);
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) t = combine_t<KIND>(t, part[g][threadIdx.x], p.kind);
    if (chunks > 1) partial_store(sh.lines + (int64_t)blockIdx.y * p.n_keep + keep, t);
    else store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
  }
  if (chunks == 1) return;
  if (!arrived_last(sh.counters + blockIdx.x, (uint32_t)chunks, &word)) return;
  fold_partial_lines<COLS, KIND>(p, sh, (int64_t)blockIdx.x * COLS, chunks, &part[0][0]);
  if (threadIdx.x == 0) __hip_atomic_store(sh.counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Any element type, alignment and extents, kept axis contiguous (or at least not the strided one): a workgroup owns 64 kept
// indices, one per lane of a wave (a wave's loads cover 64 consecutive elements of one reduced index), its four waves share
// out a chunk of the reduced axis with four loads in flight each and meet in LDS; chunks as in reduce_cols_strip_kernel
// (float combiners only: the partial lines are fp32).
__global__ __launch_bounds__(256) void reduce_cols_any_kernel(ReduceParams p, Shared sh, int32_t per_chunk) {
  __shared__ float part[4][64 + 1];
  __shared__ uint32_t word;
  const int cl = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int64_t keep = (int64_t)blockIdx.x * 64 + cl;
  const int32_t r_begin = blockIdx.y * per_chunk, r_end = min(p.n_red, r_begin + per_chunk);
  const int32_t chunks = gridDim.y;
  float acc = identity_of(p.kind, p.src_dtype);
  if (keep < p.n_keep) {
    int32_t r = r_begin + rg;
    for (; r + 12 < r_end; r += 16) {
      float f[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) f[u] = load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)(r + 4 * u) * p.s_red);
#pragma unroll
      for (int u = 0; u < 4; ++u) acc = combine_any(acc, f[u], p.kind, p.src_dtype);
    }
    for (; r < r_end; r += 4) acc = combine_any(acc, load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)r * p.s_red), p.kind, p.src_dtype);
  }
  part[rg][cl] = acc;
  __syncthreads();
  if (rg == 0 && keep < p.n_keep) {
    const int k = p.kind, d = p.src_dtype;
    float t = combine_any(combine_any(part[0][cl], part[1][cl], k, d), combine_any(part[2][cl], part[3][cl], k, d), k, d);
    if (chunks > 1) partial_store(sh.lines + (int64_t)blockIdx.y * p.n_keep + keep, t);
    else store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
  }
  if (chunks == 1) return;
  if (!arrived_last(sh.counters + blockIdx.x, (uint32_t)chunks, &word)) return;
  fold_partial_lines<64, 1>(p, sh, (int64_t)blockIdx.x * 64, chunks, &part[0][0]);
  if (threadIdx.x == 0) __hip_atomic_store(sh.counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// KAPY_REDUCE_REFERENCE: the lowering's own fold of one wavefront's tile (ReduceOpToLLVM.cpp:51-172 on 64 lanes).  A lane
// holds the elements `layout` gives it (map 1: positions past the tensor wrap, as the reference's own loads replicate them);
// per kept loop index it folds its elements along the reduced axis in loop order, every application of the combiner an op
// on the element type; then `rounds` butterfly exchanges at lane distances lane_offset << i; every lane stores what it holds
// (lanes that hold replicas store the same value).
__global__ __launch_bounds__(64) void reduce_reference_kernel(ReduceParams p, Fragments layout, Idx2 shape, int axis, int lane_offset, int rounds) {
  const int lane = threadIdx.x;
  const Idx2 ls = layout.loop_space(shape);
  const int64_t n_keep_iv = axis == 1 ? ls.v0 : ls.v1, n_red_iv = axis == 1 ? ls.v1 : ls.v0;
  const bool is_float = p.kind < KAPY_REDUCE_ADDI;
  for (int64_t k = 0; k < n_keep_iv; ++k) {
    float acc = 0.f;
    Idx2 at{0, 0};
    for (int64_t r = 0; r < n_red_iv; ++r) {
      const int64_t iv0 = axis == 1 ? k : r, iv1 = axis == 1 ? r : k;
      const int64_t iv = layout.row_major() ? iv0 * ls.v1 + iv1 : iv0 + iv1 * ls.v0;
      const Idx2 e = layout.to_index(shape, lane, iv, true);
      const float v = load_as_f32(p.src, p.src_dtype, (axis == 1 ? e.v0 : e.v1) * p.s_keep + (axis == 1 ? e.v1 : e.v0) * p.s_red);
      if (r == 0) { acc = v; at = e; }
      else {
        acc = combine_any(acc, v, p.kind, p.src_dtype);
        if (is_float) acc = round_to_dtype(acc, p.src_dtype, true);
      }
    }
    for (int i = 0; i < rounds; ++i) {
      const float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ (lane_offset << i)) << 2, (int)f32_bits(acc)));
      acc = combine_any(acc, other, p.kind, p.src_dtype);
      if (is_float) acc = round_to_dtype(acc, p.src_dtype, true);
    }
    store_from_f32(p.dst, p.dst_dtype, (axis == 1 ? at.v0 : at.v1) * p.d_keep, acc);
  }
}

}  // namespace
}  // namespace kapy

// The library's own workspace: 16 KiB of arrival counters (zero when the code object is loaded, and every launch leaves them
// zero) and 4 MiB of partial lines, one copy per device.  In host code the array's name is a handle, not a device address.
static __device__ __align__(256) unsigned char reduce_scratch[kapy::kCounterBytes + kapy::kScratchLineBytes];

namespace kapy {

// This device's copy of the array (asked for once per device; a race between two first calls only repeats the query).
void *reduce_scratch_address() {
  constexpr int kMaxDevices = 64;
  static void *on_device[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void *ws = __atomic_load_n(&on_device[dev], __ATOMIC_ACQUIRE);
  if (!ws) {
    if (hipGetSymbolAddress(&ws, HIP_SYMBOL(reduce_scratch)) != hipSuccess || !ws) {
      (void)hipGetLastError();
      return nullptr;
    }
    __atomic_store_n(&on_device[dev], ws, __ATOMIC_RELEASE);
  }
  return ws;
}
// The partial-line part of the library's own array for the column programs of kapy_elementwise (elementwise.hip), which
// run their reduces as launches of their own on the caller's stream: like every call without a workspace they must not
// overlap in time with another such call on the same GPU.
float *reduce_scratch_lines(size_t *bytes, uint32_t **counters) {
  char *ws = (char *)reduce_scratch_address();
  if (!ws) return nullptr;
  *bytes = kScratchLineBytes;
  if (counters) *counters = (uint32_t *)ws;
  return (float *)(ws + kCounterBytes);
}

namespace {

// counters and lines of the call: the caller's workspace if it gave one, else the library's array; empty if neither is usable
Shared shared_of(const kapy_reduce_cfg &cfg) {
  Shared sh;
  char *base = (char *)cfg.workspace;
  int64_t bytes = cfg.workspace_bytes;
  if (!base) {
    base = (char *)reduce_scratch_address();
    bytes = (int64_t)(kCounterBytes + kScratchLineBytes);
  }
  if (!base || bytes <= kCounterBytes || ((uintptr_t)base & 15)) return sh;
  sh.counters = (uint32_t *)base;
  sh.lines = (float *)(base + kCounterBytes);
  sh.floats = (bytes - kCounterBytes) / 4;
  return sh;
}

Fragments to_internal(const kapy_fragments *f) {
  return Fragments{f->lane_array[0], f->lane_array[1], f->lane_loops[0], f->lane_loops[1], f->major_axis};
}

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" {

int kapy_change(const uint32_t *lane_values_in, const kapy_fragments *src, const kapy_fragments *dst, const int64_t shape[2],
                uint32_t *lane_values_out, void *stream) {
  if (!lane_values_in || !lane_values_out || !src || !dst || !shape) return fail(KAPY_ERR_INVALID, "change: null argument");
  for (const kapy_fragments *f : {src, dst}) {
    if (f->lane_array[0] * f->lane_array[1] != kWaveSize)
      return fail(KAPY_ERR_VERIFY, "change: a fragments layout must cover the %d lanes of a wavefront", kWaveSize);
    if (f->lane_loops[0] <= 0 || f->lane_loops[1] <= 0 || (f->major_axis != 0 && f->major_axis != 1) ||
        f->minor_axis != 1 - f->major_axis)
      return fail(KAPY_ERR_VERIFY, "change: malformed fragments layout");
  }
  for (int i = 0; i < 2; ++i)
    if (shape[i] <= 0 || (shape[i] & (shape[i] - 1)))
      return fail(KAPY_ERR_VERIFY, "change: tensor shape must be a positive power of two on every axis");
  Fragments s = to_internal(src), d = to_internal(dst);
  Idx2 sh{shape[0], shape[1]};
  int64_t ns = s.loop_size(sh), nd = d.loop_size(sh);
  if (ns > kMaxLoop || nd > kMaxLoop) return fail(KAPY_ERR_UNSUPPORTED, "change: more than %d values per lane", kMaxLoop);
  int rc = ensure_device();
  if (rc) return rc;
  change_kernel<<<1, 64, 0, (hipStream_t)stream>>>(lane_values_in, lane_values_out, s, d, sh, (int)ns, (int)nd);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

// LAUNCH(source kind, KIND) for the call's source type; KIND 0: the kernels' compiled-in addf, 1: the combiner read from p.kind
#define KAPY_BY_SOURCE(LAUNCH)                                                                  \
  do {                                                                                          \
    if (src_kind == 0) { if (kind == 0) LAUNCH(0, 0); else LAUNCH(0, 1); }                      \
    else if (src_kind == 1) { if (kind == 0) LAUNCH(1, 0); else LAUNCH(1, 1); }                 \
    else { if (kind == 0) LAUNCH(2, 0); else LAUNCH(2, 1); }                                    \
  } while (0)

int64_t kapy_reduce_workspace_bytes(void) { return (int64_t)(kCounterBytes + kScratchLineBytes); }

int kapy_reduce(const kapy_global *src, const kapy_global *dst, int32_t axis, int32_t kind, void *stream) {
  kapy_reduce_cfg cfg = {kind, KAPY_REDUCE_WIDE, nullptr, nullptr, 0};
  return kapy_reduce_ex(src, dst, axis, &cfg, stream);
}

int kapy_reduce_ex(const kapy_global *src, const kapy_global *dst, int32_t axis, const kapy_reduce_cfg *cfg_in, void *stream) {
  int rc = check_global(src, "reduce source");
  if (!rc) rc = check_global(dst, "reduce result");
  if (rc) return rc;
  kapy_reduce_cfg cfg = {KAPY_REDUCE_ADDF, KAPY_REDUCE_WIDE, nullptr, nullptr, 0};
  if (cfg_in) cfg = *cfg_in;
  const int kind = cfg.combiner;
  if (axis != 0 && axis != 1) return fail(KAPY_ERR_VERIFY, "reduce: axis must be 0 or 1");
  if (kind < KAPY_REDUCE_ADDF || kind > KAPY_REDUCE_XORI) return fail(KAPY_ERR_INVALID, "reduce: unknown combiner %d", kind);
  if (cfg.arithmetic != KAPY_REDUCE_WIDE && cfg.arithmetic != KAPY_REDUCE_REFERENCE) return fail(KAPY_ERR_INVALID, "reduce: unknown arithmetic %d", cfg.arithmetic);
  if (cfg.workspace && cfg.workspace_bytes < 0) return fail(KAPY_ERR_INVALID, "reduce: negative workspace size");
  const int64_t s0 = extent0(src), s1 = extent1(src);
  // Kapy.cpp ReduceOp::verify: the result keeps the other axis and has one element along `axis`
  if (axis == 1 ? (extent1(dst) != 1 || extent0(dst) != s0) : (extent0(dst) != 1 || extent1(dst) != s1))
    return fail(KAPY_ERR_VERIFY, "reduce: number of elements in result is incorrect");
  const bool on_ints = kind >= KAPY_REDUCE_ADDI;
  if (on_ints) {
    if (!is_int(src->dtype) || src->dtype == KAPY_I1 || dst->dtype != src->dtype)
      return fail(KAPY_ERR_VERIFY, "reduce: an integer combiner needs i8, i16 or i32 tensors, source and result of one type");
  } else if (!is_float(src->dtype) || is_f8(src->dtype) || !is_float(dst->dtype) || is_f8(dst->dtype))
    return fail(KAPY_ERR_UNSUPPORTED, "reduce: a float combiner needs f16, bf16 or f32 tensors");
  if (src->start0 < 0 || src->start1 < 0 || dst->start0 < 0 || dst->start1 < 0) return fail(KAPY_ERR_INVALID, "reduce: negative view start");
  rc = ensure_device();
  if (rc) return rc;
  ReduceParams p;
  p.src = view_base(src);
  p.dst = (char *)view_base(dst);
  p.s_keep = axis == 1 ? src->stride0 : src->stride1;
  p.s_red = axis == 1 ? src->stride1 : src->stride0;
  p.d_keep = axis == 1 ? dst->stride0 : dst->stride1;
  p.n_keep = (int32_t)(axis == 1 ? s0 : s1);
  p.n_red = (int32_t)(axis == 1 ? s1 : s0);
  p.src_dtype = src->dtype;
  p.dst_dtype = dst->dtype;
  p.kind = kind;
  if (p.n_keep == 0) return KAPY_OK;
  hipStream_t s = (hipStream_t)stream;
  if (cfg.arithmetic == KAPY_REDUCE_REFERENCE) {
    if (dst->dtype != src->dtype) return fail(KAPY_ERR_VERIFY, "reduce: in the reference's arithmetic the result has the source's element type");
    if ((s0 & (s0 - 1)) || (s1 & (s1 - 1))) return fail(KAPY_ERR_VERIFY, "reduce: a wavefront's tile has power-of-two extents");
    const Idx2 shape{s0, s1};
    Fragments layout = default_fragments(Idx2{1, 1}, shape, true);
    if (cfg.layout) {
      const kapy_fragments *f = cfg.layout;
      if (f->lane_array[0] * f->lane_array[1] != kWaveSize || f->lane_loops[0] <= 0 || f->lane_loops[1] <= 0 || (f->major_axis != 0 && f->major_axis != 1) ||
          f->minor_axis != 1 - f->major_axis)
        return fail(KAPY_ERR_VERIFY, "reduce: malformed fragments layout");
      layout = to_internal(f);
    }
    if (layout.loop_size(shape) > 4096) return fail(KAPY_ERR_UNSUPPORTED, "reduce: more than 4096 values per lane in the reference's arithmetic");
    // laneOffset and the number of exchange rounds: LayoutUtils.cpp:26-49
    const int lane_offset = layout.major == axis ? 1 : (axis == 1 ? layout.a0 : layout.a1);
    bool seen[kWaveSize] = {false};
    int distinct = 0;
    for (int64_t i = 0; i < (axis == 0 ? s0 : s1); ++i) {
      const int64_t lane = axis == 0 ? layout.to_lane_iv(shape, i, 0).v0 : layout.to_lane_iv(shape, 0, i).v0;
      if (!seen[lane]) { seen[lane] = true; ++distinct; }
    }
    int rounds = 0;
    while ((1 << (rounds + 1)) <= distinct) ++rounds;
    reduce_reference_kernel<<<1, 64, 0, s>>>(p, layout, shape, axis, lane_offset, rounds);
    KAPY_HIP_CHECK(hipGetLastError());
    return KAPY_OK;
  }
  // the vector kernels: f16, bf16 or f32 source read in 128-bit pieces of E elements
  const bool vec_ok = !on_ints && (src->dtype == KAPY_F16 || src->dtype == KAPY_BF16 || src->dtype == KAPY_F32);
  const int src_kind = src->dtype == KAPY_F32 ? 2 : src->dtype == KAPY_BF16 ? 1 : 0, E = src_kind == 2 ? 4 : 8, EB = 16 / E;
  const bool aligned = ((uintptr_t)p.src & 15) == 0;
  // how far a launch may share a reduced axis out: as many chunks as the partial lines of `lines_of` values each and the
  // counters of `groups` line groups allow (integer combiners: no sharing, the partial lines are fp32)
  Shared sh;
  auto chunks_allowed = [&](int64_t groups, int64_t values_per_chunk) -> int64_t {
    if (on_ints || groups > kMaxGroups) return 1;
    sh = shared_of(cfg);
    return sh.lines ? std::max<int64_t>(1, sh.floats / std::max<int64_t>(1, values_per_chunk)) : 1;
  };
  if (vec_ok && aligned && p.s_red == 1 && p.n_red % E == 0 && (p.s_keep * EB) % 16 == 0 && p.n_red <= 64 * E && p.n_red >= E) {
    const int vecs = p.n_red / E, group = vecs <= 8 ? 8 : vecs <= 16 ? 16 : vecs <= 32 ? 32 : 64;
    const int64_t wgs = ((int64_t)p.n_keep + 256 / group - 1) / (256 / group);
    if (wgs > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "reduce: more than 2^31 workgroups");
    dim3 grid((unsigned)wgs);
#define KAPY_SHORT(SRC_, KIND_)                                                                      \
  do {                                                                                               \
    if (group == 8) reduce_rows_short_kernel<SRC_, KIND_, 8><<<grid, 256, 0, s>>>(p);                \
    else if (group == 16) reduce_rows_short_kernel<SRC_, KIND_, 16><<<grid, 256, 0, s>>>(p);         \
    else if (group == 32) reduce_rows_short_kernel<SRC_, KIND_, 32><<<grid, 256, 0, s>>>(p);         \
    else reduce_rows_short_kernel<SRC_, KIND_, 64><<<grid, 256, 0, s>>>(p);                          \
  } while (0)
    KAPY_BY_SOURCE(KAPY_SHORT);
#undef KAPY_SHORT
  } else if (vec_ok && aligned && p.s_red == 1 && p.n_red % E == 0 && (p.s_keep * EB) % 16 == 0 && p.n_red > 64 * E) {
    // four lines per workgroup; with fewer workgroups than CUs, chunks of at least 256 vectors of the reduced axis as well,
    // up to four workgroups per CU: 64 lines of 1 Mi elements 312 -> 33 us, 256 lines of 256 Ki 82 -> 30 us.
    const int64_t wgs = ((int64_t)p.n_keep + 3) / 4, want = 4 * (int64_t)device_cus(), vecs = p.n_red / E;
    int64_t chunks = wgs >= device_cus() ? 1 : std::max<int64_t>(1, std::min<int64_t>({(want + wgs - 1) / wgs, vecs / 256, 512}));
    if (chunks > 1) chunks = std::min(chunks, chunks_allowed(wgs, p.n_keep));
    const int32_t vecs_per_chunk = (int32_t)((vecs + chunks - 1) / chunks);
    chunks = (vecs + vecs_per_chunk - 1) / vecs_per_chunk;
    dim3 grid((unsigned)wgs, (unsigned)chunks);
#define KAPY_ROWS(SRC_, KIND_) reduce_rows_vec_kernel<SRC_, KIND_><<<grid, 256, 0, s>>>(p, sh, vecs_per_chunk)
    KAPY_BY_SOURCE(KAPY_ROWS);
#undef KAPY_ROWS
  } else if (vec_ok && aligned && p.s_keep == 1 && p.n_keep % E == 0 && (p.s_red * EB) % 16 == 0 && p.n_red >= 32) {
    // strips of 256 kept indices (512-byte runs per reduced index), of 64 for narrow sources; the reduced axis in as many
    // chunks as bring the launch to about four workgroups per CU, of at least 128 reduced indices each, as far as their
    // partial lines fit the workspace.
    const int lpr = p.n_keep >= 32 * E ? 32 : 8, cols = lpr * E;
    const int64_t strips = ((int64_t)p.n_keep + cols - 1) / cols, want = 4 * (int64_t)device_cus();
    if (strips > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "reduce: more than 2^31 strips of results");
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>({(want + strips - 1) / strips, (int64_t)p.n_red / 128, 512}));
    if (chunks > 1) chunks = std::min(chunks, chunks_allowed(strips, p.n_keep));
    const int32_t per_chunk = (int32_t)((p.n_red + chunks - 1) / chunks);
    chunks = (p.n_red + per_chunk - 1) / per_chunk;
    dim3 grid((unsigned)strips, (unsigned)chunks);
#define KAPY_STRIP(SRC_, KIND_)                                                                                                       \
  do {                                                                                                                                \
    if (lpr == 32) reduce_cols_strip_kernel<SRC_, KIND_, 32><<<grid, 256, 0, s>>>(p, sh, per_chunk);                                  \
    else reduce_cols_strip_kernel<SRC_, KIND_, 8><<<grid, 256, 0, s>>>(p, sh, per_chunk);                                             \
  } while (0)
    KAPY_BY_SOURCE(KAPY_STRIP);
#undef KAPY_STRIP
  } else if (p.s_keep == 1 && p.s_red != 1) {
    const int64_t strips = ((int64_t)p.n_keep + 63) / 64, want = 4 * (int64_t)device_cus();
    if (strips > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "reduce: more than 2^31 strips of results");
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>({(want + strips - 1) / strips, (int64_t)p.n_red / 64, 512}));
    if (chunks > 1) chunks = std::min(chunks, chunks_allowed(strips, p.n_keep));
    const int32_t per_chunk = (int32_t)((p.n_red + chunks - 1) / chunks);
    chunks = (p.n_red + per_chunk - 1) / per_chunk;
    reduce_cols_any_kernel<<<dim3((unsigned)strips, (unsigned)chunks), 256, 0, s>>>(p, sh, per_chunk);
  }
  else reduce_wave_kernel<<<(p.n_keep + 3) / 4, 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}
#undef KAPY_BY_SOURCE

}  // extern "C"
