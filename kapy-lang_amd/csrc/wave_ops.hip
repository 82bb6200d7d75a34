// wave_ops.hip — cross-lane ops of one wavefront: kgpu.change (register re-layout by shuffles)
// and kapy.reduce (butterfly reduction).
//
// Reference: ChangeOpToLLVM.cpp:21-93 — result (lane, iv) takes the value of source
// (lane', iv') = srcMap3(dstMap2(lane, iv)); every source iv that some lane needs from another
// lane is shuffled with shfl.sync.idx and a select chain keeps the one whose iv' matches.
// ReduceOpToLLVM.cpp:51-172 — an in-lane tree over the loop ivs, then shfl.sync.bfly rounds over
// the lanes that share the reduced axis.  On gfx950 the shuffles are ds_bpermute_b32 over 64 lanes.
#include <algorithm>
#include <mutex>

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
  int32_t src_dtype, dst_dtype, kind;
};

__device__ __forceinline__ float combine(float a, float b, int kind) {
  if (kind == 0) return a + b;
  return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b);
}

// A sum starts from -0, the identity of IEEE addition (-0 + x = x for every x, -0 included): the result is that of folding
// the elements themselves, as ReduceOpToLLVM.cpp:60-101 does, and a line of only -0 sums to -0.
// One wavefront per kept index: lanes stride over the reduced axis, then 6 butterfly rounds.
__global__ __launch_bounds__(256) void reduce_wave_kernel(ReduceParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t keep = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (keep >= p.n_keep) return;
  float acc = p.kind == 0 ? -0.f : -__builtin_inff();
  int32_t r = lane;
  for (; r + 192 < p.n_red; r += 256) {  // four loads in flight
    float f[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) f[u] = load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)(r + 64 * u) * p.s_red);
#pragma unroll
    for (int u = 0; u < 4; ++u) acc = combine(acc, f[u], p.kind);
  }
  for (; r < p.n_red; r += 64) acc = combine(acc, load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)r * p.s_red), p.kind);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ off) << 2, (int)f32_bits(acc)));
    acc = combine(acc, other, p.kind);
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
template <int SRC>
__device__ __forceinline__ float fold_vec(const float (&f)[per_vec<SRC>()], int kind) {
  if constexpr (SRC == 2) return combine(combine(f[0], f[1], kind), combine(f[2], f[3], kind), kind);
  else return combine(combine(combine(f[0], f[1], kind), combine(f[2], f[3], kind), kind), combine(combine(f[4], f[5], kind), combine(f[6], f[7], kind), kind), kind);
}
template <int SRC, int KIND>
__global__ __launch_bounds__(256) void reduce_rows_vec_kernel(ReduceParams p, float *partials, int32_t vecs_per_chunk) {
  const int lane = threadIdx.x & 63;
  const int64_t keep = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (keep >= p.n_keep) return;
  constexpr int E = per_vec<SRC>();
  const u32x4_t *row = (const u32x4_t *)(p.src + keep * p.s_keep * (16 / E));
  const int32_t vecs = min(p.n_red / E, (int32_t)(blockIdx.y + 1) * vecs_per_chunk);
  float acc = KIND == 0 ? -0.f : -__builtin_inff();
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
      const float t = fold_vec<SRC>(f, KIND);
      acc = combine(acc, t, KIND);
    }
  }
  for (; v < vecs; v += 64) {
    float f[E];
    widen<SRC>(__builtin_nontemporal_load(row + v), f);
#pragma unroll
    for (int e = 0; e < E; ++e) acc = combine(acc, f[e], KIND);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ off) << 2, (int)f32_bits(acc)));
    acc = combine(acc, other, KIND);
  }
  if (lane == 0) {
    if (partials) partials[keep * gridDim.y + blockIdx.y] = acc;
    else store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
  }
}

// The same for lines of up to 512 elements: a line takes GROUP lanes (8, 16, 32 or 64: the next power of two from its
// vectors), a wave 64 / GROUP lines at a time, each lane one 128-bit load; the butterfly stays inside the group.
template <int SRC, int KIND, int GROUP>
__global__ __launch_bounds__(256) void reduce_rows_short_kernel(ReduceParams p) {
  const int64_t keep = (int64_t)blockIdx.x * (256 / GROUP) + threadIdx.x / GROUP;
  const int32_t jv = threadIdx.x % GROUP;
  float acc = KIND == 0 ? -0.f : -__builtin_inff();
  constexpr int E = per_vec<SRC>();
  if (keep < p.n_keep && jv < p.n_red / E) {
    float f[E];
    widen<SRC>(__builtin_nontemporal_load((const u32x4_t *)(p.src + keep * p.s_keep * (16 / E)) + jv), f);
    acc = fold_vec<SRC>(f, KIND);
  }
#pragma unroll
  for (int off = GROUP / 2; off >= 1; off >>= 1) {
    float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute(((threadIdx.x & 63) ^ off) << 2, (int)f32_bits(acc)));
    acc = combine(acc, other, KIND);
  }
  if (jv == 0 && keep < p.n_keep) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
}

// 16-bit elements, kept axis contiguous: a workgroup of 256 lanes owns a strip of 8 * LPR kept indices - LPR lanes x one
// 128-bit load per reduced index - and a chunk of the reduced axis, which its 256 / LPR groups of lanes walk with four
// loads in flight each; the groups' partial results meet in LDS.  With one chunk the strip's results go to the result;
// with more (few kept indices, many reduced ones: a tall matrix would otherwise keep a handful of CUs busy) every chunk
// leaves an fp32 partial line and reduce_partials_kernel folds the lines in chunk order.
template <int SRC, int KIND, int LPR>
__global__ __launch_bounds__(256) void reduce_cols_strip_kernel(ReduceParams p, float *partials, int32_t per_chunk) {
  constexpr int E = per_vec<SRC>(), EB = 16 / E, GROUPS = 256 / LPR, COLS = LPR * E;
  __shared__ float part[GROUPS][COLS + 1];
  const int cl = threadIdx.x % LPR, rg = threadIdx.x / LPR;
  const int64_t keep0 = (int64_t)blockIdx.x * COLS + cl * E;
  const int32_t r_begin = blockIdx.y * per_chunk, r_end = min(p.n_red, r_begin + per_chunk);
  float acc[E];
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = KIND == 0 ? -0.f : -__builtin_inff();
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
        for (int e = 0; e < E; ++e) acc[e] = combine(acc[e], f[e], KIND);
      }
    }
    for (; r < r_end; r += GROUPS) {
      float f[E];
      widen<SRC>(__builtin_nontemporal_load((const u32x4_t *)(col + (int64_t)r * p.s_red * EB)), f);
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] = combine(acc[e], f[e], KIND);
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) part[rg][cl * E + e] = acc[e];
  __syncthreads();
  const int64_t keep = (int64_t)blockIdx.x * COLS + threadIdx.x;
  if (threadIdx.x < COLS && keep < p.n_keep) {
    float t = KIND == 0 ? -0.f : -__builtin_inff();
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) t = combine(t, part[g][threadIdx.x], KIND);
    if (partials) partials[(int64_t)blockIdx.y * p.n_keep + keep] = t;
    else store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
  }
}

// The second pass over `chunks` fp32 partial lines of n_keep values: 64 kept indices per workgroup, 16 groups of lanes
// share out the lines, folded in chunk order within a group and in group order across them (the same result every run).
template <int KIND>
__global__ __launch_bounds__(1024) void reduce_partials_kernel(ReduceParams p, const float *partials, int32_t chunks) {
  __shared__ float part[16][64 + 1];
  const int cl = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int64_t keep = (int64_t)blockIdx.x * 64 + cl;
  float acc = KIND == 0 ? -0.f : -__builtin_inff();
  if (keep < p.n_keep)
    for (int32_t c = rg; c < chunks; c += 16) acc = combine(acc, partials[(int64_t)c * p.n_keep + keep], KIND);
  part[rg][cl] = acc;
  __syncthreads();
  if (threadIdx.x < 64 && keep < p.n_keep) {
    float t = KIND == 0 ? -0.f : -__builtin_inff();
#pragma unroll
    for (int g = 0; g < 16; ++g) t = combine(t, part[g][cl], KIND);
    store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
  }
}

// Memory for the partial lines: one block per device, allocated at the first call that wants it and kept.  Calls on one
// stream use it in turn by stream order; a call on another stream first makes its stream wait for the event that the last
// user recorded behind its second pass.  The mutex is held from that wait to the new record, so calls from several host
// threads cannot interleave.  Not available - and then the caller reduces in one pass - while the stream is being
// captured (an event of another stream's work cannot be waited for inside a capture) or when the allocation fails.
constexpr int kMaxPartialsDevices = 16;
constexpr size_t kPartialsBytes = size_t(4) << 20;  // the launches keep what they leave there within this
struct Partials {
  float *lines = nullptr;
  hipEvent_t free_again = nullptr;
  hipStream_t last_stream = nullptr;
  bool used = false;
  int state = 0;  // 0 not tried, 1 ready, -1 not available
};
std::mutex partials_mutex;
Partials partials_of[kMaxPartialsDevices];

// Call with partials_mutex held.  The device's block, ready for work on `s`, or nullptr.
Partials *partials_for(hipStream_t s) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxPartialsDevices) return nullptr;
  Partials &P = partials_of[dev];
  if (P.state == 0) {
    if (hipMalloc((void **)&P.lines, kPartialsBytes) == hipSuccess && hipEventCreateWithFlags(&P.free_again, hipEventDisableTiming) == hipSuccess) P.state = 1;
    else {
      (void)hipGetLastError();
      P.state = -1;
    }
  }
  if (P.state != 1) return nullptr;
  if (P.used && P.last_stream != s && hipStreamWaitEvent(s, P.free_again, 0) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return &P;
}

// The block for a call that wants `chunks` > 1 partial lines, with `lock` taken - or nullptr, chunks = 1 and no lock.
Partials *take_partials(int64_t &chunks, std::unique_lock<std::mutex> &lock, hipStream_t s) {
  Partials *P = nullptr;
  if (chunks > 1) {
    lock.lock();
    P = partials_for(s);
    if (!P) lock.unlock();
  }
  if (!P) chunks = 1;
  return P;
}

// After the call's launches (lock still held): whatever was launched reads or writes the block, so the next user waits for
// all of it.
int partials_used(Partials *P, hipStream_t s) {
  const hipError_t launched = hipGetLastError(), recorded = hipEventRecord(P->free_again, s);
  P->last_stream = s;
  P->used = true;
  if (launched != hipSuccess) return fail(KAPY_ERR_HIP, "reduce: %s", hipGetErrorString(launched));
  if (recorded != hipSuccess) {
    P->state = -1;  // nobody could wait for this call's use of the block: it is not handed out again
    return fail(KAPY_ERR_HIP, "reduce: hipEventRecord: %s", hipGetErrorString(recorded));
  }
  return KAPY_OK;
}

}  // namespace

// The same block for the column programs of kapy_elementwise (elementwise.hip): acquire returns it ready for work on `s`
// with the mutex held, or nullptr (then nothing is held); release, after the caller's last launch that touches it, records
// the event the next user waits for and lets go of the mutex.
float *partials_acquire(hipStream_t s, size_t *bytes) {
  partials_mutex.lock();
  Partials *P = partials_for(s);
  if (!P) {
    partials_mutex.unlock();
    return nullptr;
  }
  *bytes = kPartialsBytes;
  return P->lines;
}
int partials_release(hipStream_t s) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  const int rc = partials_used(&partials_of[dev], s);
  partials_mutex.unlock();
  return rc;
}

namespace {

// Any element type, alignment and extents, kept axis contiguous (or at least not the strided one): a workgroup owns 64 kept
// indices, one per lane of a wave (a wave's loads cover 64 consecutive elements of one reduced index), its four waves share
// out a chunk of the reduced axis with four loads in flight each and meet in LDS; chunks as in reduce_cols_strip_kernel.
__global__ __launch_bounds__(256) void reduce_cols_any_kernel(ReduceParams p, float *partials, int32_t per_chunk) {
  __shared__ float part[4][64];
  const int cl = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int64_t keep = (int64_t)blockIdx.x * 64 + cl;
  const int32_t r_begin = blockIdx.y * per_chunk, r_end = min(p.n_red, r_begin + per_chunk);
  float acc = p.kind == 0 ? -0.f : -__builtin_inff();
  if (keep < p.n_keep) {
    int32_t r = r_begin + rg;
    for (; r + 12 < r_end; r += 16) {
      float f[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) f[u] = load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)(r + 4 * u) * p.s_red);
#pragma unroll
      for (int u = 0; u < 4; ++u) acc = combine(acc, f[u], p.kind);
    }
    for (; r < r_end; r += 4) acc = combine(acc, load_as_f32(p.src, p.src_dtype, keep * p.s_keep + (int64_t)r * p.s_red), p.kind);
  }
  part[rg][cl] = acc;
  __syncthreads();
  if (rg == 0 && keep < p.n_keep) {
    float t = combine(combine(part[0][cl], part[1][cl], p.kind), combine(part[2][cl], part[3][cl], p.kind), p.kind);
    if (partials) partials[(int64_t)blockIdx.y * p.n_keep + keep] = t;
    else store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, t);
  }
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

// LAUNCH(source kind, reduce kind) for the call's source type and reduce kind
#define KAPY_BY_SOURCE(LAUNCH)                                                                  \
  do {                                                                                          \
    if (src_kind == 0) { if (kind == 0) LAUNCH(0, 0); else LAUNCH(0, 1); }                      \
    else if (src_kind == 1) { if (kind == 0) LAUNCH(1, 0); else LAUNCH(1, 1); }                 \
    else { if (kind == 0) LAUNCH(2, 0); else LAUNCH(2, 1); }                                    \
  } while (0)

int kapy_reduce(const kapy_global *src, const kapy_global *dst, int32_t axis, int32_t kind, void *stream) {
  int rc = check_global(src, "reduce source");
  if (!rc) rc = check_global(dst, "reduce result");
  if (rc) return rc;
  if (axis != 0 && axis != 1) return fail(KAPY_ERR_VERIFY, "reduce: axis must be 0 or 1");
  if (kind != 0 && kind != 1) return fail(KAPY_ERR_INVALID, "reduce: kind must be 0 (sum) or 1 (max)");
  const int64_t s0 = extent0(src), s1 = extent1(src);
  // Kapy.cpp ReduceOp::verify: the result keeps the other axis and has one element along `axis`
  if (axis == 1 ? (extent1(dst) != 1 || extent0(dst) != s0) : (extent0(dst) != 1 || extent1(dst) != s1))
    return fail(KAPY_ERR_VERIFY, "reduce: number of elements in result is incorrect");
  if (!is_float(src->dtype) || is_f8(src->dtype) || !is_float(dst->dtype) || is_f8(dst->dtype))
    return fail(KAPY_ERR_UNSUPPORTED, "reduce: only f16, bf16 and f32 tensors are supported");
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
  // the vector kernels: f16, bf16 or f32 source read in 128-bit pieces of E elements
  const bool vec_ok = src->dtype == KAPY_F16 || src->dtype == KAPY_BF16 || src->dtype == KAPY_F32;
  const int src_kind = src->dtype == KAPY_F32 ? 2 : src->dtype == KAPY_BF16 ? 1 : 0, E = src_kind == 2 ? 4 : 8, EB = 16 / E;
  const bool aligned = ((uintptr_t)p.src & 15) == 0;
  std::unique_lock<std::mutex> lock(partials_mutex, std::defer_lock);
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
    // up to four workgroups per CU (their partial results within the block): 64 lines of 1 Mi elements 312 -> 33 us, 256
    // lines of 256 Ki 82 -> 30 us.  The second launch costs about 6 us: 1024 lines of 64 Ki elements are faster whole.
    const int64_t wgs = ((int64_t)p.n_keep + 3) / 4, want = 4 * (int64_t)device_cus(), vecs = p.n_red / E;
    int64_t chunks = wgs >= device_cus() ? 1 : std::max<int64_t>(1, std::min<int64_t>({(want + wgs - 1) / wgs, vecs / 256, 512, (int64_t)(kPartialsBytes / sizeof(float)) / p.n_keep}));
    Partials *P = take_partials(chunks, lock, s);
    const int32_t vecs_per_chunk = (int32_t)((vecs + chunks - 1) / chunks);
    chunks = (vecs + vecs_per_chunk - 1) / vecs_per_chunk;
    float *lines = P ? P->lines : nullptr;
    dim3 grid((unsigned)wgs, (unsigned)chunks);
#define KAPY_ROWS(SRC_, KIND_) reduce_rows_vec_kernel<SRC_, KIND_><<<grid, 256, 0, s>>>(p, lines, vecs_per_chunk)
    KAPY_BY_SOURCE(KAPY_ROWS);
#undef KAPY_ROWS
    if (P) {
      // the partial results as an fp32 source of n_keep lines of `chunks` values: one wave per line folds them
      ReduceParams q = p;
      q.src = (const char *)lines;
      q.s_keep = chunks;
      q.s_red = 1;
      q.n_red = (int32_t)chunks;
      q.src_dtype = KAPY_F32;
      reduce_wave_kernel<<<(p.n_keep + 3) / 4, 256, 0, s>>>(q);
      return partials_used(P, s);
    }
  } else if (vec_ok && aligned && p.s_keep == 1 && p.n_keep % E == 0 && (p.s_red * EB) % 16 == 0 && p.n_red >= 32) {
    // strips of 256 kept indices (512-byte runs per reduced index), of 64 for narrow sources; the reduced axis in as many
    // chunks as bring the launch to about four workgroups per CU, of at least 128 reduced indices each, as far as their
    // partial lines fit the block.  Measured for 128 MiB of fp16: 8192 x 8192 46 -> 29 us (64-wide strips: 31, eight
    // workgroups per CU: 31, eight loads in flight per lane: 30), 1 Mi x 64 4335 -> 34 us.
    const int lpr = p.n_keep >= 32 * E ? 32 : 8, cols = lpr * E;
    const int64_t strips = ((int64_t)p.n_keep + cols - 1) / cols, want = 4 * (int64_t)device_cus();
    if (strips > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "reduce: more than 2^31 strips of results");
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>({(want + strips - 1) / strips, (int64_t)p.n_red / 128, 512, (int64_t)(kPartialsBytes / sizeof(float)) / p.n_keep}));
    Partials *P = take_partials(chunks, lock, s);
    const int32_t per_chunk = (int32_t)((p.n_red + chunks - 1) / chunks);
    chunks = (p.n_red + per_chunk - 1) / per_chunk;
    float *lines = P ? P->lines : nullptr;
    dim3 grid((unsigned)strips, (unsigned)chunks);
#define KAPY_STRIP(SRC_, KIND_)                                                                                                       \
  do {                                                                                                                                \
    if (lpr == 32) reduce_cols_strip_kernel<SRC_, KIND_, 32><<<grid, 256, 0, s>>>(p, lines, per_chunk);                               \
    else reduce_cols_strip_kernel<SRC_, KIND_, 8><<<grid, 256, 0, s>>>(p, lines, per_chunk);                                          \
  } while (0)
    KAPY_BY_SOURCE(KAPY_STRIP);
#undef KAPY_STRIP
    if (P) {
      if (kind == 0) reduce_partials_kernel<0><<<dim3((unsigned)((p.n_keep + 63) / 64)), 1024, 0, s>>>(p, lines, (int32_t)chunks);
      else reduce_partials_kernel<1><<<dim3((unsigned)((p.n_keep + 63) / 64)), 1024, 0, s>>>(p, lines, (int32_t)chunks);
      return partials_used(P, s);
    }
  } else if (p.s_keep == 1 && p.s_red != 1) {
    const int64_t strips = ((int64_t)p.n_keep + 63) / 64, want = 4 * (int64_t)device_cus();
    if (strips > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "reduce: more than 2^31 strips of results");
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>({(want + strips - 1) / strips, (int64_t)p.n_red / 64, 512, (int64_t)(kPartialsBytes / sizeof(float)) / p.n_keep}));
    Partials *P = take_partials(chunks, lock, s);
    const int32_t per_chunk = (int32_t)((p.n_red + chunks - 1) / chunks);
    chunks = (p.n_red + per_chunk - 1) / per_chunk;
    float *lines = P ? P->lines : nullptr;
    reduce_cols_any_kernel<<<dim3((unsigned)strips, (unsigned)chunks), 256, 0, s>>>(p, lines, per_chunk);
    if (P) {
      if (kind == 0) reduce_partials_kernel<0><<<dim3((unsigned)strips), 1024, 0, s>>>(p, lines, (int32_t)chunks);
      else reduce_partials_kernel<1><<<dim3((unsigned)strips), 1024, 0, s>>>(p, lines, (int32_t)chunks);
      return partials_used(P, s);
    }
  }
  else reduce_wave_kernel<<<(p.n_keep + 3) / 4, 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}
#undef KAPY_BY_SOURCE

}  // extern "C"
