// wave_ops.hip — cross-lane ops of one wavefront: kgpu.change (register re-layout by shuffles)
// and kapy.reduce (butterfly reduction).
//
// Reference: ChangeOpToLLVM.cpp:21-93 — result (lane, iv) takes the value of source
// (lane', iv') = srcMap3(dstMap2(lane, iv)); every source iv that some lane needs from another
// lane is shuffled with shfl.sync.idx and a select chain keeps the one whose iv' matches.
// ReduceOpToLLVM.cpp:51-172 — an in-lane tree over the loop ivs, then shfl.sync.bfly rounds over
// the lanes that share the reduced axis.  On gfx950 the shuffles are ds_bpermute_b32 over 64 lanes.
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

// One wavefront per kept index: lanes stride over the reduced axis, then 6 butterfly rounds.
__global__ __launch_bounds__(256) void reduce_wave_kernel(ReduceParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t keep = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (keep >= p.n_keep) return;
  float acc = p.kind == 0 ? 0.f : -__builtin_inff();
  for (int32_t r = lane; r < p.n_red; r += 64) acc = combine(acc, load_as_f32(p.src, p.src_dtype, keep * p.s_keep + r * p.s_red), p.kind);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    float other = bits_f32((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ off) << 2, (int)f32_bits(acc)));
    acc = combine(acc, other, p.kind);
  }
  if (lane == 0) store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
}

// One lane per kept index: used when the kept axis is the contiguous one (coalesced as is).
__global__ __launch_bounds__(256) void reduce_lane_kernel(ReduceParams p) {
  const int64_t keep = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (keep >= p.n_keep) return;
  float acc = p.kind == 0 ? 0.f : -__builtin_inff();
  for (int32_t r = 0; r < p.n_red; ++r) acc = combine(acc, load_as_f32(p.src, p.src_dtype, keep * p.s_keep + r * p.s_red), p.kind);
  store_from_f32(p.dst, p.dst_dtype, keep * p.d_keep, acc);
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
  if (p.s_keep == 1 && p.s_red != 1) reduce_lane_kernel<<<(p.n_keep + 255) / 256, 256, 0, s>>>(p);
  else reduce_wave_kernel<<<(p.n_keep + 3) / 4, 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // extern "C"
