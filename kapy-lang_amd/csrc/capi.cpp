// capi.cpp — host-only entry points of the C ABI: library state, descriptors, and the layout
// engine.  Device ops live beside their kernels (copy.hip, elementwise.hip, matmul*.hip, ...).
#include <string.h>

#include <mutex>

#include "common.hpp"
#include <algorithm>
#include <cstring>
#include <string>
#include <utility>
#include <vector>
#include "layout.hpp"

namespace kapy {

char *last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return status;
}

int check_global(const kapy_global *g, const char *what) {
  if (!g) return fail(KAPY_ERR_INVALID, "%s: null descriptor", what);
  if (!g->ptr) return fail(KAPY_ERR_INVALID, "%s: null pointer in descriptor", what);
  if (!dtype_bytes(g->dtype)) return fail(KAPY_ERR_INVALID, "%s: unknown element type %d", what, g->dtype);
  if (g->end0 < g->start0 || g->end1 < g->start1) return fail(KAPY_ERR_INVALID, "%s: end before start", what);
  return KAPY_OK;
}

namespace {
struct DeviceState {
  std::once_flag once;
  int status = KAPY_OK;
  int cus = 0, wave = 0, lds = 0;
  char arch[64] = {0};
  char err[256] = {0};
};
DeviceState g_dev;

void probe_device() {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n == 0) {
    g_dev.status = KAPY_ERR_HIP;
    snprintf(g_dev.err, sizeof g_dev.err, "no HIP device available (%s); this library has no CPU fallback",
             e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    (void)hipGetLastError();
    return;
  }
  int dev = 0;
  hipDeviceProp_t p;
  if ((e = hipGetDevice(&dev)) != hipSuccess || (e = hipGetDeviceProperties(&p, dev)) != hipSuccess) {
    g_dev.status = KAPY_ERR_HIP;
    snprintf(g_dev.err, sizeof g_dev.err, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    return;
  }
  g_dev.cus = p.multiProcessorCount;
  g_dev.wave = p.warpSize;
  g_dev.lds = (int)p.sharedMemPerBlock;
  snprintf(g_dev.arch, sizeof g_dev.arch, "%s", p.gcnArchName);
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    g_dev.status = KAPY_ERR_HIP;
    snprintf(g_dev.err, sizeof g_dev.err, "device is %s; the kernels of this library are built for gfx950 only", p.gcnArchName);
  }
}
}  // namespace

int ensure_device() {
  std::call_once(g_dev.once, probe_device);
  if (g_dev.status != KAPY_OK) return fail(g_dev.status, "%s", g_dev.err);
  return KAPY_OK;
}
int device_cus() { return g_dev.cus > 0 ? g_dev.cus : 256; }

static Fragments to_internal(const kapy_fragments *f) {
  return Fragments{f->lane_array[0], f->lane_array[1], f->lane_loops[0], f->lane_loops[1], f->major_axis};
}
static void to_public(const Fragments &f, kapy_fragments *out) {
  out->lane_array[0] = f.a0;
  out->lane_array[1] = f.a1;
  out->lane_loops[0] = f.l0;
  out->lane_loops[1] = f.l1;
  out->major_axis = f.major;
  out->minor_axis = 1 - f.major;
}
// FragmentsLayoutAttr::verify-style checks: positive powers of two, distinct axes.
static int check_fragments(const kapy_fragments *f, const char *what) {
  if (!f) return fail(KAPY_ERR_INVALID, "%s: null layout", what);
  for (int i = 0; i < 2; ++i) {
    int32_t a = f->lane_array[i], l = f->lane_loops[i];
    if (a <= 0 || (a & (a - 1)) || l <= 0 || (l & (l - 1)))
      return fail(KAPY_ERR_VERIFY, "%s: lane array and lane loops must be positive powers of two", what);
  }
  if (!((f->minor_axis == 0 && f->major_axis == 1) || (f->minor_axis == 1 && f->major_axis == 0)))
    return fail(KAPY_ERR_VERIFY, "%s: (minor, major) must be (0, 1) or (1, 0)", what);
  return KAPY_OK;
}
// Power-of-two static tile shapes (lib/Dialect/Kapy/IR/OpTraits.cpp:43-58).
static int check_shape(const int64_t shape[2], const char *what) {
  if (!shape) return fail(KAPY_ERR_INVALID, "%s: null shape", what);
  for (int i = 0; i < 2; ++i)
    if (shape[i] <= 0 || (shape[i] & (shape[i] - 1)))
      return fail(KAPY_ERR_VERIFY, "%s: tensor shape must be a positive power of two on every axis", what);
  return KAPY_OK;
}

}  // namespace kapy

using namespace kapy;

extern "C" {

int kapy_version(void) { return 100; }
const char *kapy_last_error(void) { return last_error_buffer(); }

int kapy_device_info(int32_t *num_cus, int32_t *wave_size, int32_t *lds_bytes, char *arch, int32_t arch_len) {
  int rc = ensure_device();
  if (rc && g_dev.cus == 0) return rc;
  if (num_cus) *num_cus = g_dev.cus;
  if (wave_size) *wave_size = g_dev.wave;
  if (lds_bytes) *lds_bytes = g_dev.lds;
  if (arch && arch_len > 0) snprintf(arch, (size_t)arch_len, "%s", g_dev.arch);
  return rc;
}

int kapy_mk_global(kapy_global *out, void *ptr, int32_t dynamic_offset, int32_t size0, int32_t size1, int32_t stride0,
                   int32_t stride1, int32_t dtype, int32_t alignment) {
  if (!out || !ptr) return fail(KAPY_ERR_INVALID, "mk_global: null argument");
  int b = dtype_bytes(dtype);
  if (!b) return fail(KAPY_ERR_INVALID, "mk_global: unknown element type %d", dtype);
  if (size0 < 0 || size1 < 0) return fail(KAPY_ERR_INVALID, "mk_global: negative size");
  // kapy.alignment must be a power of two of at least 4 bytes (CoalesceAccess.cpp:181-190); 0 = default 128
  // with the reference's warning (Kapy.cpp:865-872) replaced by silence.
  if (alignment == 0) alignment = 128;
  if (alignment < 0 || (alignment & (alignment - 1))) return fail(KAPY_ERR_VERIFY, "mk_global: alignment must be a power of two");
  out->ptr = (char *)ptr + int64_t(dynamic_offset) * b;
  out->start0 = out->start1 = 0;
  out->end0 = size0;
  out->end1 = size1;
  out->stride0 = stride0;
  out->stride1 = stride1;
  out->dtype = dtype;
  out->alignment = alignment;
  return KAPY_OK;
}

int kapy_sv_global(kapy_global *out, const kapy_global *src, int32_t start0, int32_t end0, int32_t start1, int32_t end1) {
  if (!out) return fail(KAPY_ERR_INVALID, "sv_global: null result");
  int rc = check_global(src, "sv_global source");
  if (rc) return rc;
  if (end0 < start0 || end1 < start1) return fail(KAPY_ERR_INVALID, "sv_global: end before start");
  kapy_global r = *src;
  r.start0 = src->start0 + start0;
  r.start1 = src->start1 + start1;
  r.end0 = src->start0 + end0;
  r.end1 = src->start1 + end1;
  *out = r;
  return KAPY_OK;
}

int kapy_mk_shared(kapy_shared *out, int64_t byte_offset, int32_t size0, int32_t size1, int32_t dtype, int32_t row_major,
                   int32_t bank_param, int32_t line_param) {
  if (!out) return fail(KAPY_ERR_INVALID, "mk_shared: null result");
  int b = dtype_bytes(dtype);
  if (!b) return fail(KAPY_ERR_INVALID, "mk_shared: unknown element type %d", dtype);
  // static power-of-two shapes (OpTraits.cpp:43-58)
  if (size0 <= 0 || size1 <= 0 || (size0 & (size0 - 1)) || (size1 & (size1 - 1)))
    return fail(KAPY_ERR_VERIFY, "mk_shared: shape must be static and every extent a power of two");
  if (byte_offset < 0 || byte_offset % 128) return fail(KAPY_ERR_INVALID, "mk_shared: the offset must be a non-negative multiple of 128 bytes");
  if (bank_param == 0 && line_param == 0) { bank_param = 4; line_param = 1; }  // unswizzled
  if ((bank_param != 4 && bank_param != 2 && bank_param != 1) || line_param < 1 || line_param > kLdsBanks / bank_param || (line_param & (line_param - 1)))
    return fail(KAPY_ERR_INVALID, "mk_shared: swizzling parameters (%d, %d) out of range", bank_param, line_param);
  if (byte_offset + int64_t(size0) * size1 * b > 160 * 1024)
    return fail(KAPY_ERR_VERIFY, "mk_shared: the tensor ends beyond the 160 KiB of a workgroup's shared memory");
  out->offset = byte_offset;
  out->start0 = out->start1 = 0;
  out->end0 = size0;
  out->end1 = size1;
  out->dtype = dtype;
  // row-major strides (size1, 1), column-major (1, size0): Analyze.cpp:82-95
  out->layout.stride0 = row_major ? size1 : 1;
  out->layout.stride1 = row_major ? 1 : size0;
  out->layout.bank_param = bank_param;
  out->layout.line_param = line_param;
  out->layout.rotate = 0;
  return KAPY_OK;
}

int kapy_sv_shared(kapy_shared *out, const kapy_shared *src, int32_t start0, int32_t end0, int32_t start1, int32_t end1) {
  if (!out || !src) return fail(KAPY_ERR_INVALID, "sv_shared: null argument");
  if (end0 < start0 || end1 < start1) return fail(KAPY_ERR_INVALID, "sv_shared: end before start");
  kapy_shared r = *src;  // same base, element type and layout (Kapy.cpp:301-313)
  r.start0 = src->start0 + start0;
  r.start1 = src->start1 + start1;
  r.end0 = src->start0 + end0;
  r.end1 = src->start1 + end1;
  *out = r;
  return KAPY_OK;
}

int64_t kapy_shared_address(const kapy_shared *tensor, int64_t i0, int64_t i1) {
  if (!tensor) return fail(KAPY_ERR_INVALID, "shared_address: null tensor");
  int b = dtype_bytes(tensor->dtype);
  if (!b) return fail(KAPY_ERR_INVALID, "shared_address: unknown element type %d", tensor->dtype);
  // in bounds iff (start + i) <u end on both axes, the unsigned compare of the loads and stores
  const uint32_t a0 = (uint32_t)(tensor->start0 + i0), a1 = (uint32_t)(tensor->start1 + i1);
  if (a0 >= (uint32_t)tensor->end0 || a1 >= (uint32_t)tensor->end1) return KAPY_ERR_VERIFY;
  const Swizzle sw{tensor->layout.stride0, tensor->layout.stride1, tensor->layout.bank_param, tensor->layout.line_param, tensor->layout.rotate};
  return tensor->offset + sw.offset(b * 8, a0, a1) * b;
}

int kapy_fragments_loops(const kapy_fragments *layout, const int64_t shape[2], int64_t warp_loops[2], int64_t loop_space[2]) {
  int rc = check_fragments(layout, "fragments");
  if (rc) return rc;
  if (!shape) return fail(KAPY_ERR_INVALID, "fragments: null shape");
  Fragments f = to_internal(layout);
  Idx2 w = f.warp_loops({shape[0], shape[1]}), s = f.loop_space({shape[0], shape[1]});
  if (warp_loops) { warp_loops[0] = w.v0; warp_loops[1] = w.v1; }
  if (loop_space) { loop_space[0] = s.v0; loop_space[1] = s.v1; }
  return KAPY_OK;
}

int kapy_fragments_map(const kapy_fragments *layout, const int64_t shape[2], int32_t option, const int64_t in[2], int64_t out[2]) {
  int rc = check_fragments(layout, "fragments");
  if (rc) return rc;
  if (!shape || !in || !out) return fail(KAPY_ERR_INVALID, "fragments map: null argument");
  if (option < 1 || option > 3) return fail(KAPY_ERR_INVALID, "fragments map: option must be 1, 2 or 3");
  Fragments f = to_internal(layout);
  Idx2 r = option == 3 ? f.to_lane_iv({shape[0], shape[1]}, in[0], in[1])
                       : f.to_index({shape[0], shape[1]}, in[0], in[1], option == 1);
  out[0] = r.v0;
  out[1] = r.v1;
  return KAPY_OK;
}

int64_t kapy_layout_string(const kapy_fragments *layout, const int64_t shape[2], char *out, int64_t out_len) {
  int rc = check_fragments(layout, "fragments");
  if (rc) return rc;
  if (!shape || shape[0] <= 0 || shape[1] <= 0) return fail(KAPY_ERR_INVALID, "layout string: shape must be positive");
  const Fragments f = to_internal(layout);
  const Idx2 sh{shape[0], shape[1]};
  const int64_t lanes = f.a0 * f.a1, loop_size = f.loop_size(sh), numel = shape[0] * shape[1];
  if (lanes > 9999 || loop_size > 9999) return fail(KAPY_ERR_UNSUPPORTED, "layout string: ids of more than four digits");
  // owners of every element, in (lane, iv) order
  std::vector<std::vector<std::pair<int64_t, int64_t>>> owners((size_t)numel);
  for (int64_t lane = 0; lane < lanes; ++lane)
    for (int64_t iv = 0; iv < loop_size; ++iv) {
      const Idx2 at = f.to_index(sh, lane, iv, true);
      owners[(size_t)(at.v0 * shape[1] + at.v1)].push_back({lane, iv});
    }
  auto width = [](int64_t id) { return id >= 1000 ? 4 : id >= 100 ? 3 : id >= 10 ? 2 : 1; };
  const int lane_w = width(lanes - 1), iv_w = width(loop_size - 1);
  std::string text;
  for (size_t round = 0; round < owners[0].size(); ++round) {
    if (round) text += "\n\n";
    for (int64_t e = 0; e < numel; ++e) {
      if (e % shape[1] == 0) text += e == 0 ? "[[" : "\n [";
      if (round >= owners[(size_t)e].size()) return fail(KAPY_ERR_INVALID, "layout string: elements are not owned equally often");
      const auto &o = owners[(size_t)e][round];
      text.append((size_t)(lane_w - width(o.first)), ' ');
      text += "T" + std::to_string(o.first) + ":";
      text.append((size_t)(iv_w - width(o.second)), ' ');
      text += std::to_string(o.second);
      text += (e + 1) % shape[1] ? ", " : ((e + 1) == numel ? "]]" : "],");
    }
  }
  if (out && out_len > 0) {
    const size_t n = std::min(text.size(), (size_t)out_len - 1);
    memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return (int64_t)text.size();
}

int kapy_fragments_transpose(const kapy_fragments *layout, kapy_fragments *out) {
  int rc = check_fragments(layout, "fragments");
  if (rc) return rc;
  if (!out) return fail(KAPY_ERR_INVALID, "fragments transpose: null result");
  to_public(to_internal(layout).transposed(), out);
  return KAPY_OK;
}

int kapy_fragments_exchange_axes(const kapy_fragments *layout, kapy_fragments *out) {
  int rc = check_fragments(layout, "fragments");
  if (rc) return rc;
  if (!out) return fail(KAPY_ERR_INVALID, "fragments exchange_axes: null result");
  to_public(to_internal(layout).axes_exchanged(), out);
  return KAPY_OK;
}

int kapy_fragments_default(const int64_t lane_loops[2], const int64_t shape[2], int32_t row_major, kapy_fragments *out) {
  if (!lane_loops || !out) return fail(KAPY_ERR_INVALID, "fragments default: null argument");
  int rc = check_shape(shape, "fragments default");
  if (rc) return rc;
  to_public(default_fragments({lane_loops[0], lane_loops[1]}, {shape[0], shape[1]}, row_major != 0), out);
  return KAPY_OK;
}

int64_t kapy_access_simd_size(int64_t alignment, int64_t bits, int64_t numel) {
  if (bits <= 0 || alignment <= 0) return fail(KAPY_ERR_INVALID, "access_simd_size: bits and alignment must be positive");
  return access_simd_size(alignment, bits, numel);
}

int kapy_change_source(const kapy_fragments *src, const kapy_fragments *dst, const int64_t shape[2], int64_t lane,
                       int64_t iv, int64_t *src_lane, int64_t *src_iv) {
  int rc = check_fragments(src, "change source layout");
  if (!rc) rc = check_fragments(dst, "change result layout");
  if (rc) return rc;
  if (!shape || !src_lane || !src_iv) return fail(KAPY_ERR_INVALID, "change: null argument");
  Idx2 r = change_source(to_internal(src), to_internal(dst), {shape[0], shape[1]}, lane, iv);
  *src_lane = r.v0;
  *src_iv = r.v1;
  return KAPY_OK;
}

int64_t kapy_change_num_shuffles(const kapy_fragments *src, const kapy_fragments *dst, const int64_t shape[2]) {
  int rc = check_fragments(src, "change source layout");
  if (!rc) rc = check_fragments(dst, "change result layout");
  if (rc) return rc;
  if (!shape) return fail(KAPY_ERR_INVALID, "change: null shape");
  Fragments s = to_internal(src), d = to_internal(dst);
  Idx2 sh{shape[0], shape[1]};
  int64_t n = d.loop_size(sh), ns = s.loop_size(sh);
  // distinct source ivs that some lane must fetch from another lane
  int64_t distinct = 0;
  bool *needs = new bool[(size_t)ns]();
  for (int64_t lane = 0; lane < kWaveSize; ++lane)
    for (int64_t iv = 0; iv < n; ++iv) {
      Idx2 r = change_source(s, d, sh, lane, iv);
      if (r.v0 != lane && r.v1 >= 0 && r.v1 < ns && !needs[r.v1]) {
        needs[r.v1] = true;
        ++distinct;
      }
    }
  delete[] needs;
  return n * distinct;
}

int64_t kapy_swizzle_offset(const kapy_swizzling *layout, int64_t bits, int64_t i0, int64_t i1) {
  if (!layout || layout->bank_param <= 0 || layout->line_param <= 0 || bits <= 0)
    return fail(KAPY_ERR_INVALID, "swizzle_offset: bad layout");
  if (layout->rotate < 0) return fail(KAPY_ERR_INVALID, "swizzle_offset: bad layout");
  return Swizzle{layout->stride0, layout->stride1, layout->bank_param, layout->line_param, layout->rotate}.offset(bits, i0, i1);
}

int kapy_swizzle_search(const kapy_fragments *access, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                        int64_t alignment, int32_t *pairs, int32_t max_pairs) {
  int rc = check_fragments(access, "swizzle search access layout");
  if (rc) return rc;
  if (!shape || (max_pairs > 0 && !pairs)) return fail(KAPY_ERR_INVALID, "swizzle search: null argument");
  // a contiguous axis must exist (CoalesceAccess.cpp:38-40)
  if (stride0 != 1 && stride1 != 1) return fail(KAPY_ERR_VERIFY, "swizzle search: can not find a contiguous axis");
  return swizzle_search(to_internal(access), {shape[0], shape[1]}, (int32_t)stride0, (int32_t)stride1, bits, alignment, pairs,
                        max_pairs);
}

int kapy_swizzle_search_gfx950(const kapy_fragments *access, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                               int64_t alignment, int32_t *triples, int32_t max_triples) {
  int rc = check_fragments(access, "swizzle search access layout");
  if (rc) return rc;
  if (!shape || (max_triples > 0 && !triples)) return fail(KAPY_ERR_INVALID, "swizzle search: null argument");
  if (stride0 != 1 && stride1 != 1) return fail(KAPY_ERR_VERIFY, "swizzle search: can not find a contiguous axis");
  if (access->lane_array[0] * access->lane_array[1] != kWaveSize)
    return fail(KAPY_ERR_VERIFY, "swizzle search: the read phases of gfx950 are phases of a 64-lane wavefront; the access layout has %d lanes",
                access->lane_array[0] * access->lane_array[1]);
  return swizzle_search_gfx950(to_internal(access), {shape[0], shape[1]}, (int32_t)stride0, (int32_t)stride1, bits, alignment, triples, max_triples);
}

int kapy_matmul_layouts(int32_t impl_way, int32_t which, kapy_fragments *out, int32_t mnk[3]) {
  MfmaShape s;
  switch (impl_way) {
  case KAPY_MFMA_32X32X16_16B: s = kMfma32x32x16; break;
  case KAPY_MFMA_16X16X32_16B: case KAPY_MMA_M16N8K8_F16: case KAPY_MMA_M16N8K16_F16: s = kMfma16x16x32; break;
  case KAPY_MFMA_16X16X128_F8: case KAPY_MMA_M16N8K16_F8: s = kMfma16x16x128F8; break;
  case KAPY_MFMA_32X32X64_F8: s = kMfma32x32x64F8; break;
  case KAPY_MMA_M16N8K8_TF32:
    return fail(KAPY_ERR_UNSUPPORTED, "mma_m16n8k8_tf32: gfx950 has no tf32 matrix instruction");
  default: return fail(KAPY_ERR_INVALID, "matmul layouts: unknown implement way %d", impl_way);
  }
  if (which < 0 || which > 3 || !out)
    return fail(KAPY_ERR_INVALID, "matmul layouts: which must be 0 (lhs), 1 (rhs), 2 (acc) or 3 (acc with the operands exchanged)");
  to_public(which == 0 ? mfma_lhs(s) : which == 1 ? mfma_rhs(s) : which == 2 ? mfma_acc(s) : mfma_acc_exchanged(s), out);
  if (mnk) { mnk[0] = s.m; mnk[1] = s.n; mnk[2] = s.k; }
  return KAPY_OK;
}

}  // extern "C"
