// kapy_oracle.cpp — CPU restatement of the kapy-lang op semantics.  TEST INFRASTRUCTURE ONLY:
// the product library never links or calls this file.  See kapy_oracle.h for what pins each part.
//
// Citations are file:line inside the kapy-lang tree.
#include "kapy_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <map>
#include <set>
#include <string>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---------------------------------------------------------------------------------------------
// Small-float codec.  One parameterised encoder covers f16, bf16, e5m2 (IEEE-like, with inf) and
// e4m3fn (OCP: no inf, NaN = S.1111.111, max finite 448).  Down-casts carry RN (ties-to-even) or
// RZ (Enums.td:102-109); casts to fp8 saturate to the largest finite value
// (cvt.rn.satfinite, ElementwiseOpToLLVM.cpp:238-276).
// ---------------------------------------------------------------------------------------------
struct Fmt {
  int ebits, mbits, bias;
  bool has_inf;   // exponent field all-ones encodes inf/NaN (IEEE style)
  bool saturate;  // overflow clamps to max finite instead of producing inf
  double max_finite;
  uint32_t nan_bits;
};
const Fmt kF16{5, 10, 15, true, false, 65504.0, 0x7E00};
const Fmt kBF16{8, 7, 127, true, false, 3.3895313892515355e38, 0x7FC0};
const Fmt kE5M2{5, 2, 15, true, true, 57344.0, 0x7F};
const Fmt kE4M3{4, 3, 7, false, true, 448.0, 0x7F};

uint32_t encode_small(double x, const Fmt &f, int rmode) {
  const uint32_t sign_bit = 1u << (f.ebits + f.mbits);
  if (std::isnan(x)) return f.nan_bits;
  uint32_t sign = std::signbit(x) ? sign_bit : 0u;
  double a = std::fabs(x);
  const uint32_t inf_bits = ((1u << f.ebits) - 1u) << f.mbits;
  auto max_bits = [&]() -> uint32_t {
    int e;
    double fr = std::frexp(f.max_finite, &e);  // max = fr * 2^e, fr in [0.5,1)
    uint32_t efield = (uint32_t)(e - 1 + f.bias);
    uint32_t mant = (uint32_t)std::llround((fr * 2.0 - 1.0) * (double)(1u << f.mbits));
    return (efield << f.mbits) | mant;
  };
  if (std::isinf(a)) return sign | ((f.saturate || !f.has_inf) ? max_bits() : inf_bits);
  if (a == 0.0) return sign;
  int e;
  std::frexp(a, &e);
  int ue = e - 1;  // a = 1.xxx * 2^ue
  const int emin = 1 - f.bias;
  int qexp = (ue < emin ? emin : ue) - f.mbits;  // exponent of the rounding quantum
  double q = std::ldexp(a, -qexp);               // exact: power-of-two scaling
  double r = std::floor(q);
  double frac = q - r;
  if (rmode == KO_RN) {
    if (frac > 0.5 || (frac == 0.5 && std::fmod(r, 2.0) == 1.0)) r += 1.0;
  }
  double v = std::ldexp(r, qexp);
  if (v > f.max_finite) return sign | ((f.saturate || !f.has_inf || rmode == KO_RZ) ? max_bits() : inf_bits);
  if (v == 0.0) return sign;
  int e2;
  double fr2 = std::frexp(v, &e2);
  int ue2 = e2 - 1;
  if (ue2 < emin) {  // subnormal
    uint32_t mant = (uint32_t)std::llround(std::ldexp(v, -(emin - f.mbits)));
    return sign | mant;
  }
  uint32_t efield = (uint32_t)(ue2 + f.bias);
  uint32_t mant = (uint32_t)std::llround((fr2 * 2.0 - 1.0) * (double)(1u << f.mbits));
  return sign | (efield << f.mbits) | mant;
}

double decode_small(uint32_t bits, const Fmt &f) {
  const uint32_t sign_bit = 1u << (f.ebits + f.mbits);
  bool neg = bits & sign_bit;
  uint32_t efield = (bits >> f.mbits) & ((1u << f.ebits) - 1u);
  uint32_t mant = bits & ((1u << f.mbits) - 1u);
  double v;
  if (f.has_inf && efield == (1u << f.ebits) - 1u) {
    v = mant ? std::numeric_limits<double>::quiet_NaN() : std::numeric_limits<double>::infinity();
  } else if (!f.has_inf && efield == (1u << f.ebits) - 1u && mant == (1u << f.mbits) - 1u) {
    v = std::numeric_limits<double>::quiet_NaN();
  } else if (efield == 0) {
    v = std::ldexp((double)mant, 1 - f.bias - f.mbits);
  } else {
    v = std::ldexp(1.0 + (double)mant / (double)(1u << f.mbits), (int)efield - f.bias);
  }
  return neg ? -v : v;
}

float f64_to_f32_mode(double x, int rmode) {
  float r = (float)x;  // RN-even
  if (rmode == KO_RZ && std::isfinite(x)) {
    if (std::isinf(r)) return std::copysign(std::numeric_limits<float>::max(), r);
    if (std::fabs((double)r) > std::fabs(x)) r = std::nextafterf(r, 0.0f);
  }
  return r;
}

inline int dtype_bytes(int dtype) {
  switch (dtype) {
  case KO_F16: case KO_BF16: case KO_I16: return 2;
  case KO_F32: case KO_I32: return 4;
  case KO_F8E4M3: case KO_F8E5M2: case KO_I8: case KO_I1: return 1;
  }
  return 0;
}

inline int64_t elem_offset(const ko_global *g, int64_t i, int64_t j) {
  return ((int64_t)g->start0 + i) * g->stride0 + ((int64_t)g->start1 + j) * g->stride1;
}
// Predicate of LdGlobalOpToLLVM.cpp:84-97 / StGlobalOpToLLVM.cpp: unsigned compares on i32.
inline bool in_bounds(const ko_global *g, int64_t i, int64_t j) {
  uint32_t a = (uint32_t)(g->start0 + (int32_t)i), b = (uint32_t)(g->start1 + (int32_t)j);
  return a < (uint32_t)g->end0 && b < (uint32_t)g->end1;
}
inline int64_t extent0(const ko_global *g) { return (int64_t)g->end0 - g->start0; }
inline int64_t extent1(const ko_global *g) { return (int64_t)g->end1 - g->start1; }

double padding_value(int dtype, int padding) {
  switch (padding) {
  case KO_PAD_QNAN: return std::numeric_limits<double>::quiet_NaN();
  case KO_PAD_PINF: return std::numeric_limits<double>::infinity();
  case KO_PAD_NINF: return -std::numeric_limits<double>::infinity();
  }
  (void)dtype;
  return 0.0;
}

}  // namespace

extern "C" {

int ko_dtype_bits(int dtype) { return dtype_bytes(dtype) * 8; }

uint16_t ko_f64_to_f16(double x, int rmode) { return (uint16_t)encode_small(x, kF16, rmode); }
uint16_t ko_f64_to_bf16(double x, int rmode) { return (uint16_t)encode_small(x, kBF16, rmode); }
uint8_t ko_f64_to_e4m3(double x, int rmode) { return (uint8_t)encode_small(x, kE4M3, rmode); }
uint8_t ko_f64_to_e5m2(double x, int rmode) { return (uint8_t)encode_small(x, kE5M2, rmode); }
float ko_f64_to_f32(double x, int rmode) { return f64_to_f32_mode(x, rmode); }
double ko_f16_to_f64(uint16_t h) { return decode_small(h, kF16); }
double ko_bf16_to_f64(uint16_t h) { return decode_small(h, kBF16); }
double ko_e4m3_to_f64(uint8_t b) { return decode_small(b, kE4M3); }
double ko_e5m2_to_f64(uint8_t b) { return decode_small(b, kE5M2); }

double ko_decode(const void *p, int dtype, int64_t idx) {
  switch (dtype) {
  case KO_F16: return decode_small(((const uint16_t *)p)[idx], kF16);
  case KO_BF16: return decode_small(((const uint16_t *)p)[idx], kBF16);
  case KO_F32: return (double)((const float *)p)[idx];
  case KO_F8E4M3: return decode_small(((const uint8_t *)p)[idx], kE4M3);
  case KO_F8E5M2: return decode_small(((const uint8_t *)p)[idx], kE5M2);
  case KO_I8: return (double)((const int8_t *)p)[idx];
  case KO_I16: return (double)((const int16_t *)p)[idx];
  case KO_I32: return (double)((const int32_t *)p)[idx];
  case KO_I1: return (double)(((const uint8_t *)p)[idx] & 1);
  }
  return 0.0;
}

void ko_encode(void *p, int dtype, int64_t idx, double v, int rmode) {
  switch (dtype) {
  case KO_F16: ((uint16_t *)p)[idx] = (uint16_t)encode_small(v, kF16, rmode); break;
  case KO_BF16: ((uint16_t *)p)[idx] = (uint16_t)encode_small(v, kBF16, rmode); break;
  case KO_F32: ((float *)p)[idx] = f64_to_f32_mode(v, rmode); break;
  case KO_F8E4M3: ((uint8_t *)p)[idx] = (uint8_t)encode_small(v, kE4M3, rmode); break;
  case KO_F8E5M2: ((uint8_t *)p)[idx] = (uint8_t)encode_small(v, kE5M2, rmode); break;
  case KO_I8: ((int8_t *)p)[idx] = (int8_t)(int64_t)v; break;
  case KO_I16: ((int16_t *)p)[idx] = (int16_t)(int64_t)v; break;
  case KO_I32: ((int32_t *)p)[idx] = (int32_t)(int64_t)v; break;
  case KO_I1: ((uint8_t *)p)[idx] = (uint8_t)((int64_t)v & 1); break;
  }
}

// kapy.fptofp (Ops.td:50-72; verifier Kapy.cpp:272-287; lowering ElementwiseOpToLLVM.cpp:536-605).
// Returns 0, or a negative code naming the verifier rule that rejects the cast.
// f32_to_f8_via_f16 = 1 reproduces the pre-sm_90 / RZ route of :577-594 (f32 -RZ-> f16 -> f8).
int ko_fptofp(const void *src, int sd, void *dst, int dd, int rmode, int64_t n, int via_f16) {
  bool src_f8 = sd == KO_F8E4M3 || sd == KO_F8E5M2, dst_f8 = dd == KO_F8E4M3 || dd == KO_F8E5M2;
  bool down = dtype_bytes(dd) < dtype_bytes(sd);
  if (down && rmode != KO_RZ && rmode != KO_RN) return -1;   // "rounding mode is required for down cast"
  if (sd == KO_BF16 && dst_f8 && rmode == KO_RZ) return -2;  // "unsupported rounding mode when convert bf16 to f8"
  if (src_f8 && dst_f8) return -3;                           // "convert f8 to f8 is not supported"
  for (int64_t i = 0; i < n; ++i) {
    double v = ko_decode(src, sd, i);
    if (via_f16 && sd == KO_F32 && dst_f8) v = decode_small(encode_small(v, kF16, KO_RZ), kF16);
    ko_encode(dst, dd, i, v, down ? rmode : KO_RN);
  }
  return 0;
}

// 32-bit initialisation word for masked loads (ConvertUtils.cpp:267-334).  The fp8 rows of the
// reference assume an IEEE-style e4m3 with infinities; OCP e4m3fn has none, so PINF/NINF map to
// ±max-finite (0x7E/0xFE) and QNAN to 0x7F here.
uint32_t ko_padding_word(int dtype, int padding) {
  if (padding == KO_PAD_ZERO) return 0;
  double v = padding_value(dtype, padding);
  uint32_t w = 0;
  switch (dtype) {
  case KO_F32: { float f = (float)v; std::memcpy(&w, &f, 4); return w; }
  case KO_F16: w = encode_small(v, kF16, KO_RN); return w | (w << 16);
  case KO_BF16: w = encode_small(v, kBF16, KO_RN); return w | (w << 16);
  case KO_F8E4M3: w = encode_small(v, kE4M3, KO_RN); return w * 0x01010101u;
  case KO_F8E5M2: {
    // IEEE-like e5m2 keeps its infinities for padding (ConvertUtils.cpp:321-331: 0x7C / 0xFC / 0x7E).
    uint32_t b = padding == KO_PAD_QNAN ? 0x7Eu : (padding == KO_PAD_PINF ? 0x7Cu : 0xFCu);
    return b * 0x01010101u;
  }
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Seeded, counter-based generators.  The reference has no PRNG; these define the synthetic inputs.
// ---------------------------------------------------------------------------------------------
uint64_t ko_splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}
static inline uint64_t stream_base(uint64_t seed, uint64_t stream) { return ko_splitmix64(seed * 1000003ull + stream); }

void ko_fill_uniform(void *dst, int dtype, int64_t n, uint64_t seed, uint64_t stream, double lo, double hi) {
  uint64_t base = stream_base(seed, stream);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    uint64_t h = ko_splitmix64(base ^ (uint64_t)i);
    double u = (double)(h >> 11) * 0x1.0p-53;
    ko_encode(dst, dtype, i, lo + (hi - lo) * u, KO_RN);
  }
}

void ko_fill_normal(void *dst, int dtype, int64_t n, uint64_t seed, uint64_t stream, double mean, double stddev) {
  uint64_t base = stream_base(seed, stream);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    uint64_t h1 = ko_splitmix64(base ^ (uint64_t)i);
    uint64_t h2 = ko_splitmix64(h1);
    double u1 = ((double)(h1 >> 11) + 1.0) * 0x1.0p-53;  // (0,1]
    double u2 = (double)(h2 >> 11) * 0x1.0p-53;
    double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925286766559 * u2);
    ko_encode(dst, dtype, i, mean + stddev * z, KO_RN);
  }
}

void ko_fill_bits16(uint16_t *dst, int64_t n, uint64_t seed, uint64_t stream) {
  uint64_t base = stream_base(seed, stream);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) dst[i] = (uint16_t)(ko_splitmix64(base ^ (uint64_t)i) & 0xFFFF);
}

// ---------------------------------------------------------------------------------------------
// #kgpu.fragments<[A0,A1],[L0,L1],(minor,major)>  (Kgpu.cpp:164-263, CommonUtils.h:51-124)
// ---------------------------------------------------------------------------------------------
void ko_fragments_loops(const ko_fragments *l, const int64_t shape[2], int64_t warp_loops[2], int64_t loop_space[2]) {
  for (int i = 0; i < 2; ++i) {  // Kgpu.cpp:164-184
    int64_t w = shape[i] / ((int64_t)l->lane_array[i] * l->lane_loops[i]);
    w = std::max<int64_t>(w, 1);
    if (warp_loops) warp_loops[i] = w;
    if (loop_space) loop_space[i] = w * l->lane_loops[i];
  }
}

// Options 1 and 2: (lane, iv) -> (i0, i1)   (Kgpu.cpp:221-250).
void ko_fragments_map12(const ko_fragments *l, const int64_t shape[2], int option, int64_t lane, int64_t iv, int64_t idx[2]) {
  int64_t A[2] = {l->lane_array[0], l->lane_array[1]}, L[2] = {l->lane_loops[0], l->lane_loops[1]};
  int64_t S[2], sh[2] = {shape[0], shape[1]};
  ko_fragments_loops(l, shape, nullptr, S);
  bool col_major = l->major_axis == 0;
  if (col_major) { std::swap(A[0], A[1]); std::swap(L[0], L[1]); std::swap(S[0], S[1]); std::swap(sh[0], sh[1]); }
  // delinearize(x, [s0, s1]) = [x / s1, x % s1]: the leading component is not reduced (CommonUtils.h:81-93).
  int64_t lid[2] = {lane / A[1], lane % A[1]};
  int64_t ivs[2] = {iv / S[1], iv % S[1]};
  int64_t out[2];
  for (int i = 0; i < 2; ++i) {
    int64_t c0 = ivs[i] / L[i], c1 = ivs[i] % L[i];
    out[i] = c0 * (A[i] * L[i]) + lid[i] * L[i] + c1;
    if (option == 1 && A[i] * L[i] > sh[i]) out[i] %= sh[i];
  }
  if (col_major) std::swap(out[0], out[1]);
  idx[0] = out[0];
  idx[1] = out[1];
}

// getLayoutString (Kgpu.cpp:293-353): for every element, in row-major order, the (lane, loop iv) pairs
// that own it, printed as "T<lane>:<iv>" right-aligned to the widest lane id / iv; when an element has
// several owners (replication) one block per round, separated by a blank line.
// Returns the length of the text (without the terminating NUL); writes at most out_len bytes.
static int id_width(int64_t id) { return id >= 1000 ? 4 : id >= 100 ? 3 : id >= 10 ? 2 : 1; }
int64_t ko_layout_string(const ko_fragments *l, const int64_t shape[2], char *out, int64_t out_len) {
  const int64_t lanes = l->lane_array[0] * l->lane_array[1], numel = shape[0] * shape[1];
  int64_t S[2];
  ko_fragments_loops(l, shape, nullptr, S);
  const int64_t loop_size = S[0] * S[1];
  std::vector<std::vector<std::pair<int64_t, int64_t>>> owners(numel);
  for (int64_t lane = 0; lane < lanes; ++lane)
    for (int64_t iv = 0; iv < loop_size; ++iv) {
      int64_t idx[2];
      ko_fragments_map12(l, shape, 1, lane, iv, idx);
      owners[idx[0] * shape[1] + idx[1]].push_back({lane, iv});
    }
  const int wl = id_width(lanes - 1), wi = id_width(loop_size - 1);
  std::string text;
  const size_t rounds = owners[0].size();
  for (size_t r = 0; r < rounds; ++r) {
    if (r > 0) text += "\n\n";
    for (int64_t e = 0; e < numel; ++e) {
      if (e % shape[1] == 0) text += e == 0 ? "[[" : "\n [";
      const auto pr = owners[e][r];
      text += std::string(wl - id_width(pr.first), ' ') + "T" + std::to_string(pr.first) + ":";
      text += std::string(wi - id_width(pr.second), ' ') + std::to_string(pr.second);
      if ((e + 1) % shape[1] == 0) text += (e + 1) == numel ? "]]" : "],";
      else text += ", ";
    }
  }
  if (out && out_len > 0) {
    const int64_t n = std::min<int64_t>((int64_t)text.size(), out_len - 1);
    memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return (int64_t)text.size();
}

// Option 3: (i0, i1) -> (lane, iv)   (Kgpu.cpp:196-219).
void ko_fragments_map3(const ko_fragments *l, const int64_t shape[2], int64_t i0, int64_t i1, int64_t *lane, int64_t *iv) {
  const int64_t A0 = l->lane_array[0], A1 = l->lane_array[1], L0 = l->lane_loops[0], L1 = l->lane_loops[1];
  int64_t S[2];
  ko_fragments_loops(l, shape, nullptr, S);
  bool row_major = l->major_axis == 1;
  int64_t c0[3] = {i0 / (A0 * L0), (i0 % (A0 * L0)) / L0, i0 % L0};
  int64_t c1[3] = {i1 / (A1 * L1), (i1 % (A1 * L1)) / L1, i1 % L1};
  *lane = row_major ? c0[1] * A1 + c1[1] : c0[1] + c1[1] * A0;
  int64_t iv0 = c0[0] * L0 + c0[2], iv1 = c1[0] * L1 + c1[2];
  *iv = row_major ? iv0 * S[1] + iv1 : iv0 + iv1 * S[0];
}

void ko_fragments_transpose(const ko_fragments *l, ko_fragments *out) {  // Kgpu.cpp:253-258
  ko_fragments r = {{l->lane_array[1], l->lane_array[0]}, {l->lane_loops[1], l->lane_loops[0]}, l->major_axis, l->minor_axis};
  *out = r;
}
void ko_fragments_exchange_axes(const ko_fragments *l, ko_fragments *out) {  // Kgpu.cpp:260-263
  ko_fragments r = *l;
  r.minor_axis = l->major_axis;
  r.major_axis = l->minor_axis;
  *out = r;
}

// getFragmentsLayout (LayoutUtils.cpp:92-104), warp size as a parameter (32 there, 64 on gfx950).
void ko_fragments_default(const int64_t lane_loops[2], const int64_t shape[2], int row_major, int64_t warp_size, ko_fragments *out) {
  int i = row_major ? 0 : 1, j = row_major ? 1 : 0;
  int64_t max_lanes = std::max<int64_t>(shape[j] / lane_loops[j], 1);
  int64_t A[2];
  A[j] = std::min<int64_t>(std::max<int64_t>(warp_size, 1), max_lanes);  // std::clamp(warpSize, 1, maxLanes)
  A[i] = warp_size / A[j];
  out->lane_array[0] = (int32_t)A[0];
  out->lane_array[1] = (int32_t)A[1];
  out->lane_loops[0] = (int32_t)lane_loops[0];
  out->lane_loops[1] = (int32_t)lane_loops[1];
  out->minor_axis = i;
  out->major_axis = j;
}

// Vector width of a global/shared access (CoalesceAccess.cpp:18-27).
int64_t ko_access_simd_size(int64_t alignment, int64_t bits, int64_t numel, int64_t warp_size) {
  int64_t s = std::min<int64_t>(alignment * 8 / bits, 128 / bits);
  s = std::min<int64_t>(s, (numel + warp_size - 1) / warp_size);
  s = std::max<int64_t>(s, 32 / bits);
  return s;
}

// kgpu.change: where result (lane, iv) fetches from (LayoutUtils.cpp:83-90, ChangeOpToLLVM.cpp:43-78).
void ko_change_source(const ko_fragments *src, const ko_fragments *dst, const int64_t shape[2], int64_t lane, int64_t iv,
                      int64_t *src_lane, int64_t *src_iv) {
  int64_t idx[2];
  ko_fragments_map12(dst, shape, 2, lane, iv, idx);
  ko_fragments_map3(src, shape, idx[0], idx[1], src_lane, src_iv);
}

// ChangeOpHelper::getNumShfls (LayoutUtils.cpp:61-81).
int64_t ko_change_num_shuffles(const ko_fragments *src, const ko_fragments *dst, const int64_t shape[2], int64_t warp_size) {
  int64_t S[2];
  ko_fragments_loops(dst, shape, nullptr, S);
  int64_t loop_size = S[0] * S[1];
  std::set<int64_t> ivs;
  for (int64_t lane = 0; lane < warp_size; ++lane)
    for (int64_t iv = 0; iv < loop_size; ++iv) {
      int64_t sl, si;
      ko_change_source(src, dst, shape, lane, iv, &sl, &si);
      if (sl != lane) ivs.insert(si);
    }
  return loop_size * (int64_t)ivs.size();
}

// Swizzled element offset (CpAsyncOpToLLVM.cpp:124-139 == LdMatrixOpToLLVM.cpp:106-121 ==
// Ld/StSharedOpToLLVM.cpp:97-112), with the bank count as a parameter: 32 banks x 4 B there,
// 64 banks x 4 B on gfx950.  A "line" is num_banks*4 bytes.
int64_t ko_swizzle_offset(int64_t i0, int64_t i1, int64_t stride0, int64_t stride1, int64_t bits, int64_t bank_param,
                          int64_t line_param, int64_t num_banks) {
  int64_t line_bits = num_banks * 32;
  int64_t bit_off = (i0 * stride0 + i1 * stride1) * bits;
  int64_t bank = (bit_off % line_bits) / 32;
  int64_t line = bit_off / line_bits;
  int64_t sub = bit_off % 32;  // the reference drops this (accesses are >= 4-byte aligned); kept so the map is a bijection on elements
  bank = ((bank / bank_param) ^ (line % line_param)) * bank_param + bank % bank_param;
  return (bank * 32 + line * line_bits + sub) / bits;
}

// isNoBankConflict (LayoutUtils.cpp:167-209) with warp size and bank count as parameters.
int ko_no_bank_conflict(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                        int64_t bank_param, int64_t line_param, int64_t alignment, int64_t num_banks, int64_t warp_size) {
  int64_t line_bits = num_banks * 32;
  bool shared_row_major = stride1 == 1;
  bool tensor_row_major = l->major_axis == 1;
  int64_t simd = l->lane_loops[stride0 == 1 ? 0 : 1];
  simd = std::min<int64_t>(simd, bank_param * 32 / bits);
  int64_t S[2];
  ko_fragments_loops(l, shape, nullptr, S);
  int64_t iv_step = 1;
  if (shared_row_major && !tensor_row_major) iv_step = S[0];
  if (!shared_row_major && tensor_row_major) iv_step = S[1];
  std::map<int64_t, std::set<int64_t>> bank_lines;
  for (int64_t lane = 0; lane < warp_size / bank_param; ++lane)
    for (int64_t iv = 0; iv < simd * iv_step; iv += iv_step) {
      int64_t bit_off = alignment % (line_bits / 8) * 8;
      int64_t idx[2];
      ko_fragments_map12(l, shape, 1, lane, iv, idx);
      if (shared_row_major) bit_off += (idx[0] * stride0 + idx[1]) * bits;
      else bit_off += (idx[0] + idx[1] * stride1) * bits;
      int64_t bank = bit_off % line_bits / 32, line = bit_off / line_bits;
      bank = ((bank / bank_param) ^ (line % line_param)) * bank_param + bank % bank_param;
      bank_lines[bank].insert(line);
    }
  for (auto &kv : bank_lines)
    if (kv.second.size() > 1) return 0;
  return 1;
}

// getSwizzlingLayouts (LayoutUtils.cpp:211-225): candidates in the reference's search order.
int ko_swizzle_search(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                      int64_t alignment, int64_t num_banks, int64_t warp_size, int64_t *out_pairs, int max_pairs) {
  int n = 0;
  for (int64_t bank_param : {4, 2, 1})
    for (int64_t line_param = 1; line_param <= num_banks / bank_param; line_param *= 2)
      if (ko_no_bank_conflict(l, shape, stride0, stride1, bits, bank_param, line_param, alignment, num_banks, warp_size)) {
        if (n < max_pairs) { out_pairs[2 * n] = bank_param; out_pairs[2 * n + 1] = line_param; }
        ++n;
      }
  return n;
}

// The same question for the LDS of gfx950 as the hardware serves a 64-lane wavefront (no counterpart in the reference, whose
// model above is NVIDIA's first-quarter-warp rule).  16-byte reads go in four phases of sixteen lanes, listed below; 8-byte
// reads in two halves of 32 lanes; 4-byte reads at once; a lane that reads several atoms issues one instruction per atom.
// `rotate`: the XOR key is line % line_param rotated left by that many bits within log2(line_param) bits.
// Pinned by two measurements of SQ_LDS_BANK_CONFLICT on the 16x16x128 operand reads (plain key (4, 8): conflicts on half of the
// active cycles; key rotated by one: none) and by a brute-force replay in the tests.
static const int kGfx950Phases128[4][16] = {
    {0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27},
    {4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31},
    {32, 33, 34, 35, 44, 45, 46, 47, 52, 53, 54, 55, 56, 57, 58, 59},
    {36, 37, 38, 39, 40, 41, 42, 43, 48, 49, 50, 51, 60, 61, 62, 63}};
static int64_t rotated_key(int64_t line, int64_t line_param, int64_t rotate) {
  int64_t key = line % line_param, width = 0;
  while ((int64_t(1) << width) < line_param) ++width;
  for (int64_t r = 0; width > 0 && r < rotate % width; ++r) key = ((key << 1) & (line_param - 1)) | (key >> (width - 1));
  return key;
}
int ko_no_bank_conflict_gfx950(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                               int64_t bank_param, int64_t line_param, int64_t rotate, int64_t alignment) {
  const int64_t num_banks = 64, line_bits = num_banks * 32;
  bool shared_row_major = stride1 == 1, tensor_row_major = l->major_axis == 1;
  int64_t per_lane = l->lane_loops[stride0 == 1 ? 0 : 1];
  int64_t atom = std::min<int64_t>(per_lane, bank_param * 32 / bits);
  int64_t S[2];
  ko_fragments_loops(l, shape, nullptr, S);
  int64_t iv_step = 1;
  if (shared_row_major && !tensor_row_major) iv_step = S[0];
  if (!shared_row_major && tensor_row_major) iv_step = S[1];
  std::vector<std::vector<int>> phases;
  if (bank_param >= 4) for (auto &ph : kGfx950Phases128) phases.emplace_back(ph, ph + 16);
  else if (bank_param == 2) for (int h = 0; h < 2; ++h) { phases.emplace_back(); for (int i = 0; i < 32; ++i) phases.back().push_back(32 * h + i); }
  else { phases.emplace_back(); for (int i = 0; i < 64; ++i) phases.back().push_back(i); }
  for (int64_t first = 0; first < per_lane; first += atom)   // one instruction per atom
    for (auto &phase : phases) {
      std::map<int64_t, std::set<int64_t>> bank_lines;
      for (int lane : phase)
        for (int64_t e = first; e < first + atom; ++e) {
          int64_t idx[2];
          ko_fragments_map12(l, shape, 1, lane, e * iv_step, idx);
          int64_t bit_off = alignment % (line_bits / 8) * 8 + (shared_row_major ? idx[0] * stride0 + idx[1] : idx[0] + idx[1] * stride1) * bits;
          int64_t bank = bit_off % line_bits / 32, line = bit_off / line_bits;
          bank = ((bank / bank_param) ^ rotated_key(line, line_param, rotate)) * bank_param + bank % bank_param;
          bank_lines[bank].insert(line);
        }
      for (auto &kv : bank_lines)
        if (kv.second.size() > 1) return 0;
    }
  return 1;
}
int ko_swizzle_search_gfx950(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                             int64_t alignment, int64_t *out_triples, int max_triples) {
  int n = 0;
  for (int64_t bank_param : {4, 2, 1})
    for (int64_t line_param = 1, width = 0; line_param <= 64 / bank_param; line_param *= 2, ++width)
      for (int64_t rotate = 0; rotate < std::max<int64_t>(width, 1); ++rotate)
        if (ko_no_bank_conflict_gfx950(l, shape, stride0, stride1, bits, bank_param, line_param, rotate, alignment)) {
          if (n < max_triples) { out_triples[3 * n] = bank_param; out_triples[3 * n + 1] = line_param; out_triples[3 * n + 2] = rotate; }
          ++n;
        }
  return n;
}
int64_t ko_swizzle_offset_rotated(int64_t i0, int64_t i1, int64_t stride0, int64_t stride1, int64_t bits, int64_t bank_param,
                                  int64_t line_param, int64_t rotate) {
  int64_t line_bits = 64 * 32;
  int64_t bit_off = (i0 * stride0 + i1 * stride1) * bits;
  int64_t bank = (bit_off % line_bits) / 32, line = bit_off / line_bits, sub = bit_off % 32;
  bank = ((bank / bank_param) ^ rotated_key(line, line_param, rotate)) * bank_param + bank % bank_param;
  return (bank * 32 + line * line_bits + sub) / bits;
}

// ---------------------------------------------------------------------------------------------
// Descriptors (TypeConverter.cpp:65-73) and global memory ops.
// ---------------------------------------------------------------------------------------------
// kapy.mk_global (Ops.td:95-114, MkGlobalOpToLLVM.cpp:23-47): ptr += dynamic_offset elements,
// start = 0, end = size.
int ko_mk_global(ko_global *out, void *ptr, int32_t dynamic_offset, int32_t size0, int32_t size1, int32_t stride0,
                 int32_t stride1, int dtype, int32_t alignment) {
  int b = dtype_bytes(dtype);
  if (!b) return -1;
  out->ptr = (char *)ptr + (int64_t)dynamic_offset * b;
  out->start0 = out->start1 = 0;
  out->end0 = size0;
  out->end1 = size1;
  out->stride0 = stride0;
  out->stride1 = stride1;
  out->dtype = dtype;
  out->alignment = alignment;
  return 0;
}

// kapy.sv_global (Ops.td:116-136, SvGlobalOpToLLVM.cpp:22-40): new_start = start + start_arg,
// new_end = start + end_arg (both relative to the OLD start; the old end is not consulted).
int ko_sv_global(ko_global *out, const ko_global *src, int32_t start0, int32_t end0, int32_t start1, int32_t end1) {
  ko_global r = *src;
  r.start0 = src->start0 + start0;
  r.start1 = src->start1 + start1;
  r.end0 = src->start0 + end0;
  r.end1 = src->start1 + end1;
  *out = r;
  return 0;
}

// kapy.ld_global (Ops.td:138-161, LdGlobalOpToLLVM.cpp:60-145): a shape0 x shape1 register tile,
// returned row-major.  Element (i,j) comes from ptr + (start0+i)*stride0 + (start1+j)*stride1 when
// (start0+i) <u end0 && (start1+j) <u end1, otherwise it holds the padding pattern.
void ko_ld_global(const ko_global *src, int64_t shape0, int64_t shape1, int padding, void *tile) {
  int b = dtype_bytes(src->dtype);
  uint32_t padw = ko_padding_word(src->dtype, padding);
  for (int64_t i = 0; i < shape0; ++i)
    for (int64_t j = 0; j < shape1; ++j) {
      char *d = (char *)tile + (i * shape1 + j) * b;
      if (in_bounds(src, i, j)) std::memcpy(d, (const char *)src->ptr + elem_offset(src, i, j) * b, b);
      else std::memcpy(d, &padw, b);
    }
}

// kapy.st_global (Ops.td:163-187, StGlobalOpToLLVM.cpp:60-139): masked store, same predicate.
void ko_st_global(const void *tile, int64_t shape0, int64_t shape1, const ko_global *dst) {
  int b = dtype_bytes(dst->dtype);
  for (int64_t i = 0; i < shape0; ++i)
    for (int64_t j = 0; j < shape1; ++j)
      if (in_bounds(dst, i, j))
        std::memcpy((char *)dst->ptr + elem_offset(dst, i, j) * b, (const char *)tile + (i * shape1 + j) * b, b);
}

// kapy.transpose (Ops.td:358-373, Kapy.cpp:700-720): result[j,i] = source[i,j]; on the GPU this is
// a relabel of the register layout (TransposeOpToLLVM.cpp:21-26), so values never pass an FP unit.
void ko_transpose_tile(const void *tile, int64_t shape0, int64_t shape1, int dtype, void *out) {
  int b = dtype_bytes(dtype);
  for (int64_t i = 0; i < shape0; ++i)
    for (int64_t j = 0; j < shape1; ++j)
      std::memcpy((char *)out + (j * shape0 + i) * b, (const char *)tile + (i * shape1 + j) * b, b);
}

// kgpu.change on a whole warp (ChangeOpToLLVM.cpp:21-93): lane_values[lane*loop_size_src + iv].
void ko_change_tile(const void *lane_values, const ko_fragments *src, const ko_fragments *dst, const int64_t shape[2],
                    int bytes, int64_t warp_size, void *out_lane_values) {
  int64_t Ss[2], Sd[2];
  ko_fragments_loops(src, shape, nullptr, Ss);
  ko_fragments_loops(dst, shape, nullptr, Sd);
  int64_t ns = Ss[0] * Ss[1], nd = Sd[0] * Sd[1];
  for (int64_t lane = 0; lane < warp_size; ++lane)
    for (int64_t iv = 0; iv < nd; ++iv) {
      int64_t sl, si;
      ko_change_source(src, dst, shape, lane, iv, &sl, &si);
      char *o = (char *)out_lane_values + (lane * nd + iv) * bytes;
      // A result layout larger than the tensor names positions past the tensor's edge, which the source does not
      // hold: the select chain of ChangeOpToLLVM.cpp:50-78 then matches no source iv and keeps its first candidate,
      // whatever that lane holds.  No consumer reads such a position; here it is defined as zero.
      if (sl < 0 || sl >= warp_size || si < 0 || si >= ns) std::memset(o, 0, bytes);
      else std::memcpy(o, (const char *)lane_values + (sl * ns + si) * bytes, bytes);
    }
}

// Whole-tensor ld_global -> [transpose] -> st_global.  The register tile is the destination
// view's extent (transposed back for the load when transpose != 0); out-of-bounds source
// elements read as padding, out-of-bounds destination elements are not written.
int ko_copy(const ko_global *src, const ko_global *dst, int transpose, int padding) {
  if (dtype_bytes(src->dtype) != dtype_bytes(dst->dtype) || !dtype_bytes(src->dtype)) return -1;
  int b = dtype_bytes(src->dtype);
  int64_t d0 = extent0(dst), d1 = extent1(dst);
  if (d0 <= 0 || d1 <= 0) return 0;
  uint32_t padw = ko_padding_word(src->dtype, padding);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < d0; ++i)
    for (int64_t j = 0; j < d1; ++j) {
      int64_t si = transpose ? j : i, sj = transpose ? i : j;
      char *d = (char *)dst->ptr + elem_offset(dst, i, j) * b;
      if (in_bounds(src, si, sj)) std::memcpy(d, (const char *)src->ptr + elem_offset(src, si, sj) * b, b);
      else std::memcpy(d, &padw, b);
    }
  return 0;
}

// A grid of programs (kapy.program_id axes 0,1; ParallelIdOpToLLVM.cpp:28-38), each running
// ko_copy on views whose mk_global dynamic_offset is affine in the program ids.
int ko_copy_batched(const ko_global *src, const ko_global *dst, int transpose, int padding, int32_t n0, int32_t n1,
                    int64_t src_off0, int64_t src_off1, int64_t dst_off0, int64_t dst_off1) {
  int b = dtype_bytes(src->dtype);
  for (int32_t p0 = 0; p0 < n0; ++p0)
    for (int32_t p1 = 0; p1 < n1; ++p1) {
      ko_global s = *src, d = *dst;
      s.ptr = (char *)src->ptr + (p0 * src_off0 + p1 * src_off1) * b;
      d.ptr = (char *)dst->ptr + (p0 * dst_off0 + p1 * dst_off1) * b;
      int rc = ko_copy(&s, &d, transpose, padding);
      if (rc) return rc;
    }
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Elementwise programs (ElementwiseOpToLLVM.cpp:424-534 generic; special cases :536-1166).
// Every virtual register has a dtype; an op computes the exact (or libm) result of its operands
// and rounds ONCE to the register dtype: f16/f32 native IEEE RN, bf16 single rounding as the
// fma.rn.bf16 forms of :771-892 give.
// ---------------------------------------------------------------------------------------------
enum {
  EW_LD_GLOBAL = 0, EW_SPLAT, EW_FPTOFP, EW_ADDF, EW_SUBF, EW_MULF, EW_DIVF, EW_FMA, EW_MAXIMUMF, EW_MINIMUMF,
  EW_NEGF, EW_ABSF, EW_EXP, EW_EXP2, EW_LOG, EW_LOG2, EW_SQRT, EW_RSQRT, EW_TANH, EW_ERF, EW_GELU_TANH, EW_ST_GLOBAL,
  EW_REDUCE_SUM, EW_REDUCE_MAX, EW_FLOOR, EW_CEIL, EW_SIN, EW_COS, EW_MAXNUMF, EW_MINNUMF, EW_REMF,
  // integer, compare, select and conversion ops (BinaryOpConversion / UnaryOpConversion over the arith ops,
  // ElementwiseOpToLLVM.cpp:1178-1215; arith.select, SelectOpToLLVM.cpp:21-98; kapy.arange, ArangeOpToLLVM.cpp:22-50)
  EW_ADDI, EW_SUBI, EW_MULI, EW_DIVSI, EW_DIVUI, EW_FLOORDIVSI, EW_CEILDIVSI, EW_CEILDIVUI, EW_REMSI, EW_REMUI, EW_ANDI, EW_ORI, EW_XORI,
  EW_SHLI, EW_SHRSI, EW_SHRUI, EW_MAXSI, EW_MAXUI, EW_MINSI, EW_MINUI, EW_ABSI, EW_CMPI, EW_CMPF, EW_SELECT, EW_TRUNCI, EW_EXTSI, EW_EXTUI,
  EW_SITOFP, EW_FPTOSI, EW_BITCAST, EW_ARANGE,
  EW_NUM_OPS
};
enum { EW_MAX_REGS = 16 };

// ---- signless integers (MLIR's iN): a register holds the value read as a signed number of its width (i1: 0 or 1) in a
// double.  What MLIR leaves undefined is defined as the device library defines it: x / 0 = 0, x % 0 = 0, the most negative
// value over -1 wraps (remainder 0), a shift by the width or more gives 0 (shrsi: all sign bits), fptosi saturates to i32
// and maps NaN to 0 before wrapping to the result's width.
static bool is_int_dtype(int d) { return d == KO_I8 || d == KO_I16 || d == KO_I32 || d == KO_I1; }
static bool is_arith_float(int d) { return d == KO_F16 || d == KO_BF16 || d == KO_F32; }
static int int_bits(int d) { return d == KO_I1 ? 1 : d == KO_I8 ? 8 : d == KO_I16 ? 16 : 32; }
static int64_t int_wrap(int64_t v, int d) {  // the low bits of v as the register keeps them
  const int bits = int_bits(d);
  const uint64_t low = (uint64_t)v & ((uint64_t(1) << bits) - 1);
  if (d == KO_I1) return (int64_t)low;
  return (low >> (bits - 1)) ? (int64_t)low - (int64_t(1) << bits) : (int64_t)low;
}
static int64_t int_as_signed(int64_t reg, int d) { return d == KO_I1 ? -reg : reg; }
static int64_t int_as_unsigned(int64_t reg, int d) { return d == KO_I1 ? reg : (reg < 0 ? reg + (int64_t(1) << int_bits(d)) : reg); }
static int64_t floor_div(int64_t a, int64_t b) {
  int64_t q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}
static int64_t int_binary_op(int op, int64_t ra, int64_t rb, int d) {
  const int64_t a = int_as_signed(ra, d), b = int_as_signed(rb, d), ua = int_as_unsigned(ra, d), ub = int_as_unsigned(rb, d);
  const int bits = int_bits(d);
  int64_t r = 0;
  switch (op) {
  case EW_ADDI: r = a + b; break;
  case EW_SUBI: r = a - b; break;
  case EW_MULI: r = (int64_t)((uint64_t)a * (uint64_t)b); break;
  case EW_DIVSI: r = b == 0 ? 0 : a / b; break;                      // (64-bit: the most negative value over -1 does not trap, it wraps below)
  case EW_DIVUI: r = ub == 0 ? 0 : ua / ub; break;
  case EW_FLOORDIVSI: r = b == 0 ? 0 : floor_div(a, b); break;
  case EW_CEILDIVSI: r = b == 0 ? 0 : -floor_div(-a, b); break;
  case EW_CEILDIVUI: r = ub == 0 ? 0 : (ua + ub - 1) / ub; break;
  case EW_REMSI: r = b == 0 ? 0 : a % b; break;
  case EW_REMUI: r = ub == 0 ? 0 : ua % ub; break;
  case EW_ANDI: r = ua & ub; break;
  case EW_ORI: r = ua | ub; break;
  case EW_XORI: r = ua ^ ub; break;
  case EW_SHLI: r = ub >= bits ? 0 : (int64_t)((uint64_t)ua << ub); break;
  case EW_SHRUI: r = ub >= bits ? 0 : ua >> ub; break;
  case EW_SHRSI: r = ub >= bits ? (a < 0 ? -1 : 0) : floor_div(a, int64_t(1) << ub); break;
  case EW_MAXSI: r = std::max(a, b); break;
  case EW_MINSI: r = std::min(a, b); break;
  case EW_MAXUI: r = std::max(ua, ub); break;
  case EW_MINUI: r = std::min(ua, ub); break;
  }
  return int_wrap(r, d);
}
static int64_t int_compare_op(int pred, int64_t ra, int64_t rb, int d) {
  const int64_t a = int_as_signed(ra, d), b = int_as_signed(rb, d), ua = int_as_unsigned(ra, d), ub = int_as_unsigned(rb, d);
  switch (pred) {  // arith.cmpi predicates as MLIR numbers them
  case 0: return ua == ub;
  case 1: return ua != ub;
  case 2: return a < b;
  case 3: return a <= b;
  case 4: return a > b;
  case 5: return a >= b;
  case 6: return ua < ub;
  case 7: return ua <= ub;
  case 8: return ua > ub;
  default: return ua >= ub;
  }
}
static int64_t float_compare_op(int pred, double a, double b) {
  const bool unordered = std::isnan(a) || std::isnan(b);
  if (pred == 0) return 0;
  if (pred == 15) return 1;
  if (pred == 7) return !unordered;
  if (pred == 14) return unordered;
  const int base = pred >= 8 ? pred - 7 : pred;  // oeq ogt oge olt ole one = 1..6; ueq .. une = 8..13
  bool ordered_result = false;
  switch (base) {
  case 1: ordered_result = a == b; break;
  case 2: ordered_result = a > b; break;
  case 3: ordered_result = a >= b; break;
  case 4: ordered_result = a < b; break;
  case 5: ordered_result = a <= b; break;
  case 6: ordered_result = a != b; break;
  }
  return unordered ? pred >= 8 : ordered_result;
}

static double round_to(double v, int dtype) {
  switch (dtype) {
  case KO_F32: return (double)(float)v;
  case KO_F16: return decode_small(encode_small(v, kF16, KO_RN), kF16);
  case KO_BF16: return decode_small(encode_small(v, kBF16, KO_RN), kBF16);
  }
  return v;
}

static double gelu_tanh(double v) {
  // 0.5*v*(1 + tanh(u)), u = sqrt(2/pi)*(v + 0.044715 v^3).  Written out like that, 1 + tanh(u) cancels for u << 0 (below
  // u = -17 nothing but rounding noise is left of it in fp64, while the result, ~1e-15, is an ordinary bf16 or f32 value);
  // 0.5*(1 + tanh(u)) = 1/(1 + exp(-2u)) is the same function without the cancellation.
  const double u = 0.7978845608028654 * (v + 0.044715 * v * v * v);
  if (u < -4.0) return v / (1.0 + std::exp(-2.0 * u));
  return 0.5 * v * (1.0 + std::tanh(u));
}

int ko_elementwise(const ko_ew_inst *prog, int n_inst, const ko_global *const *ins, int n_ins, const ko_global *out) {
  int reg_dtype[EW_MAX_REGS];
  for (int r = 0; r < EW_MAX_REGS; ++r) reg_dtype[r] = -1;
  // static verification pass: register dtypes, operand agreement, broadcastability
  int64_t o0 = extent0(out), o1 = extent1(out);
  bool has_store = false;
  for (int k = 0; k < n_inst; ++k) {
    const ko_ew_inst &I = prog[k];
    if (I.op < 0 || I.op >= EW_NUM_OPS) return -1;
    auto reg_ok = [&](int r) { return r >= 0 && r < EW_MAX_REGS && reg_dtype[r] >= 0; };
    if (I.op != EW_ST_GLOBAL && (I.dst < 0 || I.dst >= EW_MAX_REGS)) return -2;
    switch (I.op) {
    case EW_LD_GLOBAL: {
      if (I.a < 0 || I.a >= n_ins) return -3;
      int64_t e0 = extent0(ins[I.a]), e1 = extent1(ins[I.a]);
      // kapy.broadcast only from size-1 axes (Kapy.cpp:686-698)
      if ((e0 != o0 && e0 != 1) || (e1 != o1 && e1 != 1)) return -4;
      reg_dtype[I.dst] = ins[I.a]->dtype;
      break;
    }
    case EW_SPLAT:
      if (!is_arith_float(I.dtype) && !is_int_dtype(I.dtype)) return -5;
      reg_dtype[I.dst] = I.dtype;
      break;
    case EW_ARANGE:
      if (I.b != 0 && I.b != 1) return -14;
      reg_dtype[I.dst] = KO_I32;
      break;
    case EW_SELECT:
      if (!reg_ok(I.a) || !reg_ok(I.b) || !reg_ok(I.c)) return -6;
      if (reg_dtype[I.a] != KO_I1 || reg_dtype[I.b] != reg_dtype[I.c]) return -10;
      reg_dtype[I.dst] = reg_dtype[I.b];
      break;
    case EW_ADDI: case EW_SUBI: case EW_MULI: case EW_DIVSI: case EW_DIVUI: case EW_FLOORDIVSI: case EW_CEILDIVSI: case EW_CEILDIVUI: case EW_REMSI:
    case EW_REMUI: case EW_ANDI: case EW_ORI: case EW_XORI: case EW_SHLI: case EW_SHRSI: case EW_SHRUI: case EW_MAXSI: case EW_MAXUI: case EW_MINSI:
    case EW_MINUI: case EW_CMPI:
      if (!reg_ok(I.a) || !reg_ok(I.b)) return -6;
      if (reg_dtype[I.a] != reg_dtype[I.b] || !is_int_dtype(reg_dtype[I.a])) return -10;
      if (I.op == EW_CMPI && (I.c < 0 || I.c > 9)) return -15;
      reg_dtype[I.dst] = I.op == EW_CMPI ? (int)KO_I1 : reg_dtype[I.a];
      break;
    case EW_CMPF:
      if (!reg_ok(I.a) || !reg_ok(I.b)) return -6;
      if (reg_dtype[I.a] != reg_dtype[I.b] || !is_arith_float(reg_dtype[I.a])) return -10;
      if (I.c < 0 || I.c > 15) return -15;
      reg_dtype[I.dst] = KO_I1;
      break;
    case EW_ABSI:
      if (!reg_ok(I.a) || !is_int_dtype(reg_dtype[I.a])) return -6;
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    case EW_TRUNCI: case EW_EXTSI: case EW_EXTUI: case EW_SITOFP: case EW_FPTOSI: case EW_BITCAST: {
      if (!reg_ok(I.a)) return -6;
      const int sd = reg_dtype[I.a], dd = I.dtype;
      if (I.op == EW_TRUNCI && !(is_int_dtype(sd) && is_int_dtype(dd) && int_bits(dd) < int_bits(sd))) return -16;
      if ((I.op == EW_EXTSI || I.op == EW_EXTUI) && !(is_int_dtype(sd) && is_int_dtype(dd) && int_bits(dd) > int_bits(sd))) return -16;
      if (I.op == EW_SITOFP && !(is_int_dtype(sd) && is_arith_float(dd))) return -16;
      if (I.op == EW_FPTOSI && !(is_arith_float(sd) && is_int_dtype(dd) && dd != KO_I1)) return -16;
      if (I.op == EW_BITCAST && (sd == KO_I1 || dd == KO_I1 || dtype_bytes(sd) != dtype_bytes(dd) || dtype_bytes(dd) == 0)) return -16;
      reg_dtype[I.dst] = dd;
      break;
    }
    case EW_FPTOFP: {
      if (!reg_ok(I.a)) return -6;
      int sd = reg_dtype[I.a], dd = I.dtype;
      bool down = dtype_bytes(dd) < dtype_bytes(sd);
      bool sf8 = sd == KO_F8E4M3 || sd == KO_F8E5M2, df8 = dd == KO_F8E4M3 || dd == KO_F8E5M2;
      if (down && I.rmode != KO_RN && I.rmode != KO_RZ) return -7;
      if (sd == KO_BF16 && df8 && I.rmode == KO_RZ) return -8;
      if (sf8 && df8) return -9;
      reg_dtype[I.dst] = dd;
      break;
    }
    case EW_FMA:
      if (!reg_ok(I.a) || !reg_ok(I.b) || !reg_ok(I.c)) return -6;
      if (reg_dtype[I.a] != reg_dtype[I.b] || reg_dtype[I.a] != reg_dtype[I.c]) return -10;
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    case EW_ADDF: case EW_SUBF: case EW_MULF: case EW_DIVF: case EW_MAXIMUMF: case EW_MINIMUMF: case EW_MAXNUMF: case EW_MINNUMF: case EW_REMF:
      if (!reg_ok(I.a) || !reg_ok(I.b)) return -6;
      if (reg_dtype[I.a] != reg_dtype[I.b]) return -10;
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    case EW_ST_GLOBAL:
      if (!reg_ok(I.a)) return -6;
      if (reg_dtype[I.a] != out->dtype) return -11;
      has_store = true;
      break;
    case EW_REDUCE_SUM: case EW_REDUCE_MAX:
      if (!reg_ok(I.a)) return -6;
      if (I.b != 0 && I.b != 1) return -14;  // the axis
      reg_dtype[I.dst] = reg_dtype[I.a];
      break;
    default:
      if (!reg_ok(I.a)) return -6;
      reg_dtype[I.dst] = reg_dtype[I.a];
    }
    if (I.op != EW_ST_GLOBAL && I.op != EW_LD_GLOBAL && I.op != EW_FPTOFP && I.op != EW_SPLAT && I.op < EW_ADDI) {
      int d = reg_dtype[I.dst];
      if (d != KO_F16 && d != KO_BF16 && d != KO_F32) return -12;  // float arithmetic on f8 / integer registers is not defined
    }
    if (I.op == EW_FPTOFP && (is_int_dtype(reg_dtype[I.dst]) || is_int_dtype(reg_dtype[I.a] ))) return -12;
  }
  if (!has_store) return -13;

  const double qnan = std::numeric_limits<double>::quiet_NaN();
  // Registers are whole tensors (o0 x o1 doubles holding exactly representable values of the register's
  // type), instructions run one after the other over all elements: what the SSA program of whole-tensor
  // ops means.  A reduce (kapy.reduce with an addf / maximumf combiner, Ops.td:441-457, followed by the
  // kapy.broadcast that later uses imply) accumulates exactly (double) along its axis, rounds once to the
  // register type and fills the axis with the result.
  std::vector<std::vector<double>> reg(EW_MAX_REGS);
  int rd[EW_MAX_REGS];
  const int64_t total = o0 * o1;
  for (int k = 0; k < n_inst; ++k) {
    const ko_ew_inst &I = prog[k];
    const int d = (I.op == EW_ST_GLOBAL) ? 0 : I.dst;
    if (I.op == EW_REDUCE_SUM || I.op == EW_REDUCE_MAX) {
      const std::vector<double> src = reg[I.a];
      const int dt = rd[I.a];
      reg[d].assign(total, 0.0);
      rd[d] = dt;
      const int64_t n_keep = I.b == 1 ? o0 : o1, n_red = I.b == 1 ? o1 : o0;
#pragma omp parallel for schedule(static)
      for (int64_t q = 0; q < n_keep; ++q) {
        long double acc = I.op == EW_REDUCE_SUM ? -0.0L : -std::numeric_limits<long double>::infinity();
        bool nan = false;
        for (int64_t r = 0; r < n_red; ++r) {
          const double v = I.b == 1 ? src[q * o1 + r] : src[r * o1 + q];
          if (std::isnan(v)) nan = true;
          if (I.op == EW_REDUCE_SUM) acc += v;
          else if (v > acc || (v == 0.0 && acc == 0.0L && !std::signbit(v))) acc = v;  // maximumf orders -0 below +0
        }
        const double res = nan ? qnan : round_to((double)acc, dt);
        for (int64_t r = 0; r < n_red; ++r) reg[d][I.b == 1 ? q * o1 + r : r * o1 + q] = res;
      }
      continue;
    }
    std::vector<double> dstv(I.op == EW_ST_GLOBAL ? 0 : total);
    int dst_dtype = -1;
    if (I.op == EW_LD_GLOBAL) dst_dtype = ins[I.a]->dtype;
    else if (I.op == EW_SPLAT || I.op == EW_FPTOFP || (I.op >= EW_TRUNCI && I.op <= EW_BITCAST)) dst_dtype = I.dtype;
    else if (I.op == EW_ARANGE) dst_dtype = KO_I32;
    else if (I.op == EW_CMPI || I.op == EW_CMPF) dst_dtype = KO_I1;
    else if (I.op == EW_SELECT) dst_dtype = rd[I.b];
    else if (I.op != EW_ST_GLOBAL) dst_dtype = rd[I.a];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < o0; ++i) {
      for (int64_t j = 0; j < o1; ++j) {
        const int64_t at = i * o1 + j;
        const double a = (I.op != EW_LD_GLOBAL && I.op != EW_SPLAT && I.op != EW_ARANGE) ? reg[I.a][at] : 0.0;
        double r = 0.0;
        if (I.op >= EW_ADDI && I.op <= EW_MINUI) {
          dstv[at] = (double)int_binary_op(I.op, (int64_t)a, (int64_t)reg[I.b][at], dst_dtype);
          continue;
        }
        switch (I.op) {
        case EW_ARANGE: dstv[at] = (double)int_wrap((int64_t)I.a + (I.b ? j : i), KO_I32); continue;
        case EW_SELECT: dstv[at] = ((int64_t)a & 1) ? reg[I.b][at] : reg[I.c][at]; continue;
        case EW_CMPI: dstv[at] = (double)int_compare_op(I.c, (int64_t)a, (int64_t)reg[I.b][at], rd[I.a]); continue;
        case EW_CMPF: dstv[at] = (double)float_compare_op(I.c, a, reg[I.b][at]); continue;
        case EW_ABSI: {
          const int64_t v = int_as_signed((int64_t)a, dst_dtype);
          dstv[at] = (double)int_wrap(v < 0 ? -v : v, dst_dtype);
          continue;
        }
        case EW_TRUNCI: dstv[at] = (double)int_wrap((int64_t)a, dst_dtype); continue;
        case EW_EXTSI: dstv[at] = (double)int_wrap(int_as_signed((int64_t)a, rd[I.a]), dst_dtype); continue;
        case EW_EXTUI: dstv[at] = (double)int_wrap(int_as_unsigned((int64_t)a, rd[I.a]), dst_dtype); continue;
        case EW_SITOFP: {  // one rounding to nearest even of the exact integer (a double holds any i32)
          uint32_t tmp = 0;
          ko_encode(&tmp, dst_dtype, 0, (double)int_as_signed((int64_t)a, rd[I.a]), KO_RN);
          dstv[at] = ko_decode(&tmp, dst_dtype, 0);
          continue;
        }
        case EW_FPTOSI: {
          const double t = std::isnan(a) ? 0.0 : std::trunc(a);
          const int64_t v = t >= 2147483647.0 ? 2147483647 : t <= -2147483648.0 ? -2147483648LL : (int64_t)t;
          dstv[at] = (double)int_wrap(v, dst_dtype);
          continue;
        }
        case EW_BITCAST: {  // through the memory image of the operand
          uint32_t tmp = 0;
          ko_encode(&tmp, rd[I.a], 0, a, KO_RN);
          dstv[at] = ko_decode(&tmp, dst_dtype, 0);
          continue;
        }
        case EW_LD_GLOBAL: {
          const ko_global *g = ins[I.a];
          int64_t gi = extent0(g) == 1 && o0 != 1 ? 0 : i, gj = extent1(g) == 1 && o1 != 1 ? 0 : j;
          if (in_bounds(g, gi, gj)) r = ko_decode(g->ptr, g->dtype, elem_offset(g, gi, gj));
          else {
            uint32_t w = ko_padding_word(g->dtype, I.c);
            r = ko_decode(&w, g->dtype, 0);
          }
          dstv[at] = r;
          continue;
        }
        case EW_SPLAT: dstv[at] = is_int_dtype(I.dtype) ? (double)int_wrap((int64_t)I.a, I.dtype) : round_to((double)I.imm, I.dtype); continue;
        case EW_FPTOFP: {
          bool down = dtype_bytes(I.dtype) < dtype_bytes(rd[I.a]);
          uint32_t tmp = 0;
          ko_encode(&tmp, I.dtype, 0, a, down ? I.rmode : KO_RN);
          dstv[at] = ko_decode(&tmp, I.dtype, 0);
          continue;
        }
        case EW_ADDF: r = a + reg[I.b][at]; break;
        case EW_SUBF: r = a - reg[I.b][at]; break;
        case EW_MULF: r = a * reg[I.b][at]; break;
        case EW_DIVF: r = a / reg[I.b][at]; break;
        // One rounding of the exact a*b + c to the register type.  For f16 / bf16 the double-precision fma followed by the
        // rounding to 16 bits is that (a value on a 16-bit rounding boundary needs the product to supply both the boundary
        // bit and a lower one, which spans at most 22 + 11 bits: exact in a double).  For f32 it is not (add, sub, mul, div
        // survive the detour through double, fma does not), so the fma is taken in float.
        case EW_FMA:
          r = dst_dtype == KO_F32 ? (double)std::fmaf((float)a, (float)reg[I.b][at], (float)reg[I.c][at]) : std::fma(a, reg[I.b][at], reg[I.c][at]);
          break;
        // arith.maximumf / minimumf propagate NaN
        // arith.maximumf / minimumf: NaN if either operand is, and -0 orders below +0 (max.NaN / min.NaN of PTX do the same)
        case EW_MAXIMUMF: {
          const double b = reg[I.b][at];
          r = (std::isnan(a) || std::isnan(b)) ? qnan : a == b ? (std::signbit(a) ? b : a) : std::max(a, b);
          break;
        }
        case EW_MINIMUMF: {
          const double b = reg[I.b][at];
          r = (std::isnan(a) || std::isnan(b)) ? qnan : a == b ? (std::signbit(a) ? a : b) : std::min(a, b);
          break;
        }
        case EW_MAXNUMF: {  // arith.maxnumf / minnumf: a NaN operand is ignored; -0 below +0 (BinaryOpConversion, ElementwiseOpToLLVM.cpp:1201-1206)
          const double b = reg[I.b][at];
          r = std::isnan(a) ? b : std::isnan(b) ? a : a == b ? (std::signbit(a) ? b : a) : std::max(a, b);
          break;
        }
        case EW_MINNUMF: {
          const double b = reg[I.b][at];
          r = std::isnan(a) ? b : std::isnan(b) ? a : a == b ? (std::signbit(a) ? a : b) : std::min(a, b);
          break;
        }
        case EW_REMF: r = std::fmod(a, reg[I.b][at]); break;  // arith.remf (frem): exact, sign of the dividend (:1192)
        case EW_NEGF: r = -a; break;
        case EW_ABSF: r = std::fabs(a); break;
        case EW_EXP: r = std::exp(a); break;
        case EW_EXP2: r = std::exp2(a); break;
        case EW_LOG: r = std::log(a); break;
        case EW_LOG2: r = std::log2(a); break;
        case EW_SQRT: r = std::sqrt(a); break;
        case EW_RSQRT: r = 1.0 / std::sqrt(a); break;
        case EW_TANH: r = std::tanh(a); break;
        case EW_ERF: r = std::erf(a); break;
        case EW_GELU_TANH: r = gelu_tanh(a); break;
        case EW_FLOOR: r = std::floor(a); break;  // math.floor / ceil / sin / cos: UnaryOpConversion, ElementwiseOpToLLVM.cpp:1222-1225
        case EW_CEIL: r = std::ceil(a); break;
        case EW_SIN: r = std::sin(a); break;
        case EW_COS: r = std::cos(a); break;
        case EW_ST_GLOBAL:
          if (in_bounds(out, i, j)) ko_encode(out->ptr, out->dtype, elem_offset(out, i, j), a, KO_RN);
          continue;
        }
        dstv[at] = round_to(r, dst_dtype);
      }
    }
    if (I.op != EW_ST_GLOBAL) {
      reg[d].swap(dstv);
      rd[d] = dst_dtype;
    }
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------
// kapy.matmul (Ops.td:416-439; verifier Kapy.cpp:451-487): result = lhs·rhs + acc, here with an
// fp64 accumulator and one final rounding to result->dtype.
// ---------------------------------------------------------------------------------------------
static int matmul_verify(const ko_global *lhs, const ko_global *rhs, const ko_global *acc, const ko_global *res) {
  int64_t M = extent0(lhs), K = extent1(lhs), K2 = extent0(rhs), N = extent1(rhs);
  if (K != K2) return -1;
  if (extent0(res) != M || extent1(res) != N) return -2;
  if (acc && (extent0(acc) != M || extent1(acc) != N)) return -2;
  if (dtype_bytes(lhs->dtype) != dtype_bytes(rhs->dtype)) return -3;
  bool lf8 = lhs->dtype == KO_F8E4M3 || lhs->dtype == KO_F8E5M2;
  if (!lf8 && lhs->dtype != rhs->dtype) return -4;
  if (acc && acc->dtype != KO_F16 && acc->dtype != KO_F32) return -5;
  if (acc && lhs->dtype == KO_BF16 && acc->dtype == KO_F16) return -6;
  return 0;
}

int ko_matmul(const ko_global *lhs, const ko_global *rhs, const ko_global *acc, const ko_global *result, int rmode) {
  int rc = matmul_verify(lhs, rhs, acc, result);
  if (rc) return rc;
  int64_t M = extent0(lhs), K = extent1(lhs), N = extent1(rhs);
  std::vector<double> A((size_t)M * K), Bt((size_t)N * K);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t k = 0; k < K; ++k) A[i * K + k] = ko_decode(lhs->ptr, lhs->dtype, elem_offset(lhs, i, k));
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < N; ++j)
    for (int64_t k = 0; k < K; ++k) Bt[j * K + k] = ko_decode(rhs->ptr, rhs->dtype, elem_offset(rhs, k, j));
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      const double *a = &A[i * K], *b = &Bt[j * K];
      double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
      int64_t k = 0;
      for (; k + 4 <= K; k += 4) {
        s0 += a[k] * b[k]; s1 += a[k + 1] * b[k + 1]; s2 += a[k + 2] * b[k + 2]; s3 += a[k + 3] * b[k + 3];
      }
      for (; k < K; ++k) s0 += a[k] * b[k];
      double s = (s0 + s1) + (s2 + s3);
      if (acc) s += ko_decode(acc->ptr, acc->dtype, elem_offset(acc, i, j));
      ko_encode(result->ptr, result->dtype, elem_offset(result, i, j), s, rmode);
    }
  return 0;
}

// kapy.matmul in the reference's own arithmetic when the result has f16 element type: the instruction it emits for f16
// operands then carries f16 accumulators (MatmulOpToLLVM.cpp:270-291: mma.sync ... .f16.f16.f16.f16), one instruction per
// k_step columns of the lhs (8: mma_m16n8k8_f16, 16: mma_m16n8k16_f16; the loop over K of MatmulOpToLLVM.cpp:207-262 feeds
// each instruction's result to the next as its accumulator).  Restated: the accumulator is an f16 value; every step adds the
// exact sum of the step's k_step products to it and rounds once to f16 (nearest even).  What the instruction does INSIDE a
// step is not published for either vendor's matrix unit; "exact sum, one rounding" is the model, and a device whose unit adds
// in fp32 can differ from it by one f16 unit in the last place where the exact sum sits within fp32 round-off of a tie.
int ko_matmul_f16acc(const ko_global *lhs, const ko_global *rhs, const ko_global *acc, const ko_global *result, int k_step) {
  int rc = matmul_verify(lhs, rhs, acc, result);
  if (rc) return rc;
  if (lhs->dtype != KO_F16 || rhs->dtype != KO_F16 || result->dtype != KO_F16 || (acc && acc->dtype != KO_F16)) return -7;
  if (k_step != 8 && k_step != 16) return -8;
  int64_t M = extent0(lhs), K = extent1(lhs), N = extent1(rhs);
  std::vector<double> A((size_t)M * K), Bt((size_t)N * K);
  for (int64_t i = 0; i < M; ++i)
    for (int64_t k = 0; k < K; ++k) A[i * K + k] = ko_decode(lhs->ptr, lhs->dtype, elem_offset(lhs, i, k));
  for (int64_t j = 0; j < N; ++j)
    for (int64_t k = 0; k < K; ++k) Bt[j * K + k] = ko_decode(rhs->ptr, rhs->dtype, elem_offset(rhs, k, j));
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      uint16_t held = 0;  // the accumulator register: f16 bits
      if (acc) ko_encode(&held, KO_F16, 0, ko_decode(acc->ptr, acc->dtype, elem_offset(acc, i, j)), KO_RN);
      for (int64_t k0 = 0; k0 < K; k0 += k_step) {
        long double s = (long double)ko_decode(&held, KO_F16, 0);
        for (int64_t k = k0; k < std::min<int64_t>(K, k0 + k_step); ++k) s += (long double)(A[i * K + k] * Bt[j * K + k]);  // (a product of two f16 values is exact in double)
        ko_encode(&held, KO_F16, 0, (double)s, KO_RN);
      }
      ko_encode(result->ptr, result->dtype, elem_offset(result, i, j), ko_decode(&held, KO_F16, 0), KO_RN);
    }
  return 0;
}

// W8A8: result[m,n] = RN_bf16( (sum_k a8[m,k]·w8[k,n]) · row_scale[m] · col_scale[n] ), fp64 sum.
// The scale product is formed in fp32 (row_scale*col_scale) as the kapy chain
// broadcast(row) * broadcast(col) on f32 tensors would.
int ko_matmul_scaled_f8(const ko_global *a, const ko_global *w, const float *row_scale, const float *col_scale,
                        const ko_global *result) {
  int rc = matmul_verify(a, w, nullptr, result);
  if (rc) return rc;
  int64_t M = extent0(a), K = extent1(a), N = extent1(w);
  std::vector<float> A((size_t)M * K), Bt((size_t)N * K);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t k = 0; k < K; ++k) A[i * K + k] = (float)ko_decode(a->ptr, a->dtype, elem_offset(a, i, k));
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < N; ++j)
    for (int64_t k = 0; k < K; ++k) Bt[j * K + k] = (float)ko_decode(w->ptr, w->dtype, elem_offset(w, k, j));
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      const float *x = &A[i * K], *y = &Bt[j * K];
      double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
      int64_t k = 0;
      for (; k + 4 <= K; k += 4) {
        s0 += (double)x[k] * y[k]; s1 += (double)x[k + 1] * y[k + 1];
        s2 += (double)x[k + 2] * y[k + 2]; s3 += (double)x[k + 3] * y[k + 3];
      }
      for (; k < K; ++k) s0 += (double)x[k] * y[k];
      double s = ((s0 + s1) + (s2 + s3)) * (double)(row_scale[i] * col_scale[j]);
      ko_encode(result->ptr, result->dtype, elem_offset(result, i, j), s, KO_RN);
    }
  return 0;
}

// amax/448 quantisation to e4m3fn (RN-even, saturating).  along_cols = 1: one scale per row
// (amax over columns); 0: one scale per column (amax over rows).  q keeps x's index order but is
// written densely with the same strides as given.
void ko_quantize_e4m3(const float *x, int64_t rows, int64_t cols, int64_t row_stride, int64_t col_stride,
                      int along_cols, uint8_t *q, float *scale) {
  int64_t outer = along_cols ? rows : cols, inner = along_cols ? cols : rows;
#pragma omp parallel for schedule(static)
  for (int64_t o = 0; o < outer; ++o) {
    float amax = 0.f;
    for (int64_t t = 0; t < inner; ++t) {
      int64_t r = along_cols ? o : t, c = along_cols ? t : o;
      amax = std::max(amax, std::fabs(x[r * row_stride + c * col_stride]));
    }
    float s = amax / 448.0f;
    if (s == 0.f) s = 1.f;
    scale[o] = s;
    for (int64_t t = 0; t < inner; ++t) {
      int64_t r = along_cols ? o : t, c = along_cols ? t : o;
      float v = x[r * row_stride + c * col_stride] / s;  // fp32 division, then one RN rounding to e4m3
      q[r * row_stride + c * col_stride] = (uint8_t)encode_small((double)v, kE4M3, KO_RN);
    }
  }
}

// kapy.reduce (Ops.td:441-457, ReduceOpToLLVM.cpp:51-172) with a combiner region that is one arith op.
// kind (= kapy_reduce_combiner): 0 addf (fp64 accumulate), 1 maximumf, 2 minimumf, 3 mulf, 4 maxnumf, 5 minnumf; 6 addi, 7 muli,
// 8 maxsi, 9 minsi, 10 maxui, 11 minui, 12 andi, 13 ori, 14 xori on integers (wrapping).  dst extent along `axis` is 1.
// The elements themselves are folded (no identity joins them): the fold starts from the line's first element.
static double reduce_step(double acc, double v, int kind, int dtype) {
  const double qnan = std::numeric_limits<double>::quiet_NaN();
  auto lower = [](double a, double b) { return a == b ? (std::signbit(a) ? a : b) : std::min(a, b); };   // -0 orders below +0
  auto upper = [](double a, double b) { return a == b ? (std::signbit(a) ? b : a) : std::max(a, b); };
  switch (kind) {
  case 0: return acc + v;
  case 1: return (std::isnan(acc) || std::isnan(v)) ? qnan : upper(acc, v);
  case 2: return (std::isnan(acc) || std::isnan(v)) ? qnan : lower(acc, v);
  case 3: return acc * v;
  case 4: return std::isnan(acc) ? v : std::isnan(v) ? acc : upper(acc, v);
  case 5: return std::isnan(acc) ? v : std::isnan(v) ? acc : lower(acc, v);
  default: {
    static const int op_of[] = {EW_ADDI, EW_MULI, EW_MAXSI, EW_MINSI, EW_MAXUI, EW_MINUI, EW_ANDI, EW_ORI, EW_XORI};
    return (double)int_binary_op(op_of[kind - 6], (int64_t)acc, (int64_t)v, dtype);
  }
  }
}

int ko_reduce(const ko_global *src, const ko_global *dst, int axis, int kind) {
  int64_t s0 = extent0(src), s1 = extent1(src);
  int64_t outer = axis == 0 ? s1 : s0, inner = axis == 0 ? s0 : s1;
  if (axis == 0 ? (extent0(dst) != 1 || extent1(dst) != s1) : (extent1(dst) != 1 || extent0(dst) != s0)) return -1;
  if (kind < 0 || kind > 14 || inner <= 0) return -2;
  if (kind >= 6 && (!is_int_dtype(src->dtype) || src->dtype == KO_I1 || dst->dtype != src->dtype)) return -3;
#pragma omp parallel for schedule(static)
  for (int64_t o = 0; o < outer; ++o) {
    double acc = 0.0;
    for (int64_t t = 0; t < inner; ++t) {
      int64_t i = axis == 0 ? t : o, j = axis == 0 ? o : t;
      double v = ko_decode(src->ptr, src->dtype, elem_offset(src, i, j));
      acc = t == 0 ? v : reduce_step(acc, v, kind, src->dtype);
    }
    int64_t i = axis == 0 ? 0 : o, j = axis == 0 ? o : 0;
    ko_encode(dst->ptr, dst->dtype, elem_offset(dst, i, j), acc, KO_RN);
  }
  return 0;
}

// The same reduce in the lowering's own arithmetic and order for one wavefront's tile (ReduceOpToLLVM.cpp:51-172): the tile sits in
// the registers of `lanes` lanes under `layout` (map 1 of Kgpu.cpp:186-251; nullptr: getFragmentsLayout({1, 1}, tile, rowMajor =
// true), LayoutUtils.cpp:92-110).  Per kept loop index a lane folds its elements along the reduced axis in loop order (:76-101),
// then the lanes fold by butterfly exchanges at lane distances laneOffset * 2^i for i = 0 .. numShfls - 1 (:104-119; laneOffset
// and numShfls: LayoutUtils.cpp:26-49).  Every application of the combiner is an op on the ELEMENT type: a float result is
// rounded to the source's type each time.  dst has the source's element type.
int ko_reduce_reference(const ko_global *src, const ko_global *dst, int axis, int kind, const ko_fragments *layout, int64_t lanes) {
  const int64_t shape[2] = {extent0(src), extent1(src)};
  if (axis == 0 ? (extent0(dst) != 1 || extent1(dst) != shape[1]) : (extent1(dst) != 1 || extent0(dst) != shape[0])) return -1;
  if (kind < 0 || kind > 14 || dst->dtype != src->dtype) return -2;
  if (kind >= 6 && (!is_int_dtype(src->dtype) || src->dtype == KO_I1)) return -3;
  ko_fragments def;
  if (!layout) {
    const int64_t ones[2] = {1, 1};
    ko_fragments_default(ones, shape, 1, lanes, &def);
    layout = &def;
  }
  int64_t warp_loops[2], space[2];
  ko_fragments_loops(layout, shape, warp_loops, space);
  const bool row_major = layout->major_axis == 1;
  const int64_t n_keep_iv = axis == 1 ? space[0] : space[1], n_red_iv = axis == 1 ? space[1] : space[0];
  const int64_t lane_offset = layout->major_axis == axis ? 1 : layout->lane_array[axis == 1 ? 0 : 1];
  std::set<int64_t> owners;
  for (int64_t index = 0; index < shape[axis]; ++index) {
    int64_t lane, iv;
    ko_fragments_map3(layout, shape, axis == 0 ? index : 0, axis == 0 ? 0 : index, &lane, &iv);
    owners.insert(lane);
  }
  int64_t rounds = 0;
  while ((int64_t(1) << (rounds + 1)) <= (int64_t)owners.size()) ++rounds;
  auto typed = [&](double a, double b) {
    const double r = reduce_step(a, b, kind, src->dtype);
    if (kind >= 6) return r;
    uint32_t tmp = 0;
    ko_encode(&tmp, src->dtype, 0, r, KO_RN);
    return ko_decode(&tmp, src->dtype, 0);
  };
  std::vector<double> acc((size_t)lanes);
  std::vector<int64_t> kept((size_t)lanes);
  for (int64_t k = 0; k < n_keep_iv; ++k) {
    for (int64_t lane = 0; lane < lanes; ++lane) {
      for (int64_t r = 0; r < n_red_iv; ++r) {
        const int64_t iv0 = axis == 1 ? k : r, iv1 = axis == 1 ? r : k;
        const int64_t iv = row_major ? iv0 * space[1] + iv1 : iv0 + iv1 * space[0];
        int64_t idx[2];
        ko_fragments_map12(layout, shape, 1, lane, iv, idx);
        const double v = ko_decode(src->ptr, src->dtype, elem_offset(src, idx[0], idx[1]));
        if (r == 0) { acc[lane] = v; kept[lane] = idx[axis == 1 ? 0 : 1]; }
        else acc[lane] = typed(acc[lane], v);
      }
    }
    for (int64_t i = 0; i < rounds; ++i) {
      const std::vector<double> before = acc;
      for (int64_t lane = 0; lane < lanes; ++lane) acc[lane] = typed(before[lane], before[lane ^ (lane_offset << i)]);
    }
    for (int64_t lane = 0; lane < lanes; ++lane)
      ko_encode(dst->ptr, dst->dtype, axis == 1 ? elem_offset(dst, kept[lane], 0) : elem_offset(dst, 0, kept[lane]), acc[lane], KO_RN);
  }
  return 0;
}

int ko_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // extern "C"
