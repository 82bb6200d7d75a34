// layout.hpp — the affine layout algebra of kapy's kgpu dialect for wave64 / 64-bank LDS, usable
// from host code and, being constexpr, from device code and static_asserts.
//
// What it mirrors in kapy-lang:
//   Fragments        #kgpu.fragments and its three affine maps   lib/Dialect/Kgpu/IR/Kgpu.cpp:164-263
//   default_fragments, access_simd_size                           lib/Support/LayoutUtils.cpp:92-104,
//                                                                 lib/Dialect/Kgpu/Transforms/CoalesceAccess.cpp:18-27
//   Swizzle, no_bank_conflict, swizzle_search                     lib/Support/LayoutUtils.cpp:167-225,
//                                                                 lib/Conversion/KgpuToLLVM/CpAsyncOpToLLVM.cpp:124-139
// Differences from the reference are parameters, not formulas: 64 lanes per wavefront instead
// of 32, 64 LDS banks of 4 bytes (256-byte line) instead of 32 (128-byte line).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define KAPY_HD __host__ __device__
#else
#define KAPY_HD
#endif

namespace kapy {

constexpr int kWaveSize = 64;
constexpr int kLdsBanks = 64;
constexpr int kLdsLineBytes = kLdsBanks * 4;

struct Idx2 {
  int64_t v0, v1;
};

struct Fragments {
  int32_t a0, a1;  // lane array
  int32_t l0, l1;  // lane loops
  int32_t major;   // axis along which the lane id is contiguous (1 = row-major)

  KAPY_HD constexpr bool row_major() const { return major == 1; }
  KAPY_HD constexpr int lanes() const { return a0 * a1; }

  KAPY_HD constexpr Idx2 warp_loops(Idx2 shape) const {
    int64_t w0 = shape.v0 / (int64_t(a0) * l0), w1 = shape.v1 / (int64_t(a1) * l1);
    return {w0 < 1 ? 1 : w0, w1 < 1 ? 1 : w1};
  }
  KAPY_HD constexpr Idx2 loop_space(Idx2 shape) const {
    Idx2 w = warp_loops(shape);
    return {w.v0 * l0, w.v1 * l1};
  }
  KAPY_HD constexpr int64_t loop_size(Idx2 shape) const {
    Idx2 s = loop_space(shape);
    return s.v0 * s.v1;
  }

  // (lane, iv) -> (i0, i1).  wrap = true is the reference's option 1 (indices reduced modulo the
  // shape where the layout is larger than the tensor), false its option 2.
  KAPY_HD constexpr Idx2 to_index(Idx2 shape, int64_t lane, int64_t iv, bool wrap) const {
    Idx2 s = loop_space(shape);
    // Work in "minor, major" order so that one formula serves both orientations.
    const int64_t A[2] = {row_major() ? a0 : a1, row_major() ? a1 : a0};
    const int64_t L[2] = {row_major() ? l0 : l1, row_major() ? l1 : l0};
    const int64_t S[2] = {row_major() ? s.v0 : s.v1, row_major() ? s.v1 : s.v0};
    const int64_t E[2] = {row_major() ? shape.v0 : shape.v1, row_major() ? shape.v1 : shape.v0};
    const int64_t lid[2] = {lane / A[1], lane % A[1]};
    const int64_t ivs[2] = {iv / S[1], iv % S[1]};
    int64_t out[2] = {0, 0};
    for (int d = 0; d < 2; ++d) {
      int64_t span = A[d] * L[d];
      out[d] = (ivs[d] / L[d]) * span + lid[d] * L[d] + ivs[d] % L[d];
      if (wrap && span > E[d]) out[d] %= E[d];
    }
    return row_major() ? Idx2{out[0], out[1]} : Idx2{out[1], out[0]};
  }

  // (i0, i1) -> (lane, iv): the reference's option 3.
  KAPY_HD constexpr Idx2 to_lane_iv(Idx2 shape, int64_t i0, int64_t i1) const {
    Idx2 s = loop_space(shape);
    int64_t span0 = int64_t(a0) * l0, span1 = int64_t(a1) * l1;
    int64_t lane0 = (i0 % span0) / l0, lane1 = (i1 % span1) / l1;
    int64_t iv0 = (i0 / span0) * l0 + i0 % l0, iv1 = (i1 / span1) * l1 + i1 % l1;
    int64_t lane = row_major() ? lane0 * a1 + lane1 : lane0 + lane1 * a0;
    int64_t iv = row_major() ? iv0 * s.v1 + iv1 : iv0 + iv1 * s.v0;
    return {lane, iv};
  }

  KAPY_HD constexpr Fragments transposed() const { return {a1, a0, l1, l0, 1 - major}; }
  KAPY_HD constexpr Fragments axes_exchanged() const { return {a0, a1, l0, l1, 1 - major}; }
};

KAPY_HD constexpr Fragments default_fragments(Idx2 lane_loops, Idx2 shape, bool row_major) {
  int64_t extent = row_major ? shape.v1 : shape.v0, loops = row_major ? lane_loops.v1 : lane_loops.v0;
  int64_t max_lanes = extent / loops < 1 ? 1 : extent / loops;
  int64_t along = kWaveSize < max_lanes ? kWaveSize : max_lanes;
  int64_t across = kWaveSize / along;
  return row_major ? Fragments{int32_t(across), int32_t(along), int32_t(lane_loops.v0), int32_t(lane_loops.v1), 1}
                   : Fragments{int32_t(along), int32_t(across), int32_t(lane_loops.v0), int32_t(lane_loops.v1), 0};
}

KAPY_HD constexpr int64_t access_simd_size(int64_t alignment, int64_t bits, int64_t numel) {
  int64_t s = alignment * 8 / bits < 128 / bits ? alignment * 8 / bits : 128 / bits;
  int64_t per_lane = (numel + kWaveSize - 1) / kWaveSize;
  if (per_lane < s) s = per_lane;
  if (s < 32 / bits) s = 32 / bits;
  return s;
}

// result (lane, iv) of a kgpu.change reads source (lane, iv) = src.to_lane_iv(dst.to_index(lane, iv)).
KAPY_HD constexpr Idx2 change_source(const Fragments &src, const Fragments &dst, Idx2 shape, int64_t lane, int64_t iv) {
  Idx2 e = dst.to_index(shape, lane, iv, false);
  return src.to_lane_iv(shape, e.v0, e.v1);
}

struct Swizzle {
  int32_t stride0, stride1;  // elements
  int32_t bank_param;        // banks kept together: 4 -> 16-byte atoms, 2 -> 8-byte, 1 -> 4-byte
  int32_t line_param;        // how many consecutive lines take part in the XOR
  int32_t rotate = 0;        // the XOR key is (line % line_param) rotated left by this many bits within log2(line_param) bits
                             // (0: the reference's key; the search over the gfx950 read phases below also tries the others)

  KAPY_HD constexpr int64_t key(int64_t line) const {
    int64_t k = line % line_param;
    int bits = 0;
    for (int32_t v = line_param; v > 1; v >>= 1) ++bits;
    const int r = bits > 0 ? rotate % bits : 0;
    return r ? ((k << r) | (k >> (bits - r))) & (line_param - 1) : k;
  }
  // Element offset of (i0, i1) in the swizzled buffer.
  KAPY_HD constexpr int64_t offset(int64_t bits, int64_t i0, int64_t i1) const {
    int64_t line_bits = int64_t(kLdsLineBytes) * 8;
    int64_t bit_off = (i0 * stride0 + i1 * stride1) * bits;
    int64_t bank = (bit_off % line_bits) / 32, line = bit_off / line_bits, sub = bit_off % 32;
    int64_t bank_sw = ((bank / bank_param) ^ key(line)) * bank_param + bank % bank_param;
    return (line * line_bits + bank_sw * 32 + sub) / bits;
  }
};

// Does the first phase of a wave's access (kWaveSize / bank_param lanes, each touching `simd`
// contiguous elements) hit every bank from at most one line?  Same model as the reference's
// isNoBankConflict with the bank and lane counts of gfx950.  constexpr: kernels evaluate it at
// compile time to derive their LDS swizzle from the MFMA operand layout.
KAPY_HD constexpr bool no_bank_conflict(const Fragments &access, Idx2 shape, const Swizzle &sw, int64_t bits, int64_t alignment) {
  const int64_t line_bits = int64_t(kLdsLineBytes) * 8;
  bool shared_row_major = sw.stride1 == 1;
  int64_t simd = sw.stride0 == 1 ? access.l0 : access.l1;
  int64_t atom = int64_t(sw.bank_param) * 32 / bits;
  if (atom < simd) simd = atom;
  Idx2 space = access.loop_space(shape);
  int64_t iv_step = 1;
  if (shared_row_major && !access.row_major()) iv_step = space.v0;
  if (!shared_row_major && access.row_major()) iv_step = space.v1;
  // bank -> the single line seen so far (-1: none)
  int64_t seen[kLdsBanks] = {};
  for (int b = 0; b < kLdsBanks; ++b) seen[b] = -1;
  for (int64_t lane = 0; lane < kWaveSize / sw.bank_param; ++lane)
    for (int64_t iv = 0; iv < simd * iv_step; iv += iv_step) {
      Idx2 e = access.to_index(shape, lane, iv, true);
      int64_t bit_off = (alignment % kLdsLineBytes) * 8;
      bit_off += (shared_row_major ? e.v0 * sw.stride0 + e.v1 : e.v0 + e.v1 * sw.stride1) * bits;
      int64_t bank = bit_off % line_bits / 32, line = bit_off / line_bits;
      bank = ((bank / sw.bank_param) ^ sw.key(line)) * sw.bank_param + bank % sw.bank_param;
      if (seen[bank] >= 0 && seen[bank] != line) return false;
      seen[bank] = line;
    }
  return true;
}

// Candidates in the reference's order: bank_param 4, 2, 1; line_param 1, 2, 4, ... banks/bank_param.
KAPY_HD constexpr int swizzle_search(const Fragments &access, Idx2 shape, int32_t stride0, int32_t stride1, int64_t bits,
                                     int64_t alignment, int32_t *pairs, int max_pairs) {
  int n = 0;
  for (int32_t bp = 4; bp >= 1; bp /= 2)
    for (int32_t lp = 1; lp <= kLdsBanks / bp; lp *= 2)
      if (no_bank_conflict(access, shape, Swizzle{stride0, stride1, bp, lp, 0}, bits, alignment)) {
        if (n < max_pairs) {
          pairs[2 * n] = bp;
          pairs[2 * n + 1] = lp;
        }
        ++n;
      }
  return n;
}

// First conflict-free candidate of the search (the reference takes the first hit too,
// LayoutUtils.cpp:216-224); {0,0,0,0} when none exists.
KAPY_HD constexpr Swizzle first_swizzle(const Fragments &access, Idx2 shape, int32_t stride0, int32_t stride1, int64_t bits,
                                        int64_t alignment) {
  int32_t pair[2] = {0, 0};
  int n = swizzle_search(access, shape, stride0, stride1, bits, alignment, pair, 1);
  return n > 0 ? Swizzle{stride0, stride1, pair[0], pair[1], 0} : Swizzle{0, 0, 0, 0, 0};
}

// The same question asked the way the gfx950 LDS answers it.  The model above, like the reference's, looks at the first
// kWaveSize / bank_param lanes and at a lane's first access.  The hardware serves a wave's 16-byte reads (ds_read_b128) in four
// phases of sixteen lanes that are NOT consecutive - {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31} and the same plus 32 -
// 8-byte reads in two halves of 32 lanes, 4-byte reads all at once; a lane that reads more than one atom issues one
// instruction per atom, each served by itself.  Conflict-free here means: in every phase of every instruction, every bank
// is asked for at most one line.  (Measured on the 16x16x128 operand reads - row lane % 16, chunks 2 * (lane / 16) and + 1 of
// a 128-byte row: the plain key (4, 8) passes the model above and conflicts on half of the LDS's active cycles; the key
// rotated by one bit is free of conflicts.  This model says both.)
KAPY_HD constexpr int gfx950_read_phases(int32_t bank_param) { return bank_param >= 4 ? 4 : bank_param == 2 ? 2 : 1; }
KAPY_HD constexpr int gfx950_phase_lane(int32_t bank_param, int phase, int i) {
  if (bank_param >= 4) {
    constexpr int first[2][4] = {{0, 12, 20, 24}, {4, 8, 16, 28}};  // each start: four consecutive lanes
    return first[phase & 1][i / 4] + i % 4 + 32 * (phase >> 1);
  }
  return bank_param == 2 ? 32 * phase + i : i;
}
KAPY_HD constexpr bool no_bank_conflict_gfx950(const Fragments &access, Idx2 shape, const Swizzle &sw, int64_t bits, int64_t alignment) {
  const int64_t line_bits = int64_t(kLdsLineBytes) * 8;
  const bool shared_row_major = sw.stride1 == 1;
  const int64_t per_lane = sw.stride0 == 1 ? access.l0 : access.l1;
  int64_t atom = int64_t(sw.bank_param) * 32 / bits;
  if (atom > per_lane) atom = per_lane;
  const Idx2 space = access.loop_space(shape);
  int64_t iv_step = 1;
  if (shared_row_major && !access.row_major()) iv_step = space.v0;
  if (!shared_row_major && access.row_major()) iv_step = space.v1;
  const int phases = gfx950_read_phases(sw.bank_param), lanes = kWaveSize / phases;
  for (int64_t first = 0; first < per_lane; first += atom)
    for (int ph = 0; ph < phases; ++ph) {
      int64_t seen[kLdsBanks] = {};
      for (int b = 0; b < kLdsBanks; ++b) seen[b] = -1;
      for (int i = 0; i < lanes; ++i) {
        const int64_t lane = gfx950_phase_lane(sw.bank_param, ph, i);
        for (int64_t e = first; e < first + atom; ++e) {
          const Idx2 at = access.to_index(shape, lane, e * iv_step, true);
          int64_t bit_off = (alignment % kLdsLineBytes) * 8;
          bit_off += (shared_row_major ? at.v0 * sw.stride0 + at.v1 : at.v0 + at.v1 * sw.stride1) * bits;
          int64_t bank = bit_off % line_bits / 32;
          const int64_t line = bit_off / line_bits;
          bank = ((bank / sw.bank_param) ^ sw.key(line)) * sw.bank_param + bank % sw.bank_param;
          if (seen[bank] >= 0 && seen[bank] != line) return false;
          seen[bank] = line;
        }
      }
    }
  return true;
}
// Candidates (bank_param, line_param, rotate) in the reference's order with the rotations innermost; writes up to max_triples.
KAPY_HD constexpr int swizzle_search_gfx950(const Fragments &access, Idx2 shape, int32_t stride0, int32_t stride1, int64_t bits, int64_t alignment,
                                            int32_t *triples, int max_triples) {
  int n = 0;
  for (int32_t bp = 4; bp >= 1; bp /= 2)
    for (int32_t lp = 1, lp_bits = 0; lp <= kLdsBanks / bp; lp *= 2, ++lp_bits)
      for (int32_t rot = 0; rot < (lp_bits > 0 ? lp_bits : 1); ++rot)
        if (no_bank_conflict_gfx950(access, shape, Swizzle{stride0, stride1, bp, lp, rot}, bits, alignment)) {
          if (n < max_triples) {
            triples[3 * n] = bp;
            triples[3 * n + 1] = lp;
            triples[3 * n + 2] = rot;
          }
          ++n;
        }
  return n;
}
KAPY_HD constexpr Swizzle first_swizzle_gfx950(const Fragments &access, Idx2 shape, int32_t stride0, int32_t stride1, int64_t bits, int64_t alignment) {
  int32_t t[3] = {0, 0, 0};
  const int n = swizzle_search_gfx950(access, shape, stride0, stride1, bits, alignment, t, 1);
  return n > 0 ? Swizzle{stride0, stride1, t[0], t[1], t[2]} : Swizzle{0, 0, 0, 0, 0};
}

// ---------------------------------------------------------------------------------------------
// MFMA operand / accumulator layouts of gfx950 written as fragments (the counterpart of
// getDefaultLayouts(MatmulOp), lib/Support/LayoutUtils.cpp:123-149).  For v_mfma_f32_MxNxK with
// 16-bit operands a lane holds `kpack` consecutive K elements of one row (lhs) or column (rhs);
// the accumulator holds 4 consecutive rows of one column per register quad.
//   32x32x16: lhs <[32,2],[1,8],(1,0)>  rhs <[2,32],[8,1],(0,1)>  acc <[2,32],[4,1],(0,1)>
//   16x16x32: lhs <[16,4],[1,8],(1,0)>  rhs <[4,16],[8,1],(0,1)>  acc <[4,16],[4,1],(0,1)>
//   f8 16x16x128: lhs <[16,4],[1,32],(1,0)>  rhs <[4,16],[32,1],(0,1)>  acc as 16x16x32
//   f8 32x32x64:  lhs <[32,2],[1,32],(1,0)>  rhs <[2,32],[32,1],(0,1)>  acc as 32x32x16
// ---------------------------------------------------------------------------------------------
struct MfmaShape {
  int m, n, k, kpack;
};
KAPY_HD constexpr Fragments mfma_lhs(MfmaShape s) { return {s.m, kWaveSize / s.m, 1, s.kpack, 0}; }
KAPY_HD constexpr Fragments mfma_rhs(MfmaShape s) { return {kWaveSize / s.n, s.n, s.kpack, 1, 1}; }
KAPY_HD constexpr Fragments mfma_acc(MfmaShape s) { return {kWaveSize / s.n, s.n, 4, 1, 1}; }
// The accumulator when the instruction is issued with the operands exchanged (rhs fragment in the first operand
// slot, lhs fragment in the second: the mirrored operand layouts make that legal without moving a register).
// The instruction then computes the transposed block, so over the [m x n] result a lane's register quad holds
// four consecutive COLUMNS of one row - what a row-major store wants.  The tiled matmul kernels issue this form.
//   32x32x16: <[32,2],[1,4],(1,0)>   16x16x32: <[16,4],[1,4],(1,0)>
KAPY_HD constexpr Fragments mfma_acc_exchanged(MfmaShape s) { return mfma_acc(MfmaShape{s.n, s.m, s.k, s.kpack}).transposed(); }
constexpr MfmaShape kMfma32x32x16{32, 32, 16, 8};
constexpr MfmaShape kMfma16x16x32{16, 16, 32, 8};
constexpr MfmaShape kMfma16x16x128F8{16, 16, 128, 32};
constexpr MfmaShape kMfma32x32x64F8{32, 32, 64, 32};

}  // namespace kapy
