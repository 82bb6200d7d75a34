// mfma.hpp — the matrix instructions of gfx950 as operand policies, each tied to the fragments layouts
// (layout.hpp) that say which lane and register holds which element of the lhs, rhs and accumulator tiles.
//
// Reference: MatmulOpConversion maps the per-lane loop-iv slots of the lhs / rhs / acc structs to the
// registers of mma.sync through tables derived from the operands' layouts
// (lib/Conversion/KgpuToLLVM/MatmulOpToLLVM.cpp:94-123); the layouts come from getDefaultLayouts
// (lib/Support/LayoutUtils.cpp:123-149) and are checked by the kgpu verifier
// (lib/Dialect/Kgpu/IR/Kgpu.cpp:83-147).  Here every kernel takes the position of a lane's registers
// from kShape's layouts (operand_lane / acc_lane below) instead of spelling out lane % 16, lane / 16,
// and the probe kernel in matmul.hip runs each policy on registers laid out by those same layouts,
// so a layout that did not describe the hardware would give wrong numbers there.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.hpp"

namespace kapy {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

// Operand element policies: bytes per element, the K extent of one matrix instruction, how many
// 16-byte LDS chunks a lane feeds it per operand, its duration in clocks (4 per pass), and its shape.
// mfma(first, second, acc) issues the instruction with `first` in its first operand slot: acc += first . second
// with first an [m x k] block (layout mfma_lhs(kShape)), second a [k x n] block (mfma_rhs), acc [m x n] (mfma_acc).
struct Bf16 {
  static constexpr int kBytes = 2, kSliceK = 16, kChunks = 1, kMfmaClocks = 32, kM = 32;
  static constexpr MfmaShape kShape = kMfma32x32x16;
  using Acc = f32x16;
  static __device__ __forceinline__ f32x16 mfma(const u32x4 *a, const u32x4 *b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[0]), __builtin_bit_cast(bf16x8, b[0]), c, 0, 0, 0);
  }
};
struct F16 {
  static constexpr int kBytes = 2, kSliceK = 16, kChunks = 1, kMfmaClocks = 32, kM = 32;
  static constexpr MfmaShape kShape = kMfma32x32x16;
  using Acc = f32x16;
  static __device__ __forceinline__ f32x16 mfma(const u32x4 *a, const u32x4 *b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b[0]), c, 0, 0, 0);
  }
};
// The 16x16x32 forms: kM = 16 rows per operand block, four K-groups of lanes.  Same flops per clock
// as 32x32x16, but each accumulator register is read and written once per 32 K instead of per 16 K;
// under sustained load the chip holds a ~13% higher clock with them (it is power-limited), which
// outweighs the doubled operand-register reads.
struct Bf16M16 {
  static constexpr int kBytes = 2, kSliceK = 32, kChunks = 1, kMfmaClocks = 16, kM = 16;
  static constexpr MfmaShape kShape = kMfma16x16x32;
  using Acc = f32x4;
  static __device__ __forceinline__ f32x4 mfma(const u32x4 *a, const u32x4 *b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[0]), __builtin_bit_cast(bf16x8, b[0]), c, 0, 0, 0);
  }
  // The same instruction accumulating in place in an accumulator register (see F8M16::mfma_in_place): where registers are
  // not scarce the compiler moves accumulators between the two halves of the register file around the instruction,
  // several vector moves per matrix instruction, which the matrix pipe then waits for.
  static __device__ __forceinline__ void mfma_in_place(const u32x4 *a, const u32x4 *b, f32x4 &c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a[0]), "v"(b[0]));
  }
};
struct F16M16 {
  static constexpr int kBytes = 2, kSliceK = 32, kChunks = 1, kMfmaClocks = 16, kM = 16;
  static constexpr MfmaShape kShape = kMfma16x16x32;
  using Acc = f32x4;
  static __device__ __forceinline__ f32x4 mfma(const u32x4 *a, const u32x4 *b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[0]), __builtin_bit_cast(f16x8, b[0]), c, 0, 0, 0);
  }
  // The same instruction accumulating in place in an accumulator register (see F8M16::mfma_in_place): where registers are
  // not scarce the compiler moves accumulators between the two halves of the register file around the instruction,
  // several vector moves per matrix instruction, which the matrix pipe then waits for.
  static __device__ __forceinline__ void mfma_in_place(const u32x4 *a, const u32x4 *b, f32x4 &c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a[0]), "v"(b[0]));
  }
};
// OCP fp8, v_mfma_scale_f32_32x32x64_f8f6f4 with unit block scales (E8M0 127 = 2^0).  AF / BF are the
// format selectors of the first / second instruction operand: 0 = E4M3, 1 = E5M2 (kapy lets the two
// f8 types mix, Kapy.cpp:484-487).  A lane feeds 32 K-contiguous bytes per operand: two chunks.
// (Which 32 of the instruction's K positions a lane's bytes take is not observable: both operands use the
// same assignment and the sum over K does not depend on it.)
template <int AF, int BF>
struct F8 {
  static constexpr int kBytes = 1, kSliceK = 64, kChunks = 2, kMfmaClocks = 64, kM = 32;
  static constexpr MfmaShape kShape = kMfma32x32x64F8;
  using Acc = f32x16;
  static __device__ __forceinline__ f32x16 mfma(const u32x4 *a, const u32x4 *b, f32x16 c) {
    i32x8 av = {(int)a[0][0], (int)a[0][1], (int)a[0][2], (int)a[0][3], (int)a[1][0], (int)a[1][1], (int)a[1][2], (int)a[1][3]};
    i32x8 bv = {(int)b[0][0], (int)b[0][1], (int)b[0][2], (int)b[0][3], (int)b[1][0], (int)b[1][1], (int)b[1][2], (int)b[1][3]};
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, AF, BF, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  }
};
// v_mfma_scale_f32_16x16x128_f8f6f4: 16-row blocks, four K-groups of lanes with 32 bytes each.
template <int AF, int BF>
struct F8M16 {
  static constexpr int kBytes = 1, kSliceK = 128, kChunks = 2, kMfmaClocks = 32, kM = 16;
  static constexpr MfmaShape kShape = kMfma16x16x128F8;
  using Acc = f32x4;
  static __device__ __forceinline__ f32x4 mfma(const u32x4 *a, const u32x4 *b, f32x4 c) {
    i32x8 av = {(int)a[0][0], (int)a[0][1], (int)a[0][2], (int)a[0][3], (int)a[1][0], (int)a[1][1], (int)a[1][2], (int)a[1][3]};
    i32x8 bv = {(int)b[0][0], (int)b[0][1], (int)b[0][2], (int)b[0][3], (int)b[1][0], (int)b[1][1], (int)b[1][2], (int)b[1][3]};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, c, AF, BF, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  }
  // The same instruction accumulating in place in an accumulator register: the tiled kernel's 256 accumulators fill that half
  // of the register file exactly, and left to itself the compiler gives some matrix instructions a destination other than
  // their accumulator operand, which needs registers that are not there.  cbsz / blgp carry the operand formats.
  static __device__ __forceinline__ void mfma_in_place(const u32x4 *a, const u32x4 *b, f32x4 &c) {
    i32x8 av = {(int)a[0][0], (int)a[0][1], (int)a[0][2], (int)a[0][3], (int)a[1][0], (int)a[1][1], (int)a[1][2], (int)a[1][3]};
    i32x8 bv = {(int)b[0][0], (int)b[0][1], (int)b[0][2], (int)b[0][3], (int)b[1][0], (int)b[1][1], (int)b[1][2], (int)b[1][3]};
    const int unit_scales = 0x7F7F7F7F;
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0] cbsz:%4 blgp:%5"
                 : "+a"(c)
                 : "v"(av), "v"(bv), "v"(unit_scales), "n"(AF), "n"(BF));
  }
};

// Where a lane's operand registers sit in an operand block: the row (lhs) or column (rhs) they belong to and
// the position along K of the first of their kpack consecutive elements, read off the fragments layout.
// Both operands are staged K-contiguous ([rows][K] for the lhs, [columns][K] for the rhs), so one answer serves
// both as long as the two layouts mirror each other, which operand_layouts_mirror() checks at compile time.
struct OperandLane {
  int32_t row, k0;
};
KAPY_HD constexpr OperandLane operand_lane(MfmaShape s, int lane) {
  const Idx2 at = mfma_lhs(s).to_index({s.m, s.k}, lane, 0, false);
  return {(int32_t)at.v0, (int32_t)at.v1};
}
constexpr bool operand_layouts_mirror(MfmaShape s) {
  if (s.m != s.n) return false;
  for (int lane = 0; lane < kWaveSize; ++lane)
    for (int iv = 0; iv < s.kpack; ++iv) {
      const Idx2 a = mfma_lhs(s).to_index({s.m, s.k}, lane, iv, false), b = mfma_rhs(s).to_index({s.k, s.n}, lane, iv, false);
      const OperandLane o = operand_lane(s, lane);
      if (a.v0 != b.v1 || a.v1 != b.v0) return false;            // rhs(k, n) of a lane = lhs(m, k) of the same lane, transposed
      if (a.v0 != o.row || a.v1 != o.k0 + iv) return false;      // a lane's registers: kpack consecutive K of one row
    }
  return true;
}
static_assert(operand_layouts_mirror(kMfma32x32x16) && operand_layouts_mirror(kMfma16x16x32) && operand_layouts_mirror(kMfma16x16x128F8) &&
                  operand_layouts_mirror(kMfma32x32x64F8),
              "lhs and rhs fragments of a matrix instruction must mirror each other");

// Where a lane's accumulator registers sit in the [m x n] block under `layout` (mfma_acc for the instruction as
// documented, mfma_acc_exchanged for kernels that hand the rhs fragment to the first operand slot): register
// 4q + e holds element (row + e*drow, col + e*dcol) + q*(qrow, qcol), i.e. quads of four consecutive rows of
// one column (drow = 1) or four consecutive columns of one row (dcol = 1).
struct AccLane {
  int32_t row, col;      // element of register 0
  int32_t drow, dcol;    // step from register e to e + 1 inside a quad
  int32_t qrow, qcol;    // step from quad q to q + 1
};
KAPY_HD constexpr AccLane acc_lane(const Fragments &layout, MfmaShape s, int lane) {
  const Idx2 shape{s.m, s.n};
  const Idx2 r0 = layout.to_index(shape, lane, 0, false), r1 = layout.to_index(shape, lane, 1, false);
  const int64_t regs = layout.loop_size(shape);
  const Idx2 r4 = regs > 4 ? layout.to_index(shape, lane, 4, false) : r0;
  return {(int32_t)r0.v0, (int32_t)r0.v1, (int32_t)(r1.v0 - r0.v0), (int32_t)(r1.v1 - r0.v1), (int32_t)(r4.v0 - r0.v0), (int32_t)(r4.v1 - r0.v1)};
}
// every register of every lane is where acc_lane's six numbers say it is
constexpr bool acc_lane_describes(const Fragments &layout, MfmaShape s) {
  const Idx2 shape{s.m, s.n};
  if (layout.loop_size(shape) * kWaveSize != int64_t(s.m) * s.n) return false;
  for (int lane = 0; lane < kWaveSize; ++lane) {
    const AccLane a = acc_lane(layout, s, lane);
    for (int64_t iv = 0; iv < layout.loop_size(shape); ++iv) {
      const Idx2 at = layout.to_index(shape, lane, iv, false);
      const int64_t q = iv / 4, e = iv % 4;
      if (at.v0 != a.row + e * a.drow + q * a.qrow || at.v1 != a.col + e * a.dcol + q * a.qcol) return false;
    }
  }
  return true;
}
static_assert(acc_lane_describes(mfma_acc(kMfma32x32x16), kMfma32x32x16) && acc_lane_describes(mfma_acc(kMfma16x16x32), kMfma16x16x32) &&
                  acc_lane_describes(mfma_acc_exchanged(kMfma32x32x16), kMfma32x32x16) && acc_lane_describes(mfma_acc_exchanged(kMfma16x16x32), kMfma16x16x32),
              "accumulator registers come in quads along one axis");

}  // namespace kapy
