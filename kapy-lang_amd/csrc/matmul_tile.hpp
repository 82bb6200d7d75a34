// matmul_tile.hpp — what the tiled matrix-product kernels share: the LDS image of a K-contiguous operand tile, the
// transposing LDS read and its wait, wait-counter immediates, the fused elementwise tail, the element and strip epilogues,
// the tile walk over the XCDs and the meeting of split-K parts.  Included by the kernel sources (each gets its own copy:
// everything here has internal linkage).
#pragma once
#include <algorithm>
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "layout.hpp"
#include "matmul_params.hpp"
#include "mfma.hpp"
#include "ew_machine.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

// LDS image of an operand tile: [rows][ROWBYTES] bytes, K contiguous, 16-byte chunks XOR-ed with the
// line index.  The parameters come from the compile-time search (the reference's getSwizzlingLayouts for 64 banks,
// asked of the gfx950 read phases: layout.hpp) run on the access layout of the operand reads of the matrix instruction
// the kernel is built for: the lhs fragments of T::kShape counted in bytes (T::kShape.m lanes down the rows, the K-groups
// across, 16 contiguous bytes per lane and read instruction).
// BLOCK_ROWS: a kernel that computes the key once for all blocks of BLOCK_ROWS rows needs a swizzle period that divides such a
// block; where the hardware search's first hit does not, the layout falls back to the reference model's first hit.
template <int ROWBYTES, typename T, int BLOCK_ROWS = 0>
struct TileLayout {
  static constexpr int kRowBytes = ROWBYTES;
  static constexpr MfmaShape kS = T::kShape;
  static constexpr Fragments kAccess{mfma_lhs(kS).a0, mfma_lhs(kS).a1, 1, mfma_lhs(kS).l1 * T::kBytes, mfma_lhs(kS).major};
  static constexpr Swizzle kSwizzleHw = first_swizzle_gfx950(kAccess, {kS.m, kS.k * T::kBytes}, ROWBYTES, 1, 8, 1024);
  static constexpr bool kPeriodFits = BLOCK_ROWS == 0 || (BLOCK_ROWS * ROWBYTES) % (256 * kSwizzleHw.line_param) == 0;
  static constexpr Swizzle kSwizzle = kPeriodFits ? kSwizzleHw : first_swizzle(kAccess, {kS.m, kS.k * T::kBytes}, ROWBYTES, 1, 8, 1024);
  static_assert(kSwizzle.bank_param == 4, "MFMA operand reads are 16-byte: the search must return 16-byte atoms");
  static constexpr int kLineParam = kSwizzle.line_param;
  // the chunk index is XOR-ed with the line index taken modulo kLineParam and rotated as the search found it
  static __device__ __forceinline__ uint32_t key_of(uint32_t o) { return (uint32_t)kSwizzle.key((o >> 8) & (kLineParam - 1)); }
  // byte offset of 16-byte chunk `chunk` of row `row`
  static __device__ __forceinline__ uint32_t offset(uint32_t row, uint32_t chunk) {
    uint32_t o = row * kRowBytes + chunk * 16;
    return o ^ (key_of(o) << 4);
  }
  // inverse on a linear LDS byte offset: which (row, chunk) of the tile lives there
  static __device__ __forceinline__ void locate(uint32_t lds_off, uint32_t &row, uint32_t &chunk) {
    uint32_t o = lds_off ^ (key_of(lds_off) << 4);
    row = o / kRowBytes;
    chunk = (o % kRowBytes) / 16;
  }
};

// ds_read_b64_tr_b16 issued as opaque assembly.  Through the compiler's builtin every such read is
// preceded by s_waitcnt vmcnt(0) (it is taken to alias the LDS-direct loads in flight), which
// serialises the whole global->LDS pipeline; ordering against those loads is established by the
// kernel's own waits and barriers.  The result is pending until the wait below has been executed: every
// register that holds a pending result is an in/out operand of that wait, so the compiler sees each later
// use as a use of the WAIT's result and cannot place it (or a copy feeding it) before the wait.
typedef uint32_t u32x2_lds __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x2_lds tr_read_b64(const char *lds_ptr) {
  const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)lds_ptr;  // LDS pointers are 32-bit byte offsets
  u32x2_lds r;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
// The same from LDS byte address `addr` + IMM (below 64 KiB), the immediate in the instruction: no address arithmetic.
template <uint32_t IMM>
__device__ __forceinline__ u32x2_lds tr_read_b64_at(uint32_t addr) {
  static_assert(IMM < 65536, "a DS instruction's offset field has 16 bits");
  u32x2_lds r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(IMM));
  return r;
}
// Waits for the transposing reads whose results sit in h0[j], h1[j] (j < 4) and hands those registers back as its own results.
__device__ __forceinline__ void tr_reads_wait(u32x2_lds (&h0)[4], u32x2_lds (&h1)[4]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(h0[0]), "+v"(h0[1]), "+v"(h0[2]), "+v"(h0[3]), "+v"(h1[0]), "+v"(h1[1]), "+v"(h1[2]), "+v"(h1[3])
               :
               : "memory");
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose counter is a compile-time constant in the body
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }

// s_waitcnt immediate that waits only on vmcnt <= n (gfx9 encoding: vmcnt in bits [3:0] and [15:14],
// expcnt [6:4] and lgkmcnt [11:8] left at "no wait").
constexpr int vmcnt_imm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }
// Same, and also lgkmcnt(0): this wave's LDS reads have returned.  Used in front of a barrier after
// which other waves overwrite the LDS stage this wave has been reading.
constexpr int vmcnt_lgkm0_imm(int n) { return 0x0070 | (n & 15) | ((n >> 4) << 14); }


// The fused elementwise tail: every step rounds to fp32 on its own, as the separate kapy ops would.  Only activations
// that are a handful of instructions are compiled into the epilogues (every kernel variant carries hundreds of unrolled copies).
__device__ __forceinline__ bool has_tail(const GemmParams &p) { return p.bias != nullptr || p.act >= 0 || p.alpha != 1.0f; }
__device__ __forceinline__ float apply_tail(const GemmParams &p, float v, float bias) {
  if (p.alpha != 1.0f) v = __fmul_rn(v, p.alpha);
  if (p.bias) v = __fadd_rn(v, bias);
  switch (p.act) {
  case KAPY_EW_GELU_TANH: return gelu_tanh_f32(v);
  case KAPY_EW_MAXIMUMF: return max_nan(v, p.act_operand);
  case KAPY_EW_MINIMUMF: return min_nan(v, p.act_operand);
  case KAPY_EW_NEGF: return -v;
  case KAPY_EW_ABSF: return fabsf(v);
  }
  return v;
}

// The same on 8 values, with every uniform decision taken once.
__device__ __forceinline__ void apply_tail8(const GemmParams &p, float (&v)[8], const float (&bias)[8]) {
  if (p.alpha != 1.0f) {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = __fmul_rn(v[e], p.alpha);
  }
  if (p.bias) {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = __fadd_rn(v[e], bias[e]);
  }
  switch (p.act) {
  case KAPY_EW_GELU_TANH:
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = gelu_tanh_f32(v[e]);
    break;
  case KAPY_EW_MAXIMUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = max_nan(v[e], p.act_operand);
    break;
  case KAPY_EW_MINIMUMF:
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = min_nan(v[e], p.act_operand);
    break;
  case KAPY_EW_NEGF:
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = -v[e];
    break;
  case KAPY_EW_ABSF:
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = fabsf(v[e]);
    break;
  }
}

__device__ __forceinline__ void store_result(const GemmParams &p, int32_t m, int32_t n, float v) {
  if (m >= p.M || n >= p.N) return;
  if (p.row_scale) v = __fmul_rn(v, __fmul_rn(p.row_scale[m], p.col_scale[n]));
  if (has_tail(p)) v = apply_tail(p, v, p.bias ? load_as_f32(p.bias, p.bias_dtype, n) : 0.f);
  if (p.acc_dtype >= 0) v += load_as_f32(p.acc, p.acc_dtype, m * p.acc_sm + n * p.acc_sn);
  int64_t idx = m * p.d_sm + n * p.d_sn;
  switch (p.d_dtype) {
  case KAPY_F32: ((float *)p.d)[idx] = v; break;
  case KAPY_F16: ((uint16_t *)p.d)[idx] = p.rz ? f32_to_f16_rz(v) : f32_to_f16_rn(v); break;
  default: ((uint16_t *)p.d)[idx] = p.rz ? f32_to_bf16_rz(v) : f32_to_bf16_rn(v); break;
  }
}

// Epilogues of one accumulator block.  Every kernel here issues the matrix instruction with the operands
// exchanged (rhs fragment in the first slot), so the block's registers follow mfma_acc_exchanged: a lane's
// register quad holds four consecutive columns of one row.  Where each register sits is read off that layout
// (acc_lane), e.g. for 32x32: register v of lane l holds D[l%32][8*(v/4) + 4*(l/32) + v%4].
constexpr bool quads_run_along_rows(MfmaShape s) {
  const AccLane a = acc_lane(mfma_acc_exchanged(s), s, 0);
  return a.drow == 0 && a.dcol == 1 && a.qrow == 0;
}
static_assert(quads_run_along_rows(kMfma32x32x16) && quads_run_along_rows(kMfma16x16x32), "the packed epilogues store register quads as 8 contiguous bytes of a row");
// Packed form: 16-bit row-major result, block fully in range, no accumulator input, RN: one
// 8-byte store per quad.
__device__ __forceinline__ void store_block_packed(const GemmParams &p, int32_t m_base, int32_t n_base, int lane, const f32x16 &acc) {
  const AccLane at = acc_lane(mfma_acc_exchanged(kMfma32x32x16), kMfma32x32x16, lane);
  char *row = p.d + ((int64_t)(m_base + at.row) * p.d_sm + n_base + at.col) * 2;
  const bool f16 = p.d_dtype == KAPY_F16;
  const float rs = p.row_scale ? p.row_scale[m_base + at.row] : 1.0f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint16_t h[4];
    f32x4 cs = {1.0f, 1.0f, 1.0f, 1.0f};
    if (p.row_scale) cs = *(const f32x4 *)(p.col_scale + n_base + at.col + at.qcol * q);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float v = acc[4 * q + e];
      if (p.row_scale) v = __fmul_rn(v, __fmul_rn(rs, cs[e]));
      if (has_tail(p)) v = apply_tail(p, v, p.bias ? load_as_f32(p.bias, p.bias_dtype, n_base + at.col + at.qcol * q + e) : 0.f);
      h[e] = f16 ? f32_to_f16_rn(v) : f32_to_bf16_rn(v);
    }
    u32x2 w = {h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16)};
    *(u32x2 *)(row + 2 * at.qcol * q) = w;
  }
}
// General form: any result type and strides, accumulator input, ragged edges.  Out of line: it is
// large and off the roofline path.
template <int REGS>
__device__ __forceinline__ void store_block_elements(const GemmParams &p, MfmaShape s, int32_t m_base, int32_t n_base, int lane, const float (&acc)[REGS]) {
  const AccLane at = acc_lane(mfma_acc_exchanged(s), s, lane);
  for (int v = 0; v < REGS; ++v)
    store_result(p, m_base + at.row + (v & 3) * at.drow + (v >> 2) * at.qrow, n_base + at.col + (v & 3) * at.dcol + (v >> 2) * at.qcol, acc[v]);
}
__device__ __noinline__ void store_block_generic(const GemmParams &p, int32_t m_base, int32_t n_base, int lane, f32x16 acc) {
  float r[16];
  for (int v = 0; v < 16; ++v) r[v] = acc[v];
  store_block_elements(p, kMfma32x32x16, m_base, n_base, lane, r);
}
__device__ __noinline__ void store_block_generic(const GemmParams &p, int32_t m_base, int32_t n_base, int lane, f32x4 acc) {
  float r[4];
  for (int v = 0; v < 4; ++v) r[v] = acc[v];
  store_block_elements(p, kMfma16x16x32, m_base, n_base, lane, r);
}

// Packed epilogue (16-bit row-major result, 16-byte aligned rows, no accumulator input, RN) of one
// wavefront's WTM x WTN block of KM x KM accumulator blocks, by 32-row strips through a wave-private
// LDS area: accumulator quads (four consecutive columns of one row per lane) are written as fp32,
// read back 32 bytes per lane along rows, narrowed and stored so that one instruction writes whole
// 128-byte lines (64 / (WTN/8) rows x WTN*2 bytes) - the register layout itself would scatter 8-byte
// pieces over KM rows per instruction.  Row stride WTN*4 + 16 bytes: the 16-byte writes down the rows
// then use every LDS bank equally.
// The caller makes sure (barrier) that no other wave still uses the LDS area.
template <int KM, int WTM, int WTN>
struct PackedEpilogue {
  static constexpr int kBytesPerWave = 32 * (WTN * 4 + 16);  // one strip of 32 rows of fp32, rows 16 bytes apart in the banks
  static constexpr int kGroups = 64 / KM, kAccRegs = KM * KM / 64;
  static constexpr int kBlocksPerStrip = 32 / KM, kStrips = WTM / 32, kTn = WTN / KM;
  // the accumulator fragments of a KM x KM block (the operand classes share them): a lane's register quads hold 4
  // consecutive columns of one row, quads kQuadStep columns apart
  static constexpr MfmaShape kBlock{KM, KM, 0, 0};
  static constexpr Fragments kAccLayout = mfma_acc_exchanged(kBlock);
  static constexpr int kQuads = kAccRegs / 4, kQuadStep = kQuads > 1 ? acc_lane(kAccLayout, kBlock, 0).qcol : 0;
  static_assert(quads_run_along_rows(kBlock) && acc_lane_describes(kAccLayout, kBlock) && kAccLayout.loop_size({KM, KM}) == kAccRegs, "accumulator fragments");
  static_assert(WTM % 32 == 0, "strip geometry");

  // EPI: 0 = cast only, 1 = row and column scales.  The strip goes through LDS as fp32: the accumulator registers are
  // written as they are (an LDS store takes them from the accumulator file; narrowing first would cost a register move
  // per element), a lane reads back 8 consecutive columns of a row, scales, narrows and stores 16 bytes.  The stores are
  // buffer stores through a descriptor of the wavefront's part of the result: it ends with the result's last row, so
  // the rows of a tile that hangs over the edge fall out of range in hardware, and a store costs one add.
  // OUT: the result's element type - 0 bf16, 1 f16, 2 f32 (stored as it is: two 16-byte pieces per lane).
  // ACC: an accumulator input added at the end - 0 none, 1 f16, 2 f32 (row-major, rows 16-byte aligned), fetched a strip ahead
  // of its use through a descriptor bounded like the result's.
  template <int OUT, int EPI, int ACC, typename Acc>
  static __device__ __forceinline__ void strips(const GemmParams &p, Acc (&acc)[WTM / KM][WTN / KM], char *strip, int32_t m_wave, int32_t n_wave, int lane) {
    constexpr int kRowStrideF = WTN * 4 + 16, kChunksF = WTN / 8, kRowsPerPass = 64 / kChunksF, kPasses = 32 / kRowsPerPass;
    static_assert(32 * kRowStrideF <= kBytesPerWave && 64 % kChunksF == 0 && 32 % kRowsPerPass == 0, "fp32 strip geometry");
    const AccLane at = acc_lane(kAccLayout, kBlock, lane);
    const int wrow = at.row, wcol = at.col;                      // this lane's row / first column in an accumulator block
    const int rrow = lane / kChunksF, rchunk = lane % kChunksF;  // and in a read-back instruction
    const int32_t nn = n_wave + rchunk * 8;                      // (N a multiple of 8: a piece of 8 columns is in or out whole)
    // The lane's scales - of its 8 columns, of its row in every pass of every strip - are fetched once, up front and together:
    // fetched where they are used, each load would be waited for by itself (the result stores in between might alias
    // them, for all the compiler knows), some hundred exposed cache latencies per wavefront.
    constexpr int kRowsPerLane = EPI == 1 ? kStrips * kPasses : 1;
    float rs_all[kRowsPerLane];
    f32x4 cs_lo = {1.f, 1.f, 1.f, 1.f}, cs_hi = cs_lo;
    if constexpr (EPI == 1) {
      const int32_t nc = min(nn, p.N - 8);
      cs_lo = *(const f32x4 *)(p.col_scale + nc);
      cs_hi = *(const f32x4 *)(p.col_scale + nc + 4);
#pragma unroll
      for (int r = 0; r < kRowsPerLane; ++r)  // (rows past M exist only in tiles that hang over the edge; they are not stored)
        rs_all[r] = p.row_scale[min(m_wave + (r / kPasses) * 32 + (r % kPasses) * kRowsPerPass + rrow, p.M - 1)];
    }
    constexpr uint32_t kOutBytes = OUT == 2 ? 4 : 2;
    const uint32_t pitch = (uint32_t)__builtin_amdgcn_readfirstlane((int)(p.d_sm * kOutBytes));
    const int32_t rows_left = min(WTM, p.M - m_wave), cols_left = min(WTN, p.N - n_wave);
    const uint64_t bv = (uint64_t)(p.d + ((int64_t)m_wave * p.d_sm + n_wave) * kOutBytes);
    const uint32_t base_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)bv), base_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(bv >> 32));
    const int32_t records = (rows_left > 0 && cols_left > 0) ? (int32_t)((uint32_t)(rows_left - 1) * pitch + (uint32_t)cols_left * kOutBytes) : 0;
    const __amdgpu_buffer_rsrc_t d_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)base_hi << 32) | (uint64_t)base_lo), 0, __builtin_amdgcn_readfirstlane(records), 0x00020000);
    // (a lane whose columns lie past N asks for an offset beyond any descriptor)
    const uint32_t voff0 = nn < p.N ? (uint32_t)rrow * pitch + (uint32_t)rchunk * (8u * kOutBytes) : 0x80000000u;
    // the accumulator input, if any: the same geometry in its own element size
    constexpr uint32_t kAccBytes = ACC == 2 ? 4 : 2;
    const uint32_t apitch = ACC ? (uint32_t)__builtin_amdgcn_readfirstlane((int)(p.acc_sm * kAccBytes)) : 0;
    const uint64_t av = ACC ? (uint64_t)(p.acc + ((int64_t)m_wave * p.acc_sm + n_wave) * kAccBytes) : 0;
    const uint32_t abase_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)av), abase_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(av >> 32));
    const int32_t arecords = (ACC && rows_left > 0 && cols_left > 0) ? (int32_t)((uint32_t)(rows_left - 1) * apitch + (uint32_t)cols_left * kAccBytes) : 0;
    const __amdgpu_buffer_rsrc_t a_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)abase_hi << 32) | (uint64_t)abase_lo), 0, __builtin_amdgcn_readfirstlane(arecords), 0x00020000);
    const uint32_t avoff0 = nn < p.N ? (uint32_t)rrow * apitch + (uint32_t)rchunk * (8u * kAccBytes) : 0x80000000u;
    u32x4 acc_in[ACC ? kPasses : 1][ACC == 2 ? 2 : 1];
    // A result too large to be found in the L2s by whoever reads it next is stored non-temporally, so that it does not push
    // the operand panels out of them on its way (bf16 8192^3: + 2 %).
    const bool stream_out = (int64_t)p.M * p.N * kOutBytes >= (int64_t(32) << 20);
    auto store16 = [&](u32x4 w, int voff, int soff) {
      if (stream_out) __builtin_amdgcn_raw_buffer_store_b128(w, d_rsrc, voff, soff, 2);  // (cache policy bit 1: non-temporal)
      else __builtin_amdgcn_raw_buffer_store_b128(w, d_rsrc, voff, soff, 0);
    };
#pragma unroll
    for (int i = 0; i < kStrips; ++i) {
      __builtin_amdgcn_sched_barrier(0);  // keep the strips apart: hoisting accumulator reads costs registers
      if constexpr (ACC != 0) {
#pragma unroll
        for (int t = 0; t < kPasses; ++t) {
          const int avoff = (int)(avoff0 + (uint32_t)(i * 32 + t * kRowsPerPass) * apitch);
          acc_in[t][0] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, avoff, 0, 0);
          if constexpr (ACC == 2) acc_in[t][1] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, avoff, 16, 0);
        }
      }
#pragma unroll
      for (int bi = 0; bi < kBlocksPerStrip; ++bi)
#pragma unroll
        for (int j = 0; j < kTn; ++j)
#pragma unroll
          for (int q = 0; q < kQuads; ++q) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i * kBlocksPerStrip + bi][j][4 * q + e];
            *(f32x4 *)(strip + (bi * KM + wrow) * kRowStrideF + (j * KM + wcol + kQuadStep * q) * 4) = v;
          }
      // LDS executes a wave's instructions in order: the reads below see the writes above, and the next strip's writes
      // come after these reads
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < kPasses; ++t) {
        const int row = t * kRowsPerPass + rrow;
        const f32x4 lo = *(const f32x4 *)(strip + row * kRowStrideF + rchunk * 32), hi = *(const f32x4 *)(strip + row * kRowStrideF + rchunk * 32 + 16);
        float v[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
        if constexpr (EPI == 1) {
          const float rs = rs_all[i * kPasses + t];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = __fmul_rn(v[e], __fmul_rn(rs, cs_lo[e]));
            v[4 + e] = __fmul_rn(v[4 + e], __fmul_rn(rs, cs_hi[e]));
          }
        }
        if constexpr (ACC == 2) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = __fadd_rn(v[e], __uint_as_float(acc_in[t][0][e]));
            v[4 + e] = __fadd_rn(v[4 + e], __uint_as_float(acc_in[t][1][e]));
          }
        } else if constexpr (ACC == 1) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[2 * e] = __fadd_rn(v[2 * e], f16_to_f32((uint16_t)(acc_in[t][0][e] & 0xffffu)));
            v[2 * e + 1] = __fadd_rn(v[2 * e + 1], f16_to_f32((uint16_t)(acc_in[t][0][e] >> 16)));
          }
        }
        const int voff = (int)(voff0 + (uint32_t)(i * 32 + t * kRowsPerPass) * pitch);
        if constexpr (OUT == 2) {
          u32x4 w0, w1;
#pragma unroll
          for (int e = 0; e < 4; ++e) { w0[e] = __float_as_uint(v[e]); w1[e] = __float_as_uint(v[4 + e]); }
          store16(w0, voff, 0);
          store16(w1, voff, 16);  // (the scalar offset is outside the range check: the piece is in or out whole)
        } else {
          u32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = OUT == 1 ? pack2_f16_rn(v[2 * e], v[2 * e + 1]) : pack2_bf16_rn(v[2 * e], v[2 * e + 1]);
          store16(w, voff, 0);
        }
      }
    }
  }
  // The fused elementwise tail.  Its code must not sit in the unrolled accumulator loop (hundreds of copies: the compiler then
  // gives up keeping the accumulators in registers, for the whole kernel), so the strip goes through LDS as fp32 - one strip
  // of 32 x (WTN*4 + 16) bytes fits the two 16-bit strips' space - and a rolled loop applies the tail to 8 consecutive
  // columns per lane on the way out, narrows and stores 16 bytes.
  template <int OUT, typename Acc>
  static __device__ __forceinline__ void strips_tail(const GemmParams &p, Acc (&acc)[WTM / KM][WTN / KM], char *strip, int32_t m_wave, int32_t n_wave, int lane) {
    constexpr int kRowStrideF = WTN * 4 + 16, kChunksF = WTN / 8, kRowsPerPass = 64 / kChunksF, kPasses = 32 / kRowsPerPass;
    static_assert(32 * kRowStrideF <= kBytesPerWave && 64 % kChunksF == 0 && 32 % kRowsPerPass == 0, "fp32 strip geometry");
    const AccLane at = acc_lane(kAccLayout, kBlock, lane);
    const int wrow = at.row, wcol = at.col;
    const int rrow = lane / kChunksF, rchunk = lane % kChunksF;
    const bool stream_out = (int64_t)p.M * p.N * (OUT == 2 ? 4 : 2) >= (int64_t(32) << 20);  // (see strips)
    // the lane's 8 columns are the same in every pass and strip: their bias values are fetched once
    const int32_t nn = n_wave + rchunk * 8;
    float bias[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (p.bias && nn < p.N) {
#pragma unroll
      for (int e = 0; e < 8; ++e) bias[e] = load_as_f32(p.bias, p.bias_dtype, nn + e);
    }
#pragma unroll
    for (int i = 0; i < kStrips; ++i) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int bi = 0; bi < kBlocksPerStrip; ++bi)
#pragma unroll
        for (int j = 0; j < kTn; ++j)
#pragma unroll
          for (int q = 0; q < kQuads; ++q) {
            f32x4 v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i * kBlocksPerStrip + bi][j][4 * q + e];
            *(f32x4 *)(strip + (bi * KM + wrow) * kRowStrideF + (j * KM + wcol + kQuadStep * q) * 4) = v;
          }
      __builtin_amdgcn_sched_barrier(0);  // LDS executes a wave's instructions in order: the reads below see the writes above
#pragma unroll 1
      for (int t = 0; t < kPasses; ++t) {
        const int row = t * kRowsPerPass + rrow;
        const int32_t mm = m_wave + i * 32 + row;
        const f32x4 lo = *(const f32x4 *)(strip + row * kRowStrideF + rchunk * 32), hi = *(const f32x4 *)(strip + row * kRowStrideF + rchunk * 32 + 16);
        float v[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
        apply_tail8(p, v, bias);
        // (N a multiple of 8: a piece of 8 columns is in or out whole)
        if constexpr (OUT == 2) {
          if (mm < p.M && nn < p.N) {
            f32x4 *dst = (f32x4 *)(p.d + ((int64_t)mm * p.d_sm + nn) * 4);
            if (stream_out) {
              __builtin_nontemporal_store(f32x4{v[0], v[1], v[2], v[3]}, dst);
              __builtin_nontemporal_store(f32x4{v[4], v[5], v[6], v[7]}, dst + 1);
            } else {
              dst[0] = f32x4{v[0], v[1], v[2], v[3]};
              dst[1] = f32x4{v[4], v[5], v[6], v[7]};
            }
          }
        } else {
          u32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = OUT == 1 ? pack2_f16_rn(v[2 * e], v[2 * e + 1]) : pack2_bf16_rn(v[2 * e], v[2 * e + 1]);
          if (mm < p.M && nn < p.N) {
            if (stream_out) __builtin_nontemporal_store(w, (u32x4 *)(p.d + ((int64_t)mm * p.d_sm + nn) * 2));
            else *(u32x4 *)(p.d + ((int64_t)mm * p.d_sm + nn) * 2) = w;
          }
        }
      }
    }
  }
  // result type and scaling are uniform: one specialised copy of the loop each, chosen once.  TAIL: the kernel was built for
  // calls with a fused elementwise tail (a build of its own: in one kernel with the plain epilogue the extra live values
  // push the main loop's accumulators out of registers).
  template <bool TAIL = false, typename Acc>
  static __device__ __forceinline__ void run(const GemmParams &p, Acc (&acc)[WTM / KM][WTN / KM], char *strip0, int32_t m_wave, int32_t n_wave, int lane) {
    const int out = p.d_dtype == KAPY_F32 ? 2 : p.d_dtype == KAPY_F16 ? 1 : 0;
    if constexpr (TAIL) {
      if (out == 2) strips_tail<2>(p, acc, strip0, m_wave, n_wave, lane);
      else if (out == 1) strips_tail<1>(p, acc, strip0, m_wave, n_wave, lane);
      else strips_tail<0>(p, acc, strip0, m_wave, n_wave, lane);
    } else if (p.row_scale) {
      if (out == 2) strips<2, 1, 0>(p, acc, strip0, m_wave, n_wave, lane);
      else if (out == 1) strips<1, 1, 0>(p, acc, strip0, m_wave, n_wave, lane);
      else strips<0, 1, 0>(p, acc, strip0, m_wave, n_wave, lane);
    } else if (p.acc_dtype == KAPY_F32) {
      if (out == 2) strips<2, 0, 2>(p, acc, strip0, m_wave, n_wave, lane);
      else if (out == 1) strips<1, 0, 2>(p, acc, strip0, m_wave, n_wave, lane);
      else strips<0, 0, 2>(p, acc, strip0, m_wave, n_wave, lane);
    } else if (p.acc_dtype == KAPY_F16) {
      if (out == 2) strips<2, 0, 1>(p, acc, strip0, m_wave, n_wave, lane);
      else if (out == 1) strips<1, 0, 1>(p, acc, strip0, m_wave, n_wave, lane);
      else strips<0, 0, 1>(p, acc, strip0, m_wave, n_wave, lane);
    } else {
      if (out == 2) strips<2, 0, 0>(p, acc, strip0, m_wave, n_wave, lane);
      else if (out == 1) strips<1, 0, 0>(p, acc, strip0, m_wave, n_wave, lane);
      else strips<0, 0, 0>(p, acc, strip0, m_wave, n_wave, lane);
    }
  }
};

// Workgroup id -> output tile.  Consecutive workgroup ids land on different XCDs (8 of them, each
// with its own L2), so ids are first regrouped per XCD, then each XCD walks a compact band of
// tiles GROUP_M tall so that the operand panels it streams stay in its L2.
__device__ __forceinline__ void tile_of_block(const GemmParams &p, int32_t &tm, int32_t &tn) {
  constexpr int kXcds = 8, kGroupM = 8;
  int32_t total = p.tiles_m * p.tiles_n, id = blockIdx.x;
  if (total % kXcds == 0) id = (id % kXcds) * (total / kXcds) + id / kXcds;
  int32_t per_group = kGroupM * p.tiles_n;
  int32_t g = id / per_group, first_m = g * kGroupM;
  int32_t rows = std::min(p.tiles_m - first_m, kGroupM);
  int32_t in_group = id - g * per_group;
  tm = first_m + in_group % rows;
  tn = in_group / rows;
}

// Split K (GemmParams::split_k): workgroup (tile, blockIdx.y) multiplies the blockIdx.y-th part of K.  Narrows the
// kernel's own copy of the parameters to that part and returns the split index.
__device__ __forceinline__ int32_t enter_split(GemmParams &p, int element_bytes) {
  const int32_t split = blockIdx.y;
  if (p.split_k > 1) {
    const int32_t ks = p.K / p.split_k;  // (the host only splits a K that divides into whole K-tiles per part)
    p.a += (int64_t)split * ks * p.a_sk * element_bytes;
    p.b += (int64_t)split * ks * p.b_sk * element_bytes;
    p.K = ks;
  }
  return split;
}
// The meeting point: every workgroup of a tile leaves its accumulators in the workspace as they sit in registers
// (quad by quad, thread-contiguous: the reader is the same thread of another workgroup, so no layout is involved) and
// counts itself; the one that arrives last gets `true` with `acc` replaced by the sum of all parts IN SPLIT ORDER (the
// result does not depend on which workgroup was last), and sets the counter back to zero for the next call.  Nobody
// waits for anybody.
// The parts are written and read by workgroups on different XCDs, whose L2 caches do not see each other.  A release /
// acquire pair at device scope would make them visible, but costs a write-back and an invalidation of a whole L2 per
// workgroup (measured: 1024^3 took 33 us instead of 16).  Instead every access to the workspace is itself a relaxed
// device-scope access (stores write through, loads do not hit a stale line), each workgroup waits until its stores have
// been acknowledged before it counts itself, and the reader starts loading only after its count has come back.
// Accumulator blocks that lie wholly below the last row of the result (row0 + i * block_rows >= p.M) are not exchanged.
// `lds_word`: 4 bytes of LDS that no wave uses at this point.
template <int THREADS, typename Acc, int TM, int TN>
__device__ __forceinline__ bool split_k_meet(const GemmParams &p, int32_t tile, int32_t split, Acc (&acc)[TM][TN], int32_t row0, int32_t block_rows,
                                             uint32_t *lds_word) {
  constexpr int kHalves = sizeof(Acc) / 8, kPerThread = TM * TN * kHalves;  // 8-byte pieces: the widest relaxed access
  uint64_t *base = (uint64_t *)p.partial + (int64_t)tile * p.split_k * (kPerThread * THREADS) + threadIdx.x;
  uint64_t *mine = base + (int64_t)split * (kPerThread * THREADS);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (row0 + i * block_rows >= p.M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int h = 0; h < kHalves; ++h) {
        const uint64_t v = (uint64_t)__float_as_uint(acc[i][j][2 * h]) | ((uint64_t)__float_as_uint(acc[i][j][2 * h + 1]) << 32);
        __hip_atomic_store(mine + ((i * TN + j) * kHalves + h) * THREADS, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // this lane's stores have been acknowledged
  __syncthreads();                           // ... and every lane's of the workgroup
  if (threadIdx.x == 0) *lds_word = __hip_atomic_fetch_add(p.counters + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const uint32_t arrived_before = *lds_word;
  __syncthreads();  // (the word's LDS may be reused from here on)
  if (arrived_before != (uint32_t)p.split_k - 1) return false;
  // one part at a time, all of its pieces requested before the first is added: a piece-by-piece loop would pay the
  // memory latency once per piece instead of once per part (two parts per round measured no faster and cost 64 more
  // registers, which halves the occupancy of these kernels)
  for (int sp = 0; sp < p.split_k; ++sp) {
    const uint64_t *part = base + (int64_t)sp * (kPerThread * THREADS);
    uint64_t piece[TM][TN][kHalves];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (row0 + i * block_rows >= p.M) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int h = 0; h < kHalves; ++h)
          piece[i][j][h] = __hip_atomic_load(part + ((i * TN + j) * kHalves + h) * THREADS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (row0 + i * block_rows >= p.M) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int h = 0; h < kHalves; ++h) {
          const float a = __uint_as_float((uint32_t)piece[i][j][h]), b = __uint_as_float((uint32_t)(piece[i][j][h] >> 32));
          acc[i][j][2 * h] = sp ? acc[i][j][2 * h] + a : a;
          acc[i][j][2 * h + 1] = sp ? acc[i][j][2 * h + 1] + b : b;
        }
    }
  }
  if (threadIdx.x == 0) __hip_atomic_store(p.counters + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

}  // namespace
}  // namespace kapy
