// matmul.hip — kapy.matmul over whole views on CDNA4 matrix cores (f16 / bf16 operands).
//
// Reference: kapy.matmul (include/kapy/Dialect/Kapy/IR/Ops.td:416-439, verifier
// lib/Dialect/Kapy/IR/Kapy.cpp:451-574) lowered by MatmulOpToLLVM.cpp:58-311 to mma.sync, fed by
// the cp.async ring of CpAsyncOpToLLVM.cpp:22-186 and ldmatrix (LdMatrixOpToLLVM.cpp:21-174);
// the kernel shape is the fixture test/Conversion/KapyToKgpu/matmul.mlir: a 2-stage shared-memory
// ring, fragments prefetched one k-slice ahead, one barrier per wait.
//
// gfx950 counterparts used here:
//   mma.sync m16n8k16          -> v_mfma_f32_32x32x16_{f16,bf16} (fp32 accumulate)
//   cp.async + wait_group      -> global_load_lds_dwordx4 (16 B per lane, written straight into
//                                 LDS) + s_waitcnt vmcnt
//   per-lane swizzled cp.async destination (CpAsyncOpToLLVM.cpp:124-139)
//                              -> the destination of an LDS-direct load is wave-contiguous, so the
//                                 XOR swizzle is applied to WHICH global chunk a lane fetches; the
//                                 LDS image is the same swizzled one
//   ldmatrix                   -> ds_read_b128 of 8 K-contiguous elements per lane
//   swizzle (4,8) for 32 banks -> searched at compile time for 64 banks from the MFMA operand
//                                 layout (layout.hpp first_swizzle)
//
// Two kernels:
//   tn_kernel      both operands contiguous along K (lhs row-major, rhs column-major), extents
//                  multiples of the tile: the roofline path.
//   staged_kernel  any strides, ragged extents: tiles go global -> registers -> LDS, transposing
//                  on the way when an operand is contiguous along M/N.  128x128x32 tiles.
#include <algorithm>
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "layout.hpp"
#include "matmul_params.hpp"
#include "mfma.hpp"
#include "ew_machine.hpp"
#include "numeric.hpp"

// Workspace of a split K for callers that cannot bring one (kapy_matmul_static_workspace): arrival counters, then
// partial sums.  Part of the device image, so every GPU the library runs on holds its own copy until the process ends;
// zero when the image is loaded, and every kernel that uses the counters leaves them zero.  (A launch the runtime refuses has
// not run and leaves them as they were; a kernel that dies on the way takes the process's context with it, array included: there
// is no state in between for the host to repair.)
static __device__ __align__(256) unsigned char scratch[kapy::kSplitCounterBytes + (16 << 20)];

#include "matmul_tile.hpp"

namespace kapy {
namespace {

// ---------------------------------------------------------------------------------------------
// TN kernel.  BM x BN x BK workgroup tile, WM x WN wavefronts, each owning a (BM/WM) x (BN/WN)
// block of 32x32 accumulators.  STAGES-deep LDS ring filled by LDS-direct loads.
constexpr int kRing25 = 25;  // value of STAGES (and of kapy_matmul_cfg.stages) that selects the 2.5-tile ring
template <typename T, int BM, int BN, int BK, int WM, int WN, int STAGES>
struct TnConfig {
  static constexpr int kWaves = WM * WN, kThreads = 64 * kWaves;
  static constexpr int kWtm = BM / WM, kWtn = BN / WN;       // wave tile
  static constexpr int kTm = kWtm / T::kM, kTn = kWtn / T::kM;  // accumulator blocks per wave
  static constexpr int kRowBytes = BK * T::kBytes;
  static constexpr int kRowsPerLoad = 1024 / kRowBytes;      // rows one LDS-direct wave instruction fills
  static constexpr int kLoadsA = BM / kRowsPerLoad, kLoadsB = BN / kRowsPerLoad;
  static constexpr int kLoadsAPerWave = kLoadsA / kWaves, kLoadsBPerWave = kLoadsB / kWaves;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  // STAGES == kRing25: a ring of ten quarter-tile units (half an operand tile each), i.e. 2.5 tiles
  static constexpr int kUnitBytes = kStageBytes / 4;
  static constexpr int kLdsBytes = STAGES == kRing25 ? 10 * kUnitBytes : STAGES * kStageBytes;
  static_assert(kLoadsA % kWaves == 0 && kLoadsB % kWaves == 0, "loads must divide evenly over the wavefronts");
  static_assert(kWtm % 32 == 0 && kWtn % 32 == 0 && BK % T::kSliceK == 0 && 32 % T::kM == 0, "wave tile must be a multiple of the MFMA tile");
};

template <typename T, int BM, int BN, int BK, int WM, int WN, int STAGES, bool PACKED, bool KTAIL = false, bool TAIL = false>
__global__ __launch_bounds__(64 * WM * WN) void tn_kernel(GemmParams p) {
  using C = TnConfig<T, BM, BN, BK, WM, WN, STAGES>;
  using L = TileLayout<C::kRowBytes, T>;
  constexpr int EB = T::kBytes, CH = T::kChunks;
  // Static, so that the size is a property of the code object (160 KiB, a CU's whole LDS, for the 256 x 256 ring) and no
  // launch depends on the runtime honouring a raised dynamic-LDS limit: LDS-direct loads that land outside the allocation fault.
  __shared__ __attribute__((aligned(1024))) char lds[C::kLdsBytes];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave % WM, wn = wave / WM;
  int32_t tm, tn;
  tile_of_block(p, tm, tn);
  const int32_t m0 = tm * BM, n0 = tn * BN;
  // (the 128 x 128 builds, which serve the shapes with few tiles, can split K across workgroups)
  constexpr bool kCanSplit = BM == 128 && BN == 128 && STAGES == kRing25;
  int32_t split = 0;
  if constexpr (kCanSplit) split = enter_split(p, EB);

  // Per-lane global byte offsets of the chunks this lane fetches, one per load instruction.
  // Instruction q of an operand fills LDS bytes [q*1024, q*1024+1024); this lane's 16 bytes sit at
  // q*1024 + lane*16, which the (inverse) swizzle maps back to a (row, chunk) of the tile.
  uint32_t a_goff[C::kLoadsAPerWave], b_goff[C::kLoadsBPerWave];
#pragma unroll
  for (int i = 0; i < C::kLoadsAPerWave; ++i) {
    uint32_t row, chunk;
    L::locate((uint32_t)(wave + i * C::kWaves) * 1024u + lane * 16u, row, chunk);
    // (the 128-wide builds without bounded loads fetch the operand's last row in place of rows past its end: results nobody
    // stores; the 256-wide ones are only given whole tiles)
    if constexpr (STAGES != kRing25 && BM <= 128) row = min(row, (uint32_t)max(p.M - 1 - tm * BM, 0));
    a_goff[i] = (uint32_t)((row * p.a_sm + chunk * (16 / EB)) * EB);
  }
#pragma unroll
  for (int i = 0; i < C::kLoadsBPerWave; ++i) {
    uint32_t row, chunk;
    L::locate((uint32_t)(wave + i * C::kWaves) * 1024u + lane * 16u, row, chunk);
    if constexpr (STAGES != kRing25 && BN <= 128) row = min(row, (uint32_t)max(p.N - 1 - tn * BN, 0));
    b_goff[i] = (uint32_t)((row * p.b_sn + chunk * (16 / EB)) * EB);
  }
  const char *a_tile = p.a + (int64_t)m0 * p.a_sm * EB;
  const char *b_tile = p.b + (int64_t)n0 * p.b_sn * EB;

  // Load instruction `idx` (0 .. loads per tile - 1) of this wavefront for K-tile kt into `stage`.
  auto issue_load = [&](int stage, int kt, int idx) {
    char *sa = lds + stage * C::kStageBytes, *sb = sa + BM * C::kRowBytes;
    if (idx < C::kLoadsAPerWave) {
      const char *ga = a_tile + (int64_t)kt * BK * EB;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(ga + a_goff[idx]),
                                       (__attribute__((address_space(3))) void *)(sa + (wave + idx * C::kWaves) * 1024), 16, 0, 0);
    } else {
      const int i = idx - C::kLoadsAPerWave;
      const char *gb = b_tile + (int64_t)kt * BK * EB;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gb + b_goff[i]),
                                       (__attribute__((address_space(3))) void *)(sb + (wave + i * C::kWaves) * 1024), 16, 0, 0);
    }
  };
  auto issue_loads = [&](int stage, int kt) {
#pragma unroll
    for (int idx = 0; idx < C::kLoadsAPerWave + C::kLoadsBPerWave; ++idx) issue_load(stage, kt, idx);
  };

  // LDS byte offsets of this lane's operand reads, from the operand fragments of the instruction: the lane's
  // row of each KM-row block and, in K slice kk, the 16-byte chunks that hold its kpack consecutive K elements.
  constexpr int KM = T::kM;  // rows per operand block
  static_assert(T::kShape.m == KM && T::kShape.k == T::kSliceK && T::kShape.kpack * EB == 16 * CH, "policy and instruction shape disagree");
  const OperandLane frag_at = operand_lane(T::kShape, lane);
  const uint32_t frag_row = frag_at.row, frag_k0 = frag_at.k0;

  using Acc = typename T::Acc;
  constexpr int kAccRegs = KM * KM / 64;
  Acc acc[C::kTm][C::kTn];
  {
    Acc zero;
#pragma unroll
    for (int v = 0; v < kAccRegs; ++v) zero[v] = 0.f;
#pragma unroll
    for (int i = 0; i < C::kTm; ++i)
#pragma unroll
      for (int j = 0; j < C::kTn; ++j) acc[i][j] = zero;
  }

  const int KT = (p.K + BK - 1) / BK;  // (a partial last tile only in the ring variant)
  constexpr int KK = BK / T::kSliceK;                                   // matrix-instruction K-slices per tile
  constexpr int kLoadsPerTile = C::kLoadsAPerWave + C::kLoadsBPerWave;  // per wavefront
  // A fragment: the CH 16-byte chunks one lane feeds a matrix instruction for one operand block.
  struct Frag {
    u32x4 c[CH];
  };
  // Per-lane LDS offsets of the operand reads of slice kk, relative to the wave's rows of a stage.
  uint32_t frag_off[KK][CH];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk)
#pragma unroll
    for (int c = 0; c < CH; ++c) frag_off[kk][c] = L::offset(frag_row, ((kk * T::kSliceK + frag_k0) * EB) / 16 + c);
  const uint32_t a_rows = (wm * C::kWtm) * C::kRowBytes, b_rows = BM * C::kRowBytes + (wn * C::kWtn) * C::kRowBytes;
  // 32-row blocks are whole multiples of the swizzle period, so block i only adds i*32*rowBytes.
  static_assert((KM * C::kRowBytes) % (256 * L::kLineParam) == 0, "an operand block must span whole swizzle periods");
  // Read `idx` of slice kk (0 .. kReads-1): the first kTm*CH are lhs row blocks, the rest rhs column blocks.
  auto read_frag = [&](int stage, int kk, int idx, Frag *af, Frag *bf) {
    const int blk = idx / CH, c = idx % CH;
    const char *base = lds + stage * C::kStageBytes + frag_off[kk][c];
    if (blk < C::kTm) af[blk].c[c] = *(const u32x4 *)(base + a_rows + blk * KM * C::kRowBytes);
    else bf[blk - C::kTm].c[c] = *(const u32x4 *)(base + b_rows + (blk - C::kTm) * KM * C::kRowBytes);
  };
  auto read_frags = [&](int stage, int kk, Frag *af, Frag *bf) {
#pragma unroll
    for (int idx = 0; idx < (C::kTm + C::kTn) * CH; ++idx) read_frag(stage, kk, idx, af, bf);
  };

  using Yes = std::integral_constant<bool, true>;
  using No = std::integral_constant<bool, false>;
  constexpr int kReads = (C::kTm + C::kTn) * CH, kMfmas = C::kTm * C::kTn;
  constexpr int kReadsPerMfma = (kReads + kMfmas - 1) / kMfmas;  // LDS reads issued behind each matrix instruction

  if constexpr (STAGES == kRing25) {
    // Ring of ten units, a unit being half an operand tile (unit u of tile j: 0/1 = upper/lower half
    // of the lhs rows, 2/3 = left/right half of the rhs columns) at ring position (4j + u) mod 10:
    // all of the 160 KiB of LDS, 2.5 tiles.  A wavefront reads exactly one lhs unit and one rhs unit.
    // There is one barrier per tile, before the tile's last K-slice; it frees the four units of tile
    // kt, and they are refilled in this order: rhs half of tile kt+2 (needed one tile time later),
    // then lhs half of tile kt+3 (needed two tile times later).  That slack lets the loads be spread
    // evenly over the whole tile time - a steady request stream into the L2 instead of every CU
    // bursting at the L1's peak rate right after the barrier - without the last ones running late.
    // Loads for tiles past the end of K are still issued (from the last real tile) into units nobody
    // reads again: every tile step is then identical and the wait counts are constants.
    //
    // The loads are LDS-direct buffer loads: per-lane 32-bit offset (loop invariant) + scalar offset
    // (the K position) + M0 (the LDS destination), so a load costs one scalar and one vector-memory
    // instruction and no vector ALU work.  Ring positions repeat every five tiles; the steady-state
    // loop is unrolled by five so that every LDS address is a constant.
    static_assert(BM == BN && WM == 2 && WN == 2, "the unit ring assumes equal lhs / rhs halves and 2 x 2 wavefronts");
    // A tile step runs in kPhases phases with the barrier before the last one.  Normally a phase is a K-slice (all
    // kTm x kTn blocks with the fragments of that slice, the next slice's fragments fetched meanwhile).  An instruction whose
    // K extent is the whole tile (16x16x128 on 128-byte rows: KK == 1) has 2 x 8 fragment registers per block pair, too many
    // to double-buffer whole; its tile runs as two passes over the halves of the rhs blocks instead: the lhs fragments stay
    // for both passes (double-buffered across tiles), the rhs halves alternate between two buffers.
    constexpr bool kNPass = KK == 1;
    static_assert(kNPass || KK % 2 == 0, "needs an even number of K-slices per tile");
    static_assert(!kNPass || C::kTn % 2 == 0, "two passes over halves of the rhs blocks");
    constexpr int kPhases = kNPass ? 2 : KK, kPhaseMfmas = kNPass ? kMfmas / 2 : kMfmas, kHalfTn = C::kTn / 2;
    constexpr int kUnit = C::kUnitBytes, kHalf = kLoadsPerTile / 2;  // loads per wavefront per operand
    static_assert(C::kLoadsAPerWave == kHalf && C::kLoadsBPerWave == kHalf && kHalf % 2 == 0, "two equal units per operand");
    constexpr int kPerUnit = kHalf / 2;
    constexpr int kEven = (kPhases * kPhaseMfmas) / kLoadsPerTile;
    constexpr int kLoadSpacing = kEven < 1 ? 1 : kEven;
    constexpr int kEarly = kPhaseMfmas / kLoadSpacing < kLoadsPerTile ? kPhaseMfmas / kLoadSpacing : kLoadsPerTile;
    static_assert((kLoadsPerTile - kEarly) * kLoadSpacing <= (kPhases - 1) * kPhaseMfmas, "late loads must go out before the barrier that waits for them");
    // reads and loads in different gaps, where a phase has enough gaps without a load for its reads at one per gap
    constexpr int kFreeGaps = kPhaseMfmas - (kPhaseMfmas + kLoadSpacing - 1) / kLoadSpacing;
    constexpr bool kSpread = kLoadSpacing > 1 && (kNPass ? (kLoadSpacing == kHalfTn && CH <= kHalfTn - 2 && kHalfTn * CH <= kFreeGaps) : kReads <= kFreeGaps);
    // The descriptors must sit in scalar registers (a descriptor in vector registers makes every load
    // a loop over its distinct values): pin the workgroup-uniform tile pointers with readfirstlane.
    auto uniform_ptr = [](const char *ptr) {
      const uint64_t v = (uint64_t)ptr;
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      return (void *)(((uint64_t)hi << 32) | lo);
    };
    // The descriptors end where the operands end: in a tile that hangs over the last row of the lhs (M not a multiple
    // of BM) or of the rhs, the loads of the rows that do not exist are out of range, which the hardware answers with
    // zeros in LDS instead of a fault.  (An operand with 2 GiB or more behind the tile base has all of the tile's rows.)
    auto bytes_left = [&](int32_t rows, int64_t pitch) {
      const int64_t left = rows <= 0 ? 0 : ((int64_t)(rows - 1) * pitch + p.K) * EB;
      return (int)(left < 0x7fffffff ? left : 0x7fffffff);
    };
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(a_tile), 0, __builtin_amdgcn_readfirstlane(bytes_left(p.M - m0, p.a_sm)), 0x00020000);
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(b_tile), 0, __builtin_amdgcn_readfirstlane(bytes_left(p.N - n0, p.b_sn)), 0x00020000);
    const int wave_lds = wave * 1024;
    auto wrap = [](auto pos) { return pos >= 20 ? pos - 20 : (pos >= 10 ? pos - 10 : pos); };
    // ring position `pos` + D, keeping a compile-time position (an integral_constant) a compile-time position
    auto ring_add = [&](auto pos, auto d) {
      if constexpr (std::is_integral_v<decltype(pos)>) return wrap(pos + decltype(d)::value);
      else return std::integral_constant<int, (decltype(pos)::value + decltype(d)::value) % 10>{};
    };
    using Plus2 = std::integral_constant<int, 2>;
    using Plus4 = std::integral_constant<int, 4>;
    using Plus6 = std::integral_constant<int, 6>;
    // K need not be a multiple of BK (only of the 16 bytes of a chunk): the last tile is then partial, and the lanes
    // whose chunk lies past K ask for an offset beyond any descriptor, which the hardware answers with zeros in LDS.
    // Which chunk of a row a lane fetches is the same for every load it issues (the swizzle only mixes in the bit of
    // the load index that is the wavefront's own), so one mask serves all of them.
    const int k_last = (KT - 1) * BK;
    bool lane_past_k;
    {
      uint32_t row, chunk;
      L::locate((uint32_t)wave * 1024u + lane * 16u, row, chunk);
      lane_past_k = k_last + (int)(chunk * (16 / EB)) >= p.K;
    }
    constexpr int kTailFlag = (int)0x80000000;
    // (only the KTAIL build of the kernel pays the select and the mask: they cost 2 % of the aligned case)
    // Two passes: the per-lane offsets of load idx differ from load 0's by idx x (32 rows) only (the swizzle mixes in no bit of
    // the load index beyond the wavefront's own); they are formed at the load from one register per operand - through an
    // opaque add, or the compiler would keep all of them alive again - which leaves the registers to the fragments.
    auto offset_of = [&](const uint32_t(&goff)[kHalf], int idx, uint32_t row_pitch_bytes) -> uint32_t {
      if constexpr (!kNPass) return goff[idx];
      if (idx == 0) return goff[0];
      uint32_t r;
      const uint32_t delta = (uint32_t)idx * 32u * row_pitch_bytes;
      asm volatile("v_add_u32 %0, %1, %2" : "=v"(r) : "v"(goff[0]), "s"(delta));
      return r;
    };
#define KAPY_VOFF(g) ((KTAIL && soff < 0 && lane_past_k) ? kTailFlag : (int)(g))
#define KAPY_SOFF (KTAIL ? (soff & ~kTailFlag) : soff)
    // scalar byte offset of K-tile j in a row, clamped to the last real tile; the sign bit marks a partial tile
    auto k_off = [&](int j) {
      const int jj = min(j, KT - 1);
      return jj * (BK * EB) | ((KTAIL && jj == KT - 1 && k_last + BK > p.K) ? kTailFlag : 0);
    };
    const uint32_t a_pitch_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(p.a_sm * EB)), b_pitch_bytes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(p.b_sn * EB));
    auto load_a = [&](int idx, int pos_of_unit0, int soff) {  // idx: 0 .. kHalf-1, unit idx / kPerUnit
      const int u = idx / kPerUnit, i = idx % kPerUnit;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(lds + wrap(pos_of_unit0 + u) * kUnit + i * C::kWaves * 1024 + wave_lds),
                                               16, KAPY_VOFF(offset_of(a_goff, idx, a_pitch_bytes)), KAPY_SOFF, 0, 0);
    };
    auto load_b = [&](int idx, int pos_of_unit2, int soff) {
      const int u = idx / kPerUnit, i = idx % kPerUnit;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (__attribute__((address_space(3))) void *)(lds + wrap(pos_of_unit2 + u) * kUnit + i * C::kWaves * 1024 + wave_lds),
                                               16, KAPY_VOFF(offset_of(b_goff, idx, b_pitch_bytes)), KAPY_SOFF, 0, 0);
    };
#undef KAPY_VOFF
#undef KAPY_SOFF
    // Load `slot` (0 .. kLoadsPerTile-1) of the sequence issued after the barrier of the tile at ring
    // position pos0: slots [0, kHalf) = rhs units of the tile two ahead (they take positions pos0,
    // pos0+1), the rest = lhs units of the tile three ahead (positions pos0+2, pos0+3).
    auto ring_load = [&](auto pos0, int slot, int soff_b, int soff_a) {
      if (slot < kHalf) load_b(slot, pos0, soff_b);
      else load_a(slot - kHalf, pos0 + 2, soff_a);
    };
    Frag af[kNPass ? 1 : 2][C::kTm], bf[2][kNPass ? kHalfTn : C::kTn];
    // A matrix instruction every 16 (32) clocks leaves the wave 12 (28) clocks to issue anything else before the matrix
    // pipe runs dry, and a vector ALU instruction takes 8 of them, a scalar or LDS or memory instruction 4 to 8.  The
    // steady-state loop therefore computes no address: a read at a compile-time ring position is one of three copies of the
    // lane's fragment offset (the 160 KiB ring seen as 64 KiB windows, the reach of a read's immediate) plus an immediate.
    // (The build for a partial last K-tile has no registers to spare for the copies: it forms the addresses as before.)
    constexpr bool kUseWindows = !KTAIL;
    constexpr int kWindows = kUseWindows ? (C::kLdsBytes + 65535) / 65536 : 1;
    // (a tile's units start at an even ring position, so the wave's own unit - wm for the lhs, wn for the rhs - never
    // wraps on its own and can sit in the register part: one set of copies per operand)
    uint32_t frag_win[2][kWindows][KK][CH];
#pragma unroll
    for (int o = 0; o < 2; ++o)
#pragma unroll
      for (int w = 0; w < kWindows; ++w)
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
          for (int c = 0; c < CH; ++c) {
            uint32_t v = (uint32_t)(uintptr_t)lds + frag_off[kk][c] + (uint32_t)(o ? wn : wm) * kUnit + (uint32_t)w * 65536u;
            asm volatile("" : "+v"(v));  // (opaque: registers that stay, not one register and an add at every read)
            frag_win[o][w][kk][c] = v;
          }
    // The 16 bytes of chunk c, slice kk of operand o (0 lhs, 1 rhs) whose unit 0 starts at ring byte `at`, `rows` bytes in.
    auto read_at = [&](int o, auto at, uint32_t rows, int kk, int c) -> u32x4 {
      if constexpr (std::is_integral_v<decltype(at)>) {
        return *(const u32x4 *)(lds + (at + (o ? wn : wm) * kUnit + frag_off[kk][c]) + rows);
      } else if constexpr (!kUseWindows) {
        return *(const u32x4 *)(lds + (decltype(at)::value + (o ? wn : wm) * kUnit + frag_off[kk][c]) + rows);
      } else {
        const uint32_t v = decltype(at)::value + rows;
        return *(const __attribute__((address_space(3))) u32x4 *)(uintptr_t)(frag_win[o][v >> 16][kk][c] + (v & 65535u));
      }
    };
    // prologue: tiles 0 and 1 whole (lhs units first, then rhs, as the tile steps count them)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int idx = 0; idx < kHalf; ++idx) load_a(idx, 4 * t, k_off(t));
#pragma unroll
      for (int idx = 0; idx < kHalf; ++idx) load_b(idx, 4 * t + 2, k_off(t));
    }
    // ... and the part of the sequence [rhs of tile 1, lhs of tile 2] that a tile step issues in the
    // last slice of the tile before (there is none before tile 0)
    constexpr int kPrologueExtra = kEarly > kHalf ? kEarly - kHalf : 0;
#pragma unroll
    for (int slot = kHalf; slot < kHalf + kPrologueExtra; ++slot) ring_load(6, slot, 0, k_off(2));
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoadsPerTile + kPrologueExtra));
    __builtin_amdgcn_s_barrier();  // tile 0 published
    {
      const uint32_t a0 = wm * kUnit, b0 = (2 + wn) * kUnit;
      // (two passes: the lhs blocks and the first half of the rhs blocks)
#pragma unroll
      for (int idx = 0; idx < (kNPass ? (C::kTm + kHalfTn) * CH : kReads); ++idx) {
        const int blk = idx / CH, c = idx % CH;
        if (blk < C::kTm) af[0][blk].c[c] = *(const u32x4 *)(lds + a0 + frag_off[0][c] + blk * KM * C::kRowBytes);
        else bf[0][blk - C::kTm].c[c] = *(const u32x4 *)(lds + b0 + frag_off[0][c] + (blk - C::kTm) * KM * C::kRowBytes);
      }
    }
    // One tile at ring position `pos` (an int, or an integral_constant in the unrolled loop).  The
    // sequence after the barrier of tile kt-1 is [rhs of tile kt+1, lhs of tile kt+2]; its first
    // kEarly loads went out in the last slice of tile kt-1, the rest go out in the first slices of
    // tile kt.  (`first`: tile 0, where the prologue has issued the rhs part of that sequence.)
    // (`parity`: two passes only - which lhs fragment buffer holds this tile's blocks; it alternates from tile to tile)
    auto tile_step = [&](int kt, auto pos, auto first, auto parity) {
      const auto prev = ring_add(pos, Plus6{});
      const auto next = ring_add(pos, Plus4{});
      // LDS bases of this wave's operand units in this tile and the next one
      // (ring bytes of unit 0 of each operand - compile-time constants in the unrolled loop, see read_at)
      auto unit_base = [&](auto q) {
        if constexpr (std::is_integral_v<decltype(q)>) return (uint32_t)(q * kUnit);
        else return std::integral_constant<uint32_t, (uint32_t)(decltype(q)::value * kUnit)>{};
      };
      const auto a_cur_base = unit_base(pos);
      const auto b_cur_base = unit_base(ring_add(pos, Plus2{}));
      const auto a_nxt_base = unit_base(next);
      const auto b_nxt_base = unit_base(ring_add(pos, Plus6{}));
      const int soff_late_b = k_off(kt + 1), soff_late_a = k_off(kt + 2);   // sequence of tile kt-1
      const int soff_early_b = k_off(kt + 2), soff_early_a = k_off(kt + 3); // sequence of tile kt
      auto ring_read = [&](auto a_base, auto b_base, int kk, int idx, Frag *a_dst, Frag *b_dst) {
        const int blk = idx / CH, c = idx % CH;
        if (blk < C::kTm) a_dst[blk].c[c] = read_at(0, a_base, blk * KM * C::kRowBytes, kk, c);
        else b_dst[blk - C::kTm].c[c] = read_at(1, b_base, (blk - C::kTm) * KM * C::kRowBytes, kk, c);
      };
      if constexpr (kNPass) {
        (void)parity;
        Frag *a_cur = af[0];  // one buffer: a block is fetched again (for the next tile) right behind its last use in pass 1
#pragma unroll
        for (int ph = 0; ph < 2; ++ph) {
          Frag *b_cur = bf[ph];  // pass 0: rhs blocks 0 .. kHalfTn-1, pass 1: the others
          if (ph == 1) {
            // tile kt+1 has landed once only the kHalf youngest loads (lhs of tile kt+2) are in flight; this wave's reads
            // of tile kt (the last ones went out in pass 0) have returned
            __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(kHalf));
            __builtin_amdgcn_s_barrier();
          }
#pragma unroll
          for (int g = 0; g < kPhaseMfmas; ++g) {
            const int i = g / kHalfTn, j = g % kHalfTn;  // lhs-block major: block i is used kHalfTn times in a row, then rests
            T::mfma_in_place(b_cur[j].c, a_cur[i].c, acc[i][ph * kHalfTn + j]);
            if (g % kLoadSpacing != 0) __builtin_amdgcn_sched_barrier(0);  // (a load's M0 write may move ahead of the matrix instruction)
            // (a read never shares the gap behind a matrix instruction with a load: the two together, with the scalar
            // instructions a load brings, outlast the instruction, and the matrix pipe would wait for the next one)
            if (ph == 0) {  // the second half of this tile's rhs blocks, in the first gaps that carry no load
              const int r = kSpread ? (g % kLoadSpacing ? g - 1 - g / kLoadSpacing : -1) : g;
              const int blk = r / CH, c = r % CH;
              if (r >= 0 && blk < kHalfTn) bf[1][blk].c[c] = read_at(1, b_cur_base, (kHalfTn + blk) * KM * C::kRowBytes, 0, c);
            } else {
              // the next tile: lhs block i into the registers its last use has just left ...
              const int jb = kSpread ? j - 1 : j;  // (loads go out behind j == 0 when kSpread)
              if (j == kHalfTn - 1) {
#pragma unroll
                for (int c = 0; c < CH; ++c) a_cur[i].c[c] = read_at(0, a_nxt_base, i * KM * C::kRowBytes, 0, c);
              } else if (kSpread && i < kHalfTn && jb >= 0 && jb < CH) {
                // ... and the first half of its rhs blocks (block i, chunk jb) into the buffer pass 0 has left
                bf[0][i].c[jb] = read_at(1, b_nxt_base, i * KM * C::kRowBytes, 0, jb);
              } else if (!kSpread && i * (kHalfTn - 1) + j < kHalfTn * CH) {
                // (without the spread placement: the same reads, one in each gap that refills no lhs block, in order)
                const int q = i * (kHalfTn - 1) + j;
                bf[0][q / CH].c[q % CH] = read_at(1, b_nxt_base, (q / CH) * KM * C::kRowBytes, 0, q % CH);
              }
            }
            if (g % kLoadSpacing == 0) {
              const int slot = (ph * kPhaseMfmas + g) / kLoadSpacing;
              if (ph == 1 && g / kLoadSpacing < kEarly) ring_load(pos, g / kLoadSpacing, soff_early_b, soff_early_a);
              if (ph == 0 && kEarly + slot < kLoadsPerTile && (!first.value || kEarly + slot >= kHalf))
                ring_load(prev, kEarly + slot, soff_late_b, soff_late_a);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        return;
      }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        Frag *a_cur = af[kk & 1], *b_cur = bf[kk & 1], *a_nxt = af[(kk + 1) & 1], *b_nxt = bf[(kk + 1) & 1];
        if (kk == KK - 1) {
          // tile kt+1 has landed once only the kHalf youngest loads (lhs of tile kt+2) are in flight
          __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(kHalf));
          __builtin_amdgcn_s_barrier();
        } else if constexpr (!KTAIL) {
          // this slice's fragments, asked for during the previous slice, have long returned: one wait here, which never
          // waits, instead of the compiler's own wait in each of the first gaps, where it costs the gap a third of its slots
          __builtin_amdgcn_s_waitcnt(0xC07F);
        }
#pragma unroll
        for (int g = 0; g < kMfmas; ++g) {
          const int i = g / C::kTn, j = g % C::kTn;
          acc[i][j] = T::mfma(b_cur[j].c, a_cur[i].c, acc[i][j]);
          if (KTAIL || g % kLoadSpacing != 0) __builtin_amdgcn_sched_barrier(0);  // (a load's M0 write may move ahead of the matrix instruction)
#pragma unroll
          for (int t = 0; t < kReadsPerMfma; ++t) {
            // (kSpread: one read per gap, and none in the gaps that carry a load - see the two-pass step)
            const int idx = kSpread ? (g % kLoadSpacing ? g - 1 - g / kLoadSpacing : -1) : g * kReadsPerMfma + t;
            if (idx >= 0 && idx < kReads) {
              if (kk + 1 < KK) ring_read(a_cur_base, b_cur_base, kk + 1, idx, a_nxt, b_nxt);
              else ring_read(a_nxt_base, b_nxt_base, 0, idx, a_nxt, b_nxt);
            }
          }
          if (g % kLoadSpacing == 0) {
            const int slot = (kk * kMfmas + g) / kLoadSpacing;
            if (kk == KK - 1 && g / kLoadSpacing < kEarly) ring_load(pos, g / kLoadSpacing, soff_early_b, soff_early_a);
            if (kk < KK - 1 && kEarly + slot < kLoadsPerTile && (!first.value || kEarly + slot >= kHalf))
              ring_load(prev, kEarly + slot, soff_late_b, soff_late_a);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    tile_step(0, std::integral_constant<int, 0>{}, Yes{}, Even{});
    int kt = 1;
    for (; kt + 5 <= KT; kt += 5) {
      tile_step(kt, std::integral_constant<int, 4>{}, No{}, Even{});
      tile_step(kt + 1, std::integral_constant<int, 8>{}, No{}, Even{});
      tile_step(kt + 2, std::integral_constant<int, 2>{}, No{}, Even{});
      tile_step(kt + 3, std::integral_constant<int, 6>{}, No{}, Even{});
      tile_step(kt + 4, std::integral_constant<int, 0>{}, No{}, Even{});
    }
    for (int pos = 4; kt < KT; ++kt) {
      tile_step(kt, pos, No{}, Even{});
      pos = wrap(pos + 4);
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // loads issued for tiles past the end still target this workgroup's LDS
    if constexpr (kNPass) {
      // the in-place matrix instructions are opaque to the compiler, which therefore does not count the wait states their
      // results need before another kind of instruction may read the accumulators (up to 19 for this instruction)
      asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    }
  } else if constexpr (STAGES == 2) {
    // Two stages (the ring depth of the reference fixture, matmul.mlir:19-22).  The one barrier per
    // tile sits BEFORE the tile's last K-slice: by then every wave has fetched the fragments of that
    // last slice, so the stage is free to be refilled, and the next tile is waited for and published.
    // The last slice's matrix instructions then cover the first fragment reads of the next tile.
    //
    // Pacing of the LDS-direct loads: the CU's texture path moves 64 bytes per clock, i.e. one 1 KiB
    // wave-load per 16 clocks, 64 clocks for one load from each of the 4 waves - two matrix
    // instructions.  Issued any faster the loads back up, a wave blocks at the load instruction and
    // its matrix pipe starves.  So one load goes behind every kLoadSpacing-th matrix instruction:
    // the first ones (tile kt+2) in the last slice of tile kt, right after the barrier, the rest in
    // the first slices of tile kt+1.
    static_assert(KK >= 2 && KK % 2 == 0, "needs an even number of K-slices per tile");
    // (narrower tiles have fewer matrix instructions per load: they fall back to a denser spacing)
    constexpr int kWanted = 64 / T::kMfmaClocks, kFit = ((KK - 1) * kMfmas) / kLoadsPerTile;
    constexpr int kLoadSpacing = kFit < 1 ? 1 : (kFit < kWanted ? kFit : kWanted);
    constexpr int kEarly = kMfmas / kLoadSpacing < kLoadsPerTile ? kMfmas / kLoadSpacing : kLoadsPerTile;  // issued in the last slice
    static_assert((kLoadsPerTile - kEarly) * kLoadSpacing <= (KK - 1) * kMfmas, "late loads must go out before the barrier that waits for them");
    Frag af[2][C::kTm], bf[2][C::kTn];
    issue_loads(0, 0);
    if (KT > 1) {
      issue_loads(1, 1);
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoadsPerTile));
    } else {
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    }
    __builtin_amdgcn_s_barrier();  // tile 0 published
    read_frags(0, 0, af[0], bf[0]);
    // has_next: tile kt+1 exists.  early: tile kt+2 exists (its first loads go out in the last slice).
    // late: the remaining loads of tile kt+1 are still to be issued (false for tile 1: the prologue did).
    auto tile_step = [&](int kt, auto has_next, auto early, auto late) {
      const int stage = kt & 1;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        Frag *a_cur = af[kk & 1], *b_cur = bf[kk & 1], *a_nxt = af[(kk + 1) & 1], *b_nxt = bf[(kk + 1) & 1];
        if (kk == KK - 1) {
          if constexpr (has_next.value) {
            __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));  // own loads of tile kt+1 landed; own reads of this stage returned
            __builtin_amdgcn_s_barrier();
          }
        }
#pragma unroll
        for (int g = 0; g < kMfmas; ++g) {
          const int i = g / C::kTn, j = g % C::kTn;
          acc[i][j] = T::mfma(b_cur[j].c, a_cur[i].c, acc[i][j]);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int t = 0; t < kReadsPerMfma; ++t) {
            const int idx = g * kReadsPerMfma + t;
            if (idx < kReads) {
              if (kk + 1 < KK) read_frag(stage, kk + 1, idx, a_nxt, b_nxt);
              else if constexpr (has_next.value) read_frag(stage ^ 1, 0, idx, a_nxt, b_nxt);
            }
          }
          if (g % kLoadSpacing == 0) {
            const int slot = (kk * kMfmas + g) / kLoadSpacing;  // load slots counted from the start of the tile
            if constexpr (early.value)
              if (kk == KK - 1 && g / kLoadSpacing < kEarly) issue_load(stage, kt + 2, g / kLoadSpacing);
            if constexpr (late.value)
              if (kk < KK - 1 && kEarly + slot < kLoadsPerTile) issue_load(stage ^ 1, kt + 1, kEarly + slot);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    if (KT == 1) {
      tile_step(0, No{}, No{}, No{});
    } else {
      if (KT > 2) tile_step(0, Yes{}, Yes{}, No{});
      else tile_step(0, Yes{}, No{}, No{});
      int kt = 1;
      for (; kt + 2 < KT; ++kt) tile_step(kt, Yes{}, Yes{}, Yes{});
      if (KT > 2) tile_step(KT - 2, Yes{}, No{}, Yes{});
      tile_step(KT - 1, No{}, No{}, No{});
    }
  } else {
    // Three or more stages: the barrier at the top of iteration kt publishes tile kt+1, so the
    // fragments of the next K-slice are always fetched one slice ahead, across tile boundaries
    // (the register double-buffering of the reference fixture, matmul.mlir:51-91).
    static_assert(KK % 2 == 0, "fragment double-buffering needs an even number of K-slices per tile");
    Frag af[2][C::kTm], bf[2][C::kTn];
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
      if (s < KT) issue_loads(s, s);
    if (KT > STAGES - 2) __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoadsPerTile * (STAGES - 2)));
    else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __builtin_amdgcn_s_barrier();  // tile 0 published
    read_frags(0, 0, af[0], bf[0]);
    int stage = 0;  // stage of tile kt
    // One tile.  HAS_NEXT: tile kt+1 exists (publish it, prefetch its first fragments).
    // LOADS: tile kt+STAGES-1 exists (request it).  The flags are compile-time so that the
    // steady-state body is branch-free and the scheduler can interleave LDS reads with MFMAs.
    auto tile_step = [&](int kt, auto has_next, auto loads) {
      const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
      if constexpr (has_next.value) {
        // own loads of tile kt+1 have landed once only the younger tiles' loads remain in flight
        if constexpr (loads.value) __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(kLoadsPerTile * (STAGES - 3)));
        else __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));
        __builtin_amdgcn_s_barrier();  // tile kt+1 published; every wave has left tile kt-1
      }
      // Source order is issue order (sched_barrier pins it): behind each of the first matrix
      // instructions of a slice goes one LDS read of the next slice's fragments and, in the first
      // slice, one LDS-direct global load, so reads have the rest of the slice to land.
      static_assert(KK * kMfmas >= kLoadsPerTile, "not enough matrix instructions per tile to pace the global loads");
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) {
        Frag *a_cur = af[kk & 1], *b_cur = bf[kk & 1], *a_nxt = af[(kk + 1) & 1], *b_nxt = bf[(kk + 1) & 1];
#pragma unroll
        for (int g = 0; g < kMfmas; ++g) {
          const int i = g / C::kTn, j = g % C::kTn;
          acc[i][j] = T::mfma(b_cur[j].c, a_cur[i].c, acc[i][j]);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int t = 0; t < kReadsPerMfma; ++t) {
            const int idx = g * kReadsPerMfma + t;
            if (idx < kReads) {
              if (kk + 1 < KK) read_frag(stage, kk + 1, idx, a_nxt, b_nxt);
              else if constexpr (has_next.value) read_frag(next_stage, 0, idx, a_nxt, b_nxt);
            }
          }
          // the tile's LDS-direct loads are spread one per matrix instruction over the whole tile
          if constexpr (has_next.value && loads.value)
            if (kk * kMfmas + g < kLoadsPerTile) issue_load(stage == 0 ? STAGES - 1 : stage - 1, kt + STAGES - 1, kk * kMfmas + g);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      stage = next_stage;
    };
    int kt = 0;
    for (; kt + STAGES - 1 < KT; ++kt) tile_step(kt, Yes{}, Yes{});
    for (; kt + 1 < KT; ++kt) tile_step(kt, Yes{}, No{});
    tile_step(kt, No{}, No{});
  }

  if constexpr (kCanSplit) {
    if (p.split_k > 1) {
      __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));
      __builtin_amdgcn_s_barrier();  // every wave has left the ring
      if (!split_k_meet<C::kThreads>(p, tm + tn * p.tiles_m, split, acc, m0 + wm * C::kWtm, KM, (uint32_t *)lds)) return;
    }
  }
  if constexpr (PACKED) {
    static_assert(PackedEpilogue<KM, C::kWtm, C::kWtn>::kBytesPerWave * C::kWaves <= C::kLdsBytes, "two strips per wavefront must fit the ring");
    __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));
    __builtin_amdgcn_s_barrier();  // every wave has left the ring: it is reused as staging space
    PackedEpilogue<KM, C::kWtm, C::kWtn>::template run<TAIL>(p, acc, lds + wave * PackedEpilogue<KM, C::kWtm, C::kWtn>::kBytesPerWave, m0 + wm * C::kWtm,
                                              n0 + wn * C::kWtn, lane);
  } else {
#pragma unroll
    for (int i = 0; i < C::kTm; ++i)
#pragma unroll
      for (int j = 0; j < C::kTn; ++j) store_block_generic(p, m0 + wm * C::kWtm + i * KM, n0 + wn * C::kWtn + j * KM, lane, acc[i][j]);
  }
}

// ---------------------------------------------------------------------------------------------
// NN kernel: lhs row-major (K contiguous), rhs row-major (N contiguous), extents multiples of the
// 128 x 128 x BK tile.  4 wavefronts (2x2), wave tile 64x64 = 4x4 blocks of the 16x16x32 instruction.
// The rhs tile is staged as it lies in memory, [BK][128] with N contiguous, by the same LDS-direct
// buffer loads as the lhs; the K-contiguous operand registers the matrix instruction wants are made
// on the way out of LDS by ds_read_b64_tr_b16: a 16-lane group hands in 16 addresses of 8 bytes
// (4 k-rows x 16 columns) and lane i gets column i of the four rows.  This replaces the
// ldmatrix.trans of the reference (LdMatrixOpToLLVM.cpp:128-129).
// STAGES-deep ring; the barrier at the top of iteration kt publishes tile kt+1 and frees the stage of
// tile kt-1 for the loads of tile kt+STAGES-1.  Loads past the end of K re-read the last tile into
// a stage nobody reads again, so every iteration is identical.
constexpr int kNBM = 128, kNBN = 128;
// rhs image: 16-byte chunk c of k-row r sits at chunk c ^ rhs_key(r).  A transposing read of a half
// wave touches rows {0..3} + 8*{0,1} (+4) of a 32-row slice, 32 bytes of each: the key sends those
// eight to the eight 32-byte bank groups of the 256-byte row.
__device__ __forceinline__ uint32_t rhs_key(uint32_t row) { return ((row & 3) + 4 * ((row >> 3) & 1)) * 2; }

// A_TR / B_TR: how each operand lies in memory and in LDS.  false: K-contiguous (a row-major lhs, a column-major rhs): rows
// of BK elements staged under the tiled kernel's swizzle and read 16 bytes per lane.  true: contiguous along its other
// extent (a column-major lhs, a row-major rhs): k-rows of 128 elements staged as they lie and read with the transposing
// read.  <false, true> is the reference fixture's row-major x row-major; <false, false> is the tiled kernel's business.
// KTAIL: K is a multiple of 8 but not of BK.  The loads of the last K-tile are then issued with the per-lane offsets of the
// 16-byte pieces (K-contiguous operand) or k-rows (transposed operand) beyond K moved out of the descriptor's range, so that
// zeros arrive in their place; the switch is made once, beside a barrier, when the last tile's loads come up.
template <typename T, int BK, int STAGES, bool PACKED, bool A_TR = false, bool B_TR = true, bool KTAIL = false>
__global__ __launch_bounds__(256) void nn_kernel(GemmParams p) {
  static_assert(T::kM == 16 && T::kBytes == 2 && BK % 32 == 0 && STAGES >= 3, "16x16x32 instruction, 16-bit operands");
  static_assert(A_TR || B_TR, "two K-contiguous operands are the tiled kernel's");
  using LA = TileLayout<BK * 2, T, 16>;
  constexpr int kRowKc = BK * 2, kRowTr = 128 * 2;   // bytes per staged row: a row / column of BK elements, or a k-row of 128
  constexpr int kBytesOp = 128 * BK * 2, kBytesA = kBytesOp, kStage = 2 * kBytesOp;
  constexpr int kLoadsOp = kBytesOp / 1024 / 4, kLoads = 2 * kLoadsOp;  // per wavefront per tile
  constexpr int KK = BK / 32, kTm = 4, kTn = 4, kMfmas = kTm * kTn;
  static_assert(kNBM == 128 && kNBN == 128, "both operands stage 128 rows, columns or elements per k-row");
  __shared__ __attribute__((aligned(1024))) char lds[STAGES * kStage];  // static: see tn_kernel
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  int32_t tm, tn;
  tile_of_block(p, tm, tn);
  const int32_t m0 = tm * kNBM, n0 = tn * kNBN;
  const int32_t split = enter_split(p, 2);
  // (a scalar: in the builds whose epilogue calls the element store out of line the parameters live in scratch memory, and a
  // count read back from there would make every branch on it a vector compare)
  const int KT = __builtin_amdgcn_readfirstlane(KTAIL ? (p.K + BK - 1) / BK : p.K / BK);
  // elements between neighbours along the staged rows' other extent: between rows (K-contiguous) or between k-rows (transposed)
  const int32_t a_ld = (int32_t)(A_TR ? p.a_sk : p.a_sm), b_ld = (int32_t)(B_TR ? p.b_sk : p.b_sn);

  // Per-lane global byte offsets of the 16-byte chunks this lane fetches, one per load instruction (instruction q of an operand
  // fills LDS bytes [q*1024, q*1024 + 1024) of its image).
  auto goff_of = [&](bool tr, int q, int32_t ld) -> uint32_t {
    const uint32_t o = (uint32_t)(wave + q * 4) * 1024u + lane * 16u;
    uint32_t row, chunk;
    if (tr) {
      row = o / kRowTr;
      chunk = ((o % kRowTr) / 16) ^ rhs_key(row);
    } else {
      LA::locate(o, row, chunk);
    }
    return (uint32_t)((row * ld + chunk * 8) * 2);
  };
  uint32_t a_goff[kLoadsOp], b_goff[kLoadsOp];
#pragma unroll
  for (int q = 0; q < kLoadsOp; ++q) {
    a_goff[q] = goff_of(A_TR, q, a_ld);
    b_goff[q] = goff_of(B_TR, q, b_ld);
  }
  // (KTAIL) first K position, within a tile, of the piece that load instruction q of an operand brings this lane
  auto k_of = [&](bool tr, int q) -> int32_t {
    const uint32_t o = (uint32_t)(wave + q * 4) * 1024u + lane * 16u;
    uint32_t row, chunk;
    if (tr) return (int32_t)(o / kRowTr);
    LA::locate(o, row, chunk);
    return (int32_t)chunk * 8;
  };
  // From the last K-tile on (the loads past the end of K repeat it): pieces at or beyond K get an offset no descriptor covers.
  auto enter_k_tail = [&]() __attribute__((always_inline)) {
    const int32_t k_left = p.K - (KT - 1) * BK;
#pragma unroll
    for (int q = 0; q < kLoadsOp; ++q) {
      a_goff[q] = k_of(A_TR, q) >= k_left ? 0x7fffffffu : a_goff[q];
      b_goff[q] = k_of(B_TR, q) >= k_left ? 0x7fffffffu : b_goff[q];
    }
  };
  auto uniform_ptr = [](const char *ptr) {
    const uint64_t v = (uint64_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (void *)(((uint64_t)hi << 32) | lo);
  };
  // The lhs descriptor ends where the lhs ends: a tile of a K-contiguous lhs that hangs over its last rows (M not a multiple of
  // 128) gets zeros for the rows that do not exist (their per-lane offsets are out of range) instead of a fault.  (For a
  // transposed lhs the host asks for whole tiles of rows; its descriptor is bounded all the same.)
  const int64_t a_left = A_TR ? ((int64_t)(p.K - 1) * p.a_sk + (p.M - m0)) * 2 : ((int64_t)(p.M - m0 - 1) * p.a_sm + p.K) * 2;
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.a + (int64_t)m0 * (A_TR ? 1 : p.a_sm) * 2), 0,
                                                                          __builtin_amdgcn_readfirstlane((int)(a_left < 0x7fffffff ? a_left : 0x7fffffff)), 0x00020000);
  // The rhs descriptor ends where the rhs ends, too: of a tile that hangs over the last columns (N not a multiple of 128) the
  // columns that do not exist read zeros or, in a transposed rhs, the first elements of the next k-row; either way they only
  // reach results that are not stored.
  const int64_t b_left = B_TR ? ((int64_t)(p.K - 1) * p.b_sk + (p.N - n0)) * 2 : ((int64_t)(p.N - n0 - 1) * p.b_sn + p.K) * 2;
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.b + (int64_t)n0 * (B_TR ? 1 : p.b_sn) * 2), 0,
                                                                          __builtin_amdgcn_readfirstlane((int)(b_left < 0x7fffffff ? b_left : 0x7fffffff)), 0x00020000);
  const int wave_lds = wave * 1024;
  // (the scalar offsets of K-tile j, clamped to the last tile: loads past the end of K are still issued, into stages nobody reads)
  auto soff_a_of = [&](int j) { return min(j, KT - 1) * BK * (A_TR ? a_ld : 1) * 2; };
  auto soff_b_of = [&](int j) { return min(j, KT - 1) * BK * (B_TR ? b_ld : 1) * 2; };
  auto issue_load_at = [&](int soff_a, int soff_b, int stage, int idx) __attribute__((always_inline)) {
    if (idx < kLoadsOp)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(lds + stage * kStage + idx * 4096 + wave_lds), 16,
                                               (int)a_goff[idx], soff_a, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (__attribute__((address_space(3))) void *)(lds + stage * kStage + kBytesA + (idx - kLoadsOp) * 4096 + wave_lds),
                                               16, (int)b_goff[idx - kLoadsOp], soff_b, 0, 0);
  };
  auto issue_load = [&](int j, int stage, int idx) __attribute__((always_inline)) { issue_load_at(soff_a_of(j), soff_b_of(j), stage, idx); };

  // Operand reads, from the operand fragments of the instruction (l16: the lane's row of an lhs block = its column of
  // an rhs block; grp: which 8 of a slice's 32 K positions its registers hold).  K-contiguous operand: row / column l16 of each
  // 16-wide block, 16-byte chunk 4*kk + grp.  Transposed operand: the transposing read hands lane j of a 16-lane group element j
  // of the four k-rows whose 8-byte pieces the group's lanes address, so lane l16 addresses k-row (8*grp + 4*h + l16/4),
  // elements 4*(l16%4).. of the block.
  const OperandLane frag_at = operand_lane(T::kShape, lane);
  const uint32_t grp = frag_at.k0 / T::kShape.kpack, l16 = frag_at.row;
  static_assert((16 * kRowKc) % (256 * LA::kLineParam) == 0, "an operand block must span whole swizzle periods");
  const uint32_t tr_row = 8 * grp + (l16 >> 2), tr_key = rhs_key(tr_row);  // the key is the same for every kk and h
  // Byte offset, inside an operand's image of a stage, of this lane's read for block `blk` (transposed) or slice kk (K-contiguous)
  // of the wave's half `w` of the operand.
  auto tr_off = [&](int w, int blk) { return tr_row * kRowTr + (((w * 8 + blk * 2 + ((l16 & 3) >> 1)) ^ tr_key) * 16) + (l16 & 1) * 8; };
  auto kc_off = [&](int w, int kk) { return LA::offset(w * 64 + l16, 4 * kk + grp); };
  // a transposed operand's fragment comes out of LDS as two 8-byte halves (k-rows +0..3 and +4..7 of the lane's K-group)
  // (kept as two arrays of halves per fragment buffer, the form the wait for these reads takes its operands in)
  struct Frags {
    u32x4 c[4];               // K-contiguous operand: one 16-byte read per block
    u32x2_lds h0[4], h1[4];   // transposed operand
  };
  static_assert(kTm == 4 && kTn == 4, "tr_reads_wait takes the halves of four fragments");
  // Every operand read of the main loop is `register + immediate`: the stage is a compile-time constant there (the loop is
  // unrolled over the ring), and where the ring is longer than a read's 64 KiB immediate reaches, the per-lane offsets
  // are kept once per 64 KiB window (a vector add per read would cost the matrix pipe more than the read itself).
  constexpr int kWindows = (STAGES * kStage + 65535) / 65536;
  constexpr int kRegsA = A_TR ? kTm : KK, kRegsB = B_TR ? kTn : KK;
  uint32_t a_win[kWindows][kRegsA], b_win[kWindows][kRegsB];
#pragma unroll
  for (int w = 0; w < kWindows; ++w) {
#pragma unroll
    for (int x = 0; x < kRegsA; ++x) {
      uint32_t v = (uint32_t)(uintptr_t)lds + (A_TR ? tr_off(wm, x) : kc_off(wm, x)) + (uint32_t)w * 65536u;
      asm volatile("" : "+v"(v));  // (opaque: registers that stay, not one register and an add at every read)
      a_win[w][x] = v;
    }
#pragma unroll
    for (int x = 0; x < kRegsB; ++x) {
      uint32_t v = (uint32_t)(uintptr_t)lds + kBytesA + (B_TR ? tr_off(wn, x) : kc_off(wn, x)) + (uint32_t)w * 65536u;
      asm volatile("" : "+v"(v));
      b_win[w][x] = v;
    }
  }
  // read `r` (0 .. 3) of slice kk of the stage: block r of the operand
  auto read_op = [&](auto is_b, auto stage, auto kk, auto blk, Frags &dst) __attribute__((always_inline)) {
    constexpr bool kIsB = decltype(is_b)::value, kTr = kIsB ? B_TR : A_TR;
    constexpr int b = decltype(blk)::value;
    auto win = [&](uint32_t w, int x) { if constexpr (kIsB) return b_win[w][x]; else return a_win[w][x]; };
    if constexpr (kTr) {
      constexpr uint32_t c0 = decltype(stage)::value * kStage + decltype(kk)::value * 32 * kRowTr, c1 = c0 + 4 * kRowTr;
      dst.h0[b] = tr_read_b64_at<(c0 & 65535u)>(win(c0 >> 16, b));
      dst.h1[b] = tr_read_b64_at<(c1 & 65535u)>(win(c1 >> 16, b));
    } else {
      constexpr uint32_t c = decltype(stage)::value * kStage + (uint32_t)b * 16 * kRowKc;
      dst.c[b] = *(const __attribute__((address_space(3))) u32x4 *)(uintptr_t)(win(c >> 16, decltype(kk)::value) + (c & 65535u));
    }
  };
  using IsA = std::integral_constant<bool, false>;
  using IsB = std::integral_constant<bool, true>;
  auto operand_of = [](auto tr, const Frags &f, int b) __attribute__((always_inline)) -> u32x4 {
    if constexpr (decltype(tr)::value) return u32x4{f.h0[b][0], f.h0[b][1], f.h1[b][0], f.h1[b][1]};
    else return f.c[b];
  };
  using ATr = std::integral_constant<bool, A_TR>;
  using BTr = std::integral_constant<bool, B_TR>;

  using Acc = typename T::Acc;
  Acc acc[kTm][kTn];
#pragma unroll
  for (int i = 0; i < kTm; ++i)
#pragma unroll
    for (int j = 0; j < kTn; ++j) acc[i][j] = Acc{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int j = 0; j < STAGES - 1; ++j) {
    if (KTAIL && j == KT - 1) enter_k_tail();
#pragma unroll
    for (int idx = 0; idx < kLoads; ++idx) issue_load(j, j, idx);
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(kLoads * (STAGES - 2)));
  __builtin_amdgcn_s_barrier();  // tile 0 published
  Frags af[2], bf[2];
  using Zero = std::integral_constant<int, 0>;
  static_for<kTm>([&](auto i) { read_op(IsA{}, Zero{}, Zero{}, i, af[0]); });
  static_for<kTn>([&](auto j) { read_op(IsB{}, Zero{}, Zero{}, j, bf[0]); });

  constexpr int kReads = kTm + kTn;
  constexpr int kLoadSpacing = (KK * kMfmas) / kLoads;  // matrix instructions between two loads
  static_assert(kLoadSpacing >= 2 && kReads <= kMfmas - (kMfmas + kLoadSpacing - 1) / kLoadSpacing, "a slice has a gap without a load for each of its reads");
  // (Every lambda that touches the fragment buffers is always_inline.  Left to its cost model the compiler once kept tile_step
  // out of line in one build - both operands transposed, 64-deep, partial last K-tile - and the buffers it captures by
  // reference then live in scratch memory: registers with a transposing read still pending were stored there before their
  // data had arrived, and the products were wrong.)
  // One K-tile in ring stage STAGE (a type: every LDS address of the step is then a constant).  `parity` says which
  // fragment buffer holds slice 0 of this tile: with an odd number of slices per tile it alternates from tile to tile.
  // What goes behind which matrix instruction follows the tiled kernel's rule: a read never shares a gap with a load,
  // and a load's gap is left to the scheduler, which moves the M0 write ahead of the matrix instruction.
  auto tile_step = [&](int kt, auto stage_c, auto parity) __attribute__((always_inline)) {
    constexpr int stage = decltype(stage_c)::value, par = decltype(parity)::value;
    constexpr int next_stage = stage + 1 == STAGES ? 0 : stage + 1, free_stage = stage == 0 ? STAGES - 1 : stage - 1;
    // (the scalar offsets of this step's loads are formed here, beside the barrier, not in the gaps of the loads)
    int soff_a = __builtin_amdgcn_readfirstlane(soff_a_of(kt + STAGES - 1)), soff_b = __builtin_amdgcn_readfirstlane(soff_b_of(kt + STAGES - 1));
    asm volatile("" : "+s"(soff_a), "+s"(soff_b));
    if (KTAIL && kt + STAGES - 1 == KT - 1) enter_k_tail();
    // own loads of tile kt+1 have landed once only the younger tiles' loads remain in flight
    __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(kLoads * (STAGES - 3)));
    __builtin_amdgcn_s_barrier();  // tile kt+1 published; every wave has left tile kt-1
    static_for<KK>([&](auto kk_c) __attribute__((always_inline)) {
      constexpr int kk = decltype(kk_c)::value;
      Frags &a_cur = af[(kk + par) & 1], &a_nxt = af[(kk + par + 1) & 1];
      Frags &b_cur = bf[(kk + par) & 1], &b_nxt = bf[(kk + par + 1) & 1];
      // the transposed fragments of this slice were requested during the previous one
      if constexpr (A_TR) tr_reads_wait(a_cur.h0, a_cur.h1);
      if constexpr (B_TR) tr_reads_wait(b_cur.h0, b_cur.h1);
      static_for<kMfmas>([&](auto g_c) __attribute__((always_inline)) {
        constexpr int g = decltype(g_c)::value, i = g / kTn, j = g % kTn;
        constexpr bool load_here = (kk * kMfmas + g) % kLoadSpacing == kLoadSpacing - 1 && (kk * kMfmas + g) / kLoadSpacing < kLoads;
        const u32x4 a_op = operand_of(ATr{}, a_cur, i), b_op = operand_of(BTr{}, b_cur, j);
        T::mfma_in_place(&b_op, &a_op, acc[i][j]);
        if constexpr (!load_here) __builtin_amdgcn_sched_barrier(0);
        constexpr int r = load_here ? -1 : g - (g + 1) / kLoadSpacing;  // this gap's read: the gaps without a load, in order
        if constexpr (r >= 0 && r < kReads) {
          using RS = std::integral_constant<int, (kk + 1 < KK ? stage : next_stage)>;
          using RK = std::integral_constant<int, (kk + 1 < KK ? kk + 1 : 0)>;
          if constexpr (r < kTm) read_op(IsA{}, RS{}, RK{}, std::integral_constant<int, r>{}, a_nxt);
          else read_op(IsB{}, RS{}, RK{}, std::integral_constant<int, r - kTm>{}, b_nxt);
        }
        if constexpr (load_here) issue_load_at(soff_a, soff_b, free_stage, (kk * kMfmas + g) / kLoadSpacing);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  // the loop is unrolled over the ring (and over the fragment-buffer parity)
  constexpr int kUnroll = (KK & 1) && (STAGES & 1) ? 2 * STAGES : STAGES;
  int kt = 0;
  for (; kt + kUnroll <= KT; kt += kUnroll)
    static_for<kUnroll>([&](auto u) __attribute__((always_inline)) { tile_step(kt + decltype(u)::value, std::integral_constant<int, decltype(u)::value % STAGES>{}, std::integral_constant<int, (decltype(u)::value * KK) & 1>{}); });
  // Every step ends with the transposing reads of the NEXT step's first slice in flight, and only that step waits for them.  A
  // step that does not run (past the last K-tile) waits in its place, first thing, and so does the end of the kernel: the
  // compiler does not know that those registers are pending and, once nobody reads them any more, hands them out again - a
  // late result would land on top of the new value.  (These waits name no register: an asm operand may be given another
  // register than the read's, and the copy into it would itself read the pending one.  That no instruction names a pending
  // register before its wait is checked on the library's machine code by the build tests.)
  static_for<kUnroll - 1>([&](auto u) __attribute__((always_inline)) {
    if (kt + decltype(u)::value < KT)
      tile_step(kt + decltype(u)::value, std::integral_constant<int, decltype(u)::value % STAGES>{}, std::integral_constant<int, (decltype(u)::value * KK) & 1>{});
    else if constexpr (A_TR || B_TR)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  });
  __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));
  // the in-place matrix instructions are opaque to the compiler, which therefore does not count the wait states their
  // results need before another kind of instruction may read the accumulators
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
  __builtin_amdgcn_s_barrier();  // every wave has left the ring: it is reused as staging space by the packed epilogue
  if (p.split_k > 1 && !split_k_meet<256>(p, tm + tn * p.tiles_m, split, acc, m0 + wm * 64, 16, (uint32_t *)lds)) return;
  if constexpr (PACKED) {
    static_assert(PackedEpilogue<16, 64, 64>::kBytesPerWave * 4 <= STAGES * kStage, "two strips per wavefront must fit the ring");
    PackedEpilogue<16, 64, 64>::run(p, acc, lds + wave * PackedEpilogue<16, 64, 64>::kBytesPerWave, m0 + wm * 64, n0 + wn * 64, lane);
  } else {
#pragma unroll
    for (int i = 0; i < kTm; ++i)
#pragma unroll
      for (int j = 0; j < kTn; ++j) store_block_generic(p, m0 + wm * 64 + i * 16, n0 + wn * 64 + j * 16, lane, acc[i][j]);
  }
}

// ---------------------------------------------------------------------------------------------
// Staged kernel: 128x128x32 tile, 4 wavefronts (2x2), wave tile 64x64.  Any operand strides, ragged
// extents (out-of-range elements read as zero: the padding-ZERO ld_global of the reference).
constexpr int kSBM = 128, kSBN = 128, kSBK = 32;

// One operand tile [128 rows][32 k] is 512 16-byte vectors: 2 per thread.  In "k contiguous" mode a
// vector is 8 consecutive k of one row; in "row contiguous" mode it is 8 consecutive rows at one k
// and is scattered into the K-contiguous LDS image element by element.
struct StagedRegs {
  u32x4 v[2];
};

__device__ __forceinline__ u32x4 load_vec8(const char *base, int64_t s_row, int64_t s_k, int32_t row, int32_t k, int32_t rows,
                                           int32_t K, bool k_contig) {
  u32x4 r = {0, 0, 0, 0};
  const uint16_t *e = (const uint16_t *)base;
  if (k_contig) {
    if (row >= rows || k >= K) return r;
    const uint16_t *ptr = e + row * s_row + k;
    if (k + 8 <= K && (((uintptr_t)ptr) & 15) == 0) return *(const u32x4 *)ptr;
    uint16_t t[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = (k + i < K) ? ptr[i] : (uint16_t)0;
#pragma unroll
    for (int w = 0; w < 4; ++w) r[w] = t[2 * w] | ((uint32_t)t[2 * w + 1] << 16);
    return r;
  }
  if (row >= rows || k >= K) return r;
  const uint16_t *ptr = e + row + k * s_k;  // s_row == 1
  if (row + 8 <= rows && (((uintptr_t)ptr) & 15) == 0) return *(const u32x4 *)ptr;
  uint16_t t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = (row + i < rows) ? ptr[i] : (uint16_t)0;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = t[2 * w] | ((uint32_t)t[2 * w + 1] << 16);
  return r;
}

// Fully strided operand (no contiguous axis): element-wise gather of 8 consecutive k of one row.
__device__ __forceinline__ u32x4 gather_vec8(const char *base, int64_t s_row, int64_t s_k, int32_t row, int32_t k, int32_t rows,
                                             int32_t K) {
  u32x4 r = {0, 0, 0, 0};
  if (row >= rows) return r;
  const uint16_t *e = (const uint16_t *)base + row * s_row;
  uint16_t t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = (k + i < K) ? e[(k + i) * s_k] : (uint16_t)0;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = t[2 * w] | ((uint32_t)t[2 * w + 1] << 16);
  return r;
}

enum OperandMode { kKContig = 0, kRowContig = 1, kStrided = 2 };

template <typename T, bool PACKED>
__global__ __launch_bounds__(256) void staged_kernel(GemmParams p, int a_mode, int b_mode) {
  using L = TileLayout<kSBK * 2, T>;
  __shared__ __attribute__((aligned(1024))) char lds[(kSBM + kSBN) * kSBK * 2];
  char *sa = lds, *sb = lds + kSBM * kSBK * 2;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  int32_t tm, tn;
  tile_of_block(p, tm, tn);
  const int32_t m0 = tm * kSBM, n0 = tn * kSBN;

  auto fetch = [&](const char *base, int64_t s_row, int64_t s_k, int32_t row0, int32_t rows, int mode, int kt, StagedRegs &r) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int v = tid + h * 256;
      if (mode == kRowContig) {
        int k = v >> 4, rchunk = v & 15;  // 16 chunks of 8 rows at each of 32 k
        r.v[h] = load_vec8(base, s_row, s_k, row0 + rchunk * 8, kt * kSBK + k, rows, p.K, false);
      } else {
        int row = v >> 2, kchunk = v & 3;  // 4 chunks of 8 k in each of 128 rows
        r.v[h] = mode == kKContig ? load_vec8(base, s_row, s_k, row0 + row, kt * kSBK + kchunk * 8, rows, p.K, true)
                                  : gather_vec8(base, s_row, s_k, row0 + row, kt * kSBK + kchunk * 8, rows, p.K);
      }
    }
  };
  auto stash = [&](char *tile, int mode, const StagedRegs &r) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int v = tid + h * 256;
      if (mode == kRowContig) {
        int k = v >> 4, rchunk = v & 15;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          uint16_t x = (uint16_t)(r.v[h][e >> 1] >> ((e & 1) * 16));
          *(uint16_t *)(tile + L::offset(rchunk * 8 + e, k >> 3) + (k & 7) * 2) = x;
        }
      } else {
        int row = v >> 2, kchunk = v & 3;
        *(u32x4 *)(tile + L::offset(row, kchunk)) = r.v[h];
      }
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int KT = (p.K + kSBK - 1) / kSBK;
  StagedRegs ra, rb;
  fetch(p.a, p.a_sm, p.a_sk, m0, p.M, a_mode, 0, ra);
  fetch(p.b, p.b_sn, p.b_sk, n0, p.N, b_mode, 0, rb);
  const OperandLane frag_at = operand_lane(T::kShape, lane);
  const uint32_t frag_row = frag_at.row, frag_half = frag_at.k0 / T::kShape.kpack;  // the lane's row of a block; which half of a slice's 16 K
  for (int kt = 0; kt < KT; ++kt) {
    __syncthreads();  // every wave has finished reading the previous tile
    stash(sa, a_mode, ra);
    stash(sb, b_mode, rb);
    __syncthreads();
    if (kt + 1 < KT) {  // next tile's global loads fly while this one is multiplied
      fetch(p.a, p.a_sm, p.a_sk, m0, p.M, a_mode, kt + 1, ra);
      fetch(p.b, p.b_sn, p.b_sk, n0, p.N, b_mode, kt + 1, rb);
    }
#pragma unroll
    for (int kk = 0; kk < kSBK / 16; ++kk) {
      u32x4 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = *(const u32x4 *)(sa + L::offset(wm * 64 + i * 32 + frag_row, 2 * kk + frag_half));
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = *(const u32x4 *)(sb + L::offset(wn * 64 + j * 32 + frag_row, 2 * kk + frag_half));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = T::mfma(&bf[j], &af[i], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int32_t mb = m0 + wm * 64 + i * 32, nb = n0 + wn * 64 + j * 32;
      if (PACKED && mb + 32 <= p.M && nb + 32 <= p.N) store_block_packed(p, mb, nb, lane, acc[i][j]);
      else store_block_generic(p, mb, nb, lane, acc[i][j]);
    }
}

// ---------------------------------------------------------------------------------------------
// Host side.
constexpr int kMaxDevices = 64;  // device ordinals that get a slot in the per-device tables below
bool host_has_tail(const GemmParams &p) { return p.bias != nullptr || p.act >= 0 || p.alpha != 1.0f; }

// 16-bit (RN) or fp32 row-major result with 16-byte aligned rows: the packed epilogue.
bool packed_epilogue(const GemmParams &p) {
  const int64_t eb = p.d_dtype == KAPY_F32 ? 4 : 2, ab = p.acc_dtype == KAPY_F32 ? 4 : 2;
  // an accumulator input: f16 or f32, row-major with 16-byte aligned rows, and neither scales nor a fused tail beside it
  const bool acc_ok = p.acc_dtype < 0 || ((p.acc_dtype == KAPY_F16 || p.acc_dtype == KAPY_F32) && p.acc_sn == 1 && ((uintptr_t)p.acc & 15) == 0 &&
                                          (p.acc_sm * ab) % 16 == 0 && p.acc_sm * ab * 256 < (int64_t(1) << 31) && !p.row_scale && !host_has_tail(p));
  return (p.d_dtype == KAPY_F16 || p.d_dtype == KAPY_BF16 || p.d_dtype == KAPY_F32) && p.d_sn == 1 && acc_ok && (!p.rz || p.d_dtype == KAPY_F32) &&
         ((uintptr_t)p.d & 15) == 0 && (p.d_sm * eb) % 16 == 0 && p.d_sm * eb * 256 < (int64_t(1) << 31) &&  // (a wave's rows are addressed with 32-bit offsets)
         (!p.row_scale || ((uintptr_t)p.col_scale & 15) == 0);
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int STAGES, bool PACKED, bool KTAIL = false, bool TAIL = false>
int launch_tn_epi(GemmParams p, hipStream_t s) {
  using C = TnConfig<T, BM, BN, BK, WM, WN, STAGES>;
  auto kernel = tn_kernel<T, BM, BN, BK, WM, WN, STAGES, PACKED, KTAIL, TAIL>;
  p.tiles_m = (p.M + BM - 1) / BM;  // (only the ring variants are launched with tiles that hang over an edge)
  p.tiles_n = (p.N + BN - 1) / BN;
  constexpr bool kCanSplit = BM == 128 && BN == 128 && STAGES == kRing25;
  if (!kCanSplit) p.split_k = 1;
  if constexpr (C::kLdsBytes > 64 * 1024) {
    // A kernel whose LDS-direct loads address more than the 64 KiB every runtime grants: before its first launch on a device,
    // ask the runtime what it will give it - the code object's static size must be the kernel's own and within the device's
    // limit per workgroup - and refuse instead of launching loads that would land outside the workgroup's allocation.
    static int checked[kMaxDevices];  // 0 not asked, 1 fine, -1 refused (a race between two first calls only repeats the query)
    int dev = -1;
    KAPY_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(KAPY_ERR_UNSUPPORTED, "matmul: device ordinal %d beyond %d", dev, kMaxDevices);
    int state = __atomic_load_n(&checked[dev], __ATOMIC_ACQUIRE);
    if (state == 0) {
      hipFuncAttributes attr;
      int limit = 0;
      const hipError_t e1 = hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kernel));
      const hipError_t e2 = hipDeviceGetAttribute(&limit, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
      state = (e1 == hipSuccess && e2 == hipSuccess && (int64_t)attr.sharedSizeBytes == (int64_t)C::kLdsBytes && limit >= C::kLdsBytes) ? 1 : -1;
      (void)hipGetLastError();
      __atomic_store_n(&checked[dev], state, __ATOMIC_RELEASE);
    }
    if (state < 0) return fail(KAPY_ERR_HIP, "matmul: the runtime does not give this kernel the %d bytes of LDS it addresses (nothing was launched)", C::kLdsBytes);
  }
  kernel<<<dim3((unsigned)(p.tiles_m * p.tiles_n), (unsigned)p.split_k), dim3(C::kThreads), 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}


template <typename T, int BM, int BN, int BK, int WM, int WN, int STAGES>
int launch_tn(const GemmParams &p, hipStream_t s) {
  // a result that ends inside a 16-byte piece of a row takes the bounds-checked element stores
  // (tiles that hang over the edge: the ring builds' loads are bounded, the others fetch the last row again; the strip stores
  // are bounded for all of them)
  const bool whole_tiles = (p.M % BM == 0 && p.N % BN == 0) || ((STAGES == kRing25 || BM <= 128) && p.N % 8 == 0);
  const bool packed = packed_epilogue(p) && whole_tiles;
  if (host_has_tail(p)) {
    // a fused elementwise tail: the ring kernels on the 16x16 instruction have builds with it in the packed epilogue,
    // every other variant applies it in the element stores
    if constexpr (STAGES == kRing25 && T::kM == 16) {
      if (packed) return p.K % BK ? launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, true, true, true>(p, s) : launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, true, false, true>(p, s);
    }
    if constexpr (STAGES == kRing25) {
      if (p.K % BK) return launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, false, true>(p, s);
    }
    return launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, false>(p, s);
  }
  if constexpr (STAGES == kRing25) {
    if (p.K % BK)  // a partial last K-tile: the build of the kernel that masks the lanes past K
      return packed ? launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, true, true>(p, s) : launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, false, true>(p, s);
  }
  return packed ? launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, true>(p, s) : launch_tn_epi<T, BM, BN, BK, WM, WN, STAGES, false>(p, s);
}

template <typename T, int BK, int STAGES, bool A_TR = false, bool B_TR = true, bool KTAIL = false>
int launch_nn(GemmParams p, hipStream_t s) {
  p.tiles_m = (p.M + kNBM - 1) / kNBM;  // (a K-contiguous lhs need not have whole tiles of rows: see the kernel's lhs descriptor)
  p.tiles_n = (p.N + kNBN - 1) / kNBN;  // (nor whole tiles of columns: see its rhs descriptor)
  const bool packed = packed_epilogue(p) && !host_has_tail(p);  // (a fused tail goes through the element stores here)
  dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)p.split_k);
  if (packed) nn_kernel<T, BK, STAGES, true, A_TR, B_TR, KTAIL><<<grid, dim3(256), 0, s>>>(p);
  else nn_kernel<T, BK, STAGES, false, A_TR, B_TR, KTAIL><<<grid, dim3(256), 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

template <typename T>
int launch_staged(GemmParams p, int a_mode, int b_mode, hipStream_t s) {
  p.tiles_m = (p.M + kSBM - 1) / kSBM;
  p.tiles_n = (p.N + kSBN - 1) / kSBN;
  p.split_k = 1;
  dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  if (packed_epilogue(p) && p.d_dtype != KAPY_F32 && p.acc_dtype < 0) staged_kernel<T, true><<<grid, dim3(256), 0, s>>>(p, a_mode, b_mode);  // (its packed stores are 16-bit, without accumulator input)
  else staged_kernel<T, false><<<grid, dim3(256), 0, s>>>(p, a_mode, b_mode);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

// The shape and element-type rules of Kapy.cpp:451-487, with the reference's wording.  Not taken over: the minimum
// extents of :491-564 (acc at least 16x8, lhs / rhs at least 16x8, 16x16 or 8x8 per MMA way) - they bound a warp's
// register tile, and this entry point takes whole views of any extent (a decode-shaped M = 1 included) - and the rule
// that the RESULT is f16 or f32: it is applied to the accumulator operand only, because `result` here is the view the
// kernel's final fptofp stores into (f16, bf16 or f32).
int verify_matmul(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *res, int impl_way) {
  int rc = check_global(lhs, "matmul lhs");
  if (!rc) rc = check_global(rhs, "matmul rhs");
  if (!rc) rc = check_global(res, "matmul result");
  if (!rc && acc) rc = check_global(acc, "matmul acc");
  if (rc) return rc;
  if (extent1(lhs) != extent0(rhs))
    return fail(KAPY_ERR_VERIFY, "matmul: number of columns of lhs must be equal to number of rows of rhs");
  if (extent0(res) != extent0(lhs) || (acc && extent0(acc) != extent0(lhs)))
    return fail(KAPY_ERR_VERIFY, "matmul: number of rows of acc must be equal to number of rows of lhs");
  if (extent1(res) != extent1(rhs) || (acc && extent1(acc) != extent1(rhs)))
    return fail(KAPY_ERR_VERIFY, "matmul: number of columns of acc must be equal to number of columns of rhs");
  if (dtype_bytes(lhs->dtype) != dtype_bytes(rhs->dtype))
    return fail(KAPY_ERR_VERIFY, "matmul: lhs and rhs must have same element bit width");
  if (acc && acc->dtype != KAPY_F16 && acc->dtype != KAPY_F32)
    return fail(KAPY_ERR_VERIFY, "matmul: result must have f16 or f32 element type");
  if (acc && lhs->dtype == KAPY_BF16 && rhs->dtype == KAPY_BF16 && acc->dtype == KAPY_F16)
    return fail(KAPY_ERR_VERIFY, "matmul: result must have f32 element type when operands are bf16 element type");
  if (!is_f8(lhs->dtype) && lhs->dtype != rhs->dtype)
    return fail(KAPY_ERR_VERIFY, "matmul: lhs and rhs must have same element type unless they have f8 element type");
  bool f16ish = lhs->dtype == KAPY_F16 || lhs->dtype == KAPY_BF16;
  switch (impl_way) {
  case KAPY_MATMUL_AUTO: break;
  case KAPY_MMA_M16N8K8_F16: case KAPY_MMA_M16N8K16_F16: case KAPY_MFMA_32X32X16_16B: case KAPY_MFMA_16X16X32_16B:
    if (!f16ish) return fail(KAPY_ERR_VERIFY, "matmul: mma f16 operands must have f16 or bf16 element type");
    break;
  case KAPY_MMA_M16N8K8_TF32:
    if (lhs->dtype != KAPY_F32) return fail(KAPY_ERR_VERIFY, "matmul: mma_m16n8k8_tf32 operands must have f32 element type");
    return fail(KAPY_ERR_UNSUPPORTED, "matmul: mma_m16n8k8_tf32 has no counterpart on gfx950 (no tf32 matrix instruction)");
  case KAPY_MMA_M16N8K16_F8: case KAPY_MFMA_16X16X128_F8: case KAPY_MFMA_32X32X64_F8:
    if (!is_f8(lhs->dtype) || !is_f8(rhs->dtype))
      return fail(KAPY_ERR_VERIFY, "matmul: mma f8 operands must have f8E4M3 or f8E5M2 element type");
    break;
  default: return fail(KAPY_ERR_INVALID, "matmul: unknown implement way %d", impl_way);
  }
  for (const kapy_global *g : {lhs, rhs, res, acc})
    if (g && (g->start0 < 0 || g->start1 < 0)) return fail(KAPY_ERR_INVALID, "matmul: negative view start");
  return KAPY_OK;
}

// Compiled configurations of the TN kernel, in order of preference.
struct TnVariant {
  int bm, bn, bk, waves, stages, mfma;  // mfma: rows of the matrix instruction's operand block (16 or 32)
  int (*launch_bf16)(const GemmParams &, hipStream_t);
  int (*launch_f16)(const GemmParams &, hipStream_t);
};
#define KAPY_TN(BM, BN, BK, WM, WN, S) \
  { BM, BN, BK, (WM) * (WN), S, 32, launch_tn<Bf16, BM, BN, BK, WM, WN, S>, launch_tn<F16, BM, BN, BK, WM, WN, S> }
#define KAPY_TN16(BM, BN, BK, WM, WN, S) \
  { BM, BN, BK, (WM) * (WN), S, 16, launch_tn<Bf16M16, BM, BN, BK, WM, WN, S>, launch_tn<F16M16, BM, BN, BK, WM, WN, S> }
const TnVariant kTnVariants[] = {
    KAPY_TN16(256, 256, 64, 2, 2, kRing25), KAPY_TN16(256, 256, 64, 2, 2, 2),
    KAPY_TN(256, 256, 64, 2, 2, kRing25), KAPY_TN(256, 256, 64, 2, 2, 2), KAPY_TN(256, 256, 32, 2, 2, 4), KAPY_TN16(128, 128, 64, 2, 2, kRing25),
    KAPY_TN(128, 128, 64, 2, 2, 2), KAPY_TN(128, 128, 32, 2, 2, 4), KAPY_TN(128, 128, 64, 2, 2, 4),
    KAPY_TN(128, 64, 64, 2, 2, 4), KAPY_TN(64, 64, 128, 2, 2, 4),
};

int operand_mode(int64_t s_row, int64_t s_k) { return s_k == 1 ? kKContig : (s_row == 1 ? kRowContig : kStrided); }

int64_t split_workspace_bytes(int64_t tiles, int split) { return kSplitCounterBytes + tiles * split * (128 * 128 * 4); }

template <template <int, int> class P, int BM, int BN, int BK, int WM, int WN, int S>
int launch_f8(const GemmParams &p, int lhs_fmt, int rhs_fmt, hipStream_t s) {
  // the kernel issues mfma(rhs fragment, lhs fragment): the first format selector is the rhs's
  switch (rhs_fmt * 2 + lhs_fmt) {
  case 0: return launch_tn<P<0, 0>, BM, BN, BK, WM, WN, S>(p, s);
  case 1: return launch_tn<P<0, 1>, BM, BN, BK, WM, WN, S>(p, s);
  case 2: return launch_tn<P<1, 0>, BM, BN, BK, WM, WN, S>(p, s);
  default: return launch_tn<P<1, 1>, BM, BN, BK, WM, WN, S>(p, s);
  }
}

}  // namespace

// Decides whether the 128 x 128 tiled kernels split K for this problem and points the parameters at the workspace.
// cfg.split_k = 1 or no workspace: never.  0: when the tiles alone would leave at least half the device idle, the
// largest power of two that keeps tiles * split within the CUs, leaves every part at least sixteen K-tiles and fits the
// workspace.  An explicit split that cannot be honoured is an error.
int plan_split_k(GemmParams &p, const kapy_matmul_cfg &c, int tile_k) {
  p.split_k = 1;
  p.partial = nullptr;
  p.counters = nullptr;
  if (c.split_k < 0 || c.split_k > kMaxSplitK || (c.split_k & (c.split_k - 1)))
    return fail(KAPY_ERR_INVALID, "matmul: split_k must be 0 (library's choice) or a power of two up to %d, not %d", kMaxSplitK, c.split_k);
  if (c.split_k == 1) return KAPY_OK;
  if (!c.workspace) {
    if (c.split_k > 1) return fail(KAPY_ERR_INVALID, "matmul: split_k = %d needs a workspace (kapy_matmul_workspace_bytes)", c.split_k);
    return KAPY_OK;
  }
  const int64_t tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128);
  auto fits = [&](int sp) {
    return p.K % (tile_k * sp) == 0 && tiles <= kSplitCounterBytes / 4 && split_workspace_bytes(tiles, sp) <= c.workspace_bytes &&
           ((uintptr_t)c.workspace & 15) == 0;
  };
  int split = 1;
  if (c.split_k > 1) {
    if (!fits(c.split_k))
      return fail(KAPY_ERR_UNSUPPORTED, "matmul: cannot split K = %d into %d parts of whole %d-wide K-tiles with a 16-byte aligned workspace of %lld bytes (%lld needed)",
                  p.K, c.split_k, tile_k, (long long)c.workspace_bytes, (long long)split_workspace_bytes(tiles, c.split_k));
    split = c.split_k;
  } else if (tiles * 2 <= device_cus()) {
    // (meeting in the workspace costs about 10 us: parts shorter than 16 K-tiles do not earn it back)
    for (int sp = 2; sp <= kMaxSplitK && tiles * sp <= device_cus(); sp *= 2)
      if (fits(sp) && p.K / (tile_k * sp) >= 16) split = sp;
  }
  if (split > 1) {
    p.split_k = split;
    p.counters = (uint32_t *)c.workspace;
    p.partial = (float *)((char *)c.workspace + kSplitCounterBytes);
  }
  return KAPY_OK;
}

int matmul_f8_tiled(const GemmParams &p, int lhs_fmt, int rhs_fmt, int want_tile, hipStream_t s) {
  if (p.a_sm * 256 >= (int64_t(1) << 31) || p.b_sn * 256 >= (int64_t(1) << 31)) return KAPY_ERR_UNSUPPORTED;
  // the ring variants take any M, N >= 128 and any K >= 128 of whole 16-byte chunks (their loads are bounded by the
  // operands' ends); 256x256 tiles when there are at least 0.55 times as many of them as CUs, 128x128 (two workgroups per CU) below
  if (p.K % 16 == 0 && p.K >= 128 && p.M >= 1 && p.N >= 128) {
    // (want_tile: 0 = the library's choice, 128 or 256 = the caller's, kapy_matmul_cfg.tile_m)
    // (measured at N = K = 8192: 192 of the large tiles on 256 CUs already beat 768 of the small ones, 128 do not)
    if (want_tile == 256 || (want_tile == 0 && (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256) * 100 >= (int64_t)device_cus() * 55))
      return launch_f8<F8M16, 256, 256, 128, 2, 2, kRing25>(p, lhs_fmt, rhs_fmt, s);
    // At most one 128 x 128 tile per CU and K not split: the ring build's 2.5 tiles of loads in flight are sized for two
    // workgroups per CU, and one alone waits for them (N = K = 8192, 161 .. 512 rows: 50 us whatever M is).  The four-stage
    // build has three tiles (96 KiB) in flight per workgroup: 35.6 / 36.4 / 40.0 / 41.6 / 44 us at 161 / 192 / 256 / 384 / 512
    // rows (five stages measured the same).  It fetches the last row again for rows past an operand's end.
    if (want_tile == 0 && p.split_k <= 1 && p.K % 128 == 0 && (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) <= device_cus())
      return launch_f8<F8, 128, 128, 128, 2, 2, 4>(p, lhs_fmt, rhs_fmt, s);
    return launch_f8<F8M16, 128, 128, 128, 2, 2, kRing25>(p, lhs_fmt, rhs_fmt, s);
  }
  if (p.M % 256 == 0 && p.N % 256 == 0 && p.K % 128 == 0 && (int64_t)(p.M / 256) * (p.N / 256) * 2 >= device_cus())
    return launch_f8<F8M16, 256, 256, 128, 2, 2, kRing25>(p, lhs_fmt, rhs_fmt, s);
  if (p.M % 128 == 0 && p.N % 128 == 0 && p.K % 128 == 0) return launch_f8<F8, 128, 128, 128, 2, 2, 2>(p, lhs_fmt, rhs_fmt, s);
  return KAPY_ERR_UNSUPPORTED;
}

// Implemented in matmul_f8.hip.
int matmul_f8(const kapy_global *a, const kapy_global *b, const float *row_scale, const float *col_scale, const kapy_global *acc,
              const kapy_global *result, const kapy_matmul_cfg *cfg, hipStream_t s);

namespace {
// kapy.matmul with, optionally, the elementwise ops that follow it on the accumulator fused into the kernel's epilogue.
int matmul_16bit(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result,
                 const kapy_matmul_cfg *cfg, const kapy_matmul_epilogue *epi, void *stream) {
  kapy_matmul_cfg c = {KAPY_MATMUL_AUTO, 0, 0, 0, KAPY_RN, 0, 0, 0, nullptr, 0};
  if (cfg) c = *cfg;
  int rc = verify_matmul(lhs, rhs, acc, result, c.impl_way);
  if (rc) return rc;
  if (c.rmode != KAPY_RN && c.rmode != KAPY_RZ) return fail(KAPY_ERR_INVALID, "matmul: unknown rounding mode %d", c.rmode);
  if (result->dtype != KAPY_F16 && result->dtype != KAPY_BF16 && result->dtype != KAPY_F32)
    return fail(KAPY_ERR_VERIFY, "matmul: result must have f16, bf16 or f32 element type");
  if (c.accumulate != KAPY_ACCUMULATE_F32 && c.accumulate != KAPY_ACCUMULATE_ELEMENT) return fail(KAPY_ERR_INVALID, "matmul: unknown accumulate mode %d", c.accumulate);
  rc = ensure_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (c.accumulate == KAPY_ACCUMULATE_ELEMENT) {
    if (epi) return fail(KAPY_ERR_UNSUPPORTED, "matmul_fused: the fused tail exists with fp32 accumulators only");
    if (c.rmode != KAPY_RN) return fail(KAPY_ERR_UNSUPPORTED, "matmul: f16 accumulators round to nearest even, as the instruction they restate");
    return run_matmul_f16acc(lhs, rhs, acc, result, c.impl_way == KAPY_MMA_M16N8K8_F16 ? 8 : 16, s);
  }
  if (is_f8(lhs->dtype)) {
    if (epi) return fail(KAPY_ERR_UNSUPPORTED, "matmul_fused: fp8 operands take kapy_matmul_scaled_f8");
    return matmul_f8(lhs, rhs, nullptr, nullptr, acc, result, &c, s);
  }
  if (lhs->dtype != KAPY_F16 && lhs->dtype != KAPY_BF16)
    return fail(KAPY_ERR_UNSUPPORTED, "matmul: %s operands have no matrix instruction on gfx950", dtype_name(lhs->dtype));

  // A column-major result: D^T = B^T . A^T is the same problem with a row-major result, which the strip epilogues store (a
  // column-major one goes element by element).  Every dot product sums the same products in the same order, so the bits are
  // those of the problem as given.  (A bias row would turn into a bias column, which no epilogue adds: such calls stay.)
  if (result->stride0 == 1 && result->stride1 != 1 && extent0(result) > 1 && !(epi && epi->bias)) {
    auto turned = [](const kapy_global &g) {
      kapy_global t = g;
      std::swap(t.start0, t.start1);
      std::swap(t.end0, t.end1);
      std::swap(t.stride0, t.stride1);
      return t;
    };
    const kapy_global at = turned(*lhs), bt = turned(*rhs), dt = turned(*result);
    kapy_global acct;
    if (acc) acct = turned(*acc);
    kapy_matmul_cfg inner = c;
    std::swap(inner.tile_m, inner.tile_n);
    return matmul_16bit(&bt, &at, acc ? &acct : nullptr, &dt, &inner, epi, stream);
  }

  // A large problem with an operand that is contiguous along its OTHER extent (a row-major rhs, a column-major lhs).  The kernel
  // that reads such operands with transposing LDS reads works on 128 x 128 tiles and reaches 1.05-1.12 PFLOP/s where the
  // K-contiguous kernel's 256 x 256 tiles reach 1.35-1.55.  Turning the operand first costs one pass of the transposing copy
  // over it (its bytes read and written once, at 0.68 of the HBM rate) and pays from about six thousand rows on - if the caller's
  // workspace has room for the turned operand(s) behind the 16 KiB of split-K counters, which stay untouched.
  if (c.workspace && !c.tile_m && !c.tile_n && !c.tile_k && !c.stages && !c.waves && c.split_k <= 1 && c.impl_way < KAPY_MFMA_32X32X16_16B) {
    const int64_t M = extent0(lhs), K = extent1(lhs), N = extent1(rhs);
    const bool a_turn = lhs->stride0 == 1 && lhs->stride1 != 1, b_turn = rhs->stride1 == 1 && rhs->stride0 != 1;
    const bool a_kc = lhs->stride1 == 1, b_kc = rhs->stride0 == 1;
    const int64_t a_bytes = a_turn ? ((M * K * 2 + 255) & ~int64_t(255)) : 0, b_bytes = b_turn ? ((K * N * 2 + 255) & ~int64_t(255)) : 0;
    // (measured, bf16, in place -> turned: 8192^3 1237 -> 1485 TFLOP/s, 8192 x 2048 x 4096 1130 -> 1317, 8192 x 8192 x 1024 924 -> 1106;
    // 4096^3 and 2048 x 8192 x 4096 the same either way; 2048^2 x K slower by a third: the turn is paid once per operand and
    // earned back over the rows - or, for a turned lhs, the columns - that use it)
    // (a row-major rhs beside a row-major lhs with K in whole tiles of 64 is read in place by the 256-wide kernel of
    // matmul_nn256.hip, faster than turn and product together: 8192^3 bf16 0.683 ms against 0.727)
    const bool wide_in_place = b_turn && !a_turn && a_kc && N % 8 == 0 && K % 64 == 0 && ((M + 255) / 256) * ((N + 255) / 256) * 100 >= (int64_t)device_cus() * 55 &&
                               c.rmode == KAPY_RN;
    if (!wide_in_place && (a_turn || b_turn) && (a_turn || a_kc) && (b_turn || b_kc) && (!b_turn || M >= 6144) && (!a_turn || N >= 6144) && M >= 2048 && N >= 2048 && K >= 1024 &&
        M % 8 == 0 && N % 8 == 0 && K % 8 == 0 &&
        M * K < (int64_t(1) << 31) && K * N < (int64_t(1) << 31) && kSplitCounterBytes + a_bytes + b_bytes <= c.workspace_bytes &&
        ((uintptr_t)c.workspace & 255) == 0) {
      char *at = (char *)c.workspace + kSplitCounterBytes;
      kapy_global a2 = *lhs, b2 = *rhs;
      const kapy_copy_cfg turn = {1, KAPY_PAD_ZERO, 0, 0, 0, 0};
      auto dense = [](void *ptr, int64_t rows, int64_t cols, int32_t dtype) {
        kapy_global g;
        g.ptr = ptr;
        g.start0 = g.start1 = 0;
        g.end0 = (int32_t)rows;
        g.end1 = (int32_t)cols;
        g.stride0 = (int32_t)cols;
        g.stride1 = 1;
        g.dtype = dtype;
        g.alignment = 16;
        return g;
      };
      if (b_turn) {  // rhs [K x N] row-major -> [N x K] row-major in the workspace, read back as a [K x N] view with K contiguous
        const kapy_global turned = dense(at, N, K, rhs->dtype);
        rc = copy_impl(rhs, &turned, &turn, nullptr, stream);
        if (rc) return rc;
        b2 = turned;
        b2.end0 = (int32_t)K; b2.end1 = (int32_t)N;
        b2.stride0 = 1; b2.stride1 = (int32_t)K;
        at += b_bytes;
      }
      if (a_turn) {  // lhs [M x K] column-major -> row-major
        const kapy_global turned = dense(at, M, K, lhs->dtype);
        kapy_global as_rows = *lhs;  // the same memory seen as the row-major [K x M] it is, which the copy transposes
        std::swap(as_rows.start0, as_rows.start1);
        std::swap(as_rows.end0, as_rows.end1);
        std::swap(as_rows.stride0, as_rows.stride1);
        rc = copy_impl(&as_rows, &turned, &turn, nullptr, stream);
        if (rc) return rc;
        a2 = turned;
      }
      kapy_matmul_cfg inner = c;
      inner.workspace = nullptr;
      inner.workspace_bytes = 0;
      return matmul_16bit(&a2, &b2, acc, result, &inner, epi, stream);
    }
  }

  GemmParams p;
  p.a = view_base(lhs);
  p.b = view_base(rhs);
  p.acc = acc ? view_base(acc) : nullptr;
  p.d = (char *)view_base(result);
  p.row_scale = p.col_scale = nullptr;
  p.bias = epi && epi->bias ? view_base(epi->bias) : nullptr;
  p.bias_dtype = epi && epi->bias ? epi->bias->dtype : KAPY_F32;
  p.alpha = epi ? epi->alpha : 1.0f;
  p.act = epi ? epi->act : -1;
  p.act_operand = epi ? epi->act_operand : 0.f;
  p.a_sm = lhs->stride0; p.a_sk = lhs->stride1;
  p.b_sk = rhs->stride0; p.b_sn = rhs->stride1;
  p.acc_sm = acc ? acc->stride0 : 0; p.acc_sn = acc ? acc->stride1 : 0;
  p.d_sm = result->stride0; p.d_sn = result->stride1;
  p.M = (int32_t)extent0(lhs); p.K = (int32_t)extent1(lhs); p.N = (int32_t)extent1(rhs);
  p.acc_dtype = acc ? acc->dtype : -1;
  p.d_dtype = result->dtype;
  p.rz = c.rmode == KAPY_RZ;
  p.tiles_m = p.tiles_n = 0;
  p.split_k = 1;
  p.partial = nullptr;
  p.counters = nullptr;
  if (p.M == 0 || p.N == 0) return KAPY_OK;
  const bool bf16 = lhs->dtype == KAPY_BF16;

  // Roofline path: both operands K-contiguous, 16-byte aligned rows, extents multiples of the tile,
  // and offsets that fit the 32-bit per-lane address arithmetic of the loader.
  bool tn = p.a_sk == 1 && p.b_sk == 1 && vector_bytes(lhs, 1) == 16 && vector_bytes(rhs, 0) == 16 && p.K > 0 &&
            p.a_sm * 2 * 256 < (int64_t(1) << 31) && p.b_sn * 2 * 256 < (int64_t(1) << 31) && p.a_sm >= 0 && p.b_sn >= 0;
  if (tn) {
    const bool free_choice = !c.tile_m && !c.tile_n && !c.tile_k && !c.stages && !c.waves && c.impl_way < KAPY_MFMA_32X32X16_16B;
    for (const TnVariant &v : kTnVariants) {
      if ((c.tile_m && c.tile_m != v.bm) || (c.tile_n && c.tile_n != v.bn) || (c.tile_k && c.tile_k != v.bk) ||
          (c.stages && c.stages != v.stages) || (c.waves && c.waves != v.waves) ||
          (c.impl_way == KAPY_MFMA_32X32X16_16B && v.mfma != 32) || (c.impl_way == KAPY_MFMA_16X16X32_16B && v.mfma != 16))
        continue;
      // the ring variants' bounded loads let a tile hang over the last rows of either operand; the others need whole tiles
      const bool whole_tiles = p.M % v.bm == 0 && p.N % v.bn == 0;
      const bool whole_k = p.K % v.bk == 0;  // the ring variants also take a partial last K-tile of whole 16-byte chunks
      if ((!whole_k && (v.stages != kRing25 || p.K % 8)) || (!whole_tiles && v.stages != kRing25)) continue;
      // with a free choice, a 256x256 tiling with fewer than 0.55 tiles per CU yields to 128x128 (measured: 144 large tiles on
      // 256 CUs beat 576 small ones - 3072^3: 1009 against 899 TFLOP/s - 128 do not)
      if (free_choice && v.bm == 256 && (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256) * 100 < (int64_t)device_cus() * 55) continue;
      // an explicit split of K is a request for a variant that can split: with a free tile choice the others are passed over
      // (plan_split_k then honours the split or says why it cannot)
      if (c.split_k > 1 && !c.tile_m && !(v.bm == 128 && v.stages == kRing25)) continue;
      if (v.bm == 128 && v.stages == kRing25) {
        rc = plan_split_k(p, c, v.bk);
        if (rc) return rc;
        // Tiles for at most half the CUs and K not split: a workgroup alone on its CU waits for the ring's 2.5 tiles of loads.
        // The four-stage build on the 32-row instruction keeps three tiles in flight: bf16 N = K = 8192, 128 / 256 rows
        // 54 / 55 -> 48 / 52 us (level at 384 rows, behind from 512; the same depth on the 16-row instruction: 71 us).
        // Fewer still: smaller tiles put every CU to work on the operand streams.  bf16 N = K = 8192, 64 / 128 rows on
        // 64 x 64 x 128 tiles 48 / 47 -> 30 / 30 us, 256 rows on 128 x 64 x 64 tiles 47.5 -> 43; from 384 rows on (more small
        // tiles than CUs) they lose to the 128 x 128 ring.
        if (free_choice && p.split_k <= 1 && !host_has_tail(p) && p.N % 8 == 0) {
          const int64_t n64 = (p.N + 63) / 64;
          if (p.K % 128 == 0 && (int64_t)((p.M + 63) / 64) * n64 <= device_cus())
            return bf16 ? launch_tn<Bf16, 64, 64, 128, 2, 2, 4>(p, s) : launch_tn<F16, 64, 64, 128, 2, 2, 4>(p, s);
          if (p.K % 64 == 0 && (int64_t)((p.M + 127) / 128) * n64 <= device_cus())
            return bf16 ? launch_tn<Bf16, 128, 64, 64, 2, 2, 4>(p, s) : launch_tn<F16, 128, 64, 64, 2, 2, 4>(p, s);
        }
        if (free_choice && p.split_k <= 1 && !host_has_tail(p) && p.K % 64 == 0 && p.N % 8 == 0 &&
            (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * 2 <= device_cus())
          return bf16 ? launch_tn<Bf16, 128, 128, 64, 2, 2, 4>(p, s) : launch_tn<F16, 128, 128, 64, 2, 2, 4>(p, s);
      } else if (c.split_k > 1 && c.tile_m) {
        return fail(KAPY_ERR_UNSUPPORTED, "matmul: only the 128 x 128 tiles split K");
      }
      return bf16 ? v.launch_bf16(p, s) : v.launch_f16(p, s);
    }
  }
  // An operand that is contiguous along its other extent - a row-major rhs (with a row-major lhs: the reference fixture's
  // layout, matmul.mlir), a column-major lhs - is staged as it lies and read with the transposing read.
  const bool a_kc = p.a_sk == 1 && vector_bytes(lhs, 1) == 16 && p.a_sm >= 0 && p.a_sm * 2 * kNBM < (int64_t(1) << 31);
  const bool a_tr = !a_kc && p.a_sm == 1 && vector_bytes(lhs, 0) == 16 && p.a_sk >= 0 && p.M % kNBM == 0 && (int64_t)p.K * p.a_sk * 2 < (int64_t(1) << 31);
  const bool b_tr = p.b_sn == 1 && vector_bytes(rhs, 1) == 16 && p.b_sk >= 0 && (int64_t)p.K * p.b_sk * 2 < (int64_t(1) << 31);
  const bool b_kc = !b_tr && p.b_sk == 1 && vector_bytes(rhs, 0) == 16 && p.b_sn >= 0 && p.b_sn * 2 * kNBN < (int64_t(1) << 31);
  bool nn = (a_kc || a_tr) && (b_kc || b_tr) && (a_tr || b_tr) && p.M > 0 && p.N % 8 == 0 && p.K > 0 &&
            c.impl_way != KAPY_MFMA_32X32X16_16B && (!c.tile_m || c.tile_m == kNBM) && (!c.tile_n || c.tile_n == kNBN) && (!c.waves || c.waves == 4);
  if (nn) {
    struct NnVariant {
      int bk, stages;
      int (*launch_bf16[3])(GemmParams, hipStream_t);   // lhs K-contiguous x rhs transposed, both transposed, lhs transposed x rhs K-contiguous
      int (*launch_f16[3])(GemmParams, hipStream_t);
    };
#define KAPY_NN(BK, ST) {BK, ST, {launch_nn<Bf16M16, BK, ST, false, true>, launch_nn<Bf16M16, BK, ST, true, true>, launch_nn<Bf16M16, BK, ST, true, false>}, \
                         {launch_nn<F16M16, BK, ST, false, true>, launch_nn<F16M16, BK, ST, true, true>, launch_nn<F16M16, BK, ST, true, false>}}
    static const NnVariant kNn[] = {KAPY_NN(64, 4), KAPY_NN(64, 3), KAPY_NN(32, 4)};
#undef KAPY_NN
    const int form = !a_tr ? 0 : (b_tr ? 1 : 2);
    // Row-major x row-major with enough 256 x 256 tiles for the device (the rule of the K-contiguous kernel): the 256-wide
    // form, half the LDS bytes per flop of the 128-wide tiles below.
    static const bool wide = !(getenv("KAPY_NN256") && getenv("KAPY_NN256")[0] == '0');
    // (KAPY_NN256_FROM: the least number of 256 x 256 tiles per 100 CUs, for measurements)
    static const int wide_from_pct = getenv("KAPY_NN256_FROM") ? atoi(getenv("KAPY_NN256_FROM")) : 55;
    if (wide && form == 0 && !c.tile_m && !c.tile_n && !c.tile_k && !c.stages && !c.waves && c.split_k <= 1 && !p.rz && nn256_serves(p) && packed_epilogue(p) &&
        (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256) * 100 >= (int64_t)device_cus() * wide_from_pct)
      return launch_nn256(p, bf16, s);
    for (const NnVariant &v : kNn) {
      if ((c.tile_k && c.tile_k != v.bk) || (c.stages && c.stages != v.stages) || p.K % v.bk) continue;
      rc = plan_split_k(p, c, v.bk);
      if (rc) return rc;
      return bf16 ? v.launch_bf16[form](p, s) : v.launch_f16[form](p, s);
    }
    // K a multiple of 8 that no variant's K-tile divides: the builds with a partial last K-tile (never split)
    if (p.K % 8 == 0 && !c.stages && c.split_k <= 1) {
#define KAPY_NN_TAIL(BK) {launch_nn<Bf16M16, BK, 4, false, true, true>, launch_nn<Bf16M16, BK, 4, true, true, true>, launch_nn<Bf16M16, BK, 4, true, false, true>, \
                          launch_nn<F16M16, BK, 4, false, true, true>, launch_nn<F16M16, BK, 4, true, true, true>, launch_nn<F16M16, BK, 4, true, false, true>}
      static int (*const kTail64[6])(GemmParams, hipStream_t) = KAPY_NN_TAIL(64);
      static int (*const kTail32[6])(GemmParams, hipStream_t) = KAPY_NN_TAIL(32);
#undef KAPY_NN_TAIL
      const int bk = c.tile_k ? c.tile_k : (p.K >= 256 ? 64 : 32);
      if (bk == 64 || bk == 32) {
        p.split_k = 1;
        return (bk == 64 ? kTail64 : kTail32)[(bf16 ? 0 : 3) + form](p, s);
      }
    }
  }
  if ((c.tile_m && c.tile_m != kSBM) || (c.tile_n && c.tile_n != kSBN) || (c.tile_k && c.tile_k != kSBK) || (c.stages && c.stages != 1) ||
      (c.waves && c.waves != 4))
    return fail(KAPY_ERR_UNSUPPORTED, "matmul: no kernel with tile %dx%dx%d, %d stages, %d waves serves these operands "
                                      "(the general kernel is 128x128x32, 1 stage, 4 waves)",
                c.tile_m, c.tile_n, c.tile_k, c.stages, c.waves);
  int a_mode = operand_mode(p.a_sm, p.a_sk), b_mode = operand_mode(p.b_sn, p.b_sk);
  return bf16 ? launch_staged<Bf16>(p, a_mode, b_mode, s) : launch_staged<F16>(p, a_mode, b_mode, s);
}


}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" {

int kapy_matmul(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result,
                const kapy_matmul_cfg *cfg, void *stream) {
  return matmul_16bit(lhs, rhs, acc, result, cfg, nullptr, stream);
}

int64_t kapy_matmul_turn_workspace_bytes(const kapy_global *lhs, const kapy_global *rhs) {
  if (!lhs || !rhs) return 0;
  const int64_t M = extent0(lhs), K = extent1(lhs), N = extent1(rhs);
  const bool a_turn = lhs->stride0 == 1 && lhs->stride1 != 1, b_turn = rhs->stride1 == 1 && rhs->stride0 != 1;
  if (!a_turn && !b_turn) return 0;
  return kSplitCounterBytes + (a_turn ? ((M * K * 2 + 255) & ~int64_t(255)) : 0) + (b_turn ? ((K * N * 2 + 255) & ~int64_t(255)) : 0);
}

int64_t kapy_matmul_workspace_bytes(int64_t m, int64_t n) {
  if (m <= 0 || n <= 0) return 0;
  // a split keeps tiles * parts within the CUs of the device; without a device, the largest split of every tile
  const int64_t tiles = ((m + 127) / 128) * ((n + 127) / 128);
  return split_workspace_bytes(tiles, kMaxSplitK);
}

int kapy_matmul_static_workspace(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result,
                                 const kapy_matmul_cfg *cfg, void *stream) {
  kapy_matmul_cfg c = {KAPY_MATMUL_AUTO, 0, 0, 0, KAPY_RN, 0, 0, 0, nullptr, 0};
  if (cfg) c = *cfg;
  int rc = ensure_device();
  if (rc) return rc;
  // The array's name is a host-side handle, not a device address: ask the runtime once per device where this device's
  // copy lives, and hand that pointer to the kernels.
  static void *scratch_on_device[kMaxDevices];  // (a race between two first calls only repeats the query)
  int dev = -1;
  KAPY_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(KAPY_ERR_UNSUPPORTED, "matmul_static_workspace: device ordinal %d beyond %d", dev, kMaxDevices);
  void *ws = __atomic_load_n(&scratch_on_device[dev], __ATOMIC_ACQUIRE);
  if (!ws) {
    KAPY_HIP_CHECK(hipGetSymbolAddress(&ws, HIP_SYMBOL(scratch)));
    if (!ws) return fail(KAPY_ERR_HIP, "matmul_static_workspace: the runtime reports no address for the workspace array");
    __atomic_store_n(&scratch_on_device[dev], ws, __ATOMIC_RELEASE);
  }
  c.workspace = ws;
  c.workspace_bytes = (int64_t)sizeof(scratch);
  return matmul_16bit(lhs, rhs, acc, result, &c, nullptr, stream);
}

int kapy_matmul_fused(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *result, const kapy_matmul_epilogue *epi,
                      const kapy_matmul_cfg *cfg, void *stream) {
  if (!epi) return fail(KAPY_ERR_INVALID, "matmul_fused: null epilogue");
  switch (epi->act) {
  case -1: case KAPY_EW_GELU_TANH: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF: case KAPY_EW_NEGF: case KAPY_EW_ABSF:
    break;
  case KAPY_EW_EXP: case KAPY_EW_EXP2: case KAPY_EW_LOG: case KAPY_EW_LOG2: case KAPY_EW_SQRT: case KAPY_EW_RSQRT: case KAPY_EW_TANH: case KAPY_EW_ERF:
    return fail(KAPY_ERR_UNSUPPORTED, "matmul_fused: this activation is not compiled into the matmul kernels; run it as an elementwise program on the result");
  default: return fail(KAPY_ERR_INVALID, "matmul_fused: act must be a unary elementwise op, maximumf / minimumf (against act_operand) or -1, not %d", epi->act);
  }
  if (epi->bias) {
    int rc = check_global(epi->bias, "matmul_fused bias");
    if (rc) return rc;
    if (epi->bias->dtype != KAPY_F16 && epi->bias->dtype != KAPY_BF16 && epi->bias->dtype != KAPY_F32)
      return fail(KAPY_ERR_VERIFY, "matmul_fused: bias must have f16, bf16 or f32 element type");
    if (!rhs || extent0(epi->bias) != 1 || extent1(epi->bias) != extent1(rhs) || epi->bias->stride1 != 1)
      return fail(KAPY_ERR_VERIFY, "broadcast: the bias must be one contiguous row [1 x N]");
  }
  return matmul_16bit(lhs, rhs, nullptr, result, cfg, epi, stream);
}

int kapy_matmul_lds_layout(int32_t operand_dtype, int32_t tile_k, kapy_swizzling *out) {
  if (!out) return fail(KAPY_ERR_INVALID, "matmul_lds_layout: null result");
  if (operand_dtype != KAPY_F16 && operand_dtype != KAPY_BF16)
    return fail(KAPY_ERR_UNSUPPORTED, "matmul_lds_layout: only f16 / bf16 operand tiles are described here");
  Swizzle s;
  switch (tile_k) {
  case 32: s = TileLayout<64, Bf16>::kSwizzle; break;      // (f16 and bf16 share the operand layouts; the 32-deep tiles are built
  case 64: s = TileLayout<128, Bf16M16>::kSwizzle; break;  //  on the 32x32x16 instruction, the 64-deep ones on 16x16x32)
  default: return fail(KAPY_ERR_UNSUPPORTED, "matmul_lds_layout: tile_k must be 32 or 64");
  }
  s.stride0 = tile_k;  // the search runs on bytes; report the row stride in elements
  out->stride0 = s.stride0;
  out->stride1 = s.stride1;
  out->bank_param = s.bank_param;
  out->line_param = s.line_param;
  out->rotate = s.rotate;
  return KAPY_OK;
}

}  // extern "C"
