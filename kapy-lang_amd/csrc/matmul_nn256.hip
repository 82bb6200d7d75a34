// matmul_nn256.hip — large kapy.matmul on a row-major lhs and a ROW-major rhs (the layout of the reference's fixture,
// test/Conversion/KapyToKgpu/matmul.mlir) on 256 x 256 x 64 tiles.
//
// nn_kernel (matmul.hip) serves that layout on 128 x 128 tiles, which read twice the LDS bytes per flop of the 256-wide tiles
// and stop at half the matrix peak.  This kernel is the 256-wide form: 4 wavefronts (2 x 2), a wave tile of 128 x 128 =
// 8 x 8 blocks of the 16x16x32 instruction, two LDS stages of 64 KiB.  The lhs tile is staged K-contiguous under the tiled
// kernel's swizzle and read 16 bytes per lane; the rhs tile is staged as it lies in memory - for each half of its columns an
// image [64 k-rows][128 columns] with 16-byte chunk c of k-row r at chunk c ^ rhs_key(r), nn_kernel's image - and its operand
// registers are made on the way out of LDS by ds_read_b64_tr_b16 (the ldmatrix.trans of LdMatrixOpToLLVM.cpp:128-129).
// Both come in by LDS-direct buffer loads (the cp_async of CpAsyncOpToLLVM.cpp:22-186).
// One barrier per K-tile, before the tile's last K-slice: by then every wave holds that slice's fragments, so the stage is
// free; the loads of the tile after next go out behind the matrix instructions of that last slice and have the next tile's
// first slice to land.  Whole tiles only (M, N multiples of 256, K of 64), strip epilogue only: the host checks both.
#include "matmul_tile.hpp"

namespace kapy {
namespace {

constexpr int kBM = 256, kBN = 256, kBK = 64, kStageBytes = 65536, kImageB = 32768, kHalfB = 16384, kRowTr = 256;
constexpr int kLoadsOp = 8;   // LDS-direct loads per wavefront, operand and K-tile (32 KiB / 1 KiB / 4 waves)
// (nn_kernel's key: a transposing read of a half wave touches k-rows {0..3} + 8*{0,1} (+4) of a 32-row slice, 32 bytes of each;
// the key sends those eight to the eight 32-byte bank groups of the 256-byte row)
__device__ __forceinline__ uint32_t rhs_key(uint32_t row) { return ((row & 3) + 4 * ((row >> 3) & 1)) * 2; }

// Waits for the transposing reads whose results sit in h0[j], h1[j] (j < 8) and hands those registers back as its own results
// (the registers of a read still pending must not be touched by anything before this).
__device__ __forceinline__ void tr_reads_wait8(u32x2_lds (&h0)[8], u32x2_lds (&h1)[8]) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(h0[0]), "+v"(h0[1]), "+v"(h0[2]), "+v"(h0[3]), "+v"(h0[4]), "+v"(h0[5]), "+v"(h0[6]), "+v"(h0[7]), "+v"(h1[0]), "+v"(h1[1]),
                 "+v"(h1[2]), "+v"(h1[3]), "+v"(h1[4]), "+v"(h1[5]), "+v"(h1[6]), "+v"(h1[7])
               :
               : "memory");
}

// TAIL: the build for calls with a fused elementwise tail (scale, bias, activation in the strip epilogue).
template <typename T, bool TAIL = false>
__global__ __launch_bounds__(256) void nn256_kernel(GemmParams p) {
  static_assert(T::kM == 16 && T::kBytes == 2, "16x16x32 instruction, 16-bit operands");
  using LA = TileLayout<kBK * 2, T, 16>;
  constexpr int kRowKc = kBK * 2, KK = kBK / 32, kTm = 8, kTn = 8, kMfmas = kTm * kTn;
  __shared__ __attribute__((aligned(1024))) char lds[2 * kStageBytes];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  int32_t tm, tn;
  tile_of_block(p, tm, tn);
  const int32_t m0 = tm * kBM, n0 = tn * kBN;
  const int KT = __builtin_amdgcn_readfirstlane(p.K / kBK);
  const int32_t a_ld = __builtin_amdgcn_readfirstlane((int32_t)p.a_sm), b_ld = __builtin_amdgcn_readfirstlane((int32_t)p.b_sk);

  // Per-lane global byte offset of the 16-byte piece this lane fetches with load instruction 0 of an operand; instruction q
  // fills bytes [(wave + 4q) * 1024, + 1024) of the operand's image, which is 32 rows (lhs) or 16 k-rows and, from q = 4 on,
  // the other half of the columns (rhs) further on - neither swizzle mixes in a bit that q changes - so the rest of an
  // instruction's address is a scalar.
  static_assert(16 % LA::kLineParam == 0, "the lhs key must not depend on the load instruction");
  uint32_t a_goff, b_goff;
  {
    const uint32_t o = (uint32_t)wave * 1024u + lane * 16u;
    uint32_t row, chunk;
    LA::locate(o, row, chunk);
    a_goff = (uint32_t)((row * a_ld + chunk * 8) * 2);
    const uint32_t krow = o / kRowTr, c = ((o % kRowTr) / 16) ^ rhs_key(krow);
    b_goff = (uint32_t)((krow * b_ld + c * 8) * 2);
  }
  auto uniform_ptr = [](const char *ptr) {
    const uint64_t v = (uint64_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (void *)(((uint64_t)hi << 32) | lo);
  };
  // (the descriptors end where the operands end: what a tile has beyond the last row of the lhs, or beyond the last k-row's
  // N columns of the rhs, reads as zeros)
  const int64_t a_left = ((int64_t)(p.M - m0 - 1) * p.a_sm + p.K) * 2, b_left = ((int64_t)(p.K - 1) * p.b_sk + (p.N - n0)) * 2;
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.a + (int64_t)m0 * p.a_sm * 2), 0,
                                                                          __builtin_amdgcn_readfirstlane((int)(a_left < 0x7fffffff ? a_left : 0x7fffffff)), 0x00020000);
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.b + (int64_t)n0 * 2), 0,
                                                                          __builtin_amdgcn_readfirstlane((int)(b_left < 0x7fffffff ? b_left : 0x7fffffff)), 0x00020000);
  const int wave_lds = wave * 1024;
  // load instruction idx (0 .. 15: the lhs ones, then the rhs ones) of this wavefront for the K-tile at scalar offsets soff_a / soff_b
  auto issue_load = [&](int soff_a, int soff_b, int stage, int idx) __attribute__((always_inline)) {
    if (idx < kLoadsOp) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(lds + stage * kStageBytes + idx * 4096 + wave_lds), 16,
                                               (int)a_goff, soff_a + idx * 32 * a_ld * 2, 0, 0);
    } else {
      const int q = idx - kLoadsOp;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (__attribute__((address_space(3))) void *)(lds + stage * kStageBytes + kImageB + q * 4096 + wave_lds), 16,
                                               (int)b_goff, soff_b + ((q % 4) * 16 * b_ld + (q / 4) * 128) * 2, 0, 0);
    }
  };
  auto soff_a_of = [&](int j) { return min(j, KT - 1) * kBK * 2; };              // (tiles past the end of K repeat the last one,
  auto soff_b_of = [&](int j) { return min(j, KT - 1) * kBK * b_ld * 2; };       //  into a stage nobody reads again)

  // Operand reads.  lhs: row l16 of each 16-row block of the wave's 128 rows, 16-byte chunk 4 * kk + grp.  rhs: the
  // transposing read hands lane j of a 16-lane group element j of the four k-rows whose 8-byte pieces the group's lanes
  // address, so lane l16 addresses k-row 8 * grp + 4 * h + l16 / 4, elements 4 * (l16 % 4) .. of the block.
  const OperandLane frag_at = operand_lane(T::kShape, lane);
  const uint32_t grp = frag_at.k0 / T::kShape.kpack, l16 = frag_at.row;
  static_assert((16 * kRowKc) % (256 * LA::kLineParam) == 0, "an operand block must span whole swizzle periods");
  const uint32_t tr_row = 8 * grp + (l16 >> 2), tr_key = rhs_key(tr_row);  // (the key is the same for every slice and half)
  // one address register per stage and slice (lhs) / per stage and block (rhs: the key enters by XOR); the rest is an immediate
  uint32_t a_at[2][KK], b_at[2][kTn];
#pragma unroll
  for (int st = 0; st < 2; ++st) {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      uint32_t v = (uint32_t)(uintptr_t)lds + st * kStageBytes + LA::offset(wm * 128 + l16, 4 * kk + grp);
      asm volatile("" : "+v"(v));  // (opaque: registers that stay, not one register and an add at every read)
      a_at[st][kk] = v;
    }
#pragma unroll
    for (int j = 0; j < kTn; ++j) {
      uint32_t v = (uint32_t)(uintptr_t)lds + st * kStageBytes + kImageB + wn * kHalfB + tr_row * kRowTr + (((j * 2 + ((l16 & 3) >> 1)) ^ tr_key) * 16) + (l16 & 1) * 8;
      asm volatile("" : "+v"(v));
      b_at[st][j] = v;
    }
  }
  struct Frags {
    u32x4 a[kTm];
    u32x2_lds h0[kTn], h1[kTn];
  };
  // read r (0 .. 23) of slice KKc of stage STc: lhs blocks 0 .. 7, then the two halves of rhs blocks 0 .. 7
  auto read_op = [&](auto stage_c, auto kk_c, auto r_c, Frags &dst) __attribute__((always_inline)) {
    constexpr int st = decltype(stage_c)::value, kk = decltype(kk_c)::value, r = decltype(r_c)::value;
    if constexpr (r < kTm) {
      dst.a[r] = *(const __attribute__((address_space(3))) u32x4 *)(uintptr_t)(a_at[st][kk] + (uint32_t)r * 16 * kRowKc);
    } else if constexpr (r < kTm + kTn) {
      dst.h0[r - kTm] = tr_read_b64_at<(uint32_t)(kk * 32 * kRowTr)>(b_at[st][r - kTm]);
    } else {
      dst.h1[r - kTm - kTn] = tr_read_b64_at<(uint32_t)(kk * 32 * kRowTr + 4 * kRowTr)>(b_at[st][r - kTm - kTn]);
    }
  };
  constexpr int kReads = kTm + 2 * kTn;

  using Acc = typename T::Acc;
  Acc acc[kTm][kTn];
#pragma unroll
  for (int i = 0; i < kTm; ++i)
#pragma unroll
    for (int j = 0; j < kTn; ++j) acc[i][j] = Acc{0.f, 0.f, 0.f, 0.f};

  // prologue: tiles 0 and 1
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int idx = 0; idx < 2 * kLoadsOp; ++idx) issue_load(soff_a_of(t), soff_b_of(t), t, idx);
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kLoadsOp));
  __builtin_amdgcn_s_barrier();  // tile 0 published
  Frags fr[2];
  using Zero = std::integral_constant<int, 0>;
  static_for<kReads>([&](auto r) __attribute__((always_inline)) { read_op(Zero{}, Zero{}, r, fr[0]); });

  constexpr int kLoadSpacing = 4;  // one load behind every fourth matrix instruction of a tile's last slice: 16 loads in 64
  static_assert(kMfmas / kLoadSpacing == 2 * kLoadsOp && kReads <= kMfmas - kMfmas / kLoadSpacing, "gaps for the loads and, apart from them, the reads");
  // One K-tile in stage STAGE (compile time: every LDS address is then a register plus an immediate).
  auto tile_step = [&](int kt, auto stage_c) __attribute__((always_inline)) {
    constexpr int stage = decltype(stage_c)::value;
    int soff_a = __builtin_amdgcn_readfirstlane(soff_a_of(kt + 2)), soff_b = __builtin_amdgcn_readfirstlane(soff_b_of(kt + 2));
    asm volatile("" : "+s"(soff_a), "+s"(soff_b));
    static_for<KK>([&](auto kk_c) __attribute__((always_inline)) {
      constexpr int kk = decltype(kk_c)::value;
      constexpr bool last = kk == KK - 1;
      Frags &cur = fr[kk & 1], &nxt = fr[(kk + 1) & 1];
      if constexpr (last) {
        // own loads of tile kt+1 have landed and own reads of this stage have returned (the last slice's fragments among
        // them: they were asked for during the slice before); then every wave's have
        __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));
        __builtin_amdgcn_s_barrier();
      }
      tr_reads_wait8(cur.h0, cur.h1);
      static_for<kMfmas>([&](auto g_c) __attribute__((always_inline)) {
        constexpr int g = decltype(g_c)::value, i = g / kTn, j = g % kTn;
        const u32x4 b_op = u32x4{cur.h0[j][0], cur.h0[j][1], cur.h1[j][0], cur.h1[j][1]};
        T::mfma_in_place(&b_op, &cur.a[i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        constexpr bool load_here = last && g % kLoadSpacing == 0;
        constexpr int r = g % kLoadSpacing == 0 ? -1 : g - 1 - g / kLoadSpacing;  // the gaps without a load, in order
        if constexpr (r >= 0 && r < kReads) {
          using RS = std::integral_constant<int, (last ? stage ^ 1 : stage)>;
          using RK = std::integral_constant<int, (last ? 0 : kk + 1)>;
          read_op(RS{}, RK{}, std::integral_constant<int, r>{}, nxt);
        }
        if constexpr (load_here) issue_load(soff_a, soff_b, stage, g / kLoadSpacing);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  int kt = 0;
  for (; kt + 2 <= KT; kt += 2) {
    tile_step(kt, std::integral_constant<int, 0>{});
    tile_step(kt + 1, std::integral_constant<int, 1>{});
  }
  if (kt < KT) tile_step(kt, std::integral_constant<int, 0>{});
  // Every step ends with the reads of the next step's first slice in flight; nobody waits for the last ones but this.  The
  // loads issued for tiles past the end of K still target this workgroup's LDS.
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(0));
  // the in-place matrix instructions are opaque to the compiler, which therefore does not count the wait states their
  // results need before another kind of instruction may read the accumulators
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
  __builtin_amdgcn_s_barrier();  // every wave has left the stages: they are reused as staging space by the strip epilogue
  static_assert(PackedEpilogue<16, 128, 128>::kBytesPerWave * 4 <= 2 * kStageBytes, "a strip per wavefront must fit the stages");
  PackedEpilogue<16, 128, 128>::template run<TAIL>(p, acc, lds + wave * PackedEpilogue<16, 128, 128>::kBytesPerWave, m0 + wm * 128, n0 + wn * 128, lane);
}

}  // namespace

// Whether nn256_kernel serves the problem (the caller has checked the strip epilogue's own conditions): both operands with
// contiguous, 16-byte aligned rows of whole 16-byte pieces and whole K-tiles.  Tiles may hang over the last rows and columns:
// the lhs descriptor ends with the operand's last row (rows beyond it read as zeros), rhs columns beyond N are whatever
// follows in memory up to the end of the last k-row (zeros beyond) and only reach result columns that are never stored, and
// the strip stores are bounded by the result's extents.
bool nn256_serves(const GemmParams &p) {
  return p.a_sk == 1 && p.b_sn == 1 && p.M > 0 && p.N > 0 && p.N % 8 == 0 && p.K % kBK == 0 && p.K >= 2 * kBK && p.a_sm % 8 == 0 && p.b_sk % 8 == 0 &&
         ((uintptr_t)p.a & 15) == 0 && ((uintptr_t)p.b & 15) == 0 && p.a_sm > 0 && p.b_sk > 0 && p.a_sm * 2 * kBM < (int64_t(1) << 31) &&
         (int64_t)p.K * p.b_sk * 2 < (int64_t(1) << 31);
}

int launch_nn256(GemmParams p, bool bf16, hipStream_t s) {
  p.tiles_m = (p.M + kBM - 1) / kBM;
  p.tiles_n = (p.N + kBN - 1) / kBN;
  p.split_k = 1;
  // Before the first launch on a device: the runtime must give the kernel the 128 KiB of LDS its loads address.
  static int checked[64];  // 0 not asked, 1 fine, -1 refused (a race between two first calls only repeats the query)
  int dev = -1;
  KAPY_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return fail(KAPY_ERR_UNSUPPORTED, "matmul: device ordinal %d beyond 64", dev);
  int state = __atomic_load_n(&checked[dev], __ATOMIC_ACQUIRE);
  if (state == 0) {
    hipFuncAttributes attr;
    int limit = 0;
    const hipError_t e1 = hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(nn256_kernel<Bf16M16>));
    const hipError_t e2 = hipDeviceGetAttribute(&limit, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
    state = (e1 == hipSuccess && e2 == hipSuccess && (int64_t)attr.sharedSizeBytes == 2 * kStageBytes && limit >= 2 * kStageBytes) ? 1 : -1;
    (void)hipGetLastError();
    __atomic_store_n(&checked[dev], state, __ATOMIC_RELEASE);
  }
  if (state < 0) return fail(KAPY_ERR_HIP, "matmul: the runtime does not give this kernel the %d bytes of LDS it addresses (nothing was launched)", 2 * kStageBytes);
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n), 1);
  const bool tail = p.bias != nullptr || p.act >= 0 || p.alpha != 1.0f;
  if (tail) {
    if (bf16) nn256_kernel<Bf16M16, true><<<grid, 256, 0, s>>>(p);
    else nn256_kernel<F16M16, true><<<grid, 256, 0, s>>>(p);
  } else {
    if (bf16) nn256_kernel<Bf16M16><<<grid, 256, 0, s>>>(p);
    else nn256_kernel<F16M16><<<grid, 256, 0, s>>>(p);
  }
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace kapy
