// probe.hip — what this device sustains, measured by the library itself so that the roofline fractions of its kernels
// can be read against reproducible ceilings instead of data-sheet peaks alone.
//
//   kapy_probe_mfma   every CU runs a loop of nothing but independent matrix instructions, with the register blocking
//                     of the tiled matmul (8 x 8 accumulator blocks of 16x16, or 4 x 4 of 32x32, per wavefront; four
//                     wavefronts per CU) and operands taken from caller memory (the power a matrix instruction draws,
//                     and with it the clock the part holds, depends on the operand values).  No byte moves: the rate
//                     is what the matrix pipes sustain under the power limit.
//   kapy_probe_copy   a 16-byte-per-lane copy in the forms a memory-bound kernel can take (vectors per lane, ordinary or
//                     non-temporal loads and stores, one pass over a big grid or persistent workgroups striding over
//                     the buffer): the rate a read + write stream reaches on this part.
//   kapy_probe_read   the same without the stores: what a kernel that streams an operand and writes little can approach.
//   kapy_probe_l2_read  every CU reads a window that stays in its XCD's L2, over and over: the rate at which the L2s feed
//                     the CUs, which is what a tiled matmul's global->LDS traffic runs against.
//   kapy_mfma_probe   one matrix instruction on one wavefront, registers in and out (binds the exported operand layouts to
//                     the hardware in a test).
// The first two record per-workgroup shader-clock and constant-rate timer ticks, from which the sustained clock follows.
//
// The reference has no counterpart: it emits code and never runs it (its matmul instruction strings:
// lib/Conversion/KgpuToLLVM/MatmulOpToLLVM.cpp:269-311; its loads and stores: LdGlobalOpToLLVM.cpp:60-145).
#include "common.hpp"
#include "mfma.hpp"
#include "kapy_probe.h"

namespace kapy {
namespace {

// ticks[4*wg + 0/1]: shader clock at the start / end of workgroup wg; + 2/3: the constant-rate (100 MHz) timer
__device__ __forceinline__ void stamp(uint64_t *ticks, int which) {
  if (ticks && threadIdx.x == 0) {
    ticks[4 * blockIdx.x + which] = __builtin_readcyclecounter();
    ticks[4 * blockIdx.x + 2 + which] = wall_clock64();
  }
}

template <typename T, bool EXCHANGED>
__global__ __launch_bounds__(256) void mfma_loop_kernel(const char *operands, float *sink, int iterations, uint64_t *ticks) {
  constexpr int kBlocks = T::kM == 16 ? 8 : 4, kRegs = T::kShape.m * T::kShape.n / 64, CH = T::kChunks;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  u32x4 a[kBlocks][CH], b[kBlocks][CH];
#pragma unroll
  for (int i = 0; i < kBlocks; ++i)
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      a[i][c] = *(const u32x4 *)(operands + ((((wave * kBlocks + i) * 2 + 0) * CH + c) * 64 + lane) * 16);
      b[i][c] = *(const u32x4 *)(operands + ((((wave * kBlocks + i) * 2 + 1) * CH + c) * 64 + lane) * 16);
    }
  typename T::Acc acc[kBlocks][kBlocks];
#pragma unroll
  for (int i = 0; i < kBlocks; ++i)
#pragma unroll
    for (int j = 0; j < kBlocks; ++j)
#pragma unroll
      for (int v = 0; v < kRegs; ++v) acc[i][j][v] = 0.f;
  stamp(ticks, 0);
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int i = 0; i < kBlocks; ++i)
#pragma unroll
      for (int j = 0; j < kBlocks; ++j) acc[i][j] = EXCHANGED ? T::mfma(b[j], a[i], acc[i][j]) : T::mfma(a[i], b[j], acc[i][j]);
  }
  stamp(ticks, 1);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kBlocks; ++i)
#pragma unroll
    for (int j = 0; j < kBlocks; ++j)
#pragma unroll
      for (int v = 0; v < kRegs; ++v) s += acc[i][j][v];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

template <typename T>
int launch_mfma_loop(const void *operands, float *sink, int iterations, uint64_t *ticks, int workgroups, hipStream_t s) {
  mfma_loop_kernel<T, true><<<workgroups, 256, 0, s>>>((const char *)operands, sink, iterations, ticks);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

typedef uint32_t vec16 __attribute__((ext_vector_type(4)));
// one pass: workgroup b copies vectors [b*256*U, (b+1)*256*U), lane t the ones at t + u*256
template <int U, bool LNT, bool SNT>
__global__ __launch_bounds__(256) void copy_once_kernel(const vec16 *__restrict__ src, vec16 *__restrict__ dst, int64_t n, uint64_t *ticks) {
  stamp(ticks, 0);
  const int64_t base = (int64_t)blockIdx.x * 256 * U + threadIdx.x;
  vec16 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + (int64_t)u * 256;
    if (i < n) v[u] = LNT ? __builtin_nontemporal_load(src + i) : src[i];
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + (int64_t)u * 256;
    if (i < n) {
      if (SNT) __builtin_nontemporal_store(v[u], dst + i);
      else dst[i] = v[u];
    }
  }
  stamp(ticks, 1);
}
// persistent: gridDim.x workgroups stride over the buffer, U vectors per lane in flight
template <int U, bool LNT, bool SNT>
__global__ __launch_bounds__(256) void copy_stride_kernel(const vec16 *__restrict__ src, vec16 *__restrict__ dst, int64_t n, uint64_t *ticks) {
  stamp(ticks, 0);
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t base = (int64_t)blockIdx.x * 256 + threadIdx.x; base < n; base += stride * U) {
    vec16 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * stride;
      if (i < n) v[u] = LNT ? __builtin_nontemporal_load(src + i) : src[i];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * stride;
      if (i < n) {
        if (SNT) __builtin_nontemporal_store(v[u], dst + i);
        else dst[i] = v[u];
      }
    }
  }
  stamp(ticks, 1);
}

// A copy with the memory footprint of the 16-bit tile transpose: a workgroup owns 128 rows x 256 bytes of a [rows][row_bytes]
// matrix, a lane moves eight 16-byte vectors of eight different rows (rows 16 apart), so that one wave instruction touches
// four 256-byte pieces of four rows - and writes them to the SAME place of the destination (no transposition): what the
// access shape alone costs against one contiguous KiB per instruction.  THROUGH_LDS: the vectors take the detour through
// an LDS tile and a barrier that the transposing kernel needs.
template <bool THROUGH_LDS>
__global__ __launch_bounds__(256) void copy_tiled_kernel(const char *__restrict__ src, char *__restrict__ dst, int64_t row_bytes, uint32_t tiles_x, uint32_t tiles_y) {
  __shared__ __attribute__((aligned(16))) char tile[THROUGH_LDS ? 128 * 256 : 16];
  const int t = threadIdx.x;
  uint32_t bx = blockIdx.x % tiles_x, by = (blockIdx.x / tiles_x + bx) % tiles_y;  // diagonal walk, as the transpose
  const int64_t base = ((int64_t)by * 128 + t / 16) * row_bytes + (int64_t)bx * 256 + (t % 16) * 16;
  vec16 v[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) v[c] = __builtin_nontemporal_load((const vec16 *)(src + base + (int64_t)c * 16 * row_bytes));
  if (THROUGH_LDS) {
#pragma unroll
    for (int c = 0; c < 8; ++c) *(vec16 *)(tile + ((t / 16 + 16 * c) * 256) + (((t % 16) ^ (t / 16)) << 4)) = v[c];
    __syncthreads();
    const int u = (t + 64) % 256;  // read another lane's vectors back
#pragma unroll
    for (int c = 0; c < 8; ++c) v[c] = *(const vec16 *)(tile + ((u / 16 + 16 * c) * 256) + (((u % 16) ^ (u / 16)) << 4));
    const int64_t ubase = ((int64_t)by * 128 + u / 16) * row_bytes + (int64_t)bx * 256 + (u % 16) * 16;
#pragma unroll
    for (int c = 0; c < 8; ++c) __builtin_nontemporal_store(v[c], (vec16 *)(dst + ubase + (int64_t)c * 16 * row_bytes));
  } else {
#pragma unroll
    for (int c = 0; c < 8; ++c) __builtin_nontemporal_store(v[c], (vec16 *)(dst + base + (int64_t)c * 16 * row_bytes));
  }
}

// The same plain copy in pieces of RUN contiguous bytes: a workgroup owns (32 KiB / RUN) rows x RUN bytes of a [rows][row_bytes]
// matrix, 8 vectors of 16 bytes per lane.  What the length of the contiguous runs alone costs: a transposing kernel reads
// and writes runs as long as its tile is wide.
template <int RUN>
__global__ __launch_bounds__(256) void copy_runs_kernel(const char *__restrict__ src, char *__restrict__ dst, int64_t row_bytes, uint32_t tiles_x, uint32_t tiles_y) {
  constexpr int kRows = 32768 / RUN, kLanesPerRow = RUN / 16, kRowsPerPass = 256 / kLanesPerRow;
  static_assert(kRows % 8 == 0 && kRowsPerPass * 8 == kRows, "8 passes over the workgroup's rows");
  const int t = threadIdx.x;
  uint32_t bx = blockIdx.x % tiles_x, by = (blockIdx.x / tiles_x + bx) % tiles_y;  // diagonal walk, as the transpose
  const int64_t base = ((int64_t)by * kRows + t / kLanesPerRow) * row_bytes + (int64_t)bx * RUN + (t % kLanesPerRow) * 16;
  vec16 v[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) v[c] = __builtin_nontemporal_load((const vec16 *)(src + base + (int64_t)c * kRowsPerPass * row_bytes));
#pragma unroll
  for (int c = 0; c < 8; ++c) __builtin_nontemporal_store(v[c], (vec16 *)(dst + base + (int64_t)c * kRowsPerPass * row_bytes));
}

// A read-only stream: every lane folds U vectors of 16 bytes per pass into a word nobody needs (written only for a value the
// fold never takes), in one pass over a big grid or by persistent workgroups striding over the buffer.  What the memory system
// delivers when nothing is written: the ceiling of a kernel that streams a large operand and writes little (a skinny GEMM's
// weight matrix, a reduce).
template <int U, bool NT>
__global__ __launch_bounds__(256) void read_kernel(const vec16 *__restrict__ src, int64_t n, uint32_t *sink) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  uint32_t fold = 0;
  for (int64_t base = (int64_t)blockIdx.x * 256 + threadIdx.x; base < n; base += stride * U) {
    vec16 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * stride;
      v[u] = vec16{0, 0, 0, 0};
      if (i < n) v[u] = NT ? __builtin_nontemporal_load(src + i) : src[i];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) fold ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  if (fold == 0x9e3779b9u && sink) sink[blockIdx.x] = fold;
}
template <int U>
int launch_read(const void *src, int64_t n, int nt, int persistent_per_cu, uint32_t *sink, int32_t *workgroups, hipStream_t s) {
  const int64_t grid = persistent_per_cu > 0 ? (int64_t)device_cus() * persistent_per_cu : (n + 256 * U - 1) / (256 * U);
  if (workgroups) *workgroups = (int32_t)grid;
  if (nt) read_kernel<U, true><<<(unsigned)grid, 256, 0, s>>>((const vec16 *)src, n, sink);
  else read_kernel<U, false><<<(unsigned)grid, 256, 0, s>>>((const vec16 *)src, n, sink);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

template <int U, bool LNT, bool SNT>
int launch_copy(const void *src, void *dst, int64_t n, int persistent_per_cu, uint64_t *ticks, int32_t *workgroups, hipStream_t s) {
  if (persistent_per_cu > 0) {
    const int grid = device_cus() * persistent_per_cu;
    if (workgroups) *workgroups = grid;
    copy_stride_kernel<U, LNT, SNT><<<grid, 256, 0, s>>>((const vec16 *)src, (vec16 *)dst, n, ticks);
  } else {
    const int64_t grid = (n + 256 * U - 1) / (256 * U);
    if (workgroups) *workgroups = (int32_t)grid;
    copy_once_kernel<U, LNT, SNT><<<(unsigned)grid, 256, 0, s>>>((const vec16 *)src, (vec16 *)dst, n, ticks);
  }
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}
// What the L2s hand to the CUs: every workgroup reads, over and over, the window of `src` that belongs to its XCD
// (workgroup ids go to the 8 XCDs in turn; a window is sized to stay in that XCD's L2), 16 bytes per lane and instruction in
// runs of 1 KiB per wave, up to 32 instructions per wave in flight - as LDS-direct loads into a ring nobody reads (the form the
// tiled matmul kernels use) or into registers.  The workgroups of an XCD start a quarter of the window apart, so that at
// any moment they ask for different lines, as the operand panels of neighbouring GEMM tiles are.
template <bool TO_LDS>
__global__ __launch_bounds__(256) void l2_read_kernel(const char *src, int64_t window, int iterations, uint32_t *sink) {
  __shared__ __attribute__((aligned(1024))) char ring[4 * 32 * 1024];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t xcd = blockIdx.x % 8, on_xcd = blockIdx.x / 8;
  const char *base = src + xcd * window;
  const uint32_t chunks = (uint32_t)(window / 1024);  // 1 KiB runs in the window
  uint32_t at = (uint32_t)((on_xcd * 4 + wave) * (chunks / 16) % chunks);
  // (the halves go through unsigned variables: readfirstlane returns an int, and a low half with its top bit set would
  // otherwise be sign-extended over the high half when the two are joined)
  const uint64_t bv = (uint64_t)base;
  const uint32_t base_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)bv), base_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(bv >> 32));
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)base_hi << 32) | (uint64_t)base_lo), 0, (int)window, 0x00020000);
  u32x4 x = {0, 0, 0, 0};
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const uint32_t chunk = __builtin_amdgcn_readfirstlane(at + u < chunks ? at + u : at + u - chunks);
      if (TO_LDS) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)(ring + wave * 32768 + ((it & 3) * 8 + u) * 1024), 16, lane * 16,
                                                 (int)(chunk * 1024), 0, 0);
      } else {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16, (int)(chunk * 1024), 0);
        x ^= v;
      }
    }
    at = at + 8 < chunks ? at + 8 : at + 8 - chunks;
    if (TO_LDS) __builtin_amdgcn_s_waitcnt(0x0F70 | (24 & 15) | ((24 >> 4) << 14));  // vmcnt(24): four groups of eight in flight
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  if (sink && (x[0] ^ x[1] ^ x[2] ^ x[3]) == 0x9e3779b9u) sink[blockIdx.x] = x[0];  // keeps the register form's loads alive
}

// What a wave can issue beside its matrix instructions.  One wave per SIMD (the tiled matmul's occupancy) runs `iterations`
// tiles of kTileClocks of independent matrix instructions - 128 x 16x16x32 (16 clocks each) or 64 x 16x16x128 (32 clocks) - and
// in the gap behind every instruction FILL asks for: 1 = COUNT scalar instructions (s_nop), 2 = COUNT vector ALU instructions
// (v_mov), 3 = the steady-state loop of the tiled matmul: 32 LDS reads of 16 bytes per lane and 16 LDS-direct loads of 1 KiB
// per wave and tile, spread evenly and never in the same gap, from a window of 2 MiB per XCD that stays in the L2; 4 = that loop
// with the rhs kept off the LDS (16 LDS reads, 8 LDS-direct loads and 16 loads of 16 bytes per lane into registers per tile).
// MF: 0 = bf16 16x16x32, 1 = e4m3 16x16x128.
typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
template <int MF, int FILL, int COUNT>
__global__ __launch_bounds__(256) void issue_kernel(const char *src, int iterations, float *sink) {
  __shared__ __attribute__((aligned(1024))) char ring[128 * 1024];  // (with 128 KiB a workgroup has its CU to itself)
  constexpr int kMfmas = MF ? 64 : 128, kReadEvery = kMfmas / 32, kLoadEvery = kMfmas / 16;
  constexpr uint32_t kWindow = 2u << 20, kChunksInWindow = kWindow / 1024;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint64_t bv = (uint64_t)(src + (uint64_t)(blockIdx.x % 8) * kWindow);
  const uint32_t base_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)bv), base_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(bv >> 32));
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(((uint64_t)base_hi << 32) | (uint64_t)base_lo), 0, (int)kWindow, 0x00020000);
  uint32_t at = (uint32_t)(((blockIdx.x / 8) * 4 + wave) * (kChunksInWindow / 128) % kChunksInWindow);
  f32x4 acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const u32x8 op8 = {0x38383838u + lane, 0x38383838u, 0x38383838u, 0x38383838u, 0x38383838u, 0x38383838u, 0x38383838u, 0x38383838u};
  const u32x4 op4 = {0x3c003c00u + lane, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
  const uint32_t unit = 0x7f7f7f7fu, lds_rd = (uint32_t)(uintptr_t)ring + wave * 32768 + lane * 16, voff = lane * 16;
  uint32_t filler = lane;
  u32x4 r[8];
  [[maybe_unused]] u32x4 regs[16];
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int g = 0; g < kMfmas; ++g) {
      if constexpr (MF) asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0] cbsz:0 blgp:0" : "+a"(acc[g % 16]) : "v"(op8), "v"(op8), "v"(unit));
      else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[g % 16]) : "v"(op4), "v"(op4));
      if (g % (FILL == 4 ? kMfmas / 8 : kLoadEvery) != 0) __builtin_amdgcn_sched_barrier(0);  // (a load's M0 write may move ahead of the matrix instruction)
      if constexpr (FILL == 1) {
#pragma unroll
        for (int f = 0; f < COUNT; ++f) asm volatile("s_nop 0");
      }
      if constexpr (FILL == 2) {
#pragma unroll
        for (int f = 0; f < COUNT; ++f) asm volatile("v_mov_b32 %0, %1" : "=v"(filler) : "v"(lane));
      }
      if constexpr (FILL == 3) {
        if (g % kReadEvery == 0 && g % kLoadEvery != 0) {  // (the read that would share a load's gap goes one gap on)
          asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[(g / kReadEvery) % 8]) : "v"(lds_rd), "n"(((g / kReadEvery) % 16) * 1024));
        } else if (g % kLoadEvery == 1) {
          asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[(g / kReadEvery) % 8]) : "v"(lds_rd), "n"(((g / kReadEvery) % 16) * 1024));
        }
        if (g % kLoadEvery == 0) {
          const int k = g / kLoadEvery;
          const uint32_t chunk = at + k < kChunksInWindow ? at + k : at + k - kChunksInWindow;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)(ring + wave * 32768 + 16384 + k * 1024), 16, voff,
                                                   (int)(chunk * 1024), 0, 0);
        }
      }
      if constexpr (FILL == 4) {
        // one operand off the LDS: 16 LDS reads and 8 LDS-direct loads for the lhs half of the tile, and the wave's 16 rhs
        // fragments of the tile as 16-byte loads into registers (lane l: row l % 16 of a 16 KiB-pitch panel, bytes
        // 32 * (l / 16) .. + 32 of a 128-byte piece, as two loads), issued over the first half of the tile
        constexpr int kDirectEvery = kMfmas / 8, kLdsEvery = kMfmas / 16, kRegEvery = kMfmas / 32;
        if (g % kDirectEvery == 0) {
          const int k = g / kDirectEvery;
          const uint32_t chunk = at + k < kChunksInWindow ? at + k : at + k - kChunksInWindow;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)(ring + wave * 32768 + 16384 + k * 1024), 16, voff,
                                                   (int)(chunk * 1024), 0, 0);
        } else if (g % kLdsEvery == kLdsEvery / 2) {
          asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r[(g / kLdsEvery) % 8]) : "v"(lds_rd), "n"(((g / kLdsEvery) % 16) * 1024));
        } else if (g % kRegEvery == 1 && g < kMfmas / 2) {
          const int j = g / kRegEvery;  // 0 .. 15: row group j / 2, half j % 2
          regs[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (lane & 15) * 16384 + (lane >> 4) * 32 + (j & 1) * 16,
                                                          (int)((j >> 1) * 16 * 16384 + (at * 128u) % 16384u), 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (FILL == 4) {
      at = at + 8 < kChunksInWindow ? at + 8 : at + 8 - kChunksInWindow;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int k = 0; k < 8; ++k) asm volatile("" ::"v"(r[k]));
#pragma unroll
      for (int j = 0; j < 16; ++j) asm volatile("" ::"v"(regs[j]));  // (the compiler waits here for the register loads; the four LDS-direct loads behind them stay in flight)
    }
    if constexpr (FILL == 3) {
      at = at + 16 < kChunksInWindow ? at + 16 : at + 16 - kChunksInWindow;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int k = 0; k < 8; ++k) asm volatile("" ::"v"(r[k]));
      __builtin_amdgcn_s_waitcnt(0x0F70 | (16 & 15) | ((16 >> 4) << 14));  // vmcnt(16): the previous tile's loads have landed
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");  // (the compiler does not see the in-place matrix instructions' results coming)
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i];
  if (s[0] + s[1] + s[2] + s[3] == 12345.f) sink[blockIdx.x * 256 + threadIdx.x] = s[0] + (float)filler;
}

template <int MF>
int launch_issue(int filler, int count, const char *src, int iterations, float *sink, int wgs, hipStream_t s) {
#define KAPY_ISSUE(F, C) issue_kernel<MF, F, C><<<wgs, 256, 0, s>>>(src, iterations, sink)
  if (filler == 0) KAPY_ISSUE(0, 0);
  else if (filler == 3) KAPY_ISSUE(3, 0);
  else if (filler == 4) KAPY_ISSUE(4, 0);
  else if (filler == 1 && count == 1) KAPY_ISSUE(1, 1);
  else if (filler == 1 && count == 2) KAPY_ISSUE(1, 2);
  else if (filler == 1 && count == 3) KAPY_ISSUE(1, 3);
  else if (filler == 1 && count == 4) KAPY_ISSUE(1, 4);
  else if (filler == 1 && count == 6) KAPY_ISSUE(1, 6);
  else if (filler == 1 && count == 8) KAPY_ISSUE(1, 8);
  else if (filler == 2 && count == 1) KAPY_ISSUE(2, 1);
  else if (filler == 2 && count == 2) KAPY_ISSUE(2, 2);
  else if (filler == 2 && count == 3) KAPY_ISSUE(2, 3);
  else if (filler == 2 && count == 4) KAPY_ISSUE(2, 4);
  else return fail(KAPY_ERR_INVALID, "probe_issue: filler 0 (none), 1 (scalar; count 1, 2, 3, 4, 6 or 8), 2 (vector ALU; count 1 .. 4), 3 (the tiled matmul's reads and loads) or 4 (the same with the rhs loaded into registers)");
#undef KAPY_ISSUE
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

template <int U>
int launch_copy_nt(const void *src, void *dst, int64_t n, int nt_load, int nt_store, int persistent_per_cu, uint64_t *ticks, int32_t *workgroups, hipStream_t s) {
  if (nt_load && nt_store) return launch_copy<U, true, true>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
  if (nt_load) return launch_copy<U, true, false>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
  if (nt_store) return launch_copy<U, false, true>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
  return launch_copy<U, false, false>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
}

// One matrix instruction on one wavefront, registers in and registers out: lhs / rhs hold each lane's operand
// registers back to back (kpack elements per lane), acc gets each lane's accumulator registers.  The policy is
// the one the kernels multiply with, so what this shows about register positions holds for them.
template <typename T, bool EXCHANGED>
__global__ __launch_bounds__(64) void probe_kernel(const char *lhs, const char *rhs, float *acc) {
  const int lane = threadIdx.x;
  constexpr int kLaneBytes = T::kShape.kpack * T::kBytes, kRegs = T::kShape.m * T::kShape.n / 64;
  static_assert(kLaneBytes == 16 * T::kChunks, "a lane's operand registers are whole 16-byte chunks");
  u32x4 a[T::kChunks], b[T::kChunks];
#pragma unroll
  for (int c = 0; c < T::kChunks; ++c) {
    a[c] = *(const u32x4 *)(lhs + lane * kLaneBytes + 16 * c);
    b[c] = *(const u32x4 *)(rhs + lane * kLaneBytes + 16 * c);
  }
  typename T::Acc d;
#pragma unroll
  for (int v = 0; v < kRegs; ++v) d[v] = 0.f;
  d = EXCHANGED ? T::mfma(b, a, d) : T::mfma(a, b, d);
#pragma unroll
  for (int v = 0; v < kRegs; ++v) acc[lane * kRegs + v] = d[v];
}
template <typename T>
int launch_probe(bool exchanged, const void *lhs, const void *rhs, float *acc, hipStream_t s) {
  if (exchanged) probe_kernel<T, true><<<1, 64, 0, s>>>((const char *)lhs, (const char *)rhs, acc);
  else probe_kernel<T, false><<<1, 64, 0, s>>>((const char *)lhs, (const char *)rhs, acc);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}
// FIRST / SECOND: the fp8 formats of the instruction's first / second operand slot
template <template <int, int> class P>
int launch_probe_f8(int first_fmt, int second_fmt, bool exchanged, const void *lhs, const void *rhs, float *acc, hipStream_t s) {
  switch (first_fmt * 2 + second_fmt) {
  case 0: return launch_probe<P<0, 0>>(exchanged, lhs, rhs, acc, s);
  case 1: return launch_probe<P<0, 1>>(exchanged, lhs, rhs, acc, s);
  case 2: return launch_probe<P<1, 0>>(exchanged, lhs, rhs, acc, s);
  default: return launch_probe<P<1, 1>>(exchanged, lhs, rhs, acc, s);
  }
}

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" {

int kapy_mfma_probe(int32_t impl_way, int32_t lhs_dtype, int32_t rhs_dtype, int32_t exchanged, const void *lhs_regs, const void *rhs_regs,
                    float *acc_regs, void *stream) {
  if (!lhs_regs || !rhs_regs || !acc_regs) return fail(KAPY_ERR_INVALID, "mfma_probe: null register array");
  const bool f8 = is_f8(lhs_dtype) && is_f8(rhs_dtype), b16 = (lhs_dtype == KAPY_F16 || lhs_dtype == KAPY_BF16) && rhs_dtype == lhs_dtype;
  const bool way16 = impl_way == KAPY_MFMA_32X32X16_16B || impl_way == KAPY_MFMA_16X16X32_16B;
  const bool way8 = impl_way == KAPY_MFMA_16X16X128_F8 || impl_way == KAPY_MFMA_32X32X64_F8;
  if (!way16 && !way8) return fail(KAPY_ERR_INVALID, "mfma_probe: impl_way must name a matrix instruction of gfx950 (16..19), not %d", impl_way);
  if ((way16 && !b16) || (way8 && !f8)) return fail(KAPY_ERR_VERIFY, "mfma_probe: operand element types do not fit the instruction");
  int rc = ensure_device();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  const bool ex = exchanged != 0;
  if (way16) {
    const bool bf = lhs_dtype == KAPY_BF16;
    if (impl_way == KAPY_MFMA_32X32X16_16B) return bf ? launch_probe<Bf16>(ex, lhs_regs, rhs_regs, acc_regs, s) : launch_probe<F16>(ex, lhs_regs, rhs_regs, acc_regs, s);
    return bf ? launch_probe<Bf16M16>(ex, lhs_regs, rhs_regs, acc_regs, s) : launch_probe<F16M16>(ex, lhs_regs, rhs_regs, acc_regs, s);
  }
  // exchanged: the rhs fragment sits in the first operand slot, so the first format selector is the rhs's
  const int lf = lhs_dtype == KAPY_F8E5M2, rf = rhs_dtype == KAPY_F8E5M2;
  const int first = ex ? rf : lf, second = ex ? lf : rf;
  if (impl_way == KAPY_MFMA_16X16X128_F8) return launch_probe_f8<F8M16>(first, second, ex, lhs_regs, rhs_regs, acc_regs, s);
  return launch_probe_f8<F8>(first, second, ex, lhs_regs, rhs_regs, acc_regs, s);
}


int kapy_probe_mfma(int32_t impl_way, int32_t dtype, const void *operands, int32_t iterations, float *sink, uint64_t *ticks, int32_t *workgroups,
                    int64_t *flops, void *stream) {
  if (!operands || !sink || iterations <= 0) return fail(KAPY_ERR_INVALID, "probe_mfma: null buffer or no iterations");
  int rc = ensure_device();
  if (rc) return rc;
  const int wgs = device_cus();  // four wavefronts with 256 accumulator registers each: one workgroup fills a CU
  if (workgroups) *workgroups = wgs;
  hipStream_t s = (hipStream_t)stream;
  int m = 0, k = 0, blocks = 0;
  switch (impl_way) {
  case KAPY_MFMA_32X32X16_16B: m = 32; k = 16; blocks = 4; break;
  case KAPY_MFMA_16X16X32_16B: m = 16; k = 32; blocks = 8; break;
  case KAPY_MFMA_16X16X128_F8: m = 16; k = 128; blocks = 8; break;
  case KAPY_MFMA_32X32X64_F8: m = 32; k = 64; blocks = 4; break;
  default: return fail(KAPY_ERR_INVALID, "probe_mfma: impl_way must name a matrix instruction of gfx950 (16..19), not %d", impl_way);
  }
  if (flops) *flops = (int64_t)wgs * 4 * iterations * blocks * blocks * 2 * m * m * k;
  const bool b16 = dtype == KAPY_F16 || dtype == KAPY_BF16;
  if ((impl_way <= KAPY_MFMA_16X16X32_16B) != b16 || (!b16 && !is_f8(dtype))) return fail(KAPY_ERR_VERIFY, "probe_mfma: element type does not fit the instruction");
  switch (impl_way) {
  case KAPY_MFMA_32X32X16_16B: return dtype == KAPY_BF16 ? launch_mfma_loop<Bf16>(operands, sink, iterations, ticks, wgs, s) : launch_mfma_loop<F16>(operands, sink, iterations, ticks, wgs, s);
  case KAPY_MFMA_16X16X32_16B: return dtype == KAPY_BF16 ? launch_mfma_loop<Bf16M16>(operands, sink, iterations, ticks, wgs, s) : launch_mfma_loop<F16M16>(operands, sink, iterations, ticks, wgs, s);
  case KAPY_MFMA_16X16X128_F8: return dtype == KAPY_F8E4M3 ? launch_mfma_loop<F8M16<0, 0>>(operands, sink, iterations, ticks, wgs, s) : launch_mfma_loop<F8M16<1, 1>>(operands, sink, iterations, ticks, wgs, s);
  default: return dtype == KAPY_F8E4M3 ? launch_mfma_loop<F8<0, 0>>(operands, sink, iterations, ticks, wgs, s) : launch_mfma_loop<F8<1, 1>>(operands, sink, iterations, ticks, wgs, s);
  }
}

int kapy_probe_l2_read(const void *src, int64_t window_bytes, int32_t iterations, int32_t workgroups_per_cu, int32_t to_lds, uint32_t *sink,
                       int32_t *workgroups, int64_t *bytes_read, void *stream) {
  if (!src || window_bytes < 16384 || window_bytes % 16384 || window_bytes > (int64_t(1) << 30) || iterations <= 0 || workgroups_per_cu < 1 || workgroups_per_cu > 4 ||
      ((uintptr_t)src & 1023))
    return fail(KAPY_ERR_INVALID, "probe_l2_read: window must be a multiple of 16 KiB (at most 1 GiB), src 1 KiB aligned, 1 .. 4 workgroups per CU");
  int rc = ensure_device();
  if (rc) return rc;
  const int wgs = device_cus() * workgroups_per_cu;
  if (workgroups) *workgroups = wgs;
  if (bytes_read) *bytes_read = (int64_t)wgs * 4 * iterations * 8 * 1024;
  if (to_lds) l2_read_kernel<true><<<wgs, 256, 0, (hipStream_t)stream>>>((const char *)src, window_bytes, iterations, sink);
  else l2_read_kernel<false><<<wgs, 256, 0, (hipStream_t)stream>>>((const char *)src, window_bytes, iterations, sink);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int kapy_probe_issue(int32_t impl_way, int32_t filler, int32_t count, const void *src, int32_t iterations, float *sink, int32_t *workgroups, int64_t *flops,
                     void *stream) {
  if (!sink || iterations <= 0 || (filler == 3 && !src)) return fail(KAPY_ERR_INVALID, "probe_issue: null buffer or no iterations");
  if (impl_way != KAPY_MFMA_16X16X32_16B && impl_way != KAPY_MFMA_16X16X128_F8) return fail(KAPY_ERR_INVALID, "probe_issue: 16x16x32 (16-bit) or 16x16x128 (f8) only");
  int rc = ensure_device();
  if (rc) return rc;
  const int wgs = device_cus();
  if (workgroups) *workgroups = wgs;
  const bool f8 = impl_way == KAPY_MFMA_16X16X128_F8;
  if (flops) *flops = (int64_t)wgs * 4 * iterations * (f8 ? 64 : 128) * (f8 ? 65536 : 16384);
  return f8 ? launch_issue<1>(filler, count, (const char *)src, iterations, sink, wgs, (hipStream_t)stream)
            : launch_issue<0>(filler, count, (const char *)src, iterations, sink, wgs, (hipStream_t)stream);
}

int kapy_probe_copy_tiled(const void *src, void *dst, int64_t rows, int64_t row_bytes, int32_t through_lds, void *stream) {
  if (!src || !dst || rows <= 0 || rows % 128 || row_bytes <= 0 || row_bytes % 256 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
    return fail(KAPY_ERR_INVALID, "probe_copy_tiled: rows must be a multiple of 128, row_bytes of 256, buffers 16-byte aligned");
  int rc = ensure_device();
  if (rc) return rc;
  const uint32_t tx = (uint32_t)(row_bytes / 256), ty = (uint32_t)(rows / 128);
  if (through_lds) copy_tiled_kernel<true><<<tx * ty, 256, 0, (hipStream_t)stream>>>((const char *)src, (char *)dst, row_bytes, tx, ty);
  else copy_tiled_kernel<false><<<tx * ty, 256, 0, (hipStream_t)stream>>>((const char *)src, (char *)dst, row_bytes, tx, ty);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int kapy_probe_copy_runs(const void *src, void *dst, int64_t rows, int64_t row_bytes, int32_t run_bytes, void *stream) {
  if (!src || !dst || rows <= 0 || row_bytes <= 0 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
    return fail(KAPY_ERR_INVALID, "probe_copy_runs: null or misaligned buffer, or an empty matrix");
  if (run_bytes != 256 && run_bytes != 512 && run_bytes != 1024 && run_bytes != 2048 && run_bytes != 4096)
    return fail(KAPY_ERR_INVALID, "probe_copy_runs: runs of 256, 512, 1024, 2048 or 4096 bytes");
  if (row_bytes % run_bytes || rows % (32768 / run_bytes))
    return fail(KAPY_ERR_INVALID, "probe_copy_runs: row_bytes must be a multiple of the run, rows of 32768 / run");
  int rc = ensure_device();
  if (rc) return rc;
  const uint32_t tx = (uint32_t)(row_bytes / run_bytes), ty = (uint32_t)(rows / (32768 / run_bytes));
  hipStream_t s = (hipStream_t)stream;
  switch (run_bytes) {
  case 256: copy_runs_kernel<256><<<tx * ty, 256, 0, s>>>((const char *)src, (char *)dst, row_bytes, tx, ty); break;
  case 512: copy_runs_kernel<512><<<tx * ty, 256, 0, s>>>((const char *)src, (char *)dst, row_bytes, tx, ty); break;
  case 1024: copy_runs_kernel<1024><<<tx * ty, 256, 0, s>>>((const char *)src, (char *)dst, row_bytes, tx, ty); break;
  case 2048: copy_runs_kernel<2048><<<tx * ty, 256, 0, s>>>((const char *)src, (char *)dst, row_bytes, tx, ty); break;
  default: copy_runs_kernel<4096><<<tx * ty, 256, 0, s>>>((const char *)src, (char *)dst, row_bytes, tx, ty); break;
  }
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int kapy_probe_copy(const void *src, void *dst, int64_t bytes, int32_t vectors_per_lane, int32_t nt_load, int32_t nt_store, int32_t persistent_per_cu,
                    uint64_t *ticks, int32_t *workgroups, void *stream) {
  if (!src || !dst || bytes <= 0 || bytes % 16 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15))
    return fail(KAPY_ERR_INVALID, "probe_copy: buffers must be 16-byte aligned and a whole number of 16-byte vectors long");
  if (persistent_per_cu < 0 || persistent_per_cu > 64) return fail(KAPY_ERR_INVALID, "probe_copy: persistent workgroups per CU must be 0 (one pass) .. 64");
  int rc = ensure_device();
  if (rc) return rc;
  const int64_t n = bytes / 16;
  hipStream_t s = (hipStream_t)stream;
  switch (vectors_per_lane) {
  case 1: return launch_copy_nt<1>(src, dst, n, nt_load, nt_store, persistent_per_cu, ticks, workgroups, s);
  case 2: return launch_copy_nt<2>(src, dst, n, nt_load, nt_store, persistent_per_cu, ticks, workgroups, s);
  case 4: return launch_copy_nt<4>(src, dst, n, nt_load, nt_store, persistent_per_cu, ticks, workgroups, s);
  case 8: return launch_copy_nt<8>(src, dst, n, nt_load, nt_store, persistent_per_cu, ticks, workgroups, s);
  case 16: return launch_copy_nt<16>(src, dst, n, nt_load, nt_store, persistent_per_cu, ticks, workgroups, s);
  }
  return fail(KAPY_ERR_INVALID, "probe_copy: vectors per lane must be 1, 2, 4, 8 or 16");
}

int kapy_probe_read(const void *src, int64_t bytes, int32_t vectors_per_lane, int32_t nt_load, int32_t persistent_per_cu, uint32_t *sink, int32_t *workgroups,
                    void *stream) {
  if (!src || bytes <= 0 || bytes % 16 || ((uintptr_t)src & 15)) return fail(KAPY_ERR_INVALID, "probe_read: the buffer must be 16-byte aligned and a whole number of 16-byte vectors long");
  if (persistent_per_cu < 0 || persistent_per_cu > 64) return fail(KAPY_ERR_INVALID, "probe_read: persistent workgroups per CU must be 0 (one pass) .. 64");
  int rc = ensure_device();
  if (rc) return rc;
  const int64_t n = bytes / 16;
  if ((n + 255) / 256 > 0x7fffffff) return fail(KAPY_ERR_UNSUPPORTED, "probe_read: buffer too large for one launch");
  hipStream_t s = (hipStream_t)stream;
  switch (vectors_per_lane) {
  case 1: return launch_read<1>(src, n, nt_load, persistent_per_cu, sink, workgroups, s);
  case 2: return launch_read<2>(src, n, nt_load, persistent_per_cu, sink, workgroups, s);
  case 4: return launch_read<4>(src, n, nt_load, persistent_per_cu, sink, workgroups, s);
  case 8: return launch_read<8>(src, n, nt_load, persistent_per_cu, sink, workgroups, s);
  case 16: return launch_read<16>(src, n, nt_load, persistent_per_cu, sink, workgroups, s);
  }
  return fail(KAPY_ERR_INVALID, "probe_read: vectors per lane must be 1, 2, 4, 8 or 16");
}

}  // extern "C"
