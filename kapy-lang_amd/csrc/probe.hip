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
//   kapy_probe_l2_read  every CU reads a window that stays in its XCD's L2, over and over: the rate at which the L2s feed
//                     the CUs, which is what a tiled matmul's global->LDS traffic runs against.
// The first two record per-workgroup shader-clock and constant-rate timer ticks, from which the sustained clock follows.
//
// The reference has no counterpart: it emits code and never runs it (its matmul instruction strings:
// lib/Conversion/KgpuToLLVM/MatmulOpToLLVM.cpp:269-311; its loads and stores: LdGlobalOpToLLVM.cpp:60-145).
#include "common.hpp"
#include "mfma.hpp"

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

template <int U>
int launch_copy_nt(const void *src, void *dst, int64_t n, int nt_load, int nt_store, int persistent_per_cu, uint64_t *ticks, int32_t *workgroups, hipStream_t s) {
  if (nt_load && nt_store) return launch_copy<U, true, true>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
  if (nt_load) return launch_copy<U, true, false>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
  if (nt_store) return launch_copy<U, false, true>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
  return launch_copy<U, false, false>(src, dst, n, persistent_per_cu, ticks, workgroups, s);
}

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" {

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

}  // extern "C"
