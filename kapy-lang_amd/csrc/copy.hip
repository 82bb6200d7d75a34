// copy.hip — ld_global -> [transpose] -> st_global over whole views: the affine-map-described
// layout moves of kapy (strided copies, (i,j)->(j,i) transposes, batched permutes).
//
// Reference semantics: LdGlobalOpToLLVM.cpp:60-145 (addressing, unsigned-compare predicate,
// padding pre-initialisation), StGlobalOpToLLVM.cpp:60-139, TransposeOpToLLVM.cpp:21-26 (a
// transpose is a relabel of the register layout: values never pass through an FP unit), and the
// lane re-distribution of ChangeOpToLLVM.cpp:43-78 for the in-register transpose.
//
// Three kernels, chosen from the descriptor strides:
//   rows_kernel       source and destination contiguous along the same axis: 16-byte vectors,
//                     consecutive lanes on consecutive vectors, every byte read and written once.
//   transpose_kernel  contiguous axes differ: a wavefront owns a (8V x 8V) tile (V = elements per
//                     16 bytes).  Each lane loads a V x V block as V 16-byte vectors along the
//                     source's contiguous axis, transposes it in registers, then the 8x8 grid of
//                     lanes is itself transposed with ds_bpermute so that consecutive lanes again
//                     hold consecutive 16-byte vectors for the store.  Both sides of HBM see full
//                     128-byte segments; no LDS allocation, no barrier.
//   generic_kernel    anything else (no contiguous axis, misaligned rows): one element per lane.
#include "common.hpp"

constexpr int kTransposeMap = 2;  // workgroup -> tile order of the transposes: 0 row by row, 1 column by column, 2 diagonal

namespace kapy {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// All quantities are in the destination's index space (i over d0, j over d1) after the host has
// folded the transpose flag into the source strides; strides are in elements.
struct CopyParams {
  const char *src;
  char *dst;
  int64_t es0, es1;  // source element strides along i and j
  int64_t ds0, ds1;  // destination element strides
  int32_t d0, d1;    // destination extent: elements outside are not written
  int32_t sb0, sb1;  // source bounds: elements at i >= sb0 or j >= sb1 read as padding
  uint32_t pad;      // 32-bit padding word (element pattern replicated)
  int32_t n1;        // second grid dimension; program (p0,p1) = (z / n1, z % n1)
  int32_t map_mode;  // transpose kernel: how workgroup ids walk the tile grid
  int64_t s_off0, s_off1, d_off0, d_off1;  // per-program displacement in elements
};

template <int B> struct ElemOf;
template <> struct ElemOf<1> { typedef uint8_t type; };
template <> struct ElemOf<2> { typedef uint16_t type; };
template <> struct ElemOf<4> { typedef uint32_t type; };

template <int B>
__device__ __forceinline__ void program_base(const CopyParams &p, const char *&src, char *&dst) {
  int32_t z = blockIdx.z, p0 = z / p.n1, p1 = z - p0 * p.n1;
  src = p.src + (p0 * p.s_off0 + p1 * p.s_off1) * B;
  dst = p.dst + (p0 * p.d_off0 + p1 * p.d_off1) * B;
}

template <int B>
__device__ __forceinline__ void copy_one(const CopyParams &p, const char *src, char *dst, int32_t i, int32_t j) {
  typedef typename ElemOf<B>::type T;
  if (i >= p.d0 || j >= p.d1) return;
  T v = (T)p.pad;
  if (i < p.sb0 && j < p.sb1) v = *(const T *)(src + (i * p.es0 + j * p.es1) * B);
  *(T *)(dst + (i * p.ds0 + j * p.ds1) * B) = v;
}

// A transposing move no vector kernel takes (extents that are not multiples of 8, rows that are not 16-byte aligned):
// 64 x 64 tiles through LDS, element by element, lanes along the source's contiguous axis (i) when reading and along the
// destination's (j) when writing, so that both sides see runs of 64 elements where generic_kernel strides one of them.
template <int B>
__global__ __launch_bounds__(256) void transpose_any_kernel(CopyParams p) {
  typedef typename ElemOf<B>::type T;
  __shared__ T tile[64][65];
  const char *src;
  char *dst;
  program_base<B>(p, src, dst);
  const int32_t ti = blockIdx.x * 64, tj = blockIdx.y * 64;
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
#pragma unroll 4
  for (int r = 0; r < 16; ++r) {
    const int32_t i = ti + lane, j = tj + q + 4 * r;
    T v = (T)p.pad;
    if (i < p.d0 && j < p.d1 && i < p.sb0 && j < p.sb1) v = *(const T *)(src + ((int64_t)i * p.es0 + (int64_t)j * p.es1) * B);
    tile[q + 4 * r][lane] = v;
  }
  __syncthreads();
#pragma unroll 4
  for (int r = 0; r < 16; ++r) {
    const int32_t i = ti + q + 4 * r, j = tj + lane;
    if (i < p.d0 && j < p.d1) *(T *)(dst + ((int64_t)i * p.ds0 + (int64_t)j * p.ds1) * B) = tile[lane][q + 4 * r];
  }
}

// ---------------------------------------------------------------------------------------------
template <int B>
__global__ __launch_bounds__(256) void generic_kernel(CopyParams p, int j_fastest) {
  const char *src;
  char *dst;
  program_base<B>(p, src, dst);
  int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int64_t total = (int64_t)p.d0 * p.d1;
  if (t >= total) return;
  int32_t i, j;
  if (j_fastest) { i = (int32_t)(t / p.d1); j = (int32_t)(t - (int64_t)i * p.d1); }
  else { j = (int32_t)(t / p.d0); i = (int32_t)(t - (int64_t)j * p.d0); }
  copy_one<B>(p, src, dst, i, j);
}

// ---------------------------------------------------------------------------------------------
// Rows: es1 == ds1 == 1.  A slot is one VB-byte vector of one row; a thread serves UNROLL slots a
// block-stride apart, all loads issued before the first store.
template <int VB> struct VecOf;
template <> struct VecOf<16> { typedef u32x4 type; };
template <> struct VecOf<8> { typedef u32x2 type; };
template <> struct VecOf<4> { typedef uint32_t type; };

template <int B, int VB, bool NT, bool RAGGED>
__global__ __launch_bounds__(256) void rows_kernel(CopyParams p, int32_t vec_per_row) {
  typedef typename VecOf<VB>::type Vec;
  constexpr int E = VB / B;  // elements per vector
  constexpr int UNROLL = 1;  // vectors per lane (more in flight per lane measured slower: the plain-copy probe has the figures)
  const char *src;
  char *dst;
  program_base<B>(p, src, dst);
  const uint32_t total = (uint32_t)p.d0 * (uint32_t)vec_per_row;  // the host keeps this below 2^31
  const uint32_t first = blockIdx.x * (256 * UNROLL) + threadIdx.x;
  Vec v[UNROLL];
  int32_t row[UNROLL], col[UNROLL];
  bool whole[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    uint32_t slot = first + u * 256;
    row[u] = -1;
    whole[u] = false;
    if (slot < total) {
      row[u] = (int32_t)(slot / (uint32_t)vec_per_row);
      col[u] = (int32_t)(slot - (uint32_t)row[u] * (uint32_t)vec_per_row) * E;
      whole[u] = !RAGGED || (row[u] < p.sb0 && col[u] + E <= p.sb1 && col[u] + E <= p.d1);
      if (whole[u]) {
        const Vec *s = (const Vec *)(src + ((int64_t)row[u] * p.es0 + col[u]) * B);
        v[u] = NT ? __builtin_nontemporal_load(s) : *s;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    if (row[u] < 0) continue;
    if (whole[u]) {
      Vec *d = (Vec *)(dst + ((int64_t)row[u] * p.ds0 + col[u]) * B);
      if (NT) __builtin_nontemporal_store(v[u], d);
      else *d = v[u];
    } else {
#pragma unroll 1
      for (int e = 0; e < E; ++e) copy_one<B>(p, src, dst, row[u], col[u] + e);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Transpose: es0 == 1 (source contiguous along i) and ds1 == 1 (destination contiguous along j).
template <int B, bool NT>
__global__ __launch_bounds__(256) void transpose_kernel(CopyParams p) {
  typedef typename ElemOf<B>::type T;
  constexpr int V = 16 / B;  // lane block is V x V elements
  constexpr int TILE = 8 * V;
  const char *src;
  char *dst;
  program_base<B>(p, src, dst);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  // Workgroup id -> 2x2 block of wave tiles.  mode 0: x walks the source's contiguous axis; 1: x walks
  // the destination's; 2: diagonal (consecutive workgroups differ in both), which spreads the
  // pitch-strided side of the transpose over the memory channels.
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  if (p.map_mode == 1) {
    uint32_t lin = by * gridDim.x + bx;
    by = lin % gridDim.y;
    bx = lin / gridDim.y;
  } else if (p.map_mode == 2) {
    by = (by + bx) % gridDim.y;
  }
  const int32_t ti = (bx * 2 + (wave & 1)) * TILE;
  const int32_t tj = (by * 2 + (wave >> 1)) * TILE;
  if (ti >= p.d0 || tj >= p.d1) return;
  const bool interior = ti + TILE <= p.d0 && ti + TILE <= p.sb0 && tj + TILE <= p.d1 && tj + TILE <= p.sb1;
  if (!interior) {  // ragged edge: element-wise with the ld/st predicates
    for (int e = lane; e < TILE * TILE; e += 64) copy_one<B>(p, src, dst, ti + e / TILE, tj + e % TILE);
    return;
  }
  const int la = lane & 7, lb = lane >> 3;
  union Block {
    u32x4 vec[V];
    T el[V][V];
  };
  Block in, out;
  const char *s = src + ((int64_t)(ti + V * la) + (int64_t)(tj + V * lb) * p.es1) * B;
#pragma unroll
  for (int c = 0; c < V; ++c) {
    const u32x4 *ptr = (const u32x4 *)(s + (int64_t)c * p.es1 * B);
    in.vec[c] = NT ? __builtin_nontemporal_load(ptr) : *ptr;
  }
  // in.el[c][r] = S(i = ti + V*la + r, j = tj + V*lb + c)  ->  out.el[r][c]
#pragma unroll
  for (int r = 0; r < V; ++r)
#pragma unroll
    for (int c = 0; c < V; ++c) out.el[r][c] = in.el[c][r];
  // Transpose the 8x8 grid of lanes: lane (la', lb') takes the block of lane (la = lb', lb = la'),
  // i.e. the registers of source lane lb' ... the same permutation kgpu.change would derive for
  // <[8,8],[V,V],(0,1)> -> <[8,8],[V,V],(1,0)> on the transposed tile.
  const int from = (la << 3) | lb;
#pragma unroll
  for (int r = 0; r < V; ++r)
#pragma unroll
    for (int w = 0; w < 4; ++w) out.vec[r][w] = (uint32_t)__builtin_amdgcn_ds_bpermute(from << 2, (int)out.vec[r][w]);
  // now this lane holds rows i = ti + V*lb + r, columns tj + V*la .. + V-1
  char *d = dst + ((int64_t)(ti + V * lb) * p.ds0 + (int64_t)(tj + V * la)) * B;
#pragma unroll
  for (int r = 0; r < V; ++r) {
    u32x4 *ptr = (u32x4 *)(d + (int64_t)r * p.ds0 * B);
    if (NT) __builtin_nontemporal_store(out.vec[r], ptr);
    else *ptr = out.vec[r];
  }
}

// Transpose of 16-bit elements through LDS: a workgroup owns a TI x TJ tile.  Each lane still
// transposes 8x8 blocks in registers, but the lane re-distribution goes through LDS, which frees
// the lane->block assignment on each side: consecutive lanes cover TI*2 contiguous bytes of a
// source line when loading and TJ*2 contiguous bytes of a destination line when storing.
// LDS image: [TI rows][TJ/8 chunks of 16 bytes], chunk index XOR-ed with (row/8) % 16: the 16
// lanes of an access phase differ in row/8 on the write side and in the chunk on the read side,
// so either way they land on 16 distinct chunks = all 64 banks once.
template <int TI, int TJ, bool NT>
__global__ __launch_bounds__(256) void transpose_lds_kernel(CopyParams p) {
  constexpr int NI = TI / 8, NJ = TJ / 8, ROW = TJ * 2, PER_LANE = NI * NJ / 256;
  static_assert(NI >= 16 && NJ >= 16 && (NI * NJ) % 256 == 0, "tile must hold whole 16-lane phases");
  __shared__ __attribute__((aligned(16))) char tile[TI * TJ * 2];  // static: the size is the code object's, no launch attribute to raise
  const char *src;
  char *dst;
  program_base<2>(p, src, dst);
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  if (p.map_mode == 1) {
    uint32_t lin = by * gridDim.x + bx;
    by = lin % gridDim.y;
    bx = lin / gridDim.y;
  } else if (p.map_mode == 2) {
    by = (by + bx) % gridDim.y;
  }
  const int32_t ti = bx * TI, tj = by * TJ;
  const int t = threadIdx.x;
  const bool interior = ti + TI <= p.d0 && ti + TI <= p.sb0 && tj + TJ <= p.d1 && tj + TJ <= p.sb1;
  // A tile that hangs over the edge of a matrix made of whole 8 x 8 blocks (and wholly inside the source: nothing to pad)
  // takes the same path with the blocks beyond the edge left out; only other edge tiles go element by element (a lane's 64
  // elements one after the other, each waiting for its load: 8200 x 8184 took 152 us for that, against 50).
  const bool whole_blocks = p.d0 % 8 == 0 && p.d1 % 8 == 0 && p.sb0 >= p.d0 && p.sb1 >= p.d1;
  if (!interior && !whole_blocks) {
    for (int e = t; e < TI * TJ; e += 256) copy_one<2>(p, src, dst, ti + e / TJ, tj + e % TJ);
    return;
  }
  union Block {
    u32x4 vec[8];
    uint16_t el[8][8];
  };
  Block in[PER_LANE];
#pragma unroll
  for (int k = 0; k < PER_LANE; ++k) {
    const int q = t + 256 * k, bi = q % NI, bj = q / NI;  // consecutive lanes along the source's contiguous axis
    const char *s = src + ((int64_t)(ti + 8 * bi) + (int64_t)(tj + 8 * bj) * p.es1) * 2;
    const bool live = interior || (ti + 8 * bi < p.d0 && tj + 8 * bj < p.d1);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const u32x4 *ptr = (const u32x4 *)(s + (int64_t)c * p.es1 * 2);
      in[k].vec[c] = u32x4{0, 0, 0, 0};
      if (live) in[k].vec[c] = NT ? __builtin_nontemporal_load(ptr) : *ptr;
    }
  }
#pragma unroll
  for (int k = 0; k < PER_LANE; ++k) {
    const int q = t + 256 * k, bi = q % NI, bj = q / NI;
    Block out;
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int c = 0; c < 8; ++c) out.el[r][c] = in[k].el[c][r];
#pragma unroll
    for (int r = 0; r < 8; ++r) *(u32x4 *)(tile + (8 * bi + r) * ROW + ((bj ^ (bi & 15)) << 4)) = out.vec[r];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < PER_LANE; ++k) {
    const int q = t + 256 * k, bj = q % NJ, bi = q / NJ;  // consecutive lanes along the destination's contiguous axis
    char *d = dst + ((int64_t)(ti + 8 * bi) * p.ds0 + (int64_t)(tj + 8 * bj)) * 2;
    if (!interior && !(ti + 8 * bi < p.d0 && tj + 8 * bj < p.d1)) continue;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      u32x4 v = *(const u32x4 *)(tile + (8 * bi + r) * ROW + ((bj ^ (bi & 15)) << 4));
      u32x4 *ptr = (u32x4 *)(d + (int64_t)r * p.ds0 * 2);
      if (NT) __builtin_nontemporal_store(v, ptr);
      else *ptr = v;
    }
  }
}

template <int TI, int TJ>
int launch_transpose_lds(const CopyParams &p, bool nt, int32_t batch, hipStream_t stream) {
  dim3 grid((unsigned)((p.d0 + TI - 1) / TI), (unsigned)((p.d1 + TJ - 1) / TJ), (unsigned)batch);
  if (nt) transpose_lds_kernel<TI, TJ, true><<<grid, 256, 0, stream>>>(p);
  else transpose_lds_kernel<TI, TJ, false><<<grid, 256, 0, stream>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

uint32_t padding_word(int32_t dtype, int32_t padding) {
  // ConvertUtils.cpp:267-334; e4m3 is OCP E4M3FN here (no infinities): +-inf -> +-448, qnan -> 0x7F.
  static const uint32_t f32[4] = {0, 0x7FC00000u, 0x7F800000u, 0xFF800000u};
  static const uint32_t f16[4] = {0, 0x7E007E00u, 0x7C007C00u, 0xFC00FC00u};
  static const uint32_t bf16[4] = {0, 0x7FC07FC0u, 0x7F807F80u, 0xFF80FF80u};
  static const uint32_t e4m3[4] = {0, 0x7F7F7F7Fu, 0x7E7E7E7Eu, 0xFEFEFEFEu};
  static const uint32_t e5m2[4] = {0, 0x7E7E7E7Eu, 0x7C7C7C7Cu, 0xFCFCFCFCu};
  switch (dtype) {
  case KAPY_F32: return f32[padding];
  case KAPY_F16: return f16[padding];
  case KAPY_BF16: return bf16[padding];
  case KAPY_F8E4M3: return e4m3[padding];
  case KAPY_F8E5M2: return e5m2[padding];
  }
  return 0;
}

template <int B>
int launch(const CopyParams &p0, int vb_src, int vb_dst, bool nt, int32_t batch, hipStream_t stream) {
  CopyParams p = p0;
  if (p.d0 <= 0 || p.d1 <= 0 || batch <= 0) return KAPY_OK;
  // Make "destination contiguous along j" the canonical orientation.
  if (p.ds1 != 1 && p.ds0 == 1) {
    std::swap(p.es0, p.es1);
    std::swap(p.ds0, p.ds1);
    std::swap(p.d0, p.d1);
    std::swap(p.sb0, p.sb1);
  }
  if (batch > 65535) return fail(KAPY_ERR_UNSUPPORTED, "copy: more than 65535 programs in one launch");
  if (p.ds1 == 1 && p.es1 == 1) {
    int vb = std::min(vb_src, vb_dst);
    int64_t slots_at_vb = (int64_t)p.d0 * ((p.d1 + vb / B - 1) / (vb / B));
    if (vb >= 4 && slots_at_vb < (int64_t(1) << 31) - 1024) {
      int e = vb / B;
      int32_t vpr = (p.d1 + e - 1) / e;
      int64_t slots = slots_at_vb;
      dim3 grid((unsigned)((slots + 256 - 1) / (256)), 1, (unsigned)batch);
      // no ragged vector anywhere: every slot is a whole in-bounds vector on both sides
      bool ragged = p.d1 % e != 0 || p.sb1 < p.d1 || p.sb0 < p.d0;
      if (vb == 16 && !ragged) {
        if (nt) rows_kernel<B, 16, true, false><<<grid, 256, 0, stream>>>(p, vpr);
        else rows_kernel<B, 16, false, false><<<grid, 256, 0, stream>>>(p, vpr);
      } else if (vb == 16) {
        rows_kernel<B, 16, false, true><<<grid, 256, 0, stream>>>(p, vpr);
      } else if (vb == 8) {
        rows_kernel<B, 8, false, true><<<grid, 256, 0, stream>>>(p, vpr);
      } else {
        rows_kernel<B, 4, false, true><<<grid, 256, 0, stream>>>(p, vpr);
      }
      KAPY_HIP_CHECK(hipGetLastError());
      return KAPY_OK;
    }
  } else if (B == 2 && p.ds1 == 1 && p.es0 == 1 && vb_src == 16 && vb_dst == 16 && p.d0 >= 128 && p.d1 >= 128 &&
             (p.d1 + 127) / 128 <= 65535) {
    // 256 x 256 tiles where they divide the matrix and still fill the chip (one workgroup per CU: the tile takes 128 KiB of
    // LDS): a tile side is the length of the contiguous runs the kernel reads and writes, and 512-byte runs move at
    // 5.7 TB/s where 256-byte runs move at 5.4 (1 KiB runs would reach the plain copy's 6.1, but no tile that big fits).
    if (p.d0 % 256 == 0 && p.d1 % 256 == 0 && p.sb0 >= p.d0 && p.sb1 >= p.d1 && (int64_t)(p.d0 / 256) * (p.d1 / 256) * batch >= 2 * (int64_t)device_cus())
      return launch_transpose_lds<256, 256>(p, nt, batch, stream);
    return launch_transpose_lds<128, 128>(p, nt, batch, stream);
  } else if (p.ds1 == 1 && p.es0 == 1 && vb_src == 16 && vb_dst == 16) {
    constexpr int TILE = 8 * (16 / B);
    unsigned gx = (unsigned)((p.d0 + 2 * TILE - 1) / (2 * TILE)), gy = (unsigned)((p.d1 + 2 * TILE - 1) / (2 * TILE));
    if (gy <= 65535) {
      dim3 grid(gx, gy, (unsigned)batch);
      if (nt) transpose_kernel<B, true><<<grid, 256, 0, stream>>>(p);
      else transpose_kernel<B, false><<<grid, 256, 0, stream>>>(p);
      KAPY_HIP_CHECK(hipGetLastError());
      return KAPY_OK;
    }
  }
  if (p.ds1 == 1 && p.es0 == 1 && p.d0 >= 16 && p.d1 >= 16 && (p.d1 + 63) / 64 <= 65535) {
    transpose_any_kernel<B><<<dim3((unsigned)((p.d0 + 63) / 64), (unsigned)((p.d1 + 63) / 64), (unsigned)batch), 256, 0, stream>>>(p);
    KAPY_HIP_CHECK(hipGetLastError());
    return KAPY_OK;
  }
  int64_t total = (int64_t)p.d0 * p.d1;
  int j_fastest = p.ds1 <= p.ds0;
  dim3 grid((unsigned)((total + 255) / 256), 1, (unsigned)batch);
  generic_kernel<B><<<grid, 256, 0, stream>>>(p, j_fastest);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace

int copy_impl(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg, const kapy_grid2 *grid, void *stream) {
  int rc = check_global(src, "copy source");
  if (!rc) rc = check_global(dst, "copy target");
  if (rc) return rc;
  int B = dtype_bytes(src->dtype);
  // st_global carries SameOperandsElementType (Ops.td:163-170); a move only needs equal widths, so
  // re-typed views of the same bits (f16 <-> i16 ...) are let through.
  if (B != dtype_bytes(dst->dtype))
    return fail(KAPY_ERR_VERIFY, "copy: source (%s) and target (%s) must have the same element width", dtype_name(src->dtype),
                dtype_name(dst->dtype));
  kapy_copy_cfg c = {0, KAPY_PAD_ZERO, KAPY_CACHE_NONE, KAPY_EVICT_NORMAL, 0, 0};
  if (cfg) c = *cfg;
  if (c.padding_option < 0 || c.padding_option > 3) return fail(KAPY_ERR_INVALID, "copy: unknown padding option %d", c.padding_option);
  if (c.cache_modifier < KAPY_CACHE_NONE || c.cache_modifier > KAPY_CACHE_CV) return fail(KAPY_ERR_INVALID, "copy: unknown cache modifier %d", c.cache_modifier);
  if (c.evict_priority < KAPY_EVICT_NORMAL || c.evict_priority > KAPY_NO_ALLOCATE) return fail(KAPY_ERR_INVALID, "copy: unknown evict priority %d", c.evict_priority);
  if (c.padding_option != KAPY_PAD_ZERO && !is_float(src->dtype))
    return fail(KAPY_ERR_VERIFY, "copy: integer tensors only take zero padding");
  if (src->start0 < 0 || src->start1 < 0 || dst->start0 < 0 || dst->start1 < 0)
    return fail(KAPY_ERR_INVALID, "copy: negative view start");
  kapy_grid2 g = {1, 1, 0, 0, 0, 0};
  if (grid) g = *grid;
  if (g.n0 < 0 || g.n1 < 0) return fail(KAPY_ERR_INVALID, "copy: negative grid size");
  rc = ensure_device();
  if (rc) return rc;

  CopyParams p;
  p.src = view_base(src);
  p.dst = (char *)view_base(dst);
  bool t = c.transpose != 0;
  p.es0 = t ? src->stride1 : src->stride0;
  p.es1 = t ? src->stride0 : src->stride1;
  p.ds0 = dst->stride0;
  p.ds1 = dst->stride1;
  p.d0 = (int32_t)extent0(dst);
  p.d1 = (int32_t)extent1(dst);
  p.sb0 = (int32_t)(t ? extent1(src) : extent0(src));
  p.sb1 = (int32_t)(t ? extent0(src) : extent1(src));
  p.pad = padding_word(src->dtype, c.padding_option);
  p.n1 = g.n1 > 0 ? g.n1 : 1;
  p.map_mode = kTransposeMap;
  p.s_off0 = g.src_off0;
  p.s_off1 = g.src_off1;
  p.d_off0 = g.dst_off0;
  p.d_off1 = g.dst_off1;
  // vector width each side may use along its contiguous axis, also honouring the batch displacements
  auto side_vb = [&](const kapy_global *v, int64_t o0, int64_t o1) {
    int axis = v->stride1 == 1 ? 1 : (v->stride0 == 1 ? 0 : -1);
    if (axis < 0) return B;
    int vb = vector_bytes(v, axis);
    uint64_t bits = (uint64_t)((o0 < 0 ? -o0 : o0) * B) | (uint64_t)((o1 < 0 ? -o1 : o1) * B);
    while (vb > B && (bits & (uint64_t)(vb - 1))) vb >>= 1;
    return vb;
  };
  int vb_src = side_vb(src, g.n0 > 1 ? g.src_off0 : 0, g.n1 > 1 ? g.src_off1 : 0);
  int vb_dst = side_vb(dst, g.n0 > 1 ? g.dst_off0 : 0, g.n1 > 1 ? g.dst_off1 : 0);
  // Two dense matrices of the same shape (pitch = extent on both sides, nothing to pad) are one line of d0 * d1 elements:
  // whatever the extents, the line moves in 128-bit pieces from an aligned base, where rows of 5001 16-bit elements would
  // move element by element (3001 x 5001: 40 -> 10 us).
  if (g.n0 * g.n1 == 1 && p.ds1 == 1 && p.es1 == 1 && p.d0 > 1 && p.ds0 == p.d1 && p.es0 == p.d1 && p.sb1 >= p.d1 && p.sb0 >= p.d0 &&
      (int64_t)p.d0 * p.d1 < (int64_t(1) << 31) - 1024) {
    p.d1 = p.sb1 = p.d0 * p.d1;
    p.d0 = p.sb0 = 1;
    p.ds0 = p.es0 = p.d1;
    auto base_vb = [&](const void *ptr) {
      int vb = 16;
      while (vb > B && ((uintptr_t)ptr & (uintptr_t)(vb - 1))) vb >>= 1;
      return vb;
    };
    vb_src = base_vb(p.src);
    vb_dst = base_vb(p.dst);
  }
  // Streaming (non-temporal) access when asked for (cs / cg), and by default for moves too large to
  // be re-read from the 256 MB Infinity Cache anyway.
  const int64_t moved = (int64_t)p.d0 * p.d1 * B * (g.n0 > 0 ? g.n0 : 1) * (g.n1 > 0 ? g.n1 : 1);
  // The hints in the reference's order of precedence (LdGlobalOpToLLVM.cpp:103-109): volatile drops all of them, then
  // the cache modifier, then the eviction priority.
  bool nt = false;
  if (c.is_volatile) nt = false;
  else if (c.cache_modifier != KAPY_CACHE_NONE) nt = c.cache_modifier == KAPY_CACHE_CS || c.cache_modifier == KAPY_CACHE_CG;
  else if (c.evict_priority == KAPY_EVICT_FIRST || c.evict_priority == KAPY_NO_ALLOCATE) nt = true;
  else if (c.evict_priority == KAPY_EVICT_NORMAL) nt = moved >= (int64_t(32) << 20);
  int32_t batch = g.n0 * g.n1;
  hipStream_t s = (hipStream_t)stream;
  switch (B) {
  case 1: return launch<1>(p, vb_src, vb_dst, nt, batch, s);
  case 2: return launch<2>(p, vb_src, vb_dst, nt, batch, s);
  default: return launch<4>(p, vb_src, vb_dst, nt, batch, s);
  }
}

}  // namespace kapy

extern "C" {

int kapy_copy(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg, void *stream) {
  return kapy::copy_impl(src, dst, cfg, nullptr, stream);
}

int kapy_copy_batched(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg, const kapy_grid2 *grid, void *stream) {
  if (!grid) return kapy::fail(KAPY_ERR_INVALID, "copy_batched: null grid");
  return kapy::copy_impl(src, dst, cfg, grid, stream);
}

}  // extern "C"
