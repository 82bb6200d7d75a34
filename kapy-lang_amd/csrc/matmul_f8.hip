// matmul_f8.hip — kapy.matmul on OCP fp8 operands (E4M3FN / E5M2, mixable) with fp32 accumulate,
// and the W8A8 form with fp32 row/column scales applied in the epilogue.
//
// Reference: MatmulImplWay::MMA_M16N8K16_F8 (lib/Dialect/Kapy/IR/Kapy.cpp:545-564 verifier,
// MatmulOpToLLVM.cpp:269-311 mma.sync.m16n8k16 e4m3/e5m2 strings, operand layouts
// LayoutUtils.cpp:141-147) followed by mulf with broadcast scales and fptofp rn.
// gfx950: v_mfma_scale_f32_16x16x128_f8f6f4 with unit E8M0 block scales (2^0); the operand format
// selectors (cbsz / blgp: 0 = E4M3, 1 = E5M2) carry kapy's mixed-f8 rule.
//
//   skinny_stream_kernel  few rows of lhs (decode shape), K a multiple of 1024: HBM-bound on the weight;
//                  row-contiguous LDS-direct loads into per-wave rings, regrouped into operands by LDS reads.
//   skinny_kernel  the same shape for other K (multiples of 128).  One workgroup per 16*NG
//                  output columns, its 8 wavefronts split K; every weight byte is read once,
//                  straight from global memory into the MFMA operand registers (each lane's 32
//                  K-contiguous bytes are exactly its operand), partial sums meet in LDS.
//   naive_kernel   any strides / ragged K: one output element per lane, software decode.
#include "common.hpp"
#include "layout.hpp"
#include "matmul_params.hpp"
#include "mfma.hpp"
#include "numeric.hpp"

namespace kapy {
namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Both decode-shaped kernels multiply with v_mfma_scale_f32_16x16x128_f8f6f4 issued as documented (activation block
// in the first operand slot, weight block in the second), so a lane's registers sit where the instruction's own
// fragments layouts say: operand registers = 32 consecutive K bytes of row (lhs) / column (rhs) operand_lane().row,
// accumulator register v = element (row + v, col) of the 16x16 block (mfma_acc: a quad runs down a column).
constexpr MfmaShape kF8Shape = kMfma16x16x128F8;
constexpr bool acc_quad_runs_down_a_column() {
  const AccLane a = acc_lane(mfma_acc(kF8Shape), kF8Shape, 0);
  return a.drow == 1 && a.dcol == 0 && acc_lane_describes(mfma_acc(kF8Shape), kF8Shape);
}
static_assert(acc_quad_runs_down_a_column(), "accumulator fragments of the 16x16x128 instruction");
template <int A_FMT, int B_FMT>
__device__ __forceinline__ f32x4 mfma_f8(const i32x8 &a, const i32x8 &b, f32x4 c) {
  const u32x4 av[2] = {{(uint32_t)a[0], (uint32_t)a[1], (uint32_t)a[2], (uint32_t)a[3]}, {(uint32_t)a[4], (uint32_t)a[5], (uint32_t)a[6], (uint32_t)a[7]}};
  const u32x4 bv[2] = {{(uint32_t)b[0], (uint32_t)b[1], (uint32_t)b[2], (uint32_t)b[3]}, {(uint32_t)b[4], (uint32_t)b[5], (uint32_t)b[6], (uint32_t)b[7]}};
  return F8M16<A_FMT, B_FMT>::mfma(av, bv, c);
}

struct F8Params {
  const uint8_t *a, *b;
  const char *acc;
  char *d;
  const float *row_scale, *col_scale;
  int64_t a_sm, a_sk, b_sn, b_sk, acc_sm, acc_sn, d_sm, d_sn;
  int32_t M, N, K;
  int32_t a_dtype, b_dtype, acc_dtype, d_dtype, rz;
};

__device__ __forceinline__ void finish(const F8Params &p, int32_t m, int32_t n, float v) {
  if (m >= p.M || n >= p.N) return;
  if (p.row_scale) v *= __fmul_rn(p.row_scale[m], p.col_scale[n]);
  if (p.acc_dtype >= 0) v += load_as_f32(p.acc, p.acc_dtype, m * p.acc_sm + n * p.acc_sn);
  int64_t idx = m * p.d_sm + n * p.d_sn;
  switch (p.d_dtype) {
  case KAPY_F32: ((float *)p.d)[idx] = v; break;
  case KAPY_F16: ((uint16_t *)p.d)[idx] = p.rz ? f32_to_f16_rz(v) : f32_to_f16_rn(v); break;
  default: ((uint16_t *)p.d)[idx] = p.rz ? f32_to_bf16_rz(v) : f32_to_bf16_rn(v); break;
  }
}

__global__ __launch_bounds__(256) void naive_kernel(F8Params p) {
  int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= (int64_t)p.M * p.N) return;
  int32_t m = (int32_t)(t / p.N), n = (int32_t)(t - (int64_t)m * p.N);
  float s = 0.f;
  for (int32_t k = 0; k < p.K; ++k) {
    float x = load_as_f32(p.a, p.a_dtype, m * p.a_sm + k * p.a_sk);
    float y = load_as_f32(p.b, p.b_dtype, n * p.b_sn + k * p.b_sk);
    s = __fmaf_rn(x, y, s);
  }
  finish(p, m, n, s);
}

// What no other kernel takes (operand rows that are not 16-byte aligned, K not a multiple of 16, strided operands): 64 x 64
// results per workgroup, 4 x 4 per lane, K in steps of 32 whose operand elements are loaded one by one (lanes along K),
// decoded to fp32 into LDS and multiplied there on the vector ALU.  About fifty times the one-lane-per-result kernel above.
__global__ __launch_bounds__(256) void tiled_any_kernel(F8Params p) {
  constexpr int T = 64, KS = 32, PITCH = KS + 1;
  __shared__ float as[T * PITCH], bs[T * PITCH];
  const int t = threadIdx.x, ty = t >> 4, tx = t & 15;
  const int32_t tiles_n = (p.N + T - 1) / T;
  const int32_t m0 = (int32_t)(blockIdx.x / tiles_n) * T, n0 = (int32_t)(blockIdx.x % tiles_n) * T;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int32_t k0 = 0; k0 < p.K; k0 += KS) {
#pragma unroll
    for (int i = 0; i < T * KS / 256; ++i) {
      const int e = t + 256 * i, row = e / KS, k = e % KS;
      const bool k_in = k0 + k < p.K;
      as[row * PITCH + k] = (k_in && m0 + row < p.M) ? load_as_f32(p.a, p.a_dtype, (int64_t)(m0 + row) * p.a_sm + (int64_t)(k0 + k) * p.a_sk) : 0.f;
      bs[row * PITCH + k] = (k_in && n0 + row < p.N) ? load_as_f32(p.b, p.b_dtype, (int64_t)(n0 + row) * p.b_sn + (int64_t)(k0 + k) * p.b_sk) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < KS; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = as[(ty * 4 + i) * PITCH + k];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = bs[(tx * 4 + j) * PITCH + k];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __fmaf_rn(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) finish(p, m0 + ty * 4 + i, n0 + tx * 4 + j, acc[i][j]);
}

// 32 K-contiguous bytes of one row/column as the 8-dword MFMA operand; rows past the end read zero.
__device__ __forceinline__ i32x8 load_k32(const uint8_t *base, int64_t stride, int32_t row, int32_t rows, int32_t k) {
  i32x8 r = {0, 0, 0, 0, 0, 0, 0, 0};
  if (row < rows) {
    const i32x4 *ptr = (const i32x4 *)(base + row * stride + k);
    i32x4 lo = ptr[0], hi = ptr[1];
    r = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }
  return r;
}

// Skinny kernel.  Workgroup = 8 wavefronts = 8 contiguous K ranges, NG groups of 16 output columns.
// A wave first requests everything it will multiply in a chunk of CH K-steps - the weight bytes of
// its NG column groups and the activation bytes they share - and only then starts the matrix
// instructions, so that a CU keeps >100 KiB of HBM reads in flight with only 8 resident waves.
constexpr int kSkinnyWaves = 8, kSkinnyGroups = 1, kSkinnyChunk = 8;  // wavefronts, 16-column groups per workgroup, K-steps requested ahead
template <int A_FMT, int B_FMT, int NG, int CH>
__global__ __launch_bounds__(64 * kSkinnyWaves) void skinny_kernel(F8Params p) {
  __shared__ float partial[kSkinnyWaves][NG][16][16 + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int32_t n0 = blockIdx.x * 16 * NG, m0 = blockIdx.y * 16;
  const OperandLane frag_at = operand_lane(kF8Shape, lane);
  const int32_t row = frag_at.row, kq = frag_at.k0;  // this lane's row/column and its 32-byte K quarter
  const int32_t steps = p.K / 128, per_wave = (steps + kSkinnyWaves - 1) / kSkinnyWaves;
  const int32_t s_begin = wave * per_wave, s_end = min(steps, s_begin + per_wave);
  f32x4 acc[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int32_t s = s_begin; s < s_end; s += CH) {
    i32x8 bw[NG][CH], aw[CH];
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const bool live = s + u < s_end;
#pragma unroll
      for (int g = 0; g < NG; ++g) bw[g][u] = load_k32(p.b, p.b_sn, n0 + 16 * g + row, live ? p.N : 0, (s + u) * 128 + kq);
    }
#pragma unroll
    for (int u = 0; u < CH; ++u) aw[u] = load_k32(p.a, p.a_sm, m0 + row, s + u < s_end ? p.M : 0, (s + u) * 128 + kq);
#pragma unroll
    for (int u = 0; u < CH; ++u)
#pragma unroll
      for (int g = 0; g < NG; ++g)
        acc[g] = mfma_f8<A_FMT, B_FMT>(aw[u], bw[g][u], acc[g]);
  }
  const AccLane acc_at = acc_lane(mfma_acc(kF8Shape), kF8Shape, lane);
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int v = 0; v < 4; ++v) partial[wave][g][acc_at.row + v][acc_at.col] = acc[g][v];
  __syncthreads();
  for (int e = threadIdx.x; e < NG * 256; e += 64 * kSkinnyWaves) {
    const int g = e >> 8, m = (e >> 4) & 15, n = e & 15;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kSkinnyWaves; ++w) sum += partial[w][g][m][n];
    finish(p, m0 + m, n0 + 16 * g + n, sum);
  }
}

// Streaming skinny kernel (K a multiple of 1024).  Workgroup = 4 wavefronts = 4 contiguous K ranges of
// one 16-column group; every wave works alone (no barrier until the final sum).  What decides the rate
// of this HBM-bound shape is the shape of the load instructions: the operand layout of the matrix
// instruction (lane = row % 16, 32 K-bytes per lane) asked for directly makes every load touch 16 rows
// in 16-byte pieces, and the texture path takes about twice as long over it as over contiguous runs.
// So the bytes come in as LDS-direct loads of 4 rows x 256 contiguous bytes and are regrouped on the
// way out of LDS: a wave keeps a private ring of two 8 KiB stages (weight 4 KiB + activation 4 KiB,
// 256 K-bytes of 16 rows each), 16-byte chunk c of row r stored at chunk c ^ r of the row's 256 bytes
// so that the 16 rows a quarter-wave reads fall into 16 different bank groups.
// Rows past M / N are clamped to the last valid row (never stored), so nothing is read out of range.
// Which kernel serves how many rows (thresholds measured at N = K = 8192).  Up to 16 rows: the streaming kernel below.
// From 17 rows: the block streaming kernel (32 columns x up to 128 rows per workgroup, the weight read once), where K is a
// multiple of 512; it yields to the tiled MFMA kernel from kTiledFromM rows, or from kTiledFromMSplit when the caller's
// workspace lets the tiled kernel split K across workgroups (N = K = 8192, M = 65 / 80 / 96 / 112 / 128: block kernel 20.7 /
// 22.2 / 24.8 / 27.3 / 29.4 us, split tiled kernel 27.7 / 27.7 / 28.3 / 28.3 / 29.0; 144 / 160 rows: blocks of 64 rows 44 us,
// the tiled kernel's four-stage build 35 us).  Where the block kernel cannot run, the streaming kernel
// (which reads the weight once per 16 rows) is all there is below the tiled kernel, and the tiled kernel takes over earlier.
constexpr int kTiledFromM = 129, kTiledFromMSplit = 113;
constexpr int kTiledFromMNoBlock = 81, kTiledFromMSplitNoBlock = 40;
constexpr int kStreamWaves = 4, kStreamChunk = 256, kStreamStage = 2 * 16 * kStreamChunk, kStreamStages = 2;
// NG: groups of 16 columns a wave multiplies with one activation chunk (a stage is then NG weight parts and one activation part
// of 4 KiB each).  NG = 1 re-reads the whole activation per 16 columns - as many bytes from the L2s as the weight itself at
// M = 16; NG = 2 halves that with one workgroup of 96 KiB per CU.
template <int A_FMT, int B_FMT, int NG, int STAGES>
__global__ __launch_bounds__(64 * kStreamWaves) void skinny_stream_kernel(F8Params p) {
  constexpr int kPart = 16 * kStreamChunk, kStage = (NG + 1) * kPart, kLoads = 4 * (NG + 1);
  __shared__ __attribute__((aligned(1024))) char ring[kStreamWaves * STAGES * kStage];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Workgroup id -> (block of 16 * NG columns, 16-row group).  With more than one row group the workgroups that stream the same
  // columns of the weight must meet in one L2: consecutive ids go to the 8 XCDs in turn, so the groups of a column block
  // take ids 8 apart (the same XCD, dispatched back to back) and the second reader of a weight line finds it there.
  const int32_t col_blocks = (p.N + 16 * NG - 1) / (16 * NG), groups = (p.M + 15) / 16;
  const int32_t on_xcd = blockIdx.x / 8, xcd = blockIdx.x % 8;
  const int32_t col_block = (on_xcd / groups) * 8 + xcd;
  if (col_block >= col_blocks) return;  // (the grid is padded to whole rounds of 8)
  const int32_t n0 = col_block * 16 * NG, m0 = (on_xcd % groups) * 16;
  const int32_t k_per_wave = p.K / kStreamWaves, chunks = k_per_wave / kStreamChunk;
  auto uniform_ptr = [](const uint8_t *ptr) {
    const uint64_t v = (uint64_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (void *)(((uint64_t)hi << 32) | lo);
  };
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.b + (int64_t)n0 * p.b_sn + (int64_t)wave * k_per_wave), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.a + (int64_t)m0 * p.a_sm + (int64_t)wave * k_per_wave), 0, 0x7fffffff, 0x00020000);
  // load instruction i (0..3) of a 16-row part: rows 4i .. 4i+3, this lane row 4i + lane/16, stored chunk lane%16
  uint32_t w_off[NG][4], a_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * i + (lane >> 4), c = (lane & 15) ^ r;
#pragma unroll
    for (int g = 0; g < NG; ++g) w_off[g][i] = (uint32_t)(min(16 * g + r, p.N - 1 - n0) * p.b_sn + c * 16);
    a_off[i] = (uint32_t)(min(r, p.M - 1 - m0) * p.a_sm + c * 16);
  }
  // A weight that only this workgroup reads (one group of rows) is loaded non-temporally: it then does not push the activation,
  // which every workgroup re-reads, out of the L2 (cache policy bit 1; M = 16: 14.6 -> 13.7 us).
  const bool w_once = groups == 1;
  char *my_ring = ring + wave * (STAGES * kStage);
  auto issue_chunk = [&](int chunk, int stage) {
    char *dst = my_ring + stage * kStage;
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (w_once) __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (__attribute__((address_space(3))) void *)(dst + g * kPart + i * 1024), 16, (int)w_off[g][i], chunk * kStreamChunk, 0, 2);
        else __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (__attribute__((address_space(3))) void *)(dst + g * kPart + i * 1024), 16, (int)w_off[g][i], chunk * kStreamChunk, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(dst + NG * kPart + i * 1024), 16, (int)a_off[i], chunk * kStreamChunk, 0, 0);
  };
  // operand reads: the lane's row and its 32 K bytes of a 128-byte step: chunks 8*step + 2*group, +1
  const OperandLane frag_at = operand_lane(kF8Shape, lane);
  const int r16 = frag_at.row, grp = frag_at.k0 / kF8Shape.kpack;
  uint32_t rd[2][2];
#pragma unroll
  for (int st = 0; st < 2; ++st)
#pragma unroll
    for (int h = 0; h < 2; ++h) rd[st][h] = (uint32_t)(r16 * kStreamChunk + (((8 * st + 2 * grp + h) ^ r16) * 16));
  f32x4 acc[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < STAGES; ++st)
    if (st < chunks) issue_chunk(st, st);
  constexpr auto vmcnt = [](int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); };
  int stage = 0;
  for (int32_t c = 0; c < chunks; ++c) {
    // this chunk has landed; the (up to STAGES - 1) chunks issued after it may still be in flight
    const int behind = min(STAGES - 1, chunks - 1 - c);
    if (behind >= 2) __builtin_amdgcn_s_waitcnt(vmcnt(2 * kLoads));
    else if (behind == 1) __builtin_amdgcn_s_waitcnt(vmcnt(kLoads));
    else __builtin_amdgcn_s_waitcnt(vmcnt(0));
    const char *src = my_ring + stage * kStage;
    i32x4 w[NG][2][2], a[2][2];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int g = 0; g < NG; ++g) w[g][st][h] = *(const i32x4 *)(src + g * kPart + rd[st][h]);
        a[st][h] = *(const i32x4 *)(src + NG * kPart + rd[st][h]);
      }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the stage has been read, it may be refilled
    if (c + STAGES < chunks) issue_chunk(c + STAGES, stage);
    stage = stage + 1 == STAGES ? 0 : stage + 1;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const i32x8 av = {a[st][0][0], a[st][0][1], a[st][0][2], a[st][0][3], a[st][1][0], a[st][1][1], a[st][1][2], a[st][1][3]};
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const i32x8 wv = {w[g][st][0][0], w[g][st][0][1], w[g][st][0][2], w[g][st][0][3], w[g][st][1][0], w[g][st][1][1], w[g][st][1][2], w[g][st][1][3]};
        acc[g] = mfma_f8<A_FMT, B_FMT>(av, wv, acc[g]);
      }
    }
  }
  // the four K ranges meet in LDS
  const AccLane acc_at = acc_lane(mfma_acc(kF8Shape), kF8Shape, lane);
  __syncthreads();  // every wave is done with its ring
  float *partial = (float *)ring;  // [wave][NG][16][17]
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int v = 0; v < 4; ++v) partial[((wave * NG + g) * 16 + acc_at.row + v) * 17 + acc_at.col] = acc[g][v];
  __syncthreads();
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int m = threadIdx.x >> 4, n = threadIdx.x & 15;
    float sum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < kStreamWaves; ++w2) sum += partial[((w2 * NG + g) * 16 + m) * 17 + n];
    finish(p, m0 + m, n0 + 16 * g + n, sum);
  }
}

// Block streaming kernel: the same idea for 17 .. 128 rows of lhs (and, in blocks of 64 rows, beyond).  Reading the
// weight once per 16 rows, as the kernel above does, asks the L2 for it M/16 times, and a workgroup of 16 columns re-reads
// the whole activation: at M = 64 the activation traffic is four times the weight's.  Here a workgroup owns 32 columns and
// 16*RG rows (RG = 2 .. 8), so at N = 8192 there is one workgroup per CU, every weight byte crosses the fabric once, and the activation
// (M x K bytes, L2-resident) is read N/32 times.  Its 4 waves split K and work alone on private rings of kBlockStages
// stages; a stage is one 128-byte K step: 32 weight rows and 16*RG activation rows of 128 contiguous bytes, brought in by
// LDS-direct loads of 8 rows each, 16-byte chunk c of row r stored at chunk c ^ block_key(r % 16) - the 16 lanes of a
// read phase then cover all 64 banks once.  RG x 2 accumulator blocks per wave; the four K ranges meet in LDS.
constexpr int kBlockStep = 128, kBlockCols = 32;
// (the lanes of one phase of a 16-byte LDS read are 0-3, 12-15, 20-23, 24-27 and so on: rows r16 = 0-3 and 12-15 of one K
// group with rows 4-11 of the next; with this key they fall into 16 different groups of four banks)
__device__ __forceinline__ constexpr int block_key(int r) { return (r & 7) ^ ((r >> 3) & 1); }
constexpr int block_stages(int rg) { return rg >= 5 ? 2 : 3; }  // (four for 32 rows fits the LDS too and measured no faster; 80 rows and more leave room for two)
constexpr int waitcnt_vm(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }  // s_waitcnt vmcnt(n), nothing else waited for
template <int A_FMT, int B_FMT, int RG>
__global__ __launch_bounds__(256) void skinny_block_kernel(F8Params p) {
  constexpr int kBlockStages = block_stages(RG), kRows = 16 * RG, kStage = (kBlockCols + kRows) * kBlockStep, kLoadsW = kBlockCols / 8, kLoadsA = kRows / 8, kLoads = kLoadsW + kLoadsA;
  static_assert(4 * kBlockStages * kStage <= 160 * 1024 && (kBlockStages - 1) * kLoads <= 63, "rings must fit the LDS, loads in flight the counter");
  __shared__ __attribute__((aligned(1024))) char ring[4 * kBlockStages * kStage];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // workgroup id -> (32-column block, row block): the row blocks of a column block take ids 8 apart (one XCD, dispatched
  // back to back), so that the second reader of a weight line finds it in that XCD's L2
  const int32_t col_blocks = (p.N + kBlockCols - 1) / kBlockCols, row_blocks = (p.M + kRows - 1) / kRows;
  const int32_t on_xcd = blockIdx.x / 8, xcd = blockIdx.x % 8;
  const int32_t col_block = (on_xcd / row_blocks) * 8 + xcd;
  if (col_block >= col_blocks) return;  // (the grid is padded to whole rounds of 8)
  const int32_t n0 = col_block * kBlockCols, m0 = (on_xcd % row_blocks) * kRows;
  const int32_t k_per_wave = p.K / 4, steps = k_per_wave / kBlockStep;
  auto uniform_ptr = [](const uint8_t *ptr) {
    const uint64_t v = (uint64_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (void *)(((uint64_t)hi << 32) | lo);
  };
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.b + (int64_t)n0 * p.b_sn + (int64_t)wave * k_per_wave), 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(p.a + (int64_t)m0 * p.a_sm + (int64_t)wave * k_per_wave), 0, 0x7fffffff, 0x00020000);
  // load instruction i of an operand: rows 8i .. 8i+7, this lane row 8i + lane/8, filling chunk position lane%8 of it.
  // Rows past N / M are clamped to the last valid row (their results are never stored), so nothing is read out of range.
  uint32_t w_off[kLoadsW], a_off[kLoadsA];
#pragma unroll
  for (int i = 0; i < kLoadsW; ++i) {
    const int r = 8 * i + (lane >> 3), c = (lane & 7) ^ block_key(r);
    w_off[i] = (uint32_t)(min(r, p.N - 1 - n0) * p.b_sn + c * 16);
  }
#pragma unroll
  for (int i = 0; i < kLoadsA; ++i) {
    const int r = 8 * i + (lane >> 3), c = (lane & 7) ^ block_key(r);
    a_off[i] = (uint32_t)(min(r, p.M - 1 - m0) * p.a_sm + c * 16);
  }
  const bool w_once = row_blocks == 1;  // (see the streaming kernel: non-temporal loads for a weight read once)
  char *my_ring = ring + wave * (kBlockStages * kStage);
  auto issue_step = [&](int step, int stage) {
    char *dst = my_ring + stage * kStage;
#pragma unroll
    for (int i = 0; i < kLoadsW; ++i)
      if (w_once) __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (__attribute__((address_space(3))) void *)(dst + i * 1024), 16, (int)w_off[i], step * kBlockStep, 0, 2);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (__attribute__((address_space(3))) void *)(dst + i * 1024), 16, (int)w_off[i], step * kBlockStep, 0, 0);
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(dst + kBlockCols * kBlockStep + i * 1024), 16, (int)a_off[i], step * kBlockStep, 0, 0);
  };
  // operand reads: the lane's row of a 16-row block and its 32 K bytes of the step, chunks 2*group and 2*group + 1
  const OperandLane frag_at = operand_lane(kF8Shape, lane);
  const int r16 = frag_at.row, grp = frag_at.k0 / kF8Shape.kpack;
  uint32_t rd[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) rd[h] = (uint32_t)(r16 * kBlockStep + (((2 * grp + h) ^ block_key(r16)) * 16));
  f32x4 acc[RG][2];
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int g = 0; g < 2; ++g) acc[r][g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < kBlockStages; ++st)
    if (st < steps) issue_step(st, st);
  int stage = 0;
  for (int32_t c = 0; c < steps; ++c) {
    // this step has landed once only the younger steps' loads remain in flight
    const int32_t younger = min(steps - 1 - c, kBlockStages - 1);
    if (younger >= 3) __builtin_amdgcn_s_waitcnt(waitcnt_vm(3 * kLoads));
    else if (younger == 2) __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * kLoads));
    else if (younger == 1) __builtin_amdgcn_s_waitcnt(waitcnt_vm(kLoads));
    else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    static_assert(kBlockStages <= 4, "the waits above are written for up to four stages");
    const char *src = my_ring + stage * kStage;
    i32x4 w[2][2], a[RG][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int g = 0; g < 2; ++g) w[g][h] = *(const i32x4 *)(src + g * 16 * kBlockStep + rd[h]);
#pragma unroll
      for (int r = 0; r < RG; ++r) a[r][h] = *(const i32x4 *)(src + (kBlockCols + r * 16) * kBlockStep + rd[h]);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the stage has been read, it may be refilled
    if (c + kBlockStages < steps) issue_step(c + kBlockStages, stage);
#pragma unroll
    for (int r = 0; r < RG; ++r) {
      const i32x8 av = {a[r][0][0], a[r][0][1], a[r][0][2], a[r][0][3], a[r][1][0], a[r][1][1], a[r][1][2], a[r][1][3]};
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        const i32x8 wv = {w[g][0][0], w[g][0][1], w[g][0][2], w[g][0][3], w[g][1][0], w[g][1][1], w[g][1][2], w[g][1][3]};
        acc[r][g] = mfma_f8<A_FMT, B_FMT>(av, wv, acc[r][g]);
      }
    }
    stage = stage + 1 == kBlockStages ? 0 : stage + 1;
  }
  // the four K ranges meet in LDS
  const AccLane acc_at = acc_lane(mfma_acc(kF8Shape), kF8Shape, lane);
  __syncthreads();  // every wave is done with its ring
  float *partial = (float *)ring;  // [wave][kRows][kBlockCols + 1]
  constexpr int kPitch = kBlockCols + 1;
  static_assert(4 * kRows * kPitch * 4 <= 4 * kBlockStages * kStage, "the partial sums reuse the rings");
#pragma unroll
  for (int r = 0; r < RG; ++r)
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int v = 0; v < 4; ++v) partial[(wave * kRows + 16 * r + acc_at.row + v) * kPitch + 16 * g + acc_at.col] = acc[r][g][v];
  __syncthreads();
  for (int e = threadIdx.x; e < kRows * kBlockCols; e += 256) {
    const int m = e / kBlockCols, n = e % kBlockCols;
    float sum = 0.f;
#pragma unroll
    for (int w2 = 0; w2 < 4; ++w2) sum += partial[(w2 * kRows + m) * kPitch + n];
    finish(p, m0 + m, n0 + n, sum);
  }
}

template <int RG>
int launch_skinny_block(const F8Params &p, int fa, int fb, hipStream_t s) {
  const int64_t col_rounds = ((p.N + kBlockCols - 1) / kBlockCols + 7) / 8, row_blocks = (p.M + 16 * RG - 1) / (16 * RG);
  dim3 grid((unsigned)(col_rounds * 8 * row_blocks));
  if (fa == 0 && fb == 0) skinny_block_kernel<0, 0, RG><<<grid, 256, 0, s>>>(p);
  else if (fa == 0) skinny_block_kernel<0, 1, RG><<<grid, 256, 0, s>>>(p);
  else if (fb == 0) skinny_block_kernel<1, 0, RG><<<grid, 256, 0, s>>>(p);
  else skinny_block_kernel<1, 1, RG><<<grid, 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

int fmt_of(int dtype) { return dtype == KAPY_F8E5M2 ? 1 : 0; }

}  // namespace

int matmul_f8(const kapy_global *a, const kapy_global *b, const float *row_scale, const float *col_scale, const kapy_global *acc,
              const kapy_global *result, const kapy_matmul_cfg *cfg, hipStream_t s) {
  F8Params p;
  p.a = (const uint8_t *)view_base(a);
  p.b = (const uint8_t *)view_base(b);
  p.acc = acc ? view_base(acc) : nullptr;
  p.d = (char *)view_base(result);
  p.row_scale = row_scale;
  p.col_scale = col_scale;
  p.a_sm = a->stride0; p.a_sk = a->stride1;
  p.b_sk = b->stride0; p.b_sn = b->stride1;
  p.acc_sm = acc ? acc->stride0 : 0; p.acc_sn = acc ? acc->stride1 : 0;
  p.d_sm = result->stride0; p.d_sn = result->stride1;
  p.M = (int32_t)extent0(a); p.K = (int32_t)extent1(a); p.N = (int32_t)extent1(b);
  p.a_dtype = a->dtype; p.b_dtype = b->dtype;
  p.acc_dtype = acc ? acc->dtype : -1;
  p.d_dtype = result->dtype;
  p.rz = cfg && cfg->rmode == KAPY_RZ;
  if (p.M == 0 || p.N == 0) return KAPY_OK;
  // K-contiguous operands with 16-byte aligned rows of whole 16-byte pieces: what the tiled kernel needs (its ring builds take
  // a partial last K-tile); the streaming kernels below need whole 128-byte K steps
  const bool k_pieces = p.a_sk == 1 && p.b_sk == 1 && vector_bytes(a, 1) == 16 && vector_bytes(b, 0) == 16 && p.K % 16 == 0 && p.K > 0;
  const bool k_contig = k_pieces && p.K % 128 == 0;
  // Many rows: the tiled LDS-direct kernel (MFMA-bound).  Few rows: the skinny kernel (HBM-bound).
  // With a workspace the tiled kernel can split K over several workgroups per tile, which fills the device at few rows too.
  kapy_matmul_cfg c = {KAPY_MATMUL_AUTO, 0, 0, 0, KAPY_RN, 0, 0, 0, nullptr, 0};
  if (cfg) c = *cfg;
  // (offsets inside a workgroup's rows and columns are 32-bit)
  const bool block_ok = k_contig && p.M > 16 && p.K % (4 * kBlockStep) == 0 && p.a_sm * 128 < (int64_t(1) << 31) && p.b_sn * kBlockCols < (int64_t(1) << 31) &&
                        ((int64_t)(p.N + kBlockCols - 1) / kBlockCols + 8) * ((p.M + 31) / 32) < (int64_t(1) << 31);
  if (k_pieces && !acc && (result->dtype == KAPY_BF16 || result->dtype == KAPY_F16 || result->dtype == KAPY_F32)) {
    GemmParams g;
    g.a = (const char *)p.a; g.b = (const char *)p.b; g.acc = nullptr; g.d = p.d;
    g.row_scale = row_scale; g.col_scale = col_scale;
    g.bias = nullptr; g.alpha = 1.0f; g.bias_dtype = KAPY_F32; g.act = -1; g.act_operand = 0.f;
    g.a_sm = p.a_sm; g.a_sk = 1; g.b_sn = p.b_sn; g.b_sk = 1;
    g.acc_sm = g.acc_sn = 0; g.d_sm = p.d_sm; g.d_sn = p.d_sn;
    g.M = p.M; g.N = p.N; g.K = p.K;
    g.acc_dtype = -1; g.d_dtype = p.d_dtype; g.rz = p.rz; g.tiles_m = g.tiles_n = 0;
    int rc = plan_split_k(g, c, 128);
    if (rc) return rc;
    // an explicit split is a request for the tiled kernel; the library's own choice weighs it against the block kernel
    const int tiled_from = block_ok && c.split_k <= 1 ? (g.split_k > 1 ? kTiledFromMSplit : kTiledFromM) : (g.split_k > 1 ? kTiledFromMSplitNoBlock : kTiledFromMNoBlock);
    if (k_contig && p.M < tiled_from) rc = KAPY_ERR_UNSUPPORTED;  // few rows: the streaming kernels below (which need whole K steps)
    else rc = matmul_f8_tiled(g, fmt_of(a->dtype), fmt_of(b->dtype), c.tile_m == 256 || c.tile_m == 128 ? c.tile_m : 0, s);
    if (rc != KAPY_ERR_UNSUPPORTED) return rc;
  }
  if (block_ok) {
    const int fa = fmt_of(a->dtype), fb = fmt_of(b->dtype);
    if (p.M <= 32) return launch_skinny_block<2>(p, fa, fb, s);
    if (p.M <= 48) return launch_skinny_block<3>(p, fa, fb, s);
    // 65 .. 128 rows: one block of rows per workgroup still (two stages of up to 20 KiB per wave).  Two blocks of 64 rows would
    // read the weight twice through the L2s and the activation as often; N = K = 8192, M = 80 / 96 / 128: 30.0 / 30.6 / 33.8 us
    // in blocks of 64 rows, 25.2 / 26.5 / 29.5 in one of 128.  Beyond 128 rows: blocks of 64.
    if (p.M <= 64 || p.M > 128) return launch_skinny_block<4>(p, fa, fb, s);
    if (p.M <= 80) return launch_skinny_block<5>(p, fa, fb, s);
    if (p.M <= 96) return launch_skinny_block<6>(p, fa, fb, s);
    if (p.M <= 112) return launch_skinny_block<7>(p, fa, fb, s);
    return launch_skinny_block<8>(p, fa, fb, s);
  }
  if (k_contig && p.K % (kStreamWaves * kStreamChunk) == 0 && (p.M + 15) / 16 <= 65535 && p.a_sm * 16 < (int64_t(1) << 31) &&
      p.b_sn * 16 < (int64_t(1) << 31)) {
    // rows are addressed from the workgroup's first row, so the per-lane offsets stay small
    F8Params q = p;
    // two column groups per wave (half the activation traffic, 96 KiB of LDS per workgroup) where that still gives every CU a workgroup
    const int64_t groups = (p.M + 15) / 16;
    const int ng = groups == 1 && (int64_t)(p.N + 31) / 32 >= device_cus() ? 2 : 1;
    const int64_t col_rounds = ((p.N + 16 * ng - 1) / (16 * ng) + 7) / 8;
    dim3 grid((unsigned)(col_rounds * 8 * groups));
    int fa = fmt_of(a->dtype), fb = fmt_of(b->dtype);
#define KAPY_STREAM(NG_, ST_)                                                                                    \
  do {                                                                                                        \
    if (fa == 0 && fb == 0) skinny_stream_kernel<0, 0, NG_, ST_><<<grid, 64 * kStreamWaves, 0, s>>>(q);       \
    else if (fa == 0) skinny_stream_kernel<0, 1, NG_, ST_><<<grid, 64 * kStreamWaves, 0, s>>>(q);             \
    else if (fb == 0) skinny_stream_kernel<1, 0, NG_, ST_><<<grid, 64 * kStreamWaves, 0, s>>>(q);             \
    else skinny_stream_kernel<1, 1, NG_, ST_><<<grid, 64 * kStreamWaves, 0, s>>>(q);                          \
  } while (0)
    // (rings of three stages measured no faster: N = K = 8192, M = 16: 13.3 us with two column groups either way, 14.8 with one)
    if (ng == 2) KAPY_STREAM(2, kStreamStages);
    else KAPY_STREAM(1, kStreamStages);
#undef KAPY_STREAM
    KAPY_HIP_CHECK(hipGetLastError());
    return KAPY_OK;
  }
  if (k_contig) {
    constexpr int NG = kSkinnyGroups, CH = kSkinnyChunk;
    dim3 grid((unsigned)((p.N + 16 * NG - 1) / (16 * NG)), (unsigned)((p.M + 15) / 16));
    if (grid.y <= 65535) {
      int fa = fmt_of(a->dtype), fb = fmt_of(b->dtype);
      if (fa == 0 && fb == 0) skinny_kernel<0, 0, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      else if (fa == 0) skinny_kernel<0, 1, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      else if (fb == 0) skinny_kernel<1, 0, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      else skinny_kernel<1, 1, NG, CH><<<grid, 64 * kSkinnyWaves, 0, s>>>(p);
      KAPY_HIP_CHECK(hipGetLastError());
      return KAPY_OK;
    }
  }
  const int64_t tiles = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64);
  if (tiles < (int64_t(1) << 31) && (int64_t)p.M * p.N >= 4096) tiled_any_kernel<<<(unsigned)tiles, 256, 0, s>>>(p);
  else naive_kernel<<<(unsigned)(((int64_t)p.M * p.N + 255) / 256), 256, 0, s>>>(p);
  KAPY_HIP_CHECK(hipGetLastError());
  return KAPY_OK;
}

}  // namespace kapy

using namespace kapy;

extern "C" int kapy_matmul_scaled_f8(const kapy_global *a8, const kapy_global *w8, const float *row_scale, const float *col_scale,
                                     const kapy_global *result, const kapy_matmul_cfg *cfg, void *stream) {
  int rc = check_global(a8, "matmul lhs");
  if (!rc) rc = check_global(w8, "matmul rhs");
  if (!rc) rc = check_global(result, "matmul result");
  if (rc) return rc;
  if (!row_scale || !col_scale) return fail(KAPY_ERR_INVALID, "matmul_scaled_f8: null scale array");
  if (!is_f8(a8->dtype) || !is_f8(w8->dtype))
    return fail(KAPY_ERR_VERIFY, "matmul: mma f8 operands must have f8E4M3 or f8E5M2 element type");
  if (extent1(a8) != extent0(w8))
    return fail(KAPY_ERR_VERIFY, "matmul: number of columns of lhs must be equal to number of rows of rhs");
  if (extent0(result) != extent0(a8))
    return fail(KAPY_ERR_VERIFY, "matmul: number of rows of acc must be equal to number of rows of lhs");
  if (extent1(result) != extent1(w8))
    return fail(KAPY_ERR_VERIFY, "matmul: number of columns of acc must be equal to number of columns of rhs");
  if (result->dtype != KAPY_F16 && result->dtype != KAPY_BF16 && result->dtype != KAPY_F32)
    return fail(KAPY_ERR_VERIFY, "matmul: result must have f16, bf16 or f32 element type");
  for (const kapy_global *g : {a8, w8, result})
    if (g->start0 < 0 || g->start1 < 0) return fail(KAPY_ERR_INVALID, "matmul: negative view start");
  if (cfg && cfg->rmode != KAPY_RN && cfg->rmode != KAPY_RZ) return fail(KAPY_ERR_INVALID, "matmul: unknown rounding mode %d", cfg->rmode);
  rc = ensure_device();
  if (rc) return rc;
  return matmul_f8(a8, w8, row_scale, col_scale, nullptr, result, cfg, (hipStream_t)stream);
}
