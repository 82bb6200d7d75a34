/*
 * kapy_oracle.h — CPU restatement of the kapy-lang op semantics (TEST INFRASTRUCTURE ONLY).
 *
 * This library is the checker the HIP path is compared against.  It is never linked, loaded or
 * called by the product library; only tests, the smoke check and the cpu_baseline leg of the
 * benchmark use it.  Every function cites the reference file:line (relative to the kapy-lang
 * tree) whose semantics it restates.
 *
 * Pinning status (what independent evidence fixes each function; see tests/test_oracle_*.py):
 *   codecs (f16/bf16/e4m3fn/e5m2)   exhaustive against numpy.float16 / torch CPU casts, and
 *                                   against the magic constants held by the reference
 *                                   (ElementwiseOpToLLVM.cpp:83-289, ConvertUtils.cpp:267-334)
 *   fragments maps                  the lane diagram in Kgpu/IR/Attrs.td:28-78, map3∘map2 = id,
 *                                   transpose involution, brute force over power-of-two shapes
 *   swizzle                         bijection per line block, textbook 128-B XOR form at (4,8),
 *                                   brute-force bank replay
 *   descriptors / ld / st / copy    closed-form index formula vs numpy strided views, ragged edges
 *   matmul, scaled fp8 matmul       numpy float64 matmul, identity / all-ones / rank-1 closed forms
 *   elementwise                     numpy float64 closed forms, special values
 * The reference's own tests hold no golden vectors for this path, so nothing here is pinned by
 * the reference beyond the constants and diagrams named above.
 */
#ifndef KAPY_ORACLE_H
#define KAPY_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* dtype / enum numbering is shared with include/kapy_hip.h (enum values follow Enums.td). */
enum { KO_F16 = 0, KO_BF16 = 1, KO_F32 = 2, KO_F8E4M3 = 3, KO_F8E5M2 = 4, KO_I8 = 5, KO_I16 = 6, KO_I32 = 7, KO_I1 = 8 /* one byte, 0 or 1 */ };
enum { KO_RZ = 0, KO_RN = 1 };
enum { KO_PAD_ZERO = 0, KO_PAD_QNAN = 1, KO_PAD_PINF = 2, KO_PAD_NINF = 3 };

typedef struct ko_global {
  void *ptr;
  int32_t start0, start1, end0, end1, stride0, stride1;
  int32_t dtype, alignment;
} ko_global;

typedef struct ko_fragments {
  int32_t lane_array[2];
  int32_t lane_loops[2];
  int32_t minor_axis, major_axis;
} ko_fragments;

typedef struct ko_ew_inst {
  int32_t op, dst, a, b, c;
  int32_t dtype, rmode;
  float imm;
} ko_ew_inst;

int ko_dtype_bits(int dtype);

/* ---- codecs ---- */
uint16_t ko_f64_to_f16(double x, int rmode);
uint16_t ko_f64_to_bf16(double x, int rmode);
uint8_t ko_f64_to_e4m3(double x, int rmode);
uint8_t ko_f64_to_e5m2(double x, int rmode);
float ko_f64_to_f32(double x, int rmode);
double ko_f16_to_f64(uint16_t h);
double ko_bf16_to_f64(uint16_t h);
double ko_e4m3_to_f64(uint8_t b);
double ko_e5m2_to_f64(uint8_t b);
double ko_decode(const void *p, int dtype, int64_t idx);
void ko_encode(void *p, int dtype, int64_t idx, double v, int rmode);
int ko_fptofp(const void *src, int src_dtype, void *dst, int dst_dtype, int rmode, int64_t n,
              int f32_to_f8_via_f16);
uint32_t ko_padding_word(int dtype, int padding);

/* ---- seeded generators ---- */
uint64_t ko_splitmix64(uint64_t x);
void ko_fill_uniform(void *dst, int dtype, int64_t n, uint64_t seed, uint64_t stream, double lo, double hi);
void ko_fill_normal(void *dst, int dtype, int64_t n, uint64_t seed, uint64_t stream, double mean, double stddev);
void ko_fill_bits16(uint16_t *dst, int64_t n, uint64_t seed, uint64_t stream);

/* ---- layouts ---- */
void ko_fragments_loops(const ko_fragments *l, const int64_t shape[2], int64_t warp_loops[2], int64_t loop_space[2]);
int64_t ko_layout_string(const ko_fragments *l, const int64_t shape[2], char *out, int64_t out_len);
void ko_fragments_map12(const ko_fragments *l, const int64_t shape[2], int option, int64_t lane, int64_t iv, int64_t idx[2]);
void ko_fragments_map3(const ko_fragments *l, const int64_t shape[2], int64_t i0, int64_t i1, int64_t *lane, int64_t *iv);
void ko_fragments_transpose(const ko_fragments *l, ko_fragments *out);
void ko_fragments_exchange_axes(const ko_fragments *l, ko_fragments *out);
void ko_fragments_default(const int64_t lane_loops[2], const int64_t shape[2], int row_major, int64_t warp_size, ko_fragments *out);
int64_t ko_access_simd_size(int64_t alignment, int64_t bits, int64_t numel, int64_t warp_size);
void ko_change_source(const ko_fragments *src, const ko_fragments *dst, const int64_t shape[2], int64_t lane, int64_t iv,
                      int64_t *src_lane, int64_t *src_iv);
int64_t ko_change_num_shuffles(const ko_fragments *src, const ko_fragments *dst, const int64_t shape[2], int64_t warp_size);
int64_t ko_swizzle_offset(int64_t i0, int64_t i1, int64_t stride0, int64_t stride1, int64_t bits, int64_t bank_param,
                          int64_t line_param, int64_t num_banks);
int ko_no_bank_conflict(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                        int64_t bank_param, int64_t line_param, int64_t alignment, int64_t num_banks, int64_t warp_size);
int ko_swizzle_search(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                      int64_t alignment, int64_t num_banks, int64_t warp_size, int64_t *out_pairs, int max_pairs);
/* The bank-conflict question asked of the gfx950 LDS (64 banks, 64 lanes; 16-byte reads in four phases of sixteen lanes
 * {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31}, + 32; every atom of a lane's read an instruction of its own) with
 * a key that may be rotated; candidates are (bank_param, line_param, rotate) triples. */
int ko_no_bank_conflict_gfx950(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                               int64_t bank_param, int64_t line_param, int64_t rotate, int64_t alignment);
int ko_swizzle_search_gfx950(const ko_fragments *l, const int64_t shape[2], int64_t stride0, int64_t stride1, int64_t bits,
                             int64_t alignment, int64_t *out_triples, int max_triples);
int64_t ko_swizzle_offset_rotated(int64_t i0, int64_t i1, int64_t stride0, int64_t stride1, int64_t bits, int64_t bank_param,
                                  int64_t line_param, int64_t rotate);

/* ---- descriptors and memory ops ---- */
int ko_mk_global(ko_global *out, void *ptr, int32_t dynamic_offset, int32_t size0, int32_t size1, int32_t stride0,
                 int32_t stride1, int dtype, int32_t alignment);
int ko_sv_global(ko_global *out, const ko_global *src, int32_t start0, int32_t end0, int32_t start1, int32_t end1);
void ko_ld_global(const ko_global *src, int64_t shape0, int64_t shape1, int padding, void *tile);
void ko_st_global(const void *tile, int64_t shape0, int64_t shape1, const ko_global *dst);
void ko_transpose_tile(const void *tile, int64_t shape0, int64_t shape1, int dtype, void *out);
void ko_change_tile(const void *lane_values, const ko_fragments *src, const ko_fragments *dst, const int64_t shape[2],
                    int bytes, int64_t warp_size, void *out_lane_values);
int ko_copy(const ko_global *src, const ko_global *dst, int transpose, int padding);
int ko_copy_batched(const ko_global *src, const ko_global *dst, int transpose, int padding, int32_t n0, int32_t n1,
                    int64_t src_off0, int64_t src_off1, int64_t dst_off0, int64_t dst_off1);

/* ---- compute ops ---- */
int ko_elementwise(const ko_ew_inst *prog, int n_inst, const ko_global *const *ins, int n_ins, const ko_global *out);
int ko_matmul(const ko_global *lhs, const ko_global *rhs, const ko_global *acc, const ko_global *result, int rmode);
/* The same product with f16 accumulators rounded once per k_step (8 or 16) columns of the lhs: the arithmetic of the
 * reference's f16-result instruction strings (MatmulOpToLLVM.cpp:270-291).  f16 operands, accumulator and result only. */
int ko_matmul_f16acc(const ko_global *lhs, const ko_global *rhs, const ko_global *acc, const ko_global *result, int k_step);
int ko_matmul_scaled_f8(const ko_global *a, const ko_global *w, const float *row_scale, const float *col_scale,
                        const ko_global *result);
void ko_quantize_e4m3(const float *x, int64_t rows, int64_t cols, int64_t row_stride, int64_t col_stride,
                      int along_cols, uint8_t *q, float *scale);
int ko_reduce(const ko_global *src, const ko_global *dst, int axis, int kind);
int ko_reduce_reference(const ko_global *src, const ko_global *dst, int axis, int kind, const ko_fragments *layout, int64_t lanes);

int ko_num_threads(void);

/* ---- timing baselines (kapy_baseline.cpp): the benchmark workloads written for speed on the host cores
 * (packed panels + register-blocked fp32 micro-kernel, fused vector loop, cache-blocked tiles; AVX-512 forms
 * chosen at run time).  They are what the benchmark's cpu_baseline leg times; tests/test_oracle_baselines.py
 * checks each against the checker above. ---- */
int ko_baseline_gemm(const ko_global *lhs, const ko_global *rhs, const float *row_scale, const float *col_scale,
                     const ko_global *result, double *multiply_seconds);
int ko_baseline_gelu_f16(const uint16_t *x, const uint16_t *bias, float scale, uint16_t *y, int64_t rows, int64_t cols, int64_t pitch);
int ko_baseline_transpose16(const uint16_t *src, uint16_t *dst, int64_t rows, int64_t cols);
int ko_baseline_permute_bhsd_bshd16(const uint16_t *src, uint16_t *dst, int64_t b, int64_t h, int64_t s, int64_t d);

#ifdef __cplusplus
}
#endif
#endif
