/*
 * kapy_hip.h — C ABI of the MI355X (gfx950) implementation of kapy-lang's hot op path.
 *
 * kapy-lang is a compiler: it has no FFI of its own.  The boundary kept here is its op-level
 * surface — the op builders of python/src/ir.cc:480-1181 and the kernel ABI that
 * lib/Conversion/KgpuToLLVM/FuncOpToLLVM.cpp:55-92 produces (global pointers + i32 scalars, one
 * stream-ordered launch) — at whole-tensor granularity: one call runs the op over the full
 * extent of its descriptors instead of over one warp tile, and the library chooses the tiling.
 * Every entry point cites the reference interface it stands in for.
 *
 * Conventions: plain C types only; all pointers in descriptors are DEVICE pointers owned by the
 * caller (the reference never allocates global memory either); device entry points are
 * asynchronous on the given HIP stream (a hipStream_t passed as void*, NULL = default stream);
 * every function returns KAPY_OK or a negative kapy_status and never throws; the text of the
 * last failure on the calling thread is available from kapy_last_error().  There is no CPU
 * fallback: device entry points fail with KAPY_ERR_HIP when no gfx950 device is usable.
 */
#ifndef KAPY_HIP_H
#define KAPY_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum kapy_status {
  KAPY_OK = 0,
  KAPY_ERR_INVALID = -1,     /* null pointer, unknown enum value, malformed program            */
  KAPY_ERR_VERIFY = -2,      /* an op verifier of the reference rejects the operands           */
  KAPY_ERR_UNSUPPORTED = -3, /* legal in kapy, not implemented on this device                  */
  KAPY_ERR_HIP = -4          /* HIP runtime failure (including "no device")                    */
} kapy_status;

/* Element types of Kapy tensors (include/kapy/Dialect/Kapy/IR/Types.td; f8 = OCP E4M3FN / E5M2). */
typedef enum kapy_dtype {
  KAPY_F16 = 0, KAPY_BF16 = 1, KAPY_F32 = 2, KAPY_F8E4M3 = 3, KAPY_F8E5M2 = 4,
  KAPY_I8 = 5, KAPY_I16 = 6, KAPY_I32 = 7,
  KAPY_I1 = 8 /* the result type of cmpi / cmpf and the condition of select; one byte (0 or 1) in memory */
} kapy_dtype;

/* Enum values equal include/kapy/Dialect/Kapy/IR/Enums.td (python/src/ir.cc:125-156). */
typedef enum kapy_padding_option { KAPY_PAD_ZERO = 0, KAPY_PAD_QNAN = 1, KAPY_PAD_PINF = 2, KAPY_PAD_NINF = 3 } kapy_padding_option;
typedef enum kapy_cache_modifier {
  KAPY_CACHE_NONE = 0, KAPY_CACHE_CA = 1, KAPY_CACHE_CG = 2, KAPY_CACHE_CS = 3,
  KAPY_CACHE_WB = 4, KAPY_CACHE_WT = 5, KAPY_CACHE_LU = 6, KAPY_CACHE_CV = 7
} kapy_cache_modifier;
typedef enum kapy_evict_priority {
  KAPY_EVICT_NORMAL = 0, KAPY_EVICT_FIRST = 1, KAPY_EVICT_LAST = 2, KAPY_EVICT_UNCHANGED = 3, KAPY_NO_ALLOCATE = 4
} kapy_evict_priority;
typedef enum kapy_rounding_mode { KAPY_RZ = 0, KAPY_RN = 1 } kapy_rounding_mode;
/* MatmulImplWay: values 1..4 are the reference's (mma.sync shapes); on gfx950 they only select the
 * operand class (f16/bf16, tf32 — unsupported: CDNA4 has no tf32 MFMA —, f8).  0 lets the library
 * choose; 16..18 name the MFMA shape explicitly. */
typedef enum kapy_matmul_impl_way {
  KAPY_MATMUL_AUTO = 0,
  KAPY_MMA_M16N8K8_F16 = 1, KAPY_MMA_M16N8K16_F16 = 2, KAPY_MMA_M16N8K8_TF32 = 3, KAPY_MMA_M16N8K16_F8 = 4,
  KAPY_MFMA_32X32X16_16B = 16, KAPY_MFMA_16X16X32_16B = 17, KAPY_MFMA_16X16X128_F8 = 18, KAPY_MFMA_32X32X64_F8 = 19
} kapy_matmul_impl_way;

/* Global-memory tensor descriptor: the struct of lib/Conversion/KgpuToLLVM/TypeConverter.cpp:65-73
 * {ptr, start0, start1, end0, end1, stride0, stride1} plus the element type and the kapy.alignment
 * attribute (bytes) that the reference carries on the IR.  Element (i,j) of the view lives at
 * ptr + ((start0+i)*stride0 + (start1+j)*stride1) elements and is in bounds iff
 * (start0+i) <u end0 && (start1+j) <u end1. */
typedef struct kapy_global {
  void *ptr;
  int32_t start0, start1, end0, end1, stride0, stride1;
  int32_t dtype;     /* kapy_dtype */
  int32_t alignment; /* bytes the base pointer and every row start are aligned to */
} kapy_global;

/* #kgpu.fragments<[a0,a1],[l0,l1],(minor,major)> (include/kapy/Dialect/Kgpu/IR/Attrs.td:12-135).
 * The lane count is a0*a1: 64 on gfx950 (32 in the reference). */
typedef struct kapy_fragments {
  int32_t lane_array[2];
  int32_t lane_loops[2];
  int32_t minor_axis, major_axis;
} kapy_fragments;

/* #kapy.swizzling<[stride0,stride1],(bank_param,line_param)> (include/kapy/Dialect/Kapy/IR/Attrs.td:54-81).  rotate (not in
 * the reference, 0 there): the XOR key is line % line_param rotated left by this many bits within log2(line_param) bits; the
 * search over the gfx950 read phases (kapy_swizzle_search_gfx950) finds layouts that need it. */
typedef struct kapy_swizzling {
  int32_t stride0, stride1, bank_param, line_param, rotate;
} kapy_swizzling;

/* ---------------------------------------------------------------- library */
int kapy_version(void);
/* Text of the last error on this thread; mirrors the reference's emitOpError messages. */
const char *kapy_last_error(void);
/* Device facts used for dispatch: CU count, wavefront size, LDS bytes per workgroup, arch name. */
int kapy_device_info(int32_t *num_cus, int32_t *wave_size, int32_t *lds_bytes, char *arch, int32_t arch_len);

/* ---------------------------------------------------------------- descriptors (host only) */
/* kapy.mk_global — create_mk_global, python/src/ir.cc:1013-1025; MkGlobalOpToLLVM.cpp:23-47. */
int kapy_mk_global(kapy_global *out, void *ptr, int32_t dynamic_offset, int32_t size0, int32_t size1,
                   int32_t stride0, int32_t stride1, int32_t dtype, int32_t alignment);
/* kapy.sv_global — create_sv_global(src, start0, end0, start1, end1), python/src/ir.cc:1026-1034;
 * SvGlobalOpToLLVM.cpp:22-40: both new bounds are offsets from the source view's start. */
int kapy_sv_global(kapy_global *out, const kapy_global *src, int32_t start0, int32_t end0, int32_t start1, int32_t end1);

/* Shared-memory tensor descriptor: the struct of TypeConverter.cpp:74-82 {ptr AS3, start0, start1, end0, end1} with the
 * pointer as a byte offset into the workgroup's shared memory (shared_array + kapy.offset, MkSharedOpToLLVM.cpp:49-70),
 * plus the element type and the #kapy.swizzling layout that the reference carries on the tensor type. */
typedef struct kapy_shared {
  int64_t offset; /* bytes from the start of the workgroup's shared memory (kapy.offset; kapy_smem_plan assigns these) */
  int32_t start0, start1, end0, end1;
  int32_t dtype;  /* kapy_dtype */
  kapy_swizzling layout;
} kapy_shared;
/* kapy.mk_shared - create_mk_shared(shape, elementType, rowMajor), python/src/ir.cc:1050-1061; MkSharedOpToLLVM.cpp:49-70:
 * start 0, end = shape, strides (size1, 1) row-major or (1, size0) column-major (Analyze.cpp:82-95).  (bank_param,
 * line_param) is the swizzling of the buffer, (0, 0) = none; kapy_swizzle_search finds the conflict-free ones. */
int kapy_mk_shared(kapy_shared *out, int64_t byte_offset, int32_t size0, int32_t size1, int32_t dtype, int32_t row_major,
                   int32_t bank_param, int32_t line_param);
/* kapy.sv_shared - create_sv_shared(src, start0, end0, start1, end1), ir.cc:1062-1070; SvSharedOpToLLVM.cpp:20-42:
 * same base and layout, both new bounds are offsets from the source view's start. */
int kapy_sv_shared(kapy_shared *out, const kapy_shared *src, int32_t start0, int32_t end0, int32_t start1, int32_t end1);
/* Byte address in the workgroup's shared memory of element (i0, i1) of the view: offset + the swizzled position of
 * (start0 + i0, start1 + i1) (the address function of CpAsyncOpToLLVM.cpp:124-139, 64 banks); KAPY_ERR_VERIFY (negative)
 * for an element outside the view, which a load pads and a store skips. */
int64_t kapy_shared_address(const kapy_shared *tensor, int64_t i0, int64_t i1);

/* ---------------------------------------------------------------- layout engine (host only) */
/* FragmentsLayoutAttr::getWarpLoops / getLoopSpace — lib/Dialect/Kgpu/IR/Kgpu.cpp:164-184. */
int kapy_fragments_loops(const kapy_fragments *layout, const int64_t shape[2], int64_t warp_loops[2], int64_t loop_space[2]);
/* FragmentsLayoutAttr::getAffineMap(shape, option) — Kgpu.cpp:186-251.  option 1/2: in = (lane, iv),
 * out = (i0, i1); option 3: in = (i0, i1), out = (lane, iv). */
int kapy_fragments_map(const kapy_fragments *layout, const int64_t shape[2], int32_t option, const int64_t in[2], int64_t out[2]);
/* getLayoutString — Kgpu.cpp:293-353, what bin/kapy-layout.cpp prints: for every element of a tensor of
 * `shape`, row by row, the owning "T<lane>:<loop iv>", one block per replication round.  Writes at most
 * out_len bytes (NUL-terminated) and returns the full length of the text, or a negative kapy_status. */
int64_t kapy_layout_string(const kapy_fragments *layout, const int64_t shape[2], char *out, int64_t out_len);
/* FragmentsLayoutAttr::transpose / exchangeAxes — Kgpu.cpp:253-263. */
int kapy_fragments_transpose(const kapy_fragments *layout, kapy_fragments *out);
int kapy_fragments_exchange_axes(const kapy_fragments *layout, kapy_fragments *out);
/* getFragmentsLayout(laneLoops, type, rowMajor) — lib/Support/LayoutUtils.cpp:92-104, 64 lanes. */
int kapy_fragments_default(const int64_t lane_loops[2], const int64_t shape[2], int32_t row_major, kapy_fragments *out);
/* getGlobalSimdSize — lib/Dialect/Kgpu/Transforms/CoalesceAccess.cpp:18-27, 64 lanes. */
int64_t kapy_access_simd_size(int64_t alignment, int64_t bits, int64_t numel);
/* ChangeOpHelper::getShflIdxMap / getNumShfls — LayoutUtils.cpp:61-90. */
int kapy_change_source(const kapy_fragments *src, const kapy_fragments *dst, const int64_t shape[2], int64_t lane,
                       int64_t iv, int64_t *src_lane, int64_t *src_iv);
int64_t kapy_change_num_shuffles(const kapy_fragments *src, const kapy_fragments *dst, const int64_t shape[2]);
/* Swizzled element offset — CpAsyncOpToLLVM.cpp:124-139 (same in LdMatrix/LdShared/StShared), for
 * the 64-bank x 4-byte LDS of gfx950 (a line is 256 bytes). */
int64_t kapy_swizzle_offset(const kapy_swizzling *layout, int64_t bits, int64_t i0, int64_t i1);
/* getSwizzlingLayouts — LayoutUtils.cpp:167-225 re-parameterised for 64 banks and 64 lanes: writes
 * up to max_pairs (bank_param, line_param) candidates in the reference's search order, returns the count. */
int kapy_swizzle_search(const kapy_fragments *access, const int64_t shape[2], int64_t stride0, int64_t stride1,
                        int64_t bits, int64_t alignment, int32_t *pairs, int32_t max_pairs);
/* The same search asked the way the gfx950 LDS serves a wave: the model of LayoutUtils.cpp:167-209 looks at the first
 * lanes of the warp and a lane's first access (NVIDIA's quarter-warp rule for 16-byte accesses); gfx950 serves 16-byte reads
 * in four phases of sixteen lanes {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31}, the same plus 32, 8-byte reads in
 * two halves, and every 16-byte piece of a longer per-lane read as an instruction of its own.  A candidate passes when no
 * phase of no instruction asks a bank for two lines.  Candidates are (bank_param, line_param, rotate) triples in the
 * reference's order with the key rotations innermost; writes up to max_triples, returns the count.  The tiled matmul
 * kernels stage their operands in the first hit for their matrix instruction's operand reads (kapy_matmul_lds_layout). */
int kapy_swizzle_search_gfx950(const kapy_fragments *access, const int64_t shape[2], int64_t stride0, int64_t stride1,
                               int64_t bits, int64_t alignment, int32_t *triples, int32_t max_triples);
/* getDefaultLayouts(MatmulOp) — LayoutUtils.cpp:123-149 for the MFMA shapes of gfx950:
 * which = 0 lhs [m x k], 1 rhs [k x n], 2 acc [m x n] of the instruction as documented; 3 = acc [m x n] when the
 * instruction is issued with the operands exchanged (rhs fragment in the first slot: legal without moving a register
 * because the lhs and rhs layouts mirror each other; the instruction then computes the transposed block and a lane's
 * register quad holds four consecutive columns of one row).  The tiled matmul kernels issue form 3, the decode-shaped
 * fp8 kernels form 2; all of them take their lane positions from these layouts.  Also reports the tile (m, n, k). */
int kapy_matmul_layouts(int32_t impl_way, int32_t which, kapy_fragments *out, int32_t mnk[3]);
/* The LDS layout the tiled matmul stages its operands in (first hit of kapy_swizzle_search_gfx950 on the operand layout of
 * the matrix instruction the tiles of that depth are built on: tile_k 32 -> 32x32x16, tile_k 64 -> 16x16x32), so callers and
 * tests can check it is conflict-free by construction. */
int kapy_matmul_lds_layout(int32_t operand_dtype, int32_t tile_k, kapy_swizzling *out);

/* ---------------------------------------------------------------- device ops */
typedef struct kapy_copy_cfg {
  int32_t transpose;      /* 1: kapy.transpose between the load and the store (dst[i,j] = src[j,i]) */
  int32_t padding_option; /* kapy_padding_option of the ld_global                                   */
  int32_t cache_modifier; /* kapy_cache_modifier; CS / CG select non-temporal access                */
  int32_t evict_priority; /* kapy_evict_priority, looked at when cache_modifier is NONE (as the reference's lowering does,
                             LdGlobalOpToLLVM.cpp:103-109): EVICT_FIRST / NO_ALLOCATE = non-temporal access, EVICT_LAST /
                             EVICT_UNCHANGED = ordinary cached access, EVICT_NORMAL = the library's choice (non-temporal
                             for moves too large to be re-read from the Infinity Cache) */
  int32_t is_volatile;    /* the reference's ld.volatile / st.volatile drop every cache hint (same lines); here too:
                             ordinary accesses whatever cache_modifier and evict_priority say.  Every element is read
                             and written exactly once either way */
  int32_t reserved;
} kapy_copy_cfg;

/* ld_global -> [transpose] -> st_global over the destination view's full extent.
 * Stands in for create_ld_global / create_transpose / create_st_global, python/src/ir.cc:1035-1049,
 * 1087-1090 (LdGlobalOpToLLVM.cpp:60-145, TransposeOpToLLVM.cpp:21-26, StGlobalOpToLLVM.cpp:60-139).
 * Source elements out of bounds read as padding; destination elements out of bounds are not written.
 * Element types must have equal width; bits move untouched. cfg may be NULL (no transpose, zero padding). */
int kapy_copy(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg, void *stream);

/* A 2-D grid of programs (kapy.program_id axes 0 and 1, ParallelIdOpToLLVM.cpp:28-38), program (p0,p1)
 * running kapy_copy on views displaced by p0*off0 + p1*off1 ELEMENTS, i.e. mk_global's dynamic_offset
 * affine in the program ids.  (b,h,s,d)->(b,s,h,d) is grid (b,h) over [s x d] views. */
typedef struct kapy_grid2 {
  int32_t n0, n1;
  int64_t src_off0, src_off1, dst_off0, dst_off1;
} kapy_grid2;
int kapy_copy_batched(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg, const kapy_grid2 *grid, void *stream);

/* Elementwise programs: a straight-line list of kapy/arith/math ops over at most 16 virtual
 * registers, evaluated for every element of `out`'s extent (create_{addf,mulf,fma,exp,...},
 * create_fptofp, create_splat, create_broadcast, python/src/ir.cc:744-1157; lowering
 * ElementwiseOpToLLVM.cpp:424-1238).  A register has a dtype; arithmetic on f16/bf16/f32 registers
 * rounds once to that dtype after every op.  LD_GLOBAL of an input whose extent is 1 along an axis
 * broadcasts along it (kapy.broadcast, Kapy.cpp:686-698).  A program with a REDUCE is a row-wise fusion (softmax,
 * layer norm ...): it runs in one pass over HBM with each row resident on chip, and needs axis 1, rows that are
 * contiguous, a multiple of 8 and at most 32768 elements long, zero padding, and operands that are full, row,
 * column or scalar views (KAPY_ERR_UNSUPPORTED otherwise; a width that is not a multiple of 8, with rows that still
 * start aligned to 8 elements, is served by compiling a kernel on the first call, see kapy_elementwise_specialize).
 * A program whose reduces run along axis 0 (ReduceOpToLLVM.cpp:51-172 reduces either axis; at most 4 of them) takes
 * any views, shapes and padding: a workgroup owns 64 columns and re-reads its operands once per reduce, keeping only the
 * per-column results on chip, so it moves (reduces + 1) times the operand bytes and is not a one-pass kernel.  The reduces
 * of one program must all run along the same axis. */
typedef enum kapy_ew_op {
  KAPY_EW_LD_GLOBAL = 0, /* dst <- ins[a]            (c = kapy_padding_option)                  */
  KAPY_EW_SPLAT,         /* dst <- imm as `dtype`    (kapy.splat); for an integer `dtype` the value is field a */
  KAPY_EW_FPTOFP,        /* dst <- cast(a) to `dtype`, `rmode` on down-casts (kapy.fptofp/extf/truncf) */
  KAPY_EW_ADDF, KAPY_EW_SUBF, KAPY_EW_MULF, KAPY_EW_DIVF,
  KAPY_EW_FMA,           /* dst <- a*b + c                                                     */
  KAPY_EW_MAXIMUMF, KAPY_EW_MINIMUMF, KAPY_EW_NEGF, KAPY_EW_ABSF,
  KAPY_EW_EXP, KAPY_EW_EXP2, KAPY_EW_LOG, KAPY_EW_LOG2, KAPY_EW_SQRT, KAPY_EW_RSQRT,
  KAPY_EW_TANH, KAPY_EW_ERF, /* the extern-lib calls of create_elementwise_extern_lib, ir.cc:1168-1174 */
  KAPY_EW_GELU_TANH,     /* dst <- 0.5*a*(1+tanh(sqrt(2/pi)*(a+0.044715*a^3))), one rounding       */
  KAPY_EW_ST_GLOBAL,     /* out <- a                                                              */
  KAPY_EW_REDUCE_SUM,    /* dst <- sum of a along axis b, kept on every element of that axis: kapy.reduce  */
  KAPY_EW_REDUCE_MAX,    /*        with an addf / maximumf combiner followed by kapy.broadcast; accumulated */
                         /*        in fp32, rounded once to the register's type (as kapy_reduce)           */
  KAPY_EW_FLOOR, KAPY_EW_CEIL, /* math.floor / math.ceil (create_floor, create_ceil; UnaryOpConversion, ElementwiseOpToLLVM.cpp:1222-1223) */
  KAPY_EW_SIN, KAPY_EW_COS,    /* math.sin / math.cos (create_sin, create_cos; :1224-1225)                          */
  KAPY_EW_MAXNUMF, KAPY_EW_MINNUMF, /* arith.maxnumf / minnumf: a NaN operand is ignored (create_maxnumf, create_minnumf; :1201-1206) */
  KAPY_EW_REMF,          /* arith.remf: the remainder of a / b with the sign of a, exact (create_remf; :1192)   */
  /* Integer, compare, select and conversion ops on tensors (BinaryOpConversion / UnaryOpConversion over arith ops,
   * ElementwiseOpToLLVM.cpp:1178-1215; arith.select, SelectOpToLLVM.cpp:21-98; kapy.arange, ArangeOpToLLVM.cpp:22-50;
   * builders create_addi ... create_select, python/src/ir.cc:730-1167).  Integer registers (i1, i8, i16, i32) are signless
   * as in MLIR: the op names the signedness, results wrap to the register's width.  Where MLIR leaves a result undefined
   * this library and its checker define it: x / 0 = 0 and x % 0 = 0, the most negative value divided by -1 wraps (its
   * remainder is 0), a shift by the width or more gives 0 (shrsi: the sign), fptosi saturates and turns NaN into 0. */
  KAPY_EW_ADDI, KAPY_EW_SUBI, KAPY_EW_MULI, KAPY_EW_DIVSI, KAPY_EW_DIVUI, KAPY_EW_FLOORDIVSI, KAPY_EW_CEILDIVSI, KAPY_EW_CEILDIVUI,
  KAPY_EW_REMSI, KAPY_EW_REMUI, KAPY_EW_ANDI, KAPY_EW_ORI, KAPY_EW_XORI, KAPY_EW_SHLI, KAPY_EW_SHRSI, KAPY_EW_SHRUI,
  KAPY_EW_MAXSI, KAPY_EW_MAXUI, KAPY_EW_MINSI, KAPY_EW_MINUI, /* dst <- a op b, both of one integer type            */
  KAPY_EW_ABSI,          /* math.absi (create_absi)                                                              */
  KAPY_EW_CMPI,          /* dst (i1) <- a <pred> b on integers, c = a kapy_cmpi_predicate; create_cmpi_*      */
  KAPY_EW_CMPF,          /* dst (i1) <- a <pred> b on floats,   c = a kapy_cmpf_predicate; create_cmpf_*      */
  KAPY_EW_SELECT,        /* dst <- a ? b : c, a an i1 register, b and c of one type (create_select)               */
  KAPY_EW_TRUNCI, KAPY_EW_EXTSI, KAPY_EW_EXTUI, /* dst <- a as integer type `dtype` (create_intcast)             */
  KAPY_EW_SITOFP,        /* dst <- the signed integer a as float type `dtype` (f16, bf16, f32), one RN rounding    */
  KAPY_EW_FPTOSI,        /* dst <- the float a as integer type `dtype`, toward zero                               */
  KAPY_EW_BITCAST,       /* dst <- the bits of a as type `dtype` of the same width (a NaN may come out quieted)     */
  KAPY_EW_ARANGE,        /* dst (i32) <- a + the element's index along axis b: kapy.arange broadcast over the other axis */
  KAPY_EW_NUM_OPS
} kapy_ew_op;
/* arith.cmpi / arith.cmpf predicates, numbered as in MLIR's ArithBase.td (what create_cmpi_* / create_cmpf_* pass). */
typedef enum kapy_cmpi_predicate {
  KAPY_CMPI_EQ = 0, KAPY_CMPI_NE = 1, KAPY_CMPI_SLT = 2, KAPY_CMPI_SLE = 3, KAPY_CMPI_SGT = 4, KAPY_CMPI_SGE = 5,
  KAPY_CMPI_ULT = 6, KAPY_CMPI_ULE = 7, KAPY_CMPI_UGT = 8, KAPY_CMPI_UGE = 9
} kapy_cmpi_predicate;
typedef enum kapy_cmpf_predicate {
  KAPY_CMPF_FALSE = 0, KAPY_CMPF_OEQ = 1, KAPY_CMPF_OGT = 2, KAPY_CMPF_OGE = 3, KAPY_CMPF_OLT = 4, KAPY_CMPF_OLE = 5, KAPY_CMPF_ONE = 6,
  KAPY_CMPF_ORD = 7, KAPY_CMPF_UEQ = 8, KAPY_CMPF_UGT = 9, KAPY_CMPF_UGE = 10, KAPY_CMPF_ULT = 11, KAPY_CMPF_ULE = 12, KAPY_CMPF_UNE = 13,
  KAPY_CMPF_UNO = 14, KAPY_CMPF_TRUE = 15
} kapy_cmpf_predicate;
typedef struct kapy_ew_inst {
  int32_t op, dst, a, b, c;
  int32_t dtype, rmode;
  float imm;
} kapy_ew_inst;
int kapy_elementwise(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins,
                     const kapy_global *out, void *stream);

/* Compiles the program once to device code of its own, as the reference does for every function
 * (translate_mlir_to_llvm / translate_llvm_to_ptx, python/src/passes.cc:141-261), and keeps it for the current
 * device: later kapy_elementwise calls with the same program, operand element types and operand shapes of the
 * same kind (full, row, column, scalar) run it instead of the stepwise machines.  Worth it for programs that
 * none of the hand-written kernels match and that are launched many times: the first compile in a process takes
 * seconds, later ones about a quarter of a second.  The descriptors only say how operands are shaped and typed;
 * their pointers are not read (only their alignment).  Needs one store, reduces only along rows (axis 1) of at most
 * 32768 elements, zero padding, a result contiguous along one axis whose lines start aligned to 8 elements (any
 * width), full operands that are row- or column-major (a view with swapped strides: the transpose is fused; 16-byte
 * aligned along the contiguous axis), row, column or scalar operands; a program with
 * reduces is compiled for the row-length class of `out` (64, 256 or 1024 lanes times 1-4 vectors of 8) and serves
 * that class only.  KAPY_ERR_UNSUPPORTED otherwise, or when the runtime compiler (libhiprtc) is not
 * installed -- kapy_elementwise keeps working either way.  A program that the hand-written kernels already serve
 * with its activation compiled in (act(x*s + bias) with GELU or no activation, plain binary ops) returns KAPY_OK
 * without compiling anything.  Not to be called while a stream is capturing.  kapy_elementwise does this by itself
 * for a program that no hand-written kernel matches when the program comes back: its first call with an operand signature
 * runs on the stepwise machines, its second compiles (never while the stream is capturing; a program that does not compile
 * is not tried again).  KAPY_EW_AUTO_SPECIALIZE=1 in the environment: already on the first call; =0: never.
 * KAPY_EW_CACHE_DIR=<dir> keeps the compiled code objects on disk for later processes. */
int kapy_elementwise_specialize(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins,
                                const kapy_global *out);
/* How many specialised kernels this process holds and how many kapy_elementwise calls have run one (either pointer
 * may be NULL): lets a caller check that a program it specialised is the code that runs. */
int kapy_elementwise_specialize_stats(int64_t *loaded, int64_t *launches);
/* The text kapy_elementwise_specialize would compile (up to capacity-1 bytes, NUL-terminated, into source if not
 * NULL; its full length into *source_bytes if not NULL), and, if code_bytes is not NULL, the size of the gfx950
 * code object it compiles to.  Needs no GPU: the counterpart of reading the reference's generated PTX. */
int kapy_elementwise_source(const kapy_ew_inst *prog, int32_t n_inst, const kapy_global *const *ins, int32_t n_ins,
                            const kapy_global *out, char *source, int64_t capacity, int64_t *source_bytes, int64_t *code_bytes);

/* kapy.fptofp over whole tensors (create_fptofp, python/src/ir.cc:744-754; verifier
 * lib/Dialect/Kapy/IR/Kapy.cpp:272-287): dst[i,j] = cast(src[i,j]), rounding per `rmode`. */
int kapy_fptofp(const kapy_global *src, const kapy_global *dst, int32_t rmode, void *stream);

typedef struct kapy_matmul_cfg {
  int32_t impl_way;              /* kapy_matmul_impl_way                                         */
  int32_t tile_m, tile_n, tile_k; /* workgroup tile; 0 = library's choice                          */
  int32_t rmode;                 /* rounding of the final cast to result dtype (default RN)      */
  int32_t stages;                /* depth of the LDS ring in tiles (the reference fixture uses 2); 25 = the 2.5-tile
                                    ring of half-operand units; 0 = library's choice */
  int32_t waves;                 /* wavefronts per workgroup (num_warps of the reference); 0 = library's choice */
  int32_t split_k;               /* workgroups that share one output tile, each multiplying one part of K (powers of two up to 8);
                                    1 = never split; 0 = library's choice: it splits only when a workspace is given and the
                                    result has too few 128 x 128 tiles to occupy the device */
  void *workspace;               /* device memory for the partial sums and arrival counters of a split K (and, when large enough,
                                    for an operand turned K-contiguous: kapy_matmul_turn_workspace_bytes), or NULL.  Its first
                                    16 KiB (the counters) must be zero before its first use and every call leaves them zero;
                                    256-byte aligned; calls that share a workspace must not overlap in time */
  int64_t workspace_bytes;       /* kapy_matmul_workspace_bytes(m, n) is enough for any split of an [m x n] result */
  int32_t accumulate;            /* kapy_matmul_accumulate; 0 = fp32 accumulators, one cast at the end */
  int32_t reserved;              /* 0 */
} kapy_matmul_cfg;
/* What the running sum of a matmul is held in.  The reference's instruction for f16 operands and an f16 result carries f16
 * accumulators (MatmulOpToLLVM.cpp:270-291, mma.sync ... .f16.f16.f16.f16), so its K loop (MatmulOpToLLVM.cpp:207-262) rounds
 * the sum to f16 once per instruction: every 16 columns of the lhs for mma_m16n8k16_f16, every 8 for mma_m16n8k8_f16.
 * KAPY_ACCUMULATE_ELEMENT reproduces that (f16 operands, accumulator and result only; cfg->impl_way =
 * KAPY_MMA_M16N8K8_F16 selects the 8-column cadence, anything else 16; tile, stage, wave and split fields are ignored; a
 * small kernel for checking programs against the reference's numbers, not a fast path).  KAPY_ACCUMULATE_F32, the
 * default, is more accurate and what every tuned kernel does. */
typedef enum kapy_matmul_accumulate { KAPY_ACCUMULATE_F32 = 0, KAPY_ACCUMULATE_ELEMENT = 1 } kapy_matmul_accumulate;
/* Workspace size that lets the library split K for an [m x n] result whichever way it chooses. */
int64_t kapy_matmul_workspace_bytes(int64_t m, int64_t n);
/* Workspace size with which a LARGE 16-bit problem (at least 6144 rows for a row-major rhs - unless the lhs is row-major
 * too and K a multiple of 64, which a kernel of its own multiplies in place -, at least 6144 columns
 * for a column-major lhs, at least 2048 of the other, K at least 1024, all multiples of 8) is multiplied by first turning that
 * operand into the workspace (behind the 16 KiB of counters, which stay zero) with the transposing copy and then running
 * the K-contiguous kernel on 256 x 256 tiles: 1.15 - 1.2 x the rate of the kernel that reads such operands in place on
 * 128 x 128 tiles, the extra pass over the operand included.  0 when neither operand needs turning.  Used only with a free tile choice and no explicit split; a smaller
 * workspace, or a smaller problem, is multiplied in place as before.  The turned copy is scratch: nothing reads it after
 * the call's kernels have run. */
int64_t kapy_matmul_turn_workspace_bytes(const kapy_global *lhs, const kapy_global *rhs);

/* kapy.matmul — create_matmul(lhs, rhs, acc, implWay), python/src/ir.cc:1101-1105; verifier
 * lib/Dialect/Kapy/IR/Kapy.cpp:451-574; lowering MatmulOpToLLVM.cpp:58-311 with the
 * cp_async/ld_matrix pipeline of CpAsyncOpToLLVM.cpp and LdMatrixOpToLLVM.cpp.
 * result[M,N] = lhs[M,K]·rhs[K,N] (+ acc[M,N]), fp32 accumulate, one final cast to result->dtype.
 * Operand layouts come from the descriptor strides (row- or column-major, either operand).  A column-major result is
 * computed as the transposed problem (result^T = rhs^T . lhs^T, cfg->tile_m and tile_n exchanged with it): the same bits,
 * through the row-major store path.
 * acc may be NULL (zero).  cfg may be NULL. */
int kapy_matmul(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result,
                const kapy_matmul_cfg *cfg, void *stream);

/* kapy_matmul for callers that cannot allocate or hand over device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same operands, same results bit for bit as kapy_matmul with a workspace, but the
 * workspace of a split K is a 16 MiB + 16 KiB array that is part of the library's own device image (one per GPU, held until
 * the process ends); cfg->workspace is ignored.  It calls no allocating routine.  A problem whose split would need more
 * (m x n beyond 512K elements at the widest split) is multiplied without a split, exactly as kapy_matmul without a
 * workspace would.  All calls on one GPU share the array: calls that overlap in time on one GPU (different streams or
 * host threads) race; calls on one stream, or otherwise ordered, are safe.  The first call on a device asks the runtime
 * for the address of that device's copy of the array (hipGetSymbolAddress): make it before a capture begins; every later
 * call on that device records or launches kernels and nothing else.  This entry point has no counterpart in the
 * reference, which never owns device memory (its kernels get every buffer as an argument, FuncOpToLLVM.cpp:55-92). */
int kapy_matmul_static_workspace(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *acc, const kapy_global *result,
                                 const kapy_matmul_cfg *cfg, void *stream);

/* kapy.matmul with the elementwise ops that follow it on the accumulator fused into the same kernel, which is how a
 * kapy.func that multiplies and then applies bias and activation compiles (one kernel; the accumulator never leaves
 * registers): result = fptofp_rn( act( addf( mulf(matmul(lhs, rhs), splat alpha), broadcast(extf bias) ) ) ),
 * every op on fp32 with its own rounding (create_matmul, create_mulf, create_broadcast, create_addf,
 * create_elementwise_extern_lib, create_fptofp: python/src/ir.cc:744-1174).  16-bit operands (fp8: kapy_matmul_scaled_f8). */
typedef struct kapy_matmul_epilogue {
  const kapy_global *bias; /* one contiguous row [1 x N] of f16, bf16 or f32, broadcast along M; NULL = no addf */
  float alpha;             /* 1.0f = no mulf                                                                  */
  int32_t act;             /* applied last: -1 (none), KAPY_EW_GELU_TANH, NEGF, ABSF, or KAPY_EW_MAXIMUMF /
                              KAPY_EW_MINIMUMF against splat(act_operand) (relu = MAXIMUMF with 0); the other
                              unary ops: KAPY_ERR_UNSUPPORTED (run them as a program on the result)            */
  float act_operand;
} kapy_matmul_epilogue;
int kapy_matmul_fused(const kapy_global *lhs, const kapy_global *rhs, const kapy_global *result, const kapy_matmul_epilogue *epi,
                      const kapy_matmul_cfg *cfg, void *stream);

/* W8A8: result[m,n] = cast( (sum_k a8[m,k]·w8[k,n]) · row_scale[m] · col_scale[n] ).
 * In kapy terms: matmul (mma f8, f32 acc) -> mulf with broadcast(row_scale [Mx1]) and
 * broadcast(col_scale [1xN]) -> fptofp rn.  Scales are dense fp32 device arrays.
 * cfg (may be NULL): split_k / workspace as for kapy_matmul; tile_m = 128 or 256 asks for that tile of the tiled kernel
 * (0: the library's choice - 256 x 256 x 128 on the 16x16x128 instruction from 0.55 such tiles per CU, 128 x 128 x 128 below). */
int kapy_matmul_scaled_f8(const kapy_global *a8, const kapy_global *w8, const float *row_scale, const float *col_scale,
                          const kapy_global *result, const kapy_matmul_cfg *cfg, void *stream);

/* kgpu.change on one wavefront's registers (lib/Conversion/KgpuToLLVM/ChangeOpToLLVM.cpp:21-93):
 * lane_values_in[lane*n_src + iv] under `src` is re-distributed to lane_values_out[lane*n_dst + iv]
 * under `dst`, 32-bit values, moved with wave64 ds_bpermute shuffles.  n_* = loop-space sizes. */
int kapy_change(const uint32_t *lane_values_in, const kapy_fragments *src, const kapy_fragments *dst,
                const int64_t shape[2], uint32_t *lane_values_out, void *stream);

/* kapy.reduce along `axis` (Ops.td:441-457, ReduceOpToLLVM.cpp:51-172).  The op's combiner is a region; the regions that are
 * one arith op are named here (what create_reduce's callers write: addf, maximumf ... xori).  dst has extent 1 along `axis`.
 * The elements themselves are folded, as the lowering does (no identity element joins them): a line of only -0 sums to -0;
 * maximumf / minimumf order -0 below +0 and a NaN wins, maxnumf / minnumf ignore NaNs unless every element is one. */
typedef enum kapy_reduce_combiner {
  KAPY_REDUCE_ADDF = 0, KAPY_REDUCE_MAXIMUMF = 1, KAPY_REDUCE_MINIMUMF = 2, KAPY_REDUCE_MULF = 3, KAPY_REDUCE_MAXNUMF = 4, KAPY_REDUCE_MINNUMF = 5,
  KAPY_REDUCE_ADDI = 6, KAPY_REDUCE_MULI = 7, KAPY_REDUCE_MAXSI = 8, KAPY_REDUCE_MINSI = 9, KAPY_REDUCE_MAXUI = 10, KAPY_REDUCE_MINUI = 11,
  KAPY_REDUCE_ANDI = 12, KAPY_REDUCE_ORI = 13, KAPY_REDUCE_XORI = 14
} kapy_reduce_combiner;
typedef enum kapy_reduce_arithmetic {
  KAPY_REDUCE_WIDE = 0,      /* float combiners fold in fp32 and round once to dst's type (any of f16, bf16, f32); the order of the
                                additions is the library's, fixed for a given call (the same bits every run)                   */
  KAPY_REDUCE_REFERENCE = 1  /* the lowering's own arithmetic on one wavefront's tile: every combiner application is an op on the
                                ELEMENT type (an f16 addf rounds each partial sum to f16), each lane folds the elements it holds
                                under `layout` in loop order, then the lanes that share a reduced line fold by butterfly
                                exchanges at lane distances laneOffset * 2^i, i = 0, 1, ... (ReduceOpToLLVM.cpp:76-119, laneOffset
                                and the number of rounds from LayoutUtils.cpp:26-49) - on 64 lanes here.  src must be a
                                power-of-two tile, dst of src's element type                                                  */
} kapy_reduce_arithmetic;
typedef struct kapy_reduce_cfg {
  int32_t combiner;        /* kapy_reduce_combiner; the integer ones need i8 / i16 / i32 tensors, dst of src's type                */
  int32_t arithmetic;      /* kapy_reduce_arithmetic                                                                              */
  const kapy_fragments *layout; /* REFERENCE: how the tile sits in the wavefront's registers; NULL = the default layout of
                                LayoutUtils.cpp:92-110 for a row-major tile on 64 lanes                                          */
  void *workspace;         /* device memory for partial results and arrival counters of launches that share a reduced axis out over
                              workgroups, or NULL: then a 4 MiB + 16 KiB array in the library's device image serves, which every
                              call on that GPU without a workspace shares - such calls must not overlap in time (streams that run
                              concurrently: give each a workspace).  The first 16 KiB (the counters) must be zero before the
                              first use; every call leaves them zero                                                            */
  int64_t workspace_bytes; /* kapy_reduce_workspace_bytes() is enough for any call; with less the library shares out less        */
} kapy_reduce_cfg;
/* Everything on `stream`, nothing allocated, no host-side state: a workgroup that owns part of a reduced line leaves an fp32
 * partial result in the workspace and counts itself; the last to arrive folds the partials in a fixed order. */
int kapy_reduce_ex(const kapy_global *src, const kapy_global *dst, int32_t axis, const kapy_reduce_cfg *cfg, void *stream);
int64_t kapy_reduce_workspace_bytes(void);
/* kapy_reduce_ex with combiner = kind (0 = addf, 1 = maximumf, ...), WIDE arithmetic and the library's own workspace array. */
int kapy_reduce(const kapy_global *src, const kapy_global *dst, int32_t axis, int32_t kind, void *stream);

/* Static plan of a workgroup's shared memory (lib/Analysis/AllocAnalysis.cpp:187-270): buffers whose live
 * ranges [live_start, live_end) (op ids) intersect get disjoint byte ranges, others may share.  Fills
 * `offset` of every buffer (multiples of `alignment`, 0 = the reference's 128) and returns the bytes to
 * allocate, or a negative kapy_status.  Placement rule and order are the reference's; where its loop would not
 * end (it returns first-colour buffers to offset 0 on every pass) offsets are only allowed to grow. */
typedef struct kapy_smem_buffer {
  int64_t size;                  /* bytes                       */
  int64_t live_start, live_end;  /* live over [start, end)      */
  int64_t offset;                /* out                         */
} kapy_smem_buffer;
int64_t kapy_smem_plan(kapy_smem_buffer *buffers, int32_t n_buffers, int64_t alignment);

/* Where a program needs workgroup barriers (lib/Analysis/BlockAnalysis.cpp:37-88 and :114-169).  `ops` are
 * grouped by basic block in ascending block order, in program order inside a block; block 0 is the entry;
 * successors of block b are succ[succ_begin[b] .. succ_begin[b+1]).  kind 0 = an op that reads and writes the
 * byte ranges accesses[first_access .. +n_accesses) of shared memory, 1 = a barrier, 2 = cp_async_wait_group.
 * On return barrier[i] has bit 0 set when a barrier is needed before op i (a read-after-write,
 * write-after-read or write-after-write against accesses pending since the last barrier on some path) and bit 1
 * when one is needed after it (a wait_group that no barrier follows).  Returns the number of barriers, or a
 * negative kapy_status. */
typedef struct kapy_smem_op {
  int32_t block, kind, first_access, n_accesses;
} kapy_smem_op;
typedef struct kapy_smem_access {
  int64_t begin, end;  /* bytes [begin, end) of the workgroup's shared memory */
  int32_t is_write, reserved;
} kapy_smem_access;
int kapy_smem_barriers(const kapy_smem_op *ops, int32_t n_ops, const kapy_smem_access *accesses, int32_t n_accesses,
                       const int32_t *succ_begin, const int32_t *succ, int32_t n_blocks, int32_t *barrier);

/* Runs a kapy.func given in the textual form of the reference's Kapy-dialect fixtures
 * (test/Conversion/KapyToKgpu/elementwise_add.mlir, reduce_sum.mlir, matmul.mlir; op syntax from
 * include/kapy/Dialect/Kapy/IR/Ops.td) on the device: every program id of `grid` is executed in turn, for every warp id of the
 * module's kapy.num_warps, each tensor op as one call of the entry points above on
 * `stream` (mk_global/sv_global/sv_shared: MkGlobalOpToLLVM.cpp:23-47, SvGlobalOpToLLVM.cpp:22-40,
 * SvSharedOpToLLVM.cpp:20-42; ld_global/st_global/cp_async_global_to_shared/ld_matrix: kapy_copy; arith on
 * tensors, math.exp / exp2 / log / log2 / sqrt / rsqrt / tanh / erf / absf / fma, kapy.fptofp, arith.extf / truncf,
 * kapy.splat, kapy.broadcast: kapy_elementwise; kapy.transpose: kapy_copy; kapy.reduce: kapy_reduce; kapy.matmul:
 * kapy_matmul; scf.for with iter_args).
 * A chain of elementwise ops (arith / math on tensors, casts, splats, tensor constants, broadcasts, and the
 * kapy.ld_global of a whole view that feeds them) is not run op by op: it stays deferred until an op of another kind, a loop's yield or a store needs it, and
 * then runs as ONE kapy_elementwise program (at most 8 distinct tensors read, 16 values, 48 instructions; a longer
 * chain is cut where it stops fitting), a kapy.st_global storing straight into its global view (after computing
 * whatever deferred value still has to read memory the store overlaps); a kapy.reduce along axis 1 whose result is
 * broadcast back to its operand's shape is an instruction of that program: the counterpart of
 * the reference compiling the ops of a function into one kernel body.  KAPY_MLIR_FUSE=0 in the environment runs
 * every op as a call of its own instead; results are the same bit for bit.
 * The warps of a program instance advance in step: an op is executed for every warp id before the next op is, and an
 * scf.for whose bounds all warps agree on is iterated jointly, so there is in effect a barrier between any two ops
 * and warps may exchange data through shared memory wherever the program itself is race-free (the barriers
 * kapy_analyze_mlir places are a subset of these).  A loop whose bounds differ between warps runs warp after warp;
 * KAPY_MLIR_IN_STEP=0 in the environment runs every warp to the end before the next one starts.
 * The program instances of the grid advance in step too, in groups as large as the arena allows (every program its own
 * shared-memory tensors).  Where all instances and warps in flight reach a kapy.st_global of chains of one form whose views
 * - the result's and every loaded operand's - tile a rectangle over the same tensors (an operand moves with the tile along
 * an axis or is a broadcast row, column or scalar), the store runs as ONE call over the union: one launch per op for
 * the whole grid, as the reference's one kernel per function (FuncOpToLLVM.cpp:72-88).  Chains with register or shared
 * operands, an arange, or a reduce across the axis the tiles lie along run per instance as before, and so do loads,
 * copies into shared memory and kapy.matmul.  KAPY_MLIR_BATCH=0: one instance at a time, nothing merged; same results.
 * `args` follow the function's signature: a device pointer (with the size of its allocation in bytes, 0 =
 * unknown, which mk_global is checked against) for !kapy.ptr<1>, an i32 otherwise.  A sub-view that leaves
 * its parent is an error.  func_name NULL = the first function of the module.  The first call on a device allocates
 * a 2 GiB arena for shared-memory and register tensors (about 360 four-warp program instances advance in step in it), which the library keeps until the process ends; calls take
 * turns at it, and a call synchronises `stream` before it returns: it is a way to run the reference's programs against
 * this library, not a fast path.
 * The device calls of a run that succeeded are kept (the last 16 runs): a later call with the same text, function name,
 * grid, argument values (every field of every kapy_mlir_arg), device and KAPY_MLIR_* modes makes the same calls again
 * without parsing or interpreting - which calls a run makes cannot depend on the tensors' contents.  In a kept run,
 * consecutive copies, or matrix products of 16-bit row-major operands, that have one shape, lie in different places and do
 * not touch each other's results - the same kapy.ld_matrix, kapy.cp_async_global_to_shared or kapy.matmul of every
 * instance and warp in flight - are one launch each over a table of their addresses, with the bits of the calls they
 * stand for: one launch per op for the whole grid there too (a kept run with tables holds them in device memory of its
 * own, 16 bytes per copy and 32 per product, until it leaves the cache).  KAPY_MLIR_PLAN=0 in the environment turns the
 * keeping off, KAPY_MLIR_PLAN_BATCH=0 the tables. */
typedef struct kapy_mlir_arg {
  void *ptr;      /* device pointer, for a !kapy.ptr<1> argument                    */
  int64_t bytes;  /* size of the allocation behind ptr; 0 = unknown (no range check) */
  int32_t i32;    /* value, for an i32 argument                                      */
  int32_t reserved;
} kapy_mlir_arg;
int kapy_run_mlir(const char *mlir_text, const char *func_name, const kapy_mlir_arg *args, int32_t n_args,
                  const int32_t grid[3], void *stream);
/* How many kapy.st_global ops this process has run as ONE call for all program instances and warps in flight (the instances'
 * chains had the same form and their views tiled a rectangle): lets a caller check that a program took that path. */
int kapy_run_mlir_stats(int64_t *merged_stores);
/* How many runs this process has kept the calls of, how many calls of kapy_run_mlir were served from a kept run, and how
 * many launches over a table of operand addresses those made (any pointer may be NULL). */
int kapy_run_mlir_plan_stats(int64_t *plans, int64_t *replays, int64_t *table_launches);
/* The parsing half of kapy_run_mlir, without a device: KAPY_ERR_INVALID for text that does not parse,
 * KAPY_ERR_UNSUPPORTED for an op outside the set above; otherwise the function's argument count, its number
 * of ops (loop bodies included) and the module's kapy.num_warps.  Out pointers may be NULL. */
int kapy_parse_mlir(const char *mlir_text, const char *func_name, int32_t *n_args, int32_t *n_ops, int32_t *num_warps);
/* Shared-memory plan and barrier positions of a kapy.func in textual form, without a device: one buffer per
 * kapy.mk_shared in program order, live from the first to the last op that defines or uses it or a sub-view or
 * select of it (lib/Analysis/AllocAnalysis.cpp:86-185), placed by kapy_smem_plan with the reference's 128-byte
 * alignment; then kapy_smem_barriers over the function's control flow with ld_matrix / ld_shared reading and
 * cp_async_global_to_shared / st_shared writing the whole buffers their operand may alias.  barrier_lines gets
 * +line for a barrier needed before the op on that source line and -line for one after it.  kapy_run_mlir places
 * shared-memory tensors by this plan and refuses a program that needs more than a workgroup's 160 KiB. */
int kapy_analyze_mlir(const char *mlir_text, const char *func_name, int64_t *smem_bytes, int32_t *n_buffers, int64_t *offsets,
                      int32_t max_buffers, int32_t *n_barriers, int32_t *barrier_lines, int32_t max_barriers);

#ifdef __cplusplus
}
#endif
#endif /* KAPY_HIP_H */
