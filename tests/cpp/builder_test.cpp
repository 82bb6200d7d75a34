// Exercises kapy::OpBuilder (include/kapy_hip.hpp) from C++.  "cpu": what needs no device - the programs the builder
// lowers to, the verifier's refusals as exceptions, the loud failure without a GPU.  "gpu": the same graphs run on the
// device (elementwise chain, transposed store, matmul with a fused tail) against plain host arithmetic.
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "kapy_hip.hpp"

#define EXPECT(cond)                                                       \
  do {                                                                     \
    if (!(cond)) {                                                         \
      printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);             \
      exit(1);                                                             \
    }                                                                      \
  } while (0)

static kapy::Value gelu_chain(kapy::OpBuilder &b, kapy::Value x, kapy::Value bias, kapy_dtype dt) {
  kapy::Value xv = b.create_extf(b.create_ld_global(x), KAPY_F32);
  kapy::Value bv = b.create_broadcast(b.create_extf(b.create_ld_global(bias), KAPY_F32), {0, 0});
  kapy::Value v = b.create_addf(b.create_mulf(xv, b.create_splat(0.5f, KAPY_F32)), bv);
  return b.create_truncf(b.create_elementwise_extern_lib("gelu", v), dt);
}

static int run_cpu() {
  char fake[64];  // descriptors only: nothing is dereferenced on the host
  kapy::OpBuilder b;
  kapy::Value x = b.create_mk_global(fake, 0, 64, 256, 256, 1, KAPY_F16), bias = b.create_mk_global(fake, 0, 1, 256, 256, 1, KAPY_F16);
  kapy::Value y = b.create_mk_global(fake, 0, 64, 256, 256, 1, KAPY_F16);
  std::vector<kapy_global> ins;
  std::vector<kapy_ew_inst> prog = b.program_of(gelu_chain(b, x, bias, KAPY_F16), &ins);
  const int want[] = {KAPY_EW_LD_GLOBAL, KAPY_EW_FPTOFP, KAPY_EW_SPLAT, KAPY_EW_MULF, KAPY_EW_LD_GLOBAL, KAPY_EW_FPTOFP, KAPY_EW_ADDF, KAPY_EW_GELU_TANH,
                      KAPY_EW_FPTOFP, KAPY_EW_ST_GLOBAL};
  EXPECT(prog.size() == sizeof want / sizeof want[0] && ins.size() == 2);
  for (size_t k = 0; k < prog.size(); ++k) EXPECT(prog[k].op == want[k]);
  EXPECT(ins[1].end0 - ins[1].start0 == 1);  // the bias row: extent 1 along axis 0 is the broadcast
  // the library accepts the program: its verifier and the specialised-kernel generator both run without a device
  const kapy_global *ptrs[2] = {&ins[0], &ins[1]};
  kapy_global out;
  EXPECT(kapy_mk_global(&out, fake, 0, 64, 256, 256, 1, KAPY_F16, 16) == KAPY_OK);
  int64_t text = 0;
  EXPECT(kapy_elementwise_source(prog.data(), (int32_t)prog.size(), ptrs, 2, &out, nullptr, 0, &text, nullptr) == KAPY_OK && text > 1000);
  // registers are recycled: a chain of 40 ops fits the 16 registers of a program
  kapy::Value lx = b.create_ld_global(x), v = lx;
  for (int k = 0; k < 40; ++k) v = b.create_addf(v, lx);   // lx stays live throughout, every sum dies at the next one
  prog = b.program_of(v, &ins);
  EXPECT(prog.size() == 42 && ins.size() == 1);
  for (const kapy_ew_inst &I : prog) EXPECT(I.dst >= 0 && I.dst < 16);
  prog = b.program_of(b.create_clampf(lx, b.create_splat(-1.f, KAPY_F16), b.create_splat(1.f, KAPY_F16)));
  EXPECT(prog.size() == 6 && prog[2].op == KAPY_EW_MAXIMUMF && prog[4].op == KAPY_EW_MINIMUMF);
  prog = b.program_of(b.create_clampf(lx, b.create_splat(-1.f, KAPY_F16), b.create_splat(1.f, KAPY_F16), false));   // NaNs do not propagate: maxnumf / minnumf
  EXPECT(prog.size() == 6 && prog[2].op == KAPY_EW_MAXNUMF && prog[4].op == KAPY_EW_MINNUMF);
  prog = b.program_of(b.create_remf(b.create_floor(b.create_sin(lx)), b.create_ceil(b.create_cos(lx))));
  EXPECT(prog.size() == 7 && prog.back().op == KAPY_EW_ST_GLOBAL && prog[5].op == KAPY_EW_REMF);
  // integer, compare and select builders: a causal mask (column <= row) in front of a select, as a program the library verifies
  {
    kapy::Value row = b.create_arange(0, 0, 64), colv = b.create_arange(1, 0, 256);
    kapy::Value keep = b.create_cmpi_sle(colv, row);
    kapy::Value masked = b.create_select(keep, lx, b.create_splat(0.f, KAPY_F16));
    prog = b.program_of(masked, &ins);
    EXPECT(prog.size() == 7 && ins.size() == 1 && prog[5].op == KAPY_EW_SELECT && prog.back().op == KAPY_EW_ST_GLOBAL);
    int n_arange = 0, n_cmp = 0;
    for (const kapy_ew_inst &I : prog) {
      n_arange += I.op == KAPY_EW_ARANGE;
      if (I.op == KAPY_EW_CMPI) { ++n_cmp; EXPECT(I.c == KAPY_CMPI_SLE); }
    }
    EXPECT(n_arange == 2 && n_cmp == 1);
    const kapy_global *one[1] = {&ins[0]};
    EXPECT(kapy_elementwise_source(prog.data(), (int32_t)prog.size(), one, 1, &out, nullptr, 0, &text, nullptr) == KAPY_OK && text > 1000);
    // create_intcast picks the op from the widths; an integer splat carries its value in field a
    kapy::Value wide = b.create_intcast(b.create_splat(-3, KAPY_I8), KAPY_I32, true);
    prog = b.program_of(b.create_sitofp(b.create_addi(wide, b.create_intcast(b.create_splat(300, KAPY_I16), KAPY_I32, false)), KAPY_F16));
    EXPECT(prog[0].op == KAPY_EW_SPLAT && prog[0].a == -3 && prog[1].op == KAPY_EW_EXTSI && prog[3].op == KAPY_EW_EXTUI && prog[4].op == KAPY_EW_ADDI);
    EXPECT(kapy_elementwise_source(prog.data(), (int32_t)prog.size(), one, 0, &out, nullptr, 0, &text, nullptr) == KAPY_OK);
    try {
      b.create_st_global(b.create_select(lx, lx, lx), y);   // the condition is not an i1 tensor
      EXPECT(!"a select on a float condition must be refused");
    } catch (const kapy::Error &e) {
      EXPECT(e.status == KAPY_ERR_VERIFY && strstr(e.what(), "i1"));
    }
  }
  // scalar constants are splat as in the reference (create_constant_* then create_splat), and library functions answer to
  // the names of the device library the reference links
  {
    kapy::Value half = b.create_splat(b.create_constant_float16(0.5f)), three = b.create_splat(b.create_constant_int32(3));
    prog = b.program_of(b.create_mulf(lx, half));
    EXPECT(prog.size() == 4 && prog[1].op == KAPY_EW_SPLAT && prog[1].dtype == KAPY_F16 && prog[1].imm == 0.5f && prog[2].op == KAPY_EW_MULF);
    prog = b.program_of(b.create_sitofp(b.create_addi(three, b.create_splat(b.create_constant_all_ones(KAPY_I32))), KAPY_F16));
    EXPECT(prog[0].op == KAPY_EW_SPLAT && prog[0].a == 3 && prog[1].op == KAPY_EW_SPLAT && prog[1].a == -1 && prog[2].op == KAPY_EW_ADDI);
    prog = b.program_of(b.create_addf(lx, b.create_splat(b.create_constant_float64(0.25), KAPY_F16)));   // a 64-bit scalar names its tensor type
    EXPECT(prog[1].op == KAPY_EW_SPLAT && prog[1].dtype == KAPY_F16 && prog[1].imm == 0.25f);
    prog = b.program_of(b.create_addf(lx, b.create_splat(b.create_constant_zero(KAPY_F16))));
    EXPECT(prog[1].op == KAPY_EW_SPLAT && prog[1].imm == 0.f);
    prog = b.program_of(b.create_elementwise_extern_lib("__nv_tanhf", b.create_elementwise_extern_lib("__nv_expf", lx)));
    EXPECT(prog.size() == 4 && prog[1].op == KAPY_EW_EXP && prog[2].op == KAPY_EW_TANH);
    int refused = 0;
    try { b.create_splat(b.create_constant_int64(1)); } catch (const kapy::Error &e) { refused += e.status == KAPY_ERR_UNSUPPORTED; }
    try { b.create_splat(b.create_constant_float32(1.f), KAPY_I32); } catch (const kapy::Error &e) { refused += e.status == KAPY_ERR_VERIFY; }
    try { b.create_addf(lx, b.create_constant_float16(1.f)); } catch (const kapy::Error &e) { refused += e.status == KAPY_ERR_VERIFY; }
    try { b.create_elementwise_extern_lib("__nv_lgammaf", lx); } catch (const kapy::Error &e) { refused += e.status == KAPY_ERR_UNSUPPORTED; }
    EXPECT(refused == 4);
  }
  // the verifier's refusal arrives as an exception with the reference's wording
  try {
    kapy::Value h = b.create_ld_global(x), w = b.create_ld_global(b.create_mk_global(fake, 0, 64, 256, 256, 1, KAPY_BF16));
    b.create_st_global(b.create_addf(h, w), y);
    EXPECT(!"mixed element types must be refused");
  } catch (const kapy::Error &e) {
    EXPECT(e.status == KAPY_ERR_VERIFY && strstr(e.what(), "same element type"));
  }
  try {
    b.create_addf(x, x);   // a global-memory tensor is not a register tensor
    EXPECT(!"global operands must be refused");
  } catch (const kapy::Error &e) {
    EXPECT(e.status == KAPY_ERR_VERIFY);
  }
  try {
    b.create_st_global(b.create_exp(b.create_matmul(b.create_ld_global(x), b.create_ld_global(x))), y);
    EXPECT(!"exp on a matmul result is not a fusable tail");
  } catch (const kapy::Error &e) {
    EXPECT(e.status == KAPY_ERR_UNSUPPORTED || e.status == KAPY_ERR_VERIFY);
  }
  // what follows a matmul is typed like any other chain: the stored value has the target's element type, a cast to another
  // type or a missing cast is refused, and a 16-bit bias row must be widened before it joins the f32 accumulator
  {
    kapy::Value a16 = b.create_mk_global(fake, 0, 128, 128, 128, 1, KAPY_F16), c16 = b.create_mk_global(fake, 0, 128, 128, 128, 1, KAPY_F16);
    kapy::Value c32 = b.create_mk_global(fake, 0, 128, 128, 128, 1, KAPY_F32), brow = b.create_mk_global(fake, 0, 1, 128, 128, 1, KAPY_F16);
    auto mm = [&] { return b.create_matmul(b.create_ld_global(a16), b.create_ld_global(a16)); };
    auto refused = [&](kapy::Value v, kapy::Value target, int status, const char *words) {
      try {
        b.create_st_global(v, target);
      } catch (const kapy::Error &e) {
        return e.status == status && strstr(e.what(), words) != nullptr;
      }
      return false;
    };
    EXPECT(refused(mm(), c16, KAPY_ERR_VERIFY, "same element type"));                                         // f32 result, f16 view, no cast
    EXPECT(refused(b.create_truncf(mm(), KAPY_BF16), c16, KAPY_ERR_VERIFY, "same element type"));             // cast to another type than the view's
    EXPECT(refused(b.create_truncf(mm(), KAPY_F16), c32, KAPY_ERR_VERIFY, "same element type"));
    EXPECT(refused(b.create_truncf(b.create_addf(mm(), b.create_ld_global(brow)), KAPY_F16), c16, KAPY_ERR_VERIFY, "same element type"));   // f16 bias, not widened
    // a legal chain with a round-toward-zero cast passes the typing and reaches the device call (which fails without a device)
    int n_dev0 = 0;
    if (hipGetDeviceCount(&n_dev0) != hipSuccess || n_dev0 == 0)
      EXPECT(refused(b.create_fptofp(b.create_addf(mm(), b.create_extf(b.create_ld_global(brow), KAPY_F32)), KAPY_F16, KAPY_RZ), c16, KAPY_ERR_HIP, "no CPU fallback"));
  }
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev == 0) {
    try {
      b.create_st_global(gelu_chain(b, x, bias, KAPY_F16), y);
      EXPECT(!"without a device the call must fail");
    } catch (const kapy::Error &e) {
      EXPECT(e.status == KAPY_ERR_HIP && strstr(e.what(), "no CPU fallback"));
    }
  }
  printf("builder cpu ok\n");
  return 0;
}

static float h2f(uint16_t h) { return (float)*reinterpret_cast<_Float16 *>(&h); }
static uint16_t f2h(float f) { _Float16 h = (_Float16)f; return *reinterpret_cast<uint16_t *>(&h); }
static float b2f(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }
static uint16_t f2b(float f) { uint32_t u; memcpy(&u, &f, 4); return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }
#define HIP_OK(e) EXPECT((e) == hipSuccess)

static int run_gpu() {
  const int m = 96, n = 256;
  std::vector<uint16_t> x(m * n), bias(n), y(m * n), yt(m * n);
  srand(7);
  auto rnd = [] { return (float)(rand() % 65536) / 65536.f * 4.f - 2.f; };
  for (auto &v : x) v = f2h(rnd());
  for (auto &v : bias) v = f2h(rnd());
  uint16_t *dx, *db, *dy, *dt;
  HIP_OK(hipMalloc((void **)&dx, x.size() * 2)); HIP_OK(hipMalloc((void **)&db, bias.size() * 2));
  HIP_OK(hipMalloc((void **)&dy, y.size() * 2)); HIP_OK(hipMalloc((void **)&dt, y.size() * 2));
  HIP_OK(hipMemcpy(dx, x.data(), x.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(db, bias.data(), bias.size() * 2, hipMemcpyHostToDevice));
  kapy::OpBuilder b;
  kapy::Value gx = b.create_mk_global(dx, 0, m, n, n, 1, KAPY_F16), gb = b.create_mk_global(db, 0, 1, n, n, 1, KAPY_F16);
  kapy::Value gy = b.create_mk_global(dy, 0, m, n, n, 1, KAPY_F16), gt = b.create_mk_global(dt, 0, n, m, m, 1, KAPY_F16);
  b.create_st_global(gelu_chain(b, gx, gb, KAPY_F16), gy);                  // one fused kernel
  b.create_st_global(b.create_transpose(b.create_ld_global(gy)), gt);       // the layout move of its result
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(y.data(), dy, y.size() * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(yt.data(), dt, yt.size() * 2, hipMemcpyDeviceToHost));
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      const double v = (double)h2f(x[i * n + j]) * 0.5 + h2f(bias[j]);
      const double want = 0.5 * v * (1.0 + tanh(0.7978845608028654 * (v + 0.044715 * v * v * v)));
      const double got = h2f(y[i * n + j]);
      EXPECT(fabs(got - want) <= 2.5 * fmax(fabs(want), 6.1e-5) * 0.0009765625);   // 2 ulp of f16 and a rounding
      EXPECT(yt[j * m + i] == y[i * n + j]);                                       // bit-exact
    }
  // relu(A.B^T * 0.25 + bias) in bf16: matmul with the tail in its epilogue
  const int M = 128, N = 256, K = 128;
  std::vector<uint16_t> a(M * K), w(N * K), c(M * N), bb(N);
  for (auto &v : a) v = f2b(rnd() * 0.25f);
  for (auto &v : w) v = f2b(rnd() * 0.25f);
  for (auto &v : bb) v = f2b(rnd());
  uint16_t *da, *dw, *dc, *dbb;
  HIP_OK(hipMalloc((void **)&da, a.size() * 2)); HIP_OK(hipMalloc((void **)&dw, w.size() * 2));
  HIP_OK(hipMalloc((void **)&dc, c.size() * 2)); HIP_OK(hipMalloc((void **)&dbb, bb.size() * 2));
  HIP_OK(hipMemcpy(da, a.data(), a.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dw, w.data(), w.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dbb, bb.data(), bb.size() * 2, hipMemcpyHostToDevice));
  kapy::Value ga = b.create_mk_global(da, 0, M, K, K, 1, KAPY_BF16), gw = b.create_mk_global(dw, 0, K, N, 1, K, KAPY_BF16);   // B column-major
  kapy::Value gc = b.create_mk_global(dc, 0, M, N, N, 1, KAPY_BF16), gbb = b.create_mk_global(dbb, 0, 1, N, N, 1, KAPY_BF16);
  kapy::Value acc = b.create_matmul(b.create_ld_global(ga), b.create_ld_global(gw));
  kapy::Value t = b.create_addf(b.create_mulf(acc, b.create_splat(0.25f, KAPY_F32)), b.create_extf(b.create_ld_global(gbb), KAPY_F32));
  b.create_st_global(b.create_truncf(b.create_maximumf(t, b.create_splat(0.f, KAPY_F32)), KAPY_BF16), gc);
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(c.data(), dc, c.size() * 2, hipMemcpyDeviceToHost));
  double err2 = 0, ref2 = 0;
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      double s = 0;
      for (int k = 0; k < K; ++k) s += (double)b2f(a[i * K + k]) * b2f(w[j * K + k]);
      const double want = fmax(s * 0.25 + b2f(bb[j]), 0.0), got = b2f(c[i * N + j]);
      err2 += (got - want) * (got - want);
      ref2 += want * want;
    }
  EXPECT(sqrt(err2 / ref2) <= 4e-3);   // bf16 result: half an ulp (2^-9) per element at most, well inside
  // the same chain with a round-toward-zero cast: every element is the RN result or its neighbour toward zero, and never
  // larger in magnitude than the exact value
  std::vector<uint16_t> cz(M * N);
  b.create_st_global(b.create_fptofp(b.create_maximumf(t, b.create_splat(0.f, KAPY_F32)), KAPY_BF16, KAPY_RZ), gc);
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(cz.data(), dc, cz.size() * 2, hipMemcpyDeviceToHost));
  int differ = 0;
  for (int i = 0; i < M * N; ++i) {
    EXPECT(cz[i] == c[i] || cz[i] + 1 == c[i]);   // (results are >= 0 after the relu: the pattern below is the value toward zero)
    differ += cz[i] != c[i];
  }
  EXPECT(differ > M * N / 8);   // about half of all roundings go up under RN
  printf("builder gpu ok\n");
  return 0;
}

// The 256 x 256 x 64 ring kernel (all 160 KiB of a CU's LDS, declared statically) launched from a process that never loaded
// torch: bf16, A row-major, B column-major, through the C ABI with the tile named in the configuration.
static int run_gpu_large_tile() {
  const int M = 512, N = 512, K = 256;
  std::vector<uint16_t> a(M * K), w(N * K), c(M * N);
  srand(11);
  auto rnd = [] { return (float)(rand() % 65536) / 65536.f - 0.5f; };
  for (auto &v : a) v = f2b(rnd());
  for (auto &v : w) v = f2b(rnd());
  uint16_t *da, *dw, *dc;
  HIP_OK(hipMalloc((void **)&da, a.size() * 2)); HIP_OK(hipMalloc((void **)&dw, w.size() * 2)); HIP_OK(hipMalloc((void **)&dc, c.size() * 2));
  HIP_OK(hipMemcpy(da, a.data(), a.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dw, w.data(), w.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(dc, 0, c.size() * 2));
  kapy_global ga, gw, gc;
  EXPECT(kapy_mk_global(&ga, da, 0, M, K, K, 1, KAPY_BF16, 16) == KAPY_OK);
  EXPECT(kapy_mk_global(&gw, dw, 0, K, N, 1, K, KAPY_BF16, 16) == KAPY_OK);
  EXPECT(kapy_mk_global(&gc, dc, 0, M, N, N, 1, KAPY_BF16, 16) == KAPY_OK);
  kapy_matmul_cfg cfg = {KAPY_MATMUL_AUTO, 256, 256, 64, KAPY_RN, 0, 0, 0, nullptr, 0};
  printf("launching the 256 x 256 x 64 ring kernel (M = N = %d, K = %d)\n", M, K);
  fflush(stdout);
  const int rc = kapy_matmul(&ga, &gw, nullptr, &gc, &cfg, nullptr);
  if (rc != KAPY_OK) {
    printf("FAILED: kapy status %d: %s\n", rc, kapy_last_error());
    return 1;
  }
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(c.data(), dc, c.size() * 2, hipMemcpyDeviceToHost));
  double err2 = 0, ref2 = 0;
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      double s = 0;
      for (int k = 0; k < K; ++k) s += (double)b2f(a[i * K + k]) * b2f(w[j * K + k]);
      const double got = b2f(c[i * N + j]);
      err2 += (got - s) * (got - s);
      ref2 += s * s;
    }
  EXPECT(sqrt(err2 / ref2) <= 4e-3);
  printf("builder gpu large tile ok\n");
  return 0;
}

// The 256-wide kernel for row-major x row-major operands (128 KiB of LDS, declared statically) from a process that never
// loaded torch: the library picks it from 0.55 tiles of 256 x 256 per CU; 64 sampled rows against a double-precision sum.
static int run_gpu_row_major_wide() {
  const int M = 3072, N = 3072, K = 128;
  std::vector<uint16_t> a((size_t)M * K), w((size_t)K * N), c((size_t)M * N);
  srand(13);
  auto rnd = [] { return (float)(rand() % 65536) / 65536.f - 0.5f; };
  for (auto &v : a) v = f2b(rnd());
  for (auto &v : w) v = f2b(rnd());
  uint16_t *da, *dw, *dc;
  HIP_OK(hipMalloc((void **)&da, a.size() * 2)); HIP_OK(hipMalloc((void **)&dw, w.size() * 2)); HIP_OK(hipMalloc((void **)&dc, c.size() * 2));
  HIP_OK(hipMemcpy(da, a.data(), a.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dw, w.data(), w.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(dc, 0, c.size() * 2));
  kapy_global ga, gw, gc;
  EXPECT(kapy_mk_global(&ga, da, 0, M, K, K, 1, KAPY_BF16, 16) == KAPY_OK);
  EXPECT(kapy_mk_global(&gw, dw, 0, K, N, N, 1, KAPY_BF16, 16) == KAPY_OK);
  EXPECT(kapy_mk_global(&gc, dc, 0, M, N, N, 1, KAPY_BF16, 16) == KAPY_OK);
  printf("launching the row-major x row-major matmul (M = N = %d, K = %d)\n", M, K);
  fflush(stdout);
  const int rc = kapy_matmul(&ga, &gw, nullptr, &gc, nullptr, nullptr);
  if (rc != KAPY_OK) {
    printf("FAILED: kapy status %d: %s\n", rc, kapy_last_error());
    return 1;
  }
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(c.data(), dc, c.size() * 2, hipMemcpyDeviceToHost));
  double err2 = 0, ref2 = 0;
  for (int t = 0; t < 64; ++t) {
    const int i = (t * 331 + 7) % M;
    for (int j = 0; j < N; ++j) {
      double s = 0;
      for (int k = 0; k < K; ++k) s += (double)b2f(a[(size_t)i * K + k]) * b2f(w[(size_t)k * N + j]);
      const double got = b2f(c[(size_t)i * N + j]);
      err2 += (got - s) * (got - s);
      ref2 += s * s;
    }
  }
  EXPECT(ref2 > 0 && sqrt(err2 / ref2) <= 4e-3);
  printf("builder gpu row-major wide ok\n");
  return 0;
}

int main(int argc, char **argv) {
  try {
    if (argc > 1 && std::string(argv[1]) == "gpu256") return run_gpu_large_tile();
    if (argc > 1 && std::string(argv[1]) == "gpunn256") return run_gpu_row_major_wide();
    return argc > 1 && std::string(argv[1]) == "gpu" ? run_gpu() : run_cpu();
  } catch (const kapy::Error &e) {
    printf("FAILED: kapy status %d: %s\n", e.status, e.what());
    return 1;
  }
}
