// elementwise_row.hip — the row machine: elementwise programs with a reduce along the rows (softmax,
// layer norm, RMS norm ...), one pass over HBM with each row resident on chip.  kapy.reduce with an addf /
// maximumf combiner (Ops.td:441-457, ReduceOpToLLVM.cpp:51-172) and the kapy.broadcast of its result
// (BroadcastOpToLLVM.cpp:25-52) fused with the elementwise ops around them.
//
// A workgroup owns one row.  Lane t holds CH chunks of 8 elements, chunk c at vector c*THREADS + t of the
// row.  Values come in two kinds: row values (one fp32 per element: up to NS stack slots of CH*8 registers)
// and per-row values (a reduce's result, a constant, a [m x 1] operand and whatever is computed from
// those: one register each on a second stack of four).  The host compiles the program's DAG into steps
// that name their slots statically, so no register is indexed at run time; a row value used again while
// it still sits lower on the stack is copied from there, one that has been overwritten in between is
// parked in LDS by its first evaluation and read back by the lane that wrote it.
#include <string.h>

#include <algorithm>
#include <functional>
#include <vector>

#include "ew_row_machine.hpp"

namespace kapy {

// the kernels that carry the general step (elementwise_row_narrow.hip, elementwise_row_any.hip)
int launch_row_narrow(const StackProgram &P, int ns, hipStream_t s);
int launch_row_any(const StackProgram &P, int ns, hipStream_t s);

namespace {

// ---------------------------------------------------------------------------------------------
// Host: the program's DAG compiled into steps.
struct RowBuilder {
  struct N {
    int op, a = -1, b = -1, c = -1, dtype = -1, rmode = KAPY_RN, input = -1;
    float imm = 0.f;
  };
  std::vector<N> nodes;
  std::vector<char> uniform;  // one value per row?
  std::vector<int> uses, need;
  int stored = -1;
  StackProgram *P = nullptr;
  int out_dtype = 0;

  // per run
  bool full_first = false;  // a row operand before its per-row partner (keeps the row operand on the stack for the partner's own use of it)
  bool dry = true, ok = true;
  int count = 0, max_slot = 0, n_tmps = 0;
  int holder[3], holder_u[kUSlots];
  std::vector<int> tmp_of;
  std::vector<char> parked, read_back;

  void push(int op, int a, int dtype, int rmode, int slot, float imm, int flags = 0, int k = 0) {
    if (count >= kMaxPost || slot > 2 || k >= kUSlots) { ok = false; return; }
    max_slot = std::max(max_slot, slot);
    P->post[count++] = PostOp{(int16_t)op, (int16_t)a, (int16_t)dtype, (int16_t)rmode, slot | flags | (k << 8), imm};
  }
  static int reversed(int op) { return op == KAPY_EW_SUBF ? kRevSub : op == KAPY_EW_DIVF ? kRevDiv : op; }
  bool is_reduce(int id) const { return nodes[id].op == KAPY_EW_REDUCE_SUM || nodes[id].op == KAPY_EW_REDUCE_MAX; }

  // row slots an expression needs (a per-row expression needs them only while its reduces run)
  void compute_need() {
    need.assign(nodes.size(), 0);
    for (size_t id = 0; id < nodes.size(); ++id) {
      const N &n = nodes[id];
      auto nf = [&](int x) { return std::max(need[x], 1); };
      if (uniform[id]) {
        if (is_reduce((int)id)) need[id] = nf(n.a);
        else need[id] = std::max(n.a >= 0 ? need[n.a] : 0, std::max(n.b >= 0 ? need[n.b] : 0, n.c >= 0 ? need[n.c] : 0));
      } else if (n.op == KAPY_EW_LD_GLOBAL) need[id] = 1;
      else if (n.op == KAPY_EW_FMA) need[id] = std::max(nf(n.a), std::max(nf(n.b) + 1, nf(n.c) + 2));
      else if (n.b >= 0) {
        if (n.a == n.b) need[id] = nf(n.a);
        else if (uniform[n.a] || uniform[n.b]) {
          const int f = uniform[n.a] ? n.b : n.a, un = uniform[n.a] ? n.a : n.b;
          need[id] = std::max(nf(f), need[un]);  // the better of the two orders; the other needs need[un] + 1
        } else need[id] = std::min(std::max(nf(n.a), nf(n.b) + 1), std::max(nf(n.b), nf(n.a) + 1));
      } else need[id] = nf(n.a);
    }
  }

  // node id into per-row value k; row slots from d and per-row values above k are free
  void emit_uni(int id, int d, int k) {
    if (!ok) return;
    if (k >= kUSlots) { ok = false; return; }
    const N &n = nodes[id];
    if (uses[id] > 1 && n.op != KAPY_EW_SPLAT)
      for (int below = 0; below < k; ++below)
        if (holder_u[below] == id) {
          push(kPick, below, n.dtype, 0, 0, 0.f, kUniformResult, k);
          holder_u[k] = id;
          return;
        }
    switch (n.op) {
    case KAPY_EW_SPLAT: push(kPushImm, 0, n.dtype, 0, 0, n.imm, kUniformResult, k); break;
    case KAPY_EW_LD_GLOBAL: push(kPushIn, n.input, n.dtype, 0, 0, 0.f, kUniformResult, k); break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX: {
      int from = -1;
      for (int s = 0; s <= std::min(d, 2); ++s)
        if (holder[s] == n.a) from = s;  // the operand already sits on the stack: a reduce only reads it
      if (from < 0) {
        emit_full(n.a, d, k);
        from = d;
      }
      push(n.op, 0, n.dtype, 0, from, 0.f, 0, k);
      break;
    }
    case KAPY_EW_FPTOFP:
      emit_uni(n.a, d, k);
      if (n.dtype != KAPY_F32) push(kCast, 0, n.dtype, n.rmode, 0, 0.f, kUniformResult, k);  // values are fp32 images: widening changes nothing
      break;
    case KAPY_EW_FMA:
      emit_uni(n.a, d, k); emit_uni(n.b, d, k + 1); emit_uni(n.c, d, k + 2);
      push(KAPY_EW_FMA, 0, n.dtype, 0, 0, 0.f, kUniformResult, k);
      break;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF:
      emit_uni(n.a, d, k); emit_uni(n.b, d, k + 1);
      push(n.op, 0, n.dtype, 0, 0, 0.f, kUniformResult, k);
      break;
    default: emit_uni(n.a, d, k); push(n.op, 0, n.dtype, 0, 0, 0.f, kUniformResult, k);
    }
    for (int above = k + 1; above < kUSlots; ++above) holder_u[above] = -1;
    holder_u[k] = id;
  }

  // node id into row slot d; row slots above d and per-row values from k are free
  void emit_full(int id, int d, int k) {
    if (!ok) return;
    if (d > 2) { ok = false; return; }
    if (holder[d] == id) return;  // still there from an evaluation that only read it since
    const N &n = nodes[id];
    if (uniform[id]) {
      emit_uni(id, d, k);
      push(kPushU, 0, n.dtype, 0, d, 0.f, 0, k);
      holder[d] = id;
      return;
    }
    const bool shared_value = uses[id] > 1;
    if (shared_value) {
      for (int below = 0; below < d; ++below)
        if (holder[below] == id) {
          push(kPick, below, n.dtype, 0, d, 0.f);
          holder[d] = id;
          return;
        }
      if (parked[id]) {
        read_back[id] = 1;
        push(kPushTmp, dry ? 0 : tmp_of[id], n.dtype, 0, d, 0.f);
        holder[d] = id;
        return;
      }
    }
    switch (n.op) {
    case KAPY_EW_LD_GLOBAL: push(kPushIn, n.input, n.dtype, 0, d, 0.f); break;
    case KAPY_EW_FPTOFP:
      emit_full(n.a, d, k);
      // values are fp32 images, so widening changes nothing; and the store rounds to nearest itself
      if (n.dtype != KAPY_F32 && !(id == stored && n.dtype == out_dtype && n.rmode != KAPY_RZ && uses[id] == 1)) push(kCast, 0, n.dtype, n.rmode, d, 0.f);
      break;
    case KAPY_EW_FMA:
      emit_full(n.a, d, k); emit_full(n.b, d + 1, k); emit_full(n.c, d + 2, k);
      push(KAPY_EW_FMA, 0, n.dtype, 0, d, 0.f);
      break;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF:
      if (n.a == n.b) {
        emit_full(n.a, d, k);
        push(n.op, 0, n.dtype, 0, d, 0.f, kSameOperand);
      } else if (uniform[n.a] || uniform[n.b]) {
        const bool left_uniform = uniform[n.a] != 0;
        const int f = left_uniform ? n.b : n.a, un = left_uniform ? n.a : n.b;
        if (full_first && need[un] > 0) { emit_full(f, d, k); emit_uni(un, d + 1, k); }
        else { emit_uni(un, d, k); emit_full(f, d, k + 1); }
        push(left_uniform ? reversed(n.op) : n.op, 0, n.dtype, 0, d, 0.f, kUniformRight, k);
      } else {
        auto nf = [&](int x) { return std::max(need[x], 1); };
        const bool a_first = std::max(nf(n.a), nf(n.b) + 1) <= std::max(nf(n.b), nf(n.a) + 1);
        if (a_first) { emit_full(n.a, d, k); emit_full(n.b, d + 1, k); push(n.op, 0, n.dtype, 0, d, 0.f); }
        else { emit_full(n.b, d, k); emit_full(n.a, d + 1, k); push(reversed(n.op), 0, n.dtype, 0, d, 0.f); }
      }
      break;
    default: emit_full(n.a, d, k); push(n.op, 0, n.dtype, 0, d, 0.f);
    }
    for (int above = d + 1; above < 3; ++above) holder[above] = -1;
    holder[d] = id;
    if (shared_value) {
      parked[id] = 1;
      if (dry || tmp_of[id] >= 0) push(kSaveTmp, dry ? 0 : tmp_of[id], n.dtype, 0, d, 0.f);
    }
  }

  // one whole emission; returns false when the program does not fit
  bool run(bool full_first_, bool dry_) {
    full_first = full_first_;
    dry = dry_;
    ok = true;
    count = 0;
    max_slot = 0;
    for (int &h : holder) h = -1;
    for (int &h : holder_u) h = -1;
    parked.assign(nodes.size(), 0);
    emit_full(stored, 0, 0);
    push(kStore, 0, out_dtype, 0, 0, 0.f);
    return ok;
  }
  // cost of a strategy: parked values first (LDS traffic and footprint), then row slots, then steps
  bool build(bool full_first_, int *cost) {
    tmp_of.assign(nodes.size(), -1);
    read_back.assign(nodes.size(), 0);
    n_tmps = 0;
    if (!run(full_first_, true)) return false;
    for (size_t id = 0; id < nodes.size(); ++id)
      if (read_back[id]) tmp_of[id] = n_tmps++;
    if (!run(full_first_, false)) return false;
    *cost = n_tmps * 1000 + (max_slot + 1) * 100 + count;
    return true;
  }
};

}  // namespace

int run_row_program(const kapy_ew_inst *prog, int n_inst, const int *result_dtype, const kapy_global *const *ins, int n_ins, const kapy_global *out,
                    hipStream_t stream) {
  const char *why = "elementwise: a program with a reduce needs axis 1, contiguous rows of a multiple of 8 and at most 32768 elements, zero "
                    "padding, full / row / column / scalar operands of float type, one st_global and at most three row values in flight";
  RowBuilder B;
  int reg[kMaxRegs];
  for (int r = 0; r < kMaxRegs; ++r) reg[r] = -1;
  int n_store = 0;
  for (int k = 0; k < n_inst; ++k) {
    const kapy_ew_inst &I = prog[k];
    RowBuilder::N n;
    n.op = I.op;
    n.dtype = result_dtype[k];
    n.rmode = I.rmode;
    n.imm = I.imm;
    switch (I.op) {
    case KAPY_EW_LD_GLOBAL:
      n.input = I.a;
      if (I.c != KAPY_PAD_ZERO) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
      break;
    case KAPY_EW_SPLAT: break;
    case KAPY_EW_ST_GLOBAL: B.stored = reg[I.a]; ++n_store; continue;
    case KAPY_EW_FMA: n.a = reg[I.a]; n.b = reg[I.b]; n.c = reg[I.c]; break;
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case KAPY_EW_MULF: case KAPY_EW_DIVF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF:
      n.a = reg[I.a]; n.b = reg[I.b]; break;
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX:
      if (I.b != 1) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
      n.a = reg[I.a];
      break;
    default: n.a = reg[I.a];
    }
    B.nodes.push_back(n);
    reg[I.dst] = (int)B.nodes.size() - 1;
  }
  if (n_store != 1 || B.stored < 0) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  StackProgram SP;
  memset(&SP, 0, sizeof SP);
  const int64_t o0 = extent0(out), o1 = extent1(out);
  const int ob = dtype_bytes(out->dtype);
  if (!is_float(out->dtype) || out->stride1 != 1 || o1 % 8 != 0 || o1 / 8 > 4096 || ((uintptr_t)view_base(out) % (8 * ob)) || (out->stride0 * ob) % (8 * ob) ||
      o0 >= (int64_t(1) << 31) - 1)
    return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  for (int k = 0; k < n_ins; ++k) {
    const kapy_global *g = ins[k];
    StackIn &in = SP.in[k];
    in.base = view_base(g);
    in.stride0 = g->stride0;
    in.dtype = g->dtype;
    if (!is_float(g->dtype)) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
    const int64_t e0 = extent0(g), e1 = extent1(g);
    const int eb = dtype_bytes(g->dtype);
    const bool vec_ok = g->stride1 == 1 && ((uintptr_t)in.base % (8 * eb)) == 0 && (g->stride0 * eb) % (8 * eb) == 0;
    if (e0 == o0 && e1 == o1 && vec_ok) in.kind = kInFull;
    else if (e0 == 1 && e1 == o1 && vec_ok) in.kind = kInRow;
    else if (e1 == 1 && e0 == o0) in.kind = kInCol;
    else if (e0 == 1 && e1 == 1) in.kind = kInScalar;
    else return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  }
  const size_t nn = B.nodes.size();
  B.uniform.assign(nn, 0);
  for (size_t id = 0; id < nn; ++id) {
    const RowBuilder::N &n = B.nodes[id];
    if (B.is_reduce((int)id) || n.op == KAPY_EW_SPLAT) B.uniform[id] = 1;
    else if (n.op == KAPY_EW_LD_GLOBAL) B.uniform[id] = SP.in[n.input].kind == kInCol || SP.in[n.input].kind == kInScalar;
    else B.uniform[id] = (n.a < 0 || B.uniform[n.a]) && (n.b < 0 || B.uniform[n.b]) && (n.c < 0 || B.uniform[n.c]);
  }
  B.uses.assign(nn, 0);
  {
    std::vector<char> reached(nn, 0);
    std::function<void(int)> visit = [&](int id) {
      ++B.uses[id];
      if (reached[id]) return;
      reached[id] = 1;
      const RowBuilder::N &n = B.nodes[id];
      if (n.a >= 0) visit(n.a);
      if (n.b >= 0 && n.b != n.a) visit(n.b);
      if (n.c >= 0) visit(n.c);
    };
    visit(B.stored);
  }
  B.compute_need();
  B.out_dtype = out->dtype;
  // two evaluation orders for an op with one row operand and one per-row operand; the cheaper program wins
  StackProgram best;
  int best_cost = -1, best_ns = 0, best_tmps = 0;
  for (int order = 0; order < 2; ++order) {
    StackProgram cand = SP;
    B.P = &cand;
    int cost = 0;
    if (!B.build(order == 1, &cost)) continue;
    if (best_cost < 0 || cost < best_cost) {
      best = cand;
      best.n_post = B.count;
      best_cost = cost;
      best_ns = B.max_slot + 1;
      best_tmps = B.n_tmps;
    }
  }
  if (best_cost < 0) return fail(KAPY_ERR_UNSUPPORTED, "%s", why);
  best.n_ins = n_ins;
  best.out = (char *)view_base(out);
  best.out_stride0 = out->stride0;
  best.out_dtype = out->dtype;
  best.rows = (int32_t)o0;
  best.vec_per_row = (int32_t)(o1 / 8);
  best.n_tmps = best_tmps;
  bool narrow = out->dtype == KAPY_F16 || out->dtype == KAPY_BF16;
  for (int k = 0; k < n_ins; ++k) narrow = narrow && (ins[k]->dtype == KAPY_F16 || ins[k]->dtype == KAPY_BF16);
  for (int k = 0; k < n_inst; ++k) narrow = narrow && !is_f8(result_dtype[k]);
  // the light kernel takes programs whose row steps all have cheap forms
  bool light = narrow;
  for (int k = 0; k < best.n_post && light; ++k) {
    const PostOp &I = best.post[k];
    if (I.slot & kUniformResult) continue;
    switch (I.op) {
    case KAPY_EW_REDUCE_SUM: case KAPY_EW_REDUCE_MAX: case kPick: case kPushU: case kSaveTmp: case kPushTmp: case kPushIn: case kPushImm: case kStore:
    case KAPY_EW_ADDF: case KAPY_EW_SUBF: case kRevSub: case KAPY_EW_MULF: case KAPY_EW_MAXIMUMF: case KAPY_EW_MINIMUMF: case KAPY_EW_FMA:
    case KAPY_EW_NEGF: case KAPY_EW_ABSF: case KAPY_EW_RSQRT: case KAPY_EW_SQRT: case KAPY_EW_GELU_TANH:
      break;
    case KAPY_EW_EXP: light = I.dtype == KAPY_F32; break;
    case KAPY_EW_DIVF: light = (I.slot & kUniformRight) != 0; break;
    case kCast: light = I.dtype == KAPY_F32 || I.rmode != KAPY_RZ; break;
    default: light = false;
    }
  }
  if (light) return launch_row_kernel<kModeLight>(best, best_ns, stream);
  return narrow ? launch_row_narrow(best, best_ns, stream) : launch_row_any(best, best_ns, stream);
}

}  // namespace kapy
