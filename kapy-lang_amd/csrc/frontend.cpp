// frontend.cpp — executes a kapy.func written in the textual form of the reference's fixtures
// (test/Conversion/KapyToKgpu/{elementwise_add,reduce_sum,matmul}.mlir) by driving the C ABI.
//
// The reference compiles such a function to one PTX kernel; here every program of the launch grid
// and every warp of the program is run in turn on the host, and every tensor op is one library call
// on the caller's stream: mk_global / sv_global / sv_shared are descriptor arithmetic
// (MkGlobalOpToLLVM.cpp:23-47, SvGlobalOpToLLVM.cpp:22-40, SvSharedOpToLLVM.cpp:20-42), ld_global /
// st_global / cp_async_global_to_shared / ld_matrix are kapy_copy between descriptors, arith ops on
// register tensors are one-op elementwise programs, kapy.reduce and kapy.matmul are the entry points
// of the same name.  Shared-memory tensors and register tensors live in a device arena that the call
// allocates and frees.  It is a way to run the reference's own programs against this library, not a
// fast path: a program costs tens of launches.
//
// Supported: func arguments (!kapy.ptr<1>, i32), arith.constant (i32, float scalar, dense tensor), arith
// addi/subi/muli/divui/remui/cmpi/select on scalars, arith addf/subf/mulf/divf/maximumf/minimumf/negf/extf/truncf and math
// exp/exp2/log/log2/sqrt/rsqrt/tanh/erf/absf/fma on tensors, the integer arith ops (addi ... minui), cmpi / cmpf / select,
// trunci / extsi / extui / sitofp / fptosi / bitcast, math.absi and kapy.arange on tensors, kapy.fptofp / splat / broadcast / transpose,
// kapy.program_id / warp_id / mk_global / sv_global / mk_shared / sv_shared / ld_global / st_global /
// cp_async_global_to_shared / cp_async_wait_group / ld_matrix / matmul / reduce (addf or maximumf
// lambda) / return, scf.for with iter_args and scf.yield.
#include <cctype>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <atomic>
#include <climits>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "common.hpp"

namespace kapy {
namespace {

struct Type {
  enum Kind { kNone, kInt, kPtr, kFloat, kTensor } kind = kNone;
  int dtype = -1;
  int64_t shape[2] = {0, 0};  // -1 = dynamic
  std::string space;          // alias of the encoding: "global", "shared", "values"
};

struct Op {
  std::string name;
  std::vector<std::string> results;   // "%3"; a multi-result op "%34:3" is expanded to %34#0 ..
  std::vector<std::string> operands;  // every %value of the operand section, in order
  std::vector<std::string> words;     // bare words of the operand section (cmpi predicate, matmul way, constants)
  std::map<std::string, std::string> attrs;
  std::vector<Type> types;            // every type after the top-level ':'
  std::vector<std::string> region_args;  // scf.for: induction variable, then iter_args names
  std::vector<Op> body;
  int line = 0;
};

struct Func {
  std::string name;
  std::vector<std::string> arg_names;
  std::vector<Type> arg_types;
  std::vector<Op> body;
  int num_warps = 1;
};

struct Token {
  enum Kind { kWord, kValue, kNumber, kPunct, kNewline, kEnd } kind;
  std::string text;
  int line;
};

std::vector<Token> tokenize(const char *s) {
  std::vector<Token> out;
  int line = 1;
  while (*s) {
    if (*s == '\n') { out.push_back({Token::kNewline, "\n", line++}); ++s; continue; }
    if (isspace((unsigned char)*s)) { ++s; continue; }
    if (s[0] == '/' && s[1] == '/') { while (*s && *s != '\n') ++s; continue; }
    if (*s == '%' || *s == '#' || *s == '@' || *s == '!') {
      const char *b = s++;
      while (isalnum((unsigned char)*s) || *s == '_' || *s == '.' || *s == '#' || *s == '$') ++s;
      out.push_back({b[0] == '%' ? Token::kValue : Token::kWord, std::string(b, s), line});
      continue;
    }
    if (isalpha((unsigned char)*s) || *s == '_') {
      const char *b = s;
      while (isalnum((unsigned char)*s) || *s == '_' || *s == '.') ++s;
      out.push_back({Token::kWord, std::string(b, s), line});
      continue;
    }
    if (isdigit((unsigned char)*s) || ((*s == '-' || *s == '+') && isdigit((unsigned char)s[1]))) {
      const char *b = s++;
      while (isalnum((unsigned char)*s) || *s == '.' || ((*s == '+' || *s == '-') && (s[-1] == 'e' || s[-1] == 'E'))) ++s;
      out.push_back({Token::kNumber, std::string(b, s), line});
      continue;
    }
    if (s[0] == '-' && s[1] == '>') { out.push_back({Token::kPunct, "->", line}); s += 2; continue; }
    out.push_back({Token::kPunct, std::string(1, *s), line});
    ++s;
  }
  out.push_back({Token::kEnd, "", line});
  return out;
}

int dtype_of(const std::string &w) {
  if (w == "f16") return KAPY_F16;
  if (w == "bf16") return KAPY_BF16;
  if (w == "f32") return KAPY_F32;
  if (w == "f8E4M3" || w == "f8E4M3FN") return KAPY_F8E4M3;
  if (w == "f8E5M2") return KAPY_F8E5M2;
  if (w == "i32") return KAPY_I32;
  if (w == "i16") return KAPY_I16;
  if (w == "i8") return KAPY_I8;
  if (w == "i1") return KAPY_I1;
  return -1;
}

// A float literal as MLIR prints it: decimal, or the value's bit pattern in hexadecimal (how infinities and NaNs are written).
double float_literal(const std::string &w, int dtype) {
  if (w.size() > 2 && w[0] == '0' && (w[1] == 'x' || w[1] == 'X')) {
    const uint64_t bits = strtoull(w.c_str(), nullptr, 16);
    if (dtype == KAPY_F16) {
      const int e = (int)((bits >> 10) & 31);
      const double m = (double)(bits & 1023), sign = (bits & 0x8000) ? -1.0 : 1.0;
      if (e == 31) return m != 0 ? (double)NAN : sign * (double)INFINITY;
      return sign * (e == 0 ? ldexp(m, -24) : ldexp(1024.0 + m, e - 25));
    }
    uint32_t u = dtype == KAPY_BF16 ? (uint32_t)bits << 16 : (uint32_t)bits;
    float f;
    memcpy(&f, &u, 4);
    return (double)f;
  }
  return atof(w.c_str());
}

struct Parser {
  std::vector<Token> t;
  size_t p = 0;
  std::string err;
  std::map<std::string, std::string> aliases;  // "#global" -> "global_memory"
  const Token &peek(int k = 0) const { return t[std::min(p + k, t.size() - 1)]; }
  bool is(const char *text) const { return peek().text == text; }
  bool accept(const char *text) { if (is(text)) { ++p; return true; } return false; }
  bool fail_at(const std::string &m) { if (err.empty()) err = "line " + std::to_string(peek().line) + ": " + m; return false; }
  void skip_newlines() { while (peek().kind == Token::kNewline) ++p; }

  // tensor<64x?xf16, #values> | i32 | i1 | f16 | !kapy.ptr<1>
  bool parse_type(Type &ty) {
    const Token &k = peek();
    if (k.text == "tensor") {
      ++p;
      if (!accept("<")) return fail_at("expected '<' after tensor");
      ty.kind = Type::kTensor;
      // the dims and the element type arrive as "64x64xf16", "?", "x", "?xf16" word / number / punct tokens
      std::string dims;
      while (!is(",") && !is(">") && peek().kind != Token::kEnd) dims += t[p++].text;
      size_t pos = 0;
      int nd = 0;
      while (pos < dims.size()) {
        size_t x = dims.find('x', pos);
        std::string part = dims.substr(pos, x == std::string::npos ? std::string::npos : x - pos);
        if (x == std::string::npos || dtype_of(dims.substr(pos)) >= 0) { ty.dtype = dtype_of(dims.substr(pos)); break; }
        if (nd < 2) ty.shape[nd++] = part == "?" ? -1 : atoll(part.c_str());
        pos = x + 1;
      }
      if (ty.dtype < 0) return fail_at("unsupported tensor element type in '" + dims + "'");
      if (accept(",")) {
        std::string enc = t[p++].text;  // #alias
        if (is("<")) { int depth = 0; do { if (is("<")) ++depth; if (is(">")) --depth; enc += t[p++].text; } while (depth > 0); }
        auto it = aliases.find(enc);
        const std::string &full = it == aliases.end() ? enc : it->second;
        ty.space = full.find("global") != std::string::npos ? "global" : full.find("shared") != std::string::npos ? "shared" : "values";
      }
      if (!accept(">")) return fail_at("expected '>' closing tensor type");
      return true;
    }
    if (k.text == "!kapy.ptr") {
      ++p;
      if (accept("<")) { while (!is(">") && peek().kind != Token::kEnd) ++p; accept(">"); }
      ty.kind = Type::kPtr;
      return true;
    }
    if (k.text == "i32" || k.text == "i1" || k.text == "i8" || k.text == "i16" || k.text == "i64" || k.text == "index") { ++p; ty.kind = Type::kInt; ty.dtype = KAPY_I32; return true; }
    if (dtype_of(k.text) >= 0) { ++p; ty.kind = Type::kFloat; ty.dtype = dtype_of(k.text); return true; }
    return fail_at("unknown type '" + k.text + "'");
  }

  // {a = 1 : i32, b = true}
  bool parse_attr_dict(std::map<std::string, std::string> &attrs) {
    while (!is("}") && peek().kind != Token::kEnd) {
      std::string key = t[p++].text;
      std::string val = "true";
      if (accept("=")) {
        val = t[p++].text;
        if (accept(":")) { Type ty; if (!parse_type(ty)) return false; }
      }
      attrs[key] = val;
      accept(",");
    }
    return accept("}") || fail_at("unterminated attribute dictionary");
  }

  bool parse_region(std::vector<Op> &body) {
    for (;;) {
      skip_newlines();
      if (accept("}")) return true;
      if (peek().kind == Token::kEnd) return fail_at("unterminated region");
      Op op;
      if (!parse_op(op)) return false;
      body.push_back(std::move(op));
    }
  }

  bool parse_op(Op &op) {
    op.line = peek().line;
    // results
    if (peek().kind == Token::kValue) {
      for (;;) {
        std::string r = t[p++].text;
        if (accept(":")) {
          int n = atoi(t[p++].text.c_str());
          for (int i = 0; i < n; ++i) op.results.push_back(r + "#" + std::to_string(i));
        } else op.results.push_back(r);
        if (!accept(",")) break;
      }
      if (!accept("=")) return fail_at("expected '=' after results");
    }
    if (peek().kind != Token::kWord) return fail_at("expected an operation name");
    op.name = t[p++].text;
    if (op.name == "scf.for") {
      // %iv = %lo to %hi step %st iter_args(%a = %init, ...) -> (types) : i32 { region }
      op.region_args.push_back(t[p++].text);
      if (!accept("=")) return fail_at("scf.for: expected '='");
      op.operands.push_back(t[p++].text);
      if (!accept("to")) return fail_at("scf.for: expected 'to'");
      op.operands.push_back(t[p++].text);
      if (!accept("step")) return fail_at("scf.for: expected 'step'");
      op.operands.push_back(t[p++].text);
      if (accept("iter_args")) {
        if (!accept("(")) return fail_at("scf.for: expected '('");
        while (!is(")")) {
          op.region_args.push_back(t[p++].text);
          if (!accept("=")) return fail_at("scf.for: expected '=' in iter_args");
          op.operands.push_back(t[p++].text);
          accept(",");
        }
        accept(")");
        if (accept("->")) {
          if (accept("(")) { while (!is(")")) { Type ty; if (!parse_type(ty)) return false; op.types.push_back(ty); accept(","); } accept(")"); }
          else { Type ty; if (!parse_type(ty)) return false; op.types.push_back(ty); }
        }
      }
      if (accept(":")) { Type ty; if (!parse_type(ty)) return false; }
      if (!accept("{")) return fail_at("scf.for: expected '{'");
      return parse_region(op.body);
    }
    // operand section: up to the top-level ':' or the end of the line
    int depth = 0;
    while (peek().kind != Token::kEnd) {
      const Token &k = peek();
      if (k.kind == Token::kNewline && depth == 0) break;
      if (k.text == ":" && depth == 0) break;
      if (k.text == "{") {
        ++p;
        if (peek().kind == Token::kNewline) {  // a region (kapy.reduce lambda)
          if (!parse_region(op.body)) return false;
        } else if (!parse_attr_dict(op.attrs)) return false;
        continue;
      }
      if (k.text == "lambda") {  // lambda(%a: f16, %b: f16)
        ++p;
        accept("(");
        while (!is(")") && peek().kind != Token::kEnd) {
          op.region_args.push_back(t[p++].text);
          if (accept(":")) { Type ty; if (!parse_type(ty)) return false; }
          accept(",");
        }
        accept(")");
        continue;
      }
      if (k.text == "dense") {  // dense<0.000000e+00>
        ++p;
        accept("<");
        op.words.push_back(t[p++].text);
        accept(">");
        continue;
      }
      if (k.text == "(" || k.text == "[") ++depth;
      if (k.text == ")" || k.text == "]") --depth;
      if (k.kind == Token::kValue) op.operands.push_back(k.text);
      else if (k.kind == Token::kWord || k.kind == Token::kNumber) op.words.push_back(k.text);
      ++p;
    }
    if (accept(":")) {
      while (peek().kind != Token::kNewline && peek().kind != Token::kEnd) {
        if (accept(",") || accept("->") || accept("(") || accept(")") || accept("to")) continue;
        Type ty;
        if (!parse_type(ty)) return false;
        op.types.push_back(ty);
      }
    }
    return true;
  }

  bool parse_module(Func &f, const char *want) {
    for (;;) {
      skip_newlines();
      const Token &k = peek();
      if (k.kind == Token::kEnd) return fail_at(std::string("no kapy.func") + (want ? std::string(" named ") + want : std::string()) + " found");
      if (k.kind == Token::kWord && k.text[0] == '#' && peek(1).text == "=") {  // #global = #kapy.encoding<global_memory>
        std::string name = k.text;
        p += 2;
        std::string rhs;
        while (peek().kind != Token::kNewline && peek().kind != Token::kEnd) rhs += t[p++].text;
        aliases[name] = rhs;
        continue;
      }
      if (k.text == "module") {
        ++p;
        if (accept("attributes")) {
          if (!accept("{")) return fail_at("expected '{' after attributes");
          std::map<std::string, std::string> attrs;
          if (!parse_attr_dict(attrs)) return false;
          if (attrs.count("kapy.num_warps")) f.num_warps = atoi(attrs["kapy.num_warps"].c_str());
        }
        if (!accept("{")) return fail_at("expected '{' opening the module");
        continue;
      }
      if (k.text == "kapy.func") {
        ++p;
        accept("public");
        accept("private");
        std::string name = t[p++].text;  // @name
        if (!accept("(")) return fail_at("kapy.func: expected '('");
        Func g;
        g.num_warps = f.num_warps;
        g.name = name.substr(1);
        while (!is(")") && peek().kind != Token::kEnd) {
          g.arg_names.push_back(t[p++].text);
          if (!accept(":")) return fail_at("kapy.func: expected ':' after an argument");
          Type ty;
          if (!parse_type(ty)) return false;
          g.arg_types.push_back(ty);
          if (accept("{")) { std::map<std::string, std::string> a; if (!parse_attr_dict(a)) return false; }
          accept(",");
        }
        accept(")");
        if (!accept("{")) return fail_at("kapy.func: expected '{'");
        if (!parse_region(g.body)) return false;
        if (!want || g.name == want) { f = std::move(g); return true; }
        continue;
      }
      ++p;  // closing braces of the module etc.
    }
  }
};

// ---------------------------------------------------------------------------------------------
// ---------------------------------------------------------------------------------------------
// Shared-memory plan and barrier positions of a parsed function: buffers and their live ranges as
// lib/Analysis/AllocAnalysis.cpp:86-185 finds them (one buffer per mk_shared in walk order; op ids in post-order,
// so that a loop op's id is larger than its body's; a buffer is live over [first id, last id) of the ops that
// define or use it or a value aliasing it), placed by kapy_smem_plan; then the function's structured control flow
// unrolled into a block graph (entry, loop header, loop body, continuation) and handed to kapy_smem_barriers.
// Unlike BlockAnalysis.cpp:145-152, which looks buffers up by the mk_shared result only, accesses through
// sub-views and selects are attributed to every buffer they may alias.
struct SharedBuffer {
  std::string name;
  int line = 0;
  int64_t size = 0, first = INT64_MAX, last = INT64_MIN, offset = 0;
};
struct Analysis {
  std::vector<SharedBuffer> buffers;
  int64_t total = 0;
  std::vector<int> barrier_lines;  // +line: before the op on that line, -line: after it
};

struct Analyzer {
  const Func &f;
  Analysis &out;
  std::map<std::string, std::set<int>> alias;        // value -> buffers it may point into
  std::map<std::string, std::vector<const Op *>> def_chain;  // value -> ops enclosing its definition, outermost first, then the defining op
  std::map<const Op *, int64_t> id;
  std::vector<kapy_smem_op> ops;
  std::vector<int> op_line;
  std::vector<kapy_smem_access> accesses;
  std::vector<std::vector<int>> succ;
  Analyzer(const Func &fn, Analysis &a) : f(fn), out(a) {}

  void number(const std::vector<Op> &body) {
    for (const Op &op : body) {
      number(op.body);
      id[&op] = (int64_t)id.size();
    }
  }
  void define(const std::vector<Op> &body, std::vector<const Op *> &chain) {
    for (const Op &op : body) {
      chain.push_back(&op);
      for (auto &r : op.results) def_chain[r] = chain;
      for (auto &r : op.region_args) def_chain[r] = chain;  // live from the op that owns the region
      if (op.name == "kapy.mk_shared" && !op.types.empty() && !op.results.empty()) {
        SharedBuffer b;
        b.name = op.results[0];
        b.line = op.line;
        const Type &ty = op.types.back();
        b.size = std::max<int64_t>(ty.shape[0], 0) * std::max<int64_t>(ty.shape[1], 0) * dtype_bytes(ty.dtype);
        alias[b.name].insert((int)out.buffers.size());
        out.buffers.push_back(b);
      }
      define(op.body, chain);
      chain.pop_back();
    }
  }
  // one pass of alias propagation; returns whether anything grew
  bool propagate(const std::vector<Op> &body, const Op *loop) {
    bool grew = false;
    auto flow = [&](const std::string &from, const std::string &to) {
      auto it = alias.find(from);
      if (it == alias.end()) return;
      auto &dst = alias[to];
      const size_t before = dst.size();
      dst.insert(it->second.begin(), it->second.end());
      grew |= dst.size() != before;
    };
    for (const Op &op : body) {
      if (op.name == "kapy.sv_shared" && !op.results.empty() && !op.operands.empty()) flow(op.operands[0], op.results[0]);
      if (op.name == "arith.select" && op.operands.size() == 3 && !op.results.empty()) { flow(op.operands[1], op.results[0]); flow(op.operands[2], op.results[0]); }
      if (op.name == "scf.for") {
        for (size_t k = 1; k < op.region_args.size() && 2 + k < op.operands.size(); ++k) flow(op.operands[2 + k], op.region_args[k]);
        grew |= propagate(op.body, &op);
      }
      if (op.name == "scf.yield" && loop)
        for (size_t k = 0; k < op.operands.size(); ++k) {
          if (k + 1 < loop->region_args.size()) flow(op.operands[k], loop->region_args[k + 1]);
          if (k < loop->results.size()) flow(op.operands[k], loop->results[k]);
        }
    }
    return grew;
  }
  void touch(const std::string &value, int64_t at) {
    auto it = alias.find(value);
    if (it == alias.end()) return;
    for (int b : it->second) {
      out.buffers[b].first = std::min(out.buffers[b].first, at);
      out.buffers[b].last = std::max(out.buffers[b].last, at);
    }
  }
  // every op that defines or uses an aliasing value extends the buffer's range; a use inside a loop of a value
  // defined outside it counts at the loop op, whose id closes the loop's body
  void liveness(const std::vector<Op> &body, std::vector<const Op *> &chain) {
    for (const Op &op : body) {
      chain.push_back(&op);
      for (auto &r : op.results) touch(r, id[&op]);
      for (auto &u : op.operands) {
        auto d = def_chain.find(u);
        if (d == def_chain.end()) continue;
        size_t depth = d->second.size() - 1;  // nesting depth of the definition
        if (!d->second.empty() && std::find(d->second.back()->region_args.begin(), d->second.back()->region_args.end(), u) != d->second.back()->region_args.end())
          depth += 1;                          // a region argument lives inside the region
        const Op *at = depth < chain.size() ? chain[depth] : &op;
        touch(u, id[at]);
      }
      liveness(op.body, chain);
      chain.pop_back();
    }
  }
  int new_block() { succ.emplace_back(); return (int)succ.size() - 1; }
  void add_access(const std::string &value, bool is_write) {
    auto it = alias.find(value);
    if (it == alias.end()) return;
    for (int b : it->second) accesses.push_back({out.buffers[b].offset, out.buffers[b].offset + out.buffers[b].size, is_write ? 1 : 0, 0});
  }
  int blocks_of(const std::vector<Op> &body, int cur) {
    for (const Op &op : body) {
      if (op.name == "scf.for") {
        const int header = new_block(), first = new_block();
        succ[cur].push_back(header);
        succ[header].push_back(first);
        const int last = blocks_of(op.body, first);
        succ[last].push_back(header);
        const int cont = new_block();
        succ[header].push_back(cont);
        cur = cont;
        continue;
      }
      kapy_smem_op so{cur, 0, (int32_t)accesses.size(), 0};
      if (op.name == "nvvm.barrier0") so.kind = 1;
      else if (op.name == "kapy.cp_async_wait_group") so.kind = 2;
      else if ((op.name == "kapy.ld_matrix" || op.name == "kapy.ld_shared") && !op.operands.empty()) add_access(op.operands[0], false);
      else if ((op.name == "kapy.cp_async_global_to_shared" || op.name == "kapy.st_shared") && op.operands.size() > 1) add_access(op.operands[1], true);
      so.n_accesses = (int32_t)accesses.size() - so.first_access;
      ops.push_back(so);
      op_line.push_back(op.line);
    }
    return cur;
  }
  int run(std::string &err) {
    std::vector<const Op *> chain;
    number(f.body);
    define(f.body, chain);
    while (propagate(f.body, nullptr)) {}
    liveness(f.body, chain);
    std::vector<kapy_smem_buffer> plan(out.buffers.size());
    for (size_t k = 0; k < plan.size(); ++k) {
      const SharedBuffer &b = out.buffers[k];
      plan[k] = {b.size, b.first, std::max(b.first, b.last), 0};  // [first id, last id): AllocAnalysis.cpp:150-160
    }
    out.total = kapy_smem_plan(plan.data(), (int32_t)plan.size(), 128);
    if (out.total < 0) { err = kapy_last_error(); return (int)out.total; }
    for (size_t k = 0; k < plan.size(); ++k) out.buffers[k].offset = plan[k].offset;
    new_block();
    blocks_of(f.body, 0);
    std::vector<int32_t> succ_begin{0}, flat;
    for (auto &s : succ) { flat.insert(flat.end(), s.begin(), s.end()); succ_begin.push_back((int32_t)flat.size()); }
    std::vector<int32_t> flags(ops.size() + 1, 0);
    int n = kapy_smem_barriers(ops.data(), (int32_t)ops.size(), accesses.data(), (int32_t)accesses.size(), succ_begin.data(), flat.data(),
                               (int32_t)succ.size(), flags.data());
    if (n < 0) { err = kapy_last_error(); return n; }
    for (size_t k = 0; k < ops.size(); ++k) {
      if (flags[k] & 1) out.barrier_lines.push_back(op_line[k]);
      if (flags[k] & 2) out.barrier_lines.push_back(-op_line[k]);
    }
    return KAPY_OK;
  }
};

// Bytes of LDS one gfx950 workgroup can have.
constexpr int64_t kLdsBytes = 160 * 1024;

// A register tensor that has not been computed yet: one elementwise op over computed register tensors (leaves) and other
// deferred tensors.  A chain of arith / math / cast / splat / broadcast ops stays deferred until an op that is not
// elementwise needs its value; a kapy.st_global then runs the whole chain as ONE program that stores straight into the
// global view, which is what the reference's pipeline compiles such a chain to (one fused kernel body, no temporaries).
struct Expr {
  int ew = KAPY_EW_LD_GLOBAL;  // KAPY_EW_LD_GLOBAL: a leaf (`leaf` is the computed tensor); -1: the operand itself (broadcast)
  int dtype = 0, rmode = KAPY_RN;
  float imm = 0.f;
  int32_t ia = 0, ib = 0, ic = 0;  // integer fields of the instruction: an integer splat's value, arange's start and axis, a compare's predicate
  std::shared_ptr<Expr> in[3];
  int n_in = 0;
  kapy_global leaf;
  bool global_leaf = false;  // the leaf is a view of the caller's memory (a deferred kapy.ld_global), which a later store may change
  // KAPY_EW_REDUCE_SUM / _MAX along `axis`: inside a program the result sits on every element of the reduced line, so the node
  // can only be part of a program whose result has the operand's shape (rows x cols) and element type (operand_dtype)
  int32_t rows = 0, cols = 0, operand_dtype = 0, axis = 1;
};

struct Value {
  enum Kind { kNone, kInt, kPtr, kTensor, kFloat } kind = kNone;
  std::shared_ptr<Expr> lazy;  // kTensor: set while the tensor is deferred; g then only carries its shape and type
  int64_t i = 0;
  double f = 0.0;     // kFloat: a scalar of float type
  void *ptr = nullptr;
  int64_t bytes = 0;  // kPtr: size of the allocation behind ptr, 0 = unknown
  kapy_global g;      // global views, shared-memory tensors and register tensors alike
};

// Shared-memory tensors take the first part of the arena and live for the whole call; register tensors
// take the rest and die with their program instance.
// A call runs its program instances in groups (all programs of a group and all their warps in step): every program of a group
// has its own shared part, the group one region for the register tensors of calls merged over instances, every warp its share.
constexpr size_t kSharedArena = size_t(256) << 10, kArena = size_t(2048) << 20, kMergedArena = size_t(512) << 20, kMinShare = size_t(1) << 20;

// A device call of a run, as recorded for the plan cache: which entry point, and copies of everything it was given.
struct PlannedCall {
  enum Kind { kCopy, kElementwise, kReduce, kReduceEx, kMatmul } kind;
  kapy_global g[4];
  bool has[4] = {false, false, false, false};
  kapy_copy_cfg copy_cfg;
  kapy_matmul_cfg matmul_cfg;
  kapy_reduce_cfg reduce_cfg;
  bool has_cfg = false;
  int32_t axis = 0, reduce_kind = 0;
  std::vector<kapy_ew_inst> prog;
  std::vector<kapy_global> ins;
};

struct Interp {
  const Func &f;
  hipStream_t stream;
  char *arena = nullptr;
  size_t top = kSharedArena, limit = kArena;
  std::map<std::string, Value> env;
  // The warps of one program instance, run in step: every op is executed for warp 0, 1, ... before the next op is looked at,
  // which is the reference's workgroup of concurrent warps (FuncOpToLLVM.cpp:72-88) with a barrier between any two ops - so a
  // program whose warps exchange data through shared memory between the barriers BlockAnalysis would insert
  // (BlockAnalysis.cpp:114-169) sees what it would see on the reference's target.  Each warp has its own values and its own
  // share of the register arena; the state of the warp being executed is swapped into env / top / limit / warp.
  struct WarpState {
    std::map<std::string, Value> env;
    size_t top = 0, limit = 0;
    int64_t pid[3] = {0, 0, 0}, warp = 0;  // which program instance, which of its warps
    size_t shared_base = 0;                // where that program's shared-memory tensors start in the arena
  };
  std::vector<WarpState> warps;  // every warp of every program of the group in flight
  int current = -1;              // the state swapped in
  void enter(int w) {
    std::swap(env, warps[w].env);
    top = warps[w].top;
    limit = warps[w].limit;
    warp = warps[w].warp;
    for (int k = 0; k < 3; ++k) pid[k] = warps[w].pid[k];
    shared_base = warps[w].shared_base;
    current = w;
  }
  void leave(int w) {
    std::swap(env, warps[w].env);
    warps[w].top = top;
    current = -1;
  }
  size_t shared_base = 0, register_base = kSharedArena;  // (register_base: where the shared parts of the group end)
  size_t merged_base = 0, merged_top = 0;                // the group's region for merged calls, and how much of it is taken
  bool merge = true;                                     // KAPY_MLIR_BATCH=0: no call is merged over instances
  const Analysis *plan = nullptr;  // where each mk_shared lives inside the shared part of the arena
  int64_t pid[3] = {0, 0, 0}, warp = 0;
  std::string err;

  Interp(const Func &fn, hipStream_t s) : f(fn), stream(s) {}
  int fail_op(const Op &op, const std::string &m) {
    if (err.empty()) err = "line " + std::to_string(op.line) + " (" + op.name + "): " + m;
    return KAPY_ERR_INVALID;
  }
  void *alloc(size_t bytes) {
    top = (top + 255) & ~size_t(255);
    if (top + bytes > limit) return nullptr;
    void *r = arena + top;
    top += bytes;
    return r;
  }
  bool get(const Op &op, size_t k, Value::Kind kind, Value &v) {
    if (k >= op.operands.size()) { fail_op(op, "missing operand"); return false; }
    auto it = env.find(op.operands[k]);
    if (it == env.end()) { fail_op(op, "use of undefined value " + op.operands[k]); return false; }
    if (it->second.kind != kind) { fail_op(op, "operand " + op.operands[k] + " has the wrong kind"); return false; }
    if (it->second.lazy && force(op, it->second) != KAPY_OK) return false;
    v = it->second;
    return true;
  }

  // ---- deferred elementwise chains ----
  bool fuse = true;  // KAPY_MLIR_FUSE=0: every op runs by itself, as one call
  bool is_register_tensor(const kapy_global &g) const {
    const char *p = (const char *)g.ptr;
    return p >= arena + register_base && p < arena + kArena;
  }
  // [first, last] byte of a view (strides are positive: mk_global refuses others)
  static void byte_range(const kapy_global &g, const char **lo, const char **hi) {
    const int eb = dtype_bytes(g.dtype);
    *lo = view_base(&g);
    *hi = *lo + (int64_t(g.end0 - g.start0 - 1) * g.stride0 + int64_t(g.end1 - g.start1 - 1) * g.stride1 + 1) * eb - 1;
  }
  // does the chain read, through a deferred load, memory that a store into `dst` writes
  bool reads_under(const std::shared_ptr<Expr> &e, const kapy_global &dst) {
    if (e->ew == KAPY_EW_LD_GLOBAL && e->n_in == 0) {
      if (!e->global_leaf) return false;
      const char *a0, *a1, *b0, *b1;
      byte_range(e->leaf, &a0, &a1);
      byte_range(dst, &b0, &b1);
      return a0 <= b1 && b0 <= a1;
    }
    for (int k = 0; k < e->n_in; ++k)
      if (reads_under(e->in[k], dst)) return true;
    return false;
  }
  // before a store into `dst`: every deferred value that still has to read that memory is computed now
  // (the values of every warp: another warp's deferred load stands earlier in program order than this store, too)
  // (with a thousand warps in step, a store per warp that looks through every warp's values is a million looks: a scan that
  // met no deferred value at all holds until the next one is made - copies of values cannot make one out of none)
  int64_t lazy_made = 0, none_lazy_at = -1;
  int settle_readers(const Op &op, const kapy_global &dst) {
    if (none_lazy_at == lazy_made) return KAPY_OK;
    bool any_lazy = false;
    auto settle = [&](std::map<std::string, Value> &values) {
      for (auto &kv : values)
        if (kv.second.kind == Value::kTensor && kv.second.lazy) {
          any_lazy = true;
          if (!reads_under(kv.second.lazy, dst)) continue;
          int rc = force(op, kv.second);
          if (rc != KAPY_OK) return rc;
        }
      return (int)KAPY_OK;
    };
    int rc = settle(env);
    for (size_t w = 0; rc == KAPY_OK && w < warps.size(); ++w)
      if ((int)w != current) rc = settle(warps[w].env);
    if (rc == KAPY_OK && !any_lazy) none_lazy_at = lazy_made;
    return rc;
  }
  // the operand as an expression: deferred tensors as they are, computed ones as leaves
  std::shared_ptr<Expr> as_expr(const Value &v) {
    if (v.lazy) return v.lazy;
    auto e = std::make_shared<Expr>();
    e->leaf = v.g;
    return e;
  }
  static constexpr int kMaxProgram = 48, kMaxRegisters = 16;  // what one kapy_elementwise program may hold
  struct Emit {
    kapy_ew_inst prog[kMaxProgram];
    const kapy_global *ins[8];
    int n = 0, n_ins = 0, regs = 0;
    std::map<const Expr *, int> reg;
    bool ok = true;
  };
  int emit(const std::shared_ptr<Expr> &e, Emit &m) {
    auto it = m.reg.find(e.get());
    if (it != m.reg.end()) return it->second;
    int src[3] = {0, 0, 0};
    for (int k = 0; k < e->n_in; ++k) src[k] = emit(e->in[k], m);
    if (!m.ok) return 0;
    if (e->ew < 0) return m.reg[e.get()] = src[0];
    if (m.regs >= kMaxRegisters || m.n >= kMaxProgram - 1) { m.ok = false; return 0; }
    const int dst = m.regs++;
    if (e->ew == KAPY_EW_LD_GLOBAL) {
      int slot = -1;
      for (int k = 0; k < m.n_ins; ++k)
        if (!memcmp(m.ins[k], &e->leaf, sizeof(kapy_global))) slot = k;
      if (slot < 0) {
        if (m.n_ins >= 8) { m.ok = false; return 0; }
        m.ins[slot = m.n_ins++] = &e->leaf;
      }
      m.prog[m.n++] = {KAPY_EW_LD_GLOBAL, dst, slot, 0, 0, 0, KAPY_RN, 0.f};
    } else if (e->ew == KAPY_EW_REDUCE_SUM || e->ew == KAPY_EW_REDUCE_MAX) {
      m.prog[m.n++] = {e->ew, dst, src[0], e->axis, 0, 0, KAPY_RN, 0.f};
    } else if (e->ew == KAPY_EW_ARANGE || (e->ew == KAPY_EW_SPLAT && e->dtype >= KAPY_I8)) {
      m.prog[m.n++] = {e->ew, dst, e->ia, e->ib, 0, e->dtype, KAPY_RN, 0.f};
    } else {
      m.prog[m.n++] = {e->ew, dst, src[0], src[1], (e->ew == KAPY_EW_CMPI || e->ew == KAPY_EW_CMPF) ? e->ic : src[2], e->dtype, e->rmode, e->imm};
    }
    return m.reg[e.get()] = dst;
  }
  static bool is_reduce(const Expr &e) { return e.ew == KAPY_EW_REDUCE_SUM || e.ew == KAPY_EW_REDUCE_MAX; }
  // the outermost reduce of the chain that `skip` does not exempt
  template <class Skip>
  Expr *find_reduce(const std::shared_ptr<Expr> &e, Skip skip) {
    if (is_reduce(*e) && !skip(*e)) return e.get();
    for (int k = 0; k < e->n_in; ++k)
      if (Expr *r = find_reduce(e->in[k], skip)) return r;
    return nullptr;
  }
  // runs a deferred reduce by itself (its operand computed first, then kapy_reduce): the node becomes a computed [rows x 1]
  // (axis 1) or [1 x cols] (axis 0) tensor
  int compute_reduce(const Op &op, Expr *r) {
    Value operand;
    operand.kind = Value::kTensor;
    operand.lazy = r->in[0];
    memset(&operand.g, 0, sizeof operand.g);
    int rc = lib(op, kapy_mk_global(&operand.g, arena, 0, r->rows, r->cols, r->cols, 1, r->operand_dtype, 16));
    if (rc == KAPY_OK && !(operand.lazy->ew == KAPY_EW_LD_GLOBAL && operand.lazy->n_in == 0)) rc = force(op, operand);
    if (rc != KAPY_OK) return rc;
    if (operand.lazy) operand.g = operand.lazy->leaf;
    const int32_t kept0 = r->axis == 1 ? r->rows : 1, kept1 = r->axis == 1 ? 1 : r->cols;
    void *ptr = alloc((size_t)kept0 * kept1 * dtype_bytes(r->operand_dtype));
    if (!ptr) return fail_op(op, "register tensors of one program instance exceed the arena");
    kapy_global g;
    rc = lib(op, kapy_mk_global(&g, ptr, 0, kept0, kept1, kept1, 1, r->operand_dtype, 256));
    if (rc == KAPY_OK) rc = lib(op, do_reduce(&operand.g, &g, r->axis, r->ew == KAPY_EW_REDUCE_MAX ? 1 : 0));
    if (rc != KAPY_OK) return rc;
    r->ew = KAPY_EW_LD_GLOBAL;
    r->n_in = 0;
    for (auto &p : r->in) p.reset();
    r->leaf = g;
    return KAPY_OK;
  }
  int run_program(const std::shared_ptr<Expr> &e, const kapy_global *out) {
    Emit m;
    const int r = emit(e, m);
    if (!m.ok) return fail(KAPY_ERR_UNSUPPORTED, "the deferred chain does not fit one program");
    m.prog[m.n++] = {KAPY_EW_ST_GLOBAL, 0, r, 0, 0, 0, KAPY_RN, 0.f};
    return do_elementwise(m.prog, m.n, m.ins, m.n_ins, out);
  }
  // the chain as one program that stores into `out`.  Reduces stay inside the program when its result has their
  // operand's shape (the row programs of kapy_elementwise: softmax, normalisations); the others, and all of them
  // when that program is refused (rows too long, a width that is no multiple of 8, ...), run as kapy_reduce first.
  int run_chain(const Op &op, const std::shared_ptr<Expr> &e, const kapy_global *out) {
    const int32_t rows = out->end0 - out->start0, cols = out->end1 - out->start1;
    while (Expr *r = find_reduce(e, [&](const Expr &x) { return x.rows == rows && x.cols == cols; })) {
      int rc = compute_reduce(op, r);
      if (rc != KAPY_OK) return rc;
    }
    int rc = run_program(e, out);
    if (rc == KAPY_OK || !find_reduce(e, [](const Expr &) { return false; })) return rc;
    while (Expr *r = find_reduce(e, [](const Expr &) { return false; })) {
      rc = compute_reduce(op, r);
      if (rc != KAPY_OK) return rc;
    }
    return run_program(e, out);
  }
  bool fits(const std::shared_ptr<Expr> &e) {
    Emit m;
    emit(e, m);
    return m.ok;
  }
  // computes a deferred tensor into a new register tensor; `v` (an entry of env, or a copy of one) becomes that tensor
  int force(const Op &op, Value &v) {
    if (!v.lazy) return KAPY_OK;
    const int32_t rows = v.g.end0 - v.g.start0, cols = v.g.end1 - v.g.start1;
    void *ptr = alloc((size_t)rows * cols * dtype_bytes(v.g.dtype));
    if (!ptr) return fail_op(op, "register tensors of one program instance exceed the arena");
    kapy_global g;
    int rc = lib(op, kapy_mk_global(&g, ptr, 0, rows, cols, cols, 1, v.g.dtype, 256));
    if (rc == KAPY_OK) {
      // a deferred load by itself is the copy kapy.ld_global always was (any element type, any strides)
      if (v.lazy->ew == KAPY_EW_LD_GLOBAL && v.lazy->n_in == 0) rc = lib(op, do_copy(&v.lazy->leaf, &g, nullptr));
      else rc = lib(op, run_chain(op, v.lazy, &g));
    }
    if (rc != KAPY_OK) return rc;
    // every other holder of the same expression now reads the computed tensor as well
    v.lazy->ew = KAPY_EW_LD_GLOBAL;
    v.lazy->n_in = 0;
    for (auto &p : v.lazy->in) p.reset();
    v.lazy->leaf = g;
    v.lazy->global_leaf = false;
    v.lazy.reset();
    v.g = g;
    for (auto &kv : env)
      if (kv.second.lazy && kv.second.lazy->ew == KAPY_EW_LD_GLOBAL && kv.second.lazy->n_in == 0 && !memcmp(&kv.second.lazy->leaf, &g, sizeof g)) {
        kv.second.lazy.reset();
        kv.second.g = g;
      }
    return KAPY_OK;
  }
  // result <- ew(operands...) without running anything; falls back to computing operands when the chain would outgrow one
  // program, and to computing the result at once when an operand is memory the program can still change
  int defer(const Op &op, int n_operands, int ew, int dtype, int rmode, float imm, int32_t ia = 0, int32_t ib = 0, int32_t ic = 0) {
    if (op.types.empty()) return fail_op(op, "missing result type");
    const Type &ty = op.types.back();
    if (ty.kind != Type::kTensor || ty.shape[0] <= 0 || ty.shape[1] <= 0) return fail_op(op, "result must be a statically shaped tensor");
    auto e = std::make_shared<Expr>();
    e->ew = ew; e->dtype = dtype; e->rmode = rmode; e->imm = imm; e->n_in = n_operands;
    e->ia = ia; e->ib = ib; e->ic = ic;
    bool at_once = !fuse;
    for (int k = 0; k < n_operands; ++k) {
      if (k >= (int)op.operands.size()) return fail_op(op, "missing operand");
      auto it = env.find(op.operands[k]);
      if (it == env.end()) return fail_op(op, "use of undefined value " + op.operands[k]);
      if (it->second.kind != Value::kTensor) return fail_op(op, "operand " + op.operands[k] + " has the wrong kind");
      if (!it->second.lazy && !is_register_tensor(it->second.g)) at_once = true;
      e->in[k] = as_expr(it->second);
    }
    if (!fits(e)) {  // compute the deferred operands, which leaves a program of one instruction
      for (int k = 0; k < n_operands; ++k) {
        Value &v = env[op.operands[k]];
        if (v.lazy) {
          int rc = force(op, v);
          if (rc != KAPY_OK) return rc;
        }
        e->in[k] = as_expr(v);
      }
    }
    Value r;
    r.kind = Value::kTensor;
    r.lazy = e;
    ++lazy_made;
    memset(&r.g, 0, sizeof r.g);
    if (kapy_mk_global(&r.g, arena, 0, (int32_t)ty.shape[0], (int32_t)ty.shape[1], (int32_t)ty.shape[1], 1, ty.dtype, 16) != KAPY_OK)
      return fail_op(op, kapy_last_error());
    if (at_once) {
      int rc = force(op, r);
      if (rc != KAPY_OK) return rc;
    }
    env[op.results[0]] = r;
    return KAPY_OK;
  }
  // a new row-major register tensor of the op's result type
  bool new_tensor(const Op &op, const Type &ty, Value &v) {
    if (ty.kind != Type::kTensor || ty.shape[0] <= 0 || ty.shape[1] <= 0) { fail_op(op, "result must be a statically shaped tensor"); return false; }
    void *ptr = alloc((size_t)ty.shape[0] * ty.shape[1] * dtype_bytes(ty.dtype));
    if (!ptr) { fail_op(op, "register tensors of one program instance exceed the arena"); return false; }
    v.kind = Value::kTensor;
    if (kapy_mk_global(&v.g, ptr, 0, (int32_t)ty.shape[0], (int32_t)ty.shape[1], (int32_t)ty.shape[1], 1, ty.dtype, 256) != KAPY_OK) {
      fail_op(op, kapy_last_error());
      return false;
    }
    return true;
  }
  // a shared-memory tensor sits at its planned offset in its program's shared part of the arena, the same for every warp
  int mk_shared(const Op &op) {
    const Type &ty = op.types.back();
    for (const SharedBuffer &b : plan->buffers) {
      if (b.name != op.results[0] || b.line != op.line) continue;
      Value r;
      r.kind = Value::kTensor;
      if (ty.kind != Type::kTensor || ty.shape[0] <= 0 || ty.shape[1] <= 0) return fail_op(op, "result must be a statically shaped tensor");
      int rc = lib(op, kapy_mk_global(&r.g, arena + shared_base + b.offset, 0, (int32_t)ty.shape[0], (int32_t)ty.shape[1], (int32_t)ty.shape[1], 1, ty.dtype, 128));
      if (rc == KAPY_OK) env[op.results[0]] = r;
      return rc;
    }
    return fail_op(op, "no shared-memory plan for this tensor");
  }
  int lib(const Op &op, int rc) { return rc == KAPY_OK ? KAPY_OK : (fail_op(op, kapy_last_error()), rc); }

  // The device calls of the run.  With `record` set every call that succeeded is kept, with copies of its arguments: a later
  // run of the same program on the same arguments makes the same calls (nothing in a program can read a tensor's data into
  // a scalar, so which calls a run makes depends on the text, the grid and the argument values alone).
  std::vector<PlannedCall> *record = nullptr;
  int do_copy(const kapy_global *src, const kapy_global *dst, const kapy_copy_cfg *cfg) {
    int rc = kapy_copy(src, dst, cfg, stream);
    if (rc == KAPY_OK && record) {
      record->emplace_back();
      PlannedCall &c = record->back();
      c.kind = PlannedCall::kCopy;
      c.g[0] = *src; c.g[1] = *dst;
      if (cfg) { c.copy_cfg = *cfg; c.has_cfg = true; }
    }
    return rc;
  }
  int do_elementwise(const kapy_ew_inst *prog, int32_t n, const kapy_global *const *ins, int32_t n_ins, const kapy_global *out) {
    int rc = kapy_elementwise(prog, n, ins, n_ins, out, stream);
    if (rc == KAPY_OK && record) {
      record->emplace_back();
      PlannedCall &c = record->back();
      c.kind = PlannedCall::kElementwise;
      c.prog.assign(prog, prog + n);
      for (int i = 0; i < n_ins; ++i) c.ins.push_back(*ins[i]);
      c.g[0] = *out;
    }
    return rc;
  }
  int do_reduce(const kapy_global *src, const kapy_global *dst, int32_t axis, int32_t kind) {
    int rc = kapy_reduce(src, dst, axis, kind, stream);
    if (rc == KAPY_OK && record) {
      record->emplace_back();
      PlannedCall &c = record->back();
      c.kind = PlannedCall::kReduce;
      c.g[0] = *src; c.g[1] = *dst; c.axis = axis; c.reduce_kind = kind;
    }
    return rc;
  }
  int do_reduce_ex(const kapy_global *src, const kapy_global *dst, int32_t axis, const kapy_reduce_cfg *cfg) {
    int rc = kapy_reduce_ex(src, dst, axis, cfg, stream);
    if (rc == KAPY_OK && record) {
      record->emplace_back();
      PlannedCall &c = record->back();
      c.kind = PlannedCall::kReduceEx;
      c.g[0] = *src; c.g[1] = *dst; c.axis = axis;
      if (cfg) { c.reduce_cfg = *cfg; c.has_cfg = true; }
    }
    return rc;
  }
  int do_matmul(const kapy_global *a, const kapy_global *b, const kapy_global *acc, const kapy_global *r, const kapy_matmul_cfg *cfg) {
    int rc = kapy_matmul(a, b, acc, r, cfg, stream);
    if (rc == KAPY_OK && record) {
      record->emplace_back();
      PlannedCall &c = record->back();
      c.kind = PlannedCall::kMatmul;
      c.g[0] = *a; c.g[1] = *b; c.g[3] = *r;
      if (acc) { c.g[2] = *acc; c.has[2] = true; }
      if (cfg) { c.matmul_cfg = *cfg; c.has_cfg = true; }
    }
    return rc;
  }

  int binary_tensor(const Op &op, int ew) { return defer(op, 2, ew, 0, KAPY_RN, 0.f); }

  // result <- one instruction over the tensor operands (ew < 0: none, the operand itself; this is kapy.broadcast when
  // the operand has extent 1 where the result does not)
  int mapped_tensor(const Op &op, int n_operands, int ew, int dtype = 0, int rmode = KAPY_RN) {
    return defer(op, n_operands, ew, dtype, rmode, 0.f);
  }

  // ---- one call for all instances ----
  // The instances in flight all execute the same kapy.st_global.  When every one of them stores a deferred chain of the same
  // form, and their views - the result's and every loaded operand's - are the tiles of a rectangular grid over the same
  // tensors (an operand either moves with the tile along an axis or has extent 1 there: a broadcast row, column or scalar),
  // the instances together are ONE program over the union of the tiles, and it runs as one call: what the reference's one
  // kernel over the whole grid does.  Anything else (register or shared operands, which differ per instance; an arange,
  // whose values depend on the tile's origin; a reduce across the axis the tiles are laid out along) is left to the
  // instances one by one.
  static bool same_bits(float a, float b) { return !memcmp(&a, &b, sizeof a); }
  static bool is_leaf(const Expr &e) { return e.ew == KAPY_EW_LD_GLOBAL && e.n_in == 0; }
  // do two chains have the same form (leaves may differ in where their views start)?  pairs: node of a -> node of b
  bool same_form(const Expr *a, const Expr *b, std::map<const Expr *, const Expr *> &pairs, std::vector<const Expr *> *leaves_b) {
    auto seen = pairs.find(a);
    if (seen != pairs.end()) return seen->second == b;
    if (a->ew != b->ew || a->n_in != b->n_in) return false;
    if (is_leaf(*a)) {
      const kapy_global &x = a->leaf, &y = b->leaf;
      if (x.ptr != y.ptr || x.stride0 != y.stride0 || x.stride1 != y.stride1 || x.dtype != y.dtype || x.alignment != y.alignment ||
          x.end0 - x.start0 != y.end0 - y.start0 || x.end1 - x.start1 != y.end1 - y.start1 || a->global_leaf != b->global_leaf)
        return false;
      if (leaves_b) leaves_b->push_back(b);
    } else {
      if (a->dtype != b->dtype || a->rmode != b->rmode || !same_bits(a->imm, b->imm) || a->ia != b->ia || a->ib != b->ib || a->ic != b->ic ||
          a->rows != b->rows || a->cols != b->cols || a->operand_dtype != b->operand_dtype || a->axis != b->axis)
        return false;
    }
    pairs[a] = b;
    for (int k = 0; k < a->n_in; ++k)
      if (!same_form(a->in[k].get(), b->in[k].get(), pairs, leaves_b)) return false;
    return true;
  }
  std::shared_ptr<Expr> clone(const std::shared_ptr<Expr> &e, std::map<const Expr *, std::shared_ptr<Expr>> &made) {
    auto it = made.find(e.get());
    if (it != made.end()) return it->second;
    auto c = std::make_shared<Expr>(*e);
    made[e.get()] = c;
    for (int k = 0; k < e->n_in; ++k) c->in[k] = clone(e->in[k], made);
    return c;
  }
  bool try_merged_store(const Op &op) {
    const int n = (int)warps.size();
    if (n < 2 || op.operands.size() < 2) return false;
    std::vector<std::shared_ptr<Expr>> chain(n);
    std::vector<kapy_global> out(n);
    for (int w = 0; w < n; ++w) {
      auto src = warps[w].env.find(op.operands[0]), dst = warps[w].env.find(op.operands[1]);
      if (src == warps[w].env.end() || dst == warps[w].env.end() || src->second.kind != Value::kTensor || !src->second.lazy ||
          dst->second.kind != Value::kTensor || dst->second.lazy)
        return false;
      out[w] = dst->second.g;
      const kapy_global &sg = src->second.g, &o = out[w], &o0 = out[0];
      const char *ptr = (const char *)o.ptr;
      if (ptr >= arena && ptr < arena + kArena) return false;  // (a shared or register tensor)
      if (o.end0 - o.start0 != sg.end0 - sg.start0 || o.end1 - o.start1 != sg.end1 - sg.start1 || o.dtype != sg.dtype) return false;
      if (o.ptr != o0.ptr || o.stride0 != o0.stride0 || o.stride1 != o0.stride1 || o.dtype != o0.dtype || o.alignment != o0.alignment ||
          o.end0 - o.start0 != o0.end0 - o0.start0 || o.end1 - o.start1 != o0.end1 - o0.start1)
        return false;
    }
    // the grid of tiles, from the result views
    const int32_t R = out[0].end0 - out[0].start0, C = out[0].end1 - out[0].start1;
    if (R <= 0 || C <= 0) return false;
    int32_t o0 = out[0].start0, o1 = out[0].start1;
    for (int w = 1; w < n; ++w) { o0 = std::min(o0, out[w].start0); o1 = std::min(o1, out[w].start1); }
    std::vector<int32_t> a(n), b(n);
    int32_t I = 0, J = 0;
    std::set<std::pair<int32_t, int32_t>> tiles;
    for (int w = 0; w < n; ++w) {
      if ((out[w].start0 - o0) % R || (out[w].start1 - o1) % C) return false;
      a[w] = (out[w].start0 - o0) / R;
      b[w] = (out[w].start1 - o1) / C;
      I = std::max(I, a[w] + 1);
      J = std::max(J, b[w] + 1);
      if (!tiles.insert({a[w], b[w]}).second) return false;
    }
    if ((int64_t)I * J != n) return false;
    if ((int64_t)R * I > 0x7fffffff - o0 || (int64_t)C * J > 0x7fffffff - o1) return false;
    // what a store does first: deferred values that still read the memory it writes are computed - once, for the union of the
    // instances' views (all their stores stand at this point of the program); a source that this computes is no chain any more
    kapy_global all = out[0];
    all.start0 = o0; all.end0 = o0 + R * I;
    all.start1 = o1; all.end1 = o1 + C * J;
    // (register tensors made from here on come from the group's own region of the arena, which is never handed out twice
    // while the group lives: no warp is swapped in, so no warp's share can be used)
    struct Region {
      Interp &in;
      size_t top_was, limit_was;
      explicit Region(Interp &i) : in(i), top_was(i.top), limit_was(i.limit) {
        in.top = in.merged_top;
        in.limit = in.merged_base + kMergedArena;
      }
      ~Region() {
        in.merged_top = in.top;
        in.top = top_was;
        in.limit = limit_was;
      }
    } region(*this);
    {
      const std::string before = err;
      if (settle_readers(op, all) != KAPY_OK) { err = before; return false; }  // (the instance's own run reports it)
    }
    for (int w = 0; w < n; ++w) {
      auto src = warps[w].env.find(op.operands[0]);
      if (!src->second.lazy) return false;
      chain[w] = src->second.lazy;
    }
    // the leaves of every instance's chain, in one order
    std::vector<std::vector<const Expr *>> leaves(n);
    {
      std::map<const Expr *, const Expr *> pairs;
      if (!same_form(chain[0].get(), chain[0].get(), pairs, &leaves[0])) return false;
    }
    for (int w = 1; w < n; ++w) {
      std::map<const Expr *, const Expr *> pairs;
      if (!same_form(chain[0].get(), chain[w].get(), pairs, &leaves[w]) || leaves[w].size() != leaves[0].size()) return false;
    }
    // every leaf: with the tile along an axis, or of extent 1 and the same for all
    struct Axis { int32_t origin; bool moves; };
    std::vector<Axis> l0(leaves[0].size()), l1(leaves[0].size());
    for (size_t k = 0; k < leaves[0].size(); ++k) {
      const int32_t r = leaves[0][k]->leaf.end0 - leaves[0][k]->leaf.start0, c = leaves[0][k]->leaf.end1 - leaves[0][k]->leaf.start1;
      int32_t m0 = leaves[0][k]->leaf.start0, m1 = leaves[0][k]->leaf.start1;
      for (int w = 1; w < n; ++w) { m0 = std::min(m0, leaves[w][k]->leaf.start0); m1 = std::min(m1, leaves[w][k]->leaf.start1); }
      bool moves0 = true, still0 = true, moves1 = true, still1 = true;
      for (int w = 0; w < n; ++w) {
        const int64_t d0 = leaves[w][k]->leaf.start0 - m0, d1 = leaves[w][k]->leaf.start1 - m1;
        moves0 = moves0 && d0 == (int64_t)a[w] * r;
        still0 = still0 && d0 == 0;
        moves1 = moves1 && d1 == (int64_t)b[w] * c;
        still1 = still1 && d1 == 0;
      }
      if (I > 1 ? !((moves0 && r == R) || (still0 && r == 1 && R != 1) || (R == 1 && r == 1 && (moves0 || still0))) : !still0) return false;
      if (J > 1 ? !((moves1 && c == C) || (still1 && c == 1 && C != 1) || (C == 1 && c == 1 && (moves1 || still1))) : !still1) return false;
      l0[k] = {m0, I > 1 && moves0 && !(still0)};
      l1[k] = {m1, J > 1 && moves1 && !(still1)};
      if ((int64_t)r * I > 0x7fffffff - m0 || (int64_t)c * J > 0x7fffffff - m1) return false;
    }
    // the union as one chain
    std::map<const Expr *, std::shared_ptr<Expr>> made;
    std::shared_ptr<Expr> whole = clone(chain[0], made);
    for (size_t k = 0; k < leaves[0].size(); ++k) {
      kapy_global &g = made[leaves[0][k]]->leaf;
      const int32_t r = g.end0 - g.start0, c = g.end1 - g.start1;
      g.start0 = l0[k].origin;
      g.end0 = g.start0 + (l0[k].moves ? r * I : r);
      g.start1 = l1[k].origin;
      g.end1 = g.start1 + (l1[k].moves ? c * J : c);
    }
    for (auto &kv : made) {
      Expr &e = *kv.second;
      if (e.ew == KAPY_EW_ARANGE) return false;
      if (is_reduce(e)) {
        if ((e.axis == 1 && (J > 1 || e.rows != R)) || (e.axis == 0 && (I > 1 || e.cols != C)) || (e.axis != 0 && e.axis != 1)) return false;
        if (e.axis == 1) e.rows *= I;
        else e.cols *= J;
      }
    }
    // run it from the group's own region of the arena (reduces that leave the program need register tensors of the union's size)
    const std::string before = err;
    const int rc = run_chain(op, whole, &all);
    if (rc == KAPY_OK) { ++merged_calls; return true; }
    err = before;  // refused as a whole: the instances run their own stores
    return false;
  }
  int64_t merged_calls = 0;

  int run_ops(const std::vector<Op> &ops, std::vector<Value> *yielded) {
    for (const Op &op : ops) {
      int rc = run_op(op, yielded);
      if (rc != KAPY_OK) return rc;
    }
    return KAPY_OK;
  }

  // All warps in step through `ops` (see WarpState).  yielded: one list per warp, filled by the body's scf.yield.
  int run_ops_in_step(const std::vector<Op> &ops, std::vector<std::vector<Value>> *yielded) {
    const int W = (int)warps.size();
    for (const Op &op : ops) {
      if (op.name == "scf.for") {
        int rc = run_for_in_step(op);
        if (rc != KAPY_OK) return rc;
        continue;
      }
      if (merge && fuse && op.name == "kapy.st_global" && try_merged_store(op)) continue;
      for (int w = 0; w < W; ++w) {
        enter(w);
        int rc = run_op(op, yielded ? &(*yielded)[w] : nullptr);
        leave(w);
        if (rc != KAPY_OK) return rc;
      }
    }
    return KAPY_OK;
  }
  // scf.for with every warp taking the same trips: the iterations themselves run in step.  Warps that disagree on the bounds
  // cannot meet at a barrier inside the loop, so such a loop is run warp after warp.
  int run_for_in_step(const Op &op) {
    const int W = (int)warps.size();
    if (op.region_args.empty()) return fail_op(op, "scf.for without an induction variable");
    const size_t n_iter = op.region_args.size() - 1;
    std::vector<int64_t> lo(W), hi(W), st(W);
    std::vector<std::vector<Value>> carried(W, std::vector<Value>(n_iter));
    bool same = true;
    for (int w = 0; w < W; ++w) {
      enter(w);
      Value l, h, s;
      bool ok = get(op, 0, Value::kInt, l) && get(op, 1, Value::kInt, h) && get(op, 2, Value::kInt, s);
      for (size_t k = 0; ok && k < n_iter; ++k) {
        auto it = 3 + k < op.operands.size() ? env.find(op.operands[3 + k]) : env.end();
        if (it == env.end()) { fail_op(op, "use of undefined loop operand"); ok = false; break; }
        carried[w][k] = it->second;
      }
      leave(w);
      if (!ok) return KAPY_ERR_INVALID;
      if (s.i <= 0) return fail_op(op, "step must be positive");
      lo[w] = l.i; hi[w] = h.i; st[w] = s.i;
      same = same && lo[w] == lo[0] && hi[w] == hi[0] && st[w] == st[0];
    }
    if (!same) {
      for (int w = 0; w < W; ++w) {
        enter(w);
        int rc = run_op(op, nullptr);
        leave(w);
        if (rc != KAPY_OK) return rc;
      }
      return KAPY_OK;
    }
    for (int64_t iv = lo[0]; iv < hi[0]; iv += st[0]) {
      for (int w = 0; w < W; ++w) {
        Value ivv;
        ivv.kind = Value::kInt;
        ivv.i = iv;
        warps[w].env[op.region_args[0]] = ivv;
        for (size_t k = 0; k < n_iter; ++k) warps[w].env[op.region_args[1 + k]] = carried[w][k];
      }
      std::vector<std::vector<Value>> y(W);
      int rc = run_ops_in_step(op.body, &y);
      if (rc != KAPY_OK) return rc;
      for (int w = 0; w < W; ++w) {
        if (y[w].size() != n_iter) return fail_op(op, "scf.yield does not match iter_args");
        carried[w] = y[w];
      }
    }
    for (int w = 0; w < W; ++w)
      for (size_t k = 0; k < n_iter && k < op.results.size(); ++k) warps[w].env[op.results[k]] = carried[w][k];
    return KAPY_OK;
  }

  int run_op(const Op &op, std::vector<Value> *yielded) {
    const std::string &n = op.name;
    Value a, b, c, r;
    if (n == "kapy.return") return KAPY_OK;
    if (n == "scf.yield") {
      if (!yielded) return fail_op(op, "yield outside a loop");
      yielded->clear();
      for (size_t k = 0; k < op.operands.size(); ++k) {
        auto it = env.find(op.operands[k]);
        if (it == env.end()) return fail_op(op, "use of undefined value " + op.operands[k]);
        if (it->second.lazy) {  // a loop-carried tensor is computed once per iteration
          int rc = force(op, it->second);
          if (rc != KAPY_OK) return rc;
        }
        yielded->push_back(it->second);
      }
      return KAPY_OK;
    }
    if (n == "arith.constant") {
      if (op.types.empty()) return fail_op(op, "constant without a type");
      const Type &ty = op.types.back();
      if (ty.kind == Type::kInt) {
        r.kind = Value::kInt;
        const std::string &w = op.words.empty() ? std::string("0") : op.words[0];
        r.i = w == "true" ? 1 : w == "false" ? 0 : atoll(w.c_str());
      } else if (ty.kind == Type::kFloat) {
        r.kind = Value::kFloat;
        r.f = op.words.empty() ? 0.0 : float_literal(op.words[0], ty.dtype);
      } else if (ty.kind == Type::kTensor) {
        if (ty.dtype >= KAPY_I8) {  // dense<3> : tensor<..xi32>, dense<true> : tensor<..xi1>
          const std::string &w = op.words.empty() ? std::string("0") : op.words[0];
          return defer(op, 0, KAPY_EW_SPLAT, ty.dtype, KAPY_RN, 0.f, w == "true" ? 1 : w == "false" ? 0 : (int32_t)atoll(w.c_str()));
        }
        return defer(op, 0, KAPY_EW_SPLAT, ty.dtype, KAPY_RN, op.words.empty() ? 0.f : (float)float_literal(op.words[0], ty.dtype));
      } else return fail_op(op, "unsupported constant type");
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.program_id") {
      r.kind = Value::kInt;
      int axis = op.attrs.count("axis") ? atoi(op.attrs.at("axis").c_str()) : 0;
      if (axis < 0 || axis > 2) return fail_op(op, "axis must be 0, 1 or 2");
      r.i = pid[axis];
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.warp_id") { r.kind = Value::kInt; r.i = warp; env[op.results[0]] = r; return KAPY_OK; }
    // integer, compare, select and conversion ops on tensors (ElementwiseOpToLLVM.cpp:1178-1215, SelectOpToLLVM.cpp:21-98): one
    // instruction of a deferred program each; the same ops on scalars are evaluated on the host below
    const bool on_tensor = !op.operands.empty() && env.count(op.operands[0]) && env[op.operands[0]].kind == Value::kTensor;
    if (on_tensor) {
      static const struct { const char *name; int ew; } int_binary[] = {
          {"arith.addi", KAPY_EW_ADDI}, {"arith.subi", KAPY_EW_SUBI}, {"arith.muli", KAPY_EW_MULI}, {"arith.divsi", KAPY_EW_DIVSI}, {"arith.divui", KAPY_EW_DIVUI},
          {"arith.floordivsi", KAPY_EW_FLOORDIVSI}, {"arith.ceildivsi", KAPY_EW_CEILDIVSI}, {"arith.ceildivui", KAPY_EW_CEILDIVUI}, {"arith.remsi", KAPY_EW_REMSI},
          {"arith.remui", KAPY_EW_REMUI}, {"arith.andi", KAPY_EW_ANDI}, {"arith.ori", KAPY_EW_ORI}, {"arith.xori", KAPY_EW_XORI}, {"arith.shli", KAPY_EW_SHLI},
          {"arith.shrsi", KAPY_EW_SHRSI}, {"arith.shrui", KAPY_EW_SHRUI}, {"arith.maxsi", KAPY_EW_MAXSI}, {"arith.maxui", KAPY_EW_MAXUI}, {"arith.minsi", KAPY_EW_MINSI},
          {"arith.minui", KAPY_EW_MINUI}};
      for (auto &u : int_binary)
        if (n == u.name) return binary_tensor(op, u.ew);
      if (n == "arith.cmpi" || n == "arith.cmpf") {
        static const char *const cmpi[] = {"eq", "ne", "slt", "sle", "sgt", "sge", "ult", "ule", "ugt", "uge"};
        static const char *const cmpf[] = {"false", "oeq", "ogt", "oge", "olt", "ole", "one", "ord", "ueq", "ugt", "uge", "ult", "ule", "une", "uno", "true"};
        const std::string &pr = op.words.empty() ? std::string("?") : op.words[0];
        int pred = -1;
        if (n == "arith.cmpi") { for (int k = 0; k < 10; ++k) if (pr == cmpi[k]) pred = k; }
        else { for (int k = 0; k < 16; ++k) if (pr == cmpf[k]) pred = k; }
        if (pred < 0) return fail_op(op, "unknown compare predicate '" + pr + "'");
        if (op.types.empty()) return fail_op(op, "compare without a type");
        Op typed = op;  // the type written after a compare is its operands'; the result has that shape with element type i1
        typed.types.back().dtype = KAPY_I1;
        return defer(typed, 2, n == "arith.cmpi" ? KAPY_EW_CMPI : KAPY_EW_CMPF, KAPY_I1, KAPY_RN, 0.f, 0, 0, pred);
      }
      if (n == "arith.select") return defer(op, 3, KAPY_EW_SELECT, 0, KAPY_RN, 0.f);
      static const struct { const char *name; int ew; } int_unary[] = {
          {"arith.trunci", KAPY_EW_TRUNCI}, {"arith.extsi", KAPY_EW_EXTSI}, {"arith.extui", KAPY_EW_EXTUI}, {"arith.sitofp", KAPY_EW_SITOFP},
          {"arith.fptosi", KAPY_EW_FPTOSI}, {"arith.bitcast", KAPY_EW_BITCAST}, {"math.absi", KAPY_EW_ABSI}};
      for (auto &u : int_unary)
        if (n == u.name) return mapped_tensor(op, 1, u.ew, op.types.empty() ? 0 : op.types.back().dtype);
    }
    if (n == "kapy.arange") {  // i32 values start, start + 1, ... along `axis` (ArangeOpToLLVM.cpp:22-50)
      const int axis = op.attrs.count("axis") ? atoi(op.attrs.at("axis").c_str()) : 0, start = op.attrs.count("start") ? atoi(op.attrs.at("start").c_str()) : 0;
      if (axis != 0 && axis != 1) return fail_op(op, "axis must be 0 or 1");
      return defer(op, 0, KAPY_EW_ARANGE, KAPY_I32, KAPY_RN, 0.f, start, axis);
    }
    if (n == "arith.addi" || n == "arith.subi" || n == "arith.muli" || n == "arith.divui" || n == "arith.remui" || n == "arith.cmpi") {
      if (!get(op, 0, Value::kInt, a) || !get(op, 1, Value::kInt, b)) return KAPY_ERR_INVALID;
      r.kind = Value::kInt;
      const uint32_t ua = (uint32_t)a.i, ub = (uint32_t)b.i;
      if (n == "arith.addi") r.i = (int32_t)(ua + ub);
      else if (n == "arith.subi") r.i = (int32_t)(ua - ub);
      else if (n == "arith.muli") r.i = (int32_t)(ua * ub);
      else if (n == "arith.cmpi") {
        const std::string &pr = op.words.empty() ? std::string("eq") : op.words[0];
        const int32_t sa = (int32_t)a.i, sb = (int32_t)b.i;
        r.i = pr == "eq" ? sa == sb : pr == "ne" ? sa != sb : pr == "slt" ? sa < sb : pr == "sle" ? sa <= sb : pr == "sgt" ? sa > sb :
              pr == "sge" ? sa >= sb : pr == "ult" ? ua < ub : pr == "ule" ? ua <= ub : pr == "ugt" ? ua > ub : ua >= ub;
      } else {
        if (ub == 0) return fail_op(op, "division by zero");
        r.i = n == "arith.divui" ? (int32_t)(ua / ub) : (int32_t)(ua % ub);
      }
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "arith.select") {
      if (!get(op, 0, Value::kInt, a)) return KAPY_ERR_INVALID;
      auto it = env.find(op.operands[a.i ? 1 : 2]);
      if (it == env.end()) return fail_op(op, "use of undefined value");
      env[op.results[0]] = it->second;
      return KAPY_OK;
    }
    if (n == "arith.addf") return binary_tensor(op, KAPY_EW_ADDF);
    if (n == "arith.subf") return binary_tensor(op, KAPY_EW_SUBF);
    if (n == "arith.mulf") return binary_tensor(op, KAPY_EW_MULF);
    if (n == "arith.divf") return binary_tensor(op, KAPY_EW_DIVF);
    if (n == "arith.maximumf") return binary_tensor(op, KAPY_EW_MAXIMUMF);
    if (n == "arith.minimumf") return binary_tensor(op, KAPY_EW_MINIMUMF);
    if (n == "arith.maxnumf") return binary_tensor(op, KAPY_EW_MAXNUMF);
    if (n == "arith.minnumf") return binary_tensor(op, KAPY_EW_MINNUMF);
    if (n == "arith.remf") return binary_tensor(op, KAPY_EW_REMF);
    {
      static const struct { const char *name; int ew; } unary[] = {
          {"math.exp", KAPY_EW_EXP}, {"math.exp2", KAPY_EW_EXP2}, {"math.log", KAPY_EW_LOG}, {"math.log2", KAPY_EW_LOG2},
          {"math.sqrt", KAPY_EW_SQRT}, {"math.rsqrt", KAPY_EW_RSQRT}, {"math.tanh", KAPY_EW_TANH}, {"math.erf", KAPY_EW_ERF},
          {"math.absf", KAPY_EW_ABSF}, {"arith.negf", KAPY_EW_NEGF}, {"math.floor", KAPY_EW_FLOOR}, {"math.ceil", KAPY_EW_CEIL},
          {"math.sin", KAPY_EW_SIN}, {"math.cos", KAPY_EW_COS}};
      for (auto &u : unary)
        if (n == u.name) return mapped_tensor(op, 1, u.ew);
    }
    if (n == "math.fma") return mapped_tensor(op, 3, KAPY_EW_FMA);
    if (n == "kapy.broadcast") return mapped_tensor(op, 1, -1);
    if (n == "kapy.fptofp" || n == "arith.extf" || n == "arith.truncf") {
      if (op.types.empty()) return fail_op(op, "cast without a result type");
      int rmode = KAPY_RN;  // arith.truncf rounds to nearest even; kapy.fptofp carries its mode (Enums.td: rz = 0, rn = 1)
      auto it = op.attrs.find("rounding_mode");
      if (it != op.attrs.end()) rmode = (it->second == "0" || it->second.find("rz") != std::string::npos) ? KAPY_RZ : KAPY_RN;
      return mapped_tensor(op, 1, KAPY_EW_FPTOFP, op.types.back().dtype, rmode);
    }
    if (n == "kapy.splat") {
      Value v;
      if (!op.operands.empty() && env.count(op.operands[0]) && env[op.operands[0]].kind == Value::kInt && !op.types.empty()) {  // an integer scalar
        const int64_t i = env[op.operands[0]].i;
        return defer(op, 0, KAPY_EW_SPLAT, op.types.back().dtype, KAPY_RN, (float)i, (int32_t)i);
      }
      if (!get(op, 0, Value::kFloat, v) || op.types.empty()) return KAPY_ERR_INVALID;
      return defer(op, 0, KAPY_EW_SPLAT, op.types.back().dtype, KAPY_RN, (float)v.f);
    }
    if (n == "kapy.transpose") {  // result[j, i] = source[i, j] (TransposeOpToLLVM.cpp:21-26 relabels; here the data moves)
      if (!get(op, 0, Value::kTensor, a) || op.types.empty() || !new_tensor(op, op.types.back(), r)) return KAPY_ERR_INVALID;
      kapy_copy_cfg cfg;
      memset(&cfg, 0, sizeof cfg);
      cfg.transpose = 1;
      int rc = lib(op, do_copy(&a.g, &r.g, &cfg));
      if (rc) return rc;
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.mk_global") {
      Value off, s0, s1, t0, t1;
      if (!get(op, 0, Value::kPtr, a) || !get(op, 1, Value::kInt, off) || !get(op, 2, Value::kInt, s0) || !get(op, 3, Value::kInt, s1) ||
          !get(op, 4, Value::kInt, t0) || !get(op, 5, Value::kInt, t1) || op.types.empty())
        return KAPY_ERR_INVALID;
      const int eb = dtype_bytes(op.types.back().dtype);
      if (s0.i < 0 || s1.i < 0 || t0.i < 0 || t1.i < 0 || off.i < 0) return fail_op(op, "negative size, stride or offset");
      if (a.bytes > 0 && s0.i > 0 && s1.i > 0 && (off.i + (s0.i - 1) * t0.i + (s1.i - 1) * t1.i + 1) * eb > a.bytes)
        return fail_op(op, "the tensor reaches beyond the " + std::to_string(a.bytes) + " bytes of its pointer argument");
      r.kind = Value::kTensor;
      int rc = lib(op, kapy_mk_global(&r.g, a.ptr, (int32_t)off.i, (int32_t)s0.i, (int32_t)s1.i, (int32_t)t0.i, (int32_t)t1.i, op.types.back().dtype, 16));
      if (rc) return rc;
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.mk_shared") {
      if (op.types.empty()) return fail_op(op, "mk_shared without a type");
      return mk_shared(op);
    }
    if (n == "kapy.sv_global" || n == "kapy.sv_shared") {
      Value s0, e0, s1, e1;
      if (!get(op, 0, Value::kTensor, a) || !get(op, 1, Value::kInt, s0) || !get(op, 2, Value::kInt, e0) || !get(op, 3, Value::kInt, s1) ||
          !get(op, 4, Value::kInt, e1))
        return KAPY_ERR_INVALID;
      // the reference leaves a view that leaves its parent to the load's mask; here it is an error, so that
      // no access of the program can leave the memory the caller named
      if (s0.i < 0 || s1.i < 0 || e0.i < s0.i || e1.i < s1.i || a.g.start0 + e0.i > a.g.end0 || a.g.start1 + e1.i > a.g.end1)
        return fail_op(op, "the sub-view leaves its parent");
      r.kind = Value::kTensor;
      int rc = lib(op, kapy_sv_global(&r.g, &a.g, (int32_t)s0.i, (int32_t)e0.i, (int32_t)s1.i, (int32_t)e1.i));
      if (rc) return rc;
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.ld_global" && fuse && !op.types.empty() && op.types.back().kind == Type::kTensor) {
      // a load of a whole view of the caller's memory joins the deferred chain: the program that needs the value reads the
      // view itself.  A store that could change the view before then computes the value first (settle_readers).
      Value src;
      if (!get(op, 0, Value::kTensor, src)) return KAPY_ERR_INVALID;
      const Type &ty = op.types.back();
      const char *p = (const char *)src.g.ptr;
      if (!(p >= arena && p < arena + kArena) && ty.shape[0] == src.g.end0 - src.g.start0 && ty.shape[1] == src.g.end1 - src.g.start1 &&
          ty.dtype == src.g.dtype && ty.shape[0] > 0 && ty.shape[1] > 0 && src.g.stride0 > 0 && src.g.stride1 > 0) {
        auto e = std::make_shared<Expr>();
        e->leaf = src.g;
        e->global_leaf = true;
        r.kind = Value::kTensor;
        r.lazy = e;
        ++lazy_made;
        memset(&r.g, 0, sizeof r.g);
        int rc = lib(op, kapy_mk_global(&r.g, arena, 0, (int32_t)ty.shape[0], (int32_t)ty.shape[1], (int32_t)ty.shape[1], 1, ty.dtype, 16));
        if (rc) return rc;
        env[op.results[0]] = r;
        return KAPY_OK;
      }
    }
    if (n == "kapy.ld_global" || n == "kapy.ld_matrix" || n == "kapy.ld_shared") {
      if (!get(op, 0, Value::kTensor, a) || op.types.empty() || !new_tensor(op, op.types.back(), r)) return KAPY_ERR_INVALID;
      int rc = lib(op, do_copy(&a.g, &r.g, nullptr));
      if (rc) return rc;
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.st_global" || n == "kapy.st_shared" || n == "kapy.cp_async_global_to_shared") {
      // a deferred chain stores straight into a view of its own shape; anything else (padding, a program the
      // elementwise entry point refuses) goes through a register tensor as before
      if (n == "kapy.st_global") {
        if (!get(op, 1, Value::kTensor, b)) return KAPY_ERR_INVALID;
        int rc = settle_readers(op, b.g);
        if (rc != KAPY_OK) return rc;
      }
      auto src = op.operands.empty() ? env.end() : env.find(op.operands[0]);
      if (src != env.end() && src->second.kind == Value::kTensor && src->second.lazy) {
        if (!get(op, 1, Value::kTensor, b)) return KAPY_ERR_INVALID;
        const kapy_global &sg = src->second.g;
        if (b.g.end0 - b.g.start0 == sg.end0 - sg.start0 && b.g.end1 - b.g.start1 == sg.end1 - sg.start1 && b.g.dtype == sg.dtype) {
          const std::string before = err;
          if (run_chain(op, src->second.lazy, &b.g) == KAPY_OK) return KAPY_OK;
          err = before;  // the refusal is not the call's error: the store is tried again below through a register tensor
        }
      }
      if (!get(op, 0, Value::kTensor, a) || !get(op, 1, Value::kTensor, b)) return KAPY_ERR_INVALID;
      return lib(op, do_copy(&a.g, &b.g, nullptr));
    }
    if (n == "kapy.cp_async_wait_group" || n == "nvvm.barrier0") return KAPY_OK;  // every op is complete in stream order
    if (n == "kapy.matmul") {
      if (!get(op, 0, Value::kTensor, a) || !get(op, 1, Value::kTensor, b) || !get(op, 2, Value::kTensor, c) || op.types.empty() ||
          !new_tensor(op, op.types.back(), r))
        return KAPY_ERR_INVALID;
      kapy_matmul_cfg cfg;
      memset(&cfg, 0, sizeof cfg);
      cfg.rmode = KAPY_RN;
      const std::string &way = op.words.empty() ? std::string() : op.words[0];
      cfg.impl_way = way == "mma_m16n8k8_f16" ? KAPY_MMA_M16N8K8_F16 : way == "mma_m16n8k16_f16" ? KAPY_MMA_M16N8K16_F16 :
                     way == "mma_m16n8k16_f8" ? KAPY_MMA_M16N8K16_F8 : way == "mma_m16n8k8_tf32" ? KAPY_MMA_M16N8K8_TF32 : KAPY_MATMUL_AUTO;
      // KAPY_MLIR_MATMUL=reference: f16 x f16 -> f16 products keep f16 accumulators, rounded once per instruction of the named
      // way, as the reference's .f16.f16.f16.f16 instruction does (MatmulOpToLLVM.cpp:270-291); other types have fp32 accumulators there too
      const char *matmul_mode = getenv("KAPY_MLIR_MATMUL");
      if (matmul_mode && std::string(matmul_mode) == "reference" && a.g.dtype == KAPY_F16 && b.g.dtype == KAPY_F16 && c.g.dtype == KAPY_F16 && r.g.dtype == KAPY_F16)
        cfg.accumulate = KAPY_ACCUMULATE_ELEMENT;
      int rc = lib(op, do_matmul(&a.g, &b.g, &c.g, &r.g, &cfg));
      if (rc) return rc;
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "kapy.reduce") {
      // the combiner region: one arith op on the two block arguments (what kapy_reduce_combiner names)
      static const struct { const char *name; int kind; } combiners[] = {
          {"arith.addf", KAPY_REDUCE_ADDF}, {"arith.maximumf", KAPY_REDUCE_MAXIMUMF}, {"arith.minimumf", KAPY_REDUCE_MINIMUMF}, {"arith.mulf", KAPY_REDUCE_MULF},
          {"arith.maxnumf", KAPY_REDUCE_MAXNUMF}, {"arith.minnumf", KAPY_REDUCE_MINNUMF}, {"arith.addi", KAPY_REDUCE_ADDI}, {"arith.muli", KAPY_REDUCE_MULI},
          {"arith.maxsi", KAPY_REDUCE_MAXSI}, {"arith.minsi", KAPY_REDUCE_MINSI}, {"arith.maxui", KAPY_REDUCE_MAXUI}, {"arith.minui", KAPY_REDUCE_MINUI},
          {"arith.andi", KAPY_REDUCE_ANDI}, {"arith.ori", KAPY_REDUCE_ORI}, {"arith.xori", KAPY_REDUCE_XORI}};
      int kind = -1, n_ops = 0;
      for (const Op &inner : op.body) {
        if (inner.name == "kapy.return") continue;
        ++n_ops;
        for (auto &c : combiners)
          if (inner.name == c.name) kind = c.kind;
      }
      if (kind < 0 || n_ops != 1) return fail_op(op, "the combiner must be one arith op (addf, maximumf, minimumf, mulf, maxnumf, minnumf or an integer op)");
      int axis = op.attrs.count("axis") ? atoi(op.attrs.at("axis").c_str()) : 0;
      // KAPY_MLIR_REDUCE=reference: the lowering's own arithmetic for the warp's tile (partial results on the element type, lane-serial
      // fold then butterfly, ReduceOpToLLVM.cpp:76-119) instead of fp32 accumulation; such a reduce is a call of its own
      const char *reduce_mode = getenv("KAPY_MLIR_REDUCE");
      const bool reference = reduce_mode && std::string(reduce_mode) == "reference";
      // over a register tensor the reduce joins the deferred chain: followed by a broadcast back to the operand's shape it
      // becomes an instruction of the program that consumes it (along rows: the row programs; along columns: the column machine)
      auto src = op.operands.empty() ? env.end() : env.find(op.operands[0]);
      if (fuse && !reference && kind <= KAPY_REDUCE_MAXIMUMF && (axis == 0 || axis == 1) && !op.types.empty() && op.types.back().kind == Type::kTensor && src != env.end() &&
          src->second.kind == Value::kTensor && (src->second.lazy || is_register_tensor(src->second.g))) {
        const kapy_global &sg = src->second.g;
        const Type &ty = op.types.back();
        const bool kept_shape = axis == 1 ? ty.shape[0] == sg.end0 - sg.start0 && ty.shape[1] == 1 : ty.shape[0] == 1 && ty.shape[1] == sg.end1 - sg.start1;
        if (kept_shape && ty.dtype == sg.dtype) {
          auto e = std::make_shared<Expr>();
          e->ew = kind == 1 ? KAPY_EW_REDUCE_MAX : KAPY_EW_REDUCE_SUM;
          e->axis = axis;
          e->n_in = 1;
          e->in[0] = as_expr(src->second);
          e->rows = sg.end0 - sg.start0; e->cols = sg.end1 - sg.start1; e->operand_dtype = sg.dtype;
          if (fits(e)) {
            r.kind = Value::kTensor;
            r.lazy = e;
            ++lazy_made;
            memset(&r.g, 0, sizeof r.g);
            int rc = lib(op, kapy_mk_global(&r.g, arena, 0, (int32_t)ty.shape[0], (int32_t)ty.shape[1], (int32_t)ty.shape[1], 1, ty.dtype, 16));
            if (rc) return rc;
            env[op.results[0]] = r;
            return KAPY_OK;
          }
        }
      }
      if (!get(op, 0, Value::kTensor, a) || op.types.empty() || !new_tensor(op, op.types.back(), r)) return KAPY_ERR_INVALID;
      kapy_reduce_cfg rcfg = {kind, reference ? KAPY_REDUCE_REFERENCE : KAPY_REDUCE_WIDE, nullptr, nullptr, 0};
      int rc = lib(op, do_reduce_ex(&a.g, &r.g, axis, &rcfg));
      if (rc) return rc;
      env[op.results[0]] = r;
      return KAPY_OK;
    }
    if (n == "scf.for") {
      Value lo, hi, st;
      if (!get(op, 0, Value::kInt, lo) || !get(op, 1, Value::kInt, hi) || !get(op, 2, Value::kInt, st)) return KAPY_ERR_INVALID;
      if (st.i <= 0) return fail_op(op, "step must be positive");
      const size_t n_iter = op.region_args.size() - 1;
      std::vector<Value> carried(n_iter);
      for (size_t k = 0; k < n_iter; ++k) {
        auto it = env.find(op.operands[3 + k]);
        if (it == env.end()) return fail_op(op, "use of undefined value " + op.operands[3 + k]);
        carried[k] = it->second;
      }
      for (int64_t iv = lo.i; iv < hi.i; iv += st.i) {
        Value ivv;
        ivv.kind = Value::kInt;
        ivv.i = iv;
        env[op.region_args[0]] = ivv;
        for (size_t k = 0; k < n_iter; ++k) env[op.region_args[1 + k]] = carried[k];
        std::vector<Value> y;
        int rc = run_ops(op.body, &y);
        if (rc) return rc;
        if (y.size() != n_iter) return fail_op(op, "scf.yield does not match iter_args");
        carried = y;
      }
      for (size_t k = 0; k < n_iter && k < op.results.size(); ++k) env[op.results[k]] = carried[k];
      return KAPY_OK;
    }
    return fail_op(op, "operation is not supported by this front-end");
  }
};

// The ops this front-end executes, with the number of operands each needs at least and the number of results it has
// (-1: any); the interpreter indexes operands and results by these counts without looking again.
const struct OpForm { const char *name; int min_operands, results; } kSupportedOps[] = {
    {"kapy.return", 0, 0}, {"scf.yield", 0, 0}, {"scf.for", 3, -1}, {"arith.constant", 0, 1}, {"kapy.program_id", 0, 1}, {"kapy.warp_id", 0, 1},
    {"arith.addi", 2, 1}, {"arith.subi", 2, 1}, {"arith.muli", 2, 1}, {"arith.divui", 2, 1}, {"arith.remui", 2, 1}, {"arith.cmpi", 2, 1},
    {"arith.select", 3, 1}, {"arith.addf", 2, 1}, {"arith.subf", 2, 1}, {"arith.mulf", 2, 1}, {"arith.divf", 2, 1}, {"arith.maximumf", 2, 1},
    {"arith.minimumf", 2, 1}, {"arith.maxnumf", 2, 1}, {"arith.minnumf", 2, 1}, {"arith.remf", 2, 1}, {"kapy.mk_global", 6, 1}, {"kapy.mk_shared", 0, 1}, {"kapy.sv_global", 5, 1}, {"kapy.sv_shared", 5, 1},
    {"kapy.ld_global", 1, 1}, {"kapy.ld_matrix", 1, 1}, {"kapy.ld_shared", 1, 1}, {"kapy.st_global", 2, 0}, {"kapy.st_shared", 2, 0},
    {"kapy.cp_async_global_to_shared", 2, 0}, {"kapy.cp_async_wait_group", 0, 0}, {"kapy.matmul", 3, 1}, {"kapy.reduce", 1, 1},
    {"nvvm.barrier0", 0, 0}, {"math.exp", 1, 1}, {"math.exp2", 1, 1}, {"math.log", 1, 1}, {"math.log2", 1, 1}, {"math.sqrt", 1, 1},
    {"math.rsqrt", 1, 1}, {"math.tanh", 1, 1}, {"math.erf", 1, 1}, {"math.absf", 1, 1}, {"math.floor", 1, 1}, {"math.ceil", 1, 1}, {"math.sin", 1, 1}, {"math.cos", 1, 1}, {"math.fma", 3, 1}, {"arith.negf", 1, 1},
    {"arith.extf", 1, 1}, {"arith.truncf", 1, 1}, {"kapy.fptofp", 1, 1}, {"kapy.splat", 1, 1}, {"kapy.broadcast", 1, 1}, {"kapy.transpose", 1, 1},
    {"arith.divsi", 2, 1}, {"arith.floordivsi", 2, 1}, {"arith.ceildivsi", 2, 1}, {"arith.ceildivui", 2, 1}, {"arith.remsi", 2, 1}, {"arith.andi", 2, 1},
    {"arith.ori", 2, 1}, {"arith.xori", 2, 1}, {"arith.shli", 2, 1}, {"arith.shrsi", 2, 1}, {"arith.shrui", 2, 1}, {"arith.maxsi", 2, 1}, {"arith.maxui", 2, 1},
    {"arith.minsi", 2, 1}, {"arith.minui", 2, 1}, {"arith.cmpf", 2, 1}, {"arith.trunci", 1, 1}, {"arith.extsi", 1, 1}, {"arith.extui", 1, 1},
    {"arith.sitofp", 1, 1}, {"arith.fptosi", 1, 1}, {"arith.bitcast", 1, 1}, {"math.absi", 1, 1}, {"kapy.arange", 0, 1}};

// Every op must be one this front-end executes, written with the operands and results it needs; returns the number of ops,
// regions included, -1 for an op it does not execute, -2 for one that is malformed.  (The body of a kapy.reduce is only looked at for its combiner: its ops are not executed.)
int count_ops(const std::vector<Op> &ops, bool in_reduce, std::string &err) {
  int n = 0;
  for (const Op &op : ops) {
    const OpForm *form = nullptr;
    for (const OpForm &k : kSupportedOps)
      if (op.name == k.name) form = &k;
    if (!form) {
      err = "line " + std::to_string(op.line) + ": operation '" + op.name + "' is not supported by this front-end";
      return -1;
    }
    if (!in_reduce) {
      bool well_formed = (int)op.operands.size() >= form->min_operands && (form->results < 0 || (int)op.results.size() == form->results);
      if (op.name == "scf.for")  // an induction variable, then one region argument and at most one result per carried operand
        well_formed = well_formed && !op.region_args.empty() && op.operands.size() == 2 + op.region_args.size() && op.results.size() <= op.region_args.size() - 1;
      if (!well_formed) {
        err = "line " + std::to_string(op.line) + ": '" + op.name + "' is written with " + std::to_string(op.operands.size()) + " operands and " +
              std::to_string(op.results.size()) + " results; it needs " + (op.name == "scf.for" ? "bounds, a step and one operand per iter_arg" :
              "at least " + std::to_string(form->min_operands) + " operands") + (form->results >= 0 ? " and " + std::to_string(form->results) + " results" : "");
        return -2;
      }
    }
    ++n;
    if (!op.body.empty() && !in_reduce) {
      int inner = count_ops(op.body, op.name == "kapy.reduce", err);
      if (inner < 0) return inner;
      n += inner;
    }
  }
  return n;
}

}  // namespace
}  // namespace kapy

using namespace kapy;

extern "C" int kapy_parse_mlir(const char *mlir_text, const char *func_name, int32_t *n_args, int32_t *n_ops, int32_t *num_warps) {
  if (!mlir_text) return fail(KAPY_ERR_INVALID, "parse_mlir: null text");
  Parser ps;
  ps.t = tokenize(mlir_text);
  Func f;
  if (!ps.parse_module(f, func_name)) return fail(KAPY_ERR_INVALID, "parse_mlir: %s", ps.err.c_str());
  std::string err;
  int n = count_ops(f.body, false, err);
  if (n < 0) return fail(n == -2 ? KAPY_ERR_INVALID : KAPY_ERR_UNSUPPORTED, "parse_mlir: %s", err.c_str());
  if (n_args) *n_args = (int32_t)f.arg_names.size();
  if (n_ops) *n_ops = n;
  if (num_warps) *num_warps = f.num_warps;
  return KAPY_OK;
}

extern "C" int kapy_analyze_mlir(const char *mlir_text, const char *func_name, int64_t *smem_bytes, int32_t *n_buffers, int64_t *offsets,
                                 int32_t max_buffers, int32_t *n_barriers, int32_t *barrier_lines, int32_t max_barriers) {
  if (!mlir_text) return fail(KAPY_ERR_INVALID, "analyze_mlir: null text");
  Parser ps;
  ps.t = tokenize(mlir_text);
  Func f;
  if (!ps.parse_module(f, func_name)) return fail(KAPY_ERR_INVALID, "analyze_mlir: %s", ps.err.c_str());
  std::string err;
  if (int n = count_ops(f.body, false, err); n < 0) return fail(n == -2 ? KAPY_ERR_INVALID : KAPY_ERR_UNSUPPORTED, "analyze_mlir: %s", err.c_str());
  Analysis a;
  int rc = Analyzer(f, a).run(err);
  if (rc) return fail(rc, "analyze_mlir: %s", err.c_str());
  if (smem_bytes) *smem_bytes = a.total;
  if (n_buffers) *n_buffers = (int32_t)a.buffers.size();
  for (int k = 0; offsets && k < max_buffers && k < (int)a.buffers.size(); ++k) offsets[k] = a.buffers[k].offset;
  if (n_barriers) *n_barriers = (int32_t)a.barrier_lines.size();
  for (int k = 0; barrier_lines && k < max_barriers && k < (int)a.barrier_lines.size(); ++k) barrier_lines[k] = a.barrier_lines[k];
  return KAPY_OK;
}

static std::atomic<int64_t> g_merged_calls{0}, g_plans{0}, g_replays{0}, g_table_launches{0};
extern "C" int kapy_run_mlir_stats(int64_t *merged_stores) {
  if (merged_stores) *merged_stores = g_merged_calls.load();
  return KAPY_OK;
}
extern "C" int kapy_run_mlir_plan_stats(int64_t *plans, int64_t *replays, int64_t *table_launches) {
  if (plans) *plans = g_plans.load();
  if (replays) *replays = g_replays.load();
  if (table_launches) *table_launches = g_table_launches.load();
  return KAPY_OK;
}

// The plan cache: the device calls of a run that succeeded, kept under everything that decides them - the text, the function,
// the grid, the argument values, the device and the modes read from the environment.  A later call with the same key makes
// those calls again without parsing or interpreting anything (the register tensors they name live in the device's arena, which
// is kept for the life of the process and laid out the same way every time).
namespace {
// A step of a kept run: one of its calls as it was made, or a run of consecutive calls that differ only in where their
// operands lie (the same copy or matrix product of every instance and warp in flight) as ONE launch over a table of base
// addresses (batched.hip).  The tables of all steps of a run are one device allocation, written when the run is kept.
struct PlanStep {
  enum Kind { kCall, kCopyTable, kMatmulTable } kind = kCall;
  size_t first = 0, count = 1;   // the calls it stands for
  size_t rows = 0;               // rows of its table (calls that repeat another of the group word for word have none)
  CopyTableShape copy = {};
  bool vec16 = false;
  MatmulTableShape matmul = {};
  size_t table_at = 0;           // first word of its table
};
struct Plan {
  std::string key;
  std::vector<PlannedCall> calls;
  std::vector<PlanStep> steps;
  uint64_t *device_table = nullptr;
  int64_t merged = 0;
};

// The bytes a [rows x cols] walk over a view touches.  exact: rows of contiguous elements, no longer than the pitch - then two
// regions of one pitch are compared element by element (two column ranges of one buffer interleave without meeting);
// anything else by its bounding interval.
struct Region {
  uintptr_t lo = 0, hi = 0;
  int64_t pitch = 0, row_bytes = 0, rows = 0;
  bool exact = false;
};
bool region_of(const kapy_global &g, int64_t e0, int64_t e1, Region &out) {
  if (e0 <= 0 || e1 <= 0 || g.stride0 <= 0 || g.stride1 <= 0) return false;
  const int64_t b = dtype_bytes(g.dtype);
  out.lo = (uintptr_t)view_base(&g);
  out.hi = out.lo + (uintptr_t)(((e0 - 1) * g.stride0 + (e1 - 1) * g.stride1 + 1) * b);
  out.pitch = g.stride0 * b;
  out.row_bytes = e1 * b;
  out.rows = e0;
  out.exact = g.stride1 == 1 && out.row_bytes <= out.pitch;
  return true;
}
bool regions_overlap(const Region &x, const Region &y) {
  if (!(x.lo < y.hi && y.lo < x.hi)) return false;
  if (!(x.exact && y.exact && x.pitch == y.pitch)) return true;
  const Region &a = x.lo <= y.lo ? x : y, &b = x.lo <= y.lo ? y : x;
  // b starts q rows and t bytes into a's grid: its rows meet a's where their byte ranges do, in the same or the next row of a
  const int64_t delta = (int64_t)(b.lo - a.lo), q = delta / a.pitch, t = delta % a.pitch;
  return (t < a.row_bytes && q < a.rows) || (t + b.row_bytes > a.pitch && q + 1 < a.rows);
}
// What a call reads and writes.  known = false: a view this bookkeeping does not describe (the call then stays where it is
// and nothing moves across it).
struct Footprint {
  std::vector<Region> reads;
  Region write;
  bool known = false;
};
bool add_read(Footprint &fp, const kapy_global &g, int64_t e0, int64_t e1) {
  Region r;
  if (!region_of(g, e0, e1, r)) return false;
  fp.reads.push_back(r);
  return true;
}
Footprint footprint_of(const PlannedCall &c) {
  Footprint fp;
  switch (c.kind) {
    case PlannedCall::kCopy: {
      // (the source is read where the target's extent, or its own if smaller, reaches)
      const bool t = c.has_cfg && c.copy_cfg.transpose;
      const int64_t d0 = extent0(&c.g[1]), d1 = extent1(&c.g[1]);
      const int64_t r0 = std::min(extent0(&c.g[0]), t ? d1 : d0), r1 = std::min(extent1(&c.g[0]), t ? d0 : d1);
      fp.known = region_of(c.g[1], d0, d1, fp.write) && (r0 <= 0 || r1 <= 0 || add_read(fp, c.g[0], r0, r1));
      break;
    }
    case PlannedCall::kElementwise: {
      fp.known = region_of(c.g[0], extent0(&c.g[0]), extent1(&c.g[0]), fp.write);
      for (const kapy_global &in : c.ins) fp.known = fp.known && add_read(fp, in, extent0(&in), extent1(&in));
      break;
    }
    case PlannedCall::kReduce:
    case PlannedCall::kReduceEx:
      fp.known = region_of(c.g[1], extent0(&c.g[1]), extent1(&c.g[1]), fp.write) && add_read(fp, c.g[0], extent0(&c.g[0]), extent1(&c.g[0]));
      break;
    case PlannedCall::kMatmul:
      fp.known = region_of(c.g[3], extent0(&c.g[3]), extent1(&c.g[3]), fp.write) && add_read(fp, c.g[0], extent0(&c.g[0]), extent1(&c.g[0])) &&
                 add_read(fp, c.g[1], extent0(&c.g[1]), extent1(&c.g[1])) && (!c.has[2] || add_read(fp, c.g[2], extent0(&c.g[2]), extent1(&c.g[2])));
      break;
  }
  return fp;
}
// neither writes what the other reads or writes: the two may run in either order, or at once
bool independent(const Footprint &x, const Footprint &y) {
  if (regions_overlap(x.write, y.write)) return false;
  for (const Region &r : y.reads)
    if (regions_overlap(x.write, r)) return false;
  for (const Region &r : x.reads)
    if (regions_overlap(y.write, r)) return false;
  return true;
}

// Whether a call is of a kind the table kernels reproduce bit for bit, and its shape.
bool copy_for_table(const PlannedCall &c, CopyTableShape &sh) {
  if (c.kind != PlannedCall::kCopy || (c.has_cfg && c.copy_cfg.transpose)) return false;
  const kapy_global &src = c.g[0], &dst = c.g[1];
  const int64_t d0 = extent0(&dst), d1 = extent1(&dst);
  const int b = dtype_bytes(src.dtype);
  // (nothing to pad: the source view covers the target's extent)
  if (b != dtype_bytes(dst.dtype) || (b != 1 && b != 2 && b != 4) || d0 <= 0 || d1 <= 0 || extent0(&src) < d0 || extent1(&src) < d1 || d0 > INT32_MAX || d1 > INT32_MAX ||
      src.stride0 <= 0 || src.stride1 <= 0 || dst.stride0 <= 0 || dst.stride1 <= 0)
    return false;
  sh = {(int32_t)d0, (int32_t)d1, b, src.stride0, src.stride1, dst.stride0, dst.stride1};
  return true;
}
bool matmul_for_table(const PlannedCall &c, MatmulTableShape &sh) {
  if (c.kind != PlannedCall::kMatmul) return false;
  const kapy_global &a = c.g[0], &b = c.g[1], &acc = c.g[2], &d = c.g[3];
  if (c.has_cfg) {
    const kapy_matmul_cfg &m = c.matmul_cfg;
    if (m.accumulate != KAPY_ACCUMULATE_F32 || m.rmode != KAPY_RN || m.split_k > 1 || m.workspace || m.tile_m || m.tile_n || m.tile_k || m.stages || m.waves ||
        m.impl_way >= KAPY_MFMA_32X32X16_16B)
      return false;
  }
  const int64_t M = extent0(&a), K = extent1(&a), N = extent1(&b);
  // the shapes the library multiplies with its kernel for a row-major lhs and a row-major rhs, whose arithmetic
  // matmul_table_kernel repeats: 16-byte aligned contiguous rows on both, N and K multiples of 8; and small ones only
  if ((a.dtype != KAPY_F16 && a.dtype != KAPY_BF16) || b.dtype != a.dtype || a.stride1 != 1 || b.stride1 != 1 || a.stride0 <= 0 || b.stride0 <= 0 || extent0(&b) != K ||
      M <= 0 || N <= 0 || K <= 0 || N % 8 || K % 8 || M > 256 || N > 256 || K > 1024 || vector_bytes(&a, 1) != 16 || vector_bytes(&b, 1) != 16)
    return false;
  if ((d.dtype != KAPY_F16 && d.dtype != KAPY_BF16 && d.dtype != KAPY_F32) || extent0(&d) != M || extent1(&d) != N || d.stride0 <= 0 || d.stride1 <= 0) return false;
  if (c.has[2] && ((acc.dtype != KAPY_F16 && acc.dtype != KAPY_BF16 && acc.dtype != KAPY_F32) || extent0(&acc) != M || extent1(&acc) != N || acc.stride0 <= 0 || acc.stride1 <= 0))
    return false;
  sh = {(int32_t)M, (int32_t)N, (int32_t)K, a.dtype, c.has[2] ? acc.dtype : -1, d.dtype, a.stride0, b.stride0,
        c.has[2] ? acc.stride0 : 0, c.has[2] ? acc.stride1 : 0, d.stride0, d.stride1};
  return true;
}
bool same_shape(const CopyTableShape &x, const CopyTableShape &y) {
  return x.d0 == y.d0 && x.d1 == y.d1 && x.elem_bytes == y.elem_bytes && x.ss0 == y.ss0 && x.ss1 == y.ss1 && x.ds0 == y.ds0 && x.ds1 == y.ds1;
}
bool same_shape(const MatmulTableShape &x, const MatmulTableShape &y) {
  return x.M == y.M && x.N == y.N && x.K == y.K && x.ab_dtype == y.ab_dtype && x.acc_dtype == y.acc_dtype && x.d_dtype == y.d_dtype && x.a_sm == y.a_sm &&
         x.b_sk == y.b_sk && x.acc_sm == y.acc_sm && x.acc_sn == y.acc_sn && x.d_sm == y.d_sm && x.d_sn == y.d_sn;
}

// Groups the calls of a run into steps and writes the tables.  A group starts at a copy or product the table kernels take and
// collects, from the calls behind it (a window of them), those of the same kind and shape that are independent of every
// member so far and of every call passed over on the way - such a call may move up in front of those and run with the
// group; the calls passed over keep their order.  (The instances reach an op one after the other, and some ops make two
// calls per instance - a deferred value computed, then the product that reads it - so the calls that belong together are
// not always neighbours.)  A copy from the same place to the same place as a member, with nothing in between that touches
// either, is dropped: the warps of a program that fetch one tile into one shared buffer.
constexpr size_t kMaxTableRows = 16384, kPlanWindow = 8192, kMaxOptimisedCalls = 200000;
void plan_steps(Plan &plan) {
  bool tables = true;
  if (const char *e = getenv("KAPY_MLIR_PLAN_BATCH")) tables = atoi(e) != 0;
  const std::vector<PlannedCall> &calls = plan.calls;
  auto singles = [&]() {
    plan.steps.clear();
    for (size_t i = 0; i < calls.size(); ++i) {
      PlanStep st;
      st.first = i;
      plan.steps.push_back(st);
    }
  };
  if (!tables || calls.size() > kMaxOptimisedCalls) return singles();
  std::vector<Footprint> fps;
  fps.reserve(calls.size());
  for (const PlannedCall &c : calls) fps.push_back(footprint_of(c));
  std::vector<char> taken(calls.size(), 0);
  std::vector<uint64_t> words;
  std::vector<size_t> members, passed;
  for (size_t i = 0; i < calls.size(); ++i) {
    if (taken[i]) continue;
    PlanStep st;
    st.first = i;
    CopyTableShape cs = {};
    MatmulTableShape ms = {};
    const bool is_copy = fps[i].known && copy_for_table(calls[i], cs), is_matmul = fps[i].known && !is_copy && matmul_for_table(calls[i], ms);
    if (!is_copy && !is_matmul) {
      plan.steps.push_back(st);
      continue;
    }
    members.assign(1, i);
    passed.clear();
    size_t stood_for = 1;
    for (size_t j = i + 1; j < calls.size() && j - i < kPlanWindow && members.size() < kMaxTableRows; ++j) {
      if (taken[j]) continue;
      if (!fps[j].known) break;
      CopyTableShape cs2 = {};
      MatmulTableShape ms2 = {};
      bool joins = is_copy ? copy_for_table(calls[j], cs2) && same_shape(cs, cs2) : matmul_for_table(calls[j], ms2) && same_shape(ms, ms2);
      for (size_t k = 0; k < passed.size() && joins; ++k) joins = independent(fps[j], fps[passed[k]]);
      bool repeated = false;
      if (joins && is_copy)
        for (size_t m : members)
          if (fps[m].write.lo == fps[j].write.lo && fps[m].write.hi == fps[j].write.hi && fps[m].reads[0].lo == fps[j].reads[0].lo) repeated = true;
      for (size_t k = 0; k < members.size() && joins && !repeated; ++k) joins = independent(fps[j], fps[members[k]]);
      if (!joins) {
        passed.push_back(j);
        continue;
      }
      taken[j] = 1;
      ++stood_for;
      if (!repeated) members.push_back(j);
    }
    st.count = stood_for;
    st.rows = members.size();
    if (stood_for >= 2) {
      st.table_at = words.size();
      if (is_copy) {
        st.kind = PlanStep::kCopyTable;
        st.copy = cs;
        const int64_t b = cs.elem_bytes;
        bool vec = cs.ss1 == 1 && cs.ds1 == 1 && (cs.d1 * b) % 16 == 0 && (cs.ss0 * b) % 16 == 0 && (cs.ds0 * b) % 16 == 0;
        for (size_t m : members) {
          vec = vec && fps[m].reads[0].lo % 16 == 0 && fps[m].write.lo % 16 == 0;
          words.push_back((uint64_t)fps[m].reads[0].lo);
          words.push_back((uint64_t)fps[m].write.lo);
        }
        st.vec16 = vec;
      } else {
        st.kind = PlanStep::kMatmulTable;
        st.matmul = ms;
        for (size_t m : members) {
          words.push_back((uint64_t)fps[m].reads[0].lo);
          words.push_back((uint64_t)fps[m].reads[1].lo);
          words.push_back(fps[m].reads.size() > 2 ? (uint64_t)fps[m].reads[2].lo : 0);
          words.push_back((uint64_t)fps[m].write.lo);
        }
      }
    }
    plan.steps.push_back(st);
  }
  if (words.empty()) return;
  // (a run whose tables cannot be placed keeps its calls as they were made)
  if (hipMalloc((void **)&plan.device_table, words.size() * sizeof(uint64_t)) != hipSuccess ||
      hipMemcpy(plan.device_table, words.data(), words.size() * sizeof(uint64_t), hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipGetLastError();
    if (plan.device_table) (void)hipFree(plan.device_table);
    plan.device_table = nullptr;
    singles();
  }
}
void release_plan(Plan &plan) {
  if (plan.device_table) (void)hipFree(plan.device_table);
  plan.device_table = nullptr;
}
constexpr size_t kMaxPlans = 16, kMaxPlannedCalls = 1u << 20;
std::deque<std::shared_ptr<Plan>> g_plan_cache;  // (guarded by the arena's mutex: calls take turns anyway)

std::string plan_key(const char *text, const char *func, const kapy_mlir_arg *args, int32_t n_args, const int32_t grid[3], int device) {
  std::string k(text);
  k.push_back('\0');
  if (func) k += func;
  k.push_back('\0');
  k.append((const char *)grid, 3 * sizeof(int32_t));
  k.append((const char *)&device, sizeof device);
  for (int i = 0; i < n_args; ++i) {
    // (field by field: the padding of the struct is not part of the key)
    k.append((const char *)&args[i].ptr, sizeof args[i].ptr);
    k.append((const char *)&args[i].bytes, sizeof args[i].bytes);
    k.append((const char *)&args[i].i32, sizeof args[i].i32);
  }
  for (const char *name : {"KAPY_MLIR_FUSE", "KAPY_MLIR_IN_STEP", "KAPY_MLIR_BATCH", "KAPY_MLIR_MATMUL", "KAPY_MLIR_REDUCE", "KAPY_MLIR_PLAN_BATCH"}) {
    const char *v = getenv(name);
    k += v ? v : "";
    k.push_back('\0');
  }
  return k;
}

int replay_plan(const Plan &plan, hipStream_t stream) {
  std::vector<const kapy_global *> ins;
  for (const PlanStep &st : plan.steps) {
    int rc = KAPY_OK;
    if (st.kind == PlanStep::kCopyTable) {
      rc = copy_table_launch(plan.device_table + st.table_at, (int32_t)st.rows, st.copy, st.vec16, stream);
      if (rc != KAPY_OK) return rc;
      g_table_launches.fetch_add(1, std::memory_order_relaxed);
      continue;
    }
    if (st.kind == PlanStep::kMatmulTable) {
      rc = matmul_table_launch(plan.device_table + st.table_at, (int32_t)st.rows, st.matmul, stream);
      if (rc != KAPY_OK) return rc;
      g_table_launches.fetch_add(1, std::memory_order_relaxed);
      continue;
    }
    const PlannedCall &c = plan.calls[st.first];
    switch (c.kind) {
      case PlannedCall::kCopy: rc = kapy_copy(&c.g[0], &c.g[1], c.has_cfg ? &c.copy_cfg : nullptr, stream); break;
      case PlannedCall::kElementwise:
        ins.clear();
        for (const kapy_global &g : c.ins) ins.push_back(&g);
        rc = kapy_elementwise(c.prog.data(), (int32_t)c.prog.size(), ins.data(), (int32_t)ins.size(), &c.g[0], stream);
        break;
      case PlannedCall::kReduce: rc = kapy_reduce(&c.g[0], &c.g[1], c.axis, c.reduce_kind, stream); break;
      case PlannedCall::kReduceEx: rc = kapy_reduce_ex(&c.g[0], &c.g[1], c.axis, c.has_cfg ? &c.reduce_cfg : nullptr, stream); break;
      case PlannedCall::kMatmul: rc = kapy_matmul(&c.g[0], &c.g[1], c.has[2] ? &c.g[2] : nullptr, &c.g[3], c.has_cfg ? &c.matmul_cfg : nullptr, stream); break;
    }
    if (rc != KAPY_OK) return rc;
  }
  return KAPY_OK;
}
}  // namespace

extern "C" int kapy_run_mlir(const char *mlir_text, const char *func_name, const kapy_mlir_arg *args, int32_t n_args, const int32_t grid[3],
                             void *stream) {
  if (!mlir_text || (n_args > 0 && !args) || !grid) return fail(KAPY_ERR_INVALID, "run_mlir: null argument");
  // The arena is allocated at the first call on a device and kept (a call used to pay an allocation and a release of its own,
  // several milliseconds); calls take turns at it.
  static std::mutex arena_mutex;
  static char *arenas[16] = {};
  std::lock_guard<std::mutex> arena_lock(arena_mutex);
  // KAPY_MLIR_PLAN=0: every call parses and interprets the text again
  bool use_plans = true;
  if (const char *e = getenv("KAPY_MLIR_PLAN")) use_plans = atoi(e) != 0;
  if (use_plans && !g_plan_cache.empty()) {  // (a kept run means a device has been in use: nothing here is a call's first touch of it)
    int device = 0;
    KAPY_HIP_CHECK(hipGetDevice(&device));
    const std::string key = plan_key(mlir_text, func_name, args, n_args, grid, device);
    for (const std::shared_ptr<Plan> &plan : g_plan_cache)
      if (plan->key == key) {
        int rc = replay_plan(*plan, (hipStream_t)stream);
        g_merged_calls.fetch_add(plan->merged, std::memory_order_relaxed);
        g_replays.fetch_add(1, std::memory_order_relaxed);
        // the next call may use the arena once the work on the stream has finished
        hipError_t e = hipStreamSynchronize((hipStream_t)stream);
        if (rc != KAPY_OK) return rc;  // (the entry point that refused has left its message)
        if (e != hipSuccess) return fail(KAPY_ERR_HIP, "run_mlir: %s", hipGetErrorString(e));
        return KAPY_OK;
      }
  }
  Parser ps;
  ps.t = tokenize(mlir_text);
  Func f;
  if (!ps.parse_module(f, func_name)) return fail(KAPY_ERR_INVALID, "run_mlir: %s", ps.err.c_str());
  {
    std::string err;
    if (int n = count_ops(f.body, false, err); n < 0) return fail(n == -2 ? KAPY_ERR_INVALID : KAPY_ERR_UNSUPPORTED, "run_mlir: %s", err.c_str());
  }
  Analysis plan;
  {
    std::string err;
    int arc = Analyzer(f, plan).run(err);
    if (arc) return fail(arc, "run_mlir: %s", err.c_str());
    if (plan.total > kLdsBytes)
      return fail(KAPY_ERR_UNSUPPORTED, "run_mlir: the program needs %lld bytes of shared memory, a gfx950 workgroup has %lld", (long long)plan.total,
                  (long long)kLdsBytes);
  }
  if ((int)f.arg_names.size() != n_args)
    return fail(KAPY_ERR_INVALID, "run_mlir: @%s takes %d arguments, %d given", f.name.c_str(), (int)f.arg_names.size(), n_args);
  for (int k = 0; k < 3; ++k)
    if (grid[k] <= 0) return fail(KAPY_ERR_INVALID, "run_mlir: grid extents must be positive");
  int rc = ensure_device();
  if (rc) return rc;
  Interp in(f, (hipStream_t)stream);
  in.plan = &plan;
  if (const char *e = getenv("KAPY_MLIR_FUSE")) in.fuse = atoi(e) != 0;
  int device = 0;
  KAPY_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= 16) return fail(KAPY_ERR_UNSUPPORTED, "run_mlir: device ordinal %d beyond 16", device);
  if (!arenas[device]) KAPY_HIP_CHECK(hipMalloc((void **)&arenas[device], kArena));
  in.arena = arenas[device];
  std::vector<PlannedCall> recorded;
  if (use_plans) in.record = &recorded;
  rc = KAPY_OK;
  // KAPY_MLIR_IN_STEP=0: the warps of an instance run one after the other to the end instead of in step (the former way;
  // only right for programs whose warps do not exchange data through shared memory)
  bool in_step = true;
  if (const char *e = getenv("KAPY_MLIR_IN_STEP")) in_step = atoi(e) != 0;
  const int W = f.num_warps > 0 ? f.num_warps : 1;
  auto bind_args = [&](std::map<std::string, Value> &values) {
    for (int k = 0; k < n_args; ++k) {
      Value v;
      if (f.arg_types[k].kind == Type::kPtr) {
        if (!args[k].ptr) { in.err = "pointer argument " + std::to_string(k) + " is null"; return (int)KAPY_ERR_INVALID; }
        v.kind = Value::kPtr; v.ptr = args[k].ptr; v.bytes = args[k].bytes;
      }
      else { v.kind = Value::kInt; v.i = args[k].i32; }
      values[f.arg_names[k]] = v;
    }
    return (int)KAPY_OK;
  };
  // KAPY_MLIR_BATCH=0: one program instance at a time (its warps in step), no call merged over instances
  bool batch = true;
  if (const char *e = getenv("KAPY_MLIR_BATCH")) batch = atoi(e) != 0;
  in.merge = batch && in_step;
  const int64_t programs = (int64_t)grid[0] * grid[1] * grid[2];
  // programs per group: every warp of the group keeps at least kMinShare of the arena for its register tensors
  int64_t per_group = 1;
  if (batch && in_step) {
    per_group = std::max<int64_t>(1, (int64_t)((kArena - kMergedArena) / (kSharedArena + (size_t)W * kMinShare)));
    per_group = std::min(per_group, programs);
  }
  for (int64_t first = 0; first < programs && rc == KAPY_OK; first += per_group) {
    const int64_t count = std::min(per_group, programs - first);
    if (in_step) {
      // register tensors of the previous group are dead.  Layout of the arena: the shared parts of the group's programs, the
      // region of merged calls, then an equal share per warp.
      in.register_base = (size_t)count * kSharedArena;
      in.merged_base = in.merged_top = in.register_base;
      const size_t shares_at = in.merged_base + kMergedArena;
      const size_t share = ((kArena - shares_at) / (size_t)(count * W)) & ~size_t(255);
      in.warps.assign((size_t)(count * W), Interp::WarpState());
      for (int64_t g = 0; g < count && rc == KAPY_OK; ++g) {
        const int64_t id = first + g;
        for (int w = 0; w < W && rc == KAPY_OK; ++w) {
          Interp::WarpState &st = in.warps[(size_t)(g * W + w)];
          st.pid[0] = id % grid[0];
          st.pid[1] = id / grid[0] % grid[1];
          st.pid[2] = id / ((int64_t)grid[0] * grid[1]);
          st.warp = w;
          st.shared_base = (size_t)g * kSharedArena;
          st.top = shares_at + (size_t)(g * W + w) * share;
          st.limit = st.top + share;
          rc = bind_args(st.env);
        }
      }
      in.env.clear();
      if (rc == KAPY_OK) rc = in.run_ops_in_step(f.body, nullptr);
      continue;
    }
    in.pid[0] = first % grid[0];
    in.pid[1] = first / grid[0] % grid[1];
    in.pid[2] = first / ((int64_t)grid[0] * grid[1]);
    in.register_base = kSharedArena;
    in.shared_base = 0;
    for (int w = 0; w < W && rc == KAPY_OK; ++w) {
      in.warp = w;
      in.env.clear();
      in.top = kSharedArena;
      in.limit = kArena;
      rc = bind_args(in.env);
      if (rc == KAPY_OK) rc = in.run_ops(f.body, nullptr);
    }
  }
  g_merged_calls.fetch_add(in.merged_calls, std::memory_order_relaxed);
  // the next call may use the arena once the work on the stream has finished
  hipError_t e = hipStreamSynchronize((hipStream_t)stream);
  if (rc != KAPY_OK) return fail(rc, "run_mlir: %s", in.err.c_str());
  if (e != hipSuccess) return fail(KAPY_ERR_HIP, "run_mlir: %s", hipGetErrorString(e));
  if (use_plans && recorded.size() <= kMaxPlannedCalls) {
    auto plan = std::make_shared<Plan>();
    plan->key = plan_key(mlir_text, func_name, args, n_args, grid, device);
    plan->calls = std::move(recorded);
    plan->merged = in.merged_calls;
    plan_steps(*plan);
    if (g_plan_cache.size() >= kMaxPlans) {
      release_plan(*g_plan_cache.front());
      g_plan_cache.pop_front();
    }
    g_plan_cache.push_back(std::move(plan));
    g_plans.fetch_add(1, std::memory_order_relaxed);
  }
  return KAPY_OK;
}
