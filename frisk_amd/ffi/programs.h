// Recognisers for the two programs of the reference's design sketches that go beyond a lone GEMM:
//   @online_softmax  tmp/ir.mlir:21-75   per row, chunks through copy -> reduce max -> block exp2 -> reduce sum -> block
//                                        running log-sum; then a second sweep exp2(x * cst - lse)
//   @attention       tmp/ir.mlir:88-158  copy Q; for every key tile { copy K; gemm; reduce max; block rescale factor; block
//                                        exp2; reduce sum; block running sum; cast; block rescale acc; copy V; gemm };
//                                        block normalise; copy O
// written with the dialect's structure ops and frisk.block bodies of affine.load / arith / math / affine.store
// (FriskOps.td:143-190).  The sketches themselves are pseudo-code that no parser reads (free-form headers, `i` for `%i`,
// an undefined %8, a misspelt buffer, a second fill that would zero the scores, no division by the running sum); what is
// matched here is the same op sequence in the printed form of the ops, with the running maximum accumulating
// (clear = false) and the final division present.  A matched program is lowered to one library call
// (frisk_hip_softmax / frisk_hip_attention), which computes the same function with its own tiling.
//
// A block body is compared as an expression tree: the value each affine.store writes, built from loads, constants and
// arith / math ops (width casts are transparent), against a pattern such as
//     exp2(sub(mul($x[i], #c), mul($m[0], #c)))
// where $name binds a buffer, #name a constant, i / j are the block's induction variables and integers are constant
// indices; mul and add match in either operand order.
#pragma once
#include <cmath>
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "mini_ir.h"

namespace frisk_ir {

struct Expr {
  std::string op;  // "load", "const", or mul / add / sub / div / max / min / neg / exp2 / log2
  std::vector<Expr> kids;
  Value buffer;                  // load
  std::vector<AffineExpr> index;  // load: one expression per buffer dimension over the block's induction variables (dims)
  double value = 0.0;            // const
};

struct Bindings {
  std::map<std::string, Value> buffers;
  std::map<std::string, double> constants;
};

class BodyMatcher {
 public:
  explicit BodyMatcher(const char* what) : what_(what) {}
  [[noreturn]] void bad(const std::string& m) const { throw std::invalid_argument(std::string("not ") + what_ + ": " + m); }

  // expression tree of `v` inside a frisk.block with induction variables `ivs`
  Expr tree(Value v, const std::vector<Value>& ivs) const {
    Operation* d = v.impl ? v.impl->def : nullptr;
    if (!d) bad("a block body uses a value that no operation defines");
    const std::string& n = d->name;
    Expr e;
    if (n == "arith.constant") {
      const Attribute* a = d->attr("value");
      e.op = "const";
      e.value = a->kind == Attribute::Float ? a->f : (double)a->i;
      return e;
    }
    if (n == "arith.extf" || n == "arith.truncf") return tree(d->operands[0], ivs);
    if (n == "affine.load") {
      e.op = "load";
      e.buffer = d->operands[0];
      e.index = indices_over_ivs(d, 1, ivs);
      return e;
    }
    static const std::map<std::string, std::string> names = {{"arith.mulf", "mul"}, {"arith.addf", "add"}, {"arith.subf", "sub"}, {"arith.divf", "div"},
                                                              {"arith.maxnumf", "max"}, {"arith.minnumf", "min"}, {"arith.negf", "neg"},
                                                              {"math.exp2", "exp2"}, {"math.log2", "log2"}};
    auto it = names.find(n);
    if (it == names.end()) bad("operation " + n + " in a block body");
    e.op = it->second;
    for (const Value& o : d->operands) e.kids.push_back(tree(o, ivs));
    return e;
  }

  // index expressions of an affine.load / affine.store rewritten over the block's induction variables
  std::vector<AffineExpr> indices_over_ivs(const Operation* op, size_t first_index, const std::vector<Value>& ivs) const {
    const AffineMap& map = op->attr("map")->map;
    std::vector<AffineExpr> dims, syms;
    for (size_t i = first_index; i < op->operands.size(); ++i) {
      int pos = -1;
      for (size_t k = 0; k < ivs.size(); ++k) if (op->operands[i] == ivs[k]) pos = (int)k;
      if (pos < 0) bad("a block body indexes a buffer with something other than the block's induction variables");
      ((int)(i - first_index) < map.num_dims() ? dims : syms).push_back(AffineExpr::dim(pos));
    }
    std::vector<AffineExpr> out;
    for (int r = 0; r < map.num_results(); ++r) out.push_back(map.impl->results[(size_t)r].replace_dims_and_symbols(dims, syms));
    return out;
  }

  // the single store of a block: (buffer, index expressions, stored expression)
  struct Store { Value buffer; std::vector<AffineExpr> index; Expr value; };
  Store single_store(const Operation* block_op) const {
    Block* body = block_op->regions[0]->blocks[0];
    std::vector<Value> ivs;
    for (ValueImpl* a : body->args) ivs.push_back(Value{a});
    const Operation* store = nullptr;
    for (const Operation* op : body->ops)
      if (op->name == "affine.store") { if (store) bad("a block body with more than one store"); store = op; }
    if (!store) bad("a block body without a store");
    Store s;
    s.buffer = store->operands[1];
    s.index = indices_over_ivs(store, 2, ivs);
    s.value = tree(store->operands[0], ivs);
    return s;
  }

  // pattern matching; returns false without touching `b` on a mismatch
  bool match(const Expr& e, const std::string& pattern, Bindings& b) const {
    size_t p = 0;
    Bindings trial = b;
    if (!match_at(e, pattern, p, trial)) return false;
    skip(pattern, p);
    if (p != pattern.size()) return false;
    b = trial;
    return true;
  }
  // `target` like "$y[i]" or "$l[0]": the buffer and indices a store writes
  bool match_target(const Store& s, const std::string& target, Bindings& b) const {
    Expr as_load;
    as_load.op = "load";
    as_load.buffer = s.buffer;
    as_load.index = s.index;
    return match(as_load, target, b);
  }

 private:
  const char* what_;
  static void skip(const std::string& s, size_t& p) { while (p < s.size() && (s[p] == ' ' || s[p] == '\n')) ++p; }
  static std::string ident(const std::string& s, size_t& p) {
    size_t q = p;
    while (q < s.size() && (std::isalnum((unsigned char)s[q]) || s[q] == '_')) ++q;
    std::string w = s.substr(p, q - p);
    p = q;
    return w;
  }
  // end of the sub-pattern that starts at p (balanced parentheses / brackets up to a top-level ',' or ')')
  static size_t end_of(const std::string& s, size_t p) {
    int depth = 0;
    for (; p < s.size(); ++p) {
      if (s[p] == '(' || s[p] == '[') ++depth;
      else if (s[p] == ')' || s[p] == ']') { if (depth == 0) return p; --depth; }
      else if (s[p] == ',' && depth == 0) return p;
    }
    return p;
  }
  bool match_at(const Expr& e, const std::string& s, size_t& p, Bindings& b) const {
    skip(s, p);
    if (p >= s.size()) return false;
    if (s[p] == '#') {
      ++p;
      const std::string name = ident(s, p);
      if (e.op != "const") return false;
      auto it = b.constants.find(name);
      if (it == b.constants.end()) { b.constants[name] = e.value; return true; }
      return it->second == e.value || (std::isnan(it->second) && std::isnan(e.value));
    }
    if (s[p] == '$') {
      ++p;
      const std::string name = ident(s, p);
      if (e.op != "load") return false;
      auto it = b.buffers.find(name);
      if (it == b.buffers.end()) b.buffers[name] = e.buffer;
      else if (!(it->second == e.buffer)) return false;
      skip(s, p);
      if (p >= s.size() || s[p] != '[') return false;
      ++p;
      for (size_t k = 0;; ++k) {
        skip(s, p);
        const std::string w = ident(s, p);
        if (k >= e.index.size()) return false;
        AffineExpr want = w == "i" ? AffineExpr::dim(0) : w == "j" ? AffineExpr::dim(1) : AffineExpr::constant(std::atoll(w.c_str()));
        if (!e.index[k].equals(want)) return false;
        skip(s, p);
        if (p < s.size() && s[p] == ',') { ++p; continue; }
        if (p < s.size() && s[p] == ']') { ++p; return k + 1 == e.index.size(); }
        return false;
      }
    }
    const std::string name = ident(s, p);
    if (name.empty() || e.op != name) return false;
    skip(s, p);
    if (p >= s.size() || s[p] != '(') return false;
    ++p;
    // sub-pattern spans
    std::vector<std::pair<size_t, size_t>> spans;
    for (;;) {
      skip(s, p);
      const size_t q = end_of(s, p);
      spans.push_back({p, q});
      p = q;
      if (p < s.size() && s[p] == ',') { ++p; continue; }
      if (p < s.size() && s[p] == ')') { ++p; break; }
      return false;
    }
    if (spans.size() != e.kids.size()) return false;
    auto try_order = [&](const std::vector<size_t>& order, Bindings& out) {
      Bindings t = b;
      for (size_t k = 0; k < order.size(); ++k) {
        const std::string sub = s.substr(spans[k].first, spans[k].second - spans[k].first);
        size_t sp = 0;
        if (!match_at(e.kids[order[k]], sub, sp, t)) return false;
        skip(sub, sp);
        if (sp != sub.size()) return false;
      }
      out = t;
      return true;
    };
    Bindings got;
    if (try_order(e.kids.size() == 2 ? std::vector<size_t>{0, 1} : e.kids.size() == 1 ? std::vector<size_t>{0} : std::vector<size_t>{}, got)) { b = got; return true; }
    if (e.kids.size() == 2 && (name == "mul" || name == "add" || name == "max" || name == "min") && try_order({1, 0}, got)) { b = got; return true; }
    return false;
  }
};

// Window origin of one side of a frisk.copy as a linear function of named index values: origin[r] = sum_v coef[r][v] * var_v +
// c0[r].  Every index operand must be one of `vars`.
struct LinearOrigin {
  std::vector<std::vector<int64_t>> coef;  // [result][var]
  std::vector<int64_t> c0;
};
inline LinearOrigin linear_origin(const BodyMatcher& m, const Operation* cp, bool dst_side, const std::vector<Value>& vars) {
  const AffineMap& map = cp->attr(dst_side ? "dstMap" : "srcMap")->map;
  const int ns = cp->src_index_count, first = dst_side ? 2 + ns : 2;
  const int count = dst_side ? (int)cp->operands.size() - 2 - ns : ns;
  if (count != map.num_inputs()) m.bad("a copy's index operands do not match its index map");
  std::vector<int> which((size_t)count, -1);
  for (int i = 0; i < count; ++i) {
    for (size_t v = 0; v < vars.size(); ++v) if (cp->operands[(size_t)(first + i)] == vars[v]) which[(size_t)i] = (int)v;
    if (which[(size_t)i] < 0) m.bad("a copy is indexed by a value that is neither a grid index nor the enclosing loop's induction variable");
  }
  auto at = [&](const std::vector<int64_t>& val) {
    std::vector<int64_t> dims, syms;
    for (int i = 0; i < count; ++i) (i < map.num_dims() ? dims : syms).push_back(val[(size_t)which[(size_t)i]]);
    std::vector<int64_t> out;
    for (int r = 0; r < map.num_results(); ++r) out.push_back(map.impl->results[(size_t)r].eval(dims, syms));
    return out;
  };
  LinearOrigin o;
  std::vector<int64_t> zero(vars.size(), 0), probe(vars.size());
  o.c0 = at(zero);
  o.coef.assign(o.c0.size(), std::vector<int64_t>(vars.size(), 0));
  for (size_t v = 0; v < vars.size(); ++v) {
    std::vector<int64_t> unit = zero;
    unit[v] = 1;
    const std::vector<int64_t> r = at(unit);
    for (size_t k = 0; k < r.size(); ++k) o.coef[k][v] = r[k] - o.c0[k];
    probe[v] = (int64_t)(2 * v + 3);
  }
  const std::vector<int64_t> r = at(probe);
  for (size_t k = 0; k < r.size(); ++k) {
    int64_t want = o.c0[k];
    for (size_t v = 0; v < vars.size(); ++v) want += o.coef[k][v] * probe[v];
    if (r[k] != want) m.bad("a copy's index map is not linear in its indices");
  }
  return o;
}

inline bool is_zero_origin(const LinearOrigin& o) {
  for (size_t r = 0; r < o.c0.size(); ++r) {
    if (o.c0[r] != 0) return false;
    for (int64_t c : o.coef[r]) if (c != 0) return false;
  }
  return true;
}

// ------------------------------------------------------------------ helpers shared by the two recognisers
struct ProgramWalk {
  const BodyMatcher& m;
  Operation* kernel = nullptr;
  Operation* par = nullptr;
  Block* body = nullptr;
  std::string target = "gfx950";

  ProgramWalk(const BodyMatcher& matcher, Operation* k, Operation* module, size_t grid_rank) : m(matcher), kernel(k) {
    if (!kernel || kernel->name != "frisk.kernel") m.bad("expected a frisk.kernel");
    if (kernel->regions.empty() || kernel->regions[0]->blocks.empty()) m.bad("kernel has no entry block");
    for (const Operation* scope : {(const Operation*)kernel, (const Operation*)module})
      if (scope) if (auto t = scope->attr("frisk.target")) { target = t->s; break; }
    if (target.rfind("gfx950", 0) != 0) m.bad("frisk.target '" + target + "' is not gfx950");
    for (Operation* op : kernel->regions[0]->blocks[0]->ops) {
      if (op->name == "frisk.parallel") { if (par) m.bad("more than one frisk.parallel"); par = op; }
      else if (op->name != "frisk.end") m.bad("unexpected '" + op->name + "' at kernel level");
    }
    if (!par) m.bad("no frisk.parallel");
    if (par->attr("ranges")->ints.size() != grid_rank) m.bad("frisk.parallel must have a " + std::to_string(grid_rank) + "-D grid");
    if (par->regions[0]->blocks.empty()) m.bad("frisk.parallel has no body");
    body = par->regions[0]->blocks[0];
  }
  // the ops of a block without constants, allocations and the terminator (those may stand anywhere)
  static std::vector<Operation*> steps(Block* b) {
    std::vector<Operation*> out;
    for (Operation* op : b->ops)
      if (op->name != "arith.constant" && op->name != "frisk.alloc_buffer" && op->name != "frisk.end") out.push_back(op);
    return out;
  }
  int arg_index(Value v) const {
    Block* entry = kernel->regions[0]->blocks[0];
    return (v.impl && v.impl->block == entry) ? v.impl->index : -1;
  }
  void expect_op(Operation* op, const char* name, const char* role) const {
    if (!op || op->name != name) m.bad(std::string("expected ") + name + " (" + role + "), found " + (op ? op->name : std::string("the end of the block")));
  }
  void expect_fill(Operation* op, Value buffer, double value, const char* role) const {
    expect_op(op, "frisk.fill", role);
    if (!(op->operands[0] == buffer)) m.bad(std::string(role) + ": fills another buffer");
    const double v = op->attr("value")->f;
    if (!(v == value)) m.bad(std::string(role) + ": wrong fill value");
  }
  void expect_reduce(Operation* op, Value src, Value dst, const char* kind, int64_t dim, bool clear, const char* role) const {
    expect_op(op, "frisk.reduce", role);
    if (!(op->operands[0] == src) || !(op->operands[1] == dst)) m.bad(std::string(role) + ": reduces other buffers");
    std::string k = op->attr("kind")->s;
    if (k == "sum") k = "add";
    if (k != kind || op->int_attr("dim") != dim || op->attr("clear")->b != clear) m.bad(std::string(role) + ": wrong kind, dimension or clear flag");
  }
  static std::vector<int64_t> shape_of(Value v) { return v.type().impl->shape; }
  // a copy whose both sides are whole buffers at origin 0 (fragment <-> fragment, possibly converting)
  void expect_whole_copy(Operation* op, Value src, Value dst, const char* role) const {
    expect_op(op, "frisk.copy", role);
    if (!(op->operands[0] == src) || !(op->operands[1] == dst)) m.bad(std::string(role) + ": copies other buffers");
    if (!is_zero_origin(linear_origin(m, op, false, {})) || !is_zero_origin(linear_origin(m, op, true, {}))) m.bad(std::string(role) + ": must copy from and to origin 0");
    int64_t n = 1;
    for (int64_t d : shape_of(dst)) n *= d;
    int64_t ns = 1, nd = 1;
    for (int64_t d : op->attr("srcExtents")->ints) ns *= d;
    for (int64_t d : op->attr("dstExtents")->ints) nd *= d;
    int64_t nsrc = 1;
    for (int64_t d : shape_of(src)) nsrc *= d;
    if (ns != n || nd != n || nsrc != n) m.bad(std::string(role) + ": must copy the whole buffer");
  }
};

// ------------------------------------------------------------------ @online_softmax
struct SoftmaxProgram {
  std::string kernel_name;
  int arg_src = -1, arg_dst = -1;
  Type elem;
  int64_t rows = 0, cols = 0, chunk = 0;
  double cst = 0.0;  // the sketch's constant: y = 2^(cst x) / sum 2^(cst x)
  std::string target = "gfx950";
};

inline SoftmaxProgram match_online_softmax(Operation* kernel, Operation* module = nullptr) {
  BodyMatcher m("an online-softmax kernel");
  ProgramWalk w(m, kernel, module, 1);
  SoftmaxProgram g;
  g.kernel_name = kernel->attr("sym_name")->s;
  g.target = w.target;
  g.rows = w.par->attr("ranges")->ints[0];
  const Value bx{w.body->args[0]};
  std::vector<Operation*> top = ProgramWalk::steps(w.body);
  if (top.size() != 3) m.bad("the row program is fill(lse), a first sweep and a second sweep");
  Operation *fill = top[0], *sweep1 = top[1], *sweep2 = top[2];
  w.expect_op(fill, "frisk.fill", "the initial log-sum");
  w.expect_op(sweep1, "frisk.for", "the first sweep");
  w.expect_op(sweep2, "frisk.for", "the second sweep");
  const Value lse = fill->operands[0];
  w.expect_fill(fill, lse, -INFINITY, "the initial log-sum");

  auto trips_of = [&](Operation* loop, int64_t& lo, int64_t& step) {
    lo = loop->int_attr("lower");
    step = loop->int_attr("step");
    const int64_t hi = loop->int_attr("upper");
    if (step <= 0 || hi < lo) m.bad("a sweep must count upwards");
    return (hi - lo + step - 1) / step;
  };
  // global window of a sweep's copy: row bx, columns chunk t of the row in iteration t
  auto check_global = [&](Operation* cp, bool dst_side, Value global, Value iv, int64_t lo, int64_t step, const char* role) {
    const std::vector<int64_t> gs = ProgramWalk::shape_of(global);
    if (gs.size() != 2 || gs[0] != g.rows) m.bad(std::string(role) + ": the global buffer must be rows x columns with one row per grid index");
    const LinearOrigin o = linear_origin(m, cp, dst_side, {bx, iv});
    const std::vector<int64_t>& ext = cp->attr(dst_side ? "dstExtents" : "srcExtents")->ints;
    if (o.c0.size() != 2 || ext.size() != 2 || ext[0] != 1 || ext[1] != g.chunk) m.bad(std::string(role) + ": the window must be one chunk of one row");
    const bool ok = o.coef[0][0] == 1 && o.coef[0][1] == 0 && o.c0[0] == 0 && o.coef[1][0] == 0 && o.coef[1][1] * step == g.chunk && o.c0[1] + o.coef[1][1] * lo == 0;
    if (!ok) m.bad(std::string(role) + ": the window is not chunk t of row bx in iteration t");
    return gs[1];
  };
  auto check_fragment_side = [&](Operation* cp, bool dst_side, const char* role) {
    if (!is_zero_origin(linear_origin(m, cp, dst_side, {}))) m.bad(std::string(role) + ": the fragment side must start at 0");
  };

  // ---- first sweep: copy, reduce max, block exp2, reduce sum, block log-sum update
  int64_t lo1, st1;
  const int64_t trips1 = trips_of(sweep1, lo1, st1);
  Block* b1 = sweep1->regions[0]->blocks[0];
  const Value i1{b1->args[0]};
  std::vector<Operation*> s1 = ProgramWalk::steps(b1);
  if (s1.size() != 5) m.bad("the first sweep is copy, reduce max, block, reduce sum, block");
  w.expect_op(s1[0], "frisk.copy", "loading a chunk");
  const Value src = s1[0]->operands[0], x = s1[0]->operands[1];
  g.arg_src = w.arg_index(src);
  if (g.arg_src < 0) m.bad("the source must be a kernel argument");
  if (ProgramWalk::shape_of(x).size() != 1) m.bad("the chunk buffer must be rank-1");
  g.chunk = ProgramWalk::shape_of(x)[0];
  g.cols = check_global(s1[0], false, src, i1, lo1, st1, "loading a chunk");
  check_fragment_side(s1[0], true, "loading a chunk");
  if (trips1 * g.chunk != g.cols) m.bad("the first sweep does not cover the row");
  w.expect_op(s1[1], "frisk.reduce", "the chunk maximum");
  const Value max_x = s1[1]->operands[1];
  w.expect_reduce(s1[1], x, max_x, "max", 0, true, "the chunk maximum");
  w.expect_op(s1[2], "frisk.block", "the exponentials");
  Bindings bind;
  bind.buffers["x"] = x;
  bind.buffers["m"] = max_x;
  bind.buffers["l"] = lse;
  {
    const BodyMatcher::Store st = m.single_store(s1[2]);
    if (s1[2]->attr("ranges")->ints != std::vector<int64_t>{g.chunk}) m.bad("the exponentials must cover the chunk");
    if (!m.match(st.value, "exp2(sub(mul($x[i], #c), mul($m[0], #c)))", bind) || !m.match_target(st, "$e[i]", bind))
      m.bad("the first block is not exp_x[i] = exp2(x[i] * cst - max_x[0] * cst)");
  }
  w.expect_op(s1[3], "frisk.reduce", "the chunk sum");
  const Value sum = s1[3]->operands[1];
  w.expect_reduce(s1[3], bind.buffers["e"], sum, "add", 0, true, "the chunk sum");
  bind.buffers["s"] = sum;
  w.expect_op(s1[4], "frisk.block", "the log-sum update");
  {
    const BodyMatcher::Store st = m.single_store(s1[4]);
    if (s1[4]->attr("ranges")->ints != std::vector<int64_t>{1}) m.bad("the log-sum update is a single step");
    if (!m.match(st.value, "add(mul($m[0], #c), log2(add(exp2(sub($l[0], mul($m[0], #c))), $s[0])))", bind) || !m.match_target(st, "$l[0]", bind))
      m.bad("the second block is not lse = max_x * cst + log2(exp2(lse - max_x * cst) + sum_exp_x)");
  }
  // ---- second sweep: copy, block exp2(x * cst - lse), copy out
  int64_t lo2, st2;
  const int64_t trips2 = trips_of(sweep2, lo2, st2);
  Block* b2 = sweep2->regions[0]->blocks[0];
  const Value i2{b2->args[0]};
  std::vector<Operation*> s2 = ProgramWalk::steps(b2);
  if (s2.size() != 3) m.bad("the second sweep is copy, block, copy");
  w.expect_op(s2[0], "frisk.copy", "reloading a chunk");
  if (!(s2[0]->operands[0] == src)) m.bad("the second sweep must read the same source");
  const Value x2 = s2[0]->operands[1];
  if (ProgramWalk::shape_of(x2) != std::vector<int64_t>{g.chunk}) m.bad("the second sweep must use the same chunk length");
  check_global(s2[0], false, src, i2, lo2, st2, "reloading a chunk");
  check_fragment_side(s2[0], true, "reloading a chunk");
  if (trips2 * g.chunk != g.cols) m.bad("the second sweep does not cover the row");
  w.expect_op(s2[1], "frisk.block", "the probabilities");
  Bindings bind2;
  bind2.buffers["x"] = x2;
  bind2.buffers["l"] = lse;
  bind2.constants = bind.constants;
  {
    const BodyMatcher::Store st = m.single_store(s2[1]);
    if (s2[1]->attr("ranges")->ints != std::vector<int64_t>{g.chunk}) m.bad("the probabilities must cover the chunk");
    if (!m.match(st.value, "exp2(sub(mul($x[i], #c), $l[0]))", bind2) || !m.match_target(st, "$y[i]", bind2))
      m.bad("the block of the second sweep is not y[i] = exp2(x[i] * cst - lse)");
  }
  w.expect_op(s2[2], "frisk.copy", "storing a chunk");
  if (!(s2[2]->operands[0] == bind2.buffers["y"])) m.bad("the second sweep must store the probabilities it computed");
  const Value dst = s2[2]->operands[1];
  g.arg_dst = w.arg_index(dst);
  if (g.arg_dst < 0) m.bad("the destination must be a kernel argument");
  check_fragment_side(s2[2], false, "storing a chunk");
  if (check_global(s2[2], true, dst, i2, lo2, st2, "storing a chunk") != g.cols) m.bad("source and destination rows differ in length");
  g.elem = src.type().element();
  if (!g.elem.equals(dst.type().element())) m.bad("source and destination element types differ");
  g.cst = bind.constants["c"];
  if (!std::isfinite(g.cst)) m.bad("the constant must be finite");
  return g;
}

// ------------------------------------------------------------------ @attention
struct AttentionProgram {
  std::string kernel_name;
  int arg_q = -1, arg_k = -1, arg_v = -1, arg_o = -1;
  Type elem;
  int64_t batch = 0, heads = 0, seq_q = 0, seq_k = 0, head_dim = 0;
  int64_t tile_q = 0, tile_k = 0;  // the program's own tiling
  bool k_transposed = false;       // K stored [batch, heads, head_dim, seq_k]
  double cst = 0.0;                // scores are multiplied by cst before exp2: cst = softmax scale * log2(e)
  std::string target = "gfx950";
};

inline AttentionProgram match_attention(Operation* kernel, Operation* module = nullptr) {
  BodyMatcher m("a fused-attention kernel");
  ProgramWalk w(m, kernel, module, 3);
  AttentionProgram g;
  g.kernel_name = kernel->attr("sym_name")->s;
  g.target = w.target;
  const auto& grid = w.par->attr("ranges")->ints;
  g.batch = grid[0];
  g.heads = grid[1];
  const Value bz{w.body->args[0]}, by{w.body->args[1]}, bx{w.body->args[2]};
  std::vector<Operation*> top = ProgramWalk::steps(w.body);
  // copy Q; fill acc_o 0; fill logsum 0; fill scores_max -inf (in any order); for; block normalise; copy acc_o -> o; copy o -> O
  if (top.size() != 8) m.bad("the program is copy Q, three fills, the key loop, the normalisation, two copies out");
  w.expect_op(top[0], "frisk.copy", "loading the query tile");
  Operation* loop = top[4];
  w.expect_op(loop, "frisk.for", "the key loop");
  Block* lb = loop->regions[0]->blocks[0];
  const Value kv{lb->args[0]};
  std::vector<Operation*> s = ProgramWalk::steps(lb);
  if (s.size() != 13) m.bad("the key loop is copy K, fill, gemm, copy max, reduce max, block, block, reduce sum, block, copy, block, copy V, gemm");

  // ---- the two products name most of the buffers
  Operation *gemm1 = s[2], *gemm2 = s[12];
  w.expect_op(gemm1, "frisk.gemm", "the scores");
  w.expect_op(gemm2, "frisk.gemm", "the weighted sum of V");
  const Value q = gemm1->operands[0], k = gemm1->operands[1], acc_s = gemm1->operands[2];
  const Value p16 = gemm2->operands[0], v = gemm2->operands[1], acc_o = gemm2->operands[2];
  if (gemm1->bool_attr("clear_accum") || gemm2->bool_attr("clear_accum")) m.bad("the products accumulate into buffers that fills clear");
  const std::vector<int64_t> qs = ProgramWalk::shape_of(q), ks = ProgramWalk::shape_of(k), vs = ProgramWalk::shape_of(v);
  if (qs.size() != 2 || ks.size() != 2 || vs.size() != 2) m.bad("tiles must be rank-2");
  g.tile_q = qs[0];
  g.head_dim = qs[1];
  // K tile: [head_dim][keys] (the sketch's layout), or [keys][head_dim] with transB set on the product
  const bool tb = gemm1->bool_attr("transB") && !(ks[0] == g.head_dim && ks[1] != g.head_dim);
  g.k_transposed = !tb;
  g.tile_k = tb ? ks[0] : ks[1];
  if ((tb ? ks[1] : ks[0]) != g.head_dim) m.bad("the K tile does not match the head dimension");
  if (vs != std::vector<int64_t>{g.tile_k, g.head_dim}) m.bad("the V tile must be keys x head_dim");
  if (ProgramWalk::shape_of(acc_s) != std::vector<int64_t>{g.tile_q, g.tile_k} || ProgramWalk::shape_of(acc_o) != std::vector<int64_t>{g.tile_q, g.head_dim})
    m.bad("accumulator shapes do not match the tiles");
  if (gemm1->bool_attr("transA") || gemm2->bool_attr("transA") || gemm2->bool_attr("transB")) m.bad("unexpected transpose flag");

  // ---- before the loop
  const Value gq = top[0]->operands[0];
  if (!(top[0]->operands[1] == q)) m.bad("the first copy must load the query tile the product reads");
  g.arg_q = w.arg_index(gq);
  if (g.arg_q < 0) m.bad("Q must be a kernel argument");
  const std::vector<int64_t> gqs = ProgramWalk::shape_of(gq);
  if (gqs.size() != 4 || gqs[0] != g.batch || gqs[1] != g.heads || gqs[3] != g.head_dim) m.bad("Q must be [batch, heads, seq_q, head_dim] matching the grid");
  g.seq_q = gqs[2];
  if (grid[2] * g.tile_q != g.seq_q) m.bad("the grid does not cover the queries");
  auto check_4d = [&](Operation* cp, bool dst_side, Value global, int seq_axis, Value seq_var, int64_t seq_step, int64_t seq_lo, int64_t rows, int64_t cols, const char* role) {
    // window [1, 1, rows, cols] at (bz, by, ., .): axis seq_axis advances by one tile per unit of seq_var, the other starts at 0
    const LinearOrigin o = linear_origin(m, cp, dst_side, {bz, by, bx, kv});
    const std::vector<int64_t>& ext = cp->attr(dst_side ? "dstExtents" : "srcExtents")->ints;
    if (o.c0.size() != 4 || ext != std::vector<int64_t>{1, 1, rows, cols}) m.bad(std::string(role) + ": the window must be one tile of one head");
    const int var = seq_var == bx ? 2 : 3;
    for (int r = 0; r < 4; ++r)
      for (int vv = 0; vv < 4; ++vv) {
        int64_t want = 0;
        if (r == 0 && vv == 0) want = 1;
        if (r == 1 && vv == 1) want = 1;
        if (r == seq_axis && vv == var) continue;  // checked below
        if (o.coef[(size_t)r][(size_t)vv] != want) m.bad(std::string(role) + ": the window is not the tile of (batch, head) the grid names");
      }
    const int64_t tile = seq_axis == 2 ? rows : cols;
    if (o.coef[(size_t)seq_axis][(size_t)var] * seq_step != tile || o.c0[(size_t)seq_axis] + o.coef[(size_t)seq_axis][(size_t)var] * seq_lo != 0)
      m.bad(std::string(role) + ": the window does not advance one tile per step");
    for (int r = 0; r < 4; ++r) if (r != seq_axis && o.c0[(size_t)r] != 0) m.bad(std::string(role) + ": the window has an offset");
    (void)global;
  };
  check_4d(top[0], false, gq, 2, bx, 1, 0, g.tile_q, g.head_dim, "loading the query tile");
  if (!is_zero_origin(linear_origin(m, top[0], true, {}))) m.bad("loading the query tile: the shared side must start at 0");

  // the three fills
  Value logsum, scores_max;
  {
    bool seen_o = false;
    for (int t = 1; t <= 3; ++t) {
      w.expect_op(top[(size_t)t], "frisk.fill", "clearing the running state");
      const Value b = top[(size_t)t]->operands[0];
      const double val = top[(size_t)t]->attr("value")->f;
      if (b == acc_o) { if (val != 0.0) m.bad("the output accumulator must start at 0"); seen_o = true; }
      else if (val == 0.0) logsum = b;
      else if (std::isinf(val) && val < 0) scores_max = b;
      else m.bad("unexpected fill before the key loop");
    }
    if (!seen_o || !logsum || !scores_max) m.bad("the running state is acc_o = 0, logsum = 0, scores_max = -inf");
  }

  // ---- the key loop
  const int64_t lo = loop->int_attr("lower"), hi = loop->int_attr("upper"), step = loop->int_attr("step");
  if (step <= 0 || hi < lo) m.bad("the key loop must count upwards");
  const int64_t trips = (hi - lo + step - 1) / step;
  g.seq_k = trips * g.tile_k;
  w.expect_op(s[0], "frisk.copy", "loading the key tile");
  const Value gk = s[0]->operands[0];
  if (!(s[0]->operands[1] == k)) m.bad("the key copy must fill the tile the product reads");
  g.arg_k = w.arg_index(gk);
  if (g.arg_k < 0) m.bad("K must be a kernel argument");
  const std::vector<int64_t> gks = ProgramWalk::shape_of(gk);
  if (gks.size() != 4 || gks[0] != g.batch || gks[1] != g.heads) m.bad("K must be rank-4 over (batch, heads)");
  if (g.k_transposed) {
    if (gks[2] != g.head_dim || gks[3] != g.seq_k) m.bad("K must be [batch, heads, head_dim, seq_k] covered by the key loop");
    check_4d(s[0], false, gk, 3, kv, step, lo, g.head_dim, g.tile_k, "loading the key tile");
  } else {
    if (gks[2] != g.seq_k || gks[3] != g.head_dim) m.bad("K must be [batch, heads, seq_k, head_dim] covered by the key loop");
    check_4d(s[0], false, gk, 2, kv, step, lo, g.tile_k, g.head_dim, "loading the key tile");
  }
  w.expect_fill(s[1], acc_s, 0.0, "clearing the scores");
  Value max_prev;
  w.expect_op(s[3], "frisk.copy", "keeping the previous maximum");
  max_prev = s[3]->operands[1];
  w.expect_whole_copy(s[3], scores_max, max_prev, "keeping the previous maximum");
  w.expect_reduce(s[4], acc_s, scores_max, "max", 1, false, "the running maximum");
  Bindings bind;
  bind.buffers["s"] = acc_s;
  bind.buffers["m"] = scores_max;
  bind.buffers["p"] = max_prev;
  bind.buffers["l"] = logsum;
  bind.buffers["o"] = acc_o;
  auto ranges_are = [&](Operation* op, std::vector<int64_t> r) { return op->attr("ranges")->ints == r; };
  {
    w.expect_op(s[5], "frisk.block", "the rescale factor");
    const BodyMatcher::Store st = m.single_store(s[5]);
    if (!ranges_are(s[5], {g.tile_q}) || !m.match(st.value, "exp2(sub(mul($p[i], #c), mul($m[i], #c)))", bind) || !m.match_target(st, "$f[i]", bind))
      m.bad("the first block is not scores_scale[i] = exp2(scores_max_prev[i] * cst - scores_max[i] * cst)");
  }
  {
    w.expect_op(s[6], "frisk.block", "the exponentials");
    const BodyMatcher::Store st = m.single_store(s[6]);
    if (!ranges_are(s[6], {g.tile_q, g.tile_k}) || !m.match(st.value, "exp2(sub(mul($s[i, j], #c), mul($m[i], #c)))", bind) || !m.match_target(st, "$s[i, j]", bind))
      m.bad("the second block is not acc_s[i, j] = exp2(acc_s[i, j] * cst - scores_max[i] * cst)");
  }
  w.expect_op(s[7], "frisk.reduce", "the row sums");
  const Value row_sum = s[7]->operands[1];
  w.expect_reduce(s[7], acc_s, row_sum, "add", 1, true, "the row sums");
  bind.buffers["r"] = row_sum;
  {
    w.expect_op(s[8], "frisk.block", "the running sum");
    const BodyMatcher::Store st = m.single_store(s[8]);
    if (!ranges_are(s[8], {g.tile_q}) || !m.match(st.value, "add(mul($l[i], $f[i]), $r[i])", bind) || !m.match_target(st, "$l[i]", bind))
      m.bad("the third block is not logsum[i] = logsum[i] * scores_scale[i] + scores_sum[i]");
  }
  w.expect_whole_copy(s[9], acc_s, p16, "rounding the probabilities");
  {
    w.expect_op(s[10], "frisk.block", "rescaling the output accumulator");
    const BodyMatcher::Store st = m.single_store(s[10]);
    if (!ranges_are(s[10], {g.tile_q, g.head_dim}) || !m.match(st.value, "mul($o[i, j], $f[i])", bind) || !m.match_target(st, "$o[i, j]", bind))
      m.bad("the fourth block is not acc_o[i, j] = acc_o[i, j] * scores_scale[i]");
  }
  w.expect_op(s[11], "frisk.copy", "loading the value tile");
  const Value gv = s[11]->operands[0];
  if (!(s[11]->operands[1] == v)) m.bad("the value copy must fill the tile the product reads");
  g.arg_v = w.arg_index(gv);
  if (g.arg_v < 0) m.bad("V must be a kernel argument");
  if (ProgramWalk::shape_of(gv) != std::vector<int64_t>{g.batch, g.heads, g.seq_k, g.head_dim}) m.bad("V must be [batch, heads, seq_k, head_dim]");
  check_4d(s[11], false, gv, 2, kv, step, lo, g.tile_k, g.head_dim, "loading the value tile");

  // ---- after the loop: normalise, round, store
  {
    w.expect_op(top[5], "frisk.block", "the normalisation");
    const BodyMatcher::Store st = m.single_store(top[5]);
    if (!ranges_are(top[5], {g.tile_q, g.head_dim}) || !m.match(st.value, "div($o[i, j], $l[i])", bind) || !m.match_target(st, "$o[i, j]", bind))
      m.bad("the block after the key loop is not acc_o[i, j] = acc_o[i, j] / logsum[i] (without it the result is not a softmax)");
  }
  w.expect_op(top[6], "frisk.copy", "rounding the output");
  const Value o16 = top[6]->operands[1];
  w.expect_whole_copy(top[6], acc_o, o16, "rounding the output");
  w.expect_op(top[7], "frisk.copy", "storing the output tile");
  if (!(top[7]->operands[0] == o16)) m.bad("the last copy must store the rounded output");
  const Value go = top[7]->operands[1];
  g.arg_o = w.arg_index(go);
  if (g.arg_o < 0) m.bad("O must be a kernel argument");
  if (ProgramWalk::shape_of(go) != gqs) m.bad("O must have the shape of Q");
  g.cst = bind.constants["c"];
  if (!std::isfinite(g.cst)) m.bad("the constant must be finite");
  g.elem = gq.type().element();
  for (Value t : {gk, gv, go}) if (!g.elem.equals(t.type().element())) m.bad("Q, K, V and O must have one element type");
  check_4d(top[7], true, go, 2, bx, 1, 0, g.tile_q, g.head_dim, "storing the output tile");
  if (!is_zero_origin(linear_origin(m, top[7], false, {}))) m.bad("storing the output tile: the shared side must start at 0");
  return g;
}

// ------------------------------------------------------------------ free-standing frisk.block bodies
// A kernel whose entry block holds nothing but frisk.block ops (and the constants they use): every block runs its body
// for each point of a rank-1 or rank-2 iteration space, the body loads from kernel arguments, computes with arith / math
// ops and stores one value per point (FriskOps.td:143-190).  Each block becomes one postfix program for
// frisk_hip_elementwise; blocks run in program order.
// A load or store index must be linear in the block's induction variables.  With (row, col) = (0, i) for a rank-1 block
// and (i, j) for a rank-2 one, an access is  offset + row * row_stride + col * col_stride  elements into its argument;
// loads may broadcast (col stride 0, row stride 0), the store must walk its row (col stride 1) and give every point an
// element of its own.
struct EwOperand {
  int arg = -1;
  Type elem;
  int64_t offset = 0, row_stride = 0, col_stride = 0;
  bool operator==(const EwOperand& o) const { return arg == o.arg && offset == o.offset && row_stride == o.row_stride && col_stride == o.col_stride; }
};
struct EwStep { std::string op; int operand = -1; double value = 0.0; };  // op: input | const | add sub mul div max min neg exp2 log2
struct EwBlock {
  int64_t rows = 1, cols = 1;
  EwOperand out;
  std::vector<EwOperand> inputs;
  std::vector<EwStep> steps;
  int max_stack = 0;
};
struct EwProgram {
  std::string kernel_name, target;
  std::vector<EwBlock> blocks;
};

inline bool is_elementwise_kernel(Operation* kernel) {
  if (!kernel || kernel->name != "frisk.kernel" || kernel->regions.empty() || kernel->regions[0]->blocks.empty()) return false;
  bool any = false;
  for (Operation* op : kernel->regions[0]->blocks[0]->ops) {
    if (op->name == "frisk.block") any = true;
    else if (op->name != "arith.constant" && op->name != "frisk.end") return false;
  }
  return any;
}

inline EwProgram match_elementwise(Operation* kernel, Operation* module = nullptr) {
  const BodyMatcher m("an elementwise kernel");
  if (!kernel || kernel->name != "frisk.kernel") m.bad("expected a frisk.kernel");
  if (kernel->regions.empty() || kernel->regions[0]->blocks.empty()) m.bad("kernel has no entry block");
  EwProgram g;
  g.kernel_name = kernel->attr("sym_name") ? kernel->attr("sym_name")->s : std::string();
  g.target = "gfx950";
  for (const Operation* scope : {(const Operation*)kernel, (const Operation*)module})
    if (scope) if (auto t = scope->attr("frisk.target")) { g.target = t->s; break; }
  if (g.target.rfind("gfx950", 0) != 0) m.bad("frisk.target '" + g.target + "' is not gfx950");
  for (Operation* op : kernel->regions[0]->blocks[0]->ops) {
    if (op->name == "arith.constant" || op->name == "frisk.end") continue;
    if (op->name != "frisk.block") m.bad("operation " + op->name + " beside the blocks");
    const auto& ranges = op->attr("ranges")->ints;
    if (ranges.empty() || ranges.size() > 2) m.bad("a block of rank " + std::to_string(ranges.size()) + " (1 or 2 supported)");
    EwBlock b;
    b.rows = ranges.size() == 2 ? ranges[0] : 1;
    b.cols = ranges.back();
    const BodyMatcher::Store st = m.single_store(op);
    // an access as offset + row * rs + col * cs, from the index expressions over the induction variables
    auto operand_of = [&](Value buffer, const std::vector<AffineExpr>& index, const char* what) {
      EwOperand o;
      o.arg = kernel_arg_index(kernel, buffer);
      if (o.arg < 0 || !buffer.type().is_memref()) m.bad(std::string(what) + " is not a kernel argument memref");
      const auto& sh = buffer.type().impl->shape;
      if (sh.empty() || sh.size() > 2) m.bad(std::string(what) + " must have rank 1 or 2");
      for (int64_t d : sh) if (d < 0) m.bad(std::string(what) + " has a dynamic extent");
      if (index.size() != sh.size()) m.bad(std::string(what) + " is indexed with " + std::to_string(index.size()) + " expressions for rank " + std::to_string(sh.size()));
      o.elem = buffer.type().element();
      const size_t nv = ranges.size();
      auto at = [&](int64_t i, int64_t j) {  // element offset at induction values (i, j)
        std::vector<int64_t> dims = nv == 2 ? std::vector<int64_t>{i, j} : std::vector<int64_t>{i};
        int64_t off = 0;
        for (size_t d = 0; d < sh.size(); ++d) {
          const int64_t v = index[d].eval(dims, {});
          off = off * sh[d] + v;
        }
        return off;
      };
      const int64_t c0 = at(0, 0), ci = at(1, 0) - c0, cj = nv == 2 ? at(0, 1) - c0 : 0;
      if (at(3, nv == 2 ? 5 : 0) != c0 + 3 * ci + (nv == 2 ? 5 * cj : 0)) m.bad(std::string(what) + " is not indexed linearly by the block's induction variables");
      o.offset = c0;
      o.row_stride = nv == 2 ? ci : 0;
      o.col_stride = nv == 2 ? cj : ci;
      // every point inside the memref: the corners of the iteration space bound a linear access
      int64_t total = 1;
      for (int64_t d : sh) total *= d;
      for (size_t d = 0; d < sh.size(); ++d)
        for (int64_t i : {int64_t(0), ranges[0] - 1})
          for (int64_t j : {int64_t(0), nv == 2 ? ranges[1] - 1 : int64_t(0)}) {
            std::vector<int64_t> dims = nv == 2 ? std::vector<int64_t>{i, j} : std::vector<int64_t>{i};
            const int64_t v = index[d].eval(dims, {});
            if (v < 0 || v >= sh[d]) m.bad(std::string(what) + " is indexed outside its extents");
          }
      (void)total;
      if (o.row_stride < 0 || o.col_stride < 0) m.bad(std::string(what) + " is walked backwards");
      return o;
    };
    b.out = operand_of(st.buffer, st.index, "the stored buffer");
    if (b.out.col_stride != 1) m.bad("the store must walk a row of its buffer (column stride " + std::to_string(b.out.col_stride) + ")");
    if (b.rows > 1 && b.out.row_stride < b.cols) m.bad("the stores of different rows overlap");
    // postfix program of the stored expression; the operand pushed first is the left one
    int depth = 0;
    std::function<void(const Expr&)> emit = [&](const Expr& e) {
      if (e.op == "load") {
        const EwOperand o = operand_of(e.buffer, e.index, "a loaded buffer");
        if (o.col_stride > 1) m.bad("a load with column stride " + std::to_string(o.col_stride) + " (0 or 1 supported)");
        size_t k = 0;
        while (k < b.inputs.size() && !(b.inputs[k] == o)) ++k;
        if (k == b.inputs.size()) b.inputs.push_back(o);
        b.steps.push_back(EwStep{"input", (int)k, 0.0});
        b.max_stack = std::max(b.max_stack, ++depth);
        return;
      }
      if (e.op == "const") {
        b.steps.push_back(EwStep{"const", -1, e.value});
        b.max_stack = std::max(b.max_stack, ++depth);
        return;
      }
      for (const Expr& k : e.kids) emit(k);
      b.steps.push_back(EwStep{e.op, -1, 0.0});
      depth -= (int)e.kids.size() - 1;
    };
    emit(st.value);
    // an in-place block may only read the element it writes
    for (const EwOperand& o : b.inputs)
      if (o.arg == b.out.arg && !(o == b.out)) m.bad("a block reads its own output buffer at other elements than the one it writes");
    g.blocks.push_back(b);
  }
  if (g.blocks.empty()) m.bad("the kernel holds no frisk.block");
  return g;
}

}  // namespace frisk_ir
