// Text -> IR: reads back the textual form the printer of mini_ir.h writes, i.e. the form the reference's custom
// printers give its ops (lib/Dialect/Frisk/IR/FriskOps.cpp:953-973 kernel, :1023-1038 parallel, :1147-1162 block,
// :1250-1259 for, :1519-1545 alloc_buffer, :1642-1665 copy; assembly formats of fill / reduce / gemm / end,
// include/Dialect/Frisk/IR/FriskOps.td:244,288,409,442), so that a saved module such as tmp/log_11_18 can be loaded,
// verified, planned and launched.  It takes the place of the reference's custom parsers (:922-951, :991-1021,
// :1118-1145, :1220-1248, :1483-1516, :1593-1640).  Those do not read what their own printers write in three places
// (frisk.for wants `step =` and a parenthesised argument list the printer never emits; frisk.copy wants the types
// before the attribute dictionary; frisk.alloc_buffer wants a generic attribute dictionary where the printer writes
// `scope = "..."`): the printed form is the one that exists in the reference's saved outputs, and it is the grammar here.
// `frisk.for ... step = N` is accepted whether or not the step is 1.
#pragma once
#include <cctype>
#include <cstdlib>

#include "mini_ir.h"

namespace frisk_ir {

struct ParseError : std::invalid_argument {
  explicit ParseError(const std::string& m) : std::invalid_argument(m) {}
};

class IrParser {
 public:
  IrParser(Context& ctx, const std::string& text) : ctx_(ctx), s_(text) {}

  // `module [attributes {...}] { kernels }`; a bare list of kernels is wrapped in a module, as MLIR does
  Operation* parse_module() {
    Operation* mod = ctx_.new_op("builtin.module");
    Region* rg = ctx_.new_region(mod);
    Block* body = ctx_.new_block();
    body->parent = rg;
    rg->blocks.push_back(body);
    skip();
    if (try_word("module")) {
      if (try_word("attributes")) parse_attr_dict(mod);
      expect("{");
      while (!try_tok("}")) parse_top_level(body);
    } else {
      while (!at_end()) parse_top_level(body);
    }
    skip();
    if (!at_end()) fail("unexpected text after the module");
    return mod;
  }

 private:
  Context& ctx_;
  const std::string& s_;
  size_t p_ = 0;
  std::vector<std::map<std::string, ValueImpl*>> scopes_;

  // ------------------------------------------------------------ lexing
  [[noreturn]] void fail(const std::string& msg) const {
    size_t line = 1, col = 1;
    for (size_t i = 0; i < p_ && i < s_.size(); ++i) { if (s_[i] == '\n') { ++line; col = 1; } else ++col; }
    throw ParseError("line " + std::to_string(line) + ", column " + std::to_string(col) + ": " + msg);
  }
  bool at_end() { skip(); return p_ >= s_.size(); }
  void skip() {
    for (;;) {
      while (p_ < s_.size() && std::isspace((unsigned char)s_[p_])) ++p_;
      if (p_ + 1 < s_.size() && s_[p_] == '/' && s_[p_ + 1] == '/') { while (p_ < s_.size() && s_[p_] != '\n') ++p_; continue; }
      return;
    }
  }
  bool peek_tok(const std::string& t) { skip(); return s_.compare(p_, t.size(), t) == 0; }
  bool try_tok(const std::string& t) { if (!peek_tok(t)) return false; p_ += t.size(); return true; }
  void expect(const std::string& t) { if (!try_tok(t)) fail("expected '" + t + "'"); }
  static bool word_char(char c) { return std::isalnum((unsigned char)c) || c == '_' || c == '.' || c == '$'; }
  std::string peek_word() {
    skip();
    size_t q = p_;
    while (q < s_.size() && word_char(s_[q])) ++q;
    return s_.substr(p_, q - p_);
  }
  bool try_word(const std::string& w) { if (peek_word() != w) return false; p_ += w.size(); return true; }
  void expect_word(const std::string& w) { if (!try_word(w)) fail("expected '" + w + "'"); }
  std::string word() { std::string w = peek_word(); if (w.empty()) fail("expected an identifier"); p_ += w.size(); return w; }
  int64_t integer() {
    skip();
    size_t q = p_;
    if (q < s_.size() && (s_[q] == '-' || s_[q] == '+')) ++q;
    size_t d = q;
    while (q < s_.size() && std::isdigit((unsigned char)s_[q])) ++q;
    if (q == d) fail("expected an integer");
    int64_t v = std::strtoll(s_.substr(p_, q - p_).c_str(), nullptr, 10);
    p_ = q;
    return v;
  }
  std::string ssa_name() {
    skip();
    if (p_ >= s_.size() || s_[p_] != '%') fail("expected an SSA value name");
    size_t q = p_ + 1;
    while (q < s_.size() && word_char(s_[q])) ++q;
    if (q == p_ + 1) fail("expected an SSA value name");
    std::string n = s_.substr(p_, q - p_);
    p_ = q;
    return n;
  }
  std::string string_literal() {
    skip();
    if (p_ >= s_.size() || s_[p_] != '"') fail("expected a string");
    size_t q = ++p_;
    while (q < s_.size() && s_[q] != '"') ++q;
    if (q >= s_.size()) fail("unterminated string");
    std::string v = s_.substr(p_, q - p_);
    p_ = q + 1;
    return v;
  }

  // ------------------------------------------------------------ SSA scopes
  void define(const std::string& name, ValueImpl* v) {
    if (scopes_.empty()) scopes_.emplace_back();
    if (lookup_or_null(name)) fail("redefinition of SSA value '" + name + "'");
    scopes_.back()[name] = v;
  }
  ValueImpl* lookup_or_null(const std::string& name) const {
    for (auto it = scopes_.rbegin(); it != scopes_.rend(); ++it) {
      auto f = it->find(name);
      if (f != it->end()) return f->second;
    }
    return nullptr;
  }
  Value use(const std::string& name) {
    ValueImpl* v = lookup_or_null(name);
    if (!v) fail("use of undeclared SSA value name '" + name + "'");
    return Value{v};
  }

  // ------------------------------------------------------------ types
  Type parse_type() {
    skip();
    if (peek_tok("(")) {  // function type
      std::vector<Type> in = parse_type_list_parens(), out;
      expect("->");
      if (peek_tok("(")) out = parse_type_list_parens(); else out.push_back(parse_type());
      return Type::function(in, out);
    }
    std::string w = word();
    static const std::map<std::string, TypeKind> scalars = {
        {"f16", TypeKind::F16}, {"bf16", TypeKind::BF16}, {"f32", TypeKind::F32}, {"f64", TypeKind::F64}, {"f8E4M3FN", TypeKind::F8E4M3FN},
        {"f8E5M2", TypeKind::F8E5M2}, {"i1", TypeKind::I1}, {"i8", TypeKind::I8}, {"i32", TypeKind::I32}, {"i64", TypeKind::I64}, {"index", TypeKind::Index}};
    auto it = scalars.find(w);
    if (it != scalars.end()) return Type::scalar(it->second);
    if (w != "memref" && w != "tensor") fail("unknown type '" + w + "'");
    expect("<");
    std::vector<int64_t> shape;
    Type elem;
    for (;;) {  // 4096x4096xf16 : extents, then the element type, separated by 'x'
      skip();
      if (p_ < s_.size() && s_[p_] == '?') { ++p_; shape.push_back(-1); }
      else if (p_ < s_.size() && std::isdigit((unsigned char)s_[p_])) {
        size_t q = p_;
        while (q < s_.size() && std::isdigit((unsigned char)s_[q])) ++q;
        shape.push_back(std::strtoll(s_.substr(p_, q - p_).c_str(), nullptr, 10));
        p_ = q;
      } else { elem = parse_type(); break; }
      if (p_ >= s_.size() || s_[p_] != 'x') fail("expected 'x' in a shape");
      ++p_;
    }
    AffineMap layout;
    int space = 0;
    if (w == "memref") {
      while (try_tok(",")) {
        if (try_word("affine_map")) { expect("<"); layout = parse_affine_map(); expect(">"); }
        else space = (int)integer();
      }
    }
    expect(">");
    return w == "memref" ? Type::memref(shape, elem, layout, space) : Type::tensor(shape, elem);
  }
  std::vector<Type> parse_type_list_parens() {
    std::vector<Type> out;
    expect("(");
    if (try_tok(")")) return out;
    do out.push_back(parse_type()); while (try_tok(","));
    expect(")");
    return out;
  }

  // ------------------------------------------------------------ affine expressions and maps
  // names: identifier -> expression (d0, s0 of a map; SSA names of an index list)
  using Names = std::function<AffineExpr(const std::string&)>;
  AffineExpr affine_expr(const Names& names) {  // sums bind weakest
    AffineExpr v = affine_term(names);
    for (;;) {
      if (try_tok("+")) v = v + affine_term(names);
      else if (peek_tok("-") && !peek_tok("->")) { ++p_; v = v - affine_term(names); }
      else return v;
    }
  }
  AffineExpr affine_term(const Names& names) {  // * floordiv ceildiv mod, left to right
    AffineExpr v = affine_factor(names);
    for (;;) {
      if (try_tok("*")) v = v * affine_factor(names);
      else if (try_word("floordiv")) v = v.floor_div(affine_factor(names));
      else if (try_word("ceildiv")) v = v.ceil_div(affine_factor(names));
      else if (try_word("mod")) v = v.mod(affine_factor(names));
      else return v;
    }
  }
  AffineExpr affine_factor(const Names& names) {
    skip();
    if (try_tok("(")) { AffineExpr v = affine_expr(names); expect(")"); return v; }
    if (peek_tok("-") && !peek_tok("->")) { ++p_; return -affine_factor(names); }
    if (p_ < s_.size() && std::isdigit((unsigned char)s_[p_])) return AffineExpr::constant(integer());
    if (p_ < s_.size() && s_[p_] == '%') return names(ssa_name());
    return names(word());
  }
  AffineMap parse_affine_map() {  // (d0, d1)[s0] -> (e0, e1)
    std::map<std::string, AffineExpr> ids;
    int nd = 0, ns = 0;
    expect("(");
    if (!try_tok(")")) { do ids[word()] = AffineExpr::dim(nd++); while (try_tok(",")); expect(")"); }
    if (try_tok("[")) { if (!try_tok("]")) { do ids[word()] = AffineExpr::symbol(ns++); while (try_tok(",")); expect("]"); } }
    expect("->");
    expect("(");
    std::vector<AffineExpr> results;
    Names names = [&](const std::string& n) -> AffineExpr {
      auto it = ids.find(n);
      if (it == ids.end()) fail("use of undeclared identifier '" + n + "' in an affine map");
      return it->second;
    };
    if (!try_tok(")")) { do results.push_back(affine_expr(names)); while (try_tok(",")); expect(")"); }
    return AffineMap(nd, ns, results);
  }
  // `[e0, e1]` over SSA ids: every distinct id becomes a dim, in order of first appearance (parseAffineMapOfSSAIds)
  AffineMap parse_map_of_ssa_ids(std::vector<Value>& operands) {
    std::vector<std::string> seen;
    Names names = [&](const std::string& n) -> AffineExpr {
      for (size_t i = 0; i < seen.size(); ++i) if (seen[i] == n) return AffineExpr::dim((int64_t)i);
      operands.push_back(use(n));
      seen.push_back(n);
      return AffineExpr::dim((int64_t)seen.size() - 1);
    };
    std::vector<AffineExpr> results;
    expect("[");
    if (!try_tok("]")) { do results.push_back(affine_expr(names)); while (try_tok(",")); expect("]"); }
    return AffineMap((int)seen.size(), 0, results);
  }

  // ------------------------------------------------------------ attributes
  Attribute parse_attribute() {
    skip();
    if (peek_tok("\"")) return Attribute::string(string_literal());
    if (try_word("true")) return Attribute::boolean(true);
    if (try_word("false")) return Attribute::boolean(false);
    if (try_tok("#frisk<")) {
      expect_word("gemm_warp_policy");
      std::string p = word();
      expect(">");
      if (p == "Square") return Attribute::policy(GemmWarpPolicy::Square);
      if (p == "FullRow") return Attribute::policy(GemmWarpPolicy::FullRow);
      if (p == "FullCol") return Attribute::policy(GemmWarpPolicy::FullCol);
      fail("unknown gemm_warp_policy '" + p + "'");
    }
    if (try_word("affine_map")) { expect("<"); AffineMap m = parse_affine_map(); expect(">"); return Attribute::affine_map(m); }
    if (try_word("array")) {
      expect("<");
      expect_word("i64");
      std::vector<int64_t> v;
      if (try_tok(":")) do v.push_back(integer()); while (try_tok(","));
      expect(">");
      return Attribute::int_array(v);
    }
    if (peek_tok("[")) {  // the bare integer lists of src_extents / dst_extents
      ++p_;
      std::vector<int64_t> v;
      if (!try_tok("]")) { do v.push_back(integer()); while (try_tok(",")); expect("]"); }
      return Attribute::int_array(v);
    }
    // number: integer `N [: iW]`, float `1.000000e+00 : f16`, or the hexadecimal bit pattern of a non-finite float
    skip();
    size_t q = p_;
    if (q < s_.size() && (s_[q] == '-' || s_[q] == '+')) ++q;
    if (q < s_.size() && std::isdigit((unsigned char)s_[q])) {
      bool is_float = false, is_hex = false;
      if (s_[q] == '0' && q + 1 < s_.size() && (s_[q + 1] == 'x' || s_[q + 1] == 'X')) { is_hex = true; q += 2; while (q < s_.size() && std::isxdigit((unsigned char)s_[q])) ++q; }
      else {
        while (q < s_.size() && (std::isdigit((unsigned char)s_[q]) || s_[q] == '.' || s_[q] == 'e' || s_[q] == 'E' ||
                                 ((s_[q] == '-' || s_[q] == '+') && (s_[q - 1] == 'e' || s_[q - 1] == 'E')))) {
          if (s_[q] == '.' || s_[q] == 'e' || s_[q] == 'E') is_float = true;
          ++q;
        }
      }
      const std::string num = s_.substr(p_, q - p_);
      p_ = q;
      if (is_float || is_hex) {
        double v;
        if (is_hex) {
          const unsigned long bits = std::strtoul(num.c_str(), nullptr, 16);
          v = bits == 0x7F800000ul ? INFINITY : bits == 0xFF800000ul ? -INFINITY : NAN;
        } else v = std::strtod(num.c_str(), nullptr);
        expect(":");
        return Attribute::floating(v, parse_type());
      }
      const int64_t v = std::strtoll(num.c_str(), nullptr, 10);
      int width = 64;
      if (try_tok(":")) {
        Type t = parse_type();
        if (t.is_float()) return Attribute::floating((double)v, t);
        width = t.bit_width();
      }
      return Attribute::integer(v, width);
    }
    // anything else that starts a type is a type attribute
    return Attribute::type_attr(parse_type());
  }
  void parse_attr_dict(Operation* op) {
    expect("{");
    if (try_tok("}")) return;
    do {
      skip();
      std::string key = peek_tok("\"") ? string_literal() : word();
      if (try_tok("=")) op->attrs[key] = parse_attribute();
      else op->attrs[key] = Attribute::boolean(true);  // unit attribute
    } while (try_tok(","));
    expect("}");
  }
  bool try_attr_dict(Operation* op) {
    if (!peek_tok("{")) return false;
    parse_attr_dict(op);
    return true;
  }

  // ------------------------------------------------------------ regions and operations
  // `{ ops }` into a fresh block whose arguments (already created, with their names) come from the op's header
  void parse_region(Operation* op, const std::vector<std::pair<std::string, Type>>& args) {
    Region* rg = ctx_.new_region(op);
    Block* body = ctx_.new_block();
    body->parent = rg;
    rg->blocks.push_back(body);
    scopes_.emplace_back();
    for (auto& a : args) {
      Value v = ctx_.add_block_arg(body, a.second);
      if (!a.first.empty()) define(a.first, v.impl);
    }
    expect("{");
    while (!try_tok("}")) parse_operation(body);
    // the printer drops the terminator (printBlockTerminators = false); every region of the dialect ends in frisk.end
    if (!body->has_terminator()) { Operation* end = ctx_.new_op("frisk.end"); end->block = body; body->ops.push_back(end); }
    scopes_.pop_back();
  }
  void parse_top_level(Block* body) {
    if (peek_word() != "frisk.kernel") fail("expected 'frisk.kernel'");
    // a kernel is isolated from above: names do not leak between kernels
    auto saved = std::move(scopes_);
    scopes_.clear();
    parse_operation(body);
    scopes_ = std::move(saved);
  }
  std::vector<std::string> arg_name_list() {  // (%a, %b)
    std::vector<std::string> names;
    expect("(");
    if (!try_tok(")")) { do names.push_back(ssa_name()); while (try_tok(",")); expect(")"); }
    return names;
  }
  std::vector<int64_t> int_list_parens() {
    std::vector<int64_t> v;
    expect("(");
    if (!try_tok(")")) { do v.push_back(integer()); while (try_tok(",")); expect(")"); }
    return v;
  }
  Type memref_type(const char* what) {
    Type t = parse_type();
    if (!t.is_memref()) fail(std::string("expected memref type for ") + what);
    return t;
  }
  void check_operand_type(const Value& v, const Type& t, const std::string& name) {
    if (!v.type().equals(t)) fail("use of value '" + name + "' expects different type than prior uses: '" + t.str() + "' vs '" + v.type().str() + "'");
  }

  void one_result(Operation* op, std::vector<std::string>& results, const Type& t) {
    if (results.size() != 1) fail("operation '" + op->name + "' defines one result");
    define(results[0], ctx_.add_result(op, t).impl);
    results.clear();
  }

  void parse_operation(Block* block) {
    skip();
    std::vector<std::string> results;
    if (peek_tok("%")) {
      do results.push_back(ssa_name()); while (try_tok(","));
      expect("=");
    }
    const std::string n = word();
    Operation* op = ctx_.new_op(n);
    op->block = block;
    if (n == "frisk.kernel") {
      expect("@");
      op->attrs["sym_name"] = Attribute::string(word());
      std::vector<Type> in = parse_type_list_parens(), out;
      if (try_tok("->")) out = parse_type_list_parens();
      op->attrs["function_type"] = Attribute::type_attr(Type::function(in, out));
      std::vector<std::pair<std::string, Type>> args;
      for (size_t i = 0; i < in.size(); ++i) args.push_back({"%arg" + std::to_string(i), in[i]});
      parse_region(op, args);
      try_attr_dict(op);
    } else if (n == "frisk.parallel" || n == "frisk.block") {
      std::vector<std::string> ivs = arg_name_list();
      if (n == "frisk.parallel") expect("="); else expect_word("to");
      op->attrs["ranges"] = Attribute::int_array(int_list_parens());
      if (n == "frisk.parallel") {
        expect(",");
        expect_word("threads");
        expect("=");
        op->attrs["threads"] = Attribute::integer(integer());
      }
      if (ivs.size() != op->attrs["ranges"].ints.size()) fail("number of induction variables does not match the number of ranges");
      std::vector<std::pair<std::string, Type>> args;
      for (auto& v : ivs) args.push_back({v, Type::scalar(TypeKind::Index)});
      parse_region(op, args);
      if (n == "frisk.block") try_attr_dict(op);
    } else if (n == "frisk.for") {
      std::string iv = ssa_name();
      expect("=");
      op->attrs["lower"] = Attribute::integer(integer());
      expect_word("to");
      op->attrs["upper"] = Attribute::integer(integer());
      int64_t step = 1;
      if (try_word("step")) { expect("="); step = integer(); }
      op->attrs["step"] = Attribute::integer(step);
      parse_region(op, {{iv, Type::scalar(TypeKind::Index)}});
    } else if (n == "frisk.alloc_buffer") {
      // {scope = "shared", alignment = 1024} -> memref<...>: the attributes are derived from the keys and the type
      expect("{");
      std::string scope;
      int64_t alignment = 0;
      if (!try_tok("}")) {
        do {
          std::string key = word();
          expect("=");
          if (key == "scope") scope = string_literal();
          else if (key == "alignment") alignment = integer();
          else fail("unknown alloc_buffer key '" + key + "'");
        } while (try_tok(","));
        expect("}");
      }
      expect("->");
      Type t = memref_type("result");
      const int space = t.impl->memory_space;
      const char* want = space == (int)MemorySpace::Shared ? "shared" : space == (int)MemorySpace::Global ? "global" : space == (int)MemorySpace::Local ? "local" : "unknown";
      if (!scope.empty() && scope != want) fail("scope \"" + scope + "\" does not match the memory space of the result type");
      op->attrs["shape"] = Attribute::int_array(t.impl->shape);
      op->attrs["elementType"] = Attribute::type_attr(t.element());
      op->attrs["memory_space"] = Attribute::integer(space);
      op->attrs["alignment"] = Attribute::integer(alignment);
      if (results.size() != 1) fail("frisk.alloc_buffer defines one result");
      define(results[0], ctx_.add_result(op, t).impl);
      results.clear();
    } else if (n == "frisk.copy") {
      const std::string src = ssa_name();
      std::vector<Value> si, di;
      AffineMap sm = parse_map_of_ssa_ids(si);
      expect(",");
      const std::string dst = ssa_name();
      AffineMap dm = parse_map_of_ssa_ids(di);
      expect("{");
      expect_word("src_extents");
      expect("=");
      Attribute se = parse_attribute();
      expect(",");
      expect_word("dst_extents");
      expect("=");
      Attribute de = parse_attribute();
      expect("}");
      if (se.kind != Attribute::IntArray || de.kind != Attribute::IntArray) fail("extents must be integer lists");
      try_attr_dict(op);
      expect(":");
      Type st = memref_type("the copy source");
      expect(",");
      Type dt = memref_type("the copy destination");
      Value sv = use(src), dv = use(dst);
      check_operand_type(sv, st, src);
      check_operand_type(dv, dt, dst);
      op->operands = {sv, dv};
      op->operands.insert(op->operands.end(), si.begin(), si.end());
      op->operands.insert(op->operands.end(), di.begin(), di.end());
      op->src_index_count = (int)si.size();
      op->attrs["srcMap"] = Attribute::affine_map(sm);
      op->attrs["dstMap"] = Attribute::affine_map(dm);
      op->attrs["srcExtents"] = se;
      op->attrs["dstExtents"] = de;
    } else if (n == "frisk.gemm") {
      expect("(");
      std::vector<std::string> names = {ssa_name()};
      expect(",");
      names.push_back(ssa_name());
      expect(",");
      names.push_back(ssa_name());
      expect(")");
      try_attr_dict(op);
      expect(":");
      for (size_t i = 0; i < 3; ++i) {
        if (i) expect(",");
        Type t = parse_type();
        Value v = use(names[i]);
        check_operand_type(v, t, names[i]);
        op->operands.push_back(v);
      }
    } else if (n == "frisk.fill" || n == "frisk.reduce") {
      std::vector<std::string> names = {ssa_name()};
      if (n == "frisk.reduce") { expect(","); names.push_back(ssa_name()); }
      try_attr_dict(op);
      expect(":");
      for (size_t i = 0; i < names.size(); ++i) {
        if (i) expect(",");
        Type t = parse_type();
        Value v = use(names[i]);
        check_operand_type(v, t, names[i]);
        op->operands.push_back(v);
      }
    } else if (n == "frisk.end") {
      try_attr_dict(op);
    } else if (n == "arith.constant") {
      Attribute v = parse_attribute();
      if (v.kind != Attribute::Float && v.kind != Attribute::Int) fail("arith.constant expects a number with its type");
      op->attrs["value"] = v;
      one_result(op, results, v.kind == Attribute::Float ? v.type : Type::scalar(v.int_width == 32 ? TypeKind::I32 : TypeKind::I64));
    } else if (n == "affine.load" || n == "affine.store") {
      std::string stored;
      if (n == "affine.store") { stored = ssa_name(); expect(","); }
      const std::string mem = ssa_name();
      std::vector<Value> idx;
      AffineMap map = parse_map_of_ssa_ids(idx);
      expect(":");
      Type mt = memref_type("the accessed buffer");
      Value mv = use(mem);
      check_operand_type(mv, mt, mem);
      if (n == "affine.store") op->operands.push_back(use(stored));
      op->operands.push_back(mv);
      op->operands.insert(op->operands.end(), idx.begin(), idx.end());
      op->attrs["map"] = Attribute::affine_map(map);
      if (n == "affine.load") one_result(op, results, mt.element());
    } else if (is_scalar_binary(n) || is_scalar_unary(n)) {
      std::vector<std::string> names = {ssa_name()};
      if (is_scalar_binary(n)) { expect(","); names.push_back(ssa_name()); }
      expect(":");
      Type t = parse_type();
      for (auto& nm : names) { Value v = use(nm); check_operand_type(v, t, nm); op->operands.push_back(v); }
      one_result(op, results, t);
    } else if (is_scalar_cast(n)) {
      const std::string nm = ssa_name();
      expect(":");
      Type from = parse_type();
      expect_word("to");
      Type to = parse_type();
      Value v = use(nm);
      check_operand_type(v, from, nm);
      op->operands.push_back(v);
      one_result(op, results, to);
    } else {
      fail("unknown operation '" + n + "'");
    }
    if (!results.empty()) fail("operation '" + n + "' defines no results");
    block->ops.push_back(op);
  }
};

inline Operation* parse_module_text(Context& ctx, const std::string& text) { return IrParser(ctx, text).parse_module(); }

}  // namespace frisk_ir
