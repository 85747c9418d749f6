// A small, MLIR-free IR that carries the Frisk dialect's GEMM program:
// module / kernel / parallel / block / for / end / alloc_buffer / copy / fill /
// reduce / gemm, memref and function types, affine maps, and the textual form
// MLIR prints for them.
//
// The reference builds these ops with MLIR (include/Dialect/Frisk/IR/FriskOps.td,
// lib/Dialect/Frisk/IR/FriskOps.cpp) and exposes an OpBuilder to Python
// (ffi/ir.cpp).  MLIR is not available where this runs, so the data model,
// the custom printers (FriskOps.cpp:953-973 kernel, :1023-1038 parallel,
// :1147-1162 block, :1250-1259 for, :1519-1545 alloc_buffer, :1642-1665 copy,
// assembly formats FriskOps.td:244,288,409,442) and the verifiers
// (:901-920 kernel, :1264-1283 gemm, :1436-1481 alloc_buffer, :1666-1683 copy,
// :1688-1701 fill, :1725-1767 reduce) are restated here over plain structs.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace frisk_ir {

// ------------------------------------------------------------------ enums
// numeric values as in include/Dialect/Frisk/IR/FriskEnums.td:6-25; the memory
// space number is what a memref type prints (", 1>" global, ", 3>" shared, nothing for local)
enum class MemorySpace : int { Local = 0, Global = 1, Shared = 3 };
enum class GemmWarpPolicy : int { Square = 0, FullRow = 1, FullCol = 2 };

inline const char* policy_name(GemmWarpPolicy p) {
  switch (p) {
    case GemmWarpPolicy::Square: return "Square";
    case GemmWarpPolicy::FullRow: return "FullRow";
    default: return "FullCol";
  }
}

// ------------------------------------------------------------------ affine expressions
enum class ExprKind : int { Add = 0, Mul = 1, Mod = 2, FloorDiv = 3, CeilDiv = 4, Constant = 5, DimId = 6, SymbolId = 7, Null = -1 };

struct AffineExprImpl {
  ExprKind kind;
  int64_t value;  // constant value or position
  std::shared_ptr<const AffineExprImpl> lhs, rhs;
};

struct AffineExpr {
  std::shared_ptr<const AffineExprImpl> impl;
  AffineExpr() = default;
  explicit AffineExpr(std::shared_ptr<const AffineExprImpl> i) : impl(std::move(i)) {}
  explicit operator bool() const { return (bool)impl; }
  ExprKind kind() const { return impl ? impl->kind : ExprKind::Null; }
  static AffineExpr constant(int64_t v) { return AffineExpr(std::make_shared<AffineExprImpl>(AffineExprImpl{ExprKind::Constant, v, nullptr, nullptr})); }
  static AffineExpr dim(int64_t p) { return AffineExpr(std::make_shared<AffineExprImpl>(AffineExprImpl{ExprKind::DimId, p, nullptr, nullptr})); }
  static AffineExpr symbol(int64_t p) { return AffineExpr(std::make_shared<AffineExprImpl>(AffineExprImpl{ExprKind::SymbolId, p, nullptr, nullptr})); }
  bool is_constant() const { return kind() == ExprKind::Constant; }
  int64_t constant_value() const { return impl->value; }
  bool equals(const AffineExpr& o) const {
    if (!impl || !o.impl) return !impl && !o.impl;
    if (impl->kind != o.impl->kind) return false;
    if (impl->kind >= ExprKind::Constant) return impl->value == o.impl->value;
    return AffineExpr(impl->lhs).equals(AffineExpr(o.impl->lhs)) && AffineExpr(impl->rhs).equals(AffineExpr(o.impl->rhs));
  }
  static int64_t floordiv(int64_t a, int64_t b) { int64_t q = a / b; return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; }
  static AffineExpr raw(ExprKind k, const AffineExpr& l, const AffineExpr& r) {
    return AffineExpr(std::make_shared<AffineExprImpl>(AffineExprImpl{k, 0, l.impl, r.impl}));
  }
  bool is_kind_with_const_rhs(ExprKind k) const { return kind() == k && AffineExpr(impl->rhs).is_constant(); }
  // The folding constructor: the simplifications MLIR applies when an affine expression is built (constant folding,
  // constants and symbolic operands to the right, merged constants and coefficients, "e - q * (e floordiv q)" = "e mod q",
  // divisions and remainders of known multiples), so that expressions built the way the reference builds its layouts
  // print the way the reference's logs show them.
  static AffineExpr binary(ExprKind k, AffineExpr l, AffineExpr r) {
    if (!l || !r) throw std::invalid_argument("affine expression operand is null");
    if (l.is_constant() && r.is_constant()) {
      int64_t a = l.constant_value(), b = r.constant_value();
      switch (k) {
        case ExprKind::Add: return constant(a + b);
        case ExprKind::Mul: return constant(a * b);
        case ExprKind::Mod: if (b > 0) return constant(a - floordiv(a, b) * b); break;
        case ExprKind::FloorDiv: if (b > 0) return constant(floordiv(a, b)); break;
        case ExprKind::CeilDiv: if (b > 0) return constant(-floordiv(-a, b)); break;
        default: break;
      }
    }
    switch (k) {
      case ExprKind::Add: return make_add(l, r);
      case ExprKind::Mul: return make_mul(l, r);
      case ExprKind::Mod: return make_mod(l, r);
      case ExprKind::FloorDiv: return make_div(ExprKind::FloorDiv, l, r);
      case ExprKind::CeilDiv: return make_div(ExprKind::CeilDiv, l, r);
      default: throw std::invalid_argument("not a binary affine expression kind");
    }
  }
  static AffineExpr make_add(AffineExpr l, AffineExpr r) {
    // constants, then symbolic expressions, go to the right
    if (l.is_constant() || (l.is_symbolic_or_constant() && !r.is_symbolic_or_constant())) return binary(ExprKind::Add, r, l);
    if (r.is_constant()) {
      if (r.constant_value() == 0) return l;
      if (l.is_kind_with_const_rhs(ExprKind::Add)) return binary(ExprKind::Add, l.lhs(), constant(l.rhs().constant_value() + r.constant_value()));
    }
    // c1 * e + c2 * e = (c1 + c2) * e
    {
      int64_t cl = 1, cr = 1;
      AffineExpr bl = l, br = r;
      if (l.is_kind_with_const_rhs(ExprKind::Mul)) { cl = l.rhs().constant_value(); bl = l.lhs(); }
      if (r.is_kind_with_const_rhs(ExprKind::Mul)) { cr = r.rhs().constant_value(); br = r.lhs(); }
      if (bl.equals(br)) return binary(ExprKind::Mul, bl, constant(cl + cr));
    }
    // (e + c) + f = (e + f) + c
    if (l.is_kind_with_const_rhs(ExprKind::Add)) return binary(ExprKind::Add, binary(ExprKind::Add, l.lhs(), r), l.rhs());
    // e + (e floordiv q) * -q = e mod q, also in the form e + (q * (e floordiv q)) * -1
    if (r.is_kind_with_const_rhs(ExprKind::Mul)) {
      AffineExpr inner = r.lhs();
      int64_t c = r.rhs().constant_value();
      if (c == -1 && inner.is_kind_with_const_rhs(ExprKind::Mul)) { c = -inner.rhs().constant_value(); inner = inner.lhs(); }
      if (c < 0 && inner.is_kind_with_const_rhs(ExprKind::FloorDiv) && inner.rhs().constant_value() == -c && inner.lhs().equals(l))
        return binary(ExprKind::Mod, l, constant(-c));
    }
    return raw(ExprKind::Add, l, r);
  }
  static AffineExpr make_mul(AffineExpr l, AffineExpr r) {
    // the constant or symbolic factor goes to the right
    if (l.is_constant() || (!r.is_symbolic_or_constant() && l.is_symbolic_or_constant())) return binary(ExprKind::Mul, r, l);
    if (r.is_constant()) {
      if (r.constant_value() == 1) return l;
      if (r.constant_value() == 0) return constant(0);
      if (l.is_kind_with_const_rhs(ExprKind::Mul)) return binary(ExprKind::Mul, l.lhs(), constant(l.rhs().constant_value() * r.constant_value()));
    }
    // (e * c) * f = (e * f) * c
    if (l.is_kind_with_const_rhs(ExprKind::Mul)) return binary(ExprKind::Mul, binary(ExprKind::Mul, l.lhs(), r), l.rhs());
    return raw(ExprKind::Mul, l, r);
  }
  static AffineExpr make_div(ExprKind k, const AffineExpr& l, const AffineExpr& r) {
    if (r.is_constant() && r.constant_value() >= 1) {
      const int64_t q = r.constant_value();
      if (q == 1) return l;
      // (e * c) div q with q | c
      if (l.is_kind_with_const_rhs(ExprKind::Mul) && l.rhs().constant_value() % q == 0) return binary(ExprKind::Mul, l.lhs(), constant(l.rhs().constant_value() / q));
      // (a + b) floordiv q with q | a or q | b splits
      if (k == ExprKind::FloorDiv && l.kind() == ExprKind::Add &&
          (l.lhs().largest_known_divisor() % q == 0 || l.rhs().largest_known_divisor() % q == 0))
        return binary(ExprKind::Add, binary(k, l.lhs(), r), binary(k, l.rhs(), r));
    }
    return raw(k, l, r);
  }
  static AffineExpr make_mod(const AffineExpr& l, const AffineExpr& r) {
    if (r.is_constant() && r.constant_value() >= 1) {
      const int64_t q = r.constant_value();
      if (l.largest_known_divisor() % q == 0) return constant(0);
      if (l.kind() == ExprKind::Add) {
        if (l.lhs().largest_known_divisor() % q == 0) return binary(ExprKind::Mod, l.rhs(), r);
        if (l.rhs().largest_known_divisor() % q == 0) return binary(ExprKind::Mod, l.lhs(), r);
      }
      // (e mod c) mod q with q | c
      if (l.is_kind_with_const_rhs(ExprKind::Mod) && l.rhs().constant_value() >= 1 && l.rhs().constant_value() % q == 0) return binary(ExprKind::Mod, l.lhs(), r);
    }
    return raw(ExprKind::Mod, l, r);
  }
  AffineExpr operator+(const AffineExpr& o) const { return binary(ExprKind::Add, *this, o); }
  AffineExpr operator+(int64_t v) const { return *this + constant(v); }
  AffineExpr operator*(const AffineExpr& o) const { return binary(ExprKind::Mul, *this, o); }
  AffineExpr operator*(int64_t v) const { return *this * constant(v); }
  AffineExpr operator-() const { return *this * constant(-1); }
  AffineExpr operator-(const AffineExpr& o) const { return *this + (-o); }
  AffineExpr operator-(int64_t v) const { return *this + constant(-v); }
  AffineExpr floor_div(const AffineExpr& o) const { return binary(ExprKind::FloorDiv, *this, o); }
  AffineExpr ceil_div(const AffineExpr& o) const { return binary(ExprKind::CeilDiv, *this, o); }
  AffineExpr mod(const AffineExpr& o) const { return binary(ExprKind::Mod, *this, o); }

  int64_t eval(const std::vector<int64_t>& dims, const std::vector<int64_t>& syms) const {
    switch (kind()) {
      case ExprKind::Constant: return impl->value;
      case ExprKind::DimId: return dims.at((size_t)impl->value);
      case ExprKind::SymbolId: return syms.at((size_t)impl->value);
      default: break;
    }
    int64_t a = AffineExpr(impl->lhs).eval(dims, syms), b = AffineExpr(impl->rhs).eval(dims, syms);
    switch (kind()) {
      case ExprKind::Add: return a + b;
      case ExprKind::Mul: return a * b;
      case ExprKind::Mod: return a - floordiv(a, b) * b;
      case ExprKind::FloorDiv: return floordiv(a, b);
      case ExprKind::CeilDiv: return -floordiv(-a, b);
      default: throw std::invalid_argument("cannot evaluate a null affine expression");
    }
  }
  // ---- analysis and rewriting, following the documented behaviour of mlir::AffineExpr
  AffineExpr lhs() const { return AffineExpr(impl->lhs); }
  AffineExpr rhs() const { return AffineExpr(impl->rhs); }
  bool is_binary() const { return impl && (int)impl->kind <= (int)ExprKind::CeilDiv && (int)impl->kind >= 0; }
  bool is_symbolic_or_constant() const {
    switch (kind()) {
      case ExprKind::Constant: case ExprKind::SymbolId: return true;
      case ExprKind::DimId: case ExprKind::Null: return false;
      default: return lhs().is_symbolic_or_constant() && rhs().is_symbolic_or_constant();
    }
  }
  bool is_pure_affine() const {
    switch (kind()) {
      case ExprKind::Constant: case ExprKind::SymbolId: case ExprKind::DimId: return true;
      case ExprKind::Null: return false;
      case ExprKind::Add: return lhs().is_pure_affine() && rhs().is_pure_affine();
      case ExprKind::Mul: return lhs().is_pure_affine() && rhs().is_pure_affine() && (lhs().is_constant() || rhs().is_constant());
      default: return lhs().is_pure_affine() && rhs().is_constant();  // mod, floordiv, ceildiv by a constant
    }
  }
  static int64_t gcd(int64_t a, int64_t b) { a = a < 0 ? -a : a; b = b < 0 ? -b : b; while (b) { int64_t t = a % b; a = b; b = t; } return a; }
  int64_t largest_known_divisor() const {
    switch (kind()) {
      case ExprKind::Constant: return impl->value < 0 ? -impl->value : impl->value;
      case ExprKind::DimId: case ExprKind::SymbolId: case ExprKind::Null: return 1;
      case ExprKind::Mul: return lhs().largest_known_divisor() * rhs().largest_known_divisor();
      case ExprKind::Add: case ExprKind::Mod: return gcd(lhs().largest_known_divisor(), rhs().largest_known_divisor());
      default: {  // floordiv, ceildiv: exact only when the constant divisor divides what is known of the dividend
        if (rhs().is_constant() && rhs().constant_value() != 0) {
          int64_t l = lhs().largest_known_divisor(), r = rhs().constant_value();
          if (l % r == 0) return l / r < 0 ? -(l / r) : l / r;
        }
        return 1;
      }
    }
  }
  bool is_multiple_of(int64_t factor) const {
    if (factor == 0) return false;
    switch (kind()) {
      case ExprKind::Constant: return impl->value % factor == 0;
      case ExprKind::DimId: case ExprKind::SymbolId: return factor * factor == 1;
      case ExprKind::Null: return false;
      case ExprKind::Mul: {
        int64_t l = lhs().largest_known_divisor();
        return l % factor == 0 || rhs().largest_known_divisor() % factor == 0 || (l * rhs().largest_known_divisor()) % factor == 0;
      }
      default: return largest_known_divisor() % factor == 0;
    }
  }
  bool is_function_of(ExprKind leaf, int64_t position) const {
    if (kind() == leaf) return impl->value == position;
    if (!is_binary()) return false;
    return lhs().is_function_of(leaf, position) || rhs().is_function_of(leaf, position);
  }
  // dims / symbols with a replacement in the lists are substituted; the others stay
  AffineExpr replace_dims_and_symbols(const std::vector<AffineExpr>& dims, const std::vector<AffineExpr>& syms) const {
    switch (kind()) {
      case ExprKind::Constant: case ExprKind::Null: return *this;
      case ExprKind::DimId: return (size_t)impl->value < dims.size() ? dims[(size_t)impl->value] : *this;
      case ExprKind::SymbolId: return (size_t)impl->value < syms.size() ? syms[(size_t)impl->value] : *this;
      default: return binary(kind(), lhs().replace_dims_and_symbols(dims, syms), rhs().replace_dims_and_symbols(dims, syms));
    }
  }
  AffineExpr replace(const AffineExpr& target, const AffineExpr& with) const {
    if (equals(target)) return with;
    if (!is_binary()) return *this;
    return binary(kind(), lhs().replace(target, with), rhs().replace(target, with));
  }
  AffineExpr shift(ExprKind leaf, int64_t shift_by, int64_t offset) const {
    if (kind() == leaf) return impl->value >= offset ? (leaf == ExprKind::DimId ? dim(impl->value + shift_by) : symbol(impl->value + shift_by)) : *this;
    if (!is_binary()) return *this;
    return binary(kind(), lhs().shift(leaf, shift_by, offset), rhs().shift(leaf, shift_by, offset));
  }
  AffineExpr simplified() const {  // rebuild bottom-up through the folding constructor
    if (!is_binary()) return *this;
    return binary(kind(), lhs().simplified(), rhs().simplified());
  }

  // MLIR's spelling; `names` substitutes SSA names for dims (then symbols) when given
  std::string str(const std::vector<std::string>* names = nullptr, int num_dims = 0, bool nested = false) const {
    switch (kind()) {
      case ExprKind::Null: return "<<NULL AFFINE EXPR>>";
      case ExprKind::Constant: return std::to_string(impl->value);
      case ExprKind::DimId: return names ? names->at((size_t)impl->value) : "d" + std::to_string(impl->value);
      case ExprKind::SymbolId: return names ? names->at((size_t)(num_dims + impl->value)) : "s" + std::to_string(impl->value);
      default: break;
    }
    AffineExpr l(impl->lhs), r(impl->rhs);
    std::string out;
    // binding strength as in MLIR's printer: operands of * mod floordiv ceildiv are parenthesised whenever
    // they are binary expressions themselves; operands of a sum never are
    if (kind() == ExprKind::Add) {
      // a + (-1) * b and a + (-c) print as subtractions
      if (r.kind() == ExprKind::Mul && AffineExpr(r.impl->rhs).is_constant() && AffineExpr(r.impl->rhs).constant_value() == -1)
        out = l.str(names, num_dims, false) + " - " + AffineExpr(r.impl->lhs).str(names, num_dims, true);
      else if (r.is_constant() && r.constant_value() < 0)
        out = l.str(names, num_dims, false) + " - " + std::to_string(-r.constant_value());
      else
        out = l.str(names, num_dims, false) + " + " + r.str(names, num_dims, false);
      return nested ? "(" + out + ")" : out;
    }
    const char* op = kind() == ExprKind::Mul ? " * " : kind() == ExprKind::Mod ? " mod " : kind() == ExprKind::FloorDiv ? " floordiv " : " ceildiv ";
    if (kind() == ExprKind::Mul && r.is_constant() && r.constant_value() == -1) out = "-" + l.str(names, num_dims, true);
    else out = l.str(names, num_dims, true) + op + r.str(names, num_dims, true);
    return nested ? "(" + out + ")" : out;
  }
};

struct AffineMapImpl {
  int num_dims, num_symbols;
  std::vector<AffineExpr> results;
};

// default-constructed = "no map" (falsy), as the reference's AffineMap() default argument (ffi/ir.cpp:252-256, 649)
struct AffineMap {
  std::shared_ptr<const AffineMapImpl> impl;
  AffineMap() = default;
  AffineMap(int dims, int syms, std::vector<AffineExpr> results) : impl(std::make_shared<AffineMapImpl>(AffineMapImpl{dims, syms, std::move(results)})) {}
  explicit operator bool() const { return (bool)impl; }
  static AffineMap identity(int n) {
    std::vector<AffineExpr> r;
    for (int i = 0; i < n; ++i) r.push_back(AffineExpr::dim(i));
    return AffineMap(n, 0, r);
  }
  int num_dims() const { return impl ? impl->num_dims : 0; }
  int num_symbols() const { return impl ? impl->num_symbols : 0; }
  int num_inputs() const { return num_dims() + num_symbols(); }
  int num_results() const { return impl ? (int)impl->results.size() : 0; }
  bool is_identity() const {
    if (!impl || impl->num_symbols || num_results() != num_dims()) return false;
    for (int i = 0; i < num_results(); ++i)
      if (impl->results[i].kind() != ExprKind::DimId || impl->results[i].impl->value != i) return false;
    return true;
  }
  // every result a distinct dim (or, if allowed, the constant 0), no symbols
  bool is_projected_permutation(bool allow_zero_in_results) const {
    if (!impl || impl->num_symbols) return false;
    if (num_results() > num_dims() && !allow_zero_in_results) return false;
    std::vector<bool> seen((size_t)num_dims(), false);
    for (const AffineExpr& e : impl->results) {
      if (e.kind() == ExprKind::DimId) {
        if (e.impl->value >= num_dims() || seen[(size_t)e.impl->value]) return false;
        seen[(size_t)e.impl->value] = true;
      } else if (!(allow_zero_in_results && e.is_constant() && e.constant_value() == 0)) {
        return false;
      }
    }
    return true;
  }
  bool equals(const AffineMap& o) const {
    if (!impl || !o.impl) return !impl && !o.impl;
    if (impl->num_dims != o.impl->num_dims || impl->num_symbols != o.impl->num_symbols || impl->results.size() != o.impl->results.size()) return false;
    for (size_t i = 0; i < impl->results.size(); ++i)
      if (!impl->results[i].equals(o.impl->results[i])) return false;
    return true;
  }
  std::string str() const {
    if (!impl) return "<<NULL AFFINE MAP>>";
    std::ostringstream os;
    os << "(";
    for (int i = 0; i < impl->num_dims; ++i) os << (i ? ", " : "") << "d" << i;
    os << ")";
    if (impl->num_symbols) {
      os << "[";
      for (int i = 0; i < impl->num_symbols; ++i) os << (i ? ", " : "") << "s" << i;
      os << "]";
    }
    os << " -> (";
    for (size_t i = 0; i < impl->results.size(); ++i) os << (i ? ", " : "") << impl->results[i].str();
    os << ")";
    return os.str();
  }
};

// ------------------------------------------------------------------ types
enum class TypeKind { None, F16, BF16, F32, F64, F8E4M3FN, F8E5M2, I1, I8, I32, I64, Index, MemRef, Function, RankedTensor };

struct TypeImpl {
  TypeKind kind = TypeKind::None;
  std::vector<int64_t> shape;                            // memref / tensor
  std::shared_ptr<const TypeImpl> element;               // memref / tensor
  int memory_space = 0;                                  // memref
  AffineMap layout;                                      // memref (only the default is printed away)
  std::vector<std::shared_ptr<const TypeImpl>> inputs, results;  // function
};

struct Type {
  std::shared_ptr<const TypeImpl> impl;
  Type() = default;
  explicit Type(std::shared_ptr<const TypeImpl> i) : impl(std::move(i)) {}
  explicit operator bool() const { return (bool)impl; }
  TypeKind kind() const { return impl ? impl->kind : TypeKind::None; }
  static Type scalar(TypeKind k) { auto t = std::make_shared<TypeImpl>(); t->kind = k; return Type(t); }
  static Type memref(std::vector<int64_t> shape, Type elem, AffineMap layout, int space) {
    auto t = std::make_shared<TypeImpl>();
    t->kind = TypeKind::MemRef; t->shape = std::move(shape); t->element = elem.impl; t->memory_space = space; t->layout = layout;
    return Type(t);
  }
  static Type tensor(std::vector<int64_t> shape, Type elem) {
    auto t = std::make_shared<TypeImpl>();
    t->kind = TypeKind::RankedTensor; t->shape = std::move(shape); t->element = elem.impl;
    return Type(t);
  }
  static Type function(const std::vector<Type>& in, const std::vector<Type>& out) {
    auto t = std::make_shared<TypeImpl>();
    t->kind = TypeKind::Function;
    for (auto& x : in) t->inputs.push_back(x.impl);
    for (auto& x : out) t->results.push_back(x.impl);
    return Type(t);
  }
  bool is_float() const {
    switch (kind()) { case TypeKind::F16: case TypeKind::BF16: case TypeKind::F32: case TypeKind::F64: case TypeKind::F8E4M3FN: case TypeKind::F8E5M2: return true; default: return false; }
  }
  bool is_int() const { return kind() == TypeKind::I1 || kind() == TypeKind::I8 || kind() == TypeKind::I32 || kind() == TypeKind::I64; }
  bool is_memref() const { return kind() == TypeKind::MemRef; }
  Type element() const { return Type(impl->element); }
  int bit_width() const {
    switch (kind()) {
      case TypeKind::F16: case TypeKind::BF16: return 16;
      case TypeKind::F32: case TypeKind::I32: return 32;
      case TypeKind::F64: case TypeKind::I64: case TypeKind::Index: return 64;
      case TypeKind::F8E4M3FN: case TypeKind::F8E5M2: case TypeKind::I8: return 8;
      case TypeKind::I1: return 1;
      default: return 0;
    }
  }
  bool equals(const Type& o) const {
    if (!impl || !o.impl) return !impl && !o.impl;
    if (impl->kind != o.impl->kind) return false;
    if (impl->kind == TypeKind::MemRef || impl->kind == TypeKind::RankedTensor)
      return impl->shape == o.impl->shape && element().equals(o.element()) && impl->memory_space == o.impl->memory_space &&
             impl->layout.equals(o.impl->layout);
    if (impl->kind == TypeKind::Function) {
      if (impl->inputs.size() != o.impl->inputs.size() || impl->results.size() != o.impl->results.size()) return false;
      for (size_t i = 0; i < impl->inputs.size(); ++i) if (!Type(impl->inputs[i]).equals(Type(o.impl->inputs[i]))) return false;
      for (size_t i = 0; i < impl->results.size(); ++i) if (!Type(impl->results[i]).equals(Type(o.impl->results[i]))) return false;
    }
    return true;
  }
  std::string str() const {
    switch (kind()) {
      case TypeKind::None: return "<<NULL TYPE>>";
      case TypeKind::F16: return "f16";
      case TypeKind::BF16: return "bf16";
      case TypeKind::F32: return "f32";
      case TypeKind::F64: return "f64";
      case TypeKind::F8E4M3FN: return "f8E4M3FN";
      case TypeKind::F8E5M2: return "f8E5M2";
      case TypeKind::I1: return "i1";
      case TypeKind::I8: return "i8";
      case TypeKind::I32: return "i32";
      case TypeKind::I64: return "i64";
      case TypeKind::Index: return "index";
      default: break;
    }
    std::ostringstream os;
    if (kind() == TypeKind::MemRef || kind() == TypeKind::RankedTensor) {
      os << (kind() == TypeKind::MemRef ? "memref<" : "tensor<");
      for (int64_t d : impl->shape) { if (d < 0) os << "?x"; else os << d << "x"; }
      os << element().str();
      if (kind() == TypeKind::MemRef) {
        if (impl->layout && !impl->layout.is_identity()) os << ", affine_map<" << impl->layout.str() << ">";
        if (impl->memory_space != 0) os << ", " << impl->memory_space;
      }
      os << ">";
      return os.str();
    }
    os << "(";
    for (size_t i = 0; i < impl->inputs.size(); ++i) os << (i ? ", " : "") << Type(impl->inputs[i]).str();
    os << ") -> ";
    if (impl->results.size() == 1 && Type(impl->results[0]).kind() != TypeKind::Function) os << Type(impl->results[0]).str();
    else {
      os << "(";
      for (size_t i = 0; i < impl->results.size(); ++i) os << (i ? ", " : "") << Type(impl->results[i]).str();
      os << ")";
    }
    return os.str();
  }
};

// ------------------------------------------------------------------ attributes
struct Attribute {
  enum Kind { None, Bool, Int, Float, String, Policy, IntArray, Map, TypeAttr } kind = None;
  bool b = false;
  int64_t i = 0;
  int int_width = 64;
  double f = 0.0;
  Type type;  // of a float / type attribute
  std::string s;
  std::vector<int64_t> ints;
  AffineMap map;
  static Attribute boolean(bool v) { Attribute a; a.kind = Bool; a.b = v; return a; }
  static Attribute integer(int64_t v, int width = 64) { Attribute a; a.kind = Int; a.i = v; a.int_width = width; return a; }
  static Attribute floating(double v, Type t) { Attribute a; a.kind = Float; a.f = v; a.type = t; return a; }
  static Attribute string(std::string v) { Attribute a; a.kind = String; a.s = std::move(v); return a; }
  static Attribute policy(GemmWarpPolicy p) { Attribute a; a.kind = Policy; a.i = (int)p; return a; }
  static Attribute int_array(std::vector<int64_t> v) { Attribute a; a.kind = IntArray; a.ints = std::move(v); return a; }
  static Attribute affine_map(AffineMap m) { Attribute a; a.kind = Map; a.map = m; return a; }
  static Attribute type_attr(Type t) { Attribute a; a.kind = TypeAttr; a.type = t; return a; }

  static std::string float_str(double v) {
    // MLIR prints "%.6e" style when that round-trips, otherwise more digits
    if (std::isnan(v)) return "0x7FC00000";
    if (std::isinf(v)) return v > 0 ? "0x7F800000" : "0xFF800000";
    char buf[64];
    std::snprintf(buf, sizeof buf, "%.6e", v);
    if (std::strtod(buf, nullptr) == v) return buf;
    std::snprintf(buf, sizeof buf, "%.17g", v);
    return buf;
  }
  std::string str() const {
    switch (kind) {
      case Bool: return b ? "true" : "false";
      case Int: return std::to_string(i) + " : i" + std::to_string(int_width);
      case Float: return float_str(f) + " : " + type.str();
      case String: return "\"" + s + "\"";
      case Policy: return std::string("#frisk<gemm_warp_policy ") + policy_name((GemmWarpPolicy)i) + ">";
      case IntArray: {
        std::string o = "array<i64";
        for (size_t k = 0; k < ints.size(); ++k) o += (k ? ", " : ": ") + std::to_string(ints[k]);
        return o + ">";
      }
      case Map: return "affine_map<" + map.str() + ">";
      case TypeAttr: return type.str();
      default: return "<<NULL ATTRIBUTE>>";
    }
  }
};

// ------------------------------------------------------------------ values, operations, blocks, regions
struct Operation;
struct Block;
struct Region;

struct ValueImpl {
  Type type;
  Operation* def = nullptr;  // result of this operation ...
  Block* block = nullptr;    // ... or argument of this block
  int index = 0;
};

struct Value {
  ValueImpl* impl = nullptr;
  explicit operator bool() const { return impl != nullptr; }
  Type type() const { return impl ? impl->type : Type(); }
  bool operator==(const Value& o) const { return impl == o.impl; }
};

struct Region {
  Operation* parent = nullptr;
  std::vector<Block*> blocks;
};

struct Block {
  Region* parent = nullptr;
  std::vector<ValueImpl*> args;
  std::vector<Operation*> ops;
  bool has_terminator() const;
};

struct Operation {
  std::string name;  // "frisk.gemm", "builtin.module", ...
  std::vector<Value> operands;
  std::vector<ValueImpl*> results;
  std::map<std::string, Attribute> attrs;  // sorted by name, as MLIR stores them
  std::vector<Region*> regions;
  Block* block = nullptr;  // where it is inserted
  int src_index_count = 0; // frisk.copy: operands are [src, dst, srcIndices..., dstIndices...]
  bool is_terminator() const { return name == "frisk.end" || name == "func.return"; }
  const Attribute* attr(const std::string& n) const { auto it = attrs.find(n); return it == attrs.end() ? nullptr : &it->second; }
  int64_t int_attr(const std::string& n) const { auto a = attr(n); if (!a) throw std::invalid_argument("missing attribute " + n); return a->i; }
  bool bool_attr(const std::string& n) const { auto a = attr(n); return a && a->b; }
};

inline bool Block::has_terminator() const { return !ops.empty() && ops.back()->is_terminator(); }

// Owns every IR object created through it; handles on the Python side are raw
// pointers, valid for as long as the context lives (the tests keep it alive by
// stashing it on the module, as they do for the reference).
struct Context {
  std::deque<std::unique_ptr<Operation>> ops;
  std::deque<std::unique_ptr<Block>> blocks;
  std::deque<std::unique_ptr<Region>> regions;
  std::deque<std::unique_ptr<ValueImpl>> values;
  bool dialects_loaded = false;
  bool multithreading = true;
  Operation* new_op(const std::string& name) { ops.emplace_back(new Operation()); ops.back()->name = name; return ops.back().get(); }
  Block* new_block() { blocks.emplace_back(new Block()); return blocks.back().get(); }
  Region* new_region(Operation* parent) { regions.emplace_back(new Region()); regions.back()->parent = parent; parent->regions.push_back(regions.back().get()); return regions.back().get(); }
  ValueImpl* new_value(Type t) { values.emplace_back(new ValueImpl()); values.back()->type = t; return values.back().get(); }
  Value add_result(Operation* op, Type t) { ValueImpl* v = new_value(t); v->def = op; v->index = (int)op->results.size(); op->results.push_back(v); return Value{v}; }
  Value add_block_arg(Block* b, Type t) { ValueImpl* v = new_value(t); v->block = b; v->index = (int)b->args.size(); b->args.push_back(v); return Value{v}; }
};

// The scalar ops of frisk.block bodies (the element-wise steps of the reference's sketches, tmp/ir.mlir:39-47, 49-60,
// 114-147): constants, affine.load / affine.store, floating binary and unary ops, width casts.  Upstream MLIR ops, printed
// in their standard forms.
inline bool is_scalar_binary(const std::string& n) {
  return n == "arith.mulf" || n == "arith.addf" || n == "arith.subf" || n == "arith.divf" || n == "arith.maxnumf" || n == "arith.minnumf";
}
inline bool is_scalar_unary(const std::string& n) { return n == "math.exp2" || n == "math.log2" || n == "arith.negf"; }
inline bool is_scalar_cast(const std::string& n) { return n == "arith.extf" || n == "arith.truncf"; }

// ------------------------------------------------------------------ printer
struct Printer {
  std::map<const ValueImpl*, std::string> names;
  int next_arg = 0, next_result = 0;
  std::ostringstream os;

  void number_block(Block* b) {
    for (ValueImpl* a : b->args) names[a] = "%arg" + std::to_string(next_arg++);
    for (Operation* op : b->ops) {
      for (ValueImpl* r : op->results) names[r] = "%" + std::to_string(next_result++);
      for (Region* rg : op->regions) for (Block* nb : rg->blocks) number_block(nb);
    }
  }
  // SSA names restart inside every kernel / function (they are isolated from above)
  void number_isolated(Operation* op) {
    next_arg = next_result = 0;
    for (Region* rg : op->regions) for (Block* b : rg->blocks) number_block(b);
  }
  std::string name(Value v) {
    auto it = names.find(v.impl);
    return it == names.end() ? "<<UNKNOWN SSA VALUE>>" : it->second;
  }
  void indent(int n) { for (int i = 0; i < n; ++i) os << "  "; }
  void attr_dict(const Operation* op, const std::vector<std::string>& elided, bool leading_space = true) {
    std::vector<std::pair<std::string, const Attribute*>> shown;
    for (auto& kv : op->attrs) {
      bool skip = false;
      for (auto& e : elided) skip = skip || e == kv.first;
      if (!skip) shown.push_back({kv.first, &kv.second});
    }
    if (shown.empty()) return;
    os << (leading_space ? " {" : "{");
    for (size_t i = 0; i < shown.size(); ++i) os << (i ? ", " : "") << shown[i].first << " = " << shown[i].second->str();
    os << "}";
  }
  void region(Region* rg, int ind) {
    os << "{\n";
    for (Block* b : rg->blocks)
      for (Operation* op : b->ops) {
        if (op->name == "frisk.end") continue;  // printBlockTerminators = false
        operation(op, ind + 1);
      }
    indent(ind);
    os << "}";
  }
  void map_of_ssa_ids(const AffineMap& m, const std::vector<Value>& ids) {
    std::vector<std::string> n;
    for (auto& v : ids) n.push_back(name(v));
    for (int i = 0; i < m.num_results(); ++i) os << (i ? ", " : "") << m.impl->results[i].str(&n, m.num_dims());
  }
  void operation(Operation* op, int ind) {
    indent(ind);
    if (!op->results.empty()) {
      for (size_t i = 0; i < op->results.size(); ++i) os << (i ? ", " : "") << names[op->results[i]];
      os << " = ";
    }
    const std::string& n = op->name;
    if (n == "builtin.module") {
      os << "module";
      if (!op->attrs.empty()) os << " attributes";
      attr_dict(op, {}, true);
      os << " {\n";
      for (Operation* k : op->regions[0]->blocks[0]->ops) {
        if (k->name == "frisk.kernel" || k->name == "func.func") number_isolated(k);
        operation(k, ind + 1);
      }
      indent(ind);
      os << "}";
    } else if (n == "frisk.kernel") {
      os << "frisk.kernel @" << op->attr("sym_name")->s << "(";
      const Type& ft = op->attr("function_type")->type;
      for (size_t i = 0; i < ft.impl->inputs.size(); ++i) os << (i ? ", " : "") << Type(ft.impl->inputs[i]).str();
      os << ")";
      if (!ft.impl->results.empty()) {
        os << " -> (";
        for (size_t i = 0; i < ft.impl->results.size(); ++i) os << (i ? ", " : "") << Type(ft.impl->results[i]).str();
        os << ")";
      }
      os << " ";
      region(op->regions[0], ind);
      attr_dict(op, {"sym_name", "function_type"});
    } else if (n == "frisk.parallel" || n == "frisk.block") {
      os << n << " (";
      Block* body = op->regions[0]->blocks.empty() ? nullptr : op->regions[0]->blocks[0];
      if (body) for (size_t i = 0; i < body->args.size(); ++i) os << (i ? ", " : "") << names[body->args[i]];
      os << ")";
      const auto& r = op->attr(n == "frisk.parallel" ? "ranges" : "ranges")->ints;
      os << (n == "frisk.parallel" ? " = (" : " to (");
      for (size_t i = 0; i < r.size(); ++i) os << (i ? ", " : "") << r[i];
      os << ")";
      if (n == "frisk.parallel") os << ", threads = " << op->int_attr("threads");
      os << " ";
      region(op->regions[0], ind);
    } else if (n == "frisk.for") {
      Block* body = op->regions[0]->blocks[0];
      os << "frisk.for " << names[body->args[0]] << " = " << op->int_attr("lower") << " to " << op->int_attr("upper");
      if (op->int_attr("step") > 1) os << " step = " << op->int_attr("step");
      os << " ";
      region(op->regions[0], ind);
    } else if (n == "frisk.alloc_buffer") {
      os << "frisk.alloc_buffer {scope = \"";
      switch ((MemorySpace)op->int_attr("memory_space")) {
        case MemorySpace::Local: os << "local"; break;
        case MemorySpace::Global: os << "global"; break;
        case MemorySpace::Shared: os << "shared"; break;
        default: os << "unknown";
      }
      os << "\"";
      if (op->int_attr("alignment") != 0) os << ", alignment = " << op->int_attr("alignment");
      os << "} -> " << op->results[0]->type.str();
    } else if (n == "frisk.copy") {
      std::vector<Value> si(op->operands.begin() + 2, op->operands.begin() + 2 + op->src_index_count);
      std::vector<Value> di(op->operands.begin() + 2 + op->src_index_count, op->operands.end());
      os << "frisk.copy " << name(op->operands[0]) << "[";
      map_of_ssa_ids(op->attr("srcMap")->map, si);
      os << "], " << name(op->operands[1]) << "[";
      map_of_ssa_ids(op->attr("dstMap")->map, di);
      os << "] {src_extents = [";
      const auto& se = op->attr("srcExtents")->ints;
      const auto& de = op->attr("dstExtents")->ints;
      for (size_t i = 0; i < se.size(); ++i) os << (i ? ", " : "") << se[i];
      os << "], dst_extents = [";
      for (size_t i = 0; i < de.size(); ++i) os << (i ? ", " : "") << de[i];
      os << "]} ";
      attr_dict(op, {"srcMap", "dstMap", "srcExtents", "dstExtents"});
      os << " : " << op->operands[0].type().str() << ", " << op->operands[1].type().str();
    } else if (n == "frisk.gemm") {
      os << "frisk.gemm(" << name(op->operands[0]) << ", " << name(op->operands[1]) << ", " << name(op->operands[2]) << ")";
      attr_dict(op, {});
      os << " : " << op->operands[0].type().str() << ", " << op->operands[1].type().str() << ", " << op->operands[2].type().str();
    } else if (n == "frisk.fill") {
      os << "frisk.fill " << name(op->operands[0]);
      attr_dict(op, {});
      os << " : " << op->operands[0].type().str();
    } else if (n == "frisk.reduce") {
      os << "frisk.reduce " << name(op->operands[0]) << ", " << name(op->operands[1]);
      attr_dict(op, {});
      os << " : " << op->operands[0].type().str() << ", " << op->operands[1].type().str();
    } else if (n == "frisk.end") {
      os << "frisk.end";
    } else if (n == "arith.constant") {
      os << "arith.constant " << op->attr("value")->str();
    } else if (n == "affine.load") {
      os << "affine.load " << name(op->operands[0]) << "[";
      map_of_ssa_ids(op->attr("map")->map, std::vector<Value>(op->operands.begin() + 1, op->operands.end()));
      os << "] : " << op->operands[0].type().str();
    } else if (n == "affine.store") {
      os << "affine.store " << name(op->operands[0]) << ", " << name(op->operands[1]) << "[";
      map_of_ssa_ids(op->attr("map")->map, std::vector<Value>(op->operands.begin() + 2, op->operands.end()));
      os << "] : " << op->operands[1].type().str();
    } else if (is_scalar_binary(n)) {
      os << n << " " << name(op->operands[0]) << ", " << name(op->operands[1]) << " : " << op->results[0]->type.str();
    } else if (is_scalar_unary(n)) {
      os << n << " " << name(op->operands[0]) << " : " << op->results[0]->type.str();
    } else if (is_scalar_cast(n)) {
      os << n << " " << name(op->operands[0]) << " : " << op->operands[0].type().str() << " to " << op->results[0]->type.str();
    } else {
      os << "\"" << n << "\"(";
      for (size_t i = 0; i < op->operands.size(); ++i) os << (i ? ", " : "") << name(op->operands[i]);
      os << ")";
      attr_dict(op, {});
    }
    os << "\n";
  }
};

inline Operation* enclosing_isolated(Operation* op) {
  Operation* cur = op;
  while (cur && cur->name != "frisk.kernel" && cur->name != "func.func" && cur->name != "builtin.module")
    cur = (cur->block && cur->block->parent) ? cur->block->parent->parent : nullptr;
  return cur ? cur : op;
}

inline std::string print_operation(Operation* op) {
  Printer p;
  Operation* root = enclosing_isolated(op);
  if (root->name != "builtin.module") p.number_isolated(root);
  p.operation(op, 0);
  std::string s = p.os.str();
  if (!s.empty() && s.back() == '\n') s.pop_back();
  return s;
}

// ------------------------------------------------------------------ verifier
struct Diagnostics {
  std::vector<std::string> errors;
  void error(const Operation* op, const std::string& msg) { errors.push_back("'" + op->name + "' op " + msg); }
};

inline bool verify_operation(const Operation* op, Diagnostics& d);

inline bool verify_region_ops(const Operation* op, Diagnostics& d) {
  bool ok = true;
  for (Region* rg : op->regions)
    for (Block* b : rg->blocks)
      for (Operation* inner : b->ops) ok = verify_operation(inner, d) && ok;
  return ok;
}

inline bool verify_operation(const Operation* op, Diagnostics& d) {
  bool ok = true;
  auto fail = [&](const std::string& m) { d.error(op, m); ok = false; };
  const std::string& n = op->name;
  auto memref_operand = [&](size_t i, const char* what) -> const TypeImpl* {
    if (i >= op->operands.size() || !op->operands[i].type().is_memref()) { fail(std::string("operand ") + what + " must be a memref"); return nullptr; }
    return op->operands[i].type().impl.get();
  };
  if (n == "frisk.kernel") {
    const Attribute* ft = op->attr("function_type");
    if (!ft || ft->type.kind() != TypeKind::Function) fail("requires a 'function_type' attribute");
    else if (op->regions.empty() || op->regions[0]->blocks.empty()) fail("requires an entry block");
    else {
      Block* body = op->regions[0]->blocks[0];
      if (body->args.size() != ft->type.impl->inputs.size()) fail("region argument count does not match function type");
      else for (size_t i = 0; i < body->args.size(); ++i)
        if (!body->args[i]->type.equals(Type(ft->type.impl->inputs[i]))) fail("region argument type mismatch");
      if (!body->has_terminator()) fail("entry block must end with frisk.end");
    }
  } else if (n == "frisk.parallel" || n == "frisk.block" || n == "frisk.for") {
    if (op->regions.empty() || op->regions[0]->blocks.empty()) fail("requires a body block");
    else {
      Block* body = op->regions[0]->blocks[0];
      size_t want = n == "frisk.for" ? 1 : op->attr(n == "frisk.parallel" ? "ranges" : "ranges")->ints.size();
      if (body->args.size() != want) fail("body block must carry one index argument per range");
      if (!body->has_terminator()) fail("body block must end with frisk.end");
    }
    if (n == "frisk.parallel") {
      if (op->int_attr("threads") <= 0) fail("requires a positive thread count");
      for (int64_t r : op->attr("ranges")->ints) if (r <= 0) fail("grid ranges must be positive");
    }
    if (n == "frisk.for" && op->int_attr("step") <= 0) fail("requires a positive step");
  } else if (n == "frisk.gemm") {
    const TypeImpl *a = memref_operand(0, "A"), *b = memref_operand(1, "B"), *c = memref_operand(2, "C");
    if (a && b && c) {
      if (a->shape.size() != 2 || b->shape.size() != 2 || c->shape.size() != 2) fail("expects rank-2 memrefs");
      else {
        // The reference's verifier (FriskOps.cpp:1264-1283) reads A as [M][K] and B as [K][N] and ignores the transpose
        // flags.  Here a set flag may also mean the operand is stored transposed ([K][M], [N][K]): either reading that
        // fits the op's M, N, K is accepted.
        const bool ta = op->bool_attr("transA"), tb = op->bool_attr("transB");
        const int64_t M = op->int_attr("M"), N = op->int_attr("N"), K = op->int_attr("K");
        auto fits = [](const TypeImpl* t, bool swapped, int64_t r, int64_t cc) { return t->shape[swapped ? 1 : 0] == r && t->shape[swapped ? 0 : 1] == cc; };
        if (!fits(a, ta, M, K) && !fits(a, false, M, K)) fail("A shape does not match M x K");
        if (!fits(b, tb, K, N) && !fits(b, false, K, N)) fail("B shape does not match K x N");
        if (c->shape[0] != M || c->shape[1] != N) fail("C shape does not match M x N");
      }
      if (!Type(a->element).equals(Type(b->element))) fail("A and B must have the same element type");
    }
  } else if (n == "frisk.alloc_buffer") {
    const Type& t = op->results[0]->type;
    if (!t.is_memref()) fail("result must be a memref");
    else {
      if (t.impl->shape != op->attr("shape")->ints) fail("result shape does not match the shape attribute");
      for (int64_t s : t.impl->shape) if (s <= 0) fail("shape must be static and positive");
      if (!t.element().equals(op->attr("elementType")->type)) fail("result element type does not match the elementType attribute");
      if (t.impl->memory_space != op->int_attr("memory_space")) fail("result memory space does not match the memory_space attribute");
      int64_t al = op->int_attr("alignment");
      if (al < 0 || (al & (al - 1)) != 0) fail("alignment must be zero or a power of two");
    }
  } else if (n == "frisk.copy") {
    const TypeImpl *s = memref_operand(0, "src"), *t = memref_operand(1, "dst");
    const AffineMap& sm = op->attr("srcMap")->map;
    const AffineMap& dm = op->attr("dstMap")->map;
    int ns = op->src_index_count, nd = (int)op->operands.size() - 2 - ns;
    if (ns != sm.num_inputs()) fail("expected " + std::to_string(sm.num_inputs()) + " source indices, but got " + std::to_string(ns));
    if (nd != dm.num_inputs()) fail("expected " + std::to_string(dm.num_inputs()) + " destination indices, but got " + std::to_string(nd));
    if (s && sm.num_results() != (int)s->shape.size()) fail("source map must produce one index per source dimension");
    if (t && dm.num_results() != (int)t->shape.size()) fail("destination map must produce one index per destination dimension");
  } else if (n == "arith.constant") {
    const Attribute* v = op->attr("value");
    if (!v || (v->kind != Attribute::Float && v->kind != Attribute::Int)) fail("requires a numeric 'value' attribute");
    else if (op->results.size() != 1) fail("defines one result");
    else if (v->kind == Attribute::Float && !op->results[0]->type.equals(v->type)) fail("result type does not match the value's type");
  } else if (n == "affine.load" || n == "affine.store") {
    const size_t at = n == "affine.load" ? 0 : 1;
    const TypeImpl* m = memref_operand(at, "memref");
    const Attribute* map = op->attr("map");
    if (!map || map->kind != Attribute::Map) fail("requires a 'map' attribute");
    else if (m) {
      if (map->map.num_results() != (int)m->shape.size()) fail("map must produce one index per memref dimension");
      if ((int)op->operands.size() - (int)at - 1 != map->map.num_inputs()) fail("index operand count does not match the map");
      for (size_t i = at + 1; i < op->operands.size(); ++i) if (op->operands[i].type().kind() != TypeKind::Index) fail("indices must have index type");
      const Type elem(m->element);
      if (n == "affine.load" && (op->results.size() != 1 || !op->results[0]->type.equals(elem))) fail("result type must be the memref element type");
      if (n == "affine.store" && !op->operands[0].type().equals(elem)) fail("stored value type must be the memref element type");
    }
  } else if (is_scalar_binary(n) || is_scalar_unary(n)) {
    const size_t want = is_scalar_binary(n) ? 2 : 1;
    if (op->operands.size() != want || op->results.size() != 1) fail("wrong number of operands or results");
    else {
      const Type& t = op->results[0]->type;
      if (!t.is_float()) fail("operates on floating-point values");
      for (const Value& v : op->operands) if (!v.type().equals(t)) fail("operand and result types must be the same");
    }
  } else if (is_scalar_cast(n)) {
    if (op->operands.size() != 1 || op->results.size() != 1) fail("wrong number of operands or results");
    else {
      const Type from = op->operands[0].type(), to = op->results[0]->type;
      if (!from.is_float() || !to.is_float()) fail("casts between floating-point types");
      else if (n == "arith.extf" ? from.bit_width() >= to.bit_width() : from.bit_width() <= to.bit_width()) fail(n == "arith.extf" ? "result must be wider than the operand" : "result must be narrower than the operand");
    }
  } else if (n == "frisk.fill") {
    const TypeImpl* m = memref_operand(0, "memref");
    if (m && !Type(m->element).equals(op->attr("value")->type)) fail("fill value type does not match the memref element type");
  } else if (n == "frisk.reduce") {
    const TypeImpl *s = memref_operand(0, "src"), *t = memref_operand(1, "dst");
    const std::string& kind = op->attr("kind")->s;
    if (kind != "add" && kind != "mul" && kind != "min" && kind != "max" && kind != "sum") fail("unknown reduce kind '" + kind + "'");
    if (s) {
      int64_t dim = op->int_attr("dim");
      if (dim < 0 || dim >= (int64_t)s->shape.size()) fail("reduce dimension out of range");
      else if (t) {
        std::vector<int64_t> want = s->shape;
        want.erase(want.begin() + dim);
        std::vector<int64_t> keep = s->shape;
        keep[(size_t)dim] = 1;
        if (t->shape != want && t->shape != keep) fail("destination shape must be the source shape without (or with extent 1 in) the reduced dimension");
      }
    }
  }
  return verify_region_ops(op, d) && ok;
}

// ------------------------------------------------------------------ the tiled GEMM program
// What the runtime extracts from
//   kernel(A, B, C [, ...]) { parallel (by, bx) = (gm, gn), threads = T {
//     sA = alloc_buffer shared; sB = alloc_buffer shared; acc = alloc_buffer local
//     fill acc, 0 ; for k { copy A -> sA ; copy B -> sB ; gemm(sA, sB, acc) } ; copy acc -> C } }
// (the program shape of the reference's tmp/ir.mlir:1-17).
struct GemmProgram {
  std::string kernel_name;
  int arg_a = -1, arg_b = -1, arg_c = -1;  // kernel argument positions
  Type elem_ab, elem_acc, elem_out;
  int64_t M = 0, N = 0, K = 0;
  int64_t tile_m = 0, tile_n = 0, tile_k = 0;
  int64_t grid_m = 0, grid_n = 0, threads = 0;
  bool transA = false, transB = false, clear_accum = true;
  GemmWarpPolicy policy = GemmWarpPolicy::Square;
  std::string target = "gfx950";
};

inline int kernel_arg_index(const Operation* kernel, Value v) {
  Block* entry = kernel->regions[0]->blocks[0];
  if (v.impl && v.impl->block == entry) return v.impl->index;
  return -1;
}

// The window origin one side of a frisk.copy addresses, as an affine function of (grid index along M, grid index along N,
// K induction variable): origin[r] = cm[r] * by + cn[r] * bx + ck[r] * k + c0[r] for result r of the side's index map.
// Index operands must be those three values; the map must be linear in them.
struct CopyOrigin {
  std::vector<int64_t> cm, cn, ck, c0;
};

inline CopyOrigin copy_origin(const Operation* cp, bool dst_side, Value by, Value bx, Value k) {
  const AffineMap& map = cp->attr(dst_side ? "dstMap" : "srcMap")->map;
  const int ns = cp->src_index_count, first = dst_side ? 2 + ns : 2;
  const int count = dst_side ? (int)cp->operands.size() - 2 - ns : ns;
  if (count != map.num_inputs()) throw std::invalid_argument("not a tiled GEMM kernel: a copy's index operands do not match its index map");
  std::vector<int> which((size_t)count);  // 0 by, 1 bx, 2 k
  for (int i = 0; i < count; ++i) {
    const Value v = cp->operands[(size_t)(first + i)];
    if (v == by) which[(size_t)i] = 0;
    else if (v == bx) which[(size_t)i] = 1;
    else if (k && v == k) which[(size_t)i] = 2;
    else throw std::invalid_argument("not a tiled GEMM kernel: a copy is indexed by something other than the grid indices and the K induction variable");
  }
  auto at = [&](int64_t vby, int64_t vbx, int64_t vk) {
    const int64_t val[3] = {vby, vbx, vk};
    std::vector<int64_t> dims, syms;
    for (int i = 0; i < count; ++i) (i < map.num_dims() ? dims : syms).push_back(val[which[(size_t)i]]);
    std::vector<int64_t> out;
    for (int r = 0; r < map.num_results(); ++r) out.push_back(map.impl->results[(size_t)r].eval(dims, syms));
    return out;
  };
  CopyOrigin o;
  o.c0 = at(0, 0, 0);
  const std::vector<int64_t> m1 = at(1, 0, 0), n1 = at(0, 1, 0), k1 = at(0, 0, 1), probe = at(2, 3, 5);
  for (size_t r = 0; r < o.c0.size(); ++r) {
    o.cm.push_back(m1[r] - o.c0[r]);
    o.cn.push_back(n1[r] - o.c0[r]);
    o.ck.push_back(k1[r] - o.c0[r]);
    if (probe[r] != o.c0[r] + 2 * o.cm[r] + 3 * o.cn[r] + 5 * o.ck[r]) throw std::invalid_argument("not a tiled GEMM kernel: a copy's index map is not linear in the grid and K indices");
  }
  return o;
}

inline GemmProgram match_tiled_gemm(Operation* kernel, Operation* module = nullptr) {
  auto bad = [](const std::string& m) -> GemmProgram { throw std::invalid_argument("not a tiled GEMM kernel: " + m); };
  if (!kernel || kernel->name != "frisk.kernel") return bad("expected a frisk.kernel");
  if (kernel->regions.empty() || kernel->regions[0]->blocks.empty()) return bad("kernel has no entry block");
  GemmProgram g;
  g.kernel_name = kernel->attr("sym_name")->s;
  for (const Operation* scope : {(const Operation*)kernel, (const Operation*)module})
    if (scope) if (auto t = scope->attr("frisk.target")) { g.target = t->s; break; }
  if (g.target.rfind("gfx950", 0) != 0) return bad("frisk.target '" + g.target + "' is not gfx950");
  Block* entry = kernel->regions[0]->blocks[0];
  Operation* par = nullptr;
  for (Operation* op : entry->ops) {
    if (op->name == "frisk.parallel") { if (par) return bad("more than one frisk.parallel"); par = op; }
    else if (op->name != "frisk.end") return bad("unexpected '" + op->name + "' at kernel level");
  }
  if (!par) return bad("no frisk.parallel");
  const auto& grid = par->attr("ranges")->ints;
  if (grid.size() != 2) return bad("frisk.parallel must have a 2-D grid (tiles along M, tiles along N)");
  g.grid_m = grid[0]; g.grid_n = grid[1]; g.threads = par->int_attr("threads");
  if (par->regions[0]->blocks.empty()) return bad("frisk.parallel has no body");
  Block* body = par->regions[0]->blocks[0];

  Operation *loop = nullptr, *gemm = nullptr, *store = nullptr, *fill = nullptr;
  std::vector<Operation*> allocs;
  for (Operation* op : body->ops) {
    if (op->name == "frisk.alloc_buffer") allocs.push_back(op);
    else if (op->name == "frisk.fill") { if (fill) return bad("more than one frisk.fill"); if (loop) return bad("frisk.fill after the K loop"); fill = op; }
    else if (op->name == "frisk.for") { if (loop) return bad("more than one frisk.for"); loop = op; }
    else if (op->name == "frisk.copy") { if (store) return bad("more than one copy after the K loop"); if (!loop) return bad("copy before the K loop"); store = op; }
    else if (op->name != "frisk.end") return bad("unexpected '" + op->name + "' in frisk.parallel");
  }
  if (!loop) return bad("no frisk.for over K");
  if (!store) return bad("no copy of the accumulator to global memory");
  std::vector<Operation*> loads;
  for (Operation* op : loop->regions[0]->blocks[0]->ops) {
    if (op->name == "frisk.copy") loads.push_back(op);
    else if (op->name == "frisk.gemm") { if (gemm) return bad("more than one frisk.gemm"); gemm = op; }
    else if (op->name != "frisk.end") return bad("unexpected '" + op->name + "' in the K loop");
  }
  if (!gemm) return bad("no frisk.gemm in the K loop");
  if (loads.size() != 2) return bad("the K loop must stage exactly A and B");

  Value sA = gemm->operands[0], sB = gemm->operands[1], acc = gemm->operands[2];
  auto space_of = [](Value v) { return v.type().impl->memory_space; };
  if (space_of(sA) != (int)MemorySpace::Shared || space_of(sB) != (int)MemorySpace::Shared) return bad("gemm operands A and B must live in shared memory");
  if (space_of(acc) != (int)MemorySpace::Local) return bad("gemm operand C must be a local fragment");
  Value gA, gB;
  for (Operation* cp : loads) {
    if (cp->operands[1] == sA) gA = cp->operands[0];
    else if (cp->operands[1] == sB) gB = cp->operands[0];
    else return bad("a copy in the K loop does not feed the gemm");
  }
  if (!gA || !gB) return bad("A or B is not staged in the K loop");
  if (!(store->operands[0] == acc)) return bad("the copy after the K loop must read the accumulator");
  Value gC = store->operands[1];
  g.arg_a = kernel_arg_index(kernel, gA); g.arg_b = kernel_arg_index(kernel, gB); g.arg_c = kernel_arg_index(kernel, gC);
  if (g.arg_a < 0 || g.arg_b < 0 || g.arg_c < 0) return bad("A, B and C must be kernel arguments");
  for (Value v : {gA, gB, gC}) if (space_of(v) != (int)MemorySpace::Global) return bad("kernel arguments must be global memrefs");

  g.transA = gemm->bool_attr("transA"); g.transB = gemm->bool_attr("transB");
  {
    // A set flag means the operand is stored transposed; when the op's M, N, K fit only the un-transposed reading of its
    // operand shapes (the reference's reading, where the flag is a layout hint), the operand is taken as stored.
    const auto& ha = sA.type().impl->shape; const auto& hb = sB.type().impl->shape;
    const int64_t gm = gemm->int_attr("M"), gn = gemm->int_attr("N"), gk = gemm->int_attr("K");
    if (g.transA && ha.size() == 2 && ha[0] != ha[1] && ha[0] == gm && ha[1] == gk) g.transA = false;
    if (g.transB && hb.size() == 2 && hb[0] != hb[1] && hb[0] == gk && hb[1] == gn) g.transB = false;
  }
  g.policy = (GemmWarpPolicy)gemm->attr("policy")->i;
  // clear_accum on the gemm restarts the sum every K step; the tiled program clears once with fill 0
  if (gemm->bool_attr("clear_accum")) return bad("gemm inside the K loop must accumulate (clear_accum = false)");
  // The program only ever copies the accumulator to C, so C is never read: the result is (fill value) + A.B.  Only the
  // fill value 0 has a kernel here; without a fill the accumulator would start undefined.
  if (!fill || !(fill->operands[0] == acc)) return bad("the accumulator must be cleared by a frisk.fill before the K loop");
  if (fill->attr("value")->f != 0.0) return bad("the accumulator must be filled with 0 (a GEMM on top of another fill value is not lowered)");
  g.clear_accum = true;
  g.tile_m = gemm->int_attr("M"); g.tile_n = gemm->int_attr("N"); g.tile_k = gemm->int_attr("K");
  const auto& sa = sA.type().impl->shape; const auto& sb = sB.type().impl->shape; const auto& sc = acc.type().impl->shape;
  if (sa.size() != 2 || sb.size() != 2) return bad("the shared tiles of A and B must be rank-2");
  const auto& ga = gA.type().impl->shape; const auto& gb = gB.type().impl->shape; const auto& gc = gC.type().impl->shape;
  if (ga.size() != 2 || gb.size() != 2 || gc.size() != 2) return bad("A, B and C must be rank-2");
  g.M = gc[0]; g.N = gc[1];
  g.K = g.transA ? ga[0] : ga[1];
  int64_t mA = g.transA ? ga[1] : ga[0], kB = g.transB ? gb[1] : gb[0], nB = g.transB ? gb[0] : gb[1];
  if (mA != g.M || nB != g.N || kB != g.K) return bad("global operand shapes are inconsistent");
  // tile extents as staged: op(A) tile is tile_m x tile_k, op(B) tile is tile_k x tile_n
  int64_t tm = g.transA ? sa[1] : sa[0], tkA = g.transA ? sa[0] : sa[1];
  int64_t tkB = g.transB ? sb[1] : sb[0], tn = g.transB ? sb[0] : sb[1];
  if (tkA != tkB) return bad("shared A and B tiles disagree on the K extent");
  if (sc.size() != 2 || sc[0] != tm || sc[1] != tn) return bad("accumulator fragment does not match the staged tiles");
  g.tile_m = tm; g.tile_n = tn; g.tile_k = tkA;
  if (g.grid_m * g.tile_m != g.M || g.grid_n * g.tile_n != g.N) return bad("grid x tile does not cover C exactly");
  int64_t lo = loop->int_attr("lower"), hi = loop->int_attr("upper"), step = loop->int_attr("step");
  if (step <= 0 || hi < lo) return bad("the K loop must count upwards");
  int64_t trips = (hi - lo + step - 1) / step;
  if (trips * g.tile_k != g.K) return bad("the K loop does not cover K exactly");
  // The kernels compute the canonical tiling: tile (by, bx) of C from row band by of op(A) and column band bx of op(B),
  // K tile t of both in iteration t.  Check that the copies address exactly those windows.
  Block* loop_body = loop->regions[0]->blocks[0];
  if (body->args.size() != 2 || loop_body->args.size() != 1) return bad("unexpected block arguments");
  const Value by{body->args[0]}, bx{body->args[1]}, kv{loop_body->args[0]};
  auto window = [&](const Operation* cp, bool dst_side, bool is_global, int64_t rows, int64_t cols, int m_axis, int n_axis, int k_axis, const char* what) {
    const CopyOrigin o = copy_origin(cp, dst_side, by, bx, cp == store ? Value{} : kv);
    if (o.c0.size() != 2) throw std::invalid_argument(std::string("not a tiled GEMM kernel: ") + what + " is not addressed with two indices");
    const std::vector<int64_t>& ext = cp->attr(dst_side ? "dstExtents" : "srcExtents")->ints;
    if (!(ext.size() == 2 && ext[0] == rows && ext[1] == cols)) throw std::invalid_argument(std::string("not a tiled GEMM kernel: the window of ") + what + " is not one whole tile");
    for (int r = 0; r < 2; ++r) {
      const int64_t want_m = (is_global && r == m_axis) ? (m_axis == 0 ? rows : cols) : 0;
      const int64_t want_n = (is_global && r == n_axis) ? (n_axis == 0 ? rows : cols) : 0;
      const bool k_here = is_global && r == k_axis;
      const bool ok = o.cm[(size_t)r] == want_m && o.cn[(size_t)r] == want_n &&
                      (k_here ? (o.ck[(size_t)r] * step == g.tile_k && o.c0[(size_t)r] + o.ck[(size_t)r] * lo == 0) : (o.ck[(size_t)r] == 0 && o.c0[(size_t)r] == 0));
      if (!ok) throw std::invalid_argument(std::string("not a tiled GEMM kernel: ") + what + " is not the window of the canonical tiling (tile (by, bx) of C, K tile of the loop iteration)");
    }
  };
  for (Operation* cp : loads) {
    const bool is_a = cp->operands[1] == sA;
    const auto& sh = is_a ? sa : sb;
    // stored [M][K] / [K][M] for A, [K][N] / [N][K] for B
    const bool k_first = is_a ? g.transA : !g.transB;
    window(cp, false, true, sh[0], sh[1], is_a ? (k_first ? 1 : 0) : -1, is_a ? -1 : (k_first ? 1 : 0), k_first ? 0 : 1, is_a ? "the source of A" : "the source of B");
    window(cp, true, false, sh[0], sh[1], -1, -1, -1, is_a ? "the shared tile of A" : "the shared tile of B");
  }
  window(store, false, false, g.tile_m, g.tile_n, -1, -1, -1, "the accumulator");
  window(store, true, true, g.tile_m, g.tile_n, 0, 1, -1, "the destination in C");
  g.elem_ab = sA.type().element();
  if (!g.elem_ab.equals(sB.type().element()) || !g.elem_ab.equals(gA.type().element()) || !g.elem_ab.equals(gB.type().element()))
    return bad("A and B element types differ between global and shared memory");
  g.elem_acc = acc.type().element();
  g.elem_out = gC.type().element();
  return g;
}

// ------------------------------------------------------------------ data-movement programs
// What the runtime extracts from a kernel made of
//   frisk.fill %arg            frisk.copy %a[map(indices)], %b[map(indices)] {src_extents, dst_extents}
//   frisk.reduce %arg, %arg {kind, dim, clear}
// on kernel arguments of rank 1 or 2 (global memrefs): one entry per op, in program order.  A copy's window origin is its
// index map applied to its index operands; extents follow the op (default: the destination shape left-padded with 1s,
// FriskOps.cpp:1564-1591).  Copies may sit under frisk.parallel and frisk.for and be indexed by their grid indices and
// induction variables: the windows of all iterations must then tile one rectangle of each side without gaps or overlap
// (every index moves the window by whole tiles along one dimension); when every index moves both sides alike the copy is
// lowered as one copy of that rectangle, otherwise (tiles placed transposed, say) as one tile-by-tile copy.  A tile may also pass through one frisk.alloc_buffer (global -> buffer -> global in
// the same block, the buffer used by nothing else): the pair is lowered as the direct copy.  A staged tile may be reduced
// on its way (copy -> buffer, reduce buffer -> vector buffer, copy vector buffer -> global) when the indices move it along
// the kept dimension only: the tiles' reductions are then ONE reduction of the rectangle they cover.  Fill and reduce on
// whole arguments must not be repeated by an enclosing grid or loop.
struct TileOpDesc {
  enum Kind { Fill, Copy, Reduce, CopyTiles } kind = Fill;
  int arg_src = -1, arg_dst = -1;          // kernel argument positions (fill: arg_dst only)
  Type elem_src, elem_dst;
  int64_t src_offset = 0, dst_offset = 0;  // elements from the start of the argument
  int64_t rows = 0, cols = 0, src_ld = 0, dst_ld = 0;
  double value = 0.0;                      // fill
  // CopyTiles: rows x cols is one tile; tile (a, b) of n0 x n1 lies a * step0 + b * step1 elements further on each side
  int64_t n0 = 1, n1 = 1, src_step0 = 0, src_step1 = 0, dst_step0 = 0, dst_step1 = 0;
  std::string reduce_kind;                 // add | mul | min | max
  int64_t dim = 0;
  bool clear = true;
};

// an index a copy may use: value lower + step * i for i in [0, count)
struct IndexRange {
  Value value;
  int64_t lower = 0, step = 1, count = 1;
};

// Window origin of one side of a frisk.copy as a linear function of the iteration numbers i_v of `vars`:
// origin[r] = c0[r] + sum_v stride[r][v] * i_v.  Every index operand must be one of `vars`.
struct TiledOrigin {
  std::vector<int64_t> c0;
  std::vector<std::vector<int64_t>> stride;  // [result][var]
};

inline TiledOrigin tiled_origin(const Operation* cp, bool dst_side, const std::vector<IndexRange>& vars, const std::function<void(const std::string&)>& bad) {
  const AffineMap& map = cp->attr(dst_side ? "dstMap" : "srcMap")->map;
  const int ns = cp->src_index_count, first = dst_side ? 2 + ns : 2;
  const int count = dst_side ? (int)cp->operands.size() - 2 - ns : ns;
  if (count != map.num_inputs()) bad("a copy's index operands do not match its index map");
  std::vector<int> which((size_t)count, -1);
  for (int i = 0; i < count; ++i) {
    for (size_t v = 0; v < vars.size(); ++v) if (cp->operands[(size_t)(first + i)] == vars[v].value) which[(size_t)i] = (int)v;
    if (which[(size_t)i] < 0) bad("a copy is indexed by a value that is neither a grid index nor an enclosing loop's induction variable");
  }
  auto at = [&](const std::vector<int64_t>& iter) {  // origin at iteration numbers `iter`
    std::vector<int64_t> dims, syms;
    for (int i = 0; i < count; ++i) {
      const IndexRange& r = vars[(size_t)which[(size_t)i]];
      (i < map.num_dims() ? dims : syms).push_back(r.lower + r.step * iter[(size_t)which[(size_t)i]]);
    }
    std::vector<int64_t> out;
    for (int r = 0; r < map.num_results(); ++r) out.push_back(map.impl->results[(size_t)r].eval(dims, syms));
    return out;
  };
  TiledOrigin o;
  std::vector<int64_t> zero(vars.size(), 0), probe(vars.size());
  o.c0 = at(zero);
  o.stride.assign(o.c0.size(), std::vector<int64_t>(vars.size(), 0));
  for (size_t v = 0; v < vars.size(); ++v) {
    std::vector<int64_t> unit = zero;
    unit[v] = 1;
    const std::vector<int64_t> r = at(unit);
    for (size_t k = 0; k < r.size(); ++k) o.stride[k][v] = r[k] - o.c0[k];
    probe[v] = (int64_t)(2 * v + 3);
  }
  const std::vector<int64_t> r = at(probe);
  for (size_t k = 0; k < r.size(); ++k) {
    int64_t want = o.c0[k];
    for (size_t v = 0; v < vars.size(); ++v) want += o.stride[k][v] * probe[v];
    if (r[k] != want) bad("a copy's index map is not linear in its indices");
  }
  return o;
}

inline std::vector<TileOpDesc> match_data_movement(Operation* kernel) {
  auto bad = [](const std::string& m) -> std::vector<TileOpDesc> { throw std::invalid_argument("not a data-movement kernel: " + m); };
  const std::function<void(const std::string&)> fail = [](const std::string& m) { throw std::invalid_argument("not a data-movement kernel: " + m); };
  if (!kernel || kernel->name != "frisk.kernel") return bad("expected a frisk.kernel");
  if (kernel->regions.empty() || kernel->regions[0]->blocks.empty()) return bad("kernel has no entry block");
  Block* entry = kernel->regions[0]->blocks[0];
  struct View { int arg; Type elem; int64_t rows, cols; size_t rank; };
  auto view_of = [&](Value v, const char* what) -> View {
    int a = kernel_arg_index(kernel, v);
    if (a < 0 || !v.type().is_memref()) fail(std::string(what) + " is not a kernel argument memref");
    const auto& sh = v.type().impl->shape;
    if (sh.empty() || sh.size() > 2) fail(std::string(what) + " must have rank 1 or 2");
    for (int64_t d : sh) if (d < 0) fail(std::string(what) + " has a dynamic extent");
    return View{a, v.type().element(), sh.size() == 2 ? sh[0] : 1, sh.back(), sh.size()};
  };
  // One side of a copy: the rectangle (r0, c0, rows, cols) that the windows of all iterations cover, in the side's last two
  // dimensions, the tile (tr, tc) one iteration moves, and per index the (dimension from the end, stride) it moves the tile by.
  struct Side { int64_t r0 = 0, c0 = 0, rows = 1, cols = 1, tr = 1, tc = 1; std::vector<std::pair<int, int64_t>> moves; };
  auto side_of = [&](const Operation* cp, bool dst_side, size_t rank, const std::vector<IndexRange>& vars, const char* what) -> Side {
    const TiledOrigin o = tiled_origin(cp, dst_side, vars, fail);
    const auto& ext = cp->attr(dst_side ? "dstExtents" : "srcExtents")->ints;
    if (o.c0.size() != rank) fail(std::string("the ") + what + " map must give one origin per dimension");
    // extents may carry leading 1s (source rank > destination rank): the window is their last `rank` entries
    if (ext.size() < rank) fail(std::string("too few ") + what + " extents");
    for (size_t i = 0; i + rank < ext.size(); ++i) if (ext[i] != 1) fail(std::string("leading ") + what + " extents must be 1");
    Side sd;
    sd.moves.assign(vars.size(), {-1, 0});
    for (size_t r = 0; r < rank; ++r) {
      const int from_end = (int)(rank - 1 - r);
      int64_t tile = ext[ext.size() - rank + r], cover = tile;
      if (tile <= 0) fail(std::string("a ") + what + " extent is not positive");
      std::vector<std::pair<int64_t, size_t>> movers;  // (stride, var)
      for (size_t v = 0; v < vars.size(); ++v) {
        if (vars[v].count <= 1 || o.stride[r][v] == 0) continue;
        if (sd.moves[v].first >= 0) fail(std::string("an index moves the ") + what + " window along two dimensions");
        if (o.stride[r][v] < 0) fail(std::string("an index moves the ") + what + " window backwards");
        sd.moves[v] = {from_end, o.stride[r][v]};
        movers.push_back({o.stride[r][v], v});
      }
      std::sort(movers.begin(), movers.end());
      for (const auto& mv : movers) {
        if (mv.first != cover) fail(std::string("the ") + what + " windows of the iterations do not tile a rectangle (stride " + std::to_string(mv.first) + " where " + std::to_string(cover) + " would continue it)");
        cover *= vars[mv.second].count;
      }
      if (from_end == 0) { sd.c0 = o.c0[r]; sd.cols = cover; sd.tc = tile; } else { sd.r0 = o.c0[r]; sd.rows = cover; sd.tr = tile; }
    }
    return sd;
  };
  auto check_inside = [&](const Side& sd, const View& v, const char* what) {
    if (sd.r0 < 0 || sd.c0 < 0 || sd.r0 + sd.rows > v.rows || sd.c0 + sd.cols > v.cols) fail(std::string("the ") + what + " window leaves the memref");
  };
  auto uses_of = [&](Value buf) {
    int n = 0;
    std::function<void(Block*)> walk = [&](Block* b) {
      for (Operation* op : b->ops) {
        for (const Value& v : op->operands) if (v == buf) ++n;
        for (Region* r : op->regions) for (Block* inner : r->blocks) walk(inner);
      }
    };
    walk(entry);
    return n;
  };

  std::vector<TileOpDesc> out;
  std::vector<IndexRange> vars;
  struct Staged { Value buffer; Operation* load; Block* block; Operation* reduce = nullptr; };  // reduce: the tile was reduced into `buffer` on the way
  std::function<void(Block*)> walk = [&](Block* block) {
    std::vector<Staged> staged;  // tiles loaded into a buffer in this block and not yet stored
    for (Operation* op : block->ops) {
      TileOpDesc d;
      if (op->name == "frisk.end" || op->name == "frisk.alloc_buffer") continue;
      if (op->name == "frisk.parallel" || op->name == "frisk.for") {
        if (!staged.empty()) fail("a tile staged in a buffer must be stored in the block that loaded it");
        if (op->regions.empty() || op->regions[0]->blocks.empty()) fail(op->name + " has no body");
        Block* body = op->regions[0]->blocks[0];
        const size_t depth = vars.size();
        if (op->name == "frisk.parallel") {
          const auto& ranges = op->attr("ranges")->ints;
          for (size_t i = 0; i < ranges.size(); ++i) vars.push_back(IndexRange{Value{body->args[i]}, 0, 1, ranges[i]});
        } else {
          const int64_t lo = op->int_attr("lower"), hi = op->int_attr("upper"), step = op->int_attr("step");
          if (hi <= lo) fail("a frisk.for runs no iteration");
          vars.push_back(IndexRange{Value{body->args[0]}, lo, step, (hi - lo + step - 1) / step});
        }
        walk(body);
        vars.resize(depth);
        continue;
      }
      bool repeated = false;
      for (const IndexRange& r : vars) repeated = repeated || r.count > 1;
      if (op->name == "frisk.fill") {
        if (repeated) fail("a fill under a grid or a loop would run once per iteration");
        View v = view_of(op->operands[0], "the fill target");
        d.kind = TileOpDesc::Fill;
        d.arg_dst = v.arg; d.elem_dst = v.elem; d.rows = v.rows; d.cols = v.cols; d.dst_ld = v.cols;
        d.value = op->attr("value")->f;
      } else if (op->name == "frisk.copy") {
        Operation* load = op;  // the op whose source side is the global source
        const Value src_v = op->operands[0], dst_v = op->operands[1];
        const bool src_is_arg = kernel_arg_index(kernel, src_v) >= 0, dst_is_arg = kernel_arg_index(kernel, dst_v) >= 0;
        auto whole_buffer = [&](const Operation* cp, bool dst_side, Value buf) {
          const TiledOrigin o = tiled_origin(cp, dst_side, vars, fail);
          for (size_t r = 0; r < o.c0.size(); ++r) {
            if (o.c0[r] != 0) fail("the buffer side of a staged copy must start at 0");
            for (size_t v = 0; v < vars.size(); ++v) if (o.stride[r][v] != 0 && vars[v].count > 1) fail("the buffer side of a staged copy must not move");
          }
          const auto& sh = buf.type().impl->shape;
          const auto& ext = cp->attr(dst_side ? "dstExtents" : "srcExtents")->ints;
          if (ext.size() < sh.size()) fail("too few extents on the buffer side of a staged copy");
          for (size_t i = 0; i + sh.size() < ext.size(); ++i) if (ext[i] != 1) fail("leading extents on the buffer side of a staged copy must be 1");
          for (size_t i = 0; i < sh.size(); ++i) if (ext[ext.size() - sh.size() + i] != sh[i]) fail("a staged copy must move the whole buffer");
        };
        if (src_is_arg && !dst_is_arg) {  // global -> buffer: remember it, the store completes it
          if (!dst_v.impl || !dst_v.impl->def || dst_v.impl->def->name != "frisk.alloc_buffer") fail("a copy's destination is neither a kernel argument nor a frisk.alloc_buffer");
          if (uses_of(dst_v) != 2) fail("a staging buffer must be used by exactly one load and one store");
          whole_buffer(op, true, dst_v);
          staged.push_back(Staged{dst_v, op, block});
          continue;
        }
        if (!src_is_arg) {  // buffer -> global: complete the staged copy
          if (!dst_is_arg) fail("a copy moves between two buffers");
          size_t at = staged.size();
          for (size_t i = 0; i < staged.size(); ++i) if (staged[i].buffer == src_v) at = i;
          if (at == staged.size()) fail("a copy stores a buffer that no copy in the same block has loaded");
          whole_buffer(op, false, src_v);
          load = staged[at].load;
          Operation* reduced_by = staged[at].reduce;
          staged.erase(staged.begin() + (long)at);
          if (reduced_by) {
            // copy tile -> buffer; reduce buffer -> vector buffer; copy vector buffer -> global, under a grid or loop whose
            // indices move the source tile along the kept dimension only: ONE reduction of the rectangle all tiles cover
            View s = view_of(load->operands[0], "the reduce source"), t = view_of(dst_v, "the reduce destination");
            if (s.rank != 2) fail("the source of a tiled reduction must have rank 2");
            const Side ss = side_of(load, false, s.rank, vars, "source"), ts = side_of(op, true, t.rank, vars, "destination");
            check_inside(ss, s, "source");
            check_inside(ts, t, "destination");
            d.kind = TileOpDesc::Reduce;
            d.dim = reduced_by->int_attr("dim");
            if (d.dim != 0 && d.dim != 1) fail("reduce dimension out of range");
            if (!reduced_by->attr("clear")->b) fail("a tiled reduction must clear its staging vector (clear = true): the buffer holds nothing before");
            const int kept_from_end = d.dim == 1 ? 1 : 0;   // the source dimension that survives, counted from the last
            if ((d.dim == 1 ? ss.cols != ss.tc : ss.rows != ss.tr)) fail("the grid of a tiled reduction tiles the reduced dimension: partial results of different tiles would have to be combined");
            const int64_t kept = d.dim == 1 ? ss.rows : ss.cols, kept_tile = d.dim == 1 ? ss.tr : ss.tc;
            if (ts.rows != 1 && ts.cols != 1) fail("the destination windows of a tiled reduction do not form a vector");
            const bool dst_along_cols = ts.rows == 1;
            if ((dst_along_cols ? ts.cols : ts.rows) != kept || (dst_along_cols ? ts.tc : ts.tr) != kept_tile) fail("the destination of a tiled reduction does not hold one element per kept index");
            if (!dst_along_cols && t.cols != 1) fail("the destination of a tiled reduction must be contiguous");
            for (size_t v = 0; v < vars.size(); ++v) {
              if (vars[v].count <= 1) continue;
              if (ss.moves[v].first != kept_from_end) fail("an index of a tiled reduction does not move the source tile along the kept dimension");
              if (ts.moves[v].first != (dst_along_cols ? 0 : 1) || ts.moves[v].second != ss.moves[v].second) fail("an index moves the source tile and the destination window of a tiled reduction differently");
            }
            if (!s.elem.equals(t.elem) || !s.elem.equals(load->operands[1].type().element()) || !t.elem.equals(src_v.type().element()))
              fail("the element types of a tiled reduction differ between source, buffers and destination");
            d.arg_src = s.arg; d.arg_dst = t.arg; d.elem_src = s.elem; d.elem_dst = t.elem;
            d.rows = ss.rows; d.cols = ss.cols; d.src_ld = s.cols;
            d.src_offset = ss.r0 * s.cols + ss.c0;
            d.dst_offset = ts.r0 * t.cols + ts.c0;
            d.reduce_kind = reduced_by->attr("kind")->s == "sum" ? "add" : reduced_by->attr("kind")->s;
            d.clear = true;
            out.push_back(d);
            continue;
          }
          const Type via = src_v.type().element();
          if (!via.equals(load->operands[0].type().element()) && !via.equals(dst_v.type().element())) fail("a staging buffer's element type is neither the source's nor the destination's");
        }
        View s = view_of(load->operands[0], "the copy source"), t = view_of(dst_v, "the copy destination");
        d.kind = TileOpDesc::Copy;
        d.arg_src = s.arg; d.arg_dst = t.arg; d.elem_src = s.elem; d.elem_dst = t.elem; d.src_ld = s.cols; d.dst_ld = t.cols;
        const Side ss = side_of(load, false, s.rank, vars, "source"), ts = side_of(op, true, t.rank, vars, "destination");
        check_inside(ss, s, "source");
        check_inside(ts, t, "destination");
        d.src_offset = ss.r0 * s.cols + ss.c0;
        d.dst_offset = ts.r0 * t.cols + ts.c0;
        if (!repeated) {
          // one window on each side: equal shapes, or a dense window against a row
          if (ss.rows * ss.cols != ts.rows * ts.cols) fail("source and destination windows of a copy hold different numbers of elements");
          if (ss.rows == ts.rows && ss.cols == ts.cols) { d.rows = ss.rows; d.cols = ss.cols; }
          else if (ss.rows == 1 && ts.rows == 1) { d.rows = 1; d.cols = ss.cols; }
          else if ((ss.rows == 1 || ts.rows == 1) && (ss.cols == s.cols || ss.rows == 1) && (ts.cols == t.cols || ts.rows == 1)) { d.rows = 1; d.cols = ss.rows * ss.cols; d.src_ld = d.dst_ld = d.cols; }
          else fail("source and destination windows of a copy have different shapes");
        } else {
          if (ss.tr != ts.tr || ss.tc != ts.tc) fail("source and destination tiles of a tiled copy have different shapes");
          bool same_placement = true;
          std::vector<size_t> movers;
          for (size_t v = 0; v < vars.size(); ++v) {
            if (vars[v].count <= 1) continue;
            if (ss.moves[v].first < 0 || ts.moves[v].first < 0) fail("an enclosing grid index or induction variable does not move both windows of a copy: its iterations would repeat or overwrite one another");
            same_placement = same_placement && ss.moves[v] == ts.moves[v];
            movers.push_back(v);
          }
          if (same_placement) {
            d.rows = ss.rows; d.cols = ss.cols;  // equal on both sides by the checks above
          } else {
            // The tiles land elsewhere than they came from (placed transposed, or at another pitch): each side still tiles
            // its own rectangle without gap or overlap (side_of), so every destination element is written once.  One
            // launch copies tile by tile, each index displacing the two sides by its own steps.
            if (movers.size() > 2) fail("a tiled copy that rearranges its tiles may be indexed by at most two grid indices or induction variables");
            d.kind = TileOpDesc::CopyTiles;
            d.rows = ss.tr; d.cols = ss.tc;
            auto step = [](const std::pair<int, int64_t>& mv, int64_t ld) { return mv.first == 0 ? mv.second : mv.second * ld; };
            d.n0 = vars[movers[0]].count;
            d.src_step0 = step(ss.moves[movers[0]], s.cols); d.dst_step0 = step(ts.moves[movers[0]], t.cols);
            if (movers.size() == 2) {
              d.n1 = vars[movers[1]].count;
              d.src_step1 = step(ss.moves[movers[1]], s.cols); d.dst_step1 = step(ts.moves[movers[1]], t.cols);
            }
          }
        }
      } else if (op->name == "frisk.reduce" && kernel_arg_index(kernel, op->operands[0]) < 0) {
        // a reduction of a staged tile into a second buffer: completed by the copy that stores that buffer
        size_t at = staged.size();
        for (size_t i = 0; i < staged.size(); ++i) if (staged[i].buffer == op->operands[0] && !staged[i].reduce) at = i;
        if (at == staged.size()) fail("a reduce reads a buffer that no copy in the same block has loaded");
        const Value vec = op->operands[1];
        if (!vec.impl || !vec.impl->def || vec.impl->def->name != "frisk.alloc_buffer") fail("a reduce of a staged tile must write a frisk.alloc_buffer");
        if (uses_of(vec) != 2) fail("the vector buffer of a tiled reduction must be used by exactly the reduce and one store");
        const auto& tile_shape = op->operands[0].type().impl->shape;
        const auto& vec_shape = vec.type().impl->shape;
        const int64_t dim = op->int_attr("dim");
        if (tile_shape.size() != 2 || vec_shape.size() != 1 || dim < 0 || dim > 1 || vec_shape[0] != tile_shape[(size_t)(1 - dim)]) fail("a reduce of a staged tile must go from a rank-2 buffer to a vector of the kept extent");
        staged[at].buffer = vec;
        staged[at].reduce = op;
        continue;
      } else if (op->name == "frisk.reduce") {
        if (repeated) fail("a reduce under a grid or a loop would run once per iteration");
        View s = view_of(op->operands[0], "the reduce source"), t = view_of(op->operands[1], "the reduce destination");
        if (op->operands[0].type().impl->shape.size() != 2) fail("the reduce source must have rank 2");
        d.kind = TileOpDesc::Reduce;
        d.arg_src = s.arg; d.arg_dst = t.arg; d.elem_src = s.elem; d.elem_dst = t.elem; d.rows = s.rows; d.cols = s.cols; d.src_ld = s.cols;
        d.dim = op->int_attr("dim");
        d.reduce_kind = op->attr("kind")->s == "sum" ? "add" : op->attr("kind")->s;
        d.clear = op->attr("clear")->b;
        if (d.dim != 0 && d.dim != 1) fail("reduce dimension out of range");
        if (t.rows * t.cols != (d.dim == 1 ? s.rows : s.cols)) fail("the reduce destination does not hold one element per kept index");
        if (!s.elem.equals(t.elem)) fail("reduce source and destination element types differ");
      } else {
        fail("operation " + op->name + " is not fill, copy or reduce");
      }
      out.push_back(d);
    }
    if (!staged.empty()) fail("a tile is loaded into a buffer and never stored");
  };
  walk(entry);
  if (out.empty()) return bad("the kernel holds no fill, copy or reduce");
  return out;
}

}  // namespace frisk_ir
