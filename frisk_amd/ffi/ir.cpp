// Builder surface of the Frisk Python API over the MLIR-free IR of mini_ir.h.
// Names, argument orders, defaults and error behaviour follow the reference's
// ffi/ir.cpp (cited per binding); only the calls the GEMM path uses are provided.
#include <iostream>
#include <optional>

#include "ffi.h"
#include "mini_ir.h"
#include "ir_parser.h"

namespace frisk_ffi {

using namespace frisk_ir;
using ret = py::return_value_policy;

struct PyContext {
  std::shared_ptr<Context> ctx = std::make_shared<Context>();
};

// non-owning op handle, as mlir::OpState is
struct OpState {
  Operation* op = nullptr;
  Context* ctx = nullptr;
};
template <int Tag> struct OpT : OpState {};
using ModuleOp = OpT<0>;
using KernelOp = OpT<1>;
using ParallelOp = OpT<2>;
using BlockOp = OpT<3>;
using ForOp = OpT<4>;
using AllocBufferOp = OpT<5>;
using CopyOp = OpT<6>;
using FillOp = OpT<7>;
using ReduceOp = OpT<8>;
using GemmOp = OpT<9>;
using EndOp = OpT<10>;

struct PyBlock {
  Block* block = nullptr;
  Context* ctx = nullptr;
};
struct PyRegion {
  Region* region = nullptr;
  Context* ctx = nullptr;
};

// OpBuilder + insertion point (the reference's OpBuilderWithLoc, include/Dialect/Frisk/Utils/Utils.h:17-92).
// An insertion point is "before `before` in `block`"; before == nullptr means the end of the block.
struct Builder {
  Context* ctx;
  std::shared_ptr<Context> keep;
  Block* block = nullptr;
  Operation* before = nullptr;
  explicit Builder(PyContext& c) : ctx(c.ctx.get()), keep(c.ctx) {}

  void insert(Operation* op) {
    if (!block) return;  // detached, like an OpBuilder without insertion point
    op->block = block;
    auto& ops = block->ops;
    auto it = ops.end();
    if (before)
      for (auto i = ops.begin(); i != ops.end(); ++i)
        if (*i == before) { it = i; break; }
    ops.insert(it, op);
  }
  void set_to_start(Block* b) { block = b; before = b->ops.empty() ? nullptr : b->ops.front(); }
  void set_to_end(Block* b) { block = b; before = nullptr; }
  void set_after(Operation* op) {
    block = op->block;
    before = nullptr;
    if (!block) return;
    for (size_t i = 0; i + 1 < block->ops.size(); ++i)
      if (block->ops[i] == op) before = block->ops[i + 1];
  }
  Operation* make_end() { return ctx->new_op("frisk.end"); }
  template <class T> T wrap(Operation* op) { T t; t.op = op; t.ctx = ctx; return t; }
  // scalar ops of frisk.block bodies: one result each
  Value constant(const Attribute& v) {
    Operation* op = ctx->new_op("arith.constant");
    op->attrs["value"] = v;
    Value r = ctx->add_result(op, v.kind == Attribute::Float ? v.type : Type::scalar(TypeKind::I64));
    insert(op);
    return r;
  }
  Value scalar_op(const std::string& name, std::vector<Value> operands) {
    const Type t = operands.at(0).type();
    if (!t.is_float()) throw std::invalid_argument(name + " expects floating-point operands");
    for (const Value& v : operands)
      if (!v.type().equals(t)) throw std::invalid_argument(name + " expects operands of one type, got " + t.str() + " and " + v.type().str());
    Operation* op = ctx->new_op(name);
    op->operands = operands;
    Value r = ctx->add_result(op, t);
    insert(op);
    return r;
  }
  Value cast_op(const std::string& name, Value x, const Type& to) {
    const Type from = x.type();
    if (!from.is_float() || !to.is_float()) throw std::invalid_argument(name + " casts between floating-point types");
    if (name == "arith.extf" ? from.bit_width() >= to.bit_width() : from.bit_width() <= to.bit_width())
      throw std::invalid_argument(name + ": " + from.str() + " to " + to.str() + " is not " + (name == "arith.extf" ? "a widening" : "a narrowing"));
    Operation* op = ctx->new_op(name);
    op->operands = {x};
    Value r = ctx->add_result(op, to);
    insert(op);
    return r;
  }
};

static Type parse_dtype(const std::string& dtype) {
  // the reference accepts e4m3fn, e5m2, fp16, fp32, fp64 (ffi/ir.cpp:411-423); bf16, int8 and
  // int32 are added because the GEMM path computes in them
  if (dtype == "e4m3fn") return Type::scalar(TypeKind::F8E4M3FN);
  if (dtype == "e5m2") return Type::scalar(TypeKind::F8E5M2);
  if (dtype == "fp16") return Type::scalar(TypeKind::F16);
  if (dtype == "bf16") return Type::scalar(TypeKind::BF16);
  if (dtype == "fp32") return Type::scalar(TypeKind::F32);
  if (dtype == "fp64") return Type::scalar(TypeKind::F64);
  if (dtype == "int8") return Type::scalar(TypeKind::I8);
  if (dtype == "int32") return Type::scalar(TypeKind::I32);
  throw std::invalid_argument("invalid float type");
}

static Block* add_body_block(Context* ctx, Operation* op, const std::vector<Type>& arg_types) {
  Region* rg = op->regions[0];
  if (!rg->blocks.empty()) throw std::invalid_argument("entry block already exists");
  Block* b = ctx->new_block();
  b->parent = rg;
  rg->blocks.push_back(b);
  for (auto& t : arg_types) ctx->add_block_arg(b, t);
  Operation* end = ctx->new_op("frisk.end");
  end->block = b;
  b->ops.push_back(end);
  return b;
}

static void print_diagnostics(const Diagnostics& d) {
  for (auto& e : d.errors) std::cerr << "error: " << e << "\n";
}

template <class OpClass> static void def_common(py::class_<OpClass, OpState>&) {}

// an affine expression typed by its kind, as the reference's dyn_casts return (ffi/ir.cpp:811-858)
struct AffineBinaryOpExpr : AffineExpr { explicit AffineBinaryOpExpr(const AffineExpr& e) : AffineExpr(e) {} };
struct AffineDimExpr : AffineExpr { explicit AffineDimExpr(const AffineExpr& e) : AffineExpr(e) {} };
struct AffineSymbolExpr : AffineExpr { explicit AffineSymbolExpr(const AffineExpr& e) : AffineExpr(e) {} };
struct AffineConstantExpr : AffineExpr { explicit AffineConstantExpr(const AffineExpr& e) : AffineExpr(e) {} };

void init_ffi_ir(py::module_&& m) {
  // ---------------------------------------------------------------- context, types, values (ffi/ir.cpp:883-1078)
  py::class_<PyContext>(m, "context", py::module_local())
      .def(py::init<>())
      .def("disable_multithreading", [](PyContext& self) { self.ctx->multithreading = false; });

  py::enum_<MemorySpace>(m, "MemorySpace", py::arithmetic())  // ffi/ir.cpp:137-141
      .value("GLOBAL", MemorySpace::Global)
      .value("SHARED", MemorySpace::Shared)
      .value("LOCAL", MemorySpace::Local)
      .export_values();

  // ---------------------------------------------------------------- affine expressions and maps (ffi/ir.cpp:646-881)
  py::enum_<ExprKind>(m, "AffineExprKind", py::module_local())  // values and order of mlir::AffineExprKind
      .value("Add", ExprKind::Add)
      .value("Mul", ExprKind::Mul)
      .value("Mod", ExprKind::Mod)
      .value("FloorDiv", ExprKind::FloorDiv)
      .value("CeilDiv", ExprKind::CeilDiv)
      .value("LAST_AFFINE_BINARY_OP", ExprKind::CeilDiv)
      .value("Constant", ExprKind::Constant)
      .value("DimId", ExprKind::DimId)
      .value("SymbolId", ExprKind::SymbolId)
      .export_values();

  auto require_binary_kind = [](ExprKind k) {
    if ((int)k < 0 || (int)k > (int)ExprKind::CeilDiv) throw std::invalid_argument("not a binary affine expression kind");
  };

  py::class_<AffineExpr>(m, "AffineExpr", py::module_local())  // ffi/ir.cpp:760-858
      .def(py::init<>())
      .def("__eq__", [](const AffineExpr& a, const AffineExpr& b) { return a.equals(b); })
      .def("__eq__", [](const AffineExpr& a, int64_t v) { return a.is_constant() && a.constant_value() == v; })
      .def("__ne__", [](const AffineExpr& a, const AffineExpr& b) { return !a.equals(b); })
      .def("__ne__", [](const AffineExpr& a, int64_t v) { return !(a.is_constant() && a.constant_value() == v); })
      .def("__bool__", [](const AffineExpr& a) { return (bool)a; })
      .def("__nonzero__", [](const AffineExpr& a) { return (bool)a; })
      .def("__hash__", [](const AffineExpr& a) { return std::hash<std::string>()(a.str()); })
      .def("__str__", [](const AffineExpr& a) { return a.str(); })
      .def("__repr__", [](const AffineExpr& a) { return "AffineExpr(" + a.str() + ")"; })
      .def("get_kind", [](const AffineExpr& a) { return a.kind(); })
      .def("is_symbolic_or_constant", &AffineExpr::is_symbolic_or_constant)
      .def("is_pure_affine", &AffineExpr::is_pure_affine)
      .def("get_largest_known_divisor", &AffineExpr::largest_known_divisor)
      .def("is_multiple_of", &AffineExpr::is_multiple_of)
      .def("is_function_of_dim", [](const AffineExpr& a, unsigned p) { return a.is_function_of(ExprKind::DimId, p); })
      .def("is_function_of_symbol", [](const AffineExpr& a, unsigned p) { return a.is_function_of(ExprKind::SymbolId, p); })
      .def("replace_dims_and_symbols", &AffineExpr::replace_dims_and_symbols)
      .def("replace_dims", [](const AffineExpr& a, std::vector<AffineExpr> dims) { return a.replace_dims_and_symbols(dims, {}); })
      .def("replace_symbols", [](const AffineExpr& a, std::vector<AffineExpr> syms) { return a.replace_dims_and_symbols({}, syms); })
      .def("replace", &AffineExpr::replace)
      .def("replace_with_map", [](const AffineExpr& a, std::vector<std::pair<AffineExpr, AffineExpr>> pairs) {
        AffineExpr out = a;
        for (auto& p : pairs) out = out.replace(p.first, p.second);
        return out;
      })
      .def("shift_dims", [](const AffineExpr& a, unsigned, unsigned shift, unsigned offset) { return a.shift(ExprKind::DimId, shift, offset); },
           py::arg("num_dims"), py::arg("shift"), py::arg("offset") = 0)
      .def("shift_symbols", [](const AffineExpr& a, unsigned, unsigned shift, unsigned offset) { return a.shift(ExprKind::SymbolId, shift, offset); },
           py::arg("num_symbols"), py::arg("shift"), py::arg("offset") = 0)
      .def("__add__", [](const AffineExpr& a, int64_t v) { return a + v; })
      .def("__add__", [](const AffineExpr& a, const AffineExpr& b) { return a + b; })
      .def("__radd__", [](const AffineExpr& a, int64_t v) { return a + v; })
      .def("__neg__", [](const AffineExpr& a) { return -a; })
      .def("__sub__", [](const AffineExpr& a, int64_t v) { return a - v; })
      .def("__sub__", [](const AffineExpr& a, const AffineExpr& b) { return a - b; })
      .def("__rsub__", [](const AffineExpr& a, int64_t v) { return AffineExpr::constant(v) - a; })
      .def("__mul__", [](const AffineExpr& a, int64_t v) { return a * v; })
      .def("__mul__", [](const AffineExpr& a, const AffineExpr& b) { return a * b; })
      .def("__rmul__", [](const AffineExpr& a, int64_t v) { return a * v; })
      .def("floor_div", [](const AffineExpr& a, int64_t v) { return a.floor_div(AffineExpr::constant(v)); })
      .def("floor_div", [](const AffineExpr& a, const AffineExpr& b) { return a.floor_div(b); })
      .def("ceil_div", [](const AffineExpr& a, int64_t v) { return a.ceil_div(AffineExpr::constant(v)); })
      .def("ceil_div", [](const AffineExpr& a, const AffineExpr& b) { return a.ceil_div(b); })
      .def("__mod__", [](const AffineExpr& a, int64_t v) { return a.mod(AffineExpr::constant(v)); })
      .def("__mod__", [](const AffineExpr& a, const AffineExpr& b) { return a.mod(b); })
      .def("__floordiv__", [](const AffineExpr& a, int64_t v) { return a.floor_div(AffineExpr::constant(v)); })  // not in the reference: `//` for floor_div
      .def("__floordiv__", [](const AffineExpr& a, const AffineExpr& b) { return a.floor_div(b); })
      .def("compose", [](const AffineExpr& a, const AffineMap& map) {  // dims of the expression := results of the map
        return a.replace_dims_and_symbols(map.impl ? map.impl->results : std::vector<AffineExpr>(), {});
      })
      // the dyn_casts of the reference: the same expression typed by its kind, or None
      .def("as_binary", [](const AffineExpr& a) -> py::object { return a.is_binary() ? py::cast(AffineBinaryOpExpr(a)) : py::none(); })
      .def("as_dim", [](const AffineExpr& a) -> py::object { return a.kind() == ExprKind::DimId ? py::cast(AffineDimExpr(a)) : py::none(); })
      .def("as_symbol", [](const AffineExpr& a) -> py::object { return a.kind() == ExprKind::SymbolId ? py::cast(AffineSymbolExpr(a)) : py::none(); })
      .def("as_constant", [](const AffineExpr& a) -> py::object { return a.is_constant() ? py::cast(AffineConstantExpr(a)) : py::none(); })
      .def("evaluate", [](const AffineExpr& a, std::vector<int64_t> dims, std::vector<int64_t> syms) { return a.eval(dims, syms); },
           py::arg("dims"), py::arg("symbols") = std::vector<int64_t>());

  py::class_<AffineBinaryOpExpr, AffineExpr>(m, "AffineBinaryOpExpr", py::module_local())
      .def("get_lhs", [](const AffineBinaryOpExpr& a) { return a.lhs(); })
      .def("get_rhs", [](const AffineBinaryOpExpr& a) { return a.rhs(); });
  py::class_<AffineDimExpr, AffineExpr>(m, "AffineDimExpr", py::module_local()).def("get_position", [](const AffineDimExpr& a) { return a.impl->value; });
  py::class_<AffineSymbolExpr, AffineExpr>(m, "AffineSymbolExpr", py::module_local()).def("get_position", [](const AffineSymbolExpr& a) { return a.impl->value; });
  py::class_<AffineConstantExpr, AffineExpr>(m, "AffineConstantExpr", py::module_local()).def("get_value", [](const AffineConstantExpr& a) { return a.impl->value; });

  m.def("get_affine_dim_expr", [](unsigned p, PyContext*) { return AffineExpr::dim(p); }, py::arg("position"), py::arg("context") = nullptr);
  m.def("get_affine_symbol_expr", [](unsigned p, PyContext*) { return AffineExpr::symbol(p); }, py::arg("position"), py::arg("context") = nullptr);
  m.def("get_affine_constant_expr", [](int64_t v, PyContext*) { return AffineExpr::constant(v); }, py::arg("constant"), py::arg("context") = nullptr);
  m.def("get_affine_constant_exprs", [](std::vector<int64_t> vs, PyContext*) {
    std::vector<AffineExpr> out;
    for (int64_t v : vs) out.push_back(AffineExpr::constant(v));
    return out;
  }, py::arg("constants"), py::arg("context") = nullptr);
  m.def("get_affine_binary_op_expr", [require_binary_kind](ExprKind k, AffineExpr l, AffineExpr r) { require_binary_kind(k); return AffineExpr::binary(k, l, r); });
  // sum over dims, then symbols, of coefficient * variable, plus the trailing constant (local expressions are not supported)
  m.def("get_affine_expr_from_flat_form", [](std::vector<int64_t> flat, unsigned num_dims, unsigned num_symbols, std::vector<AffineExpr> locals, PyContext*) {
    if (flat.size() != (size_t)num_dims + num_symbols + locals.size() + 1) throw std::invalid_argument("flat form must hold one coefficient per dim, symbol and local, and a constant");
    AffineExpr e = AffineExpr::constant(0);
    for (unsigned i = 0; i < num_dims + num_symbols + locals.size(); ++i) {
      if (flat[i] == 0) continue;
      AffineExpr v = i < num_dims ? AffineExpr::dim(i) : (i < num_dims + num_symbols ? AffineExpr::symbol(i - num_dims) : locals[i - num_dims - num_symbols]);
      e = e + v * flat[i];
    }
    return e + flat.back();
  }, py::arg("flat_exprs"), py::arg("num_dims"), py::arg("num_symbols"), py::arg("local_exprs") = std::vector<AffineExpr>(), py::arg("context") = nullptr);
  m.def("simplify_affine_expr", [](const AffineExpr& e, unsigned, unsigned) { return e.simplified(); }, py::arg("expr"), py::arg("num_dims") = 0,
        py::arg("num_symbols") = 0);

  py::class_<AffineMap>(m, "AffineMap", py::module_local())  // ffi/ir.cpp:646-757
      .def(py::init<>())
      .def_static("get", [](PyContext*) { return AffineMap(0, 0, {}); })
      .def_static("get", [](unsigned dims, unsigned syms, PyContext*) { return AffineMap((int)dims, (int)syms, {}); })
      .def_static("get", [](unsigned dims, unsigned syms, AffineExpr result) { return AffineMap((int)dims, (int)syms, {result}); })
      .def_static("get", [](unsigned dims, unsigned syms, std::vector<AffineExpr> results, PyContext*) { return AffineMap((int)dims, (int)syms, results); },
                  py::arg("dim_count"), py::arg("symbol_count"), py::arg("results"), py::arg("context") = nullptr)
      .def_static("get_constant_map", [](int64_t v, PyContext*) { return AffineMap(0, 0, {AffineExpr::constant(v)}); }, py::arg("value"),
                  py::arg("context") = nullptr)
      .def_static("get_multi_dim_identity_map", [](unsigned n, PyContext*) { return AffineMap::identity((int)n); }, py::arg("num_dims"),
                  py::arg("context") = nullptr)
      .def_static("get_multi_dim_map_with_targets", [](unsigned n, PyContext*) { return AffineMap::identity((int)n); }, py::arg("num_dims"),
                  py::arg("context") = nullptr)
      .def_static("get_minor_identity_map", [](unsigned dims, unsigned results, PyContext*) {
        if (results > dims) throw std::invalid_argument("a minor identity map cannot have more results than dims");
        std::vector<AffineExpr> r;
        for (unsigned i = dims - results; i < dims; ++i) r.push_back(AffineExpr::dim(i));
        return AffineMap((int)dims, 0, r);
      }, py::arg("dims"), py::arg("results"), py::arg("context") = nullptr)
      .def_static("get_permutation_map", [](std::vector<int64_t> perm, PyContext*) {
        std::vector<bool> seen(perm.size(), false);
        std::vector<AffineExpr> r;
        for (int64_t p : perm) {
          if (p < 0 || (size_t)p >= perm.size() || seen[(size_t)p]) throw std::invalid_argument("not a permutation");
          seen[(size_t)p] = true;
          r.push_back(AffineExpr::dim(p));
        }
        return AffineMap((int)perm.size(), 0, r);
      }, py::arg("permutation"), py::arg("context") = nullptr)
      .def("__eq__", [](const AffineMap& a, const AffineMap& b) { return a.equals(b); })
      .def("__ne__", [](const AffineMap& a, const AffineMap& b) { return !a.equals(b); })
      .def("__bool__", [](const AffineMap& a) { return (bool)a; })
      .def("__nonzero__", [](const AffineMap& a) { return (bool)a; })
      .def("__str__", [](const AffineMap& a) { return a.str(); })
      .def("__repr__", [](const AffineMap& a) { return "AffineMap(" + a.str() + ")"; })
      .def("get_num_dims", &AffineMap::num_dims)
      .def("get_num_symbols", &AffineMap::num_symbols)
      .def("get_num_results", &AffineMap::num_results)
      .def("get_num_inputs", &AffineMap::num_inputs)
      .def("get_results", [](const AffineMap& a) { return a.impl ? a.impl->results : std::vector<AffineExpr>(); })
      .def("get_result", [](const AffineMap& a, unsigned i) { return a.impl->results.at(i); })
      .def("is_identity", &AffineMap::is_identity)
      .def("is_symbol_identity", [](const AffineMap& a) {
        if (!a.impl || a.num_symbols() != a.num_results()) return false;
        for (int i = 0; i < a.num_results(); ++i)
          if (a.impl->results[(size_t)i].kind() != ExprKind::SymbolId || a.impl->results[(size_t)i].impl->value != i) return false;
        return true;
      })
      .def("is_minor_identity", [](const AffineMap& a) {
        if (!a.impl || a.num_symbols() || a.num_results() > a.num_dims()) return false;
        int first = a.num_dims() - a.num_results();
        for (int i = 0; i < a.num_results(); ++i)
          if (a.impl->results[(size_t)i].kind() != ExprKind::DimId || a.impl->results[(size_t)i].impl->value != first + i) return false;
        return true;
      })
      .def("is_empty", [](const AffineMap& a) { return a.num_dims() == 0 && a.num_symbols() == 0 && a.num_results() == 0; })
      .def("is_single_constant", [](const AffineMap& a) { return a.num_results() == 1 && a.impl->results[0].is_constant(); })
      .def("is_constant", [](const AffineMap& a) {
        if (!a.impl) return false;
        for (auto& e : a.impl->results) if (!e.is_constant()) return false;
        return true;
      })
      .def("is_permutation", [](const AffineMap& a) { return a.num_dims() == a.num_results() && a.is_projected_permutation(false); })
      .def("is_projected_permutation", &AffineMap::is_projected_permutation, py::arg("allow_zero_in_results") = false)
      .def("get_single_constant_result", [](const AffineMap& a) {
        if (a.num_results() != 1 || !a.impl->results[0].is_constant()) throw std::invalid_argument("map does not have a single constant result");
        return a.impl->results[0].constant_value();
      })
      .def("get_constant_results", [](const AffineMap& a) {
        std::vector<int64_t> out;
        if (a.impl) for (auto& e : a.impl->results) {
          if (!e.is_constant()) throw std::invalid_argument("map has a non-constant result");
          out.push_back(e.constant_value());
        }
        return out;
      })
      .def("get_dim_position", [](const AffineMap& a, unsigned idx) {
        const AffineExpr& e = a.impl->results.at(idx);
        if (e.kind() != ExprKind::DimId) throw std::invalid_argument("result is not a dimension");
        return e.impl->value;
      }, py::arg("idx"))
      .def("get_result_position", [](const AffineMap& a, const AffineExpr& input) -> py::object {
        if (input.kind() != ExprKind::DimId || !a.impl) return py::none();
        for (size_t i = 0; i < a.impl->results.size(); ++i)
          if (a.impl->results[i].equals(input)) return py::cast((unsigned)i);
        return py::none();
      }, py::arg("input"));

  py::class_<Type>(m, "type", py::module_local())  // ffi/ir.cpp:888-937
      .def("__str__", [](const Type& t) { return t.str(); })
      .def("__repr__", [](const Type& t) { return t.str(); })
      .def("__eq__", [](const Type& a, const Type& b) { return a.equals(b); })
      .def("is_f16", [](const Type& t) { return t.kind() == TypeKind::F16; })
      .def("is_bf16", [](const Type& t) { return t.kind() == TypeKind::BF16; })
      .def("is_f32", [](const Type& t) { return t.kind() == TypeKind::F32; })
      .def("is_f64", [](const Type& t) { return t.kind() == TypeKind::F64; })
      .def("is_float", &Type::is_float)
      .def("is_index", [](const Type& t) { return t.kind() == TypeKind::Index; })
      .def("is_int", &Type::is_int)
      .def("get_rank", [](const Type& t) { return (int64_t)t.impl->shape.size(); })
      .def("get_dim_size", [](const Type& t, unsigned i) { return t.impl->shape.at(i); })
      .def("get_elem_width", [](const Type& t) { return t.element().bit_width(); })
      .def("get_shape", [](const Type& t) { return t.impl->shape; })
      .def("get_element_ty", [](const Type& t) { return t.element(); })
      .def("get_memory_space", [](const Type& t) -> std::optional<MemorySpace> {
        if (!t.is_memref()) return std::nullopt;
        return (MemorySpace)t.impl->memory_space;
      })
      .def("get_layout_map", [](const Type& t) { return t.impl->layout ? t.impl->layout : AffineMap::identity((int)t.impl->shape.size()); })
      .def("param_types", [](const Type& t) {
        std::vector<Type> out;
        for (auto& i : t.impl->inputs) out.push_back(Type(i));
        return out;
      });
  m.attr("memref_buffer") = m.attr("type");
  m.attr("function_type") = m.attr("type");
  m.attr("ranked_tensor") = m.attr("type");

  py::class_<Value>(m, "value", py::module_local())  // ffi/ir.cpp:949-975
      .def("get_type", &Value::type)
      .def("id", [](const Value& v) { return (uint64_t)(uintptr_t)v.impl; })
      .def("__eq__", [](const Value& a, const Value& b) { return a == b; })
      .def("__hash__", [](const Value& v) { return (size_t)(uintptr_t)v.impl; })
      .def("__repr__", [](const Value& v) { return "<value of type " + v.type().str() + ">"; })
      .def("__str__", [](const Value& v) { return "<value of type " + v.type().str() + ">"; });
  m.attr("block_argument") = m.attr("value");
  m.attr("op_result") = m.attr("value");

  py::class_<PyRegion>(m, "region", py::module_local())
      .def("size", [](PyRegion& r) { return r.region->blocks.size(); })
      .def("empty", [](PyRegion& r) { return r.region->blocks.empty(); })
      .def("push_back", [](PyRegion& r, PyBlock& b) { b.block->parent = r.region; r.region->blocks.push_back(b.block); })
      .def("id", [](PyRegion& r) { return (uint64_t)(uintptr_t)r.region; });

  py::class_<PyBlock>(m, "block", py::module_local())  // ffi/ir.cpp:1021-1073
      .def("arg", [](PyBlock& b, unsigned i) {
        if (i >= b.block->args.size()) throw py::index_error("Block argument index out of range");
        return Value{b.block->args[i]};
      })
      .def("get_argument", [](PyBlock& b, unsigned i) {
        if (i >= b.block->args.size()) throw py::index_error("Block argument index out of range");
        return Value{b.block->args[i]};
      })
      .def("add_argument", [](PyBlock& b, Type t) { return b.ctx->add_block_arg(b.block, t); })
      .def("get_num_arguments", [](PyBlock& b) { return b.block->args.size(); })
      .def("has_terminator", [](PyBlock& b) { return b.block->has_terminator(); })
      .def("get_num_operations", [](PyBlock& b) { return b.block->ops.size(); })
      .def("id", [](PyBlock& b) { return (uint64_t)(uintptr_t)b.block; });

  // ---------------------------------------------------------------- op handles (ffi/ir.cpp:476-644, 33-130)
  py::class_<OpState>(m, "OpState", py::module_local())
      .def("get_num_results", [](OpState& s) { return s.op->results.size(); })
      .def("get_result", [](OpState& s, unsigned i) {
        if (i >= s.op->results.size()) throw py::index_error("Op result index out of range");
        return Value{s.op->results[i]};
      })
      .def("get_region", [](OpState& s, unsigned i) {
        if (i >= s.op->regions.size()) throw py::index_error("Op region index out of range");
        return PyRegion{s.op->regions[i], s.ctx};
      })
      .def("get_name", [](OpState& s) { return s.op->name; })
      .def("set_attr", [](OpState& s, const std::string& name, py::object v) {
        if (py::isinstance<py::bool_>(v)) s.op->attrs[name] = Attribute::boolean(v.cast<bool>());
        else if (py::isinstance<py::int_>(v)) s.op->attrs[name] = Attribute::integer(v.cast<int64_t>());
        else if (py::isinstance<py::str>(v)) s.op->attrs[name] = Attribute::string(v.cast<std::string>());
        else throw std::invalid_argument("set_attr takes a bool, an int or a str");
      })
      .def("get_str_attr", [](OpState& s, const std::string& name) -> py::object {
        auto a = s.op->attr(name);
        if (!a || a->kind != Attribute::String) return py::none();
        return py::str(a->s);
      })
      .def("dump", [](OpState& s) { std::cerr << print_operation(s.op) << std::endl; })
      .def("__str__", [](OpState& s) { return print_operation(s.op); })
      .def("verify", [](OpState& s) {  // failures are reported on stderr, not raised (ffi/ir.cpp:595)
        Diagnostics d;
        bool ok = verify_operation(s.op, d);
        print_diagnostics(d);
        return ok;
      });

  py::class_<ModuleOp, OpState>(m, "module", py::module_local(), py::dynamic_attr())
      .def("dump", [](ModuleOp& s, const std::string& log) {
        if (!log.empty()) std::cout << log << "\n";
        std::cout << print_operation(s.op) << std::endl;
      }, py::arg("log") = "")
      .def("push_back", [](ModuleOp& s, KernelOp& k) {
        Block* body = s.op->regions[0]->blocks[0];
        if (k.op->block) throw std::invalid_argument("kernel is already in a module");
        k.op->block = body;
        body->ops.push_back(k.op);
      })
      .def("get_kernel", [](ModuleOp& s, const std::string& name) -> py::object {
        for (Operation* op : s.op->regions[0]->blocks[0]->ops)
          if (op->name == "frisk.kernel" && op->attr("sym_name")->s == name) { KernelOp k; k.op = op; k.ctx = s.ctx; return py::cast(k); }
        return py::none();
      }, py::keep_alive<0, 1>())  // the kernel handle keeps the module object (and through its `context` attribute the IR) alive
      .def("has_kernel", [](ModuleOp& s, const std::string& name) {
        for (Operation* op : s.op->regions[0]->blocks[0]->ops)
          if (op->name == "frisk.kernel" && op->attr("sym_name")->s == name) return true;
        return false;
      });

  py::class_<GemmOp, OpState>(m, "GemmOp", py::module_local())
      .def("get_matrix_A", [](GemmOp& s) { return s.op->operands[0]; })
      .def("get_matrix_B", [](GemmOp& s) { return s.op->operands[1]; })
      .def("get_matrix_C", [](GemmOp& s) { return s.op->operands[2]; })
      .def("get_all_matrix", [](GemmOp& s) { return s.op->operands; })
      .def("get_m", [](GemmOp& s) { return s.op->int_attr("M"); })
      .def("get_n", [](GemmOp& s) { return s.op->int_attr("N"); })
      .def("get_k", [](GemmOp& s) { return s.op->int_attr("K"); });
  py::class_<KernelOp, OpState>(m, "KernelOp", py::module_local())
      .def("arg", [](KernelOp& s, unsigned i) {
        if (s.op->regions[0]->blocks.empty() || i >= s.op->regions[0]->blocks[0]->args.size()) throw py::index_error("Kernel argument index out of range");
        return Value{s.op->regions[0]->blocks[0]->args[i]};
      })
      .def("get_num_arguments", [](KernelOp& s) { return s.op->attr("function_type")->type.impl->inputs.size(); })
      .def("add_entry_block", [](KernelOp& s) {  // block arguments of the kernel type + frisk.end (FriskOps.td:56-73)
        std::vector<Type> types;
        for (auto& t : s.op->attr("function_type")->type.impl->inputs) types.push_back(Type(t));
        return PyBlock{add_body_block(s.ctx, s.op, types), s.ctx};
      })
      .def_property_readonly("type", [](KernelOp& s) { return s.op->attr("function_type")->type; });
  py::class_<ParallelOp, OpState>(m, "ParallelOp", py::module_local())
      .def("get_ivs", [](ParallelOp& s) {
        std::vector<Value> v;
        if (!s.op->regions[0]->blocks.empty()) for (auto* a : s.op->regions[0]->blocks[0]->args) v.push_back(Value{a});
        return v;
      })
      .def("get_grid", [](ParallelOp& s) { return s.op->attr("ranges")->ints; })
      .def("get_thread_num", [](ParallelOp& s) { return s.op->int_attr("threads"); })
      .def("get_grid_dim", [](ParallelOp& s) { return s.op->attr("ranges")->ints.size(); })
      .def("add_entry_block", [](ParallelOp& s) {  // one index argument per grid dimension + frisk.end (FriskOps.td:119-132)
        std::vector<Type> types(s.op->attr("ranges")->ints.size(), Type::scalar(TypeKind::Index));
        return PyBlock{add_body_block(s.ctx, s.op, types), s.ctx};
      });
  py::class_<BlockOp, OpState>(m, "BlockOp", py::module_local())
      .def("get_ivs", [](BlockOp& s) {
        std::vector<Value> v;
        for (auto* a : s.op->regions[0]->blocks[0]->args) v.push_back(Value{a});
        return v;
      })
      .def("get_block_ranges", [](BlockOp& s) { return s.op->attr("ranges")->ints; })
      .def("get_block_dim", [](BlockOp& s) { return s.op->attr("ranges")->ints.size(); });
  py::class_<ForOp, OpState>(m, "ForOp", py::module_local())
      .def("get_induction_var", [](ForOp& s) { return Value{s.op->regions[0]->blocks[0]->args[0]}; })
      .def("get_lower_bound", [](ForOp& s) { return s.op->int_attr("lower"); })
      .def("get_upper_bound", [](ForOp& s) { return s.op->int_attr("upper"); })
      .def("get_step", [](ForOp& s) { return s.op->int_attr("step"); });
  py::class_<AllocBufferOp, OpState>(m, "AllocBufferOp", py::module_local())
      .def("get_alignment", [](AllocBufferOp& s) { return s.op->int_attr("alignment"); })
      .def("get_memroy_space", [](AllocBufferOp& s) { return (MemorySpace)s.op->int_attr("memory_space"); })
      .def("get_result", [](AllocBufferOp& s) { return Value{s.op->results[0]}; })
      .def("get_memref_ty", [](AllocBufferOp& s) { return s.op->results[0]->type; });
  py::class_<CopyOp, OpState>(m, "CopyOp", py::module_local())
      .def("get_src_affine_map", [](CopyOp& s) { return s.op->attr("srcMap")->map; })
      .def("get_dst_affine_map", [](CopyOp& s) { return s.op->attr("dstMap")->map; })
      .def("get_src_memref", [](CopyOp& s) { return s.op->operands[0]; })
      .def("get_dst_memref", [](CopyOp& s) { return s.op->operands[1]; })
      .def("get_src_indices", [](CopyOp& s) { return std::vector<Value>(s.op->operands.begin() + 2, s.op->operands.begin() + 2 + s.op->src_index_count); })
      .def("get_dst_indices", [](CopyOp& s) { return std::vector<Value>(s.op->operands.begin() + 2 + s.op->src_index_count, s.op->operands.end()); })
      .def("get_src_extents", [](CopyOp& s) { return s.op->attr("srcExtents")->ints; })
      .def("get_dst_extents", [](CopyOp& s) { return s.op->attr("dstExtents")->ints; });
  py::class_<FillOp, OpState>(m, "FillOp", py::module_local()).def("get_memref", [](FillOp& s) { return s.op->operands[0]; });
  py::class_<ReduceOp, OpState>(m, "ReduceOp", py::module_local())
      .def("get_src_memref", [](ReduceOp& s) { return s.op->operands[0]; })
      .def("get_dst_memref", [](ReduceOp& s) { return s.op->operands[1]; })
      .def("get_reduce_dim", [](ReduceOp& s) { return s.op->int_attr("dim"); });

  // Text -> module: what mlir::parseSourceString gives a user of the reference's dialect; the grammar is the printed
  // form (ir_parser.h).  The returned module carries the context as its `context` attribute, which keeps the IR alive.
  m.def("parse_module", [](PyContext& c, const std::string& text) {
    ModuleOp mo;
    mo.op = parse_module_text(*c.ctx, text);
    mo.ctx = c.ctx.get();
    py::object o = py::cast(mo);
    o.attr("context") = py::cast(c);
    return o;
  }, py::arg("context"), py::arg("text"), "parses the textual form of a module of frisk kernels; ValueError with line and column on a syntax error");

  // ---------------------------------------------------------------- builder (ffi/ir.cpp:144-471)
  py::class_<Builder>(m, "builder")
      .def(py::init<PyContext&>())
      .def("create_module", [](Builder& b) {
        Operation* op = b.ctx->new_op("builtin.module");
        Region* rg = b.ctx->new_region(op);
        Block* body = b.ctx->new_block();
        body->parent = rg;
        rg->blocks.push_back(body);
        return b.wrap<ModuleOp>(op);
      })
      .def("set_insertion_point_to_start", [](Builder& b, PyBlock& blk) { b.set_to_start(blk.block); })
      .def("set_insertion_point_to_end", [](Builder& b, PyBlock& blk) { b.set_to_end(blk.block); })
      .def("set_insertion_point_after", [](Builder& b, OpState& op) { b.set_after(op.op); })
      .def("get_insertion_block", [](Builder& b) -> py::object {
        if (!b.block) return py::none();
        return py::cast(PyBlock{b.block, b.ctx});
      })
      .def("new_block", [](Builder& b) { return PyBlock{b.ctx->new_block(), b.ctx}; })
      .def("get_bool_ty", [](Builder&) { return Type::scalar(TypeKind::I8); })
      .def("get_int8_ty", [](Builder&) { return Type::scalar(TypeKind::I8); })
      .def("get_int32_ty", [](Builder&) { return Type::scalar(TypeKind::I32); })
      .def("get_int64_ty", [](Builder&) { return Type::scalar(TypeKind::I64); })
      .def("get_index_ty", [](Builder&) { return Type::scalar(TypeKind::Index); })
      .def("get_f64_ty", [](Builder&) { return Type::scalar(TypeKind::F64); })
      .def("get_f32_ty", [](Builder&) { return Type::scalar(TypeKind::F32); })
      .def("get_f16_ty", [](Builder&) { return Type::scalar(TypeKind::F16); })
      .def("get_bf16_ty", [](Builder&) { return Type::scalar(TypeKind::BF16); })
      .def("get_f8e4m3fn_ty", [](Builder&) { return Type::scalar(TypeKind::F8E4M3FN); })
      .def("get_memref_ty", [](Builder&, Type elem, std::vector<int64_t> shape, AffineMap map, MemorySpace space) {
        return Type::memref(shape, elem, map, (int)space);
      }, py::arg("elementType"), py::arg("shape"), py::arg("map") = AffineMap(), py::arg("space") = MemorySpace::Global)
      .def("get_function_ty", [](Builder&, std::vector<Type> in, std::vector<Type> out) { return Type::function(in, out); })
      .def("get_kernel_ty", [](Builder&, std::vector<Type> in) { return Type::function(in, {}); })
      .def("get_affine_dim_expr", [](Builder&, unsigned p) { return AffineExpr::dim(p); })
      .def("get_affine_symbol_expr", [](Builder&, unsigned p) { return AffineExpr::symbol(p); })
      .def("get_affine_constant_expr", [](Builder&, int64_t v) { return AffineExpr::constant(v); })
      .def("get_multi_dim_identity_map", [](Builder&, unsigned n) { return AffineMap::identity((int)n); })
      // ---- frisk ops
      .def("create_gemm_op", [](Builder& b, Value& A, Value& B, Value& C, bool transA, bool transB, bool clearAccum) {
        auto require_memref = [](Value& v, const char* name) -> const TypeImpl* {
          if (!v.type().is_memref()) throw std::invalid_argument(std::string("create_gemm_op expects memref for operand ") + name);
          return v.type().impl.get();
        };
        auto require_static = [](int64_t dim, const char* desc) -> int64_t {
          if (dim < 0) throw std::invalid_argument(std::string("create_gemm_op requires static ") + desc);
          return dim;
        };
        const TypeImpl *a = require_memref(A, "A"), *bt = require_memref(B, "B"), *c = require_memref(C, "C");
        if (a->shape.size() != 2 || bt->shape.size() != 2 || c->shape.size() != 2) throw std::invalid_argument("create_gemm_op expects rank-2 memrefs");
        // The reference reads A as [M][K] and B as [K][N] whatever the flags say (ffi/ir.cpp:346-355, GemmOp::verify
        // FriskOps.cpp:1264-1283); its flags only pick the shared-memory layout (FriskOps.cpp:1359, 1376).  A path that
        // executes the GEMM needs operands that really are stored transposed (B as [N][K]), so here a set flag first
        // means "stored transposed" ([K][M] for A, [N][K] for B).  When the shapes do not fit that reading but fit the
        // reference's, the reference's is taken: the flag is then a layout hint without effect on the arithmetic.
        for (int d = 0; d < 2; ++d) {
          require_static(a->shape[(size_t)d], d == 0 ? "M dimension of A" : "K dimension of A");
          require_static(bt->shape[(size_t)d], d == 0 ? "K dimension of B" : "N dimension of B");
          require_static(c->shape[(size_t)d], d == 0 ? "M dimension of C" : "N dimension of C");
        }
        const int64_t cm = c->shape[0], cn = c->shape[1];
        int64_t mm = 0, n = 0, k = 0;
        auto reading = [&](bool ta, bool tb) {
          mm = a->shape[ta ? 1 : 0]; k = a->shape[ta ? 0 : 1];
          n = bt->shape[tb ? 0 : 1];
          return k == bt->shape[tb ? 1 : 0] && mm == cm && n == cn;
        };
        if (!reading(transA, transB) && !((transA || transB) && reading(false, false))) {
          reading(transA, transB);
          if (k != bt->shape[transB ? 1 : 0]) throw std::invalid_argument("create_gemm_op expects A and B inner dimensions to match");
          throw std::invalid_argument("create_gemm_op expects C shape to match A/B product");
        }
        Type ea(a->element), eb(bt->element), ec(c->element);
        // same element type for all three as in the reference (ffi/ir.cpp:357-359), or C in the accumulator
        // type of the inputs (f32 for floating inputs, i32 for i8), which the MFMA path needs
        bool acc_ok = (ea.is_float() && ec.kind() == TypeKind::F32) || (ea.kind() == TypeKind::I8 && ec.kind() == TypeKind::I32);
        if (!ea.equals(eb) || !(ea.equals(ec) || acc_ok)) throw std::invalid_argument("create_gemm_op expects operands to have matching element types");
        Operation* op = b.ctx->new_op("frisk.gemm");
        op->operands = {A, B, C};
        op->attrs["transA"] = Attribute::boolean(transA);
        op->attrs["transB"] = Attribute::boolean(transB);
        op->attrs["M"] = Attribute::integer(mm);
        op->attrs["N"] = Attribute::integer(n);
        op->attrs["K"] = Attribute::integer(k);
        op->attrs["policy"] = Attribute::policy(GemmWarpPolicy::Square);
        op->attrs["clear_accum"] = Attribute::boolean(clearAccum);
        b.insert(op);
        return b.wrap<GemmOp>(op);
      }, py::arg("A"), py::arg("B"), py::arg("C"), py::arg("transA") = false, py::arg("transB") = false, py::arg("clear_accum") = false)
      .def("create_kernel_op", [](Builder& b, ModuleOp& module, const std::string& name, Type& type) {
        for (Operation* op : module.op->regions[0]->blocks[0]->ops)
          if (op->name == "frisk.kernel" && op->attr("sym_name")->s == name) return b.wrap<KernelOp>(op);
        if (type.kind() != TypeKind::Function) throw std::invalid_argument("invalid kernel function type");
        Operation* op = b.ctx->new_op("frisk.kernel");  // created detached; the caller pushes it into the module
        op->attrs["sym_name"] = Attribute::string(name);
        op->attrs["function_type"] = Attribute::type_attr(type);
        b.ctx->new_region(op);
        return b.wrap<KernelOp>(op);
      })
      .def("create_parallel_op", [](Builder& b, std::vector<int64_t>& grid, int64_t threads) {
        // only as the first op of a block that so far holds just its terminator (ffi/ir.cpp:375-382)
        if (!b.block || b.block->ops.size() != 1) throw std::invalid_argument("invalid parallel create");
        Operation* op = b.ctx->new_op("frisk.parallel");
        op->attrs["threads"] = Attribute::integer(threads);
        op->attrs["ranges"] = Attribute::int_array(grid);
        b.ctx->new_region(op);
        b.insert(op);
        return b.wrap<ParallelOp>(op);
      })
      .def("create_block_op", [](py::object self, std::vector<int64_t>& ranges, py::function fn) {
        Builder& b = self.cast<Builder&>();
        Operation* op = b.ctx->new_op("frisk.block");
        op->attrs["ranges"] = Attribute::int_array(ranges);
        Region* rg = b.ctx->new_region(op);
        Block* body = b.ctx->new_block();
        body->parent = rg;
        rg->blocks.push_back(body);
        std::vector<Value> ivs;
        for (size_t i = 0; i < ranges.size(); ++i) ivs.push_back(b.ctx->add_block_arg(body, Type::scalar(TypeKind::Index)));
        Block* saved_block = b.block; Operation* saved_before = b.before;  // InsertionGuard (FriskOps.cpp:1097-1116)
        b.set_to_start(body);
        try { fn(self, ivs); } catch (py::error_already_set& e) {
          std::cerr << "Python exception in frisk block op: " << e.what() << "\n";
          b.block = saved_block; b.before = saved_before;
          throw;
        }
        Operation* end = b.make_end(); end->block = body; body->ops.push_back(end);
        b.block = saved_block; b.before = saved_before;
        b.insert(op);
        return b.wrap<BlockOp>(op);
      })
      .def("create_for_op", [](py::object self, int64_t lower, int64_t upper, int64_t step, py::function fn) {
        Builder& b = self.cast<Builder&>();
        Operation* op = b.ctx->new_op("frisk.for");
        op->attrs["lower"] = Attribute::integer(lower);
        op->attrs["upper"] = Attribute::integer(upper);
        op->attrs["step"] = Attribute::integer(step);
        Region* rg = b.ctx->new_region(op);
        Block* body = b.ctx->new_block();
        body->parent = rg;
        rg->blocks.push_back(body);
        Value iv = b.ctx->add_block_arg(body, Type::scalar(TypeKind::Index));
        Block* saved_block = b.block; Operation* saved_before = b.before;  // InsertionGuard (FriskOps.cpp:1198-1218)
        b.set_to_start(body);
        try { fn(self, iv); } catch (py::error_already_set& e) {
          std::cerr << "Python exception in frisk for op: " << e.what() << "\n";
          b.block = saved_block; b.before = saved_before;
          throw;
        }
        Operation* end = b.make_end(); end->block = body; body->ops.push_back(end);
        b.block = saved_block; b.before = saved_before;
        b.insert(op);
        return b.wrap<ForOp>(op);
      })
      .def("create_alloc_buffer_op", [](Builder& b, std::vector<int64_t> shape, const std::string& dtype, MemorySpace space, int64_t alignment) {
        Type elem = parse_dtype(dtype);
        if (alignment < 0) throw std::invalid_argument("alignment must be non-negative");
        Operation* op = b.ctx->new_op("frisk.alloc_buffer");
        op->attrs["shape"] = Attribute::int_array(shape);
        op->attrs["elementType"] = Attribute::type_attr(elem);
        op->attrs["alignment"] = Attribute::integer(alignment);
        op->attrs["memory_space"] = Attribute::integer((int)space);
        b.ctx->add_result(op, Type::memref(shape, elem, AffineMap(), (int)space));
        b.insert(op);
        return b.wrap<AllocBufferOp>(op);
      }, py::arg("shape"), py::arg("dtype"), py::arg("space") = MemorySpace::Global, py::arg("alignment") = 0)
      .def("create_copy_op", [](Builder& b, Value src, Value dst, std::vector<Value> srcIndices, std::vector<Value> dstIndices, AffineMap srcMap,
                                AffineMap dstMap, std::vector<int64_t> srcExtents, std::vector<int64_t> dstExtents) {
        if (!src.type().is_memref() || !dst.type().is_memref()) throw std::invalid_argument("create_copy_op expects memref operands");
        const auto& sshape = src.type().impl->shape; const auto& dshape = dst.type().impl->shape;
        bool no_maps = !srcMap && !dstMap, both_maps = srcMap && dstMap, no_ext = srcExtents.empty() && dstExtents.empty();
        bool both_ext = !srcExtents.empty() && !dstExtents.empty();
        // identity maps + extents from the destination shape, explicit maps, or explicit maps and extents;
        // the fourth form (extents with default maps) is what a tile copy with plain tile indices needs.
        // Any other mix ends the process in the reference (a bare `throw;`, ffi/ir.cpp:443-446); here it raises.
        if (!((no_maps || both_maps) && (no_ext || both_ext))) throw std::invalid_argument("copy op map error.");
        if (no_maps) { srcMap = AffineMap::identity((int)sshape.size()); dstMap = AffineMap::identity((int)dshape.size()); }
        if ((int)srcIndices.size() != srcMap.num_inputs()) throw std::invalid_argument("source map inputs must match source indices count");
        if ((int)dstIndices.size() != dstMap.num_inputs()) throw std::invalid_argument("destination map inputs must match destination indices count");
        if (no_ext) {  // destination shape, left-padded with 1s to the source rank (FriskOps.cpp:1564-1591)
          if (sshape.size() < dshape.size()) throw std::invalid_argument("src rank must be >= dst rank");
          size_t pad = sshape.size() - dshape.size();
          for (size_t i = 0; i < sshape.size(); ++i) srcExtents.push_back(i < pad ? 1 : dshape[i - pad]);
          dstExtents = dshape;
        }
        Operation* op = b.ctx->new_op("frisk.copy");
        op->operands = {src, dst};
        op->operands.insert(op->operands.end(), srcIndices.begin(), srcIndices.end());
        op->operands.insert(op->operands.end(), dstIndices.begin(), dstIndices.end());
        op->src_index_count = (int)srcIndices.size();
        op->attrs["srcMap"] = Attribute::affine_map(srcMap);
        op->attrs["dstMap"] = Attribute::affine_map(dstMap);
        op->attrs["srcExtents"] = Attribute::int_array(srcExtents);
        op->attrs["dstExtents"] = Attribute::int_array(dstExtents);
        b.insert(op);
        return b.wrap<CopyOp>(op);
      }, py::arg("src"), py::arg("dst"), py::arg("srcIndices"), py::arg("dstIndices"), py::arg("srcMap") = AffineMap(), py::arg("dstMap") = AffineMap(),
         py::arg("srcExtents") = std::vector<int64_t>(), py::arg("dstExtents") = std::vector<int64_t>())
      .def("create_fill_op", [](Builder& b, Value memref, float value, const std::string& dtype) {
        Type t = parse_dtype(dtype);
        Operation* op = b.ctx->new_op("frisk.fill");
        op->operands = {memref};
        op->attrs["value"] = Attribute::floating((double)value, t);
        b.insert(op);
        return b.wrap<FillOp>(op);
      })
      .def("create_reduce_op", [](Builder& b, Value src, Value dst, const std::string& kind, int64_t dim, bool clear) {
        Operation* op = b.ctx->new_op("frisk.reduce");
        op->operands = {src, dst};
        op->attrs["kind"] = Attribute::string(kind);
        op->attrs["dim"] = Attribute::integer(dim);
        op->attrs["clear"] = Attribute::boolean(clear);
        b.insert(op);
        return b.wrap<ReduceOp>(op);
      }, py::arg("src"), py::arg("dst"), py::arg("kind"), py::arg("dim"), py::arg("clear") = true)
      // ---- scalar values: the constants of the reference's builder (ffi/ir.cpp:178-193) ...
      .def("get_f16", [](Builder& b, float v) { return b.constant(Attribute::floating((double)v, Type::scalar(TypeKind::F16))); })
      .def("get_f32", [](Builder& b, float v) { return b.constant(Attribute::floating((double)v, Type::scalar(TypeKind::F32))); })
      .def("get_f64", [](Builder& b, double v) { return b.constant(Attribute::floating(v, Type::scalar(TypeKind::F64))); })
      .def("get_int64", [](Builder& b, int64_t v) { return b.constant(Attribute::integer(v, 64)); })
      // ... and what the bodies of frisk.block need beyond them (tmp/ir.mlir:39-47, 114-147 use affine.load / affine.store,
      // arith.mulf / subf / addf, math.exp2 / log2; the reference's builder has no creators for these)
      .def("create_load_op", [](Builder& b, Value memref, std::vector<Value> indices, AffineMap map) {
        if (!memref.type().is_memref()) throw std::invalid_argument("create_load_op expects a memref");
        if (!map) map = AffineMap::identity((int)memref.type().impl->shape.size());
        if ((int)indices.size() != map.num_inputs()) throw std::invalid_argument("create_load_op: the map takes " + std::to_string(map.num_inputs()) + " indices, got " + std::to_string(indices.size()));
        if (map.num_results() != (int)memref.type().impl->shape.size()) throw std::invalid_argument("create_load_op: the map must give one index per memref dimension");
        Operation* op = b.ctx->new_op("affine.load");
        op->operands = {memref};
        op->operands.insert(op->operands.end(), indices.begin(), indices.end());
        op->attrs["map"] = Attribute::affine_map(map);
        Value r = b.ctx->add_result(op, memref.type().element());
        b.insert(op);
        return r;
      }, py::arg("memref"), py::arg("indices"), py::arg("map") = AffineMap())
      .def("create_store_op", [](Builder& b, Value value, Value memref, std::vector<Value> indices, AffineMap map) {
        if (!memref.type().is_memref()) throw std::invalid_argument("create_store_op expects a memref");
        if (!map) map = AffineMap::identity((int)memref.type().impl->shape.size());
        if ((int)indices.size() != map.num_inputs()) throw std::invalid_argument("create_store_op: the map takes " + std::to_string(map.num_inputs()) + " indices, got " + std::to_string(indices.size()));
        if (map.num_results() != (int)memref.type().impl->shape.size()) throw std::invalid_argument("create_store_op: the map must give one index per memref dimension");
        if (!value.type().equals(memref.type().element())) throw std::invalid_argument("create_store_op: the value's type is not the memref's element type");
        Operation* op = b.ctx->new_op("affine.store");
        op->operands = {value, memref};
        op->operands.insert(op->operands.end(), indices.begin(), indices.end());
        op->attrs["map"] = Attribute::affine_map(map);
        b.insert(op);
        return OpState{op, b.ctx};
      }, py::arg("value"), py::arg("memref"), py::arg("indices"), py::arg("map") = AffineMap())
      .def("create_mulf", [](Builder& b, Value l, Value r) { return b.scalar_op("arith.mulf", {l, r}); })
      .def("create_addf", [](Builder& b, Value l, Value r) { return b.scalar_op("arith.addf", {l, r}); })
      .def("create_subf", [](Builder& b, Value l, Value r) { return b.scalar_op("arith.subf", {l, r}); })
      .def("create_divf", [](Builder& b, Value l, Value r) { return b.scalar_op("arith.divf", {l, r}); })
      .def("create_maxnumf", [](Builder& b, Value l, Value r) { return b.scalar_op("arith.maxnumf", {l, r}); })
      .def("create_minnumf", [](Builder& b, Value l, Value r) { return b.scalar_op("arith.minnumf", {l, r}); })
      .def("create_negf", [](Builder& b, Value x) { return b.scalar_op("arith.negf", {x}); })
      .def("create_exp2", [](Builder& b, Value x) { return b.scalar_op("math.exp2", {x}); })
      .def("create_log2", [](Builder& b, Value x) { return b.scalar_op("math.log2", {x}); })
      .def("create_extf", [](Builder& b, Value x, Type to) { return b.cast_op("arith.extf", x, to); })
      .def("create_truncf", [](Builder& b, Value x, Type to) { return b.cast_op("arith.truncf", x, to); });

  // ---------------------------------------------------------------- dialect registration (ffi/ir.cpp:33-47)
  auto frisk = m.def_submodule("frisk");
  frisk.def("load_dialects", [](PyContext& c) { c.ctx->dialects_loaded = true; });
}

// used by runtime.cpp
frisk_ir::Operation* op_of_handle(py::handle h) { return h.cast<OpState&>().op; }

}  // namespace frisk_ffi
