// `frisk_ffi.runtime`: lowers a tiled-GEMM kernel built with the IR builder to a
// frisk_gemm_desc, or a straight line of fill / copy / reduce ops to the tile-op
// entry points, and launches it through the C ABI of libfrisk_hip.so
// (include/frisk_hip.h).  This fills the slot the reference reserves for
// `init_ffi_passes` (ffi/ffi.h:14, ffi/ffi.cpp:6): the reference has nothing
// below its builder, so what it would lower to is the library's entry points.
// There is no other execution path: without the library every call here raises.
#include <dlfcn.h>

#include <mutex>
#include <sstream>

#include "ffi.h"
#include "frisk_hip.h"
#include "mini_ir.h"
#include "layout_infer.h"
#include "programs.h"

namespace frisk_ffi {

using namespace frisk_ir;
frisk_ir::Operation* op_of_handle(py::handle h);

namespace {

struct HipLibrary {
  void* handle = nullptr;
  std::string path;
  decltype(&frisk_hip_plan) plan = nullptr;
  decltype(&frisk_hip_gemm) gemm = nullptr;
  decltype(&frisk_hip_last_error) last_error = nullptr;
  decltype(&frisk_hip_abi_version) abi_version = nullptr;
  decltype(&frisk_hip_kernel_name) kernel_name = nullptr;
  decltype(&frisk_hip_fill) fill = nullptr;
  decltype(&frisk_hip_copy) copy = nullptr;
  decltype(&frisk_hip_reduce) reduce = nullptr;
  decltype(&frisk_hip_reduce_workspace_bytes) reduce_workspace_bytes = nullptr;
  decltype(&frisk_hip_softmax) softmax = nullptr;
  decltype(&frisk_hip_softmax_workspace_bytes) softmax_workspace_bytes = nullptr;
  decltype(&frisk_hip_attention) attention = nullptr;
  decltype(&frisk_hip_elementwise) elementwise = nullptr;
  decltype(&frisk_hip_copy_tiles) copy_tiles = nullptr;
};

HipLibrary g_lib;
std::string g_lib_path;
std::mutex g_lib_mutex;

HipLibrary& library() {
  std::lock_guard<std::mutex> lock(g_lib_mutex);
  if (g_lib.handle) return g_lib;
  if (g_lib_path.empty()) throw std::runtime_error("frisk runtime: the path of libfrisk_hip.so has not been set (runtime.set_library)");
  void* h = dlopen(g_lib_path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!h) throw std::runtime_error(std::string("frisk runtime: cannot load ") + g_lib_path + ": " + dlerror());
  HipLibrary lib;
  lib.handle = h;
  lib.path = g_lib_path;
  lib.plan = (decltype(lib.plan))dlsym(h, "frisk_hip_plan");
  lib.gemm = (decltype(lib.gemm))dlsym(h, "frisk_hip_gemm");
  lib.last_error = (decltype(lib.last_error))dlsym(h, "frisk_hip_last_error");
  lib.abi_version = (decltype(lib.abi_version))dlsym(h, "frisk_hip_abi_version");
  lib.kernel_name = (decltype(lib.kernel_name))dlsym(h, "frisk_hip_kernel_name");
  lib.fill = (decltype(lib.fill))dlsym(h, "frisk_hip_fill");
  lib.copy = (decltype(lib.copy))dlsym(h, "frisk_hip_copy");
  lib.reduce = (decltype(lib.reduce))dlsym(h, "frisk_hip_reduce");
  lib.reduce_workspace_bytes = (decltype(lib.reduce_workspace_bytes))dlsym(h, "frisk_hip_reduce_workspace_bytes");
  lib.softmax = (decltype(lib.softmax))dlsym(h, "frisk_hip_softmax");
  lib.softmax_workspace_bytes = (decltype(lib.softmax_workspace_bytes))dlsym(h, "frisk_hip_softmax_workspace_bytes");
  lib.attention = (decltype(lib.attention))dlsym(h, "frisk_hip_attention");
  lib.elementwise = (decltype(lib.elementwise))dlsym(h, "frisk_hip_elementwise");
  lib.copy_tiles = (decltype(lib.copy_tiles))dlsym(h, "frisk_hip_copy_tiles");
  if (!lib.elementwise || !lib.copy_tiles || !lib.softmax || !lib.softmax_workspace_bytes || !lib.attention || !lib.plan || !lib.gemm || !lib.last_error || !lib.abi_version || !lib.kernel_name || !lib.fill || !lib.copy || !lib.reduce || !lib.reduce_workspace_bytes)
    throw std::runtime_error("frisk runtime: " + g_lib_path + " does not export the frisk_hip entry points");
  if (lib.abi_version() != FRISK_HIP_ABI_VERSION) throw std::runtime_error("frisk runtime: libfrisk_hip.so ABI version mismatch");
  g_lib = lib;
  return g_lib;
}

int dtype_of(const Type& t) {
  switch (t.kind()) {
    case TypeKind::F32: return FRISK_F32;
    case TypeKind::F16: return FRISK_F16;
    case TypeKind::BF16: return FRISK_BF16;
    case TypeKind::I8: return FRISK_I8;
    case TypeKind::F8E4M3FN: return FRISK_E4M3;
    case TypeKind::I32: return FRISK_I32;
    default: throw std::invalid_argument("element type " + t.str() + " has no gfx950 GEMM kernel");
  }
}

int epilogue_of(const std::string& e) {
  if (e == "none") return FRISK_EPI_NONE;
  if (e == "row_col_scale") return FRISK_EPI_ROW_COL_SCALE;
  if (e == "tensor_scale") return FRISK_EPI_TENSOR_SCALE;
  throw std::invalid_argument("unknown epilogue '" + e + "' (none, row_col_scale, tensor_scale)");
}

frisk_gemm_desc desc_of(const GemmProgram& g, int epilogue) {
  frisk_gemm_desc d{};
  d.abi_version = FRISK_HIP_ABI_VERSION;
  d.dtype_ab = dtype_of(g.elem_ab);
  d.dtype_acc = dtype_of(g.elem_acc);
  d.dtype_out = dtype_of(g.elem_out);
  d.M = g.M; d.N = g.N; d.K = g.K;
  d.lda = g.transA ? g.M : g.K;
  d.ldb = g.transB ? g.K : g.N;
  d.ldc = g.N;
  d.transA = g.transA; d.transB = g.transB; d.clear_accum = g.clear_accum;
  d.epilogue = epilogue;
  d.policy = (int)g.policy;
  d.tile_m = (int)g.tile_m; d.tile_n = (int)g.tile_n; d.tile_k = (int)g.tile_k;
  return d;
}

// The descriptor `launch` hands to the C ABI, shared with `plan` so that the plan describes the kernel that runs.  The tile
// sizes in the IR describe the program; which kernel variant computes it best is the planner's call for the whole problem
// (1024^3 fp32 written with 128 x 128 tiles is 64 work-groups on 256 CUs).  retile = false keeps the IR's tile.
frisk_gemm_desc launch_desc_of(const GemmProgram& g, int epilogue, bool retile) {
  frisk_gemm_desc d = desc_of(g, epilogue);
  if (retile) d.tile_m = d.tile_n = d.tile_k = 0;
  return d;
}

GemmProgram program_of(py::object kernel, py::object module) {
  Operation* k = op_of_handle(kernel);
  Operation* m = module.is_none() ? nullptr : op_of_handle(module);
  return match_tiled_gemm(k, m);
}

// Index map of an LDS tile in the form the reference prints its LayoutAttr (printLayoutDebug,
// lib/Dialect/Frisk/IR/FriskAttributes.cpp:38-56): Layout(shape=[rows, cols], index=affine_map<(d0, d1) -> (...)>),
// element (d0, d1) of the tile as stored -> element offset in LDS.  The XOR of the 16-byte chunk index with row bits is
// written with sums and floordiv, bit by bit, as the reference writes its bank swizzles (FriskOps.cpp:123-143, 500-558).
std::string lds_layout_debug(const frisk_lds_layout& L, int elem_bytes) {
  const int64_t vec = 16 / elem_bytes, cols = L.row_bytes / elem_bytes;
  AffineExpr i = AffineExpr::dim(0), j = AffineExpr::dim(1);
  AffineExpr chunk = j.floor_div(AffineExpr::constant(vec));
  AffineExpr stored = chunk;
  // one XOR term applied to the chunk index as stored so far
  auto apply = [&](int row_shift, int row_mask, int chunk_shift) {
    if (!row_mask) return;
    const int64_t lo = (int64_t)1 << chunk_shift, span = (int64_t)row_mask + 1;
    AffineExpr field = stored.floor_div(AffineExpr::constant(lo)).mod(AffineExpr::constant(span));  // the chunk bits the swizzle touches
    AffineExpr key = i.floor_div(AffineExpr::constant((int64_t)1 << row_shift)).mod(AffineExpr::constant(span));
    AffineExpr x = AffineExpr::constant(0);
    for (int64_t b = 1; b < span; b *= 2) {
      AffineExpr fb = field.floor_div(AffineExpr::constant(b)).mod(AffineExpr::constant(2));
      AffineExpr kb = key.floor_div(AffineExpr::constant(b)).mod(AffineExpr::constant(2));
      x = x + (fb + kb).mod(AffineExpr::constant(2)) * b;
    }
    stored = stored + (x - field) * lo;
  };
  apply(L.row_shift, L.row_mask, L.chunk_shift);
  apply(L.row_shift2, L.row_mask2, L.chunk_shift2);
  AffineExpr index = i * cols + stored * vec + j.mod(AffineExpr::constant(vec));
  AffineMap map(2, 0, {index});
  return "Layout(shape=[" + std::to_string(L.rows) + ", " + std::to_string(cols) + "], index=affine_map<" + map.str() + ">)";
}

// Accumulator fragment of a work-group tile in the same debug form: Fragment(shape, index, thread, replicate).
std::string accumulator_layout_debug(int64_t bm, int64_t bn, int64_t wm, int64_t wn) { return accumulator_layout(bm, bn, wm, wn).debug(); }

// LayoutAttr <-> Python: {"shape": [..], "index": AffineMap, "thread": AffineMap or None, "replicate": int or None}; to
// Python also "debug", the text printLayoutDebug gives.
py::object layout_to_py(const LayoutAttr& l) {
  if (!l) return py::none();
  py::dict d;
  d["shape"] = l.shape;
  d["index"] = l.index ? py::cast(l.index) : py::object(py::none());
  d["thread"] = l.thread ? py::cast(l.thread) : py::object(py::none());
  d["replicate"] = l.replicate ? py::object(py::int_(*l.replicate)) : py::object(py::none());
  d["debug"] = l.debug();
  return std::move(d);
}
LayoutAttr layout_from_py(const py::object& o) {
  if (o.is_none()) return LayoutAttr::none();
  py::dict d = o.cast<py::dict>();
  LayoutAttr l;
  l.shape = d["shape"].cast<std::vector<int64_t>>();
  if (d.contains("index") && !d["index"].is_none()) l.index = d["index"].cast<AffineMap>();
  if (d.contains("thread") && !d["thread"].is_none()) l.thread = d["thread"].cast<AffineMap>();
  if (d.contains("replicate") && !d["replicate"].is_none()) l.replicate = d["replicate"].cast<int64_t>();
  return l;
}

py::dict program_dict(const GemmProgram& g) {
  py::dict d;
  d["kernel"] = g.kernel_name;
  d["M"] = g.M; d["N"] = g.N; d["K"] = g.K;
  d["tile"] = py::make_tuple(g.tile_m, g.tile_n, g.tile_k);
  d["grid"] = py::make_tuple(g.grid_m, g.grid_n);
  d["threads"] = g.threads;
  d["transA"] = g.transA; d["transB"] = g.transB; d["clear_accum"] = g.clear_accum;
  d["dtype_ab"] = g.elem_ab.str(); d["dtype_acc"] = g.elem_acc.str(); d["dtype_out"] = g.elem_out.str();
  d["args"] = py::make_tuple(g.arg_a, g.arg_b, g.arg_c);
  d["target"] = g.target;
  return d;
}

int reduce_kind_of(const std::string& k) {
  if (k == "add") return FRISK_REDUCE_ADD;
  if (k == "mul") return FRISK_REDUCE_MUL;
  if (k == "min") return FRISK_REDUCE_MIN;
  if (k == "max") return FRISK_REDUCE_MAX;
  throw std::invalid_argument("unsupported reduce kind: " + k + ". Supported: add, mul, min, max");
}

py::dict tile_op_dict(const TileOpDesc& d) {
  py::dict o;
  o["op"] = d.kind == TileOpDesc::Fill ? "fill" : d.kind == TileOpDesc::Copy ? "copy" : d.kind == TileOpDesc::CopyTiles ? "copy_tiles" : "reduce";
  if (d.kind == TileOpDesc::CopyTiles) {
    o["tiles"] = py::make_tuple(d.n0, d.n1);
    o["src_steps"] = py::make_tuple(d.src_step0, d.src_step1);
    o["dst_steps"] = py::make_tuple(d.dst_step0, d.dst_step1);
  }
  o["rows"] = d.rows; o["cols"] = d.cols;
  if (d.kind != TileOpDesc::Fill) { o["src"] = d.arg_src; o["src_offset"] = d.src_offset; o["src_ld"] = d.src_ld; o["src_dtype"] = d.elem_src.str(); }
  o["dst"] = d.arg_dst; o["dst_offset"] = d.dst_offset; o["dst_dtype"] = d.elem_dst.str();
  if (d.kind != TileOpDesc::Reduce) o["dst_ld"] = d.dst_ld;
  if (d.kind == TileOpDesc::Fill) o["value"] = d.value;
  if (d.kind == TileOpDesc::Reduce) { o["kind"] = d.reduce_kind; o["dim"] = d.dim; o["clear"] = d.clear; }
  return o;
}

// Which of the recognised programs a kernel is, by the ops it holds: frisk.block bodies only occur in the softmax and
// attention programs; two products make the attention program.
enum class ProgramKind { TiledGemm, OnlineSoftmax, Attention, Elementwise };
ProgramKind classify(Operation* kernel) {
  if (is_elementwise_kernel(kernel)) return ProgramKind::Elementwise;  // nothing but free-standing frisk.block ops
  int gemms = 0, blocks = 0;
  std::function<void(Operation*)> walk = [&](Operation* op) {
    if (op->name == "frisk.gemm") ++gemms;
    if (op->name == "frisk.block") ++blocks;
    for (Region* r : op->regions)
      for (Block* b : r->blocks)
        for (Operation* inner : b->ops) walk(inner);
  };
  if (kernel) walk(kernel);
  if (blocks > 0 && gemms == 0) return ProgramKind::OnlineSoftmax;
  if (blocks > 0 && gemms >= 2) return ProgramKind::Attention;
  return ProgramKind::TiledGemm;
}

py::dict softmax_dict(const SoftmaxProgram& g) {
  py::dict o;
  o["program"] = "online_softmax";
  o["kernel"] = g.kernel_name;
  o["rows"] = g.rows; o["cols"] = g.cols; o["chunk"] = g.chunk;
  o["scale_log2"] = g.cst;
  o["dtype"] = g.elem.str();
  o["args"] = py::make_tuple(g.arg_src, g.arg_dst);
  o["target"] = g.target;
  return o;
}

int ew_opcode(const std::string& op) {
  static const std::map<std::string, int> codes = {{"input", FRISK_EW_INPUT}, {"const", FRISK_EW_CONST}, {"add", FRISK_EW_ADD}, {"sub", FRISK_EW_SUB},
                                                    {"mul", FRISK_EW_MUL}, {"div", FRISK_EW_DIV}, {"max", FRISK_EW_MAX}, {"min", FRISK_EW_MIN},
                                                    {"neg", FRISK_EW_NEG}, {"exp2", FRISK_EW_EXP2}, {"log2", FRISK_EW_LOG2}};
  auto it = codes.find(op);
  if (it == codes.end()) throw std::invalid_argument("operation '" + op + "' has no elementwise opcode");
  return it->second;
}

// the postfix program of a block as text: x<k> operand k, c<value> constant, else the operation
std::string ew_text(const EwBlock& b) {
  std::ostringstream os;
  for (size_t i = 0; i < b.steps.size(); ++i) {
    if (i) os << ' ';
    if (b.steps[i].op == "input") os << 'x' << b.steps[i].operand;
    else if (b.steps[i].op == "const") os << 'c' << b.steps[i].value;
    else os << b.steps[i].op;
  }
  return os.str();
}

py::dict elementwise_dict(const EwProgram& g) {
  py::dict o;
  o["program"] = "elementwise";
  o["kernel"] = g.kernel_name;
  o["target"] = g.target;
  py::list blocks;
  for (const EwBlock& b : g.blocks) {
    py::dict d;
    d["rows"] = b.rows; d["cols"] = b.cols;
    d["out"] = py::make_tuple(b.out.arg, b.out.offset, b.out.row_stride, b.out.elem.str());
    py::list ins;
    for (const EwOperand& x : b.inputs) ins.append(py::make_tuple(x.arg, x.offset, x.row_stride, x.col_stride, x.elem.str()));
    d["inputs"] = ins;
    d["postfix"] = ew_text(b);
    d["stack"] = b.max_stack;
    blocks.append(d);
  }
  o["blocks"] = blocks;
  return o;
}

// descriptor of one block for frisk_hip_elementwise; throws what the library would refuse, with the block's own words
frisk_elementwise_desc ew_desc_of(const EwBlock& b) {
  if (b.inputs.size() > FRISK_EW_MAX_INPUTS) throw std::invalid_argument("a block body reads " + std::to_string(b.inputs.size()) + " different operands, at most " + std::to_string(FRISK_EW_MAX_INPUTS) + " are supported");
  if (b.steps.size() > FRISK_EW_MAX_OPS) throw std::invalid_argument("a block body of " + std::to_string(b.steps.size()) + " steps, at most " + std::to_string(FRISK_EW_MAX_OPS) + " are supported");
  if (b.max_stack > FRISK_EW_MAX_STACK) throw std::invalid_argument("a block body needs an evaluation stack of " + std::to_string(b.max_stack) + ", at most " + std::to_string(FRISK_EW_MAX_STACK) + " is supported");
  frisk_elementwise_desc d{};
  d.abi_version = FRISK_HIP_ABI_VERSION;
  d.n_inputs = (int)b.inputs.size();
  d.n_ops = (int)b.steps.size();
  d.out_dtype = dtype_of(b.out.elem);
  d.rows = b.rows; d.cols = b.cols;
  d.out_ld = b.rows > 1 ? b.out.row_stride : b.cols;
  for (size_t k = 0; k < b.inputs.size(); ++k) {
    d.in_dtype[k] = dtype_of(b.inputs[k].elem);
    d.in_row_stride[k] = b.inputs[k].row_stride;
    d.in_col_stride[k] = (int)b.inputs[k].col_stride;
  }
  for (size_t i = 0; i < b.steps.size(); ++i) {
    d.op[i] = ew_opcode(b.steps[i].op);
    d.arg[i] = b.steps[i].operand < 0 ? 0 : b.steps[i].operand;
    d.imm[i] = (float)b.steps[i].value;
  }
  return d;
}

py::dict attention_dict(const AttentionProgram& g) {
  py::dict o;
  o["program"] = "attention";
  o["kernel"] = g.kernel_name;
  o["batch"] = g.batch; o["heads"] = g.heads; o["seq_q"] = g.seq_q; o["seq_k"] = g.seq_k; o["head_dim"] = g.head_dim;
  o["tile"] = py::make_tuple(g.tile_q, g.tile_k);
  o["k_transposed"] = g.k_transposed;
  o["scale_log2"] = g.cst;
  o["scale"] = g.cst / 1.4426950408889634;
  o["dtype"] = g.elem.str();
  o["args"] = py::make_tuple(g.arg_q, g.arg_k, g.arg_v, g.arg_o);
  o["target"] = g.target;
  return o;
}

}  // namespace

void init_ffi_runtime(py::module_&& m) {
  m.def("set_library", [](const std::string& path) {
    std::lock_guard<std::mutex> lock(g_lib_mutex);
    g_lib_path = path;
  }, "path of libfrisk_hip.so; loaded on first use");
  m.def("library_path", []() { return g_lib_path; });

  m.def("match", [](py::object kernel, py::object module) {
    Operation* k = op_of_handle(kernel);
    Operation* mod = module.is_none() ? nullptr : op_of_handle(module);
    switch (classify(k)) {
      case ProgramKind::Elementwise: {
        const EwProgram g = match_elementwise(k, mod);
        for (const EwBlock& b : g.blocks) (void)ew_desc_of(b);  // what the library could not run is refused here already
        return elementwise_dict(g);
      }
      case ProgramKind::OnlineSoftmax: return softmax_dict(match_online_softmax(k, mod));
      case ProgramKind::Attention: return attention_dict(match_attention(k, mod));
      default: break;
    }
    py::dict d = program_dict(match_tiled_gemm(k, mod));
    d["program"] = "tiled_gemm";
    return d;
  }, py::arg("kernel"), py::arg("module") = py::none(),
        "recognise one of the programs of the reference's design sketches and return what it computes: the tiled GEMM "
        "kernel{parallel{alloc x3, fill, for{copy, copy, gemm}, copy}}, the row softmax with a running log-sum, the fused attention, or a kernel of "
        "free-standing frisk.block bodies (one postfix program per block); pure host");

  m.def("plan", [](py::object kernel, py::object module, const std::string& epilogue, bool retile) {
    GemmProgram g = program_of(kernel, module);
    frisk_gemm_desc d = launch_desc_of(g, epilogue_of(epilogue), retile);
    HipLibrary& lib = library();
    frisk_gemm_plan p{};
    if (int st = lib.plan(&d, &p)) throw std::invalid_argument(std::string("frisk_hip_plan: ") + lib.last_error() + " (status " + std::to_string(st) + ")");
    py::dict out = program_dict(g);
    out["hip_kernel"] = p.kernel_id >= 0 ? std::string(lib.kernel_name(p.kernel_id)) : std::string();
    out["hip_tile"] = py::make_tuple(p.tile_m, p.tile_n, p.tile_k);
    out["hip_waves"] = py::make_tuple(p.waves_m, p.waves_n);
    out["hip_grid"] = py::make_tuple(p.grid_y, p.grid_x);
    out["lds_bytes"] = p.lds_bytes;
    out["stages"] = py::make_tuple(p.stages, p.stages_b);
    const int es = (int)(g.elem_ab.bit_width() / 8);
    out["lds_a"] = lds_layout_debug(p.lds_a, es);
    out["lds_b"] = lds_layout_debug(p.lds_b, es);
    out["lds_swizzle"] = py::make_tuple(py::make_tuple(p.lds_a.row_shift, p.lds_a.row_mask, p.lds_a.chunk_shift),
                                        py::make_tuple(p.lds_b.row_shift, p.lds_b.row_mask, p.lds_b.chunk_shift));
    out["lds_swizzle2"] = py::make_tuple(py::make_tuple(p.lds_a.row_shift2, p.lds_a.row_mask2, p.lds_a.chunk_shift2),
                                         py::make_tuple(p.lds_b.row_shift2, p.lds_b.row_mask2, p.lds_b.chunk_shift2));
    out["flops"] = p.flops;
    out["bytes"] = p.bytes;
    return out;
  }, py::arg("kernel"), py::arg("module") = py::none(), py::arg("epilogue") = "none", py::arg("retile") = true,
     "the plan of the kernel that `launch` runs for the same `retile`: by default the planner's own tile for the whole problem, with "
     "retile = False the tile the program is written with; pure host");

  m.def("lds_layout_string", [](int rows, int row_bytes, int elem_bytes, int row_shift, int row_mask, int chunk_shift,
                                int row_shift2, int row_mask2, int chunk_shift2) {
    frisk_lds_layout L{};
    L.rows = rows; L.row_bytes = row_bytes; L.row_shift = row_shift; L.row_mask = row_mask; L.chunk_shift = chunk_shift;
    L.row_shift2 = row_shift2; L.row_mask2 = row_mask2; L.chunk_shift2 = chunk_shift2;
    if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) throw std::invalid_argument("element size must be 1, 2 or 4 bytes");
    return lds_layout_debug(L, elem_bytes);
  }, py::arg("rows"), py::arg("row_bytes"), py::arg("elem_bytes"), py::arg("row_shift"), py::arg("row_mask"), py::arg("chunk_shift"),
     py::arg("row_shift2") = 0, py::arg("row_mask2") = 0, py::arg("chunk_shift2") = 0,
     "Layout(shape=[...], index=affine_map<...>) of an LDS tile with the XOR swizzle (row_shift, row_mask, chunk_shift) and the optional second term; pure host");
  m.def("accumulator_layout_string", &accumulator_layout_debug, py::arg("tile_m"), py::arg("tile_n"), py::arg("waves_m"), py::arg("waves_n"),
        "Fragment(shape, index, thread, replicate) of the MFMA accumulators of a work-group tile; pure host");

  m.def("accumulator_layout", [](int64_t bm, int64_t bn, int64_t wm, int64_t wn) { return layout_to_py(accumulator_layout(bm, bn, wm, wn)); },
        py::arg("tile_m"), py::arg("tile_n"), py::arg("waves_m"), py::arg("waves_n"),
        "layout attribute (shape, index map, thread map, replicate) of the MFMA accumulators of a work-group tile; pure host");
  m.def("used_extent_for_dim", [](const AffineMap& map, int pos, int64_t extent) -> py::object {
    auto v = compute_used_extent_for_dim(map, pos, extent);
    return v ? py::object(py::int_(*v)) : py::object(py::none());
  }, py::arg("map"), py::arg("dim"), py::arg("extent"),
        "number of distinct values the map's results take along one dim of the given extent (None: not analysable); pure host");
  m.def("infer_reduce_layout", [](py::object src, std::vector<int64_t> src_shape, std::vector<int64_t> dst_shape, int64_t dim, int64_t threads,
                                  py::object existing) {
    const LayoutAttr have = layout_from_py(existing);
    return layout_to_py(infer_reduce_layout(layout_from_py(src), src_shape, dst_shape, dim, threads, existing.is_none() ? nullptr : &have));
  }, py::arg("src"), py::arg("src_shape"), py::arg("dst_shape"), py::arg("dim"), py::arg("threads") = 0, py::arg("existing") = py::none(),
        "layout of the destination of frisk.reduce from the layout of its source (both in registers); None when the source has no "
        "index or thread map; ValueError with the op's diagnostic otherwise; pure host");
  m.def("default_buffer_layout", [](std::vector<int64_t> shape, int element_bits, py::object space, int wave_size, int64_t threads) {
    return layout_to_py(default_buffer_layout((MemorySpace)py::int_(space).cast<int>(), shape, element_bits, wave_size, threads));
  }, py::arg("shape"), py::arg("element_bits"), py::arg("space"), py::arg("wave_size") = 64, py::arg("threads") = 1,
        "default layout of a buffer that no GEMM uses: padded row-major (shared), a lane grid over the last two dims (local), row-major "
        "(global); one-element buffers are replicated over all threads; pure host");
  m.def("infer_layouts", [](py::object kernel) {
    // ParallelOp::inferLayout (lib/Dialect/Frisk/IR/FriskOps.cpp:1040-1092), the part that is not GEMM specific: every
    // frisk.alloc_buffer under the kernel's frisk.parallel that no frisk.gemm uses gets its default layout; buffers a
    // GEMM uses are left to the GEMM planner (runtime.plan) and reported with layout None.
    Operation* k = op_of_handle(kernel);
    if (!k || k->name != "frisk.kernel" || k->regions.empty() || k->regions[0]->blocks.empty()) throw std::invalid_argument("expected a frisk.kernel with a body");
    Operation* par = nullptr;
    for (Operation* op : k->regions[0]->blocks[0]->ops)
      if (op->name == "frisk.parallel") { par = op; break; }
    if (!par) throw std::invalid_argument("the kernel has no frisk.parallel");
    const int64_t threads = par->int_attr("threads");
    std::vector<Operation*> all;
    std::function<void(Operation*)> walk = [&](Operation* op) {
      for (Region* r : op->regions)
        for (Block* b : r->blocks)
          for (Operation* inner : b->ops) { all.push_back(inner); walk(inner); }
    };
    walk(par);
    py::list out;
    int n = 0;
    for (Operation* op : all) {
      if (op->name != "frisk.alloc_buffer" || op->results.empty()) continue;
      ValueImpl* buf = op->results[0];
      bool gemm_operand = false;
      for (Operation* user : all)
        if (user->name == "frisk.gemm")
          for (const Value& v : user->operands) gemm_operand = gemm_operand || v.impl == buf;
      const Type t = buf->type;
      py::dict d;
      d["buffer"] = n++;
      d["shape"] = t.impl->shape;
      d["memory_space"] = (int)op->int_attr("memory_space");
      d["used_by_gemm"] = gemm_operand;
      d["layout"] = gemm_operand ? py::object(py::none())
                                 : layout_to_py(default_buffer_layout((MemorySpace)op->int_attr("memory_space"), t.impl->shape, t.element().bit_width(), 64, threads));
      out.append(d);
    }
    return out;
  }, py::arg("kernel"),
        "default layouts of the kernel's alloc_buffers that no GEMM uses, in program order (wave of 64 lanes); pure host");
  m.def("match_ops", [](py::object kernel) {
    py::list out;
    for (const TileOpDesc& d : match_data_movement(op_of_handle(kernel))) out.append(tile_op_dict(d));
    return out;
  }, py::arg("kernel"), "recognise a kernel whose body is a straight line of fill / copy / reduce on its arguments; pure host");

  m.def("ops_workspace_bytes", [](py::object kernel) {
    HipLibrary& lib = library();
    size_t need = 0;
    for (const TileOpDesc& d : match_data_movement(op_of_handle(kernel)))
      if (d.kind == TileOpDesc::Reduce) need = std::max(need, lib.reduce_workspace_bytes(dtype_of(d.elem_src), d.rows, d.cols, (int)d.dim));
    return need;
  }, py::arg("kernel"), "device workspace launch_ops can use for the kernel's longest reduction (0 if none needs one)");

  m.def("launch_ops", [](py::object kernel, std::vector<uint64_t> args, uint64_t stream, uint64_t workspace, size_t workspace_bytes) {
    std::vector<TileOpDesc> ops = match_data_movement(op_of_handle(kernel));
    HipLibrary& lib = library();
    auto ptr = [&](int arg, int64_t offset, const Type& elem) -> void* {
      if (arg < 0 || (size_t)arg >= args.size()) throw std::invalid_argument("launch_ops needs one device pointer per kernel argument");
      return (void*)(args[(size_t)arg] + (uint64_t)offset * (uint64_t)(elem.bit_width() / 8));
    };
    py::gil_scoped_release release;
    for (const TileOpDesc& d : ops) {  // program order on one stream: each op sees the results of the ones before it
      int st = 0;
      if (d.kind == TileOpDesc::Fill)
        st = lib.fill(dtype_of(d.elem_dst), ptr(d.arg_dst, d.dst_offset, d.elem_dst), d.rows, d.cols, d.dst_ld, d.value, (void*)stream);
      else if (d.kind == TileOpDesc::CopyTiles)
        st = lib.copy_tiles(dtype_of(d.elem_src), ptr(d.arg_src, d.src_offset, d.elem_src), d.src_ld, dtype_of(d.elem_dst), ptr(d.arg_dst, d.dst_offset, d.elem_dst),
                            d.dst_ld, d.rows, d.cols, d.n0, d.src_step0, d.dst_step0, d.n1, d.src_step1, d.dst_step1, (void*)stream);
      else if (d.kind == TileOpDesc::Copy)
        st = lib.copy(dtype_of(d.elem_src), ptr(d.arg_src, d.src_offset, d.elem_src), d.src_ld, dtype_of(d.elem_dst), ptr(d.arg_dst, d.dst_offset, d.elem_dst),
                      d.dst_ld, d.rows, d.cols, (void*)stream);
      else
        st = lib.reduce(dtype_of(d.elem_src), ptr(d.arg_src, d.src_offset, d.elem_src), d.rows, d.cols, d.src_ld, (int)d.dim, reduce_kind_of(d.reduce_kind),
                        d.clear ? 1 : 0, ptr(d.arg_dst, d.dst_offset, d.elem_dst), (void*)workspace, workspace_bytes, (void*)stream);
      if (st) {
        py::gil_scoped_acquire acquire;
        throw std::runtime_error(std::string("frisk_hip tile op: ") + lib.last_error() + " (status " + std::to_string(st) + ")");
      }
    }
  }, py::arg("kernel"), py::arg("args"), py::arg("stream") = 0, py::arg("workspace") = 0, py::arg("workspace_bytes") = 0,
     "asynchronous launch, in program order on `stream`, of a kernel made of fill / copy / reduce on its arguments");

  m.def("launch", [](py::object kernel, std::vector<uint64_t> args, uint64_t stream, py::object module, const std::string& epilogue,
                     uint64_t scale_a, uint64_t scale_b, bool retile) {
    Operation* k = op_of_handle(kernel);
    Operation* mod = module.is_none() ? nullptr : op_of_handle(module);
    const ProgramKind kind = classify(k);
    if (kind == ProgramKind::Elementwise) {
      const EwProgram g = match_elementwise(k, mod);
      HipLibrary& lib = library();
      for (const EwBlock& b : g.blocks) {  // program order on one stream: a block sees what the blocks before it stored
        const frisk_elementwise_desc d = ew_desc_of(b);
        auto ptr = [&](const EwOperand& o) -> uint64_t {
          if ((size_t)o.arg >= args.size()) throw std::invalid_argument("launch needs one device pointer per kernel argument");
          return args[(size_t)o.arg] + (uint64_t)o.offset * (uint64_t)(o.elem.bit_width() / 8);
        };
        const void* inputs[FRISK_EW_MAX_INPUTS] = {};
        for (size_t i = 0; i < b.inputs.size(); ++i) inputs[i] = (const void*)ptr(b.inputs[i]);
        void* out = (void*)ptr(b.out);
        int st;
        {
          py::gil_scoped_release release;
          st = lib.elementwise(&d, inputs, out, (void*)stream);
        }
        if (st) throw std::runtime_error(std::string("frisk_hip_elementwise: ") + lib.last_error() + " (status " + std::to_string(st) + ")");
      }
      return;
    }
    if (kind == ProgramKind::OnlineSoftmax) {
      const SoftmaxProgram g = match_online_softmax(k, mod);
      if (args.size() < (size_t)std::max(g.arg_src, g.arg_dst) + 1) throw std::invalid_argument("launch needs one device pointer per kernel argument");
      HipLibrary& lib = library();
      int st;
      {
        py::gil_scoped_release release;
        st = lib.softmax(dtype_of(g.elem), (const void*)args[(size_t)g.arg_src], g.cols, (void*)args[(size_t)g.arg_dst], g.cols, g.rows, g.cols, (float)g.cst, nullptr,
                         nullptr, 0, (void*)stream);
      }
      if (st) throw std::runtime_error(std::string("frisk_hip_softmax: ") + lib.last_error() + " (status " + std::to_string(st) + ")");
      return;
    }
    if (kind == ProgramKind::Attention) {
      const AttentionProgram g = match_attention(k, mod);
      if (args.size() < (size_t)std::max(std::max(g.arg_q, g.arg_k), std::max(g.arg_v, g.arg_o)) + 1) throw std::invalid_argument("launch needs one device pointer per kernel argument");
      if (!(g.cst > 0)) throw std::invalid_argument("the attention program's constant must be positive");
      frisk_attention_desc d{};
      d.abi_version = FRISK_HIP_ABI_VERSION;
      d.dtype = dtype_of(g.elem);
      d.batch = g.batch; d.heads = g.heads; d.seq_q = g.seq_q; d.seq_k = g.seq_k; d.head_dim = g.head_dim;
      d.scale = (float)(g.cst / 1.4426950408889634);
      d.k_transposed = g.k_transposed ? 1 : 0;
      HipLibrary& lib = library();
      int st;
      {
        py::gil_scoped_release release;
        st = lib.attention(&d, (const void*)args[(size_t)g.arg_q], (const void*)args[(size_t)g.arg_k], (const void*)args[(size_t)g.arg_v], (void*)args[(size_t)g.arg_o],
                           nullptr, (void*)stream);
      }
      if (st) throw std::runtime_error(std::string("frisk_hip_attention: ") + lib.last_error() + " (status " + std::to_string(st) + ")");
      return;
    }
    GemmProgram g = match_tiled_gemm(k, mod);
    size_t need = (size_t)std::max(g.arg_a, std::max(g.arg_b, g.arg_c)) + 1;
    if (args.size() < need) throw std::invalid_argument("launch needs one device pointer per kernel argument");
    frisk_gemm_desc d = launch_desc_of(g, epilogue_of(epilogue), retile);
    HipLibrary& lib = library();
    int st;
    {
      py::gil_scoped_release release;
      st = lib.gemm(&d, (const void*)args[(size_t)g.arg_a], (const void*)args[(size_t)g.arg_b], (void*)args[(size_t)g.arg_c], (const float*)scale_a,
                    (const float*)scale_b, nullptr, 0, (void*)stream);
    }
    if (st) throw std::runtime_error(std::string("frisk_hip_gemm: ") + lib.last_error() + " (status " + std::to_string(st) + ")");
  }, py::arg("kernel"), py::arg("args"), py::arg("stream") = 0, py::arg("module") = py::none(), py::arg("epilogue") = "none",
     py::arg("scale_a") = 0, py::arg("scale_b") = 0, py::arg("retile") = true,
     "asynchronous launch on `stream` (a hipStream_t value) of a recognised program (tiled GEMM, online softmax, fused attention, "
     "free-standing frisk.block bodies); "
     "`args` holds one raw device pointer per kernel argument");
}

}  // namespace frisk_ffi
