// Generic (non-GEMM) layout inference of the dialect, restated over the MLIR-free affine maps of mini_ir.h:
//   * the layout attribute and its debug print (include/Dialect/Frisk/IR/FriskAttributes.td:17-30,
//     lib/Dialect/Frisk/IR/FriskAttributes.cpp:38-56),
//   * how many distinct values a map takes along one dim (computeUsedExtentForDim,
//     lib/Dialect/Frisk/Utils/LayoutUtils.cpp:36-218),
//   * the layout of a reduction's destination from its source's (ReduceOp::inferLayout,
//     lib/Dialect/Frisk/IR/FriskOps_Reduce.cpp:51-163, 214-357),
//   * the default layouts of buffers no specialised inference covers (lib/Dialect/Frisk/IR/FriskOps.cpp:641-823),
//     with the wave of the target (64 lanes on gfx950) where the reference's default is a warp of 32,
//   * the accumulator fragment of a work-group tile of the MFMA kernels, as such an attribute, so that the
//     reduction inference applies to what the kernels really hold (row maxima / sums of a score tile).
#pragma once
#include <algorithm>
#include <optional>
#include <set>
#include <utility>

#include "mini_ir.h"

namespace frisk_ir {

struct LayoutAttr {
  std::vector<int64_t> shape;
  AffineMap index;                  // logical coordinates -> storage / register index
  AffineMap thread;                 // logical coordinates (and, for a reduced buffer, one symbol) -> thread; empty for memory layouts
  std::optional<int64_t> replicate; // number of threads that hold a copy of every element
  bool null = false;
  static LayoutAttr none() { LayoutAttr l; l.null = true; return l; }
  explicit operator bool() const { return !null; }
  // printLayoutDebug, FriskAttributes.cpp:38-56
  std::string debug() const {
    if (null) return "<null layout>";
    std::string s = std::string(thread ? "Fragment" : "Layout") + "(shape=[";
    for (size_t i = 0; i < shape.size(); ++i) s += (i ? ", " : "") + std::to_string(shape[i]);
    s += "], index=" + (index ? "affine_map<" + index.str() + ">" : std::string("<null>"));
    if (thread) s += ", thread=affine_map<" + thread.str() + ">";
    if (replicate) s += ", replicate=" + std::to_string(*replicate);
    return s + ")";
  }
  bool equals(const LayoutAttr& o) const {
    return null == o.null && shape == o.shape && index.equals(o.index) && thread.equals(o.thread) && replicate == o.replicate;
  }
};

// ------------------------------------------------------------------ LayoutUtils.cpp
namespace detail {
inline bool uses_dim(const AffineExpr& e, int64_t dim) { return e.is_function_of(ExprKind::DimId, dim); }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// number of values `e` can take when dim `dim` ranges over base_span values and everything else is fixed (an upper
// bound built structurally; computeSpan, LayoutUtils.cpp:36-114)
inline std::optional<int64_t> compute_span(const AffineExpr& e, int64_t dim, int64_t base_span) {
  switch (e.kind()) {
    case ExprKind::Constant: case ExprKind::SymbolId: return 1;
    case ExprKind::DimId: return e.impl->value == dim ? base_span : 1;
    default: break;
  }
  if (!e.is_binary()) return std::nullopt;
  auto l = compute_span(e.lhs(), dim, base_span), r = compute_span(e.rhs(), dim, base_span);
  if (!l || !r) return std::nullopt;
  switch (e.kind()) {
    case ExprKind::Add: return std::max<int64_t>(1, *l + *r - 1);
    case ExprKind::Mul:
      if (e.rhs().is_constant()) return *l * std::abs(e.rhs().constant_value());
      if (e.lhs().is_constant()) return *r * std::abs(e.lhs().constant_value());
      return std::nullopt;
    case ExprKind::FloorDiv:
      if (!e.rhs().is_constant() || e.rhs().constant_value() <= 0) return std::nullopt;
      return ceil_div(*l, e.rhs().constant_value());
    case ExprKind::Mod:
      if (!e.rhs().is_constant() || e.rhs().constant_value() <= 0) return std::nullopt;
      return std::min<int64_t>(*l, e.rhs().constant_value());
    default: return std::nullopt;
  }
}

// every occurrence of the dim, with the extent the operations above it leave of it (collectSplits, :116-177)
inline bool collect_splits(const AffineExpr& e, int64_t dim, int64_t base_extent, int64_t lower, std::vector<std::pair<int64_t, int64_t>>& out) {
  if (!uses_dim(e, dim)) return true;
  if (e.kind() == ExprKind::DimId) { out.push_back({lower, base_extent}); return true; }
  if (!e.is_binary()) return false;
  switch (e.kind()) {
    case ExprKind::Add:
      return collect_splits(e.lhs(), dim, base_extent, lower, out) && collect_splits(e.rhs(), dim, base_extent, lower, out);
    case ExprKind::Mul:
      if (e.lhs().is_constant()) return collect_splits(e.rhs(), dim, base_extent, lower, out);
      if (e.rhs().is_constant()) return collect_splits(e.lhs(), dim, base_extent, lower, out);
      return false;
    case ExprKind::FloorDiv: {
      if (!e.rhs().is_constant() || e.rhs().constant_value() <= 0) return false;
      auto span = compute_span(e.lhs(), dim, base_extent);
      if (!span) return false;
      return collect_splits(e.lhs(), dim, ceil_div(*span, e.rhs().constant_value()), lower * e.rhs().constant_value(), out);
    }
    case ExprKind::Mod: {
      if (!e.rhs().is_constant() || e.rhs().constant_value() <= 0) return false;
      auto span = compute_span(e.lhs(), dim, base_extent);
      if (!span) return false;
      return collect_splits(e.lhs(), dim, std::min<int64_t>(*span, e.rhs().constant_value()), lower, out);
    }
    default: return false;
  }
}
}  // namespace detail

// Product of the extents of the distinct (lower factor, extent) pieces into which the map's results split dim `pos`
// of extent `extent`: for maps that use the pieces of a dim as digits this is the number of distinct results along it
// (computeUsedExtentForDim, :181-218).  No map: 1.  nullopt: the map cannot be analysed.
inline std::optional<int64_t> compute_used_extent_for_dim(const AffineMap& map, int pos, int64_t extent) {
  if (!map) return 1;
  if (extent <= 0 || pos < 0 || pos >= map.num_dims()) return std::nullopt;
  std::vector<std::pair<int64_t, int64_t>> splits;
  for (const AffineExpr& r : map.impl->results) {
    if (!detail::uses_dim(r, pos)) continue;
    if (!detail::collect_splits(r, pos, extent, 1, splits)) return std::nullopt;
  }
  if (splits.empty()) return 1;
  std::set<std::pair<int64_t, int64_t>> seen;
  int64_t used = 1;
  for (const auto& s : splits) {
    if (!seen.insert(s).second) continue;
    if (s.second <= 0) return std::nullopt;
    used *= s.second;
  }
  return used;
}

// ------------------------------------------------------------------ FriskOps_Reduce.cpp
// The map with dim `remove` taken out: later dims shift down, and a placeholder dim appended at the end stands for
// the removed one, as `placeholder mod extent` (or floordiv) -- 0 when the extent is 1 (remapReduceDimension, :51-107).
inline AffineMap remap_reduce_dimension(const AffineMap& map, int remove, int64_t extent, bool use_floor_div) {
  if (!map || remove >= map.num_dims()) return AffineMap();
  const int src_dims = map.num_dims(), placeholder = src_dims - 1;
  std::vector<AffineExpr> dims, syms;
  for (int i = 0; i < src_dims; ++i) {
    if (i < remove) dims.push_back(AffineExpr::dim(i));
    else if (i == remove) {
      AffineExpr p = AffineExpr::dim(placeholder);
      if (extent < 0) dims.push_back(p);
      else if (extent == 1) dims.push_back(AffineExpr::constant(0));
      else dims.push_back(use_floor_div ? p.floor_div(AffineExpr::constant(extent)) : p.mod(AffineExpr::constant(extent)));
    } else dims.push_back(AffineExpr::dim(i - 1));
  }
  for (int i = 0; i < map.num_symbols(); ++i) syms.push_back(AffineExpr::symbol(i));
  std::vector<AffineExpr> results;
  for (const AffineExpr& r : map.impl->results) results.push_back(r.replace_dims_and_symbols(dims, syms));
  return AffineMap(src_dims, map.num_symbols(), results);
}

// The last dim (the placeholder) goes away: replaced by 0, or by a new trailing symbol when the map uses it and
// `keep_symbol` (condensePlaceholderDimension, :121-163).
inline AffineMap condense_placeholder_dimension(const AffineMap& map, bool keep_symbol) {
  if (!map) return AffineMap();
  const int n = map.num_dims();
  if (n == 0) return map;
  const int placeholder = n - 1;
  bool used = false;
  for (const AffineExpr& r : map.impl->results) used = used || detail::uses_dim(r, placeholder);
  int syms_out = map.num_symbols();
  AffineExpr value = AffineExpr::constant(0);
  if (keep_symbol && used) value = AffineExpr::symbol(syms_out++);
  std::vector<AffineExpr> dims, syms;
  for (int i = 0; i < n; ++i) dims.push_back(i < placeholder ? AffineExpr::dim(i) : value);
  for (int i = 0; i < map.num_symbols(); ++i) syms.push_back(AffineExpr::symbol(i));
  std::vector<AffineExpr> results;
  for (const AffineExpr& r : map.impl->results) results.push_back(r.replace_dims_and_symbols(dims, syms));
  return AffineMap(n - 1, syms_out, results);
}

// ReduceOp::inferLayout (:214-357) for a source and a destination in registers (the reference does nothing for other
// memory spaces).  The destination keeps the source's maps with the reduced dim removed; in the thread map the reduced
// dim survives as a symbol ("any of these threads"), and replicate grows by the number of distinct threads along it.
// Errors carry the reference's diagnostics.  `threads` <= 0: unknown.  `existing`: a layout the destination already
// has; it must agree (checkLayoutCompatibility, :185-209) and is kept.
inline LayoutAttr infer_reduce_layout(const LayoutAttr& src, const std::vector<int64_t>& src_shape, const std::vector<int64_t>& dst_shape, int64_t dim,
                                      int64_t threads, const LayoutAttr* existing = nullptr) {
  if (!src.index || !src.thread) return LayoutAttr::none();  // nothing to infer from
  if (src.shape.empty()) throw std::invalid_argument("source layout missing input shape metadata");
  if (src.shape.size() != src_shape.size()) throw std::invalid_argument("source layout rank does not match source memref rank");
  if (dim < 0 || dim >= (int64_t)src_shape.size()) throw std::invalid_argument("invalid reduce dimension " + std::to_string(dim));
  const int64_t extent = src_shape[(size_t)dim];
  if (extent < 0) throw std::invalid_argument("layout inference requires static extent along the reduce dimension");
  if (extent == 0) throw std::invalid_argument("reduce extent must be positive for layout inference");
  AffineMap index = remap_reduce_dimension(src.index, (int)dim, extent, false);
  AffineMap thread = remap_reduce_dimension(src.thread, (int)dim, extent, false);
  int64_t factor = 1;
  if (thread) {
    if (thread.num_dims() == 0) throw std::invalid_argument("thread layout missing placeholder dimension");
    auto used = compute_used_extent_for_dim(thread, thread.num_dims() - 1, extent);
    if (!used) throw std::invalid_argument("unable to analyze reduce dimension usage in thread map for layout inference");
    factor = std::max<int64_t>(1, *used);
  }
  AffineMap dst_index = condense_placeholder_dimension(index, false), dst_thread = condense_placeholder_dimension(thread, true);
  if (!dst_index || !dst_thread) throw std::invalid_argument("failed to synthesize destination layout for reduce op");
  int64_t base = 1;
  if (src.replicate) {
    if (*src.replicate <= 0) throw std::invalid_argument("source layout replicate extent must be positive");
    base = *src.replicate;
  }
  const int64_t replicate = base * factor;
  if (threads > 0 && threads % replicate != 0 && replicate % threads != 0)
    throw std::invalid_argument("reduce layout inference requires thread count divisible by replicate extent (threads=" + std::to_string(threads) +
                                ", replicate=" + std::to_string(replicate) + ")");
  LayoutAttr dst;
  dst.shape = dst_shape.empty() ? std::vector<int64_t>{1} : dst_shape;
  dst.index = dst_index;
  dst.thread = dst_thread;
  dst.replicate = replicate;
  if (existing && *existing) {
    auto conflict = [&](const char* what) {
      return std::invalid_argument(std::string("destination layout conflicts with reduce inference: ") + what + "\nexpected=" + dst.debug() +
                                   "\nactual=" + existing->debug());
    };
    if (dst.shape != existing->shape) throw conflict("input shapes disagree");
    if (!dst.index.equals(existing->index)) throw conflict("forward index maps differ");
    if (!dst.thread.equals(existing->thread)) throw conflict("thread maps differ");
    if (existing->replicate && *dst.replicate > *existing->replicate) throw conflict("existing layout replicates fewer lanes than inferred");
    return *existing;
  }
  return dst;
}

// ------------------------------------------------------------------ FriskOps.cpp:641-823
// row-major index map over all dims, optionally a thread map that puts everything on thread 0 (buildDefaultLinearLayout, :716-747)
inline LayoutAttr default_linear_layout(const std::vector<int64_t>& shape, bool attach_thread_map) {
  for (int64_t d : shape)
    if (d < 0) return LayoutAttr::none();
  LayoutAttr l;
  l.shape = shape.empty() ? std::vector<int64_t>{1} : shape;
  AffineExpr e = AffineExpr::constant(0);
  int64_t stride = 1;
  for (int i = (int)l.shape.size() - 1; i >= 0; --i) {
    e = e + AffineExpr::dim(i) * stride;
    stride *= std::max<int64_t>(1, l.shape[(size_t)i]);
  }
  l.index = AffineMap((int)l.shape.size(), 0, {e});
  if (attach_thread_map) l.thread = AffineMap((int)l.shape.size(), 0, {AffineExpr::constant(0)});
  return l;
}

// Default layout of an alloc_buffer that no GEMM uses (inferLayoutForAllocBuffer, :792-823):
//   shared  the last two dims row-major, rows padded by 128 bits when a row is a multiple of 256 bits
//           (buildSharedLayoutForType :662-674, buildLinearLayoutAttr :641-660); rank < 2: plain row-major
//   local   the last two dims row-major in registers, lane = (row mod min(rows,16)) * laneN + col mod laneN with
//           laneN = min(cols, 8) clamped so that a wave holds the lane grid (buildFragmentLayoutAttr :676-704)
//   global  plain row-major
// A buffer of one element is replicated over all `thread_count` threads (:815-820).
inline LayoutAttr default_buffer_layout(MemorySpace space, const std::vector<int64_t>& shape, int element_bits, int wave_size, int64_t thread_count) {
  LayoutAttr l = LayoutAttr::none();
  const bool matrix = shape.size() >= 2 && shape[shape.size() - 2] >= 0 && shape[shape.size() - 1] >= 0;
  const int64_t rows = matrix ? shape[shape.size() - 2] : 0, cols = matrix ? shape[shape.size() - 1] : 0;
  AffineExpr row = AffineExpr::dim(0), col = AffineExpr::dim(1);
  if (space == MemorySpace::Shared) {
    if (matrix) {
      int64_t padded = cols;
      if (element_bits > 0 && (element_bits * cols) % 256 == 0) padded += 128 / element_bits;
      l = LayoutAttr();
      l.shape = {rows, cols};
      l.index = AffineMap(2, 0, {row * padded + col});
    } else {
      l = default_linear_layout(shape, false);
    }
  } else if (space == MemorySpace::Local) {
    if (matrix) {
      l = LayoutAttr();
      l.shape = {rows, cols};
      l.index = AffineMap(2, 0, {row * cols + col});
      const int64_t lane_m = std::max<int64_t>(1, std::min<int64_t>(rows, 16));
      int64_t lane_n = std::max<int64_t>(1, std::min<int64_t>(cols, 8));
      if (lane_m * lane_n > wave_size) lane_n = std::max<int64_t>(1, wave_size / lane_m);
      l.thread = AffineMap(2, 0, {row.mod(AffineExpr::constant(lane_m)) * lane_n + col.mod(AffineExpr::constant(lane_n))});
      l.replicate = 1;
    } else {
      l = default_linear_layout(shape, true);
    }
  } else {
    l = default_linear_layout(shape, false);
  }
  if (!l) return l;
  int64_t elements = 1;
  bool is_static = true;
  for (int64_t d : shape) { if (d < 0) is_static = false; else elements *= d; }
  if (is_static && elements == 1 && std::max<int64_t>(1, thread_count) > 1) l.replicate = std::max<int64_t>(1, thread_count);
  return l;
}

// ------------------------------------------------------------------ the MFMA accumulator fragment
// A wave owns a (BM / WM) x (BN / WN) block as 32x32 MFMA atoms kept transposed: inside an atom, element (m, n)
// lives in lane (m mod 32) + 32 * ((n mod 8) floordiv 4), accumulator register (n mod 4) + 4 * ((n mod 32) floordiv 8).
inline LayoutAttr accumulator_layout(int64_t bm, int64_t bn, int64_t wm, int64_t wn) {
  if (wm <= 0 || wn <= 0 || bm % (wm * 32) || bn % (wn * 32)) throw std::invalid_argument("the wave grid must split the tile into whole 32x32 atoms");
  const int64_t wtm = bm / wm, wtn = bn / wn, an = wtn / 32;
  auto c = [](int64_t v) { return AffineExpr::constant(v); };
  AffineExpr i = AffineExpr::dim(0), j = AffineExpr::dim(1);
  AffineExpr lane = i.mod(c(32)) + j.mod(c(8)).floor_div(c(4)) * 32;
  AffineExpr wave = i.floor_div(c(wtm)) * wn + j.floor_div(c(wtn));
  AffineExpr reg = j.mod(c(4)) + j.mod(c(32)).floor_div(c(8)) * 4;
  AffineExpr atom = i.mod(c(wtm)).floor_div(c(32)) * an + j.mod(c(wtn)).floor_div(c(32));
  LayoutAttr l;
  l.shape = {bm, bn};
  l.index = AffineMap(2, 0, {reg + atom * 16});
  l.thread = AffineMap(2, 0, {lane + wave * 64});
  l.replicate = 1;
  return l;
}

}  // namespace frisk_ir
