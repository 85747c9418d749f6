"""The builder's affine expressions against MLIR's own output, as the reference holds it: the layout strings of
tests/golden/nvidia_gemm_layouts.json were printed by MLIR after MLIR's construction-time simplifications.  Driving the
oracle's restatement of the reference's layout construction (oracle/layouts.py: the same operations in the same order as
lib/Dialect/Frisk/IR/FriskOps.cpp:106-618) with this build's AffineExpr objects instead of numbers must reproduce those
strings character for character: that pins the folding constructor (constants and symbols to the right, merged
constants, `e - q * (e floordiv q)` = `e mod q`, ...) and the printer's parenthesisation."""
import json
import os

import pytest

import frisk_amd  # noqa: F401
import frisk as F
from oracle import layouts as L

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "nvidia_gemm_layouts.json")))
POLICY = {"Square": L.SQUARE, "FullRow": L.FULL_ROW, "FullCol": L.FULL_COL}


def _map_text(results):
    return "affine_map<%s>" % F.AffineMap.get(2, 0, list(results))


@pytest.mark.parametrize("case", GOLD["cases"], ids=[c["name"] for c in GOLD["cases"]])
def test_layout_strings_are_reproduced_character_for_character(case):
    d0, d1 = F.get_affine_dim_expr(0), F.get_affine_dim_expr(1)
    got = L.infer_gemm_layouts(case["target"], case["threads"], case["M"], case["N"], case["K"], case["spaces"], case["element_bits"],
                               case["transA"], case["transB"], POLICY[case["policy"]])
    for op, gold in case["layouts"].items():
        if got[op][0] == "shared":
            assert _map_text(got[op][2](d0, d1)) == gold["index"], (case["name"], op)
        else:
            frag = got[op][1]
            assert _map_text([frag.index(d0, d1)]) == gold["index"], (case["name"], op, "index")
            if "thread" in gold:
                assert _map_text([frag.thread(d0, d1)]) == gold["thread"], (case["name"], op, "thread")


def test_constructor_simplifications():
    d0, d1, s0 = F.get_affine_dim_expr(0), F.get_affine_dim_expr(1), F.get_affine_symbol_expr(0)
    c = F.get_affine_constant_expr
    assert str(d0 - c(8) * d0.floor_div(8)) == "d0 mod 8"                      # the reference's modConst (FriskOps.cpp:119-121)
    assert str((d0 + 2) + 3) == "d0 + 5" and str((d0 + 2) + d1) == "d0 + d1 + 2"
    assert str(5 * d0) == "d0 * 5" and str((d0 * 2) * 3) == "d0 * 6" and str((d0 * 2) * d1) == "(d0 * d1) * 2"
    assert str(s0 + d0) == "d0 + s0" and str(s0 * d0) == "d0 * s0"
    assert str(d0 * 3 + d0 * 4) == "d0 * 7" and str(d0 + d0) == "d0 * 2" and str(d0 - d0) == "0"
    assert str((d0 * 8).floor_div(4)) == "d0 * 2" and str((d0 * 8 + d1).floor_div(8)) == "d0 + d1 floordiv 8"
    assert str((d0 * 8) % 4) == "0" and str((d0 * 8 + d1) % 8) == "d1 mod 8" and str((d0 % 8) % 4) == "d0 mod 4"
    assert str(d0 % 1) == "0" and str(d0.floor_div(1)) == "d0" and str((d0 * 6).ceil_div(3)) == "d0 * 2"
    assert str(-d0) == "-d0" and str(d0 - d1) == "d0 - d1" and str(d0 - 3) == "d0 - 3"


def test_affine_api_of_the_reference_script():
    """the call sequence of test/python/map_expr_test.py:3-24 and the rest of the surface of ffi/ir.cpp:646-881"""
    ctx = F.context()
    b = F.builder(ctx)
    dim0, sym, c0, c5 = b.get_affine_dim_expr(0), b.get_affine_symbol_expr(0), b.get_affine_constant_expr(0), b.get_affine_constant_expr(5)
    e = dim0 * c5 + sym + c0
    assert str(e) == "d0 * 5 + s0" and e.get_kind() == F.AffineExprKind.Add == F.Add
    e2 = F.get_affine_binary_op_expr(e.get_kind(), e, e)
    assert str(e2) == "(d0 * 5 + s0) * 2"
    be = e.as_binary()
    assert str(be.get_lhs()) == "d0 * 5" and str(be.get_rhs()) == "s0" and e.as_dim() is None and e.as_constant() is None
    assert dim0.as_dim().get_position() == 0 and sym.as_symbol().get_position() == 0 and c5.as_constant().get_value() == 5
    m = F.AffineMap.get(1, 1, [e2], ctx)
    assert str(m) == "(d0)[s0] -> ((d0 * 5 + s0) * 2)" and repr(m).startswith("AffineMap(")
    assert m.get_result(0) == e2 and m.get_results() == [e2] and (m.get_num_dims(), m.get_num_symbols(), m.get_num_inputs()) == (1, 1, 2)
    # queries
    assert (dim0 * 12).get_largest_known_divisor() == 12 and (dim0 * 12 + 8).get_largest_known_divisor() == 4 and (dim0 * 12).is_multiple_of(6)
    assert e.is_pure_affine() and not (dim0 * dim0).is_pure_affine() and (sym * 3 + 1).is_symbolic_or_constant() and not e.is_symbolic_or_constant()
    assert e.is_function_of_dim(0) and not e.is_function_of_dim(1) and e.is_function_of_symbol(0)
    d1 = b.get_affine_dim_expr(1)
    assert str(e.replace_dims([d1 + 1])) == "(d1 + 1) * 5 + s0" and str(e.replace_symbols([c5])) == "d0 * 5 + 5"
    assert str(e.replace(sym, d1)) == "d0 * 5 + d1" and str(e.shift_dims(1, 2)) == "d2 * 5 + s0" and str(e.shift_symbols(1, 1)) == "d0 * 5 + s1"
    assert str(e.compose(F.AffineMap.get(2, 0, [d1 * 2]))) == "d1 * 10 + s0"
    assert str(F.get_affine_expr_from_flat_form([2, 0, 3, 7], 2, 1)) == "d0 * 2 + s0 * 3 + 7"
    assert [x.as_constant().get_value() for x in F.get_affine_constant_exprs([1, 2, 3])] == [1, 2, 3]
    # maps
    assert str(F.AffineMap.get_constant_map(4, ctx)) == "() -> (4)" and F.AffineMap.get_constant_map(4, ctx).get_single_constant_result() == 4
    assert str(F.AffineMap.get_minor_identity_map(3, 2, ctx)) == "(d0, d1, d2) -> (d1, d2)" and F.AffineMap.get_minor_identity_map(3, 2, ctx).is_minor_identity()
    p = F.AffineMap.get_permutation_map([2, 0, 1], ctx)
    assert str(p) == "(d0, d1, d2) -> (d2, d0, d1)" and p.is_permutation() and p.is_projected_permutation() and not p.is_identity()
    assert p.get_dim_position(0) == 2 and p.get_result_position(F.get_affine_dim_expr(0)) == 1 and p.get_result_position(F.get_affine_dim_expr(5)) is None
    assert F.AffineMap.get(ctx).is_empty() and F.AffineMap.get(2, 1, ctx).get_num_results() == 0 and not F.AffineMap()
    assert F.AffineMap.get(0, 0, [c5, c0]).is_constant() and F.AffineMap.get(0, 0, [c5, c0]).get_constant_results() == [5, 0]
    assert F.AffineMap.get(0, 2, [F.get_affine_symbol_expr(0), F.get_affine_symbol_expr(1)]).is_symbol_identity()
    with pytest.raises(ValueError):
        F.AffineMap.get_permutation_map([0, 0], ctx)
