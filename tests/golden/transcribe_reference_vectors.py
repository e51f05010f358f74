#!/usr/bin/env python3
"""Writes tests/golden/reference_vectors.json: known-answer vectors TRANSCRIBED (as data) from the reference's own
documentation and docstrings — the only literal expected values the reference holds for the tensor-backend path.
Nothing is executed from the reference; each entry cites the file:line it was read from.

Format of an entry: id, cite, fn (a key of tests/golden_ops.py), args (list of {dtype, data} or plain scalars/lists),
expect ({dtype, data} or a plain value), atol (0 = exact).  Values printed with 4-5 significant digits in the docs carry
atol 6e-5 (relative for large magnitudes via rtol).  Three docstring values are typos, not behaviour, and are corrected
from the closed form: acos(-1) printed 3.15159 (pi = 3.14159), log 4 printed 1.38529 (1.38629), tan(+-1.57079) printed
158057.9134 (158057.913...).  The corrected value is stored and the printed one kept under "printed".
"""
import json
import os

D = "Tensor/Tensor.Docs/articles/"
T = "Tensor/Tensor/Tensor.fs"


def t(dtype, data):
    return {"dtype": dtype, "data": data}


V = []


def add(id, cite, fn, args, expect, atol=0.0, rtol=0.0, **extra):
    V.append(dict(id=id, cite=cite, fn=fn, args=args, expect=expect, atol=atol, rtol=rtol, **extra))


f64, i32, i64, b = "float64", "int32", "int64", "bool"
A567 = t(f64, [5.0, 6.0, 7.0])
A234 = t(f64, [2.0, 3.0, 4.0])
M2x4 = t(f64, [[1.0, 2.0, 3.0, 4.0], [5.0, 6.0, 7.0, 8.0]])
HALFPI = t(f64, [-1.57079, 0.0, 1.57079])

# --- Guide-Operations.md -------------------------------------------------------------------------------------------------
add("ops_add", D + "Guide-Operations.md:10-22", "add", [t(f64, [0.0, 1.0, 2.0, 3.0]), t(f64, [0.0, 10.0, 20.0, 30.0])], t(f64, [0.0, 11.0, 22.0, 33.0]))
add("ops_scalar_mul", D + "Guide-Operations.md:28-30", "mul_scalar", [t(f64, [0.0, 1.0, 2.0, 3.0]), 100.0], t(f64, [0.0, 100.0, 200.0, 300.0]))
add("ops_broadcast_add", D + "Guide-Operations.md:44-75", "add",
    [t(f64, [[[0.0], [0.1], [0.2]], [[1.0], [1.1], [1.2]], [[2.0], [2.1], [2.2]], [[3.0], [3.1], [3.2]]]), t(f64, [0.0, 10.0])],
    t(f64, [[[0.0, 10.0], [0.1, 10.1], [0.2, 10.2]], [[1.0, 11.0], [1.1, 11.1], [1.2, 11.2]],
            [[2.0, 12.0], [2.1, 12.1], [2.2, 12.2]], [[3.0, 13.0], [3.1, 13.1], [3.2, 13.2]]]), atol=1e-12)
add("ops_sin", D + "Guide-Operations.md:88-90", "sin", [t(f64, [0.0, 11.0, 22.0, 33.0])], t(f64, [0.0, -1.0, -0.009, 0.9999]), atol=6e-4)
add("ops_fill_multiply_inplace", D + "Guide-Operations.md:103-115", "fill_multiply_twice",
    [t(f64, [-1.0, -1.0, 29.0, 40.0]), t(f64, [0.0, 1.0, 2.0, 3.0]), t(f64, [0.0, 10.0, 20.0, 30.0])], t(f64, [0.0, 100.0, 800.0, 2700.0]))
add("ops_dot", D + "Guide-Operations.md:129-148", "dot",
    [t(f64, [[0.0, 1.0, 2.0], [3.0, 4.0, 5.0], [6.0, 7.0, 8.0], [9.0, 10.0, 11.0], [12.0, 13.0, 14.0]]),
     t(f64, [[1.1, 0.1, 0.1], [0.1, 1.1, 0.1], [0.1, 0.1, 1.1]])],
    t(f64, [[0.3, 1.3, 2.3], [4.2, 5.2, 6.2], [8.1, 9.1, 10.1], [12.0, 13.0, 14.0], [15.9, 16.9, 17.9]]), atol=1e-12)

# --- Guide-Reductions.md -------------------------------------------------------------------------------------------------
G4 = t(i32, [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9, 10, 11], [12, 13, 14, 15]])
add("red_sum", D + "Guide-Reductions.md:9-10", "sum", [t(f64, [0.0, 11.0, 22.0, 33.0])], 66.0)
add("red_sum_axis0", D + "Guide-Reductions.md:21-29", "sumAxis", [G4, 0], t(i32, [24, 28, 32, 36]))
add("red_max_axis0", D + "Guide-Reductions.md:43-45", "maxAxis", [G4, 0], t(i32, [12, 13, 14, 15]))

# --- Guide-Logic.md ------------------------------------------------------------------------------------------------------
J = t(b, [True, False, True, False])
add("logic_equal", D + "Guide-Logic.md:12-16", "eq", [t(i32, [0, 1, 2, 3]), t(i32, [0, 10, 2, 30])], J)
add("logic_not", D + "Guide-Logic.md:33-35", "not", [J], t(b, [False, True, False, True]))
add("logic_and_not", D + "Guide-Logic.md:36-37", "and_not_self", [J], t(b, [False, False, False, False]))
TI = t(b, [[True, False, True, False], [False, True, True, False]])
add("logic_true_idx", D + "Guide-Logic.md:46-53", "trueIdx", [TI], t(i64, [[0, 0], [0, 2], [1, 1], [1, 2]]))
add("logic_if_then_else", D + "Guide-Logic.md:66-71", "ifThenElse", [t(b, [True, False, False]), A234, A567], t(f64, [2.0, 6.0, 7.0]))
MA = t(f64, [[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
MM = t(b, [[True, True, False], [False, False, True]])
add("logic_mask_get", D + "Guide-Logic.md:85-91", "mask_get", [MA, MM], t(f64, [1.0, 2.0, 6.0]))
add("logic_mask_nomask", D + "Guide-Logic.md:97-100", "mask_get_rows", [MA, t(b, [True, False])], t(f64, [[1.0, 2.0, 3.0]]))
add("logic_mask_set", D + "Guide-Logic.md:109-114", "mask_set", [MA, MM, t(f64, [8.0, 9.0, 0.0])], t(f64, [[8.0, 9.0, 3.0], [4.0, 5.0, 0.0]]))
add("logic_all", D + "Guide-Logic.md:126-128", "all", [J], False)
add("logic_all_axis0", D + "Guide-Logic.md:134-138", "allAxis", [t(b, [[True, False, False, True], [True, False, True, False]]), 0], t(b, [True, False, False, False]))

# --- Guide-Index.md ------------------------------------------------------------------------------------------------------
add("idx_argmax", D + "Guide-Index.md:21-26", "argMax", [M2x4], [1, 3])
add("idx_argmax_axis1", D + "Guide-Index.md:33-35", "argMaxAxis", [M2x4, 1], t(i64, [3, 3]))
F2 = t(f64, [[1.0, 2.0, 3.0, 4.0], [5.0, 6.0, 7.0, 3.0]])
add("idx_try_find", D + "Guide-Index.md:44-49", "tryFind", [F2, 3.0], [0, 2])
add("idx_find_axis1", D + "Guide-Index.md:52-57", "findAxis", [F2, 3.0, 1], t(i64, [2, 3]))
SRC = t(f64, [[0.0, 0.1, 0.2, 0.3], [1.0, 1.1, 1.2, 1.3], [2.0, 2.1, 2.2, 2.3]])
add("idx_gather", D + "Guide-Index.md:87-94", "gather2", [SRC, t(i64, [1, 2, 0, 0]), t(i64, [3, 1, 0, 3])], t(f64, [1.3, 2.1, 0.0, 0.3]))
add("idx_gather_none", D + "Guide-Index.md:102-105", "gather_none_first", [SRC, t(i64, [3, 1, 0])], t(f64, [0.3, 1.1, 2.0]))
add("idx_scatter", D + "Guide-Index.md:118-133", "scatter2",
    [SRC, t(i64, [[0, 0, 0, 0], [2, 2, 2, 2], [1, 1, 1, 1]]), t(i64, [[3, 3, 3, 3], [0, 1, 2, 3], [0, 1, 2, 3]]), [4, 4]],
    t(f64, [[0.0, 0.0, 0.0, 0.6], [2.0, 2.1, 2.2, 2.3], [1.0, 1.1, 1.2, 1.3], [0.0, 0.0, 0.0, 0.0]]), atol=1e-12)

# --- Guide-Shape.md / layout docstrings (pure layout algebra) ----------------------------------------------------------------
add("shape_permute_axes", D + "Guide-Shape.md:82-83", "permute_shape", [[4, 2, 2], [2, 0, 1]], [2, 2, 4])
add("shape_permute_axes_doc", T + ":588-591", "permute_shape", [[0, 11, 22, 33, 44], [3, 2, 4, 1, 0]], [44, 33, 11, 0, 22])
add("shape_swap_dim", T + ":567-570", "swap_shape", [[2, 3, 4], 0, 2], [4, 3, 2])
add("shape_reshape_remainder", T + ":528-532", "reshape_shape", [[2, 3, 4], [2, -9223372036854775805, 1]], [2, 12, 1])
add("shape_broadcast_in_dims", T + ":429-433", "broadcast_in_dims", [[1, 7, 1], [3, 4, 5], [0, 2]], [[3, 7, 5], [3, 4, 5]])
add("shape_broadcast_to", T + ":466-469", "broadcast_to", [[1, 7, 1], [2, 7, 3]], [2, 7, 3])
add("shape_pad_to_same", T + ":355-359", "pad_to_same", [[4, 5], [3, 4, 5]], [[1, 4, 5], [3, 4, 5]])
add("shape_reverse_axis", T + ":605-608", "reverse0", [t(i32, [0, 1, 2, 3])], t(i32, [3, 2, 1, 0]))

# --- Tensor.fs docstrings: unary -----------------------------------------------------------------------------------------------
add("doc_convert", T + ":794-797", "convert_f64", [t(i32, [1, 2, 3])], t(f64, [1.0, 2.0, 3.0]))
add("doc_unary_plus", T + ":821-824", "pos", [A567], A567)
add("doc_unary_minus", T + ":846-849", "neg", [A567], t(f64, [-5.0, -6.0, -7.0]))
add("doc_abs", T + ":869-872", "abs", [t(i32, [-2, -1, 1])], t(i32, [2, 1, 1]))
add("doc_sgn", T + ":891-894", "sgn", [t(i32, [-2, -1, 0, 2])], t(i32, [-1, -1, 0, 1]))
add("doc_log", T + ":914-917", "log", [t(f64, [1.0, 2.71828, 4.0])], t(f64, [0.0, 1.0, 1.38629]), atol=6e-5, printed=[0.0, 1.0, 1.38529])
add("doc_log10", T + ":936-939", "log10", [t(f64, [1.0, 10.0, 100.0])], t(f64, [0.0, 1.0, 2.0]), atol=1e-15)
add("doc_exp", T + ":959-962", "exp", [t(f64, [-1.0, 0.0, 1.0, 10.0])], t(f64, [0.36787, 1.0, 2.71828, 22026.4657]), atol=6e-5, rtol=1e-8)
add("doc_sin", T + ":982-985", "sin", [HALFPI], t(f64, [-1.0, 0.0, 1.0]), atol=6e-5)
add("doc_cos", T + ":1005-1008", "cos", [HALFPI], t(f64, [0.0, 1.0, 0.0]), atol=6e-5)
add("doc_tan", T + ":1028-1031", "tan", [HALFPI], t(f64, [-158057.9134, 0.0, 158057.9134]), rtol=1e-6)
add("doc_asin", T + ":1051-1054", "asin", [t(f64, [-1.0, 0.0, 1.0])], t(f64, [-1.57079, 0.0, 1.57079]), atol=6e-5)
add("doc_acos", T + ":1074-1077", "acos", [t(f64, [-1.0, 0.0, 1.0])], t(f64, [3.14159, 1.57079, 0.0]), atol=6e-5, printed=[3.15159, 1.57079, 0.0])
add("doc_atan", T + ":1097-1100", "atan", [t(f64, [-1.0, 0.0, 1.0])], t(f64, [-0.78539, 0.0, 0.78539]), atol=6e-5)
add("doc_sinh", T + ":1120-1123", "sinh", [HALFPI], t(f64, [-2.30128, 0.0, 2.30128]), atol=6e-5)
add("doc_cosh", T + ":1143-1146", "cosh", [HALFPI], t(f64, [2.50916, 1.0, 2.50916]), atol=6e-5)
add("doc_tanh", T + ":1166-1169", "tanh", [HALFPI], t(f64, [-0.91715, 0.0, 0.91715]), atol=6e-5)
add("doc_sqrt", T + ":1189-1192", "sqrt", [t(f64, [1.0, 4.0, 16.0])], t(f64, [1.0, 2.0, 4.0]))
R = t(f64, [-3.0, -2.7, 2.7, 3.0])
add("doc_ceil", T + ":1211-1214", "ceiling", [R], t(f64, [-3.0, -2.0, 3.0, 3.0]))
add("doc_floor", T + ":1234-1237", "floor", [R], t(f64, [-3.0, -3.0, 2.0, 3.0]))
add("doc_round", T + ":1257-1260", "round", [R], t(f64, [-3.0, -3.0, 3.0, 3.0]))
add("doc_truncate", T + ":1279-1282", "truncate", [R], t(f64, [-3.0, -2.0, 2.0, 3.0]))
add("doc_is_finite", T + ":1303-1306", "isFinite", [t(f64, ["-inf", -3.0, "nan", 3.0, "inf"])], t(b, [False, True, False, True, False]))
add("doc_negate", T + ":1326-1329", "not", [t(b, [True, False])], t(b, [False, True]))

# --- Tensor.fs docstrings: binary, logic, comparison ----------------------------------------------------------------------------
add("doc_add", T + ":1350-1354", "add", [A567, A234], t(f64, [7.0, 9.0, 11.0]))
add("doc_sub", T + ":1393-1397", "sub", [A567, A234], t(f64, [3.0, 3.0, 3.0]))
add("doc_mul", T + ":1436-1440", "mul", [A567, A234], t(f64, [10.0, 18.0, 28.0]))
add("doc_div", T + ":1479-1483", "div", [A567, A234], t(f64, [2.5, 2.0, 1.75]))
add("doc_mod", T + ":1522-1526", "mod", [A567, A234], t(f64, [1.0, 0.0, 3.0]))
add("doc_pow", T + ":1565-1569", "pow", [A567, A234], t(f64, [25.0, 216.0, 2401.0]), rtol=1e-14)
BA = t(b, [True, True, False, False])
BB = t(b, [True, False, True, False])
add("doc_and", T + ":1610-1614", "and", [BA, BB], t(b, [True, False, False, False]))
add("doc_or", T + ":1654-1658", "or", [BA, BB], t(b, [True, True, True, False]))
add("doc_xor", T + ":1698-1702", "xor", [BA, BB], t(b, [False, True, True, False]))
C246 = t(f64, [2.0, 4.0, 6.0])
C147 = t(f64, [1.0, 4.0, 7.0])
add("doc_eq", T + ":1742-1746", "eq", [C246, C147], t(b, [False, True, False]))
add("doc_ne", T + ":1786-1790", "ne", [C246, C147], t(b, [True, False, True]))
add("doc_lt", T + ":1830-1834", "lt", [C246, C147], t(b, [False, False, True]))
add("doc_le", T + ":1873-1877", "le", [C246, C147], t(b, [False, True, True]))
add("doc_gt", T + ":1917-1921", "gt", [C246, C147], t(b, [True, False, False]))
add("doc_ge", T + ":1961-1965", "ge", [C246, C147], t(b, [True, True, False]))
add("doc_max_elemwise", T + ":2004-2008", "maxElemwise", [A567, A234], A567)
add("doc_min_elemwise", T + ":2033-2037", "minElemwise", [A567, A234], A234)
add("doc_if_then_else", T + ":2064-2069", "ifThenElse", [t(b, [True, False, False]), A234, A567], t(f64, [2.0, 6.0, 7.0]))

# --- Tensor.fs docstrings: counting and reductions ------------------------------------------------------------------------------
add("doc_count_true_axis", T + ":2213-2217", "countTrueAxis", [TI, 1], t(i64, [2, 2]))
add("doc_count_true", T + ":2235-2239", "countTrue", [TI], 4)
add("doc_true_idx", T + ":2249-2256", "trueIdx", [TI], t(i64, [[0, 0], [0, 2], [1, 1], [1, 2]]))
add("doc_sum_axis", T + ":2277-2281", "sumAxis", [M2x4, 1], t(f64, [10.0, 26.0]))
add("doc_sum", T + ":2299-2303", "sum", [M2x4], 36.0)
add("doc_product_axis", T + ":2321-2325", "productAxis", [M2x4, 1], t(f64, [24.0, 1680.0]))
add("doc_product", T + ":2343-2347", "product", [M2x4], 40320.0)
add("doc_min_axis", T + ":2365-2369", "minAxis", [M2x4, 1], t(f64, [1.0, 5.0]))
add("doc_min", T + ":2387-2391", "min", [M2x4], 1.0)
add("doc_max_axis", T + ":2411-2415", "maxAxis", [M2x4, 1], t(f64, [4.0, 8.0]))
add("doc_max", T + ":2433-2437", "max", [M2x4], 8.0)
add("doc_arg_min_axis", T + ":2458-2462", "argMinAxis", [M2x4, 1], t(i64, [0, 0]))
add("doc_arg_max_axis", T + ":2484-2488", "argMaxAxis", [M2x4, 1], t(i64, [3, 3]))

if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(out, "w") as f:
        json.dump({"source": "DeepMLNet/DeepNet documentation and docstrings (transcribed data)", "vectors": V}, f, indent=1)
    print(f"wrote {len(V)} vectors to {out}")
