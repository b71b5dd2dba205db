"""Writes tests/golden/vectors.json: known-answer vectors the reference's own doctests and
regression tests hold for the hot path (inputs and expected outputs only -- data, no
code).  Short vectors are transcribed here with the file:line they come from; the long
expected vector of Issue137 is read out of the reference's test file, which is why this
script needs the reference tree (default /root/reference) and is run in the build
container only.  The parity tests read the committed JSON and never the reference.

Usage: python tests/golden/make_vectors.py [/path/to/reference]
"""
from __future__ import annotations

import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SRC = os.path.join(REF, "src", "Data", "Array", "Accelerate")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.json")

iota5x10 = [list(range(r * 10, r * 10 + 10)) for r in range(5)]
iota4x10 = [list(range(r * 10, r * 10 + 10)) for r in range(4)]

V = {}

# Language.hs:473-483  fold (+) 42 over the rows of a 5x10 iota matrix
V["fold_sum_seed42"] = {"cite": "Language.hs:473-483", "mat": iota5x10, "expected": [87, 187, 287, 387, 487]}
# Language.hs:516-518  maximum segment sum (non-commutative fold1 over 4-tuples)
V["mss"] = {"cite": "Language.hs:491-518", "vec": [-2, 1, -3, 4, -1, 2, 1, -5, 4, 0], "expected": 6}
# Language.hs:595-605  scanl
V["scanl_vec"] = {"cite": "Language.hs:595-597", "vec": list(range(10)), "seed": 10,
                  "expected": [10, 10, 11, 13, 16, 20, 25, 31, 38, 46, 55]}
V["scanl_mat"] = {"cite": "Language.hs:599-605", "mat": iota4x10, "seed": 0, "expected": [
    [0, 0, 1, 3, 6, 10, 15, 21, 28, 36, 45],
    [0, 10, 21, 33, 46, 60, 75, 91, 108, 126, 145],
    [0, 20, 41, 63, 86, 110, 135, 161, 188, 216, 245],
    [0, 30, 61, 93, 126, 160, 195, 231, 268, 306, 345]]}
# Language.hs:623-639  scanl'
V["scanl_prime_vec"] = {"cite": "Language.hs:623-628", "vec": list(range(10)), "seed": 0,
                        "expected": [0, 0, 1, 3, 6, 10, 15, 21, 28, 36], "expected_sum": 45}
V["scanl_prime_mat"] = {"cite": "Language.hs:630-639", "mat": iota4x10, "seed": 0, "expected": [
    [0, 0, 1, 3, 6, 10, 15, 21, 28, 36],
    [0, 10, 21, 33, 46, 60, 75, 91, 108, 126],
    [0, 20, 41, 63, 86, 110, 135, 161, 188, 216],
    [0, 30, 61, 93, 126, 160, 195, 231, 268, 306]], "expected_sum": [45, 145, 245, 345]}
# Language.hs:653-659  scanl1
V["scanl1_mat"] = {"cite": "Language.hs:653-659", "mat": iota4x10, "expected": [
    [0, 1, 3, 6, 10, 15, 21, 28, 36, 45],
    [10, 21, 33, 46, 60, 75, 91, 108, 126, 145],
    [20, 41, 63, 86, 110, 135, 161, 188, 216, 245],
    [30, 61, 93, 126, 160, 195, 231, 268, 306, 345]]}
# Test/NoFib/Misc/Scanl1.hs:32-39  257x31 scanl1 (+) of [1..] with a closed form
V["misc_scanl1"] = {"cite": "Test/NoFib/Misc/Scanl1.hs:32-39", "rows": 257, "cols": 31,
                    "closed_form": "out[i][j] = sum [1+i*cols .. 1+i*cols+j]"}
# Prelude.hs:689-708  foldSeg with an empty segment
V["foldseg_doctest"] = {"cite": "Prelude.hs:689-708", "mat": iota5x10, "seg": [1, 4, 0, 3], "expected": [
    [0, 10, 0, 18], [10, 50, 0, 48], [20, 90, 0, 78], [30, 130, 0, 108], [40, 170, 0, 138]]}
# Prelude.hs:958-991, 1117-1135, 1293-1312  segmented scans (same matrix and segments; one empty segment)
V["scanlseg_doctest"] = {"cite": "Prelude.hs:958-978", "mat": iota5x10, "seg": [1, 4, 0, 3], "seed": 0, "expected": [
    [0, 0, 0, 1, 3, 6, 10, 0, 0, 5, 11, 18], [0, 10, 0, 11, 23, 36, 50, 0, 0, 15, 31, 48],
    [0, 20, 0, 21, 43, 66, 90, 0, 0, 25, 51, 78], [0, 30, 0, 31, 63, 96, 130, 0, 0, 35, 71, 108],
    [0, 40, 0, 41, 83, 126, 170, 0, 0, 45, 91, 138]]}
V["scanl1seg_doctest"] = {"cite": "Prelude.hs:1117-1135", "mat": iota5x10, "seg": [1, 4, 0, 3], "expected": [
    [0, 1, 3, 6, 10, 5, 11, 18], [10, 11, 23, 36, 50, 15, 31, 48], [20, 21, 43, 66, 90, 25, 51, 78],
    [30, 31, 63, 96, 130, 35, 71, 108], [40, 41, 83, 126, 170, 45, 91, 138]]}
V["scanr1seg_doctest"] = {"cite": "Prelude.hs:1293-1312", "mat": iota5x10, "seg": [1, 4, 0, 3], "expected": [
    [0, 10, 9, 7, 4, 18, 13, 7], [10, 50, 39, 27, 14, 48, 33, 17], [20, 90, 69, 47, 24, 78, 53, 27],
    [30, 130, 99, 67, 34, 108, 73, 37], [40, 170, 129, 87, 44, 138, 93, 47]]}
# Prelude.hs:1014-1039, 1230-1257  scanl'Seg / scanr'Seg: scanned bodies and per-segment totals
V["scanlprimeseg_doctest"] = {"cite": "Prelude.hs:1014-1039", "mat": iota5x10, "seg": [1, 4, 0, 3], "seed": 0,
    "expected": [[0, 0, 1, 3, 6, 0, 5, 11], [0, 0, 11, 23, 36, 0, 15, 31], [0, 0, 21, 43, 66, 0, 25, 51],
                 [0, 0, 31, 63, 96, 0, 35, 71], [0, 0, 41, 83, 126, 0, 45, 91]],
    "expected_sums": [[0, 10, 0, 18], [10, 50, 0, 48], [20, 90, 0, 78], [30, 130, 0, 108], [40, 170, 0, 138]]}
V["scanrprimeseg_doctest"] = {"cite": "Prelude.hs:1230-1257", "mat": iota5x10, "seg": [1, 4, 0, 3], "seed": 0,
    "expected": [[0, 15, 11, 6, 0, 17, 9, 0], [0, 45, 31, 16, 0, 37, 19, 0], [0, 75, 51, 26, 0, 57, 29, 0],
                 [0, 105, 71, 36, 0, 77, 39, 0], [0, 135, 91, 46, 0, 97, 49, 0]],
    "expected_sums": [[2, 18, 0, 24], [12, 58, 0, 54], [22, 98, 0, 84], [32, 138, 0, 114], [42, 178, 0, 144]]}
# Prelude.hs:1175-1200  scanrSeg
V["scanrseg_doctest"] = {"cite": "Prelude.hs:1175-1200", "mat": iota5x10, "seg": [1, 4, 0, 3], "seed": 0, "expected": [
    [2, 0, 18, 15, 11, 6, 0, 0, 24, 17, 9, 0], [12, 0, 58, 45, 31, 16, 0, 0, 54, 37, 19, 0],
    [22, 0, 98, 75, 51, 26, 0, 0, 84, 57, 29, 0], [32, 0, 138, 105, 71, 36, 0, 0, 114, 77, 39, 0],
    [42, 0, 178, 135, 91, 46, 0, 0, 144, 97, 49, 0]]}
# Prelude.hs:656-662  foldAll
V["foldall_doctest"] = {"cite": "Prelude.hs:656-662", "vec": list(range(10)), "seed": 42, "expected_vec": 87.0,
                        "mat": iota5x10, "expected_mat": 1225.0}
# Prelude.hs:770-797  all even / any even along rows
evens_mat = [[1, 2, 3, 4, 5, 6, 7, 8, 9, 10], [1, 1, 1, 1, 1, 2, 2, 2, 2, 2], [2, 4, 6, 8, 10, 12, 14, 16, 18, 20],
             [1, 3, 5, 7, 9, 11, 13, 15, 17, 19]]
V["all_any_doctest"] = {"cite": "Prelude.hs:770-797", "mat": evens_mat, "all": [0, 0, 1, 0], "any": [1, 1, 1, 0]}
# Prelude.hs:822-878  sum, product, minimum, maximum along rows
V["reductions_doctest"] = {"cite": "Prelude.hs:822-878", "mat2x5": [list(range(5)), list(range(5, 10))], "sum": [10, 35],
                           "product": [0, 15120], "mat3x4": [[1, 4, 3, 8], [0, 2, 8, 4], [7, 9, 8, 8]],
                           "minimum": [1, 0, 7], "maximum": [8, 8, 9]}
# Prelude.hs:895-914  prescanl, postscanl
V["prepostscanl_doctest"] = {"cite": "Prelude.hs:895-914", "vec": list(range(1, 11)), "prescanl_seed": 0,
                             "prescanl": [0, 1, 3, 6, 10, 15, 21, 28, 36, 45], "postscanl_seed": 42,
                             "postscanl": [43, 45, 48, 52, 57, 63, 70, 78, 87, 97]}
# Prelude.hs:1620-1625  filter even
V["filter_doctest"] = {"cite": "Prelude.hs:1620-1625", "vec": list(range(1, 11)), "expected": [2, 4, 6, 8, 10], "count": 5}
# Prelude.hs:1696-1724, 1748-1778  gather, gatherIf, scatter, scatterIf
V["gather_scatter_doctest"] = {
    "cite": "Prelude.hs:1696-1724, 1748-1778",
    "gather": {"from": [1, 3, 7, 2, 5, 3], "input": [1, 9, 6, 4, 4, 2, 0, 1, 2], "expected": [9, 4, 1, 6, 2, 4]},
    "gatherIf": {"from": [1, 3, 7, 2, 5, 3], "mask": [3, 4, 9, 2, 7, 5], "defaults": [6.0] * 6,
                 "input": [1, 9, 6, 4, 4, 2, 0, 1, 2], "expected": [6.0, 6.0, 1.0, 6.0, 2.0, 4.0]},
    "scatter": {"to": [1, 3, 7, 2, 5, 8], "input": [1, 9, 6, 4, 4, 2, 5], "size": 10, "expected": [0, 1, 4, 9, 0, 4, 0, 6, 2, 0]},
    "scatterIf": {"to": [1, 3, 7, 2, 5, 8], "mask": [3, 4, 9, 2, 7, 5], "input": [1, 9, 6, 4, 4, 2, 5], "size": 10,
                  "expected": [0, 0, 0, 0, 0, 4, 0, 6, 2, 0]}}
# Prelude.hs:1812-1892  reverseOn, transposeOn; 1915-2010 take, drop, init, tail (the 5x10 iota matrix, the 2x3x5 iota box)
V["reindex_doctest"] = {
    "cite": "Prelude.hs:1812-1892, 1915-2010", "mat": iota5x10, "box_shape": [2, 3, 5],
    "reverseOn_1": [[r * 10 + 9 - c for c in range(10)] for r in range(5)],
    "reverseOn_2": [[(4 - r) * 10 + c for c in range(10)] for r in range(5)],
    "transposeOn_1_2_box": [0, 5, 10, 1, 6, 11, 2, 7, 12, 3, 8, 13, 4, 9, 14, 15, 20, 25, 16, 21, 26, 17, 22, 27, 18, 23, 28, 19, 24, 29],
    "transposeOn_2_3_box": [0, 1, 2, 3, 4, 15, 16, 17, 18, 19, 5, 6, 7, 8, 9, 20, 21, 22, 23, 24, 10, 11, 12, 13, 14, 25, 26, 27, 28, 29],
    "transposeOn_1_3_box": [0, 15, 5, 20, 10, 25, 1, 16, 6, 21, 11, 26, 2, 17, 7, 22, 12, 27, 3, 18, 8, 23, 13, 28, 4, 19, 9, 24, 14, 29],
    "take_5": [[r * 10 + c for c in range(5)] for r in range(5)],
    "drop_7": [[r * 10 + c for c in range(7, 10)] for r in range(5)],
    "init": [[r * 10 + c for c in range(9)] for r in range(5)],
    "tail": [[r * 10 + c for c in range(1, 10)] for r in range(5)]}
# Prelude.hs:1490-1575  (++) and concatOn
V["concat_doctest"] = {
    "cite": "Prelude.hs:1490-1575", "m1": iota5x10, "m2_10x3": [[r * 3 + c for c in range(3)] for r in range(10)],
    "append": [[r * 10 + c for c in range(10)] + [r * 3 + c for c in range(3)] for r in range(5)],
    "m2_10x5": [[r * 5 + c for c in range(5)] for r in range(10)],
    "concatOn_1": [[r * 10 + c for c in range(10)] + [r * 5 + c for c in range(5)] for r in range(5)],
    "concatOn_2": [[r * 10 + c for c in range(5)] for r in range(5)] + [[r * 5 + c for c in range(5)] for r in range(10)]}
# Language.hs:186-260  replicate; 340-400 slice (vec = [0..9], mat = the 5x10 iota matrix, cube = 3x4x5 iota)
V["replicate_slice_doctest"] = {
    "cite": "Language.hs:186-260, 340-400", "vec": list(range(10)), "mat": iota5x10, "cube_shape": [3, 4, 5],
    "replicate_4_All": [list(range(10))] * 4,
    "replicate_All_4": [[i] * 4 for i in range(10)],
    "replicate_2_All_3": [[[i] * 3 for i in range(10)]] * 2,
    "slice_2_All": list(range(20, 30)), "slice_4_2": 42,
    "sl0_vec_4": 4, "sl0_mat_4": [4, 14, 24, 34, 44], "sl1_mat_4": list(range(40, 50)),
    "sl1_cube_2": [[10, 11, 12, 13, 14], [30, 31, 32, 33, 34], [50, 51, 52, 53, 54]]}
# Language.hs:405-455  map (+1), zipWith (+) over matrices of different extents
V["map_zipwith_doctest"] = {"cite": "Language.hs:405-455", "xs": list(range(10)), "map_plus1": list(range(1, 11)),
                            "m3x5": [[r * 5 + c for c in range(5)] for r in range(3)],
                            "m5x10": [[r * 10 + c + 1 for c in range(10)] for r in range(5)],
                            "zipwith_plus": [[1, 3, 5, 7, 9], [16, 18, 20, 22, 24], [31, 33, 35, 37, 39]]}
# Prelude.hs:157-172 indexed; 1436-1478 fill, enumFromN, enumFromStepN; 1627-1635 filter odd over a matrix
V["producers_doctest"] = {"cite": "Prelude.hs:157-172, 1436-1478, 1627-1635",
                          "indexed_vec": [0.0, 1.0, 2.0, 3.0, 4.0], "indexed_mat_shape": [3, 4],
                          "enumFromN_5x10": iota5x10,
                          "enumFromStepN_5x10": [[(r * 10 + c) * 0.5 for c in range(10)] for r in range(5)],
                          "filter_odd_mat": evens_mat, "filter_odd": [1, 3, 5, 7, 9, 1, 1, 1, 1, 1, 1, 3, 5, 7, 9, 11, 13, 15, 17, 19],
                          "filter_odd_counts": [5, 5, 0, 10]}
# Test/NoFib/Misc/Cache.hs:44-73: a = [0..9], b = [10..19]
V["misc_cache"] = {"cite": "Test/NoFib/Misc/Cache.hs:44-73", "a": [float(i) for i in range(10)],
                   "b": [float(i) for i in range(10, 20)], "generate": 5 * 45.0, "backpermute": 2 * 45.0}
# Language.hs:716-728  histogram via permute (+)
V["histogram_doctest"] = {"cite": "Language.hs:716-728",
                          "keys": [0, 0, 1, 2, 1, 1, 2, 4, 8, 3, 4, 9, 8, 3, 2, 5, 5, 3, 1, 2], "bins": 10,
                          "expected": [2, 4, 4, 3, 2, 2, 0, 0, 2, 1]}
# Language.hs:734-749  identity matrix via permute const (source rank 1, destination rank 2)
V["identity_permute"] = {"cite": "Language.hs:734-749", "n": 5,
                         "expected": [[1 if i == j else 0 for j in range(5)] for i in range(5)]}
# Language.hs:821-842  transpose via backpermute
V["transpose_backpermute"] = {"cite": "Language.hs:821-842", "mat": iota5x10,
                              "expected": [[r * 10 + c for r in range(5)] for c in range(10)]}
# Test/NoFib/Issues/Issue228.hs:30-46  non-commutative pair monoid, fold with seed (1,0) and fold1
V["issue228"] = {"cite": "Test/NoFib/Issues/Issue228.hs:30-46", "fst": [1, 0, 1], "snd": [1, 0, 1],
                 "seed": [1, 0], "expected": [0, 1]}
# Test/NoFib/Issues/Issue362.hs:38-71  scanl1 over 4- and 5-tuples
V["issue362"] = {"cite": "Test/NoFib/Issues/Issue362.hs:38-71", "vec": list(range(10)),
                 "expected": [0, 1, 3, 6, 10, 15, 21, 28, 36, 45]}
# Test/NoFib/Issues/Issue185.hs:44-97  scatter / gather
V["issue185_A"] = {"cite": "Test/NoFib/Issues/Issue185.hs:44-52", "to": [1, 3, 7, 2, 5, 8],
                   "xs": [1, 9, 6, 4, 4, 2, 5], "over": [0] * 9, "expected": [0, 1, 4, 9, 0, 4, 0, 6, 2]}
V["issue185_B"] = {"cite": "Test/NoFib/Issues/Issue185.hs:55-63", "to": [1, 3, 7, 2, 5, 8],
                   "xs": [1, 9, 6], "over": [0] * 9, "expected": [0, 1, 0, 9, 0, 0, 0, 6, 0]}
V["issue185_E"] = {"cite": "Test/NoFib/Issues/Issue185.hs:96-103", "from": [1, 3, 7, 2, 5, 3],
                   "xs": [1, 9, 6, 4, 4, 2, 0, 1, 2], "expected": [9, 4, 1, 6, 2, 4]}

# Test/NoFib/Issues/Issue137.hs:33-59  permute with a min-merge combiner over pairs:
# inputs are closed forms, the 384-entry expected vector is read from the reference's file
text = open(os.path.join(SRC, "Test", "NoFib", "Issues", "Issue137.hs")).read()
m = re.search(r"ref1 = fromList \(Z:\.384\) \[(.*?)\]\s*\n", text, re.S)
pairs = [[int(a), int(b)] for a, b in re.findall(r"\((-?\d+),(-?\d+)\)", m.group(1))]
assert len(pairs) == 384
V["issue137"] = {"cite": "Test/NoFib/Issues/Issue137.hs:33-59", "size": 3000, "bins": 384, "inf": 10000,
                 "values": "abs (8 - (a mod 17)) for a in 1..size", "targets": "a div 8 for a in 1..size",
                 "expected": pairs}

# Test/NoFib/Issues/Issue119.hs: sums of and segmented scans over literal arrays ("fold and scan
# with a number of elements not a multiple of the workgroup size").  The arrays are read from the
# reference's file in the order they appear: A-E give (expected, input), F-I (expected, input,
# segments), J and K (expected bodies, expected sums, input, segments).
text = open(os.path.join(SRC, "Test", "NoFib", "Issues", "Issue119.hs")).read()
lists = [(tuple(int(d) for d in re.findall(r"\d+", sh)), [int(x) for x in body.split(",")])
         for sh, body in re.findall(r"fromList \((Z(?: *:\. *\d+)*)\)\s*\[([-0-9,\s]+)\]", text)]
totals = [int(x) for x in re.findall(r"ref\d = fromList Z \[(-?\d+)\]", text)]
assert len(totals) == 4
it = iter(lists)
for name, kind in (("A", "foldall"), ("B", "foldall"), ("C", "foldall"), ("D", "foldall"), ("E", "fold")):
    expected = [totals["ABCD".index(name)]] if name != "E" else next(it)[1]
    shape, xs = next(it)
    V["issue119_" + name] = {"cite": "Test/NoFib/Issues/Issue119.hs test " + name, "kind": kind,
                             "type": "i32" if name in "ABE" else "i64", "shape": list(shape), "xs": xs,
                             "expected": expected}
for name, kind in (("F", "scanl1Seg"), ("G", "scanr1Seg"), ("H", "scanlSeg"), ("I", "scanrSeg")):
    (_, expected), (_, xs), (_, seg) = next(it), next(it), next(it)
    V["issue119_" + name] = {"cite": "Test/NoFib/Issues/Issue119.hs test " + name, "kind": kind,
                             "xs": xs, "seg": seg, "expected": expected}
for name, kind in (("J", "scanl'Seg"), ("K", "scanr'Seg")):
    (_, ps), (_, rs), (_, xs), (_, seg) = next(it), next(it), next(it), next(it)
    V["issue119_" + name] = {"cite": "Test/NoFib/Issues/Issue119.hs test " + name, "kind": kind,
                             "xs": xs, "seg": seg, "expected": ps, "expected_sums": rs}
assert len(V["issue119_J"]["expected_sums"]) == 30 and len(V["issue119_K"]["expected"]) == 750
assert V["issue119_A"]["expected"] == [734889155] and len(V["issue119_F"]["expected"]) == 748
assert sum(V["issue119_F"]["seg"]) == 748 and len(V["issue119_H"]["expected"]) == 645

# Test/NoFib/Issues/Issue93.hs: permute (\c _ -> c) (fill (shape xs) 0) Just xs on a 1x1 matrix
V["issue93"] = {"cite": "Test/NoFib/Issues/Issue93.hs:27-34", "mat": [[5]], "expected": [[5]]}
# Test/NoFib/Issues/Issue102.hs: [4,4,4] of shape 1x3x1
V["issue102"] = {"cite": "Test/NoFib/Issues/Issue102.hs:31-62", "expected": [[[4], [4], [4]]]}
# Test/NoFib/Issues/Issue114.hs: compensated summation over pairs, fold1 and scanl1 (compared with ~=)
V["issue114"] = {"cite": "Test/NoFib/Issues/Issue114.hs:33-71", "n": 100, "x": 1.01,
                 "expected_sum": [101.0, 0.0], "expected_prefix": "(1.01 * i, 0) for i in 1..n"}
# Test/NoFib/Issues/Issue123.hs: fold (+) 0 (fill n 1) = n
V["issue123"] = {"cite": "Test/NoFib/Issues/Issue123.hs:27-38", "n": 100, "expected": 100}
# Test/NoFib/Issues/Issue184.hs test A: generate 1000 (\x -> x < 5 ? (v!!x)^2 : 0), v = [1..5]
V["issue184_A"] = {"cite": "Test/NoFib/Issues/Issue184.hs:33-41", "v": [1, 2, 3, 4, 5], "n": 1000,
                   "expected": [1, 4, 9, 16, 25] + [0] * 995}
# Test/NoFib/Issues/Issue287.hs test A: scanl1 of a six-component combination over zeros stays zero
V["issue287_A"] = {"cite": "Test/NoFib/Issues/Issue287.hs:26-56", "n": 4, "expected": [[0] * 6] * 4}
# Test/NoFib/Issues/Issue288.hs: map (while (const False) id) leaves pairs unchanged
V["issue288"] = {"cite": "Test/NoFib/Issues/Issue288.hs:26-36", "n": 10}
# Test/NoFib/Issues/Issue364.hs: scanl iappend one over the intervals (i, i) for i in 0..n-1 gives
# one, then (0, i); n = 64 and n = 65 (the second failed for integral types)
V["issue364"] = {"cite": "Test/NoFib/Issues/Issue364.hs:41-93", "sizes": [64, 65], "one": [-1, -1], "top": [-2, -2]}
# Test/NoFib/Issues/Issue407.hs: isNaN / isInfinite
V["issue407"] = {"cite": "Test/NoFib/Issues/Issue407.hs:38-46",
                 "xs": ["nan", "-inf", "nan", "0.1", "inf", "0.5", "inf"],
                 "isnan": [1, 0, 1, 0, 0, 0, 0], "isinf": [0, 1, 0, 0, 1, 0, 1]}
# Test/NoFib/Issues/Issue409.hs: y + tanh ((-y) * y) with y = recip 1  ==  1 + tanh (-1)
V["issue409"] = {"cite": "Test/NoFib/Issues/Issue409.hs:36-53", "x": 1.0, "expected": "1 + tanh(-1)"}
# Test/NoFib/Issues/Issue436.hs test A: filter (const True) (take 3 bools)
V["issue436_A"] = {"cite": "Test/NoFib/Issues/Issue436.hs:27-50", "xs": [1, 0, 1, 0, 1], "take": 3,
                   "expected": [1, 0, 1], "count": 3}
# Test/NoFib/Issues/Issue439.hs: map (* 2) over the rank-0 array fill Z 1
V["issue439"] = {"cite": "Test/NoFib/Issues/Issue439.hs:26-34", "expected": 2.0}

# Test/NoFib/Issues/Issue168.hs: fill (Z:.1) of an iterated tuple function
V["issue168"] = {"cite": "Test/NoFib/Issues/Issue168.hs:31-66", "A": [3.0, 2.0], "B": [3.0, 2.0],
                 "C": [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]}
# Test/NoFib/Issues/Issue264.hs: negate . negate = id for every number type; not . not = id and
# De Morgan's pairs over Bool (the reference checks them as properties against the host functions)
V["issue264"] = {"cite": "Test/NoFib/Issues/Issue264.hs:36-130",
                 "bool": {"not.not": "x", "not(&&)": "not (u and v)", "not(||)": "not (u or v)",
                          "not(not(&&))": "u and v", "not(not(||))": "u or v"}}
# Test/NoFib/Issues/Issue286.hs: sum . flatten . map fromIntegral over a 120x659 matrix of ones
V["issue286"] = {"cite": "Test/NoFib/Issues/Issue286.hs:47-48,107", "shape": [120, 659], "fill": 1,
                 "expected": 120.0 * 659.0}
# Test/NoFib/Issues/Issue427.hs: indices of the True cells of a matrix, row-major (property against
# a list filter; shapes n-by-64, n-by-8, n-by-m)
V["issue427"] = {"cite": "Test/NoFib/Issues/Issue427.hs:34-84", "shapes": [[33, 64], [129, 8], [0, 8], [17, 31], [1, 1]]}
# Test/NoFib/Issues/Issue437.hs: runN id returns its arguments; nothing is allocated, 4 bytes at most
# go to the device and nothing comes back
V["issue437"] = {"cite": "Test/NoFib/Issues/Issue437.hs:45-83", "unit": 42.0, "shape": [10000, 10000], "fill": 1.0}
# Test/NoFib/Issues/Issue517.hs: (Nothing, Just 2, Just 3, Just 5, Just 7) from (<>) on Maybe (Max Float)
V["issue517"] = {"cite": "Test/NoFib/Issues/Issue517.hs:31-43", "tags": [0, 1, 1, 1, 1], "values": [None, 2.0, 3.0, 5.0, 7.0]}
# Test/NoFib/Issues/Issue551.hs: equality of a nine-constructor enumeration is the 9x9 identity, the
# digits map back to 0..8
V["issue551"] = {"cite": "Test/NoFib/Issues/Issue551.hs:80-83", "n": 9}

with open(OUT, "w") as f:
    json.dump(V, f, indent=1, sort_keys=True)
print("wrote", OUT, len(V), "vectors")
