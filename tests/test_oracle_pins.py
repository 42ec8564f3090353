"""Pins of the CPU oracle (no GPU needed).

The oracle is only trusted after these pass: bit-exact known answers produced by the reference's own
sources (tests/golden/*.json), brute force on tiny inputs, scipy products and closed forms.
"""
import ctypes
import json
import math
import os
import subprocess

import numpy as np
import pytest
import scipy.sparse as sp

from flexspmv_amd import graphs
from flexspmv_amd import workloads as W
from oracle import build_oracle
from oracle.runner import run_oracle

REFERENCE_ROOT = "/root/reference"


@pytest.fixture(scope="module")
def kats():
    return build_oracle.build_kats()


@pytest.fixture(scope="module")
def merge_lib():
    lib = ctypes.CDLL(build_oracle.build_merge_capi())
    return lib


def _golden(golden_dir, name):
    with open(os.path.join(golden_dir, name + ".json")) as f:
        return json.load(f)["lines"]


# ---------------------------------------------------------------------------------------------
# value type: bit-exact against the reference header
# ---------------------------------------------------------------------------------------------
def test_tensor_semantics_match_reference_bits(kats, golden_dir):
    gold = _golden(golden_dir, "tensor_kat")
    mine = build_oracle.kat_lines(kats["tensor_kat"])
    assert set(mine) == set(gold)
    bad = {k: (mine[k], gold[k]) for k in gold if mine[k] != gold[k]}
    assert not bad, bad
    # the fixture really holds the quirks that differ from torch
    assert gold["div_same_guarded f32"].split()[1] == "0"          # x / 0 -> 0 for equal widths
    assert gold["div_scalar_unguarded f32"].split()[0] == "7f800000"  # tensor / 0 scalar -> inf
    assert gold["sign_nan_negzero f64"].split()[0] == "0"           # sign(NaN) -> 0


def test_golden_fixture_is_what_the_reference_prints(golden_dir):
    """Only where the reference tree is mounted: the committed fixtures are reproducible."""
    if not os.path.isdir(REFERENCE_ROOT):
        pytest.skip("reference tree not present")
    exes = build_oracle.build_reference_kats(REFERENCE_ROOT)
    for name, exe in exes.items():
        assert build_oracle.kat_lines(exe) == _golden(golden_dir, name)


# ---------------------------------------------------------------------------------------------
# merge-path search and fix-ups
# ---------------------------------------------------------------------------------------------
def test_merge_search_and_fixups_match_reference(kats, golden_dir):
    gold = _golden(golden_dir, "merge_kat")
    mine = build_oracle.kat_lines(kats["merge_kat"])
    for key, val in mine.items():
        assert gold[key] == val, key
    assert {k for k in gold if k not in mine} == {"map_only_T1 i64", "map_only_T3 i64", "map_only_T8 i64"}


def _brute_force_path(row_ptr):
    """All merge-path coordinates by actually merging row-end offsets with 0..nnz-1."""
    rows, nnz = len(row_ptr) - 1, int(row_ptr[-1])
    x = y = 0
    coords = [(0, 0)]
    while x < rows or y < nnz:
        if x < rows and (y >= nnz or row_ptr[x + 1] <= y):
            x += 1      # all non-zeros of row x are consumed: take its row-end item
        else:
            y += 1
        coords.append((x, y))
    return coords


@pytest.mark.parametrize("seed", range(6))
def test_merge_path_search_equals_brute_force(merge_lib, seed):
    rng = np.random.default_rng(seed)
    rows = int(rng.integers(1, 40))
    lens = rng.integers(0, 6, rows) * (rng.random(rows) < 0.6)
    if seed == 3:
        lens[rows // 2] = 50
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    nnz = int(row_ptr[-1])
    expect = _brute_force_path(row_ptr)
    assert len(expect) == rows + nnz + 1
    row_end = np.ascontiguousarray(row_ptr[1:])
    out = (ctypes.c_int * 2)()
    prev = (0, 0)
    for d, (ex, ey) in enumerate(expect):
        merge_lib.oracle_merge_path_search(d, row_end.ctypes.data_as(ctypes.c_void_p), rows, nnz, out)
        assert (out[0], out[1]) == (ex, ey), (d, row_ptr.tolist())
        assert out[0] + out[1] == d and out[0] >= prev[0] and out[1] >= prev[1]
        prev = (out[0], out[1])


def test_thread_spans_tile_the_path(merge_lib):
    row_ptr = np.array([0, 3, 3, 3, 7, 8, 8, 20, 20], dtype=np.int32)
    rows, nnz = 8, 20
    row_end = np.ascontiguousarray(row_ptr[1:])
    for T in (1, 2, 3, 5, 8, 28, 64):
        out = (ctypes.c_int * 4)()
        last = (0, 0)
        for tid in range(T):
            merge_lib.oracle_reducer_thread_span(tid, T, row_end.ctypes.data_as(ctypes.c_void_p), rows, nnz, out)
            assert (out[0], out[1]) == last
            last = (out[2], out[3])
            per = -(-(rows + nnz) // T)
            assert (out[2] + out[3]) - (out[0] + out[1]) <= per
        assert last == (rows, nnz)
        # flat split of the aggregator variant: ceil((rows+nnz)/T) edges per thread, clipped at nnz
        covered = []
        for tid in range(T):
            rng_ = (ctypes.c_int * 2)()
            merge_lib.oracle_flat_thread_range(tid, T, rows, nnz, rng_)
            covered += list(range(rng_[0], max(rng_[0], rng_[1])))
        assert covered == list(range(nnz))


def test_map_only_instance_matches_reference_generated_header(golden_dir):
    """bp_1[:] = bpoints[:, 1] on int64: the reference's checked-in generated CPU kernel, run on the
    same input, printed the fixture lines."""
    gold = _golden(golden_dir, "merge_kat")
    ne = 37
    bpoints = np.stack([1000 + np.arange(ne), 5 * np.arange(ne) - 11], axis=1).astype(np.int64)
    for T in (1, 3, 8):
        bp_1 = np.full(ne, -7, dtype=np.int64)
        outs, after = run_oracle(graphs.get("bpoints_copy"), {"bpoints": bpoints, "bp_1": bp_1}, None, ne, ne, T)
        assert outs == []
        assert " ".join(str(v) for v in after["bp_1"]) == gold[f"map_only_T{T} i64"]


# ---------------------------------------------------------------------------------------------
# reducer pass: scipy, naive loops, closed forms
# ---------------------------------------------------------------------------------------------
def _random_csr(rng, rows, cols, density, empty_frac=0.3):
    A = sp.random(rows, cols, density=density, format="csr", random_state=rng, dtype=np.float64)
    keep = rng.random(rows) > empty_frac
    A = sp.diags(keep.astype(np.float64)) @ A
    A.eliminate_zeros()
    A = A.tocsr()
    A.sort_indices()
    return A


@pytest.mark.parametrize("dtype,tol", [(np.float32, 2e-6), (np.float64, 1e-14)])
@pytest.mark.parametrize("T", [1, 2, 3, 7, 8, 64, 256])
def test_csr_spmv_oracle_equals_scipy(dtype, tol, T):
    rng = np.random.default_rng(11)
    A = _random_csr(rng, 300, 211, 0.04)
    x = rng.uniform(-1, 1, 211)
    t = {"vals": A.data.astype(dtype), "x": x.astype(dtype), "selector_idx": A.indices.astype(np.int32)}
    (y,), _ = run_oracle(graphs.get("csr_spmv"), t, A.indptr.astype(np.int32), 300, 211, T)
    ref = sp.csr_matrix((t["vals"].astype(np.float64), A.indices, A.indptr), shape=A.shape) @ t["x"].astype(np.float64)
    scale = abs(sp.csr_matrix((np.abs(t["vals"]).astype(np.float64), A.indices, A.indptr), shape=A.shape)) @ np.abs(x)
    assert np.all(np.abs(y - ref) <= tol * np.maximum(scale, 1e-30) + 0.0)
    assert np.all(y[np.diff(A.indptr) == 0] == 0)       # empty rows are written as zero


def test_thread_count_limit_of_reference_carry_arrays():
    w = W.laplacian_2d_spmv(8)
    with pytest.raises(RuntimeError):
        run_oracle(graphs.get(w.graph), w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, 257)


def test_long_row_spanning_all_threads():
    rng = np.random.default_rng(5)
    vals = rng.uniform(-1, 1, 1000)
    x = rng.uniform(-1, 1, 1000)
    ptr = np.array([0, 0, 1000, 1000], dtype=np.int32)
    t = {"vals": vals, "x": x, "selector_idx": np.arange(1000, dtype=np.int32)}
    (y,), _ = run_oracle(graphs.get("csr_spmv"), t, ptr, 3, 1000, 8)
    assert y[0] == 0 and y[2] == 0
    assert abs(y[1] - math.fsum(vals * x)) < 1e-12


def test_laplacian_closed_forms():
    n = 24
    w = W.laplacian_2d_spmv(n, dtype="float64")
    g = graphs.get(w.graph)
    # A * 1: interior rows 0, edge rows 1, corner rows 2
    t = dict(w.tensors, x=np.ones(n * n))
    (y,), _ = run_oracle(g, t, w.row_end_offsets, w.num_rows, w.num_cols, 8)
    y = y.reshape(n, n)
    assert np.all(y[1:-1, 1:-1] == 0) and np.all(y[0, 1:-1] == 1) and y[0, 0] == 2 and y[-1, -1] == 2
    # sine modes are eigenvectors of the Dirichlet Laplacian
    i = np.arange(1, n + 1)
    for pq in ((1, 1), (2, 5), (7, 3)):
        v = np.outer(np.sin(np.pi * pq[0] * i / (n + 1)), np.sin(np.pi * pq[1] * i / (n + 1))).ravel()
        lam = 4 - 2 * np.cos(np.pi * pq[0] / (n + 1)) - 2 * np.cos(np.pi * pq[1] / (n + 1))
        (y,), _ = run_oracle(g, dict(w.tensors, x=v), w.row_end_offsets, w.num_rows, w.num_cols, 5)
        assert np.allclose(y, lam * v, rtol=0, atol=1e-13)


def test_poisson_dot_aggregator_and_row_selector():
    w = W.poisson_3d_spmv_dot(10)
    (y, dot), _ = run_oracle(graphs.get(w.graph), w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, 6)
    A = sp.csr_matrix((w.tensors["vals"], w.tensors["selector_col_idx"], w.row_end_offsets), shape=(w.num_rows,) * 2)
    x = w.tensors["x"]
    assert np.allclose(y, A @ x, rtol=0, atol=1e-13)
    assert abs(dot[0] - math.fsum(x * (A @ x))) <= 1e-12 * abs(dot[0])
    assert np.array_equal(w.tensors["selector_row_idx"], np.repeat(np.arange(w.num_rows), np.diff(w.row_end_offsets)))


# ---------------------------------------------------------------------------------------------
# flat pass
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T", [1, 3, 8, 100])
def test_aggregator_only_equals_fsum(T):
    rng = np.random.default_rng(2)
    h, area = rng.uniform(0.5, 2, 5001), rng.uniform(0, 1, 5001)
    (m,), _ = run_oracle(graphs.get("mass_sum"), {"h": h, "area": area}, None, 5001, 5001, T)
    assert abs(m[0] - math.fsum(h * area)) <= 1e-13 * m[0]


# ---------------------------------------------------------------------------------------------
# physics-level invariants of the larger maps
# ---------------------------------------------------------------------------------------------
def test_spring_mass_newton_and_energy():
    w = W.spring_mass_grid(9, dtype="float64")
    (F, E), _ = run_oracle(graphs.get(w.graph), w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, 7)
    assert np.abs(F.sum(axis=0)).max() < 1e-12           # internal forces cancel
    pos, src, dst = w.tensors["pos"], w.tensors["gather_src_idx"], w.tensors["gather_dst_idx"]
    d = pos[dst] - pos[src]
    r = np.linalg.norm(d, axis=1)
    f = (w.tensors["k"] * (r - w.tensors["rest"]) / r)[:, None] * d
    Fref = np.zeros_like(F)
    np.add.at(Fref, dst, f)
    assert np.allclose(F, Fref, rtol=0, atol=1e-14)
    assert abs(E[0] - math.fsum(0.25 * w.tensors["k"] * (r - w.tensors["rest"]) ** 2)) <= 1e-12 * E[0]


def test_shallow_water_lake_at_rest():
    """Constant depth and zero velocity: no mass flux, and the pressure terms of an interior cell's
    closed polygon cancel."""
    w = W.shallow_water_mesh(3000)
    U = np.zeros_like(w.tensors["U"])
    U[:, 0] = 1.3
    outs, _ = run_oracle(graphs.get(w.graph), dict(w.tensors, U=U), w.row_end_offsets, w.num_rows, w.num_cols, 4)
    assert np.abs(outs[0]).max() < 1e-15
    interior = np.diff(w.row_end_offsets) == 3
    assert interior.sum() > 1000
    assert np.abs(outs[1][interior]).max() < 1e-13 and np.abs(outs[2][interior]).max() < 1e-13


# ---------------------------------------------------------------------------------------------
# every map op: the generated statements against a plain numpy statement of the same semantics
# ---------------------------------------------------------------------------------------------
def op_zoo_inputs(rng, ne, nv, dtype):
    t = {
        "a6": rng.uniform(-2, 2, (ne, 6)), "b3": rng.uniform(0.5, 2, (ne, 3)) * rng.choice([-1, 1], (ne, 3)),
        "c2": rng.uniform(0.5, 1.5, (ne, 2)), "acc": rng.uniform(-1, 1, (ne, 3)),
        "dst6": rng.uniform(-1, 1, (ne, 6)), "vx": rng.uniform(-1, 1, (nv, 3)),
    }
    t = {k: v.astype(dtype) for k, v in t.items()}
    t["sel_p_idx"] = rng.integers(0, nv, ne).astype(np.int32)
    q = rng.integers(0, nv, ne).astype(np.int32)
    q[::5] = t["sel_p_idx"][::5]                       # equal indices: zero differences -> guarded division
    t["sel_q_idx"] = q
    return t


def op_zoo_numpy(t, row_ptr):
    """Plain numpy statement of flexspmv_amd.graphs.op_zoo with the reference value type's rules."""
    def bc(a, n):                                      # flat-index modulo broadcast to width n
        return a[:, np.arange(n) % a.shape[1]]
    f = t["a6"].dtype.type
    a6, b3, c2, acc, vx = t["a6"], t["b3"], t["c2"], t["acc"].copy(), t["vx"]
    p, q = vx[t["sel_p_idx"]], vx[t["sel_q_idx"]]
    add = a6 + bc(b3, 6)
    sub = p - q
    mul = a6 * bc(c2, 6)
    with np.errstate(divide="ignore", invalid="ignore"):
        truediv = np.where(sub != 0, b3 / np.where(sub != 0, sub, 1), 0).astype(f)   # equal widths: guarded
        truediv_1 = a6 / bc(b3, 6)                                                     # 6 / 3: plain
    neg = -truediv
    abs_1 = np.abs(sub)
    pow_1 = abs_1 ** f(0.5)
    pow_2 = abs_1 ** bc(c2, 3)
    exp = np.exp(sub)
    sign = np.sign(sub)
    norm = np.sqrt((b3 * b3).sum(axis=1, dtype=f))
    truediv_2 = sub / norm[:, None]
    truediv_3 = f(1) / b3
    lt = (sub < 0).astype(f)
    gt = (a6 > bc(b3, 6)).astype(f)
    where = np.where(lt != 0, pow_1, exp)
    where_1 = np.where(gt != 0, add, f(0))
    where_2 = np.where(lt != 0, f(1.5), truediv_3)
    clone = a6[:, 4:5]
    mul_1 = clone * sign
    acc = acc + mul_1
    add_1 = where_1 * mul + truediv_1
    dst6 = add_1
    add_4 = where + where_2 + pow_2 + neg * f(0.001) + truediv_2
    add_5 = add_4 + acc
    rows = np.repeat(np.arange(len(row_ptr) - 1), np.diff(row_ptr))
    red = np.zeros((len(row_ptr) - 1, 3), dtype=np.float64)
    np.add.at(red, rows, add_5.astype(np.float64))
    red6 = np.zeros((len(row_ptr) - 1, 6), dtype=np.float64)
    np.add.at(red6, rows, dst6.astype(np.float64))
    return {"reducer": red, "reducer_6": red6, "sum_1": mul_1.astype(np.float64).sum(axis=0), "add_4": add_4,
            "acc": acc, "dst6": dst6}


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 2e-5)])
def test_op_zoo_oracle_equals_numpy_statement(dtype, tol):
    rng = np.random.default_rng(7)
    ne, nv, rows = 400, 37, 50
    t = op_zoo_inputs(rng, ne, nv, dtype)
    lens = rng.multinomial(ne, np.ones(rows) / rows)
    lens[3] += lens[4]; lens[4] = 0
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    outs, after = run_oracle(graphs.get("op_zoo"), t, row_ptr, rows, nv, 5)
    ref = op_zoo_numpy(t, row_ptr)
    names = ["reducer", "reducer_6", "sum_1", "add_4"]
    for name, o in zip(names, outs):
        scale = np.abs(ref[name]).max()
        assert np.abs(o - ref[name]).max() <= tol * scale, name
    for name in ("acc", "dst6"):                       # in-place results written through the inputs
        assert np.abs(after[name] - ref[name]).max() <= tol * np.abs(ref[name]).max(), name


# ---------------------------------------------------------------------------------------------
# int64 sub-graphs with reducers and aggregators: integer sums have one right answer
# ---------------------------------------------------------------------------------------------
def _segment_sums(a, row_ptr):
    """Exact per-row sums of an integer array [ne][Dim] (plain numpy, one row at a time)."""
    a = a.reshape(len(a), -1)
    out = np.zeros((len(row_ptr) - 1, a.shape[1]), dtype=np.int64)
    for r in range(len(row_ptr) - 1):
        out[r] = a[row_ptr[r]:row_ptr[r + 1]].sum(axis=0)
    return out


@pytest.mark.parametrize("T", [1, 3, 8, 64, 256])
@pytest.mark.parametrize("structure", ["mesh_with_gaps", "skewed", "one_long_row", "mostly_empty", "tiny"])
def test_int64_reducer_graphs_equal_exact_integer_sums(structure, T):
    from tests.util_inputs import make_inputs, row_structure
    rng = np.random.default_rng(33)
    row_ptr = row_structure(structure, rng)
    t, row_ptr, nr, nc, ne = make_inputs(graphs.get("index_spmv"), np.int64, rng, row_ptr=row_ptr)
    (y, total), _ = run_oracle(graphs.get("index_spmv"), t, row_ptr, nr, nc, T)
    prod = t["w"] * t["ids"][t["selector_idx"]]
    assert y.dtype == np.int64 and np.array_equal(y, _segment_sums(prod, row_ptr)[:, 0])
    assert np.array_equal(total, [prod.sum()])
    t, row_ptr, nr, nc, ne = make_inputs(graphs.get("index_sums"), np.int64, rng, row_ptr=row_ptr)
    (red, weight, total), _ = run_oracle(graphs.get("index_sums"), t, row_ptr, nr, nc, T)
    mul = t["ids"][t["sel_idx"]] * t["w"][:, None]
    rows = np.repeat(np.arange(nr), np.diff(row_ptr))
    assert np.array_equal(red, _segment_sums(mul - t["ids"][rows], row_ptr))
    assert np.array_equal(weight, _segment_sums(t["w"], row_ptr)[:, 0])
    assert np.array_equal(total, mul.sum(axis=0))


# ---------------------------------------------------------------------------------------------
# the parity criterion itself: rounding differences pass, a wrong row does not
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name, dtype", [("spring_mass", np.float32), ("swe_rusanov", np.float64),
                                         ("csr_spmv", np.float32), ("spmv_dot", np.float64)])
def test_row_criterion_accepts_reordering_and_rejects_a_wrong_edge(name, dtype):
    from oracle.parity import TOL, reducer_row_scales, row_excess
    from tests.util_inputs import make_inputs, row_structure
    rng = np.random.default_rng(44)
    row_ptr = row_structure("mesh_with_gaps", rng)
    ir = graphs.get(name)
    t, row_ptr, nr, nc, ne = make_inputs(ir, dtype, rng, row_ptr=row_ptr)
    tol = TOL[np.dtype(dtype)]
    scales = reducer_row_scales(ir, t, row_ptr, nc, 4)
    ref, _ = run_oracle(ir, t, row_ptr, nr, nc, 8)
    other, _ = run_oracle(ir, t, row_ptr, nr, nc, 1)         # another summation order
    # one edge of one row takes the value of its neighbour: a single wrong operand
    streamed = next(k for k, v in t.items() if not k.endswith("_idx") and len(v) == ne)
    bad_inputs = dict(t)
    e = int(row_ptr[nr // 2])                                 # first edge of a row in the middle
    assert row_ptr[nr // 2 + 1] > e
    changed = t[streamed].copy()
    changed[e] = changed[e] * 1.001
    bad_inputs[streamed] = changed
    wrong, _ = run_oracle(ir, bad_inputs, row_ptr, nr, nc, 8)
    for i, (scale, floor) in scales.items():
        assert row_excess(other[i], ref[i], tol, scale, floor).max() <= 1.0
        assert row_excess(wrong[i], ref[i], tol, scale, floor).max() > 1.0
        # the floor is a few ulps of the row's own terms, not a launch-wide constant
        eps = np.finfo(dtype).eps
        rows_with_edges = np.diff(row_ptr) > 0
        assert np.all(floor[~rows_with_edges] == 0)
        assert np.all(floor[rows_with_edges] <= 2000 * eps * np.maximum(scale[rows_with_edges], 1e-300) + 1e-300) \
            or name in ("spring_mass", "swe_rusanov")         # maps with a cancellation inside are allowed more
