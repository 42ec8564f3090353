"""Parity of the HIP path with the CPU oracle, through the C interface of the generated libraries
(ctypes launcher in flexspmv_amd.binding).  Tolerances: float32 1e-5, float64 1e-12.  A reducer output is held
to the tolerance row by row, relative to max(|reference|, sum of |contributions| of that row): a short row
next to a very long one gets no slack from its neighbour.  On top of that every row is allowed FLOOR_ULPS units in the last place of the
largest single contribution of the launch: a map with a cancellation inside (the spring's r - L, the flux
differences of the shallow-water map) cannot be evaluated more precisely than a few ulps of its
intermediate values, and two float32 evaluations (fused multiply-adds, sqrt, division) differ by that
much however small the contribution comes out.  For products (SpMV) the floor is far below the row
criterion and changes nothing.  Other outputs are relative to their largest
magnitude; integers and structure are exact.
"""
import zlib

import numpy as np
import pytest
import scipy.sparse as sp

torch = pytest.importorskip("torch")

from flexspmv_amd import graphs
from flexspmv_amd import workloads as W
from flexspmv_amd.binding import load_named
from oracle.runner import run_oracle
from tests.util_inputs import STRUCTURES, make_inputs, random_row_structure, row_structure
from tests.test_oracle_pins import op_zoo_inputs

pytestmark = pytest.mark.gpu

TOL = {np.dtype("float32"): 1e-5, np.dtype("float64"): 1e-12}
THREADS = 8   # oracle thread count of most cases; its rounding depends on it, which the tolerances absorb
FLOOR_ULPS = 8
THREAD_SWEEP = (1, 8, 16)   # ... and one row structure per graph is checked against all of these


def case_rng(*parts):
    """Generator seeded from the case id (crc32: the same inputs in every process, unlike hash())."""
    return np.random.default_rng(zlib.crc32("/".join(str(p) for p in parts).encode()))


def gpu_launch(name, tensors, row_ptr, num_rows, num_cols):
    """merged_spmv_launch on cuda:0; returns (outputs, value inputs after the call) as numpy."""
    ext = load_named(name, build_if_missing=False)
    args, dev_tensors = [], {}
    for pname in ext.param_names():
        if pname == "row_end_offsets":
            ro = row_ptr if row_ptr is not None else np.array([42], dtype=np.int32)
            args.append(torch.from_numpy(np.ascontiguousarray(ro)).cuda())
        elif pname == "num_rows":
            args.append(int(num_rows))
        elif pname == "num_cols":
            args.append(int(num_cols))
        else:
            dev_tensors[pname] = torch.from_numpy(np.ascontiguousarray(tensors[pname])).cuda()
            args.append(dev_tensors[pname])
    outs = ext.merged_spmv_launch(*args)
    torch.cuda.synchronize()
    outs = [] if outs is None else [o.cpu().numpy() for o in outs]
    after = {k: v.cpu().numpy() for k, v in dev_tensors.items() if k in ext.signature["value_inputs"]}
    return outs, after


def assert_close(got, ref, tol, what, row_scale=None, row_slack=None):
    assert got.shape == ref.shape and got.dtype == ref.dtype, what
    if got.dtype.kind == "i":
        assert np.array_equal(got, ref), what
        return
    if not ref.size:
        return
    diff = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    if row_scale is not None:
        scale = np.maximum(np.abs(ref.astype(np.float64)), row_scale.reshape(ref.shape))
        allowed = tol * scale + (row_slack if row_slack is not None else 0.0)
        bad = diff > allowed
        if bad.any():
            i = int(np.argmax(diff - allowed))
            raise AssertionError(f"{what}: {int(bad.sum())} elements off; worst at flat index {i}: |diff| "
                                 f"{diff.flat[i]:.3e} > {tol:g} * {scale.flat[i]:.3e} (allowed {allowed.flat[i]:.3e})")
        return
    scale = max(float(np.abs(ref).max()), 1e-300)
    err = float(diff.max())
    assert err <= tol * scale, f"{what}: max |diff| {err:.3e} > {tol:g} * {scale:.3e}"


def reducer_row_scales(ir, tensors, row_ptr, num_cols):
    """Per reducer output: (sum over each row of |what one edge contributes| as [num_rows][Dim] float64,
    the absolute floor FLOOR_ULPS * eps * largest |contribution|).

    The contributions come from the oracle itself, run on the same edges with every edge as a row of its
    own (row pointer 0, 1, 2, ...: single-term sums, no rounding); index arrays are explicit inputs, so the
    gathers are those of the real launch."""
    ne = int(row_ptr[-1])
    per_edge, _ = run_oracle(ir, tensors, np.arange(ne + 1, dtype=np.int32), ne, num_cols, THREADS)
    starts = np.asarray(row_ptr[:-1], dtype=np.int64)
    empty = np.diff(row_ptr) == 0
    scales = {}
    for i, spec in enumerate(ir.outputs):
        if spec["target"] != "reducer":
            continue
        a = np.abs(per_edge[i].astype(np.float64)).reshape(ne, -1)
        floor = FLOOR_ULPS * float(np.finfo(per_edge[i].dtype).eps) * float(a.max())
        a = np.vstack([a, np.zeros((1, a.shape[1]))])       # reduceat needs valid start indices
        s = np.add.reduceat(a, np.minimum(starts, ne), axis=0)
        s[empty] = 0.0
        scales[i] = (s, floor)
    return scales


def check_against_oracle(name, tensors, row_ptr, num_rows, num_cols, dtype, threads=THREADS, gpu_outs=None):
    ir = graphs.get(name)
    ref_outs, ref_after = run_oracle(ir, tensors, row_ptr, num_rows, num_cols, threads)
    outs, after = gpu_outs if gpu_outs is not None else gpu_launch(name, tensors, row_ptr, num_rows, num_cols)
    assert len(outs) == len(ref_outs)
    tol = TOL.get(np.dtype(dtype), 0)
    scales = {}
    if row_ptr is not None and np.dtype(dtype).kind == "f":
        scales = reducer_row_scales(ir, tensors, row_ptr, num_cols)
    # float32 aggregators: the reference adds every edge sequentially per thread, so its own result
    # drifts from the exact sum by up to (edges per thread) * eps; the centre of the comparison is the
    # same oracle evaluated in float64 on the same inputs
    ref_hi = None
    if np.dtype(dtype) == np.float32 and any(o["target"] == "sum" for o in ir.outputs):
        hi = {k: (v.astype(np.float64) if v.dtype == np.float32 else v) for k, v in tensors.items()}
        ref_hi, _ = run_oracle(ir, hi, row_ptr, num_rows, num_cols, THREADS)
    for i, (spec, o, r) in enumerate(zip(ir.outputs, outs, ref_outs)):
        if ref_hi is not None and spec["target"] == "sum":
            assert_close(o.astype(np.float64), ref_hi[i], tol, f"{name} aggregator {spec['name']} vs float64 oracle")
            # ... and the weaker statement about the float32 oracle itself: it differs from the exact sum by at
            # most (terms per thread) * eps * sum|terms| (sequential summation), the HIP result by tol
            ne = int(row_ptr[-1]) if row_ptr is not None else int(num_cols)
            chain = -(-ne // threads)
            bound = (chain * np.finfo(np.float32).eps + tol) * np.abs(ref_hi[i]).max()
            assert float(np.abs(o.astype(np.float64) - r.astype(np.float64)).max()) <= bound, \
                f"{name} aggregator {spec['name']} vs float32 oracle"
        else:
            scale, slack = scales.get(i, (None, None))
            assert_close(o, r, tol, f"{name} output {spec['name']}", row_scale=scale, row_slack=slack)
    for k in ref_after:                      # in-place map ops write through the inputs
        assert_close(after[k], ref_after[k], tol, f"{name} input {k} after the call")
    return outs


REDUCER_GRAPHS = ["csr_spmv", "spmv_dot", "spring_mass", "swe_rusanov", "system_two_selectors"]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("structure", STRUCTURES)
@pytest.mark.parametrize("name", REDUCER_GRAPHS)
def test_reducer_graphs_on_every_row_structure(name, structure, dtype):
    rng = case_rng(name, structure)
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
    print(f"case {name} {structure} {np.dtype(dtype).name} rows={nr} ne={ne}", flush=True)
    check_against_oracle(name, tensors, row_ptr, nr, nc, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("structure", ["skewed", "mesh_with_gaps"])
@pytest.mark.parametrize("name", REDUCER_GRAPHS)
def test_reducer_graphs_against_the_oracle_at_1_8_and_16_threads(name, structure, dtype):
    """The reference's result depends on its thread count (where rows are split, the order of the
    per-thread partial sums): the HIP result has to be within the tolerance of all of them."""
    rng = case_rng("threads", name, structure)
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
    gpu = gpu_launch(name, tensors, row_ptr, nr, nc)
    for threads in THREAD_SWEEP:
        print(f"case threads={threads} {name} {structure} {np.dtype(dtype).name}", flush=True)
        check_against_oracle(name, tensors, row_ptr, nr, nc, dtype, threads=threads, gpu_outs=gpu)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("structure", ["mesh", "skewed", "mostly_empty"])
def test_every_map_op(structure, dtype):
    rng = np.random.default_rng(21)
    row_ptr = row_structure(structure, rng)
    ne, nr = int(row_ptr[-1]), len(row_ptr) - 1
    t = op_zoo_inputs(rng, ne, max(nr, 64), dtype)
    print(f"case op_zoo {structure} {np.dtype(dtype).name}", flush=True)
    check_against_oracle("op_zoo", t, row_ptr, nr, max(nr, 64), dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("ne", [1, 255, 2048, 100003])
def test_flat_graphs(ne, dtype):
    rng = np.random.default_rng(ne)
    for name in ("mass_sum", "map_store"):
        tensors, _, nr, nc, _ = make_inputs(graphs.get(name), dtype, rng, ne=ne)
        print(f"case {name} ne={ne} {np.dtype(dtype).name}", flush=True)
        check_against_oracle(name, tensors, None, nr, nc, dtype)


@pytest.mark.parametrize("dtype", [np.int64, np.float64])
def test_index_shuffle_map_only_int64(dtype):
    rng = np.random.default_rng(3)
    tensors, _, nr, nc, ne = make_inputs(graphs.get("bpoints_copy"), dtype, rng, ne=77777)
    outs = check_against_oracle("bpoints_copy", tensors, None, nr, nc, dtype)
    assert outs == []
    _, after = gpu_launch("bpoints_copy", tensors, None, nr, nc)
    assert np.array_equal(after["bp_1"], tensors["bpoints"][:, 1])


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_row_structures(seed):
    """Forty random (sub-graph, dtype, row structure) combinations per seed against the oracle."""
    rng = np.random.default_rng(seed)
    names = REDUCER_GRAPHS + ["op_zoo"]
    for case in range(40):
        name = names[int(rng.integers(0, len(names)))]
        dtype = [np.float32, np.float64][int(rng.integers(0, 2))]
        row_ptr = random_row_structure(rng)
        nr, ne = len(row_ptr) - 1, int(row_ptr[-1])
        print(f"case random seed={seed} #{case} {name} {np.dtype(dtype).name} rows={nr} ne={ne}", flush=True)
        if name == "op_zoo":
            check_against_oracle(name, op_zoo_inputs(rng, ne, max(nr, 64), dtype), row_ptr, nr, max(nr, 64), dtype)
        else:
            tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
            check_against_oracle(name, tensors, row_ptr, nr, nc, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reference_harness_default_problem(dtype):
    """The default problem of the reference's CUDA harness (src/flex_spmv_full_red.cu:624-635): 1543 vertices,
    123134 edges, 12314 rows, item widths 2 / 2 / 6, random sorted row offsets with empty rows - on the
    sub-graph of its toy model - and of its CPU harness (main.cpp: 3241 rows, 324123 non-zeros, seed 12)."""
    for rows, ne, seed in ((12314, 123134, 49), (3241, 324123, 12)):
        rng = np.random.default_rng(seed)
        cuts = np.sort(rng.integers(0, ne + 1, rows - 1))
        row_ptr = np.concatenate([[0], cuts, [ne]]).astype(np.int32)
        tensors, row_ptr, nr, nc, _ = make_inputs(graphs.get("system_two_selectors"), dtype, rng, row_ptr=row_ptr,
                                                  positive=False)
        print(f"case harness rows={rows} ne={ne} {np.dtype(dtype).name}", flush=True)
        check_against_oracle("system_two_selectors", tensors, row_ptr, nr, nc, dtype)


def test_results_are_bitwise_reproducible():
    rng = np.random.default_rng(9)
    row_ptr = row_structure("skewed", rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get("spmv_dot"), np.float32, rng, row_ptr=row_ptr)
    a, _ = gpu_launch("spmv_dot", tensors, row_ptr, nr, nc)
    for _ in range(3):
        b, _ = gpu_launch("spmv_dot", tensors, row_ptr, nr, nc)
        assert all(np.array_equal(x, y) for x, y in zip(a, b))


def test_tile_table_reuse_matches_full_launches():
    """Launches that keep the tile table of the previous launch give the bits of a full launch; a
    different row structure in between invalidates the table (the launcher notices and searches again)."""
    rng = np.random.default_rng(17)
    ext = load_named("spmv_dot", build_if_missing=False)

    def arguments(structure):
        row_ptr = row_structure(structure, rng)
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get("spmv_dot"), np.float64, rng, row_ptr=row_ptr)
        out = []
        for pname in ext.param_names():
            if pname == "row_end_offsets":
                out.append(torch.from_numpy(row_ptr).cuda())
            elif pname in ("num_rows", "num_cols"):
                out.append(int(nr if pname == "num_rows" else nc))
            else:
                out.append(torch.from_numpy(np.ascontiguousarray(tensors[pname])).cuda())
        return out

    a_args, b_args = arguments("skewed"), arguments("mesh")
    full_a = [o.clone() for o in ext.merged_spmv_launch(*a_args)]
    full_b = [o.clone() for o in ext.merged_spmv_launch(*b_args)]
    ext.reuse_tiles = True
    try:
        for args, full in ((a_args, full_a), (a_args, full_a), (a_args, full_a), (b_args, full_b),
                           (b_args, full_b), (a_args, full_a)):
            got = ext.merged_spmv_launch(*args)
            torch.cuda.synchronize()
            assert all(torch.equal(g, f) for g, f in zip(got, full))
    finally:
        ext.reuse_tiles = False


# ---------------------------------------------------------------------------------------------
# the five benchmark workloads at oracle-friendly sizes
# ---------------------------------------------------------------------------------------------
def test_workload_1_laplacian_2d_fp32():
    w = W.laplacian_2d_spmv(256)
    assert (w.num_rows, w.ne, w.algorithmic_bytes) == (65536, 326656, 3399684)
    (y,), _ = gpu_launch(w.graph, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols)
    (ref,), _ = run_oracle(graphs.get(w.graph), w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, THREADS)
    A = sp.csr_matrix((np.abs(w.tensors["vals"]).astype(np.float64), w.tensors["selector_idx"], w.row_end_offsets))
    row_scale = A @ np.abs(w.tensors["x"]).astype(np.float64)
    assert np.all(np.abs(y.astype(np.float64) - ref) <= 1e-5 * np.maximum(np.abs(ref), row_scale))


def test_workload_2_spring_mass_fp32():
    w = W.spring_mass_grid(100)
    check_against_oracle(w.graph, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, np.float32)


def test_workload_3_shallow_water_fp64():
    w = W.shallow_water_mesh(60000)
    check_against_oracle(w.graph, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, np.float64)
    m = W.mass_sum_of(w)
    check_against_oracle(m.graph, m.tensors, None, m.num_rows, m.num_cols, np.float64)


def test_workload_4_rmat_fp32():
    w = W.rmat_spmv(16)
    (y,), _ = gpu_launch(w.graph, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols)
    (ref,), _ = run_oracle(graphs.get(w.graph), w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, THREADS)
    assert np.all(np.abs(y - ref) <= 1e-5 * np.abs(ref))      # all terms positive: the row scale is |ref|
    assert np.all(y[np.diff(w.row_end_offsets) == 0] == 0)


def test_workload_5_poisson_fp64():
    w = W.poisson_3d_spmv_dot(64)
    check_against_oracle(w.graph, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, np.float64)


# ---------------------------------------------------------------------------------------------
# full benchmark sizes: size-independent properties instead of the oracle
# ---------------------------------------------------------------------------------------------
def test_poisson_256_cubed_stencil_and_dot():
    w = W.poisson_3d_spmv_dot(256)
    ext = load_named(w.graph, build_if_missing=False)
    args = W.launch_arguments(w, ext.param_names(), "cuda")
    y, dot = ext.merged_spmv_launch(*args)
    x = args[ext.param_names().index("x")].view(256, 256, 256)
    ref = 6 * x.clone()
    ref[1:] -= x[:-1]; ref[:-1] -= x[1:]
    ref[:, 1:] -= x[:, :-1]; ref[:, :-1] -= x[:, 1:]
    ref[:, :, 1:] -= x[:, :, :-1]; ref[:, :, :-1] -= x[:, :, 1:]
    assert (y.view_as(ref) - ref).abs().max().item() <= 1e-12 * 12
    d_ref = (x * ref).sum().item()
    assert abs(dot.item() - d_ref) <= 1e-12 * abs(d_ref)


def test_rmat_scale_20_linearity_and_library_product():
    w = W.rmat_spmv(20)
    ext = load_named(w.graph, build_if_missing=False)
    names = ext.param_names()
    args = W.launch_arguments(w, names, "cuda")
    (y1,) = ext.merged_spmv_launch(*args)
    xi = names.index("x")
    x1 = args[xi]
    x2 = torch.rand_like(x1)
    args[xi] = x2
    (y2,) = ext.merged_spmv_launch(*args)
    args[xi] = (0.5 * x1 + 2.0 * x2).contiguous()
    (y3,) = ext.merged_spmv_launch(*args)
    scale = (0.5 * y1 + 2.0 * y2).abs().max().item()
    assert (y3 - (0.5 * y1 + 2.0 * y2)).abs().max().item() <= 1e-5 * scale
    A = torch.sparse_csr_tensor(args[names.index("row_end_offsets")].long(), args[names.index("selector_idx")].long(),
                                args[names.index("vals")].double(), size=(w.num_rows, w.num_cols))
    ref = (A @ x1.double().unsqueeze(1)).squeeze(1)
    assert ((y1.double() - ref).abs() <= 1e-5 * ref.abs()).all()


def test_shallow_water_1m_points_conservation_and_lake_at_rest():
    """Full-size mesh (about 2 M cells, 6 M half-edges).  Every interior face appears once per direction
    with opposite normals and the Rusanov flux is antisymmetric, so the fluxes summed over all cells cancel;
    a lake at rest (constant depth, no momentum) has zero mass flux everywhere and, in cells without a wall
    face, zero momentum flux (the scaled normals of a closed polygon add up to zero)."""
    w = W.shallow_water_mesh(1_000_000)
    ext = load_named(w.graph, build_if_missing=False)
    names = ext.param_names()
    args = W.launch_arguments(w, names, "cuda")
    print(f"case swe 1M cells={w.num_rows} half-edges={w.ne}", flush=True)
    fh, fu, fv = ext.merged_spmv_launch(*args)
    for f in (fh, fu, fv):
        scale = float(f.abs().sum())
        assert abs(float(f.sum())) <= 1e-12 * scale
    U = args[names.index("U")]
    rest = torch.zeros_like(U)
    rest[:, 0] = 1.25
    args[names.index("U")] = rest
    fh, fu, fv = ext.merged_spmv_launch(*args)
    assert float(fh.abs().max()) == 0.0
    ptr = args[names.index("row_end_offsets")].long()
    interior = (ptr[1:] - ptr[:-1]) == 3                      # all three faces are interior faces
    pressure_scale = 0.5 * 9.81 * 1.25 ** 2 * float(args[names.index("length")].max())
    assert float(fu[interior].abs().max()) <= 1e-12 * pressure_scale
    assert float(fv[interior].abs().max()) <= 1e-12 * pressure_scale
    assert float(fu[~interior].abs().max()) > 0              # wall cells do feel the missing face


def test_largest_supported_size_poisson_644_cubed():
    """2.134e9 merge items (rows + non-zeros), 99.4 % of what 32-bit offsets allow: the 7-point operator on
    a 644^3 grid, assembled on the device, against the stencil applied with dense shifts; one size
    larger is refused with the reference's error."""
    n, dev = 644, "cuda"
    N = n ** 3
    i = torch.arange(N, device=dev, dtype=torch.int64)
    x_, y_, z_ = i % n, (i // n) % n, i // (n * n)
    offs = [(-n * n, z_ > 0), (-n, y_ > 0), (-1, x_ > 0), (0, None), (1, x_ < n - 1), (n, y_ < n - 1), (n * n, z_ < n - 1)]
    cnt = torch.zeros(N, device=dev, dtype=torch.int64)
    for _, m in offs:
        cnt += 1 if m is None else m.to(torch.int64)
    ptr = torch.zeros(N + 1, device=dev, dtype=torch.int64)
    torch.cumsum(cnt, 0, out=ptr[1:])
    nnz = int(ptr[-1])
    assert N + nnz == 2134231456
    cols = torch.empty(nnz, device=dev, dtype=torch.int32)
    vals = torch.empty(nnz, device=dev, dtype=torch.float64)
    pos = ptr[:-1].clone()
    for o, m in offs:
        sel = i if m is None else m.nonzero().squeeze(1)
        cols[pos[sel]] = (sel + o).to(torch.int32)
        vals[pos[sel]] = 6.0 if o == 0 else -1.0
        pos[sel] += 1
    rows = torch.repeat_interleave(torch.arange(N, device=dev, dtype=torch.int32), cnt)
    del pos, cnt, x_, y_, z_, offs, sel, i
    x = torch.rand(N, device=dev, dtype=torch.float64) * 2 - 1
    ext = load_named("spmv_dot", build_if_missing=False)
    given = {"vals": vals, "x": x, "selector_col_idx": cols, "selector_row_idx": rows,
             "row_end_offsets": ptr.to(torch.int32), "num_rows": N, "num_cols": N}
    print(f"case largest size rows={N} nnz={nnz}", flush=True)
    y, dot = ext.merged_spmv_launch(*[given[k] for k in ext.param_names()])
    xb = x.view(n, n, n)
    ref = 6 * xb.clone()
    ref[1:] -= xb[:-1]; ref[:-1] -= xb[1:]
    ref[:, 1:] -= xb[:, :-1]; ref[:, :-1] -= xb[:, 1:]
    ref[:, :, 1:] -= xb[:, :, :-1]; ref[:, :, :-1] -= xb[:, :, 1:]
    assert (y.view_as(ref) - ref).abs().max().item() <= 1e-12 * 12
    d_ref = (xb * ref).sum().item()
    assert abs(dot.item() - d_ref) <= 1e-12 * abs(d_ref)
    too_many_rows = 2 ** 31 - nnz                     # rows + non-zeros would no longer fit
    with pytest.raises(RuntimeError, match="2\\^31"):
        given["num_rows"] = too_many_rows
        given["row_end_offsets"] = torch.zeros(too_many_rows + 1, device=dev, dtype=torch.int32)
        ext.merged_spmv_launch(*[given[k] for k in ext.param_names()])


def test_rmat_scale_22_against_the_library_product():
    w = W.rmat_spmv(22)
    ext = load_named(w.graph, build_if_missing=False)
    names = ext.param_names()
    args = W.launch_arguments(w, names, "cuda")
    print(f"case rmat s22 rows={w.num_rows} nnz={w.ne}", flush=True)
    (y,) = ext.merged_spmv_launch(*args)
    A = torch.sparse_csr_tensor(args[names.index("row_end_offsets")].long(), args[names.index("selector_idx")].long(),
                                args[names.index("vals")].double(), size=(w.num_rows, w.num_cols))
    ref = (A @ args[names.index("x")].double().unsqueeze(1)).squeeze(1)
    assert ((y.double() - ref).abs() <= 1e-5 * ref.abs()).all()      # all terms positive: the row scale is |ref|
    empty = (torch.diff(args[names.index("row_end_offsets")]) == 0)
    assert bool((y[empty] == 0).all())


# ---------------------------------------------------------------------------------------------
# error behaviour of the call surface (TORCH_CHECK -> RuntimeError in the reference)
# ---------------------------------------------------------------------------------------------
def test_argument_checks_raise_runtime_error():
    w = W.laplacian_2d_spmv(16)
    ext = load_named(w.graph, build_if_missing=False)
    names = ext.param_names()
    good = W.launch_arguments(w, names, "cuda")

    def call(**replace):
        a = list(good)
        for k, v in replace.items():
            a[names.index(k)] = v
        return ext.merged_spmv_launch(*a)

    with pytest.raises(RuntimeError, match="CUDA"):
        call(vals=good[names.index("vals")].cpu())
    with pytest.raises(RuntimeError, match="x dtype mismatch"):
        call(x=good[names.index("x")].double())
    with pytest.raises(RuntimeError, match="selector_idx dtype mismatch"):
        call(selector_idx=good[names.index("selector_idx")].long())
    with pytest.raises(RuntimeError, match="contiguous"):
        call(x=torch.stack([good[names.index("x")]] * 2, dim=1)[:, 0])
    with pytest.raises(RuntimeError, match="non-empty"):
        call(selector_idx=good[names.index("selector_idx")][:0])
    with pytest.raises(RuntimeError, match="Unsupported dtype"):
        call(vals=good[names.index("vals")].half())
    with pytest.raises(RuntimeError, match="num_rows \\+ 1"):
        call(row_end_offsets=good[names.index("row_end_offsets")][:-1].contiguous())
    with pytest.raises(RuntimeError, match="takes"):
        ext.merged_spmv_launch(*good, 1)
    (y,) = ext.merged_spmv_launch(**dict(zip(names, good)))          # keyword names are registered too
    assert y.shape == (w.num_rows,)


def test_repeated_calls_with_the_same_arguments_take_the_shortcut_and_stay_checked():
    """A call with the very same argument objects skips the argument checks of the call before it; the
    result is a fresh output every time, and any change to an argument brings the checks back."""
    w = W.laplacian_2d_spmv(32)
    ext = load_named(w.graph, build_if_missing=False)
    names = ext.param_names()
    good = list(W.launch_arguments(w, names, "cuda"))
    (first,) = ext.merged_spmv_launch(*good)
    assert ext._same_arguments(tuple(good)) is not None
    (second,) = ext.merged_spmv_launch(*good)
    torch.cuda.synchronize()
    assert second.data_ptr() != first.data_ptr() and torch.equal(first, second)
    # new contents in the same tensors are picked up (nothing is cached but what was checked)
    good[names.index("x")].mul_(2.0)
    (third,) = ext.merged_spmv_launch(*good)
    torch.cuda.synchronize()
    assert torch.allclose(third, 2.0 * first, rtol=1e-6)
    # another tensor object, or the same object in another state, is checked again
    bad = list(good)
    bad[names.index("x")] = good[names.index("x")].double()
    with pytest.raises(RuntimeError, match="x dtype mismatch"):
        ext.merged_spmv_launch(*bad)
    (again,) = ext.merged_spmv_launch(*good)
    x = good[names.index("x")]
    x.resize_(x.numel() // 2)                      # the same object, now too short for the gathers of the rows
    assert ext._same_arguments(tuple(good)) is None
    smaller = list(good)
    smaller[names.index("num_rows")] = w.num_rows - 1
    with pytest.raises(RuntimeError, match="num_rows \\+ 1"):
        ext.merged_spmv_launch(*smaller)


def test_row_aligned_selector_preconditions_are_checked():
    """A library that serves a selector from the merge path reads its source at every row id and never reads
    the index array: a source shorter than num_rows is refused, and the optional verification catches an
    index array that is not the row ids."""
    rng = case_rng("row_aligned_checks")
    row_ptr = np.concatenate([row_structure("mesh", rng), ]).astype(np.int32)
    row_ptr = np.concatenate([row_ptr, np.full(500, row_ptr[-1], dtype=np.int32)])      # 500 trailing empty rows
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get("spmv_dot"), np.float64, rng, row_ptr=row_ptr)
    ext = load_named("spmv_dot", build_if_missing=False)
    assert ext.signature["row_indexed_value_inputs"] == ["x"]
    names = ext.param_names()
    given = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in tensors.items()}
    given.update(row_end_offsets=torch.from_numpy(row_ptr).cuda(), num_rows=nr, num_cols=nc)
    ext.merged_spmv_launch(*[given[k] for k in names])
    short = dict(given)
    used = int(tensors["selector_col_idx"].max()) + 1
    short["x"] = given["x"][: max(used, nr - 400)].contiguous()                         # covers every column, not every row
    if short["x"].numel() < nr:
        with pytest.raises(RuntimeError, match="one item of width 1 per row"):
            ext.merged_spmv_launch(*[short[k] for k in names])
    wrong = dict(given)
    wrong["selector_row_idx"] = torch.roll(given["selector_row_idx"], 1)
    ext.verify_row_aligned = True
    try:
        ext.merged_spmv_launch(*[given[k] for k in names])
        with pytest.raises(RuntimeError, match="row_aligned"):
            ext.merged_spmv_launch(*[wrong[k] for k in names])
    finally:
        ext.verify_row_aligned = False


def test_launches_on_two_streams_do_not_share_scratch():
    """Two launches of one library on two streams get a scratch buffer each (tile table, carries, partials)."""
    rng = case_rng("two_streams")
    ext = load_named("spmv_dot", build_if_missing=False)
    cases = []
    for structure in ("skewed", "mesh_with_gaps"):
        row_ptr = row_structure(structure, rng)
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get("spmv_dot"), np.float64, rng, row_ptr=row_ptr)
        given = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in tensors.items()}
        given.update(row_end_offsets=torch.from_numpy(row_ptr).cuda(), num_rows=nr, num_cols=nc)
        args = [given[k] for k in ext.param_names()]
        cases.append((args, [o.clone() for o in ext.merged_spmv_launch(*args)]))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(20):
        got = []
        for (args, _), st in zip(cases, streams):
            with torch.cuda.stream(st):
                got.append(ext.merged_spmv_launch(*args))
        torch.cuda.synchronize()
        for (_, want), g in zip(cases, got):
            assert all(torch.equal(a, b) for a, b in zip(g, want))
    dev = torch.device("cuda", torch.cuda.current_device())
    a, b = (ext.workspace_of(dev, st) for st in streams)
    assert a is not None and b is not None and a.data_ptr() != b.data_ptr()


@pytest.mark.parametrize("case", ["one_block_walks_the_chunks", "a_block_per_chunk"])
def test_rows_that_span_hundreds_of_tiles(case):
    """A row of millions of non-zeros carries into the same row from hundreds of consecutive tiles.  The fix-up
    folds such a run with the whole block (in a fixed order), also across the chunks of tiles a block handles:
    runs longer than a chunk, runs that start in the middle of a chunk, in launches small enough for one fix-up
    block (chunks of 1024 tiles) and in larger ones (a block per 256 tiles)."""
    rng = case_rng("hub_rows", case)
    if case == "one_block_walks_the_chunks":
        lens = np.concatenate([rng.integers(0, 9, 3000), [2_600_000], rng.integers(0, 9, 500), [700_000],
                               rng.integers(0, 9, 3000)])
    else:
        lens = np.concatenate([rng.integers(0, 9, 400_000), [1_500_000], rng.integers(2, 7, 900_000), [600_000, 0, 5],
                               rng.integers(0, 9, 400_000)])
    row_ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    # float64: over a million float32 terms the reference's own sequential sums are off by more than 1e-5
    for name, dtype in (("csr_spmv", np.float64), ("swe_rusanov", np.float64)):
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
        ext = load_named(name, build_if_missing=False)
        tiles = ctypes_tiling(ext, np.dtype(dtype).name, nr, ne)
        print(f"case hub rows {case} {name} {np.dtype(dtype).name} rows={nr} ne={ne} tiles={tiles}", flush=True)
        assert (tiles <= 4096) == (case == "one_block_walks_the_chunks")
        check_against_oracle(name, tensors, row_ptr, nr, nc, dtype)


def ctypes_tiling(ext, dtype, num_rows, ne):
    import ctypes
    from flexspmv_amd.binding import DTYPE_CODES
    out = (ctypes.c_int32 * 6)()
    assert ext._lib.flexspmv_tiling(DTYPE_CODES[dtype], num_rows, ne, out) == 0
    return int(out[0])
