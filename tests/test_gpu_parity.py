"""Parity of the HIP path with the CPU oracle, through the C interface of the generated libraries
(ctypes launcher in flexspmv_amd.binding).  Tolerances: float32 1e-5, float64 1e-12; integers and structure
exact.  A reducer output is held to the tolerance row by row, relative to max(|reference|, sum of
|contributions| of that row), plus a floor of the row's own: FLOOR_ULPS ulps of its largest contribution and
twice what moves of the inputs by an ulp or two change in its contributions (the criterion and its reasons
are in oracle/parity.py).  Other outputs are relative to their largest magnitude.
"""
import zlib

import numpy as np
import pytest
import scipy.sparse as sp

torch = pytest.importorskip("torch")

from flexspmv_amd import graphs
from flexspmv_amd import workloads as W
from flexspmv_amd.binding import load_named
from oracle.parity import FLOOR_ULPS, TOL, aggregator_bounds, reducer_row_scales, row_excess
from oracle.runner import run_oracle
from tests.util_inputs import STRUCTURES, make_inputs, random_row_structure, row_structure
from tests.test_oracle_pins import op_zoo_inputs

pytestmark = pytest.mark.gpu

THREADS = 8   # oracle thread count of most cases; its rounding depends on it, which the tolerances absorb
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


def assert_close(got, ref, tol, what, row_scale=None, row_floor=None):
    assert got.shape == ref.shape and got.dtype == ref.dtype, what
    if got.dtype.kind == "i":
        assert np.array_equal(got, ref), what
        return
    if not ref.size:
        return
    if row_scale is not None:
        excess = row_excess(got, ref, tol, row_scale, row_floor)
        if (excess > 1.0).any():
            i = int(np.argmax(excess))
            raise AssertionError(f"{what}: {int((excess > 1.0).sum())} elements off; worst at flat index {i}: |diff| "
                                 f"{abs(float(got.flat[i]) - float(ref.flat[i])):.3e} is {excess.flat[i]:.2f} x what the "
                                 f"row allows (row scale {row_scale.flat[i]:.3e}, floor {row_floor.flat[i]:.3e})")
        return
    diff = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    scale = max(float(np.abs(ref).max()), 1e-300)
    err = float(diff.max())
    assert err <= tol * scale, f"{what}: max |diff| {err:.3e} > {tol:g} * {scale:.3e}"


def check_against_oracle(name, tensors, row_ptr, num_rows, num_cols, dtype, threads=THREADS, gpu_outs=None):
    ir = graphs.get(name)
    ref_outs, ref_after = run_oracle(ir, tensors, row_ptr, num_rows, num_cols, threads)
    outs, after = gpu_outs if gpu_outs is not None else gpu_launch(name, tensors, row_ptr, num_rows, num_cols)
    assert len(outs) == len(ref_outs)
    tol = TOL.get(np.dtype(dtype), 0)
    scales = {}
    if row_ptr is not None and np.dtype(dtype).kind == "f":
        scales = reducer_row_scales(ir, tensors, row_ptr, num_cols, THREADS)
    for i, (spec, o, r) in enumerate(zip(ir.outputs, outs, ref_outs)):
        agg = aggregator_bounds(ir, tensors, row_ptr, num_rows, num_cols, i, tol)
        if agg is not None:
            # float32 aggregators: centred on the oracle evaluated in float64, and within the sequential-summation
            # bound of the float32 oracle at the most threads the reference allows (oracle/parity.py)
            assert_close(o.astype(np.float64), agg["centre"], tol, f"{name} aggregator {spec['name']} vs float64 oracle")
            off = float(np.abs(o.astype(np.float64) - agg["fine"].astype(np.float64)).max())
            assert off <= agg["bound_fine"], (f"{name} aggregator {spec['name']} vs float32 oracle at 256 threads: "
                                              f"{off:.3e} > {agg['bound_fine']:.3e} (chains of {agg['chain']})")
        else:
            scale, floor = scales.get(i, (None, None))
            assert_close(o, r, tol, f"{name} output {spec['name']}", row_scale=scale, row_floor=floor)
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


INT64_REDUCER_GRAPHS = ["index_spmv", "index_sums"]


@pytest.mark.parametrize("structure", STRUCTURES)
@pytest.mark.parametrize("name", INT64_REDUCER_GRAPHS)
def test_int64_reducers_and_aggregators_are_bit_exact(name, structure):
    """Sub-graphs traced on int64 data run the reducer, the carry fix-up and the aggregator on 8-byte integers
    (the reference dispatches <long, int> for them, codegen/merged_gen_binding.py:143-157).  Integer sums have
    one right answer whatever the order: every output equals the oracle's bit for bit, on the row path
    (meshes), the merge path (skewed rows, carry runs) and with empty rows and tiles."""
    rng = case_rng("int64", name, structure)
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.int64, rng, row_ptr=row_ptr)
    print(f"case {name} {structure} int64 rows={nr} ne={ne}", flush=True)
    outs = check_against_oracle(name, tensors, row_ptr, nr, nc, np.int64)
    assert all(o.dtype == np.int64 for o in outs)
    # ... and the same library on float64 data stays within the float tolerance
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.float64, rng, row_ptr=row_ptr)
    check_against_oracle(name, tensors, row_ptr, nr, nc, np.float64)


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


def test_debug_flag_reports_every_kernel_of_a_launch(capfd):
    """FLEXSPMV_FLAG_DEBUG_SYNC is the reference's debug_synchronous (cuda_template/reducer/merged_spmv_template.cuh:
    106-124): every kernel of the launch is named on stderr with its grid, block and LDS bytes, and the result is
    the same."""
    from flexspmv_amd.binding import FLAG_DEBUG_SYNC
    w = W.laplacian_2d_spmv(64)
    ext = load_named(w.graph, build_if_missing=False)
    args = W.launch_arguments(w, ext.param_names(), "cuda")
    (plain,) = ext.merged_spmv_launch(*args)
    torch.cuda.synchronize()
    capfd.readouterr()
    ext.extra_flags = FLAG_DEBUG_SYNC
    try:
        (reported,) = ext.merged_spmv_launch(*args)
    finally:
        ext.extra_flags = 0
    err = capfd.readouterr().err
    assert torch.equal(plain, reported)
    assert "reducer launch: 4096 rows" in err and "tiles of" in err
    lines = [l for l in err.splitlines() if "<<<" in l]
    assert [l.split("]")[1].split("<<<")[0].strip() for l in lines] == \
        ["reduce_kernel (several edges per load)", "fixup_kernel (one block)"]   # a row-snapped launch of a few tiles
    assert all("static LDS" in l and "registers per thread" in l for l in lines)
    assert ", 256, 0," in lines[0]                 # 256 threads per reducer block
    # a flat (aggregator-only) library reports its two kernels
    m = W.mass_sum_of(W.shallow_water_mesh(2000))
    flat = load_named(m.graph, build_if_missing=False)
    flat.extra_flags = FLAG_DEBUG_SYNC
    try:
        flat.merged_spmv_launch(*W.launch_arguments(m, flat.param_names(), "cuda"))
    finally:
        flat.extra_flags = 0
    err = capfd.readouterr().err
    assert "flat_kernel<<<" in err and "aggregate_kernel<<<" in err
