"""The tile table the device computes, bit for bit against the CPU merge-path search.

Reference: MergePathSearch (include/merged_spmv_kernels.cuh:19-50, CPU twin
cpu_template/merged_spmv_template_reducer.h:27-51) as driven by SpmvSearchKernel (:60-99): one search per
tile boundary on diagonal t * tile_items.  The device search (flex_agent.hpp: a few interpolation probes,
then bisection - inside the reducer blocks, or in tile_search_kernel for launches that ask for it) must give exactly
the coordinates of the reference's plain bisection, restated in oracle/merge_ref.hpp and pinned there
against the reference's own code.  Where the launch moves a boundary back to a row start (row-snapped
tiles, a rule of this library stated in include/flexspmv.h), the expected coordinate is that row start and
the condition is evaluated from the oracle's coordinate.
"""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from flexspmv_amd import graphs
from flexspmv_amd import workloads as W
from flexspmv_amd.binding import DTYPE_CODES, FLAG_SEARCH_TILES, load_named
from oracle import build_oracle
from tests.test_gpu_parity import case_rng
from tests.util_inputs import STRUCTURES, make_inputs, random_row_structure, row_structure

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def merge_lib():
    lib = ctypes.CDLL(build_oracle.build_merge_capi())
    lib.oracle_merge_path_search_many.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                                                  ctypes.c_int, ctypes.c_void_p]
    return lib


def tiling_of(ext, dtype, num_rows, ne):
    out = (ctypes.c_int32 * 6)()
    rc = ext._lib.flexspmv_tiling(DTYPE_CODES[dtype], num_rows, ne, out)
    assert rc == 0, ext._lib.flexspmv_last_error().decode()
    return dict(zip(("num_tiles", "nominal", "snap_slack", "snap_rows", "capacity", "search_in_blocks"), out))


def expected_table(merge_lib, row_ptr, tl):
    """Tile boundaries 0 .. num_tiles from the oracle's search plus the snapping rule."""
    row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
    row_end = np.ascontiguousarray(row_ptr[1:])
    num_rows, nnz = len(row_end), int(row_ptr[-1])
    t = np.arange(tl["num_tiles"] + 1, dtype=np.int64)
    diag = np.minimum(t * tl["nominal"], num_rows + nnz).astype(np.int32)
    xy = np.empty((len(t), 2), dtype=np.int32)
    merge_lib.oracle_merge_path_search_many(diag.ctypes.data, len(t), row_end.ctypes.data, num_rows, nnz,
                                            xy.ctypes.data)
    assert np.array_equal(xy.sum(axis=1), diag)                      # a point on its diagonal
    if tl["snap_slack"] > 0:
        x, y = xy[:, 0].astype(np.int64), xy[:, 1].astype(np.int64)
        xs = x & ~np.int64(tl["snap_rows"] - 1)
        ys = row_ptr[xs].astype(np.int64)                            # first non-zero of row xs
        interior = (t > 0) & (t < tl["num_tiles"])
        snap = interior & ((x - xs) + (y - ys) <= tl["snap_slack"])
        xy[snap, 0] = xs[snap]
        xy[snap, 1] = ys[snap]
    return xy


def device_table(name, dtype, tensors, row_ptr, num_rows, num_cols):
    """Launch the library and read the tile table back from its workspace (every launch leaves it there,
    whether its blocks confirmed the entries of an earlier launch, searched, or a search kernel ran)."""
    ext = load_named(name, build_if_missing=False)
    args = []
    for pname in ext.param_names():
        if pname == "row_end_offsets":
            args.append(torch.from_numpy(np.ascontiguousarray(row_ptr)).cuda())
        elif pname in ("num_rows", "num_cols"):
            args.append(int(num_rows if pname == "num_rows" else num_cols))
        else:
            t = tensors[pname]
            args.append(t if isinstance(t, torch.Tensor) else torch.from_numpy(np.ascontiguousarray(t)).cuda())
    ext.merged_spmv_launch(*args)
    torch.cuda.synchronize()
    ne = int(row_ptr[-1])
    tl = tiling_of(ext, dtype, num_rows, ne)
    ws = ext.workspace_of(torch.device("cuda", torch.cuda.current_device()))
    table = ws[: 8 * (tl["num_tiles"] + 1)].view(torch.int32).view(-1, 2).cpu().numpy()
    return table, tl


def check_table(merge_lib, name, dtype, tensors, row_ptr, num_rows, num_cols):
    table, tl = device_table(name, dtype, tensors, row_ptr, num_rows, num_cols)
    want = expected_table(merge_lib, row_ptr, tl)
    assert table.shape == want.shape
    bad = np.nonzero((table != want).any(axis=1))[0]
    assert bad.size == 0, (f"{name}: {bad.size} of {len(want)} tile boundaries differ, first at tile {bad[0]}: "
                           f"device {table[bad[0]]} oracle {want[bad[0]]} ({tl})")
    sizes = np.diff(table.sum(axis=1))
    assert sizes.min() >= 0 and sizes.max() <= tl["capacity"]        # every tile fits its block
    assert tuple(table[0]) == (0, 0) and tuple(table[-1]) == (num_rows, int(row_ptr[-1]))
    return tl


@pytest.mark.parametrize("dtype", ["float32", "float64"])
@pytest.mark.parametrize("structure", STRUCTURES)
def test_tile_table_on_every_row_structure(merge_lib, structure, dtype):
    rng = case_rng("tile_table", structure)
    row_ptr = row_structure(structure, rng)
    for name in ("csr_spmv", "swe_rusanov"):                         # tiles of 2048 and of 1024 / 512 merge items
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.dtype(dtype), rng, row_ptr=row_ptr)
        print(f"case tile table {name} {structure} {dtype} rows={nr} ne={ne}", flush=True)
        check_table(merge_lib, name, dtype, tensors, row_ptr, nr, nc)


@pytest.mark.parametrize("seed", [31, 32])
def test_tile_table_on_random_row_structures(merge_lib, seed):
    rng = np.random.default_rng(seed)
    snapped = 0
    for case in range(30):
        dtype = ["float32", "float64"][int(rng.integers(0, 2))]
        row_ptr = random_row_structure(rng)
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get("csr_spmv"), np.dtype(dtype), rng, row_ptr=row_ptr)
        print(f"case tile table random seed={seed} #{case} {dtype} rows={nr} ne={ne}", flush=True)
        tl = check_table(merge_lib, "csr_spmv", dtype, tensors, row_ptr, nr, nc)
        snapped += tl["snap_slack"] > 0
    assert 0 < snapped < 30          # both kinds of tiling were exercised


def test_tile_table_of_the_two_large_workloads(merge_lib):
    """Poisson 256^3 (65 k+ tiles, written by tile_search_kernel, row-snapped) and R-MAT scale 22 (35 k tiles,
    boundaries on their diagonals)."""
    for w, dtype in ((W.poisson_3d_spmv_dot(256), "float64"), (W.rmat_spmv(22), "float32")):
        print(f"case tile table {w.name} rows={w.num_rows} ne={w.ne}", flush=True)
        tl = check_table(merge_lib, w.graph, dtype, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols)
        assert tl["search_in_blocks"] == 0
        print(f"  {tl}", flush=True)


# ---------------------------------------------------------------------------------------------
# Where the boundaries come from: by default every block tries the entries an earlier launch left in the
# scratch and confirms them against the row pointer it was given; whatever the scratch held, the launch
# must give the bits of a launch that searches everything, and leave the oracle's table behind.
# ---------------------------------------------------------------------------------------------
def _launch_args(ext, tensors, row_ptr_gpu, num_rows, num_cols):
    args = []
    for pname in ext.param_names():
        if pname == "row_end_offsets":
            args.append(row_ptr_gpu)
        elif pname in ("num_rows", "num_cols"):
            args.append(int(num_rows if pname == "num_rows" else num_cols))
        else:
            args.append(tensors[pname])
    return args


def _table_and_splits(ext, tl, row_ptr_gpu):
    ws = ext.workspace_of(torch.device("cuda", torch.cuda.current_device()), row_end_offsets=row_ptr_gpu)
    n = tl["num_tiles"] + 1
    table = ws[: 8 * n].view(torch.int32).view(-1, 2)
    at = (8 * n + 255) // 256 * 256                        # the splits follow the table, 256-byte aligned
    return ws, table, ws[at: at + 4 * n].view(torch.int32)


def _mode_libraries(name):
    """The shipped library and the same sources built for the other launch route and for small tiles, each as
    an extension of this test's own (the flags of a launch are set on the extension)."""
    from flexspmv_amd.binding import HipExtension
    from tests.launch_shapes.build_launch_shapes import library
    return [("shipped", HipExtension(load_named(name, build_if_missing=False).lib_path)),
            ("large", HipExtension(library("large", name), allow_variant=True)),
            ("tiny", HipExtension(library("tiny", name), allow_variant=True))]


@pytest.mark.parametrize("structure", ["mesh_with_gaps", "skewed", "one_long_row", "mostly_empty", "empty_tiles"])
@pytest.mark.parametrize("name,dtype", [("csr_spmv", "float32"), ("spmv_dot", "float64"), ("index_sums", "int64")])
def test_any_scratch_contents_give_the_result_of_a_full_search(merge_lib, structure, name, dtype):
    rng = case_rng("table_modes", structure, name)
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.dtype(dtype), rng, row_ptr=row_ptr)
    dev = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in tensors.items()}
    ptr = torch.from_numpy(np.ascontiguousarray(row_ptr)).cuda()
    for variant, ext in _mode_libraries(name):
        tl = tiling_of(ext, dtype, nr, ne)
        want = torch.from_numpy(expected_table(merge_lib, row_ptr, tl)).cuda()
        args = _launch_args(ext, dev, ptr, nr, nc)
        ext.extra_flags = FLAG_SEARCH_TILES                 # the reference's way: every boundary searched
        full = [o.clone() for o in ext.merged_spmv_launch(*args)]
        ext.extra_flags = 0
        ws, table, splits = _table_and_splits(ext, tl, ptr)
        assert torch.equal(table, want), (variant, "search")
        good_table, good_splits = table.clone(), splits.clone()
        n = tl["num_tiles"] + 1

        def poison(kind):
            if kind == "as_left":
                return
            if kind == "zeros":
                ws.zero_()
            elif kind == "ones":
                ws.fill_(255)                               # every int32 is -1
            elif kind == "huge":
                ws.view(torch.int32).fill_(2 ** 31 - 1)
            elif kind == "random":
                ws.view(torch.int32).random_(-2 ** 31, 2 ** 31 - 1)
            elif kind == "random_small":                    # plausible numbers: inside the matrix, in any order
                table.copy_(torch.stack([torch.randint(0, nr + 1, (n,), device="cuda", dtype=torch.int32),
                                         torch.randint(0, ne + 1, (n,), device="cuda", dtype=torch.int32)], 1))
                splits.copy_(torch.randint(0, nr + 1, (n,), device="cuda", dtype=torch.int32))
            elif kind == "wrong_splits":                    # the right boundaries with splits one row off
                table.copy_(good_table)
                splits.copy_(good_splits + 1)
            elif kind == "shifted_table":                   # the right splits with boundaries of the neighbouring tiles
                table.copy_(torch.roll(good_table, 1, 0))
                splits.copy_(good_splits)
            elif kind == "every_other_wrong":
                table.copy_(good_table)
                splits.copy_(good_splits)
                splits[::2] -= 1
            else:
                raise ValueError(kind)

        for kind in ("as_left", "zeros", "as_left", "ones", "huge", "random", "random_small", "wrong_splits",
                     "shifted_table", "every_other_wrong", "as_left"):
            poison(kind)
            print(f"case table modes {name} {dtype} {structure} {variant} scratch={kind} tiles={tl['num_tiles']}", flush=True)
            outs = ext.merged_spmv_launch(*args)
            for o, f in zip(outs, full):
                assert torch.equal(o, f), (variant, kind)
            assert torch.equal(table, want) and torch.equal(splits, good_splits), (variant, kind)


def test_a_matrix_that_changes_under_the_same_scratch(merge_lib):
    """One row-pointer tensor, rewritten between launches (same sizes, other rows): the table of the matrix before
    is confirmed where it still holds and replaced where it does not."""
    rng = np.random.default_rng(77)
    ir = graphs.get("csr_spmv")
    nr = 20_000
    lengths = rng.integers(0, 12, nr)
    for variant, ext in _mode_libraries("csr_spmv"):
        row_ptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        tensors, row_ptr, _, nc, ne = make_inputs(ir, np.dtype("float64"), rng, row_ptr=row_ptr)
        dev = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in tensors.items()}
        ptr = torch.from_numpy(row_ptr).cuda()
        args = _launch_args(ext, dev, ptr, nr, nc)
        tl = tiling_of(ext, "float64", nr, ne)
        for step in range(6):
            if step > 0:                                    # move non-zeros between rows of one part of the matrix
                lo = int(rng.integers(0, nr - 2000))
                part = lengths[lo: lo + 2000].copy()
                rng.shuffle(part)
                lengths[lo: lo + 2000] = part
                row_ptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
                ptr.copy_(torch.from_numpy(row_ptr))
            print(f"case changing matrix {variant} step={step} tiles={tl['num_tiles']}", flush=True)
            ext.extra_flags = 0
            got = ext.merged_spmv_launch(*args)[0].clone()
            _, table, _ = _table_and_splits(ext, tl, ptr)
            assert torch.equal(table, torch.from_numpy(expected_table(merge_lib, row_ptr, tl)).cuda()), (variant, step)
            ext.extra_flags = FLAG_SEARCH_TILES
            assert torch.equal(ext.merged_spmv_launch(*args)[0], got), (variant, step)


def test_which_kernels_a_launch_runs(capfd):
    """By default no launch runs a search kernel (its blocks confirm the table of the launch before, or search
    themselves); with FLEXSPMV_FLAG_SEARCH_TILES large launches run one and small ones search inside their blocks."""
    from flexspmv_amd.binding import FLAG_DEBUG_SYNC

    def kernels(w, flags):
        ext = load_named(w.graph, build_if_missing=False)
        args = W.launch_arguments(w, ext.param_names(), "cuda")
        ext.extra_flags = flags | FLAG_DEBUG_SYNC
        try:
            capfd.readouterr()
            ext.merged_spmv_launch(*args)
            torch.cuda.synchronize()
        finally:
            ext.extra_flags = 0
        return [line.split("]")[1].split("<<<")[0].strip() for line in capfd.readouterr().err.splitlines() if "<<<" in line]

    small = W.laplacian_2d_spmv(64)
    snapped = W.poisson_3d_spmv_dot(128)           # 16.7 M merge items: more than 4096 tiles, short regular rows
    skewed = W.rmat_spmv(20)                       # more than 4096 tiles, long rows: boundaries stay on their diagonals
    for w in (small, snapped, skewed):
        assert "tile_search_kernel" not in kernels(w, 0)
    assert "tile_search_kernel" not in kernels(small, FLAG_SEARCH_TILES)       # searched inside the blocks
    assert "tile_search_kernel" in kernels(snapped, FLAG_SEARCH_TILES)
    assert "tile_search_kernel" in kernels(skewed, FLAG_SEARCH_TILES)


def test_captured_launch_replayed_on_a_changing_matrix(merge_lib):
    """A launch captured into a HIP graph and replayed while the matrix behind its row pointer changes between the
    replays (same sizes, eager launches and synchronisation in between): every replay confirms what still holds of
    the table in the captured scratch, searches the rest, and equals an eager launch that searches everything."""
    rng = np.random.default_rng(91)
    ir = graphs.get("spmv_dot")
    nr = 30_000
    lengths = rng.integers(0, 10, nr)
    row_ptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    tensors, row_ptr, _, nc, ne = make_inputs(ir, np.dtype("float64"), rng, row_ptr=row_ptr)
    dev = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in tensors.items()}
    ptr = torch.from_numpy(row_ptr).cuda()
    from flexspmv_amd.binding import HipExtension
    ext = HipExtension(load_named("spmv_dot", build_if_missing=False).lib_path)
    fresh = HipExtension(ext.lib_path)
    fresh.extra_flags = FLAG_SEARCH_TILES
    args = _launch_args(ext, dev, ptr, nr, nc)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ext.merged_spmv_launch(*args)                       # allocates the scratch of that stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        y, dot = ext.merged_spmv_launch(*args)
    for step in range(5):
        if step > 0:
            lo = int(rng.integers(0, nr - 3000))
            part = lengths[lo: lo + 3000].copy()
            rng.shuffle(part)
            lengths[lo: lo + 3000] = part
            row_ptr = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
            ptr.copy_(torch.from_numpy(row_ptr))
            if "selector_row_idx" in dev:                   # the row-aligned selector follows the rows
                dev["selector_row_idx"].copy_(torch.from_numpy(
                    np.repeat(np.arange(nr, dtype=np.int32), np.diff(row_ptr))))
        print(f"case captured launch, changing matrix step={step}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        want_y, want_dot = fresh.merged_spmv_launch(*args)
        assert torch.equal(y, want_y) and torch.equal(dot, want_dot), step
