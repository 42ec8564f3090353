"""Edge-list preparation (include/flexspmv_formats.h): COO row ids -> CSR row pointer, stable sort by row,
permutation of per-edge tensors.  Integer work: every comparison is exact.

CPU part: the numpy oracle is pinned against brute force and row-pointer invariants; the library loads,
exports what the header declares and refuses bad arguments before touching a device.
GPU part: the kernels against the oracle on seeded edge lists (empty rows, runs of empty rows long enough
for the per-row search, no edges at all, int32 and int64 ids, unsorted and out-of-range ids) and, at the
benchmark sizes, through properties that do not need the oracle.
"""
import ctypes
import os
import re
import zlib

import numpy as np
import pytest

from flexspmv_amd import build, formats
from oracle import formats_oracle as FO

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib():
    if not build.formats_is_current():
        build.compile_formats()     # hipcc cross-compiles without a GPU
    return formats.load_library()


def _edge_list(rng, num_rows, ne, kind):
    if kind == "uniform":
        rows = rng.integers(0, num_rows, ne)
    elif kind == "few_rows":       # most rows empty, long runs of them
        hot = rng.choice(num_rows, size=max(1, num_rows // 5000), replace=False)
        rows = rng.choice(hot, ne)
    elif kind == "tail":           # everything in the last rows
        rows = num_rows - 1 - rng.integers(0, min(3, num_rows), ne)
    elif kind == "head":
        rows = rng.integers(0, min(3, num_rows), ne)
    elif kind == "skewed":
        rows = np.minimum((rng.pareto(1.2, ne) * num_rows / 50).astype(np.int64), num_rows - 1)
    else:
        raise ValueError(kind)
    return np.sort(rows).astype(np.int64)


# ---------------------------------------------------------------------------------------------
# oracle pins
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(6))
def test_oracle_row_pointer_counts_smaller_ids(seed):
    rng = np.random.default_rng(seed)
    num_rows, ne = int(rng.integers(1, 40)), int(rng.integers(0, 120))
    rows = np.sort(rng.integers(0, num_rows, ne))
    ptr = FO.coo_rows_to_csr(rows, num_rows)
    brute = [sum(1 for v in rows if v < r) for r in range(num_rows + 1)]
    assert ptr.tolist() == brute


@pytest.mark.parametrize("kind", ["uniform", "few_rows", "tail", "head", "skewed"])
def test_oracle_row_pointer_invariants(kind):
    rng = np.random.default_rng(11)
    num_rows, ne = 50_000, 200_000
    rows = _edge_list(rng, num_rows, ne, kind)
    ptr = FO.coo_rows_to_csr(rows, num_rows)
    assert ptr[0] == 0 and ptr[-1] == ne and ptr.dtype == np.int32
    assert np.array_equal(ptr, np.searchsorted(rows, np.arange(num_rows + 1), side="left"))
    # row r owns exactly the edges ptr[r] .. ptr[r + 1]
    assert np.array_equal(np.repeat(np.arange(num_rows), np.diff(ptr)), rows)


def test_oracle_row_pointer_refuses_bad_ids():
    with pytest.raises(RuntimeError, match="sorted"):
        FO.coo_rows_to_csr(np.array([0, 2, 1]), 3)
    with pytest.raises(RuntimeError, match="outside"):
        FO.coo_rows_to_csr(np.array([0, 3]), 3)
    with pytest.raises(RuntimeError, match="outside"):
        FO.coo_rows_to_csr(np.array([-1, 0]), 3)
    assert FO.coo_rows_to_csr(np.array([], dtype=np.int64), 4).tolist() == [0, 0, 0, 0, 0]


@pytest.mark.parametrize("seed", range(4))
def test_oracle_sort_is_stable(seed):
    rng = np.random.default_rng(seed)
    rows = rng.integers(0, 7, 200)
    sorted_rows, perm = FO.sort_edges_by_row(rows)
    expect = sorted(range(len(rows)), key=lambda k: rows[k])     # Python's sort is stable
    assert perm.tolist() == expect
    assert sorted_rows.tolist() == [int(rows[k]) for k in expect]
    vals = rng.standard_normal((200, 3))
    moved = FO.gather_rows(vals, perm)
    assert np.array_equal(moved, vals[expect])
    assert np.array_equal(FO.scatter_rows(moved, perm), vals)


# ---------------------------------------------------------------------------------------------
# the library without a GPU
# ---------------------------------------------------------------------------------------------
def test_header_symbols_are_exported():
    with open(os.path.join(ROOT, "include", "flexspmv_formats.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(flexspmv_[a-z_]+)\s*\(", header))
    assert declared == set(formats.EXPORTED_SYMBOLS)
    lib = _lib()
    for sym in declared:
        assert getattr(lib, sym) is not None
    assert lib.flexspmv_formats_abi_version() == formats.ABI_VERSION


def test_bad_arguments_are_refused_before_any_device_work():
    lib = _lib()
    p = ctypes.c_void_p(0x1000)
    assert lib.flexspmv_coo_rows_to_csr(p, 3, 10, 10, p, p, None) == -1
    assert b"index_bytes" in lib.flexspmv_formats_last_error()
    assert lib.flexspmv_coo_rows_to_csr(p, 4, -1, 10, p, p, None) == -1
    assert lib.flexspmv_coo_rows_to_csr(None, 4, 5, 10, p, p, None) == -1
    assert lib.flexspmv_coo_rows_to_csr(p, 4, 5, 10, None, p, None) == -1
    assert lib.flexspmv_coo_rows_to_csr(p, 4, 5, 10, p, None, None) == -1
    assert lib.flexspmv_coo_rows_to_csr(p, 4, 2 ** 31, 10, p, p, None) == -3
    assert b"2^31" in lib.flexspmv_formats_last_error()
    assert lib.flexspmv_sort_edges_by_row(p, 2, 5, 10, p, p, p, 1 << 20, None) == -1
    assert lib.flexspmv_sort_edges_by_row(p, 4, 5, 0, p, p, p, 1 << 20, None) == -1
    assert lib.flexspmv_sort_edges_by_row(None, 4, 5, 10, p, p, p, 1 << 20, None) == -1
    assert lib.flexspmv_sort_edges_by_row(p, 4, 0, 10, p, p, None, 0, None) == 0       # nothing to sort
    need = lib.flexspmv_sort_workspace_bytes(5, 10)
    assert need > 0
    assert lib.flexspmv_sort_edges_by_row(p, 4, 5, 10, p, p, p, need - 1, None) == -4   # scratch too small
    assert b"workspace" in lib.flexspmv_formats_last_error()
    assert lib.flexspmv_sort_edges_by_row(p, 4, 5, 10, p, p, None, need, None) == -4
    assert lib.flexspmv_gather_rows(p, p, p, 5, 6, None) == -1                           # not a multiple of 4
    assert lib.flexspmv_gather_rows(p, p, None, 5, 8, None) == -1
    assert lib.flexspmv_scatter_rows(p, p, p, -1, 8, None) == -1
    assert lib.flexspmv_scatter_rows(p, p, p, 0, 8, None) == 0


def test_sort_scratch_follows_the_number_of_digits():
    """One 8-bit digit: counters only.  More digits: a second pair of buffers of ne words each as well."""
    lib = _lib()
    one_digit = lib.flexspmv_sort_workspace_bytes(100_000, 256)
    two_digits = lib.flexspmv_sort_workspace_bytes(100_000, 257)
    four_digits = lib.flexspmv_sort_workspace_bytes(100_000, 2 ** 31 - 1)
    assert 0 < one_digit < 100_000                      # 256 counters per block of 16 384 ids, 256 sums
    assert two_digits >= one_digit + 2 * 4 * 100_000
    assert four_digits == two_digits                    # the two pairs of buffers alternate
    assert lib.flexspmv_sort_workspace_bytes(0, 10) == 0
    assert lib.flexspmv_sort_workspace_bytes(2 ** 31, 10) == 0


def test_host_side_refuses_cpu_tensors():
    import torch
    with pytest.raises(RuntimeError, match="GPU"):
        formats.coo_rows_to_csr(torch.tensor([0, 1, 2]), 3)
    with pytest.raises(RuntimeError, match="GPU"):
        formats.gather_rows(torch.zeros(3), torch.zeros(3, dtype=torch.int32))


# ---------------------------------------------------------------------------------------------
# GPU parity
# ---------------------------------------------------------------------------------------------
def _cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["uniform", "few_rows", "tail", "head", "skewed"])
@pytest.mark.parametrize("index_dtype", ["int32", "int64"])
def test_row_pointer_matches_oracle(kind, index_dtype):
    torch = _cuda()
    rng = np.random.default_rng(zlib.crc32(f"{kind}/{index_dtype}".encode()))
    for num_rows, ne in [(1, 1), (1, 700), (5, 3), (63, 64), (64, 65), (300, 0), (20_000, 0), (4097, 2),
                         (20_000, 1), (50_000, 200_000), (1_000_003, 300_017), (3000, 1_000_000)]:
        rows = _edge_list(rng, num_rows, ne, kind) if ne else np.zeros(0, dtype=np.int64)
        print(f"case kind={kind} dtype={index_dtype} rows={num_rows} ne={ne}", flush=True)
        expect = FO.coo_rows_to_csr(rows, num_rows)
        got = formats.coo_rows_to_csr(torch.from_numpy(rows.astype(index_dtype)).cuda(), num_rows)
        assert got.dtype == torch.int32 and got.shape == (num_rows + 1,)
        assert np.array_equal(got.cpu().numpy(), expect), (kind, num_rows, ne)


@pytest.mark.gpu
@pytest.mark.parametrize("index_dtype", ["int32", "int64"])
def test_row_pointer_of_ids_that_are_not_16_byte_aligned(index_dtype):
    torch = _cuda()
    rng = np.random.default_rng(21)
    rows = np.sort(rng.integers(0, 5000, 40_003))
    d_rows = torch.from_numpy(rows.astype(index_dtype)).cuda()
    for skip in (1, 2, 3):
        view = d_rows[skip:]
        assert view.data_ptr() % 16 != 0 or index_dtype == "int64" and skip == 2
        got = formats.coo_rows_to_csr(view, 5000)
        assert np.array_equal(got.cpu().numpy(), FO.coo_rows_to_csr(rows[skip:], 5000)), skip


@pytest.mark.gpu
def test_row_pointer_reports_unsorted_and_out_of_range_ids():
    torch = _cuda()
    rng = np.random.default_rng(3)
    rows = np.sort(rng.integers(0, 1000, 50_000))
    bad = rows.copy()
    bad[[17, 18]] = bad[[18, 17]] if bad[17] != bad[18] else (bad[18] + 1, bad[17])
    with pytest.raises(RuntimeError, match="sorted"):
        formats.coo_rows_to_csr(torch.from_numpy(bad).cuda(), 1000)
    for value in (-1, 1000, 2 ** 40):
        bad = rows.copy()
        bad[-1] = value
        with pytest.raises(RuntimeError, match="outside"):
            formats.coo_rows_to_csr(torch.from_numpy(bad).cuda(), 1000)
    # the findings word is cleared by every call
    good = formats.coo_rows_to_csr(torch.from_numpy(rows).cuda(), 1000)
    assert np.array_equal(good.cpu().numpy(), FO.coo_rows_to_csr(rows, 1000))


@pytest.mark.gpu
@pytest.mark.parametrize("index_dtype", ["int32", "int64"])
def test_sort_by_row_matches_oracle(index_dtype):
    torch = _cuda()
    rng = np.random.default_rng(5)
    for num_rows, ne in [(1, 1), (1, 500), (7, 200), (1000, 1), (1000, 100_000), (1 << 20, 3_000_000), (3, 2_000_000)]:
        print(f"case dtype={index_dtype} rows={num_rows} ne={ne}", flush=True)
        rows = rng.integers(0, num_rows, ne)
        exp_rows, exp_perm = FO.sort_edges_by_row(rows)
        got_rows, got_perm = formats.sort_edges_by_row(torch.from_numpy(rows.astype(index_dtype)).cuda(), num_rows)
        assert np.array_equal(got_rows.cpu().numpy(), exp_rows)
        assert np.array_equal(got_perm.cpu().numpy(), exp_perm)       # stable: one right answer
    empty_rows, empty_perm = formats.sort_edges_by_row(torch.zeros(0, dtype=torch.int64, device="cuda"), 5)
    assert empty_rows.numel() == 0 and empty_perm.numel() == 0


@pytest.mark.gpu
def test_sort_then_row_pointer_reports_out_of_range_ids():
    torch = _cuda()
    rows = np.array([5, 1, 9, 3, 2 ** 33 + 1, 0], dtype=np.int64)
    sorted_rows, _ = formats.sort_edges_by_row(torch.from_numpy(rows).cuda(), 10)
    with pytest.raises(RuntimeError, match="outside"):
        formats.coo_rows_to_csr(sorted_rows, 10)
    rows = np.array([5, 1, 12, 3, 0], dtype=np.int32)
    sorted_rows, _ = formats.sort_edges_by_row(torch.from_numpy(rows).cuda(), 10)
    with pytest.raises(RuntimeError, match="outside"):
        formats.coo_rows_to_csr(sorted_rows, 10)


@pytest.mark.gpu
def test_sort_at_tile_boundaries_and_digit_counts():
    """Lengths around one, two and four 4 096-pair tiles (what lists below 16 M pairs are cut into) and row counts
    whose ids need 1 ... 4 digits (8, 9, 16, 17, 24, 25, 31 bits): sorted ids and permutation equal numpy's stable sort."""
    torch = _cuda()
    rng = np.random.default_rng(17)
    sizes = [1, 63, 64, 65, 4095, 4096, 4097, 16383, 16384, 16385, 32767, 32768, 32769, 100_003]
    for ne in sizes:
        for num_rows in (1, 2, 255, 256, 257, 65536, 65537, (1 << 24), (1 << 24) + 1, (1 << 31) - 1):
            rows = rng.integers(0, num_rows, ne).astype(np.int64)
            rows[rng.integers(0, ne, max(1, ne // 7))] = num_rows - 1          # the last row is always there
            print(f"case ne={ne} rows={num_rows}", flush=True)
            exp_rows, exp_perm = FO.sort_edges_by_row(rows)
            got_rows, got_perm = formats.sort_edges_by_row(torch.from_numpy(rows).cuda(), num_rows)
            assert np.array_equal(got_rows.cpu().numpy(), exp_rows)
            assert np.array_equal(got_perm.cpu().numpy(), exp_perm)


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [0, 1, 16383, 16384 + 5])
def test_sort_of_long_lists_at_tile_boundaries(extra):
    """From 16 M pairs on the scatter works on tiles of 16 384 pairs (1024 threads): lengths at and around a tile end."""
    torch = _cuda()
    rng = np.random.default_rng(19 + extra)
    ne, num_rows = (16 << 20) + extra, 3_000_001
    rows = rng.integers(0, num_rows, ne).astype(np.int32)
    exp_rows, exp_perm = FO.sort_edges_by_row(rows)
    got_rows, got_perm = formats.sort_edges_by_row(torch.from_numpy(rows).cuda(), num_rows)
    assert np.array_equal(got_rows.cpu().numpy(), exp_rows)
    assert np.array_equal(got_perm.cpu().numpy(), exp_perm)


@pytest.mark.gpu
@pytest.mark.parametrize("index_dtype", ["int32", "int64"])
def test_sort_of_ids_that_are_not_16_byte_aligned(index_dtype):
    torch = _cuda()
    rng = np.random.default_rng(23)
    for skip in (1, 2, 3):
        rows = rng.integers(0, 5000, 70_001).astype(index_dtype)
        padded = torch.from_numpy(np.concatenate([np.zeros(skip, index_dtype), rows])).cuda()
        exp_rows, exp_perm = FO.sort_edges_by_row(rows)
        got_rows, got_perm = formats.sort_edges_by_row(padded[skip:], 5000)
        assert np.array_equal(got_rows.cpu().numpy(), exp_rows)
        assert np.array_equal(got_perm.cpu().numpy(), exp_perm)


@pytest.mark.gpu
def test_sort_keeps_ids_outside_the_rows_in_place_among_the_last_row():
    """Ids outside [0, num_rows) sort as the last row (in original order among its edges) and keep their value,
    -1 if it does not fit an int32; nothing else moves."""
    torch = _cuda()
    rows = np.array([5, 9, 1, 12, 9, -3, 3, 2 ** 40, 9, 0], dtype=np.int64)
    sorted_rows, perm = formats.sort_edges_by_row(torch.from_numpy(rows).cuda(), 10)
    assert sorted_rows.cpu().tolist() == [0, 1, 3, 5, 9, 12, 9, -1, -1, 9]
    assert perm.cpu().tolist() == [9, 2, 6, 0, 1, 3, 4, 5, 7, 8]


@pytest.mark.gpu
def test_sort_with_several_tiles_per_block_matches_torch():
    """Poisson-sized list (117 M ids, 16.8 M rows): more than 4096 tiles, so every scatter block walks two tiles
    and carries its digit offsets from one to the next.  torch's stable sort is the second opinion."""
    torch = _cuda()
    ne, num_rows = 117_047_296, 16_777_216
    gen = torch.Generator(device="cuda").manual_seed(3)
    rows = torch.randint(0, num_rows, (ne,), device="cuda", dtype=torch.int32, generator=gen)
    sorted_rows, perm = formats.sort_edges_by_row(rows, num_rows)
    ref_rows, ref_perm = torch.sort(rows, stable=True)
    assert torch.equal(sorted_rows, ref_rows)
    assert torch.equal(perm, ref_perm.to(torch.int32))


@pytest.mark.gpu
def test_sort_replays_in_a_hip_graph():
    """The sort clears nothing and allocates nothing: captured once, replayed on new ids in the same buffers
    (eager sorts and synchronisation between the replays), every replay equals the oracle."""
    torch = _cuda()
    rng = np.random.default_rng(37)
    num_rows, ne = 50_000, 200_000
    lib = formats.library()
    ids = torch.zeros(ne, dtype=torch.int32, device="cuda")
    out_rows = torch.empty(ne, dtype=torch.int32, device="cuda")
    out_perm = torch.empty(ne, dtype=torch.int32, device="cuda")
    need = lib.flexspmv_sort_workspace_bytes(ne, num_rows)
    workspace = torch.empty(need, dtype=torch.uint8, device="cuda")

    def sort_into_buffers():
        stream = torch.cuda.current_stream().cuda_stream
        assert lib.flexspmv_sort_edges_by_row(ids.data_ptr(), 4, ne, num_rows, out_rows.data_ptr(), out_perm.data_ptr(),
                                              workspace.data_ptr(), need, stream) == 0

    ids.copy_(torch.from_numpy(_edge_list(rng, num_rows, ne, "uniform").astype(np.int32)))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sort_into_buffers()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sort_into_buffers()
    for rep, kind in enumerate(["skewed", "few_rows", "uniform", "tail"]):
        rows = rng.permutation(_edge_list(rng, num_rows, ne, kind)).astype(np.int32)
        ids.copy_(torch.from_numpy(rows))
        graph.replay()
        torch.cuda.synchronize()
        exp_rows, exp_perm = FO.sort_edges_by_row(rows)
        assert np.array_equal(out_rows.cpu().numpy(), exp_rows), (rep, kind)
        assert np.array_equal(out_perm.cpu().numpy(), exp_perm), (rep, kind)
        eager_rows, eager_perm = formats.sort_edges_by_row(ids, num_rows)     # eager work between replays
        assert torch.equal(eager_rows, out_rows) and torch.equal(eager_perm, out_perm)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,shape", [("float32", ()), ("float64", ()), ("float32", (3,)), ("float64", (2, 2)),
                                         ("int64", ()), ("int32", (5,))])
def test_gather_and_scatter_rows_match_oracle(dtype, shape):
    torch = _cuda()
    rng = np.random.default_rng(9)
    for n in (1, 63, 1000, 250_001):
        perm = rng.permutation(n).astype(np.int32)
        src = (rng.standard_normal((n,) + shape) * 1000).astype(dtype)
        d_src, d_perm = torch.from_numpy(src).cuda(), torch.from_numpy(perm).cuda()
        gathered = formats.gather_rows(d_src, d_perm)
        assert np.array_equal(gathered.cpu().numpy(), FO.gather_rows(src, perm))
        scattered = formats.scatter_rows(d_src, d_perm)
        assert np.array_equal(scattered.cpu().numpy(), FO.scatter_rows(src, perm))
        assert torch.equal(formats.scatter_rows(gathered, d_perm), d_src)      # round trip
        out = torch.empty_like(d_src)
        assert formats.gather_rows(d_src, d_perm, out=out) is out and torch.equal(out, gathered)


@pytest.mark.gpu
def test_row_pointer_at_benchmark_size():
    """Poisson 256^3 (117 M edges, 16.8 M rows): the pointer the workload was generated from comes back."""
    torch = _cuda()
    from flexspmv_amd import workloads as W
    w = W.poisson_3d_spmv_dot(256)
    ptr = torch.from_numpy(w.row_end_offsets).cuda()
    rows = torch.repeat_interleave(torch.arange(w.num_rows, device="cuda", dtype=torch.int32),
                                   (ptr[1:] - ptr[:-1]).to(torch.int64))
    got = formats.coo_rows_to_csr(rows, w.num_rows)
    assert torch.equal(got, ptr.to(torch.int32))


@pytest.mark.gpu
def test_sort_at_benchmark_size_is_a_stable_permutation():
    """R-MAT scale 22 (67 M edges) with its edges shuffled: ascending rows, a bijection, ties in original order,
    and the row pointer of the sorted list equals the generator's."""
    torch = _cuda()
    from flexspmv_amd import workloads as W
    w = W.rmat_spmv(22)
    ptr = torch.from_numpy(w.row_end_offsets).cuda()
    rows = torch.repeat_interleave(torch.arange(w.num_rows, device="cuda", dtype=torch.int32),
                                   (ptr[1:] - ptr[:-1]).to(torch.int64))
    shuffle = torch.randperm(w.ne, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    shuffled = rows[shuffle]
    sorted_rows, perm = formats.sort_edges_by_row(shuffled, w.num_rows)
    assert torch.equal(sorted_rows, rows)
    assert torch.equal(shuffled[perm.to(torch.int64)], sorted_rows)
    seen = torch.zeros(w.ne, dtype=torch.int32, device="cuda")
    seen[perm.to(torch.int64)] = 1
    assert int(seen.sum()) == w.ne                                              # bijection
    same_row = sorted_rows[1:] == sorted_rows[:-1]
    assert bool((perm[1:][same_row] > perm[:-1][same_row]).all())               # stable
    assert torch.equal(formats.coo_rows_to_csr(sorted_rows, w.num_rows), ptr.to(torch.int32))


@pytest.mark.gpu
def test_row_pointer_and_permutation_replay_in_a_hip_graph():
    """The row-pointer call and the permutation calls are captured once and replayed on new contents of
    the same buffers (eager work and synchronisation between the replays); every replay equals the eager result."""
    torch = _cuda()
    rng = np.random.default_rng(31)
    num_rows, ne = 30_000, 120_000
    ids = torch.zeros(ne, dtype=torch.int32, device="cuda")
    vals = torch.zeros(ne, 2, dtype=torch.float64, device="cuda")
    perm = torch.from_numpy(rng.permutation(ne).astype(np.int32)).cuda()
    ids.copy_(torch.from_numpy(_edge_list(rng, num_rows, ne, "uniform").astype(np.int32)))
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for _ in range(2):
            formats.coo_rows_to_csr_async(ids, num_rows)
            formats.scatter_rows(formats.gather_rows(vals, perm), perm)
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_ptr, g_findings = formats.coo_rows_to_csr_async(ids, num_rows)
        g_moved = formats.gather_rows(vals, perm)
        g_back = formats.scatter_rows(g_moved, perm)
    for rep, kind in enumerate(["skewed", "few_rows", "uniform", "tail"]):
        rows = _edge_list(rng, num_rows, ne, kind)
        v = rng.standard_normal((ne, 2))
        ids.copy_(torch.from_numpy(rows.astype(np.int32)))
        vals.copy_(torch.from_numpy(v))
        graph.replay()
        torch.cuda.synchronize()
        assert int(g_findings[0]) == 0
        assert np.array_equal(g_ptr.cpu().numpy(), FO.coo_rows_to_csr(rows, num_rows)), (rep, kind)
        assert np.array_equal(g_moved.cpu().numpy(), FO.gather_rows(v, perm.cpu().numpy()))
        assert torch.equal(g_back, vals)
        eager_ptr = formats.coo_rows_to_csr(ids, num_rows)          # eager work between replays
        assert torch.equal(eager_ptr, g_ptr)
