"""The kernels of a launch depend on its size: up to a few thousand tiles the reducer blocks search their own
tile boundaries and one block folds carries and aggregators; beyond that a search kernel, one fix-up block per
256 tiles and a final sum run.  Inputs the CPU oracle handles in seconds only reach the first route with the
shipped libraries, so this file runs them through test-only builds of the same generated sources and the same
kernels that take the other route at every size (tests/launch_shapes/build_launch_shapes.py):

  large   the shipped tile shape on the large-launch route;
  tiny    256-item tiles (64 threads x 4 items) on the large-launch route: hundreds of tiles per launch, and a
          row of a few ten thousand non-zeros carries through more tiles than one fix-up block handles.

Same criteria as tests/test_gpu_parity.py (float32 1e-5, float64 1e-12, row by row), same oracle; the tile
tables are compared bit for bit with the oracle's merge-path search.
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from flexspmv_amd import graphs
from flexspmv_amd.binding import FLAG_SEARCH_TILES, HipExtension
from tests import test_gpu_parity as parity
from tests import test_gpu_tile_table as tile_table
from tests.launch_shapes.build_launch_shapes import GRAPHS, VARIANTS, library
from tests.test_oracle_pins import op_zoo_inputs
from tests.util_inputs import STRUCTURES, make_inputs, random_row_structure, row_structure

pytestmark = pytest.mark.gpu

merge_lib = tile_table.merge_lib      # the oracle's search behind a C interface (module-scoped fixture)

_extensions = {}


def variant_extension(variant, name):
    key = (variant, name)
    if key not in _extensions:
        path = library(variant, name)
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built: run __graft_entry__.build() "
                               "(or tests/launch_shapes/build_launch_shapes.py)")
        _extensions[key] = HipExtension(path, allow_variant=True)
        # these builds exist for the route with a search kernel and a fix-up block per 256 tiles: every launch
        # of theirs searches all boundaries afresh (the default would try the table of the launch before)
        _extensions[key].extra_flags = FLAG_SEARCH_TILES
    return _extensions[key]


@pytest.fixture(params=sorted(VARIANTS))
def variant(request, monkeypatch):
    """Point the parity and tile-table helpers at one variant's libraries."""
    def load(name, build_if_missing=False):
        return variant_extension(request.param, name)
    monkeypatch.setattr(parity, "load_named", load)
    monkeypatch.setattr(tile_table, "load_named", load)
    return request.param


def long_run_structure(rng, tile):
    """Rows that carry through many tiles, next to each other and at both ends of the matrix, between short
    and empty rows."""
    short = lambda n: rng.integers(0, 6, n)
    lens = np.concatenate([[300 * tile + 7], short(40), [0, 0], [260 * tile], [513 * tile + 1], [0], short(500),
                           [tile - 1], [tile], [tile + 1], short(3), [257 * tile + 3]])
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def test_the_variants_take_the_large_launch_route(variant):
    ext = variant_extension(variant, "csr_spmv")
    tl = tile_table.tiling_of(ext, "float32", 5000, 25000)
    assert tl["search_in_blocks"] == 0
    assert tl["capacity"] == (256 if variant == "tiny" else 2048)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("structure", STRUCTURES)
@pytest.mark.parametrize("name", parity.REDUCER_GRAPHS)
def test_reducer_graphs_on_every_row_structure(variant, name, structure, dtype):
    rng = parity.case_rng("launch shapes", name, structure)
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
    print(f"case {variant} {name} {structure} {np.dtype(dtype).name} rows={nr} ne={ne}", flush=True)
    parity.check_against_oracle(name, tensors, row_ptr, nr, nc, dtype)


@pytest.mark.parametrize("structure", STRUCTURES)
@pytest.mark.parametrize("name", parity.INT64_REDUCER_GRAPHS)
def test_int64_reducers_and_aggregators_are_bit_exact(variant, name, structure):
    """8-byte integers through the search kernel, fix-up blocks of 256 tiles (with runs that cross them on the
    256-item tiles) and the final sum: bit for bit the oracle's."""
    rng = parity.case_rng("launch shapes int64", name, structure)
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.int64, rng, row_ptr=row_ptr)
    print(f"case {variant} {name} {structure} int64 rows={nr} ne={ne}", flush=True)
    parity.check_against_oracle(name, tensors, row_ptr, nr, nc, np.int64)


def test_int64_rows_that_carry_through_several_fixup_blocks(variant):
    tile = 256 if variant == "tiny" else 2048
    for name in parity.INT64_REDUCER_GRAPHS:
        rng = parity.case_rng("long runs int64", name)
        row_ptr = long_run_structure(rng, tile)
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.int64, rng, row_ptr=row_ptr)
        print(f"case {variant} long runs {name} int64 rows={nr} ne={ne}", flush=True)
        parity.check_against_oracle(name, tensors, row_ptr, nr, nc, np.int64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("structure", ["mesh", "skewed", "mostly_empty"])
def test_every_map_op(variant, structure, dtype):
    rng = np.random.default_rng(22)
    row_ptr = row_structure(structure, rng)
    ne, nr = int(row_ptr[-1]), len(row_ptr) - 1
    t = op_zoo_inputs(rng, ne, max(nr, 64), dtype)
    print(f"case {variant} op_zoo {structure} {np.dtype(dtype).name}", flush=True)
    parity.check_against_oracle("op_zoo", t, row_ptr, nr, max(nr, 64), dtype)


@pytest.mark.parametrize("name", ["csr_spmv", "spmv_dot", "swe_rusanov"])
def test_rows_that_carry_through_several_fixup_blocks(variant, name):
    """float64: the oracle's own sequential rounding of a row of 10^5 terms is beyond 1e-5 in float32."""
    tile = 256 if variant == "tiny" else 2048
    rng = parity.case_rng("long runs", name)
    row_ptr = long_run_structure(rng, tile)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.float64, rng, row_ptr=row_ptr)
    print(f"case {variant} long runs {name} rows={nr} ne={ne}", flush=True)
    parity.check_against_oracle(name, tensors, row_ptr, nr, nc, np.float64)


@pytest.mark.parametrize("seed", [41, 42])
def test_random_row_structures(variant, seed):
    rng = np.random.default_rng(seed)
    for case in range(12):
        name = ["csr_spmv", "spmv_dot", "spring_mass", "swe_rusanov"][int(rng.integers(0, 4))]
        dtype = [np.float32, np.float64][int(rng.integers(0, 2))]
        row_ptr = random_row_structure(rng, max_edges=400_000)
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
        print(f"case {variant} random seed={seed} #{case} {name} {np.dtype(dtype).name} rows={nr} ne={ne}", flush=True)
        parity.check_against_oracle(name, tensors, row_ptr, nr, nc, dtype)


@pytest.mark.parametrize("structure", ["mesh", "skewed", "one_long_row", "empty_tiles", "rows_5"])
def test_tile_tables(variant, merge_lib, structure):
    rng = parity.case_rng("launch shapes tile table", structure)
    row_ptr = row_structure(structure, rng)
    for name, dtype in (("csr_spmv", "float32"), ("swe_rusanov", "float64")):
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), np.dtype(dtype), rng, row_ptr=row_ptr)
        print(f"case {variant} tile table {name} {structure} {dtype} rows={nr} ne={ne}", flush=True)
        tile_table.check_table(merge_lib, name, dtype, tensors, row_ptr, nr, nc)


def test_reused_tile_table_gives_the_same_bits(variant):
    ext = variant_extension(variant, "spmv_dot")
    rng = parity.case_rng("launch shapes reuse")
    results = {}
    cases = {}
    for structure in ("skewed", "mesh"):
        row_ptr = row_structure(structure, rng)
        tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get("spmv_dot"), np.float64, rng, row_ptr=row_ptr)
        args = []
        for pname in ext.param_names():
            if pname == "row_end_offsets":
                args.append(torch.from_numpy(row_ptr).cuda())
            elif pname in ("num_rows", "num_cols"):
                args.append(int(nr if pname == "num_rows" else nc))
            else:
                args.append(torch.from_numpy(np.ascontiguousarray(tensors[pname])).cuda())
        cases[structure] = args
        results[structure] = [o.clone() for o in ext.merged_spmv_launch(*args)]
    ext.reuse_tiles = True
    try:
        for structure in ("skewed", "skewed", "mesh", "mesh", "skewed"):
            got = ext.merged_spmv_launch(*cases[structure])
            torch.cuda.synchronize()
            assert all(torch.equal(g, f) for g, f in zip(got, results[structure]))
    finally:
        ext.reuse_tiles = False
