"""Seeded inputs for any sub-graph of flexspmv_amd.graphs, from its binding signature."""
import numpy as np

from flexspmv_amd.codegen.merged_gen_binding import generate_binding_code


def row_structure(kind, rng, tile=2048):
    """CSR row pointer of a named shape.  Shapes are chosen to hit every path of the reducer kernel."""
    if kind == "mesh":            # 3..7 per row: row path
        lens = rng.integers(3, 8, 5000)
    elif kind == "mesh_with_gaps":  # short rows and empty rows mixed: row path, open rows at tile ends
        lens = rng.integers(0, 9, 7000)
    elif kind == "skewed":        # empty rows, long rows spanning several tiles: merge path + carry runs
        lens = (rng.pareto(1.2, 3000) * 3).astype(np.int64)
        lens[rng.random(3000) < 0.35] = 0
        lens[100] = 3 * tile + 17
        lens[101] = 0
        lens[2000] = tile
    elif kind == "one_long_row":  # a single row far longer than a tile: every tile carries into it
        lens = np.array([0, 0, 9 * tile + 5, 0])
    elif kind == "mostly_empty":  # many row ends per tile: merge path, every row through the LDS buffer
        lens = (rng.random(20000) < 0.05).astype(np.int64) * rng.integers(1, 40, 20000)
        lens[-1] = 7
    elif kind == "tiny":
        lens = np.array([1])
    elif kind == "exact_tiles":   # rows + nnz is a multiple of the tile
        lens = np.full(512, 7)
    elif kind == "len33":         # one row just over the row-path limit inside regular rows
        lens = np.full(900, 5)
        lens[450] = 33
    elif kind == "empty_tiles":   # tiles that consist of row ends only (R = tile), between ordinary rows
        lens = np.concatenate([np.full(300, 6), np.zeros(3 * tile + 100, dtype=np.int64), np.full(300, 9)])
    elif kind == "uniform_30":    # row path, rows longer than its unrolled part
        lens = np.full(700, 30)
    elif kind == "uneven_short":  # all rows short but of very different lengths: merge path by the evenness rule
        lens = rng.integers(1, 31, 3000)
    elif kind == "rows_5":        # more rows per tile than the row path prefetches: merge path on a regular matrix
        lens = np.full(4000, 4) + (np.arange(4000) % 2)
    else:
        raise ValueError(kind)
    if lens.sum() == 0:
        lens[-1] = 1
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


def random_row_structure(rng, max_edges=1_500_000):
    """A row pointer drawn from eight families of row-length distributions (uniform short, uniform long,
    heavy-tailed, constant, isolated giants, sparse rows between empty ones, around the row-path limit,
    blocks of different character)."""
    kind = int(rng.integers(0, 8))
    n = int(rng.integers(1, 6000))
    if kind == 0:
        lens = rng.integers(0, 4, n)
    elif kind == 1:
        lens = rng.integers(0, 40, n)
    elif kind == 2:
        lens = (rng.pareto(1.1, n) * rng.integers(1, 20)).astype(np.int64)
    elif kind == 3:
        lens = np.full(n, int(rng.integers(1, 70)))
    elif kind == 4:
        lens = np.zeros(n, dtype=np.int64)
        k = rng.integers(0, n, max(1, n // 50))
        lens[k] = rng.integers(1, 5000, len(k))
    elif kind == 5:
        lens = rng.integers(0, 2, n) * rng.integers(1, 300, n)
    elif kind == 6:
        lens = rng.integers(28, 37, n)
    else:
        lens = np.concatenate([rng.integers(3, 8, n), np.zeros(int(rng.integers(0, 5000)), dtype=np.int64),
                               rng.integers(0, 3, n)])
    lens = lens.astype(np.int64)
    if lens.sum() > max_edges:
        lens = lens // (lens.sum() // max_edges + 1)
    if lens.sum() == 0:
        lens[-1] = 1
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


STRUCTURES = ["mesh", "mesh_with_gaps", "skewed", "one_long_row", "mostly_empty", "tiny", "exact_tiles", "len33",
              "empty_tiles", "uniform_30", "uneven_short", "rows_5"]


def make_inputs(ir, dtype, rng, row_ptr=None, ne=None, positive=True):
    """(tensors, row_ptr, num_rows, num_cols, ne) for a sub-graph.  Gather sources get
    max(num_rows, 64) rows so that row-aligned selectors index them safely."""
    sig = generate_binding_code(None, ir.inputs, ir.outputs, ir.selector_register)
    if sig["has_reducer"]:
        assert row_ptr is not None
        num_rows, ne = len(row_ptr) - 1, int(row_ptr[-1])
    else:
        num_rows = ne
    nv = max(num_rows, 64)
    row_aligned = {s["selector_name"] + "_idx" for s in ir.selector_register if s.get("row_aligned")}
    lo, hi = (0.5, 2.0) if positive else (-1.0, 1.0)
    tensors = {}
    for name in sig["non_gather_value_inputs"]:
        d = sig["value_dims"][name]
        tensors[name] = _values(rng, (ne, d) if d > 1 else (ne,), dtype, lo, hi)
    for name in sig["gather_value_inputs"]:
        d = sig["value_dims"][name]
        tensors[name] = _values(rng, (nv, d) if d > 1 else (nv,), dtype, lo, hi)
    for name in sig["index_inputs"]:
        if name in row_aligned and sig["has_reducer"]:
            tensors[name] = np.repeat(np.arange(num_rows, dtype=np.int32), np.diff(row_ptr)).astype(np.int32)
        elif sig["has_reducer"]:
            # never the edge's own row: keeps distances in the mesh maps away from an exact 0 / 0
            rows = np.repeat(np.arange(num_rows, dtype=np.int64), np.diff(row_ptr))
            tensors[name] = ((rows + 1 + rng.integers(0, nv - 1, ne)) % nv).astype(np.int32)
        else:
            tensors[name] = rng.integers(0, nv, ne).astype(np.int32)
    num_cols = nv if sig["gather_value_inputs"] else ne
    return tensors, row_ptr, num_rows, num_cols, ne


def _values(rng, shape, dtype, lo, hi):
    if np.dtype(dtype).kind == "i":
        return rng.integers(-1000, 1000, shape).astype(dtype)
    return rng.uniform(lo, hi, shape).astype(dtype)
