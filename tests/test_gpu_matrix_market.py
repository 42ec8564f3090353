"""MatrixMarket files through the HIP path (the reference's CUDA harness reads one with --mtx,
src/flex_spmv_full_red.cu:643): general, symmetric and pattern files with empty rows, duplicate entries and
entries in no particular order are loaded by workloads.matrix_market_spmv and run as ``y = A x`` and as the
fused ``y = A x, x . y`` on the GPU against the CPU oracle and against scipy's product of the same file.
"""
import numpy as np
import pytest
import scipy.io
import scipy.sparse as sp

torch = pytest.importorskip("torch")

from flexspmv_amd import workloads as W
from tests.test_gpu_parity import case_rng, check_against_oracle

pytestmark = pytest.mark.gpu


def write_mtx(path, n_rows, n_cols, entries, field, symmetry):
    """Coordinate-format MatrixMarket text, entries written as given (1-based in the file)."""
    with open(path, "w") as f:
        f.write(f"%%MatrixMarket matrix coordinate {field} {symmetry}\n% written by tests/test_gpu_matrix_market.py\n")
        f.write(f"{n_rows} {n_cols} {len(entries)}\n")
        for e in entries:
            if field == "pattern":
                f.write(f"{e[0] + 1} {e[1] + 1}\n")
            else:
                f.write(f"{e[0] + 1} {e[1] + 1} {e[2]!r}\n")


def random_entries(rng, n_rows, n_cols, count, lower_only=False, duplicates=0):
    r = rng.integers(0, n_rows, count)
    c = rng.integers(0, n_cols, count)
    r[r % 7 == 3] = 0                                   # rows = 3 (mod 7) stay empty
    if lower_only:
        r, c = np.maximum(r, c), np.minimum(r, c)
        keep = r % 7 != 3
        r, c = r[keep], c[keep]
        # symmetric storage lists every pair once
        _, first = np.unique(r.astype(np.int64) * n_cols + c, return_index=True)
        r, c = r[first], c[first]
    v = rng.uniform(-1.0, 1.0, len(r))
    entries = [(int(a), int(b), float(x)) for a, b, x in zip(r, c, v)]
    entries += [entries[int(i)] for i in rng.integers(0, len(entries), duplicates)]   # repeated (summed by the loader)
    order = rng.permutation(len(entries))
    return [entries[int(i)] for i in order]


CASES = [
    ("general", "real", "general", 3000, 2500, 40000, 500),
    ("general_long_rows", "real", "general", 300, 5000, 150000, 0),
    ("symmetric", "real", "symmetric", 2000, 2000, 20000, 0),
    ("pattern", "pattern", "general", 4000, 4000, 30000, 0),
    ("pattern_symmetric", "pattern", "symmetric", 1500, 1500, 9000, 0),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_matrix_market_file_through_the_hip_path(tmp_path, case):
    name, field, symmetry, n_rows, n_cols, count, dups = case
    rng = case_rng("mtx", name)
    entries = random_entries(rng, n_rows, n_cols, count, lower_only=(symmetry == "symmetric"), duplicates=dups)
    path = str(tmp_path / f"{name}.mtx")
    write_mtx(path, n_rows, n_cols, entries, field, symmetry)
    a = sp.csr_matrix(scipy.io.mmread(path))            # what any other reader of the file computes with
    for dtype in (np.float64, np.float32):
        w = W.matrix_market_spmv(path, dtype=dtype)
        assert (w.num_rows, w.num_cols, w.ne) == (n_rows, n_cols, a.nnz)
        assert np.any(np.diff(w.row_end_offsets) == 0)  # the file does have empty rows
        print(f"case mtx {name} {np.dtype(dtype).name} rows={w.num_rows} nnz={w.ne}", flush=True)
        (y,) = check_against_oracle(w.graph, w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, dtype)
        ref = a.astype(np.float64) @ w.tensors["x"].astype(np.float64)
        scale = abs(a).astype(np.float64) @ np.abs(w.tensors["x"]).astype(np.float64)
        tol = 1e-5 if dtype == np.float32 else 1e-12
        assert np.all(np.abs(y - ref) <= tol * np.maximum(np.abs(ref), scale))
        if n_rows == n_cols:
            wd = W.matrix_market_spmv(path, dtype=dtype, fused_dot=True)
            y2, dot = check_against_oracle(wd.graph, wd.tensors, wd.row_end_offsets, wd.num_rows, wd.num_cols, dtype)
            assert np.array_equal(y2, y) or np.all(np.abs(y2 - ref) <= tol * np.maximum(np.abs(ref), scale))
            d_ref = float(wd.tensors["x"].astype(np.float64) @ ref)
            d_scale = float(np.abs(wd.tensors["x"]).astype(np.float64) @ scale)
            assert abs(float(dot[0]) - d_ref) <= tol * max(abs(d_ref), d_scale)
