"""The toy ``System`` model of the reference's code-generation driver (easier_spmv.py:17-69): two
selectors on one vertex tensor, edge tensors of item shape (2,1) and (2,3), two per-edge stores and one
reducer.  The row ids are sorted by default (the reference draws them unsorted, which its own COO -> CSR
conversion cannot represent; ``sorted_rows=False`` reproduces that)."""
from __future__ import annotations

import torch

from .. import frontend as esr


class System(esr.Module):
    def __init__(self, spm_1, spm_2, vector_x, col_indices_1, col_indices_2, row_indices, output_y_map_1,
                 output_y_map_2, output_y_reducer_1, num_rows):
        super().__init__()
        self.spm_1 = esr.Tensor(spm_1, mode="partition")              # (ne, 2, 1)
        self.spm_2 = esr.Tensor(spm_2, mode="partition")              # (ne, 2, 3)
        self.vector_x = esr.Tensor(vector_x, mode="partition")        # (nv, 2, 1)
        self.y_add_1 = esr.Tensor(output_y_map_1, mode="partition")   # (ne, 2, 1)
        self.y_add_2 = esr.Tensor(output_y_map_2, mode="partition")   # (ne, 2, 3)
        self.y_reducer_1 = esr.Tensor(output_y_reducer_1, mode="partition")  # (nr, 2, 1)
        self.selector_1 = esr.Selector(col_indices_1)
        self.selector_2 = esr.Selector(col_indices_2)
        self.reducer_1 = esr.Reducer(row_indices, num_rows)

    def forward(self):
        r_1 = self.selector_1(self.vector_x)
        r_2 = self.selector_2(self.vector_x)
        add_1 = r_1 + r_2 + self.spm_1
        add_2 = r_1 + r_2 + self.spm_2
        self.y_add_1[:] = add_1
        self.y_add_2[:] = add_2
        self.y_reducer_1[:] = self.reducer_1(add_1)


def make_system(num_nnz=20, num_cols=11, num_rows=11, device="cpu", dtype=torch.float64, seed=52,
                sorted_rows=True) -> System:
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.rand(*s, generator=g, dtype=dtype).to(device)   # noqa: E731
    rows = torch.randint(0, num_rows, (num_nnz,), generator=g)
    if sorted_rows:        # False: the reference's own set-up; the replacement wrapper then sorts the edges
        rows = torch.sort(rows).values
    rows = rows.to(device)
    col_1 = torch.randint(0, num_cols, (num_nnz,), generator=g).to(device)
    col_2 = torch.randint(0, num_cols, (num_nnz,), generator=g).to(device)
    return System(rnd(num_nnz, 2, 1), rnd(num_nnz, 2, 3), rnd(num_cols, 2, 1), col_1, col_2, rows,
                  torch.zeros(num_nnz, 2, 1, dtype=dtype, device=device),
                  torch.zeros(num_nnz, 2, 3, dtype=dtype, device=device),
                  torch.zeros(num_rows, 2, 1, dtype=dtype, device=device), num_rows)
