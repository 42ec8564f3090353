"""What would another layout of the column index buy on this matrix?

    python -m flexspmv_amd.drivers.layout_study [--workload rmat] [--size 22] [--mtx FILE] [--only NAME] [--steps 30]

A power-law matrix spends most of a CSR SpMV on 4-byte gathers that miss the vector L1: each is one request
to an L2 whatever it brings back.  Before changing a model's data it is worth knowing what a layout can buy,
so this tool times the shipped ``csr_spmv`` library on the matrix as it is and on variants of its column
index, prepared with plain torch operations (set-up cost reported separately as ``prep_ms``):

``csr``                     the matrix as given
``degree_numbering``        columns renumbered by descending number of non-zeros, edge order unchanged (same
                            sums bit for bit); ``x`` has to be permuted before every launch - timed, part of
                            ``step_us``
``degree_numbering_resorted``  the same numbering with every row's edges sorted by the new column id: the
                            per-edge value tensor has to be permuted as well (once, if it is a constant of
                            the model; not part of ``step_us``)
``hot_first_<n>``           only the n most-used columns move to the front, the others keep their order
``fold_<n>`` (ablation)     every column index taken modulo n: what the launch would cost if all gathers
                            fell into n * 4 bytes of ``x`` - the bound for any scheme of column blocks of
                            that size, before it pays for combining the blocks' partial rows.  Wrong results.
``hot_free_<n>`` (ablation) the n most-used columns all read ``x[0]``: what the launch would cost if gathers
                            of those columns were free (an on-chip table).  Wrong results.

One JSON line per variant: kernel and step time, set-up time, and the largest relative difference of ``y``
from the ``csr`` result (ablations: null).  ``--only`` runs a single variant, e.g. under ``rocprofv3 --pmc``.
"""
from __future__ import annotations

import argparse
import json
import sys
import time


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workload", default="rmat", choices=["rmat", "laplacian2d"])
    ap.add_argument("--size", type=int, default=None)
    ap.add_argument("--mtx", default=None, help="a MatrixMarket file instead of a generated workload (float32 y = A x)")
    ap.add_argument("--only", default=None, help="run this variant only")
    ap.add_argument("--steps", type=int, default=30)
    a = ap.parse_args(argv)

    import torch

    from flexspmv_amd import formats
    from flexspmv_amd import workloads as W
    from flexspmv_amd.binding import load_named
    if not torch.cuda.is_available():
        print("layout_study: no GPU visible", file=sys.stderr)
        return 3
    if a.mtx:
        w = W.matrix_market_spmv(a.mtx, dtype="float32")
    else:
        w = W.WORKLOADS[a.workload](a.size if a.size is not None else {"rmat": 22, "laplacian2d": 256}[a.workload])
    ext = load_named("csr_spmv", build_if_missing=False)
    n_rows, n_cols, ne = w.num_rows, w.num_cols, w.ne
    ptr = torch.from_numpy(w.row_end_offsets).cuda()
    vals = torch.from_numpy(w.tensors["vals"]).cuda()
    x = torch.from_numpy(w.tensors["x"]).cuda()
    cols = torch.from_numpy(w.tensors["selector_idx"]).cuda()

    def timed(v, xx, c, per_call=None):
        """(kernel us, step us, y): median of the reducer kernel alone, and the wall time per step of `steps` steps -
        a step being what has to run per launch: `per_call` (the permutation of x, if the variant needs one) and the
        launch itself."""
        args = (v, xx, c, ptr, n_rows, n_cols)
        for _ in range(8):
            ext.merged_spmv_launch(*args)
        torch.cuda.synchronize()
        ext.time_kernel = True
        ks = []
        for _ in range(a.steps):
            ext.merged_spmv_launch(*args)
            ks.append(ext.last_kernel_ms())
        ext.time_kernel = False
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            if per_call is not None:
                per_call()
            out = ext.merged_spmv_launch(*args)
        torch.cuda.synchronize()
        step = (time.perf_counter() - t0) / a.steps
        ks.sort()
        return ks[len(ks) // 2] * 1e3, step * 1e6, out[0]

    prep = {}

    def degree_order():
        if "order" not in prep:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            cnt = torch.bincount(cols.long(), minlength=n_cols)
            order = torch.argsort(cnt, descending=True, stable=True)          # new id -> old id
            rank = torch.empty_like(order)
            rank[order] = torch.arange(n_cols, device="cuda")
            torch.cuda.synchronize()
            prep["order"], prep["rank"], prep["cnt_ms"] = order, rank, (time.perf_counter() - t0) * 1e3
        return prep["order"], prep["rank"], prep["cnt_ms"]

    def variant(name):
        """(vals, x, cols, per_call, prep_ms, exact) of a variant, or None."""
        if name == "csr":
            return vals, x, cols, None, 0.0, True
        if name in ("degree_numbering", "degree_numbering_resorted"):
            order, rank, ms = degree_order()
            t0 = time.perf_counter()
            c1 = rank[cols.long()].to(torch.int32).contiguous()
            v1 = vals
            if name.endswith("resorted"):
                rows = torch.repeat_interleave(torch.arange(n_rows, device="cuda"), (ptr[1:] - ptr[:-1]).long())
                edge_order = torch.argsort(rows * n_cols + c1.long())
                c1, v1 = c1[edge_order].contiguous(), vals[edge_order].contiguous()
            perm = order.to(torch.int32).contiguous()
            x1 = torch.empty_like(x)
            torch.cuda.synchronize()
            ms += (time.perf_counter() - t0) * 1e3
            formats.gather_rows(x, perm, out=x1)
            return v1, x1, c1, (lambda: formats.gather_rows(x, perm, out=x1)), ms, True
        if name.startswith("hot_first_"):
            h = min(int(name.rsplit("_", 1)[1]), n_cols)
            order, _, ms = degree_order()
            t0 = time.perf_counter()
            hot = torch.zeros(n_cols, dtype=torch.bool, device="cuda")
            hot[order[:h]] = True
            new_id = torch.empty(n_cols, dtype=torch.long, device="cuda")
            new_id[order[:h]] = torch.arange(h, device="cuda")
            cold = torch.nonzero(~hot).flatten()
            new_id[cold] = h + torch.arange(n_cols - h, device="cuda")
            inverse = torch.empty(n_cols, dtype=torch.long, device="cuda")
            inverse[new_id] = torch.arange(n_cols, device="cuda")
            c1 = new_id[cols.long()].to(torch.int32).contiguous()
            perm = inverse.to(torch.int32).contiguous()
            x1 = torch.empty_like(x)
            torch.cuda.synchronize()
            ms += (time.perf_counter() - t0) * 1e3
            formats.gather_rows(x, perm, out=x1)
            return vals, x1, c1, (lambda: formats.gather_rows(x, perm, out=x1)), ms, True
        if name.startswith("fold_"):
            m = int(name.rsplit("_", 1)[1])
            return vals, x, (cols % m).contiguous(), None, 0.0, False
        if name.startswith("hot_free_"):
            h = min(int(name.rsplit("_", 1)[1]), n_cols)
            order, _, ms = degree_order()
            hot = torch.zeros(n_cols, dtype=torch.bool, device="cuda")
            hot[order[:h]] = True
            return vals, x, torch.where(hot[cols.long()], torch.zeros_like(cols), cols).contiguous(), None, ms, False
        return None

    names = ["csr", "degree_numbering", "degree_numbering_resorted", "hot_first_65536", "hot_first_262144",
             "hot_first_1048576", "fold_524288", "fold_262144", "fold_65536", "fold_8192", "hot_free_8192",
             "hot_free_30720", "hot_free_65536", "fold_1"]
    if a.only:
        names = ["csr", a.only] if a.only != "csr" else ["csr"]
    reference = None
    for name in names:
        made = variant(name)
        if made is None:
            print(f"layout_study: unknown variant {name!r}", file=sys.stderr)
            return 2
        v, xx, c, per_call, prep_ms, exact = made
        if a.only and name == "csr" and a.only != "csr":      # the reference result only: no timing series under a profiler
            reference = ext.merged_spmv_launch(v, xx, c, ptr, n_rows, n_cols)[0].clone()
            continue
        kernel_us, step_us, y = timed(v, xx, c, per_call)
        if name == "csr":
            reference = y.clone()
        line = {"workload": w.name, "variant": name, "kernel_us": round(kernel_us, 1), "step_us": round(step_us, 1),
                "step_includes_x_permutation": per_call is not None, "prep_ms": round(prep_ms, 2),
                "max_rel_diff_vs_csr": (float(((y - reference).abs() / reference.abs().clamp_min(1e-30)).max())
                                        if exact else None),
                "share_of_edges_in_top_columns": None}
        if name == "csr":
            order, _, _ = degree_order()
            cnt = torch.bincount(cols.long(), minlength=n_cols)[order]
            share = torch.cumsum(cnt, 0).double() / ne
            line["share_of_edges_in_top_columns"] = {str(h): round(float(share[min(h, n_cols) - 1]), 4)
                                                     for h in (1024, 8192, 30720, 65536, 262144, 1048576)}
        print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
