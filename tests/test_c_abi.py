"""The C interfaces from a caller without Python or torch in it: tests/c_abi/spmv_from_c.cpp opens the
csr_spmv library and the formats library with dlopen, allocates with hipMalloc, turns COO row ids into
the row pointer, launches, and checks y = A x against a host loop (float32 to 1e-5, float64 to 1e-12 of the row
scale; the row pointer exactly)."""
import os
import subprocess

import pytest

from flexspmv_amd import build, graphs
from tests.c_abi.build_c_abi import BINARY, build as build_caller


def _binary():
    return BINARY if os.path.exists(BINARY) else build_caller()


def test_caller_builds_and_explains_itself():
    exe = _binary()
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert proc.returncode == 1 and "usage:" in proc.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("grid", [3, 300, 1500])
def test_spmv_through_the_c_interfaces(grid):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    kernel_lib = build.library_path(graphs.get("csr_spmv"))
    assert os.path.exists(kernel_lib) and os.path.exists(build.FORMATS_LIBRARY)
    print(f"case grid={grid}", flush=True)
    proc = subprocess.run([_binary(), kernel_lib, build.FORMATS_LIBRARY, str(grid)], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=100)
    assert proc.returncode == 0, proc.stdout
    assert proc.stdout.strip().endswith("OK"), proc.stdout
    assert proc.stdout.count("row pointer") == 2 and proc.stdout.count("y = A x") == 2
