"""flexspmv_launch_static: the entry point that allocates nothing (scratch in the library's own device image).

Called through the C interface (ctypes) and compared, bit for bit, with flexspmv_launch on the same inputs: a
first call on a larger input, then a second call on a smaller one - the shared scratch still holds the first
call's tile table, carries and partials, and nothing of it may leak into the second result.
"""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from flexspmv_amd import graphs
from flexspmv_amd.binding import DTYPE_CODES, FLAG_TIME_KERNEL, LaunchArgs, load_named
from tests.test_gpu_parity import case_rng
from tests.util_inputs import make_inputs, row_structure

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 4 << 20          # FLEXSPMV_STATIC_SCRATCH_BYTES of include/flexspmv.h


def device_inputs(ext, name, dtype, structure, rng):
    row_ptr = row_structure(structure, rng)
    tensors, row_ptr, nr, nc, ne = make_inputs(graphs.get(name), dtype, rng, row_ptr=row_ptr)
    given = {k: torch.from_numpy(np.ascontiguousarray(v)).cuda() for k, v in tensors.items()}
    given.update(row_end_offsets=torch.from_numpy(row_ptr).cuda(), num_rows=nr, num_cols=nc)
    return given, nr, nc, ne


def launch_static(ext, given, nr, nc, ne, dtype, outs, flags=0):
    """flexspmv_launch_static through ctypes; `outs` are preallocated output tensors in binding order."""
    sig = ext.signature
    values = [given[n] for n in sig["value_inputs"]]
    indices = [given[n] for n in sig["index_inputs"]]

    def ptr_array(tensors):
        arr = (ctypes.c_void_p * max(len(tensors), 1))()
        for i, t in enumerate(tensors):
            arr[i] = t.data_ptr()
        return arr

    v_arr, i_arr, o_arr = ptr_array(values), ptr_array(indices), ptr_array(outs)
    la = LaunchArgs()
    la.struct_size = ctypes.sizeof(LaunchArgs)
    la.dtype = DTYPE_CODES[dtype]
    la.value_inputs = ctypes.cast(v_arr, ctypes.POINTER(ctypes.c_void_p))
    la.num_value_inputs = len(values)
    la.index_inputs = ctypes.cast(i_arr, ctypes.POINTER(ctypes.c_void_p))
    la.num_index_inputs = len(indices)
    la.outputs = ctypes.cast(o_arr, ctypes.POINTER(ctypes.c_void_p))
    la.num_outputs = len(outs)
    la.row_end_offsets = given["row_end_offsets"].data_ptr()
    la.num_rows, la.num_cols, la.ne = nr, nc, ne
    la.workspace, la.workspace_bytes = None, 0
    la.stream = torch.cuda.current_stream().cuda_stream
    la.flags = flags
    rc = ext._lib.flexspmv_launch_static(ctypes.byref(la))
    return rc, ext._lib.flexspmv_last_error().decode()


@pytest.mark.parametrize("name,dtype", [("spmv_dot", "float64"), ("swe_rusanov", "float32"), ("csr_spmv", "float32")])
def test_static_scratch_launch_matches_the_allocating_one_twice_in_a_row(name, dtype):
    ext = load_named(name, build_if_missing=False)
    rng = case_rng("no_alloc", name)
    big = device_inputs(ext, name, np.dtype(dtype), "skewed", rng)           # merge path, carry runs over several tiles
    small = device_inputs(ext, name, np.dtype(dtype), "len33", rng)           # fewer tiles than the call before
    assert small[3] < big[3]
    # everything torch allocates (reference results, output buffers) exists before the calls under test
    cases = []
    for given, nr, nc, ne in (big, small):
        want = ext.merged_spmv_launch(*[given[k] for k in ext.param_names()])
        outs = [torch.full_like(o, float("nan")) for o in want]
        cases.append((given, nr, nc, ne, want, outs))
    # the first call on this GPU resolves the scratch address; the memory check compares two steady states
    given, nr, nc, ne, _, outs = cases[0]
    rc, msg = launch_static(ext, given, nr, nc, ne, dtype, outs)
    assert rc == 0, msg
    for o in outs:
        o.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for round_, (given, nr, nc, ne, _, outs) in enumerate(cases):
        print(f"case no_alloc {name} {dtype} call {round_} rows={nr} ne={ne}", flush=True)
        rc, msg = launch_static(ext, given, nr, nc, ne, dtype, outs)
        assert rc == 0, msg
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before          # no device memory was taken or returned
    for round_, (_, _, _, _, want, outs) in enumerate(cases):
        for o, w in zip(outs, want):
            assert torch.equal(o, w), f"{name}: static-scratch launch differs from flexspmv_launch (call {round_})"


def test_static_scratch_launch_under_stream_capture():
    """An allocation (or a free, or an event creation) under stream capture is an error, so a captured call
    that succeeds and replays to the bits of flexspmv_launch made none.  The graph is replayed several
    times with the program's own eager launches and synchronizations between the replays, and every replay
    is checked (the scratch keeps what the eager launches in between left there)."""
    name, dtype = "spmv_dot", "float64"
    ext = load_named(name, build_if_missing=False)
    rng = case_rng("no_alloc", "capture")
    given, nr, nc, ne = device_inputs(ext, name, np.dtype(dtype), "skewed", rng)
    other, onr, onc, one = device_inputs(ext, name, np.dtype(dtype), "mesh_with_gaps", rng)
    want = ext.merged_spmv_launch(*[given[k] for k in ext.param_names()])
    other_want = ext.merged_spmv_launch(*[other[k] for k in ext.param_names()])
    outs = [torch.full_like(o, float("nan")) for o in want]
    other_outs = [torch.full_like(o, float("nan")) for o in other_want]
    rc, msg = launch_static(ext, given, nr, nc, ne, dtype, outs)       # resolves the scratch address outside the capture
    assert rc == 0, msg
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            rc, msg = launch_static(ext, given, nr, nc, ne, dtype, outs)
    assert rc == 0, msg
    torch.cuda.current_stream().wait_stream(stream)
    for replay in range(4):
        for o in outs:
            o.fill_(float("nan"))
        # eager work of another shape through the same scratch between the replays
        rc, msg = launch_static(ext, other, onr, onc, one, dtype, other_outs)
        assert rc == 0, msg
        torch.cuda.synchronize()
        print(f"case no_alloc capture replay {replay}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        for o, w in zip(outs, want):
            assert torch.equal(o, w), f"replay {replay} differs from flexspmv_launch"
        for o, w in zip(other_outs, other_want):
            assert torch.equal(o, w)


def test_static_scratch_launch_refuses_what_it_cannot_hold():
    ext = load_named("spmv_dot", build_if_missing=False)
    rng = case_rng("no_alloc", "limits")
    given, nr, nc, ne = device_inputs(ext, "spmv_dot", np.dtype("float64"), "mesh", rng)
    outs = [torch.empty(nr, dtype=torch.float64, device="cuda"), torch.empty(1, dtype=torch.float64, device="cuda")]
    # sizes whose scratch exceeds the static buffer: refused before anything is launched
    huge_rows, huge_ne = 40_000_000, 280_000_000
    assert ext.workspace_bytes("float64", huge_rows, huge_ne) > STATIC_SCRATCH_BYTES
    rc, msg = launch_static(ext, given, huge_rows, nc, huge_ne, "float64", outs)
    assert rc == -4 and "static buffer holds" in msg and str(STATIC_SCRATCH_BYTES) in msg
    rc, msg = launch_static(ext, given, nr, nc, ne, "float64", outs, flags=FLAG_TIME_KERNEL)
    assert rc == -1 and "FLEXSPMV_FLAG_TIME_KERNEL" in msg
    # the largest benchmark problem fits
    assert ext.workspace_bytes("float64", 256 ** 3, 117047296) <= STATIC_SCRATCH_BYTES
    rc, msg = launch_static(ext, given, nr, nc, ne, "float64", outs)
    assert rc == 0, msg
    torch.cuda.synchronize()
