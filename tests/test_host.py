"""Host-side logic and the C interface of the generated libraries (no GPU needed)."""
import ctypes
import json
import os
import re

import numpy as np

import pytest

from flexspmv_amd import build, graphs
from flexspmv_amd.binding import ABI_VERSION, EXPORTED_SYMBOLS, LaunchArgs, load_library
from flexspmv_amd.codegen.merged_gen_binding import binding_plan, generate_binding_code
from flexspmv_amd.codegen.merged_gen_gpu import analyse, generate_hip_source
from flexspmv_amd.ir import GraphBuilder, get_dim_length

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _lib(name):
    ir = graphs.get(name)
    path = build.library_path(ir)
    if not build.is_current(ir):
        path = build.compile_graph(ir)     # hipcc cross-compiles without a GPU
    return load_library(path)


# ---------------------------------------------------------------------------------------------
# binding contract: argument order equals the generated bindings the reference keeps in its tree
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["system_two_selectors", "bpoints_copy"])
def test_binding_order_matches_reference_generated_binding(name, golden_dir):
    with open(os.path.join(golden_dir, "binding_fixtures.json")) as f:
        gold = json.load(f)[name]
    ir = graphs.get(name)
    sig = generate_binding_code(None, ir.inputs, ir.outputs, ir.selector_register)
    assert [p["name"] for p in sig["params"]] == gold["params"]
    assert [{k: o[k] for k in ("name", "kind", "dim")} for o in sig["outputs"]] == gold["outputs"]
    assert sig["dispatch_tensor"] == gold["dispatch_tensor"]
    assert sig["allow_int64"] == gold["allow_int64"]


def test_binding_groups():
    plan = binding_plan(*graphs.get("spring_mass").six()[:3])
    assert plan.non_gather_value_inputs == ["k", "rest"]
    assert plan.gather_value_inputs == ["pos"]
    assert plan.selector_inputs == ["gather_src", "gather_dst"]
    assert [(o.name, o.kind, o.dim) for o in plan.outputs] == [("scatter", "reducer", 3), ("sum_1", "sum", 1)]
    # a selector module used twice contributes one index tensor
    b = GraphBuilder("twice")
    b.placeholder("v", (2,)); b.placeholder("w", (1,))
    b.select("s_a", "v", module="sel"); b.select("s_b", "v", module="sel")
    b.map("add", "add", ["s_a", "s_b"]); b.reduce("red", "add"); b.output("red")
    assert binding_plan(*b.build().six()[:3]).selector_inputs == ["sel"]


def test_shape_rule_and_unknown_op():
    assert get_dim_length((2, 3)) == 6 and get_dim_length((1,)) == 1
    b = GraphBuilder("bad")
    b.placeholder("v", (1,))
    with pytest.raises(ValueError, match="not supported"):
        b.map("cosh", "c", ["v"])


# ---------------------------------------------------------------------------------------------
# generator: stage split, widths, policy
# ---------------------------------------------------------------------------------------------
def test_memory_levels_of_a_graph():
    kp = analyse(graphs.get("spmv_dot"))
    assert [v[0] for v in kp.fetch_values] == ["vals"] and kp.fetch_indices == [("selector_col", 0)]
    assert [g[0] for g in kp.gathers] == ["selector_col"] and [r[0] for r in kp.row_sources] == ["selector_row"]
    assert (kp.fetch_value_width, kp.fetch_index_width, kp.red_width, kp.agg_width, kp.row_width) == (1, 1, 1, 1, 1)
    src, sig = generate_hip_source(graphs.get("spmv_dot"))
    assert sig["row_aligned_index_inputs"] == ["selector_row_idx"] and sig["row_indexed_value_inputs"] == ["x"]
    assert "selector_row_idx_ptr +" not in src                                   # never dereferenced
    # the mesh maps: the destination selector comes from the row as well, the source selector is gathered
    kp = analyse(graphs.get("spring_mass"))
    assert (kp.fetch_value_width, kp.fetch_index_width, kp.red_width, kp.agg_width, kp.row_width) == (2, 1, 3, 1, 3)
    _, sig = generate_hip_source(graphs.get("spring_mass"))
    assert sig["row_aligned_index_inputs"] == ["gather_dst_idx"] and sig["row_indexed_value_inputs"] == ["pos"]
    kp = analyse(graphs.get("swe_rusanov"))
    assert (kp.fetch_value_width, kp.fetch_index_width, kp.red_width, kp.row_width) == (3, 1, 3, 3)


def test_plain_spmv_hands_over_value_and_column():
    kp = analyse(graphs.get("csr_spmv"))
    assert (kp.fetch_value_width, kp.fetch_index_width, kp.row_width, kp.agg_width) == (1, 1, 0, 0)
    src, sig = generate_hip_source(graphs.get("csr_spmv"))
    assert sig["policy"]["block"] == 256 and sig["policy"]["ipt"]["float64"] == 8
    assert "EDGE_PURE = true" in src
    src, _ = generate_hip_source(graphs.get("map_store"))
    assert "EDGE_PURE = false" in src                                            # it stores per edge


def test_policy_shrinks_tile_for_wide_graphs():
    _, sig = generate_hip_source(graphs.get("op_zoo"))
    ipt = sig["policy"]["ipt"]
    assert ipt["float64"] <= ipt["float32"] <= 8 and ipt["float64"] >= 1


def test_generated_source_is_deterministic_and_hash_keyed():
    a, _ = generate_hip_source(graphs.get("swe_rusanov"))
    b, _ = generate_hip_source(graphs.get("swe_rusanov"))
    assert a == b
    ir = graphs.get("swe_rusanov")
    assert ir.content_hash() in a and build.graph_dir(ir).endswith(ir.content_hash())


def test_no_cuda_or_compat_layers_in_kernel_sources():
    """Every kernel is this package's own: no CUB / hipCUB / rocPRIM primitive, no dual-platform switch."""
    bad = re.compile(r"cub::|hipcub|rocprim|__HIP_PLATFORM|cuda_runtime|triton", re.I)
    for fn in os.listdir(build.CSRC_DIR):
        with open(os.path.join(build.CSRC_DIR, fn)) as f:
            assert not bad.search(f.read()), fn


# ---------------------------------------------------------------------------------------------
# C interface: symbols, signature, argument validation (all before any GPU call)
# ---------------------------------------------------------------------------------------------
def test_header_symbols_are_exported_by_every_library():
    with open(os.path.join(ROOT, "include", "flexspmv.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(flexspmv_[a-z_]+)\s*\(", header))
    assert declared == set(EXPORTED_SYMBOLS)
    for name in graphs.REGISTRY:
        lib = _lib(name)
        for sym in declared:
            assert getattr(lib, sym) is not None
        assert lib.flexspmv_abi_version() == ABI_VERSION
        sig = json.loads(lib.flexspmv_signature().decode())
        assert sig["graph"] == name and sig["hash"] == graphs.get(name).content_hash()


def _args(lib, **over):
    sig = json.loads(lib.flexspmv_signature().decode())
    nv, ni, no = len(sig["value_inputs"]), len(sig["index_inputs"]), len(sig["outputs"])
    keep = []
    def arr(n):
        a = (ctypes.c_void_p * max(n, 1))(*([0x1000] * max(n, 1)))
        keep.append(a)
        return ctypes.cast(a, ctypes.POINTER(ctypes.c_void_p))
    la = LaunchArgs()
    la.struct_size = ctypes.sizeof(LaunchArgs)
    la.dtype = 0
    la.value_inputs, la.num_value_inputs = arr(nv), nv
    la.index_inputs, la.num_index_inputs = arr(ni), ni
    la.outputs, la.num_outputs = arr(no), no
    la.row_end_offsets = 0x1000
    la.num_rows, la.num_cols, la.ne = 10, 10, 30
    la.workspace, la.workspace_bytes = 0, 0
    for k, v in over.items():
        setattr(la, k, v)
    la._keep = keep
    return la


def test_launch_rejects_bad_arguments_without_touching_the_gpu():
    lib = _lib("csr_spmv")
    err = lambda: lib.flexspmv_last_error().decode()
    assert lib.flexspmv_launch(None) == -1
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, struct_size=8))) == -1 and "struct_size" in err()
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, flags=32))) == -1 and "flags" in err()
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, num_value_inputs=1))) == -1 and "counts" in err()
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, dtype=2))) == -2 and "Unsupported dtype" in err()
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, ne=0))) == -1 and "non-empty" in err()
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, num_rows=0))) == -1
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, ne=2**31 - 100))) == -3 and "2^31" in err()
    assert lib.flexspmv_launch(ctypes.byref(_args(lib))) == -4 and "workspace" in err()       # no scratch given
    assert lib.flexspmv_launch(ctypes.byref(_args(lib, workspace=0x1000, workspace_bytes=1 << 20,
                                                  row_end_offsets=0))) == -1 and "row_end_offsets" in err()


def test_tiling_query():
    """flexspmv_tiling: tile count, diagonal spacing and the row-snapping parameters of a launch."""
    lib = _lib("spmv_dot")
    out = (ctypes.c_int32 * 6)()
    # Poisson 256^3 in float64: 8 merge items per row, 16 rows per 128-byte output line -> slack 128
    assert lib.flexspmv_tiling(1, 16777216, 117047296, out) == 0
    num_tiles, nominal, slack, snap_rows, capacity, in_blocks = list(out)
    assert (nominal, slack, snap_rows, capacity, in_blocks) == (2048 - 128, 128, 16, 2048, 0)
    assert num_tiles == -(-(16777216 + 117047296) // nominal)
    # long rows: a line's worth of rows is more than an eighth of a tile -> boundaries stay on their diagonals
    assert lib.flexspmv_tiling(1, 1000, 1000 * 300, out) == 0
    assert list(out)[1:5] == [2048, 0, 1, 2048] and out[5] == 1
    assert lib.flexspmv_tiling(2, 1000, 7000, out) == -2             # int64 not compiled into this library
    assert lib.flexspmv_tiling(1, 2**30, 2**30, out) == -3
    flat = _lib("mass_sum")
    assert flat.flexspmv_tiling(0, 5, 100000, out) == 0 and list(out)[1:4] == [2048, 0, 1]


def test_tiles_of_a_launch_of_a_few_rounds_fill_its_last_round():
    """A launch of one to four rounds of blocks (256 CUs x the blocks a CU holds) gets smaller tiles, by a quarter at
    most, so that the last round is a full one; launches of less than a round or of more than four keep theirs."""
    out = (ctypes.c_int32 * 6)()
    spring = _lib("spring_mass")                      # float32: 25.7 KB of LDS per block, 6 blocks per CU -> 1536 per round
    assert spring.flexspmv_tiling(0, 1_000_000, 5_940_000, out) == 0
    num_tiles, nominal, slack, _, capacity, _ = list(out)
    assert nominal + slack < capacity                 # smaller than the largest tile that would fit ...
    assert 4 * nominal >= 3 * (capacity - slack)      # ... by a quarter at most
    assert num_tiles == -(-(6_940_000) // nominal) and 3 * 1536 - 8 <= num_tiles <= 3 * 1536
    assert spring.flexspmv_tiling(0, 10_000, 59_400, out) == 0 and out[1] == 1776     # less than a round: 256 average rows
    swe = _lib("swe_rusanov")                         # 6.5 rounds: left alone
    assert swe.flexspmv_tiling(1, 1_999_960, 5_999_842, out) == 0 and (out[0], out[1]) == (8334, 960)
    poisson = _lib("spmv_dot")                        # 45 rounds
    assert poisson.flexspmv_tiling(1, 16777216, 117047296, out) == 0 and (out[0], out[1]) == (69701, 1920)


def test_workspace_query():
    lib = _lib("spmv_dot")
    small = lib.flexspmv_workspace_bytes(1, 1000, 7000)
    big = lib.flexspmv_workspace_bytes(1, 16777216, 117047296)
    assert 0 < small < big < 64 << 20
    assert lib.flexspmv_workspace_bytes(2, 1000, 7000) == 0          # int64 not compiled into this library
    assert lib.flexspmv_workspace_bytes(1, 2**30, 2**30) == 0        # does not fit 32-bit offsets
    flat = _lib("bpoints_copy")
    assert flat.flexspmv_workspace_bytes(2, 100, 100) == 0           # map-only needs no scratch


def test_matrix_market_workload(tmp_path):
    """A MatrixMarket file becomes a CSR SpMV workload: symmetric storage expanded, duplicates summed,
    columns sorted; the oracle's product equals scipy's."""
    import scipy.io
    import scipy.sparse as sp
    from flexspmv_amd import graphs
    from flexspmv_amd import workloads as W
    from oracle.runner import run_oracle
    rng = np.random.default_rng(0)
    a = sp.random(40, 40, density=0.15, random_state=1, format="coo")
    a = sp.coo_matrix(a + a.T)                              # symmetric: written in symmetric storage
    path = str(tmp_path / "sym.mtx")
    scipy.io.mmwrite(path, a, symmetry="symmetric")
    w = W.matrix_market_spmv(path)
    assert w.graph == "csr_spmv" and w.num_rows == 40 and w.ne == sp.csr_matrix(a).nnz
    assert all(np.all(np.diff(w.tensors["selector_idx"][s:e]) > 0)
               for s, e in zip(w.row_end_offsets[:-1], w.row_end_offsets[1:]))
    (y,), _ = run_oracle(graphs.get("csr_spmv"), w.tensors, w.row_end_offsets, w.num_rows, w.num_cols, 3)
    assert np.allclose(y, sp.csr_matrix(a) @ w.tensors["x"], rtol=1e-13, atol=1e-15)
    wd = W.matrix_market_spmv(path, fused_dot=True)
    (y2, dot), _ = run_oracle(graphs.get("spmv_dot"), wd.tensors, wd.row_end_offsets, wd.num_rows, wd.num_cols, 3)
    assert np.allclose(y2, y) and np.isclose(dot[0], wd.tensors["x"] @ y, rtol=1e-12)
    with pytest.raises(ValueError):
        scipy.io.mmwrite(str(tmp_path / "rect.mtx"), sp.random(5, 7, density=0.5, random_state=2))
        W.matrix_market_spmv(str(tmp_path / "rect.mtx"), fused_dot=True)


def test_launcher_keeps_its_previous_arguments_by_weak_reference_only():
    """The record a launch leaves for the next call with the same arguments must not keep tensors alive."""
    import gc
    import weakref

    import torch

    from flexspmv_amd.binding import HipExtension

    class Probe(HipExtension):          # the bookkeeping alone, without a library
        def __init__(self):
            import threading
            self._tls = threading.local()
            self._param_names = ["vals", "x", "selector_idx", "row_end_offsets", "num_rows", "num_cols"]
            self._value_names, self._index_names, self._outputs = ["vals", "x"], ["selector_idx"], [None]

    ext = Probe()
    args = [torch.zeros(5), torch.zeros(4), torch.zeros(5, dtype=torch.int32), torch.zeros(5, dtype=torch.int32), 4, 4]
    ext._remember(tuple(args), [torch.zeros(4)], 4, 4, 5, "float32", torch.float32, torch.device("cuda", 0), 256)
    assert ext._same_arguments(tuple(args)) is not None
    assert ext._same_arguments(tuple(args[:4] + [4, 5])) is None            # another size
    assert ext._same_arguments(tuple([args[0].clone()] + args[1:])) is None  # another tensor object
    args[1].resize_(2)
    assert ext._same_arguments(tuple(args)) is None                          # the same object in another state
    args[1].resize_(4)
    assert ext._same_arguments(tuple(args)) is not None
    args[1].data = args[1].data.view(torch.int32)                            # same storage, size and layout: another dtype
    assert ext._same_arguments(tuple(args)) is None
    args[1].data = args[1].data.view(torch.float32)
    assert ext._same_arguments(tuple(args)) is not None
    probe = weakref.ref(args[0])
    del args
    gc.collect()
    assert probe() is None


def test_scratch_of_idle_streams_is_dropped():
    """A caller that cycles through streams does not grow the launcher's scratch table without bound: beyond a
    few entries, buffers of streams that have not launched for a while go - never one a capture recorded -
    and a tile table remembered in a dropped buffer is forgotten with it."""
    from flexspmv_amd.binding import HipExtension

    class Probe(HipExtension):          # the bookkeeping alone, without a library or a GPU
        def __init__(self):
            self._workspace, self._last_used, self._captured, self._retained = {}, {}, set(), []
            self._launch_count = 0
            self._tile_key = None

    class Buf:
        def __init__(self, ptr):
            self.ptr = ptr
        def data_ptr(self):
            return self.ptr
        def numel(self):
            return 256

    ext = Probe()
    for i in range(ext.MAX_IDLE_SCRATCH):
        ext._workspace[(0, i)] = Buf(1000 + i)
        ext._last_used[(0, i)] = 0
    ext._captured.add((0, 3))
    ext._tile_key = (1, 0, 10, 10, "float32", 1002, 0)      # table remembered in the buffer of stream 2
    ext._launch_count = ext.IDLE_LAUNCHES - 1
    ext._last_used[(0, 5)] = ext._launch_count                # stream 5 launched just now
    ext._workspace[(0, 99)] = Buf(2000)
    ext._drop_idle_scratch(keep=(0, 99))
    assert len(ext._workspace) == ext.MAX_IDLE_SCRATCH + 1    # nothing is idle long enough yet
    ext._launch_count += 1
    ext._drop_idle_scratch(keep=(0, 99))
    assert sorted(ext._workspace) == [(0, 3), (0, 5), (0, 99)]
    assert ext._tile_key is None


# ---------------------------------------------------------------------------------------------
# tuning switches: a library built with them is a measurement variant and says so
# ---------------------------------------------------------------------------------------------
def test_every_tuning_switch_of_the_sources_is_listed_in_the_fence():
    with open(os.path.join(build.CSRC_DIR, "flex_tuning.hpp")) as f:
        listed = set(re.findall(r"defined\((FLEX_TUNE_[A-Z0-9_]+)\)", f.read()))
    used = set()
    for fn in os.listdir(build.CSRC_DIR):
        if fn != "flex_tuning.hpp":
            with open(os.path.join(build.CSRC_DIR, fn)) as f:
                used |= set(re.findall(r"\bFLEX_TUNE_[A-Z0-9_]+", f.read()))
    assert used and used <= listed, sorted(used - listed)


def test_tuning_switches_are_recorded_and_variants_are_refused(tmp_path):
    from flexspmv_amd.binding import HipExtension, variant_of
    ir = graphs.get("csr_spmv")
    _, sig = generate_hip_source(ir)
    assert sig["tuning"] == [] and sig["policy_override"] == {} and variant_of(sig) == ""
    src, sig = generate_hip_source(ir, policy={"block": 128, "ipt_f32": 4}, defines=["FLEX_TUNE_NT_LOADS", "FLEX_TUNE_NOMINAL=1024"])
    assert sig["tuning"] == ["FLEX_TUNE_NOMINAL=1024", "FLEX_TUNE_NT_LOADS"]
    assert variant_of(sig) == "FLEX_TUNE_NOMINAL=1024 FLEX_TUNE_NT_LOADS block=128 ipt_f32=4"
    assert "#define FLEX_TUNING_DECLARED 1" in src
    with pytest.raises(ValueError, match="not a tuning switch"):
        generate_hip_source(ir, defines=["NDEBUG"])
    # built through the package: switches reach the generator and the compiler alike, the signature names them,
    # and only a caller that asks for a variant gets one
    lib = build.compile_graph(ir, out_dir=str(tmp_path / "variant"), extra_flags=["-DFLEX_TUNE_NT_LOADS"])
    assert json.loads(load_library(lib).flexspmv_signature().decode())["tuning"] == ["FLEX_TUNE_NT_LOADS"]
    with pytest.raises(RuntimeError, match="measurement variant"):
        HipExtension(lib)
    assert HipExtension(lib, allow_variant=True).variant == "FLEX_TUNE_NT_LOADS"
    for name in graphs.REGISTRY:                      # every shipped library is a product library
        assert variant_of(json.loads(_lib(name).flexspmv_signature().decode())) == ""


@pytest.mark.parametrize("flags, message", [
    (["-DFLEX_TUNE_NT_LOADS"], "must be the ones the generator was given"),              # not declared to the generator
    (["-DFLEX_TUNE_FORCE_MERGE"], "FLEX_TUNE_ALLOW_WRONG_RESULTS"),                      # wrong results need a second switch
    (["-DFLEX_TUNE_ABLATE_STORES"], "FLEX_TUNE_ALLOW_WRONG_RESULTS"),
    (["-DFLEX_TUNE_UNSAFE_BIG_TILE"], "FLEX_TUNE_ALLOW_WRONG_RESULTS"),
])
def test_undeclared_or_unsafe_switches_do_not_compile(tmp_path, flags, message):
    import subprocess
    ir = graphs.get("csr_spmv")
    src, _ = build.write_generated_source(ir, out_dir=str(tmp_path))        # generated without switches
    cmd = [build.hipcc_path(), *build.HIPCC_FLAGS, *flags, f"-I{build.CSRC_DIR}", f"-I{build.INCLUDE_DIR}",
           "--cuda-host-only", "-fsyntax-only", src]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode != 0 and message in proc.stdout, proc.stdout[-2000:]
