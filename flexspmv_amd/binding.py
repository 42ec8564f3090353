"""Load a generated gfx950 library and expose the reference's ``merged_spmv_launch`` on it.

The reference's binding is a generated pybind/torch CUDA translation unit
(cuda_template/merged_binding_template.cu:10-80).  Here the generated library has a C interface
(``include/flexspmv.h``) and this module is the thin host side above it: it performs the
reference's argument checks (device, contiguity, dtype, ``ne > 0``; raised as ``RuntimeError`` like
``TORCH_CHECK``), allocates outputs and scratch with torch's caching allocator, and launches on
torch's current stream.  Differences from the reference, on purpose:

* outputs are ``torch.empty`` - the kernels write every element exactly once, so the reference's
  ``torch::zeros`` fill (codegen/merged_gen_binding.py:100-104) is unnecessary traffic;
* scratch is a cached tensor per (library, device, stream) instead of ``cudaMalloc`` / ``cudaFree``
  per call (cuda_template/merged_binding_template.cu:42-49): launches of one library on different
  streams never share tile table, carries or partials, launches on one stream are ordered by it;
* an unsupported dtype raises (the reference's CUDA binding only logs and falls off the function,
  :65-68; its CPU binding raises, cpu_template/merged_binding_template_cpu.cpp:45-46).

torch is used for device memory and streams only; there is no CPU or eager fallback: without a
built library, or without a GPU, calls fail.
"""
from __future__ import annotations

import ctypes
import json
import os
import threading
import weakref
from typing import Any, Dict, List, Optional, Sequence, Tuple

from . import build as _build
from .ir import FusedGraphIR

ABI_VERSION = 5
FLAG_TIME_KERNEL = 1
FLAG_REUSE_TILES = 2
FLAG_KEEP_TILES = 4
FLAG_DEBUG_SYNC = 8
FLAG_SEARCH_TILES = 16
DTYPE_CODES = {"float32": 0, "float64": 1, "int64": 2}
EXPORTED_SYMBOLS = ("flexspmv_launch", "flexspmv_workspace_bytes", "flexspmv_signature",
                    "flexspmv_last_error", "flexspmv_abi_version", "flexspmv_last_kernel_ms", "flexspmv_tiling",
                    "flexspmv_launch_static")


class LaunchArgs(ctypes.Structure):
    """``flexspmv_launch_args`` of include/flexspmv.h."""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("dtype", ctypes.c_int32),
        ("value_inputs", ctypes.POINTER(ctypes.c_void_p)),
        ("num_value_inputs", ctypes.c_int32),
        ("index_inputs", ctypes.POINTER(ctypes.c_void_p)),
        ("num_index_inputs", ctypes.c_int32),
        ("outputs", ctypes.POINTER(ctypes.c_void_p)),
        ("num_outputs", ctypes.c_int32),
        ("row_end_offsets", ctypes.c_void_p),
        ("num_rows", ctypes.c_int64),
        ("num_cols", ctypes.c_int64),
        ("ne", ctypes.c_int64),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
        ("flags", ctypes.c_uint32),
    ]


def load_library(path: str) -> ctypes.CDLL:
    """dlopen a generated library and type its entry points."""
    if not os.path.exists(path):
        raise RuntimeError(f"FlexSpmv library {path} is not built (run __graft_entry__.build())")
    try:
        # torch ships its own HIP runtime; it has to be the one already in the process when a generated
        # library (linked against libamdhip64 by soname) is opened, or the two runtimes disagree about
        # the device
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_LOCAL)
    lib.flexspmv_launch.argtypes = [ctypes.POINTER(LaunchArgs)]
    lib.flexspmv_launch.restype = ctypes.c_int
    lib.flexspmv_launch_static.argtypes = [ctypes.POINTER(LaunchArgs)]
    lib.flexspmv_launch_static.restype = ctypes.c_int
    lib.flexspmv_workspace_bytes.argtypes = [ctypes.c_int32, ctypes.c_int64, ctypes.c_int64]
    lib.flexspmv_workspace_bytes.restype = ctypes.c_size_t
    lib.flexspmv_signature.argtypes = []
    lib.flexspmv_signature.restype = ctypes.c_char_p
    lib.flexspmv_last_error.argtypes = []
    lib.flexspmv_last_error.restype = ctypes.c_char_p
    lib.flexspmv_last_kernel_ms.argtypes = [ctypes.POINTER(ctypes.c_float)]
    lib.flexspmv_last_kernel_ms.restype = ctypes.c_int
    lib.flexspmv_abi_version.argtypes = []
    lib.flexspmv_abi_version.restype = ctypes.c_int
    lib.flexspmv_tiling.argtypes = [ctypes.c_int32, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int32)]
    lib.flexspmv_tiling.restype = ctypes.c_int
    if lib.flexspmv_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{path}: built for interface version {lib.flexspmv_abi_version()}, "
                           f"this package speaks {ABI_VERSION}")
    return lib


def variant_of(signature: Dict[str, Any]) -> str:
    """What makes a library a measurement variant - its tuning switches and tile-shape override as text -
    or "" for a product library."""
    parts = list(signature.get("tuning", []))
    parts += [f"{k}={v}" for k, v in sorted(signature.get("policy_override", {}).items())]
    return " ".join(parts)


class _CallState:
    """ctypes objects of one thread's launches of one library (kept alive together)."""
    __slots__ = ("v_arr", "i_arr", "o_arr", "la", "ref", "repeat")


class _Repeat:
    """What a launch derived from its arguments, kept (per thread) for the next call with the very same
    argument objects: a time stepper calls with the same tensors every step, and checking them again costs
    as much Python time as the launch itself."""
    __slots__ = ("args", "tensors", "state", "value_pos", "index_pos", "ro_pos", "num_rows", "num_cols", "ne", "dt",
                 "device", "index", "ws_bytes", "out_shapes", "dtype")


_DTYPE_NAMES: Dict[Any, str] = {}


def _TORCH_DTYPE_NAMES() -> Dict[Any, str]:
    if not _DTYPE_NAMES:
        import torch
        _DTYPE_NAMES.update({torch.float32: "float32", torch.float64: "float64", torch.int64: "int64"})
    return _DTYPE_NAMES


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


class HipExtension:
    """What ``torch.utils.cpp_extension.load`` returns in the reference: an object with
    ``merged_spmv_launch(values..., gathers..., index tensors..., row_end_offsets, num_rows, num_cols)``.
    """

    def __init__(self, lib_path: str, allow_variant: bool = False) -> None:
        self.lib_path = lib_path
        self._lib = load_library(lib_path)
        self.signature: Dict[str, Any] = json.loads(self._lib.flexspmv_signature().decode())
        # A library built with tuning switches or another tile shape is a measurement variant (some switches
        # give wrong results on purpose): only a caller that asks for one gets one.
        self.variant = variant_of(self.signature)
        if self.variant and not allow_variant:
            raise RuntimeError(f"{lib_path} is a measurement variant ({self.variant}), not a product library; "
                               f"pass allow_variant=True to load it for a measurement")
        self._value_names: List[str] = list(self.signature["value_inputs"])
        self._index_names: List[str] = list(self.signature["index_inputs"])
        self._row_aligned = set(self.signature.get("row_aligned_index_inputs", []))
        self._row_indexed = set(self.signature.get("row_indexed_value_inputs", []))
        # debugging aid: compare every row-aligned index array with the row ids of row_end_offsets on each
        # launch (a library that serves such a selector from the merge path never reads the array, so a
        # caller who passes another index gets the rows' own items without an error otherwise)
        self.verify_row_aligned = False
        self._outputs = self.signature["outputs"]
        self._has_reducer = bool(self.signature["has_reducer"])
        self._streamed = set(self.signature["non_gather_value_inputs"])
        self._dtypes = set(self.signature["dtypes"])
        self._param_names = [p["name"] for p in self.signature["params"]]
        self._workspace: Dict[Any, Any] = {}   # (device index, stream handle, row pointer address) -> scratch tensor
        self._last_used: Dict[Any, int] = {}   # ... -> number of the last launch that used it
        self._launch_count = 0
        self._captured = set()                 # keys whose buffer a stream capture has recorded
        self._retained: List[Any] = []         # replaced buffers that a captured graph still refers to
        self.time_kernel = False   # set True to bracket the dominant kernel of each launch with events
        # Every launch tries the tile table the launch before left in its scratch and confirms it, block by
        # block, against the row pointer it was given (the library's default).  reuse_tiles = True skips that
        # check too on launches whose row_end_offsets tensor is the same, unmodified one as in the launch before
        # (the reference's wrapper keeps it as an immutable buffer, dynamic_replace_submodule.py:118-137).
        self.reuse_tiles = False
        self._tile_key = None
        self.extra_flags = 0       # FLAG_* bits added to every launch (FLAG_DEBUG_SYNC: print every kernel's
                                   # grid / block / LDS on stderr and synchronize after it)
        # what a launch looks up, prepared once
        self._dispatch_name = self.signature["dispatch_tensor"]
        self._tensor_names = self._value_names + self._index_names + ["row_end_offsets"]
        self._dims = dict(self.signature["value_dims"])
        self._out_specs = [(o["kind"], int(o["dim"])) for o in self._outputs]
        self._ws_bytes: Dict[Any, int] = {}
        self._tls = threading.local()

    # -- helpers -------------------------------------------------------------------------
    def param_names(self) -> List[str]:
        return list(self._param_names)

    def _bind(self, args: Sequence[Any], kwargs: Dict[str, Any]) -> Dict[str, Any]:
        names = self._param_names
        _check(len(args) <= len(names), f"merged_spmv_launch() takes {len(names)} arguments "
                                         f"({', '.join(names)}), {len(args)} given")
        bound = dict(zip(names, args))
        for k, v in kwargs.items():
            _check(k in names and k not in bound, f"merged_spmv_launch(): unexpected argument {k!r}")
            bound[k] = v
        missing = [n for n in names if n not in bound]
        _check(not missing, f"merged_spmv_launch(): missing arguments {missing}")
        return bound

    def workspace_bytes(self, dtype: str, num_rows: int, ne: int) -> int:
        return int(self._lib.flexspmv_workspace_bytes(DTYPE_CODES[dtype], num_rows, ne))

    # scratch buffers kept at most, before those of streams that have not launched for a while are dropped
    MAX_IDLE_SCRATCH = 8
    IDLE_LAUNCHES = 64

    def _scratch(self, device, index: int, raw_stream: int, nbytes: int, row_ptr: int = 0):
        """Scratch of this library for launches on the stream with handle ``raw_stream`` of device ``index``
        (the current stream of the current device when this is called) with the row pointer at address
        ``row_ptr``: a launch finds the tile table of the launch before in its scratch, so a caller that
        alternates between matrices keeps one scratch - one table - per matrix.

        The buffer is allocated on that stream and only ever used on it, so when a larger launch replaces
        it - or when it is dropped - the caching allocator hands the old block out again in stream order:
        nothing still running can see it change.  A buffer that a stream capture has recorded is kept for
        the life of the library (a replayed graph keeps using its address), and growing during a capture
        is refused: run the step once eagerly first, as capture_step does.  A caller that cycles through
        many streams does not grow the table without bound: beyond MAX_IDLE_SCRATCH entries, buffers of
        streams that have not launched for IDLE_LAUNCHES launches are dropped (never a captured one)."""
        import torch
        key = (index, raw_stream, row_ptr)
        self._launch_count += 1
        buf = self._workspace.get(key)
        capturing = torch._C._cuda_isCurrentStreamCapturing()
        if buf is None or buf.numel() < nbytes:
            _check(not capturing, "FlexSpmv scratch cannot grow during a stream capture: "
                                  "launch once with these sizes before capturing")
            if buf is not None and key in self._captured:
                self._retained.append(buf)
                self._captured.discard(key)
            buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
            self._workspace[key] = buf
            if len(self._workspace) > self.MAX_IDLE_SCRATCH:
                self._drop_idle_scratch(key)
        self._last_used[key] = self._launch_count
        if capturing:
            self._captured.add(key)
        return buf

    def _drop_idle_scratch(self, keep) -> None:
        for k in list(self._workspace):
            if k != keep and k not in self._captured and \
                    self._launch_count - self._last_used.get(k, 0) >= self.IDLE_LAUNCHES:
                # a tile table remembered in the dropped buffer is gone with it (the block may come back at
                # the same address with other contents)
                if self._tile_key is not None and self._tile_key[5] == self._workspace[k].data_ptr():
                    self._tile_key = None
                del self._workspace[k]
                self._last_used.pop(k, None)

    def workspace_of(self, device, stream=None, row_end_offsets=None):
        """The scratch tensor of launches on ``stream`` (default: the current stream) of ``device`` with the
        given row pointer (default: whichever launched last on that stream), or None before the first such
        launch.  For debugging (the tile table sits at its start)."""
        import torch
        device = torch.device(device)
        stream = stream if stream is not None else torch.cuda.current_stream(device)
        index = device.index if device.index is not None else torch.cuda.current_device()
        if row_end_offsets is not None:
            return self._workspace.get((index, int(stream.cuda_stream), row_end_offsets.data_ptr()))
        mine = [k for k in self._workspace if k[0] == index and k[1] == int(stream.cuda_stream)]
        return self._workspace[max(mine, key=lambda k: self._last_used.get(k, 0))] if mine else None

    # -- the call ------------------------------------------------------------------------
    def _call_state(self):
        """Per-thread argument block of the C call, built once: the launch struct with its constant fields
        and the three pointer arrays (a launch only rewrites pointers and sizes)."""
        st = getattr(self._tls, "state", None)
        if st is None:
            nv, ni, no = len(self._value_names), len(self._index_names), len(self._outputs)
            st = _CallState()
            st.v_arr = (ctypes.c_void_p * max(nv, 1))()
            st.i_arr = (ctypes.c_void_p * max(ni, 1))()
            st.o_arr = (ctypes.c_void_p * max(no, 1))()
            la = LaunchArgs()
            la.struct_size = ctypes.sizeof(LaunchArgs)
            la.value_inputs = ctypes.cast(st.v_arr, ctypes.POINTER(ctypes.c_void_p))
            la.num_value_inputs = nv
            la.index_inputs = ctypes.cast(st.i_arr, ctypes.POINTER(ctypes.c_void_p))
            la.num_index_inputs = ni
            la.outputs = ctypes.cast(st.o_arr, ctypes.POINTER(ctypes.c_void_p))
            la.num_outputs = no
            st.la = la
            st.ref = ctypes.byref(la)
            st.repeat = None
            self._tls.state = st
        return st

    def _same_arguments(self, args):
        """The record of the previous call on this thread if ``args`` are the same objects in the same state
        (same tensors - weak references, so nothing is kept alive -, same storage, size, dtype, device and
        layout; equal sizes), else None."""
        st = getattr(self._tls, "state", None)
        rep = st.repeat if st is not None else None
        if rep is None or len(args) != len(rep.args):
            return None
        for a, known in zip(args, rep.args):
            if known.__class__ is weakref.ref:
                if known() is not a:
                    return None
            elif a.__class__ is not known.__class__ or a != known:
                return None
        for t, (ptr, count, dtype, device) in zip(rep.tensors, rep.state):
            t = t()
            if (t.data_ptr() != ptr or t.numel() != count or t.dtype != dtype or t.device != device
                    or not t.is_contiguous()):
                return None
        return rep

    def merged_spmv_launch(self, *args, **kwargs):
        import torch
        if not kwargs and not self.verify_row_aligned:
            rep = self._same_arguments(args)
            if rep is not None:
                dtype, device = rep.dtype, rep.device
                outs = [torch.empty(shape, dtype=dtype, device=device) for shape in rep.out_shapes]
                index = rep.index
                values = [args[i] for i in rep.value_pos]
                indices = [args[i] for i in rep.index_pos]
                ro = args[rep.ro_pos]
                if index != torch._C._cuda_getDevice():
                    with torch.cuda.device(device):
                        return self._launch(values, indices, outs, ro, rep.num_rows, rep.num_cols, rep.ne, rep.dt,
                                            device, index, rep.ws_bytes)
                return self._launch(values, indices, outs, ro, rep.num_rows, rep.num_cols, rep.ne, rep.dt, device,
                                    index, rep.ws_bytes)
        b = self._bind(args, kwargs)
        value_names, index_names = self._value_names, self._index_names
        values = [b[n] for n in value_names]
        indices = [b[n] for n in index_names]
        ro = b["row_end_offsets"]
        num_rows, num_cols = int(b["num_rows"]), int(b["num_cols"])

        dispatch = b[self._dispatch_name]
        _check(dispatch.is_cuda, "CUDA device required")
        for n in self._tensor_names:
            t = b[n]
            if not t.is_cuda:
                raise RuntimeError(f"{n} must be a CUDA tensor")
            if not t.is_contiguous():
                raise RuntimeError(f"{n} must be contiguous")
        dtype = dispatch.dtype
        dt = _TORCH_DTYPE_NAMES().get(dtype)
        _check(dt is not None and dt in self._dtypes and (dt != "int64" or self.signature["allow_int64"]),
               "Unsupported dtype for ValueT. Use float32 or float64.")
        for n, t in zip(value_names, values):
            if t.dtype != dtype:
                raise RuntimeError(f"{n} dtype mismatch")
        int32 = torch.int32
        for n, t in zip(index_names, indices):
            if t.dtype != int32:
                raise RuntimeError(f"{n} dtype mismatch")
        _check(ro.dtype == int32, "row_end_offsets dtype mismatch")

        ne = int(indices[0].numel()) if indices else num_cols
        _check(ne > 0, "selector index must be non-empty")
        for n, t in zip(index_names, indices):
            if t.numel() != ne:
                raise RuntimeError(f"{n} must have ne = {ne} entries")
        dims = self._dims
        for n, t in zip(value_names, values):
            d = dims[n]
            count = t.numel()
            if count % d != 0:
                raise RuntimeError(f"{n}.numel() must be a multiple of its item width {d}")
            # the kernels index a streamed tensor by edge id: a shorter one would be read out of bounds
            if n in self._streamed and count < ne * d:
                raise RuntimeError(f"{n} must hold one item of width {d} per edge ({ne})")
            # a source gathered through a row-aligned selector is read at every row id of a tile, empty
            # rows included: a tensor shorter than num_rows would be read out of bounds
            if n in self._row_indexed and count < num_rows * d and num_rows + ne < 2 ** 31:
                raise RuntimeError(f"{n} must hold one item of width {d} per row ({num_rows}): it is gathered "
                                   f"through a selector declared equal to the reducer's row ids")
        if self._has_reducer:
            _check(ro.numel() == num_rows + 1, "row_end_offsets must have length num_rows + 1")
            if self.verify_row_aligned and self._row_aligned:
                row_ids = torch.repeat_interleave(torch.arange(num_rows, device=ro.device, dtype=torch.int32),
                                                  (ro[1:] - ro[:-1]).to(torch.int64))
                for n, t in zip(index_names, indices):
                    if n in self._row_aligned:
                        _check(bool(torch.equal(t, row_ids)), f"{n} was declared equal to the reducer's row ids "
                                                              f"(row_aligned) but differs from them")

        device = dispatch.device
        outs = []
        for kind, dim in self._out_specs:
            if kind == "sum":
                shape = (dim,)
            else:
                lead = num_rows if kind == "reducer" else ne
                shape = (lead,) if dim == 1 else (lead, dim)
            outs.append(torch.empty(shape, dtype=dtype, device=device))

        size_key = (dt, num_rows, ne)
        ws_bytes = self._ws_bytes.get(size_key)
        if ws_bytes is None:
            ws_bytes = self._ws_bytes[size_key] = self.workspace_bytes(dt, num_rows, ne)
        index = device.index
        if not kwargs and len(args) == len(self._param_names):
            self._remember(args, outs, num_rows, num_cols, ne, dt, dtype, device, ws_bytes)
        other_device = index is not None and index != torch._C._cuda_getDevice()
        if other_device:
            with torch.cuda.device(device):
                return self._launch(values, indices, outs, ro, num_rows, num_cols, ne, dt, device, index, ws_bytes)
        return self._launch(values, indices, outs, ro, num_rows, num_cols, ne, dt, device,
                            index if index is not None else torch._C._cuda_getDevice(), ws_bytes)

    def _remember(self, args, outs, num_rows, num_cols, ne, dt, dtype, device, ws_bytes):
        import torch
        rep = _Repeat()
        tensors = [a for a in args if isinstance(a, torch.Tensor)]
        try:
            rep.args = tuple(weakref.ref(a) if isinstance(a, torch.Tensor) else a for a in args)
            rep.tensors = tuple(weakref.ref(t) for t in tensors)
        except TypeError:      # an argument type that cannot be weakly referenced: no shortcut
            return
        rep.state = tuple((t.data_ptr(), t.numel(), t.dtype, t.device) for t in tensors)
        where = {n: i for i, n in enumerate(self._param_names)}
        rep.value_pos = tuple(where[n] for n in self._value_names)
        rep.index_pos = tuple(where[n] for n in self._index_names)
        rep.ro_pos = where["row_end_offsets"]
        rep.num_rows, rep.num_cols, rep.ne, rep.dt, rep.dtype, rep.device = num_rows, num_cols, ne, dt, dtype, device
        rep.index = device.index if device.index is not None else torch._C._cuda_getDevice()
        rep.ws_bytes = ws_bytes
        rep.out_shapes = tuple(tuple(o.shape) for o in outs)
        self._call_state().repeat = rep

    def _launch(self, values, indices, outs, ro, num_rows, num_cols, ne, dt, device, index, ws_bytes):
        """Fill the argument block and call the library on the current stream of the (current) device."""
        import torch
        raw_stream = torch._C._cuda_getCurrentRawStream(index)
        ws = self._scratch(device, index, raw_stream, ws_bytes, ro.data_ptr() if self._has_reducer else 0)
        st = self._call_state()
        la = st.la
        for i, t in enumerate(values):
            st.v_arr[i] = t.data_ptr()
        for i, t in enumerate(indices):
            st.i_arr[i] = t.data_ptr()
        for i, t in enumerate(outs):
            st.o_arr[i] = t.data_ptr()
        la.dtype = DTYPE_CODES[dt]
        la.row_end_offsets = ro.data_ptr()
        la.num_rows, la.num_cols, la.ne = num_rows, num_cols, ne
        la.workspace, la.workspace_bytes = ws.data_ptr(), ws.numel()
        flags = (FLAG_TIME_KERNEL if self.time_kernel else 0) | int(self.extra_flags)
        if self.reuse_tiles and self._has_reducer:
            key = (ro.data_ptr(), ro._version, num_rows, ne, dt, ws.data_ptr(), index)
            if key == self._tile_key:
                flags |= FLAG_REUSE_TILES
            self._tile_key = key
        la.flags = flags
        la.stream = raw_stream
        rc = self._lib.flexspmv_launch(st.ref)
        if rc != 0:
            raise RuntimeError(f"merged_spmv_launch failed ({rc}): {self._lib.flexspmv_last_error().decode()}")
        if not outs:
            return None
        return tuple(outs)

    __call__ = merged_spmv_launch

    def last_kernel_ms(self) -> float:
        """Duration of the dominant kernel of the last launch made with ``time_kernel = True``."""
        ms = ctypes.c_float(0.0)
        rc = self._lib.flexspmv_last_kernel_ms(ctypes.byref(ms))
        if rc != 0:
            raise RuntimeError(f"flexspmv_last_kernel_ms failed ({rc}): {self._lib.flexspmv_last_error().decode()}")
        return float(ms.value)


def load_extension(ir: FusedGraphIR, build_if_missing: bool = True) -> HipExtension:
    """The library of a sub-graph: the prebuilt one when current, else built now with hipcc."""
    if _build.is_current(ir):
        return HipExtension(_build.library_path(ir))
    if not build_if_missing:
        raise RuntimeError(f"FlexSpmv library for sub-graph {ir.name!r} is not built")
    return HipExtension(_build.compile_graph(ir))


def load_named(name: str, build_if_missing: bool = True) -> HipExtension:
    from . import graphs
    return load_extension(graphs.get(name), build_if_missing=build_if_missing)
