"""The six-list description of one fused sub-graph, and a builder for writing it by hand.

The reference derives six lists of dicts from a fused ``torch.fx`` sub-graph
(``trace/graph_trace.py:32-328``): ``inputs``, ``outputs``, ``selector_register``,
``map_operations``, ``reducer_operations`` and ``aggregator_operations``.  Every generator in
this package (HIP kernels, the launch binding, the CPU oracle used by the tests) consumes exactly
those lists, with the same keys:

* ``inputs``             ``{name, target, dtype: 'scalar_t'|'int', shape, op, args, dtype_data}``
  (``graph_trace.py:133-156``): placeholders in graph order, plus one ``'int'`` entry per Selector
  call whose ``target`` is the selector module name.
* ``outputs``            ``{op, name, target: 'reducer'|'sum'|<other>, dtype, shape, args, dtype_data}``
  (``graph_trace.py:106-116``).
* ``selector_register``  ``{name, target, dtype, selector: 0|1, selector_name, shape, dtype_data}``
  (``graph_trace.py:179-204``): ``selector == 0`` is a tensor streamed by edge id, ``selector == 1``
  a vertex tensor gathered through index array ``selector_name``.
* ``map_operations``     ``{name, target, op, shape, dtype_data, args}`` (``graph_trace.py:220-286``).
* ``reducer_operations`` / ``aggregator_operations``  ``{name, op, shape, dtype_data, args}``
  (``graph_trace.py:302-319``).

Shapes drop the leading edge/vertex dimension and scalars become ``(1,)``
(``graph_trace.py:21-28``).  Argument entries are variable names (``str``), Python numbers, or - for
``getitem``/``setitem`` - the index tuple.

One key is added to what the reference records: a ``selector_register`` entry may carry
``row_aligned: True``.  It declares that the selector's index array equals the reducer's (sorted)
row ids, so a kernel may take the row id from the merge path instead of reading the array.
"""
from __future__ import annotations

import hashlib
import json
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

# Map operation names the reference's emitters accept (codegen/merged_gen_core.py:146-234).
MAP_OPS = (
    "add", "sub", "mul", "pow", "truediv", "neg", "add_", "exp", "norm", "reducer", "getitem",
    "clone", "copy_", "setitem", "sum", "abs", "sign", "lt", "gt", "where",
)

_DTYPE_NAMES = {"float32": "float32", "float": "float32", "torch.float32": "float32",
                "float64": "float64", "double": "float64", "torch.float64": "float64",
                "int64": "int64", "long": "int64", "torch.int64": "int64"}


# Node names become C++ locals of the generated code (as they do in the reference).  The generators keep
# their own identifiers under the prefix ``q_``; what is left to refuse are C++ keywords and that prefix.
RESERVED_NAMES = frozenset("""
    alignas alignof and asm auto bool break case catch char class const constexpr continue decltype default
    delete do double else enum explicit extern false float for friend goto if inline int long mutable
    namespace new not nullptr operator or private protected public register return short signed sizeof static
    struct switch template this throw true try typedef typename union unsigned using virtual void volatile
    while xor flex oracle ValueT OffsetT
""".split())


def dtype_name(dtype: Any) -> str:
    """Canonical 'float32' | 'float64' | 'int64' for a torch/numpy dtype or its name."""
    key = str(dtype)
    if key in _DTYPE_NAMES:
        return _DTYPE_NAMES[key]
    name = getattr(dtype, "name", None) or getattr(dtype, "__name__", None)
    if name in _DTYPE_NAMES:
        return _DTYPE_NAMES[name]
    raise ValueError(f"unsupported value dtype {dtype!r}")


def arg_name(arg: Any) -> Any:
    """fx nodes appear by name in generated statements; everything else passes through."""
    return arg.name if hasattr(arg, "name") and not isinstance(arg, str) else arg


def get_dim_length(shape: Sequence[int]) -> int:
    """Flattened per-item width (codegen/utils.py:5-12)."""
    n = 1
    for s in shape:
        n *= int(s)
    return n


@dataclass
class FusedGraphIR:
    """The six lists for one fused sub-graph plus a stable name."""

    name: str
    inputs: List[Dict[str, Any]]
    outputs: List[Dict[str, Any]]
    selector_register: List[Dict[str, Any]]
    map_operations: List[Dict[str, Any]]
    reducer_operations: List[Dict[str, Any]]
    aggregator_operations: List[Dict[str, Any]]
    doc: str = ""

    def six(self) -> Tuple[list, list, list, list, list, list]:
        return (self.inputs, self.outputs, self.selector_register, self.map_operations,
                self.reducer_operations, self.aggregator_operations)

    @property
    def has_reducer(self) -> bool:
        return bool(self.reducer_operations)

    @property
    def has_aggregator(self) -> bool:
        return bool(self.aggregator_operations)

    def canonical(self) -> str:
        """Deterministic text form: the content key for build caches."""
        def clean(v):
            if isinstance(v, dict):
                # one library serves float32 and float64 alike: the two spell the same key
                return {k: ("float" if k == "dtype_data" and str(x).endswith(("float32", "float64")) else clean(x))
                        for k, x in sorted(v.items()) if not k.startswith("_")}
            if isinstance(v, (list, tuple)):
                return [clean(x) for x in v]
            if isinstance(v, slice):
                return ["slice", v.start, v.stop, v.step]
            if isinstance(v, (str, int, float, bool)) or v is None:
                return v
            return str(arg_name(v))
        return json.dumps({"name": self.name, "six": clean(list(self.six()))}, sort_keys=True)

    def content_hash(self) -> str:
        return hashlib.sha1(self.canonical().encode()).hexdigest()[:12]


class GraphBuilder:
    """Write the six lists the way ``trace_graph`` would have produced them, node by node.

    Nodes are appended in graph order, which fixes the binding's argument order
    (codegen/merged_gen_binding.py:27-78).
    """

    def __init__(self, name: str, dtype: Any = "float32", doc: str = "") -> None:
        self.name = name
        self.dtype = dtype_name(dtype)
        self.doc = doc
        self._nodes: List[Dict[str, Any]] = []
        self._shape: Dict[str, Tuple[int, ...]] = {}
        self._outputs: List[str] = []

    # -- graph nodes ---------------------------------------------------------------------
    def _shape_of(self, shape) -> Tuple[int, ...]:
        shape = tuple(int(s) for s in shape)
        return shape if shape else (1,)

    @staticmethod
    def _check_name(name: str) -> None:
        if name in RESERVED_NAMES or not name.isidentifier() or name.startswith(("__", "q_")):
            raise ValueError(f"Operation on a value called {name!r} not supported: the name is not usable as a "
                             "variable of the generated code")

    def placeholder(self, name: str, shape=(1,)) -> str:
        """A tensor argument of the fused sub-graph (edge tensor unless a selector gathers it)."""
        self._check_name(name)
        self._shape[name] = self._shape_of(shape)
        self._nodes.append({"kind": "placeholder", "name": name})
        return name

    def select(self, name: str, source: str, module: Optional[str] = None,
               row_aligned: bool = False) -> str:
        """``name = <Selector module>(source)``: gather rows of ``source`` by the module's idx."""
        self._check_name(name)
        self._shape[name] = self._shape[source]
        self._nodes.append({"kind": "selector", "name": name, "source": source,
                            "module": (module or name).replace(".", "_"),
                            "row_aligned": bool(row_aligned)})
        return name

    def map(self, op: str, name: str, args: Sequence[Any], shape=None) -> str:
        """One element-wise call_function / call_method node classified as ``op``."""
        if op not in MAP_OPS or op in ("reducer", "sum"):
            raise ValueError(f"Operation {op} not supported")
        if shape is None:
            shape = self._infer_shape(op, args)
        self._check_name(name)
        self._shape[name] = self._shape_of(shape)
        self._nodes.append({"kind": "map", "op": op, "name": name, "args": list(args)})
        return name

    def reduce(self, name: str, arg: str, module: Optional[str] = None) -> str:
        """``name = <Reducer module>(arg)``: segment-sum by CSR row."""
        self._check_name(name)
        self._shape[name] = self._shape[arg]
        self._nodes.append({"kind": "reducer", "name": name, "args": [arg],
                            "module": (module or name).replace(".", "_")})
        return name

    def aggregate(self, name: str, arg: str) -> str:
        """``name = sum(arg)`` over all edges."""
        self._check_name(name)
        self._shape[name] = self._shape[arg]
        self._nodes.append({"kind": "sum", "name": name, "args": [arg]})
        return name

    def output(self, *names: str) -> None:
        self._outputs.extend(names)

    def _infer_shape(self, op: str, args: Sequence[Any]):
        if op in ("norm", "getitem"):
            return (1,)
        if op == "setitem":
            return self._shape[args[0]]
        best: Tuple[int, ...] = (1,)
        for a in args:
            if isinstance(a, str) and a in self._shape and \
                    get_dim_length(self._shape[a]) > get_dim_length(best):
                best = self._shape[a]
        return best

    # -- emit the six lists ---------------------------------------------------------------
    def build(self) -> FusedGraphIR:
        dt = self.dtype
        out_set = set(self._outputs)
        kinds = {n["name"]: n for n in self._nodes}
        gathered = {n["source"] for n in self._nodes if n["kind"] == "selector"}

        inputs, selector_register, map_ops, red_ops, agg_ops, outputs = [], [], [], [], [], []
        for n in self._nodes:
            name = n["name"]
            shape = self._shape[name]
            if n["kind"] in ("reducer", "sum") and name not in out_set:
                continue        # a reduction nobody reads: it has no output buffer, so it is not generated
            if n["kind"] == "placeholder":
                if name in out_set:
                    continue
                inputs.append({"name": name, "target": name, "dtype": "scalar_t", "shape": shape,
                               "op": "placeholder", "args": (), "dtype_data": dt})
                if name not in gathered:
                    selector_register.append({"name": name, "target": name, "dtype": "TensorT",
                                              "selector": 0, "selector_name": name, "shape": shape,
                                              "dtype_data": dt})
            elif n["kind"] == "selector":
                inputs.append({"name": name, "target": n["module"], "dtype": "int", "shape": shape,
                               "op": "call_module", "args": (n["source"],), "dtype_data": dt})
                entry = {"name": name, "target": n["source"], "dtype": "TensorKeyT", "selector": 1,
                         "selector_name": n["module"], "shape": shape, "dtype_data": dt}
                if n["row_aligned"]:
                    entry["row_aligned"] = True
                selector_register.append(entry)
            elif n["kind"] == "map":
                map_ops.append({"name": name, "target": n["op"], "op": n["op"], "shape": shape,
                                "dtype_data": dt, "args": list(n["args"])})
            elif n["kind"] == "reducer":
                map_ops.append({"name": name, "target": n["module"], "op": "reducer", "shape": shape,
                                "dtype_data": dt, "args": list(n["args"])})
                red_ops.append({"name": name, "op": "reducer", "shape": shape, "dtype_data": dt,
                                "args": list(n["args"])})
            elif n["kind"] == "sum":
                map_ops.append({"name": name, "target": "sum", "op": "sum", "shape": shape,
                                "dtype_data": dt, "args": list(n["args"])})
                agg_ops.append({"name": name, "op": "sum", "shape": shape, "dtype_data": dt,
                                "args": list(n["args"])})
        for name in self._outputs:
            n = kinds[name]
            if n["kind"] == "reducer":
                op, target = "call_module", "reducer"
            elif n["kind"] == "sum":
                op, target = "call_function", "sum"
            elif n["kind"] == "map":
                op, target = "call_function", n["op"]
            elif n["kind"] == "selector":     # a gathered value handed on as it is: a per-edge (map) output
                op, target = "call_module", n["module"]
            else:
                raise ValueError(f"{name}: a {n['kind']} node cannot be a sub-graph output")
            outputs.append({"op": op, "name": name, "target": target, "dtype": "ValueT",
                            "shape": self._shape[name], "args": tuple(n.get("args", ())),
                            "dtype_data": dt})
        return FusedGraphIR(self.name, inputs, outputs, selector_register, map_ops, red_ops,
                            agg_ops, doc=self.doc)
