"""Host-side tests of the modelling front end, the tracer and the replacement wrapper (no GPU).

The fused sub-modules are executed three ways and must agree: the model run eagerly, the compiled model
(fused torch sub-modules called in stage order), and the compiled model with its sub-modules replaced by
an extension object backed by the CPU oracle - which checks the whole host path (trace -> six lists ->
binding order -> wrapper arguments) without a device.
"""
import operator

import numpy as np
import pytest
import torch

from flexspmv_amd import frontend as esr
from flexspmv_amd import graphs
from flexspmv_amd.codegen.merged_gen_binding import binding_plan
from flexspmv_amd.drivers import ab_check
from flexspmv_amd.drivers.prebuilt import MODELS
from flexspmv_amd.drivers.shallow_water import ShallowWaterEquation, synthetic_mesh
from flexspmv_amd.drivers.spring_mass import SpringMass, lattice
from flexspmv_amd.drivers.system_model import make_system
from flexspmv_amd.ir import FusedGraphIR
from flexspmv_amd.python_wrapper import edge_order
from flexspmv_amd.python_wrapper.accelerate import fused_call_nodes, lower_submodules
from flexspmv_amd.python_wrapper.dynamic_replace_submodule import (_coo_rows_to_csr_ptr, _DynamicCudaWrapper,
                                                                    dynamic_replace_submodule)
from flexspmv_amd.trace.graph_trace import classify, trace_graph
from oracle.runner import run_oracle


class OracleExtension:
    """``merged_spmv_launch`` of one sub-graph served by the CPU oracle (test double of a built library)."""

    def __init__(self, ir: FusedGraphIR):
        self.ir = ir
        self.plan = binding_plan(ir.inputs, ir.outputs, ir.selector_register)
        self.calls = 0

    def param_names(self):
        return [n for n, _ in self.plan.bind_params]

    def merged_spmv_launch(self, *args):
        self.calls += 1
        bound = dict(zip(self.param_names(), args))
        tensors = {k: v.detach().numpy() for k, v in bound.items() if isinstance(v, torch.Tensor)
                   and k != "row_end_offsets"}
        ro = bound["row_end_offsets"].numpy() if self.ir.has_reducer else None
        outs, after = run_oracle(self.ir, tensors, ro, bound["num_rows"], bound["num_cols"], num_threads=3)
        for k, v in after.items():           # in-place map ops write through the inputs - through their memory, as
            # a library does through raw pointers: torch sees no operation and bumps no version counter
            np.copyto(bound[k].detach().numpy().reshape(-1), v.reshape(-1))
        return tuple(torch.from_numpy(o) for o in outs) if outs else None


def replace_all_with_oracle(compiled, prefix):
    irs, skipped = lower_submodules(compiled, prefix)
    exts = {}
    for name, ir in irs.items():
        exts[name] = OracleExtension(ir)
        assert dynamic_replace_submodule(compiled, exts[name], name)
    return exts, skipped


def test_system_model_fuses_into_the_sub_graph_the_reference_generates():
    [compiled] = esr.compile([make_system()], "torch")
    names = [n.name for n in fused_call_nodes(compiled)]
    assert len(names) == 2 and names[0].endswith("select_reduce") and names[1].endswith("map")
    six = trace_graph(compiled.get_submodule(names[0]), compiled)
    ref = graphs.get("system_two_selectors")
    strip = lambda ops: [(o["name"], o["op"], tuple(o["shape"]), [str(a) for a in o["args"]]) for o in ops]  # noqa: E731
    assert strip(six[3]) == strip(ref.map_operations)
    assert strip(six[4]) == strip(ref.reducer_operations)
    key = lambda s: (s["name"], s["target"], s["selector"], s["selector_name"], tuple(s["shape"]))  # noqa: E731
    assert sorted(map(key, six[2])) == sorted(map(key, ref.selector_register))
    assert [(o["name"], o["target"]) for o in six[1]] == [("reducer_1", "reducer")]
    assert {i["name"] for i in six[0]} == {i["name"] for i in ref.inputs}


@pytest.mark.parametrize("name", sorted(MODELS))
def test_compiled_model_equals_eager_model(name):
    eager, traced = MODELS[name](), MODELS[name]()
    [compiled] = esr.compile([traced], "torch")
    for _ in range(4):
        eager()
        compiled()
    for (k, a), (_, b) in zip(eager.named_parameters(), traced.named_parameters()):
        assert torch.equal(a, b), k


def test_swe_groups_and_row_alignment():
    [compiled] = esr.compile([MODELS["swe"]()], "torch")
    nodes = fused_call_nodes(compiled)
    kinds = [n.name.split("_", 1)[1] for n in nodes]
    # per Runge-Kutta stage: interior faces, wall faces, one flat cell update; plus the final update
    assert kinds.count("select_reduce") == 8 and kinds.count("map") == 5
    irs, skipped = lower_submodules(compiled, "swe")
    assert not skipped
    interior = irs[nodes[0].name]
    assert len(interior.reducer_operations) == 3
    aligned = [s for s in interior.selector_register if s.get("row_aligned")]
    assert aligned and all(s["selector_name"] == "gather_dst" for s in aligned)


def test_read_after_write_and_write_after_read_keep_program_order():
    class Chain(esr.Module):
        def __init__(self):
            super().__init__()
            self.a = esr.Tensor(torch.arange(8.0))
            self.b = esr.Tensor(torch.ones(8))
            self.c = esr.Tensor(torch.zeros(8))
            self.pick = esr.Selector(torch.tensor([7, 6, 5, 4, 3, 2, 1, 0]))

        def forward(self):
            g = self.pick(self.a)         # reads a ...
            self.a[:] = self.b * 2.0      # ... before it is overwritten
            self.c[:] = self.a + g        # reads the new a
            self.b.add_(self.c)           # and the next step sees the new b

    eager, traced = Chain(), Chain()
    [compiled] = esr.compile([traced], "torch")
    for _ in range(3):
        eager()
        compiled()
    for k in ("a", "b", "c"):
        assert torch.equal(getattr(eager, k), getattr(traced, k)), k


def test_operations_are_classified_by_identity_not_by_text():
    import torch.fx as fx

    def padded_where_thing(x):     # the text of this target contains 'add' and 'where'
        return x

    g = fx.Graph()
    x = g.placeholder("x")
    bad = g.call_function(padded_where_thing, (x,))
    good = g.call_function(torch.where, (x, x, x))
    ia = g.call_method("add_", (x, x))
    with pytest.raises(ValueError, match="not supported"):
        classify(bad)
    assert classify(good) == "where" and classify(ia) == "add_"
    assert classify(g.call_function(operator.truediv, (1.0, x))) == "truediv"


def test_broadcast_along_the_edge_dimension_is_rejected_not_generated():
    class Scaled(esr.Module):
        def __init__(self):
            super().__init__()
            self.v = esr.Tensor(torch.rand(16))
            self.total = esr.Tensor(torch.zeros(1))
            self.out = esr.Tensor(torch.zeros(16))

        def forward(self):
            self.total[:] = esr.sum(self.v)
            self.out[:] = self.v / self.total     # [16] / [1]

    [compiled] = esr.compile([Scaled()], "torch")
    irs, skipped = lower_submodules(compiled, "scaled")
    assert any("different lengths" in why for why in skipped.values())
    compiled()                                     # the torch sub-modules still run
    assert torch.allclose(compiled.out.sum(), torch.tensor(1.0))


@pytest.mark.parametrize("name,steps,tol", [("system", 2, 1e-14), ("spring", 3, 2e-5), ("swe", 2, 1e-12),
                                            ("swe_parts", 1, 0), ("swe_init", 1, 1e-13)])
def test_replaced_model_matches_original_through_the_wrapper(name, steps, tol):
    eager, traced = MODELS[name](), MODELS[name]()
    [compiled] = esr.compile([traced], "torch")
    exts, skipped = replace_all_with_oracle(compiled, f"t_{name}")
    assert not skipped
    for _ in range(steps):
        eager()
        compiled()
    assert all(e.calls == steps for e in exts.values())
    want, got = ab_check.save_state(eager), ab_check.save_state(traced)
    if name == "system":
        # (2,1) + (2,3): the reference's value type pairs flat element k of the wide operand with element
        # k % 2 of the narrow one (data_struct_shared.cuh:611-636), torch pairs it with element k // 3.
        # The generated code follows the reference, so this one tensor differs from torch by design.
        narrow = (traced.selector_1(traced.vector_x) + traced.selector_2(traced.vector_x)).reshape(-1, 2)
        k = torch.arange(6)
        expected = narrow[:, k % 2] + traced.spm_2.reshape(-1, 6)
        assert torch.allclose(got.pop("y_add_2").reshape(-1, 6), expected, rtol=1e-14, atol=0)
        assert not torch.allclose(want.pop("y_add_2").reshape(-1, 6), expected)
    worst, ok = ab_check.compare_states(want, got, tol)
    assert ok, worst


def test_wrapper_argument_order_and_shapes():
    [compiled] = esr.compile([make_system(30, 9, 7)], "torch")
    node = fused_call_nodes(compiled)[0]
    seen = {}

    class Probe:
        def merged_spmv_launch(self, *args):
            seen["args"] = args
            return (torch.zeros(7, 2),)

    assert dynamic_replace_submodule(compiled, Probe(), node.name)
    assert not dynamic_replace_submodule(compiled, Probe(), "no_such_node")
    wrapper = getattr(compiled, node.target)
    assert isinstance(wrapper, _DynamicCudaWrapper)
    compiled()
    a = seen["args"]
    # non-gather values in placeholder order, the gather source, two int32 index tensors, CSR, sizes
    assert [tuple(t.shape) for t in a[:5]] == [(30, 2, 1), (30, 2, 3), (30, 2, 1), (30, 2, 3), (9, 2, 1)]
    assert a[5].dtype == a[6].dtype == a[7].dtype == torch.int32
    assert a[7].numel() == 8 and int(a[7][-1]) == 30 and a[8:] == (7, 9)
    # the result is handed back in the shape the fused sub-module produces
    assert tuple(compiled.y_reducer_1.shape) == (7, 2, 1)


def test_coo_to_csr_and_unsorted_rows():
    rows = torch.tensor([0, 0, 2, 2, 2, 5])
    ptr, n = _coo_rows_to_csr_ptr(rows, 7)
    assert n == 7 and ptr.tolist() == [0, 2, 2, 5, 5, 5, 6, 6]
    assert _coo_rows_to_csr_ptr(rows)[1] == 6
    with pytest.raises(RuntimeError, match="sorted"):
        _coo_rows_to_csr_ptr(torch.tensor([1, 0, 2]), 3)
    with pytest.raises(RuntimeError, match="outside"):
        _coo_rows_to_csr_ptr(torch.tensor([0, 3]), 3)
    assert edge_order.coo_to_csr(rows, 7).dtype == torch.int32


def test_edge_ordering_helpers():
    g = torch.Generator().manual_seed(0)
    dst = torch.randint(0, 10, (50,), generator=g)
    w = torch.rand(50, 3, generator=g)
    sorted_dst, perm, w2 = edge_order.sort_edges_by_row(dst, w)
    assert bool((sorted_dst[1:] >= sorted_dst[:-1]).all()) and torch.equal(w2, w[perm])
    # stable: equal rows keep their original order
    for r in range(10):
        p = perm[sorted_dst == r]
        assert bool((p[1:] > p[:-1]).all())
    a, b = torch.tensor([0, 1, 2]), torch.tensor([1, 2, 0])
    s2, d2, sign, origin, w3 = edge_order.half_edges(a, b, torch.tensor([10.0, 20.0, 30.0]))
    assert d2.tolist() == sorted(d2.tolist()) and len(d2) == 6
    pairs = {(int(s), int(d)) for s, d in zip(s2, d2)}
    assert pairs == {(0, 1), (1, 2), (2, 0), (1, 0), (2, 1), (0, 2)}
    assert torch.equal(w3, torch.tensor([10.0, 20.0, 30.0])[origin])
    assert all((sg > 0) == ((int(s), int(d)) in {(0, 1), (1, 2), (2, 0)}) for s, d, sg in zip(s2, d2, sign))


def test_assembled_geometry_is_closed_and_feeds_the_model():
    from flexspmv_amd.drivers.shallow_water_assembly import assemble, mesh_for_model
    mesh, parts, init = assemble(400)
    nc = mesh["cells"].shape[0]
    # the collected ids are the cells' point ids seen from each face
    assert torch.equal(torch.stack([p.data for p in parts.src_p], 1), mesh["cells"][mesh["src"]])
    assert torch.equal(torch.stack([p.data for p in parts.bp], 1), mesh["bpoints"])
    # every cell's inward face normals (interior + wall) close the polygon; areas tile the unit square
    for a, b in ((init.sx, init.bsx), (init.sy, init.bsy)):
        closed = torch.zeros(nc, dtype=torch.float64).index_add_(0, mesh["dst"], a.data).index_add_(0, mesh["bcells"], b.data)
        assert float(closed.abs().max()) < 1e-14
    assert abs(float(init.area.sum()) - 1.0) < 1e-13
    assert 0.0 < float(init.alpha.min()) and float(init.alpha.max()) < 1.0
    model = ShallowWaterEquation(mesh_for_model(mesh, init), dt=0.002)
    mass = float((model.h * model.area).sum())
    for _ in range(20):
        model()
    assert abs(float((model.h * model.area).sum()) - mass) < 1e-13 and float(model.h.max()) < 1.2


def test_swe_conserves_mass():
    mesh = synthetic_mesh(400)
    m = ShallowWaterEquation(mesh, dt=0.002)
    mass = float((m.h * m.area).sum())
    for _ in range(10):
        m()
    assert abs(float((m.h * m.area).sum()) - mass) < 1e-13
    assert float(m.uh.abs().max()) > 0          # the bump started to move


def test_spring_energy_is_half_k_stretch_squared():
    pos, springs = lattice(4, dtype=torch.float64)
    m = SpringMass(pos, springs, stiffness=3.0)
    with torch.no_grad():
        m.pos.mul_(1.1)                          # stretch every spring by 10 %
    a, b = springs[:, 0], springs[:, 1]
    rest = (pos[a] - pos[b]).norm(dim=1)
    m()
    expected = float((0.5 * 3.0 * (0.1 * rest) ** 2).sum())
    assert abs(float(m.energy) - expected) < 1e-12 * expected
    # internal forces cancel
    assert float(m.force.sum(dim=0).abs().max()) < 1e-12


def test_reference_named_entry_point_writes_the_hip_source(tmp_path):
    """``generate_cuda_code_from_graph(submodule, traced_model)`` - the call the reference's drivers make
    (easier_spmv.py:157) - traces the fused sub-module and writes its translation unit."""
    from flexspmv_amd.codegen.merged_gen_gpu import generate_cuda_code_from_graph
    from flexspmv_amd.python_wrapper.accelerate import get_submodules
    [compiled] = esr.compile([make_system()], "torch")
    submodules, nodes = get_submodules(compiled)
    path, signature = generate_cuda_code_from_graph(submodules[0], compiled, out_dir=str(tmp_path))
    text = open(path).read()
    assert path.endswith(".hip") and "flexspmv_launch" in text and "struct Graph" in text
    assert [p["name"] for p in signature["params"]][-3:] == ["row_end_offsets", "num_rows", "num_cols"]
    assert signature["index_inputs"] == ["selector_1_idx", "selector_2_idx"]


def test_unsorted_reducer_rows_are_sorted_behind_the_wrapper():
    """The reference's toy model draws its row ids unsorted (easier_spmv.py:126-127).  The wrapper sorts the
    edges once, feeds the kernel sorted copies and puts per-edge results back in the model's edge order."""
    class Unsorted(esr.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(3)
            ne, nv, nr = 300, 40, 25
            self.w = esr.Tensor(torch.rand(ne, 2, generator=g, dtype=torch.float64))
            self.v = esr.Tensor(torch.rand(nv, 2, generator=g, dtype=torch.float64))
            self.per_edge = esr.Tensor(torch.zeros(ne, 2, dtype=torch.float64))
            self.per_row = esr.Tensor(torch.zeros(nr, 2, dtype=torch.float64))
            self.total = esr.Tensor(torch.zeros(1, 2, dtype=torch.float64))
            self.pick = esr.Selector(torch.randint(0, nv, (ne,), generator=g))
            rows = torch.randint(0, nr, (ne,), generator=g)                               # not sorted
            self.scatter = esr.Reducer(rows, nr)
            self.row_of_edge = esr.Selector(rows)
            self.per_edge_2 = esr.Tensor(torch.zeros(ne, 2, dtype=torch.float64))

        def forward(self):
            prod = self.pick(self.v) * self.w
            self.per_edge[:] = prod
            self.per_row[:] = self.scatter(prod)
            self.total[:] = esr.sum(prod + self.w)
            # a later kernel takes the per-edge value of the first one and gathers the fresh row sums
            self.per_edge_2[:] = prod * self.row_of_edge(self.per_row)

    eager, traced = Unsorted(), Unsorted()
    assert bool((traced.scatter.idx[1:] < traced.scatter.idx[:-1]).any())
    [compiled] = esr.compile([traced], "torch")
    exts, skipped = replace_all_with_oracle(compiled, "t_unsorted")
    assert not skipped
    eager()
    compiled()
    assert torch.equal(eager.per_edge, traced.per_edge)                        # back in the model's edge order
    assert torch.allclose(eager.per_edge_2, traced.per_edge_2, rtol=1e-13, atol=0)
    assert len(exts) >= 3
    assert torch.allclose(eager.per_row, traced.per_row, rtol=1e-13, atol=0)
    assert torch.allclose(eager.total, traced.total, rtol=1e-13, atol=0)
    # A streamed tensor that has not changed since the previous call is not permuted again; one that was
    # modified in place (its version counter moved) is.
    wrappers = [m for m in compiled.modules() if type(m).__name__ == "_DynamicCudaWrapper" and m._sorted_inputs]
    assert wrappers
    kept = {id(w): {n: v[2] for n, v in w._sorted_inputs.items()} for w in wrappers}
    eager()
    compiled()
    constant = [n for w in wrappers for n, v in w._sorted_inputs.items() if v[2] is kept[id(w)][n]]
    assert constant                                                            # e.g. the model tensor w
    assert torch.allclose(eager.per_row, traced.per_row, rtol=1e-13, atol=0)
    with torch.no_grad():
        eager.w.mul_(1.5)
        traced.w.mul_(1.5)
    eager()
    compiled()
    assert torch.equal(eager.per_edge, traced.per_edge)
    assert torch.allclose(eager.per_row, traced.per_row, rtol=1e-13, atol=0)


def _random_model_source(rng, n_stmts=14, rich=False):
    """Python source of a random model: gathers, per-edge and per-vertex arithmetic, reductions, in-place
    stores and re-reads of model tensors, in random order.  ``rich`` adds the rest of the operation set
    (neg, abs, powers, exp, division, comparisons with where, norm, column picks with clone / copy_)."""
    lines = []
    edge_vals, vert_vals, edge_cols, vert_cols = [], [], [], []
    counter = [0]

    def fresh(prefix):
        counter[0] += 1
        return f"{prefix}{counter[0]}"

    def pick(pool):
        return pool[int(rng.integers(0, len(pool)))]

    def edge_operand():
        return pick(edge_vals + [f"self.E{i}" for i in range(3)])

    def vert_operand():
        return pick(vert_vals + [f"self.V{i}" for i in range(3)])

    def unary(x):
        k = int(rng.integers(0, 7))
        return [f"-{x}", f"abs({x} - 0.5)", f"{x} ** 2", f"({x} * {x} + 0.5) ** 0.5", f"torch.exp(-({x} * {x}))",
                f"{x} / ({x} * {x} + 1.0)", f"esr.norm({x}) * {x}"][k]

    def binary(a, b):
        k = int(rng.integers(0, 4))
        return [f"torch.where({a} > {b}, {a}, {b})", f"torch.where({a} < {b}, {a}, {b} * 0.5)", f"{a} / ({b} * {b} + 1.0)",
                f"{a} * {b} - {a}"][k]

    for _ in range(n_stmts):
        kind = int(rng.integers(0, 14 if rich else 9))
        if kind <= 1:
            name = fresh("e")
            lines.append(f"{name} = self.sel{int(rng.integers(0, 2))}({vert_operand()})")
            edge_vals.append(name)
        elif kind == 2:
            name = fresh("e")
            lines.append(f"{name} = {edge_operand()} {'+-*'[int(rng.integers(0, 3))]} {edge_operand()}")
            edge_vals.append(name)
        elif kind == 3:
            name = fresh("v")
            lines.append(f"{name} = {vert_operand()} {'+-*'[int(rng.integers(0, 3))]} {vert_operand()}")
            vert_vals.append(name)
        elif kind == 4 and edge_vals:
            name = fresh("v")
            lines.append(f"{name} = self.red({pick(edge_vals)})")
            vert_vals.append(name)
        elif kind == 5 and vert_vals:
            lines.append(f"self.V{int(rng.integers(0, 3))}[:] = {pick(vert_vals)} * 0.5")
        elif kind == 6 and edge_vals:
            lines.append(f"self.E{int(rng.integers(0, 3))}[:] = {pick(edge_vals)} * 0.5")
        elif kind == 7 and vert_vals:
            lines.append(f"self.V{int(rng.integers(0, 3))}.add_({pick(vert_vals)} * 0.25)")
        elif kind == 8 and edge_vals:
            lines.append(f"self.S[:] = esr.sum({pick(edge_vals)})")
        elif kind == 9:
            name = fresh("e")
            lines.append(f"{name} = {unary(edge_operand())}")
            edge_vals.append(name)
        elif kind == 10:
            name = fresh("v")
            lines.append(f"{name} = {binary(vert_operand(), vert_operand())}")
            vert_vals.append(name)
        elif kind == 11:
            name = fresh("e")
            lines.append(f"{name} = {binary(edge_operand(), edge_operand())}")
            edge_vals.append(name)
        elif kind == 12:                      # column picks: (n, 2) -> (n,), stored into 1-D tensors
            name = fresh("c")
            lines.append(f"{name} = {edge_operand()}[:, {int(rng.integers(0, 2))}].clone()")
            edge_cols.append(name)
            if len(edge_cols) > 1 and rng.random() < 0.5:
                lines.append(f"self.EC.copy_({pick(edge_cols)} * {pick(edge_cols)})")
            else:
                lines.append(f"self.EC[:] = {name} * 0.5")
        elif kind == 13:
            name = fresh("d")
            lines.append(f"{name} = {vert_operand()}[:, {int(rng.integers(0, 2))}].clone()")
            vert_cols.append(name)
            lines.append(f"self.VC.copy_({name})")
    if not any(l.startswith("self.") for l in lines):
        lines.append("self.V0[:] = self.V1 * 0.5")
    body = "\n".join("        " + l for l in lines)
    return f"""
class Random(esr.Module):
    def __init__(self):
        super().__init__()
        g = torch.Generator().manual_seed(5)
        ne, nv = 60, 17
        for i in range(3):
            setattr(self, f"E{{i}}", esr.Tensor(torch.rand(ne, 2, generator=g, dtype=torch.float64)))
            setattr(self, f"V{{i}}", esr.Tensor(torch.rand(nv, 2, generator=g, dtype=torch.float64)))
        self.EC = esr.Tensor(torch.zeros(ne, dtype=torch.float64))
        self.VC = esr.Tensor(torch.zeros(nv, dtype=torch.float64))
        self.S = esr.Tensor(torch.zeros(1, 2, dtype=torch.float64))
        self.sel0 = esr.Selector(torch.randint(0, nv, (ne,), generator=g))
        self.sel1 = esr.Selector(torch.randint(0, nv, (ne,), generator=g))
        self.red = esr.Reducer(torch.sort(torch.randint(0, nv, (ne,), generator=g)).values, nv)

    def forward(self):
{body}
"""


@pytest.mark.parametrize("seed", range(40))
def test_random_models_compile_to_the_same_results(seed):
    """Dataflow fusion keeps program order: a random model run eagerly and as fused sub-modules agrees
    bit for bit over three steps (reads before and after in-place stores, gathers of freshly stored
    tensors, reductions feeding later gathers)."""
    rng = np.random.default_rng(1000 + seed)
    source = _random_model_source(rng, n_stmts=16, rich=(seed % 2 == 1))
    scope = {"esr": esr, "torch": torch}
    exec(source, scope)
    eager, traced = scope["Random"](), scope["Random"]()
    [compiled] = esr.compile([traced], "torch")
    for _ in range(3):
        eager()
        compiled()
    for (k, a), (_, b) in zip(eager.named_parameters(), traced.named_parameters()):
        assert torch.equal(a, b), (k, source)


def test_aggregator_sees_the_inputs_as_handed_over_when_the_same_kernel_overwrites_them():
    """One fused kernel stores into an edge tensor, reduces per row and aggregates a value computed from
    that tensor's original contents.  The oracle runs a reducer and an aggregator as two passes; the
    aggregator pass must not see the reducer pass's stores."""
    class StoreAndSum(esr.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(8)
            ne, nv = 90, 12
            self.a = esr.Tensor(torch.rand(ne, generator=g, dtype=torch.float64))
            self.b = esr.Tensor(torch.rand(ne, generator=g, dtype=torch.float64))
            self.rows = esr.Tensor(torch.zeros(nv, dtype=torch.float64))
            self.total = esr.Tensor(torch.zeros(1, dtype=torch.float64))
            self.red = esr.Reducer(torch.sort(torch.randint(0, nv, (ne,), generator=g)).values, nv)

        def forward(self):
            prod = self.a * self.b
            self.a[:] = prod * 0.5
            self.rows[:] = self.red(prod)
            self.total[:] = esr.sum(prod * self.b)

    eager, traced = StoreAndSum(), StoreAndSum()
    [compiled] = esr.compile([traced], "torch")
    exts, skipped = replace_all_with_oracle(compiled, "t_store_sum")
    assert not skipped
    fused = [e for e in exts.values() if e.ir.has_reducer and e.ir.has_aggregator]
    assert len(fused) == 1                    # the store, the reducer and the aggregator share a kernel
    for _ in range(2):
        eager()
        compiled()
    for k in ("a", "rows", "total"):
        assert torch.allclose(getattr(eager, k), getattr(traced, k), rtol=1e-13, atol=0), k


def test_tensor_names_that_look_like_kernel_internals_and_a_gathered_output():
    """Model tensors called ``e``, ``total``, ``row`` or ``p`` and a selector whose node shares the name of a
    value handed on to a later kernel must not collide with anything in the generated code (the generators
    keep their own identifiers under ``q_`` and index pointers under ``<module>_idx_ptr``); a gathered value
    may itself be a per-edge output."""
    class Names(esr.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(8)
            self.p = esr.Tensor(torch.rand(12, 2, generator=g, dtype=torch.float64))
            self.e = esr.Tensor(torch.zeros(50, 2, dtype=torch.float64))
            self.total = esr.Tensor(torch.zeros(12, 2, dtype=torch.float64))
            self.row = esr.Tensor(torch.rand(50, 2, generator=g, dtype=torch.float64))
            self.sel = esr.Selector(torch.randint(0, 12, (50,), generator=g))
            self.red = esr.Reducer(torch.sort(torch.randint(0, 12, (50,), generator=g)).values, 12)

        def forward(self):
            s = self.sel(self.p)
            self.e[:] = s * self.row
            self.total[:] = self.red(s)
            self.p[:] = self.total * 0.5
            self.e.add_(s * self.sel(self.p))          # s crosses into a later kernel as a placeholder "sel"

    eager, traced = Names(), Names()
    [compiled] = esr.compile([traced], "torch")
    irs, skipped = lower_submodules(compiled, "t_names")
    assert not skipped
    first = irs[fused_call_nodes(compiled)[0].name]
    assert any(o["name"] == "sel" and o["op"] == "call_module" for o in first.outputs)
    from flexspmv_amd.codegen.merged_gen_gpu import generate_hip_source
    for ir in irs.values():
        text, _ = generate_hip_source(ir)
        assert "q_p." in text and ("_idx_ptr" in text or not ir.inputs or all(i["dtype"] != "int" for i in ir.inputs))
    exts, _ = replace_all_with_oracle(compiled, "t_names")
    for _ in range(2):
        eager()
        compiled()
    for (k, a), (_, b) in zip(eager.named_parameters(), traced.named_parameters()):
        assert torch.allclose(a, b, rtol=1e-13, atol=0), k
    with pytest.raises(ValueError, match="not usable"):
        from flexspmv_amd.ir import GraphBuilder
        GraphBuilder("bad").placeholder("q_e")
    with pytest.raises(ValueError, match="not usable"):
        GraphBuilder("bad").placeholder("double")


# ---------------------------------------------------------------------------------------------
# named arrays from files (the esr.hdf5 stand-in)
# ---------------------------------------------------------------------------------------------
def test_mesh_file_round_trip_gives_the_same_model(tmp_path):
    from flexspmv_amd.drivers.shallow_water import ShallowWaterEquation, load_mesh, save_mesh, synthetic_mesh
    mesh = synthetic_mesh(400, seed=5)
    path = str(tmp_path / "mesh.npz")
    save_mesh(mesh, path)
    assert set(esr.datasets(path)) >= {"src", "dst", "bcells", "x", "h", "nc"}
    assert esr.hdf5(path, "src", dtype=torch.long).dtype == torch.int64
    assert esr.hdf5(path, "h", dtype=torch.float32).dtype == torch.float32
    loaded = load_mesh(path)
    for k, v in mesh.items():
        assert (loaded[k] == v) if k == "nc" else torch.equal(loaded[k], v), k
    a, b = ShallowWaterEquation(mesh, dt=0.0005), ShallowWaterEquation(loaded, dt=0.0005)
    for _ in range(3):
        a()
        b()
    assert torch.equal(a.h, b.h) and torch.equal(a.uh, b.uh)


def test_array_files_fail_loudly(tmp_path):
    import numpy as np
    path = str(tmp_path / "arrays.npz")
    esr.save_arrays(path, {"a": torch.arange(4), "b": np.ones((2, 2)), "n": 3})
    assert esr.hdf5(path, "a").tolist() == [0, 1, 2, 3] and int(esr.hdf5(path, "n")) == 3
    with pytest.raises(KeyError, match="no array 'c'"):
        esr.hdf5(path, "c")
    with pytest.raises(FileNotFoundError):
        esr.hdf5(str(tmp_path / "missing.npz"), "a")
    with pytest.raises(RuntimeError, match="unknown container"):
        esr.save_arrays(str(tmp_path / "arrays.bin"), {"a": torch.arange(4)})
    h5 = str(tmp_path / "mesh.hdf5")
    try:
        import h5py  # noqa: F401
    except ImportError:
        open(h5, "wb").close()
        with pytest.raises(RuntimeError, match="h5py"):
            esr.hdf5(h5, "src")
        with pytest.raises(RuntimeError, match="h5py"):
            esr.save_arrays(h5, {"a": torch.arange(4)})
    else:
        esr.save_arrays(h5, {"a": torch.arange(4)})
        assert esr.hdf5(h5, "a").tolist() == [0, 1, 2, 3]
    from flexspmv_amd.drivers.shallow_water import load_mesh, save_mesh, synthetic_mesh
    mesh = synthetic_mesh(100, seed=1)
    mesh["src"] = mesh["src"].clone()
    mesh["src"][0] = mesh["nc"]              # a face that refers to a cell that does not exist
    bad = str(tmp_path / "bad.npz")
    save_mesh(mesh, bad)
    with pytest.raises(ValueError, match="outside"):
        load_mesh(bad)


def test_edge_tensor_written_by_one_kernel_and_streamed_by_the_next_is_never_stale():
    """Kernel A stores a per-edge tensor in place (through the raw pointer, not a torch operation); kernel B,
    whose reducer ids are unsorted, streams that tensor through the edge permutation.  The wrapper keeps the
    permuted copy of a streamed tensor only while the tensor is unchanged, so the store of A has to count as
    a change: every call must see the fresh values."""
    class TwoKernels(esr.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(5)
            ne, nv, nr = 240, 30, 20
            self.w = esr.Tensor(torch.rand(ne, generator=g, dtype=torch.float64))
            self.v = esr.Tensor(torch.rand(nv, generator=g, dtype=torch.float64))
            self.per_edge = esr.Tensor(torch.zeros(ne, dtype=torch.float64))
            self.per_row = esr.Tensor(torch.zeros(nr, dtype=torch.float64))
            self.per_row_2 = esr.Tensor(torch.zeros(nr, dtype=torch.float64))
            self.pick = esr.Selector(torch.randint(0, nv, (ne,), generator=g))
            rows = torch.randint(0, nr, (ne,), generator=g)                               # not sorted
            ascending = torch.sort(rows).values
            self.scatter = esr.Reducer(ascending, nr)                 # A: sorted ids, stores straight into per_edge
            self.scatter_2 = esr.Reducer(rows, nr)                    # B: unsorted ids, streams through a permutation
            self.row_of_edge = esr.Selector(ascending)

        def forward(self):
            prod = self.pick(self.v) * self.w
            self.per_edge[:] = prod                                   # kernel A writes the edge tensor
            self.per_row[:] = self.scatter(prod)
            fresh = self.row_of_edge(self.per_row)                    # gather of A's result: kernel B starts here
            self.per_row_2[:] = self.scatter_2(self.per_edge * fresh)  # B streams the tensor A wrote

    eager, traced = TwoKernels(), TwoKernels()
    [compiled] = esr.compile([traced], "torch")
    exts, skipped = replace_all_with_oracle(compiled, "t_two_kernels")
    assert not skipped and len(exts) >= 2
    wrappers = [m for m in compiled.modules() if type(m).__name__ == "_DynamicCudaWrapper"]
    assert any("per_edge" in w._written_inputs and w.edge_permutation is None for w in wrappers)
    assert any("per_edge" in w._non_gather_value_inputs and "per_edge" not in w._written_inputs
               and w.edge_permutation is not None for w in wrappers)
    for step in range(3):
        eager()
        compiled()
        assert torch.allclose(eager.per_row_2, traced.per_row_2, rtol=1e-13, atol=0), step
        with torch.no_grad():                                         # other vertex data for the next step
            eager.v.mul_(1.25)
            traced.v.mul_(1.25)


def test_permutation_into_a_given_tensor_counts_as_a_write():
    from flexspmv_amd.formats import mark_written
    t = torch.zeros(4)
    before = t._version
    mark_written(t)
    assert t._version == before + 1
