"""Whole models on the GPU: every fused sub-module replaced by its prebuilt gfx950 library, N steps
compared with the same model on its torch sub-modules (the flow of the reference's A/B driver,
test_full/easier_full.py:484-578, whose tolerance of 1e-10 is used for float64)."""
import pytest
import torch

from flexspmv_amd import frontend as esr
from flexspmv_amd.drivers import ab_check
from flexspmv_amd.drivers.prebuilt import MODELS
from flexspmv_amd.python_wrapper.accelerate import accelerate

pytestmark = pytest.mark.gpu


def run(name, steps, tolerance, skip=(), **kw):
    print(f"case model {name} steps={steps} {kw}", flush=True)
    model = MODELS[name](device="cuda", **kw)
    [compiled] = esr.compile([model], "torch")
    initial = ab_check.save_state(compiled)
    for _ in range(steps):
        compiled()
    original = ab_check.save_state(compiled)
    report = accelerate(compiled, prefix=name, build_if_missing=False)
    assert report and all(v == "replaced" for v in report.values()), report
    ab_check.restore_state(compiled, initial)
    for _ in range(steps):
        compiled()
    torch.cuda.synchronize()
    replaced = ab_check.save_state(compiled)
    for k in skip:
        original.pop(k), replaced.pop(k)
    worst, ok = ab_check.compare_states(original, replaced, tolerance)
    assert ok, worst
    return compiled


def test_system_model_float64():
    # y_add_2 pairs a (2,1) with a (2,3) operand: the reference's flat-index-modulo rule, not torch's
    c = run("system", 3, 1e-12, skip=("y_add_2",))
    narrow = (c.selector_1(c.vector_x) + c.selector_2(c.vector_x)).reshape(-1, 2)
    expected = narrow[:, torch.arange(6, device="cuda") % 2] + c.spm_2.reshape(-1, 6)
    assert torch.allclose(c.y_add_2.reshape(-1, 6), expected, rtol=1e-14, atol=0)


def test_system_model_with_unsorted_rows():
    """The reference's own set-up of the toy model: row ids in random order, sorted behind the wrapper."""
    c = run("system", 2, 1e-12, skip=("y_add_2",), num_nnz=5000, sorted_rows=False)
    assert bool((c.reducer_1.idx[1:] < c.reducer_1.idx[:-1]).any())


def test_system_model_float32():
    run("system", 3, 1e-5, skip=("y_add_2",), dtype=torch.float32)


@pytest.mark.parametrize("points", [900, 40000])
def test_shallow_water_runge_kutta_steps(points):
    c = run("swe", 10, 1e-10, points=points)
    assert float(c.uh.abs().max()) > 0


def float32_against_float64_yardstick(name, steps, keys, **kw):
    """Float32 results of ill-conditioned quantities (small differences of large terms) are only as
    good as float32 arithmetic allows.  The float64 model is the yardstick: the generated kernels may
    not be further from it than the same model on torch's float32 kernels."""
    def final_state(dtype, replace):
        model = MODELS[name](device="cuda", dtype=dtype, **kw)
        [compiled] = esr.compile([model], "torch")
        if replace:
            report = accelerate(compiled, prefix=name, build_if_missing=False)
            assert all(v == "replaced" for v in report.values()), report
        for _ in range(steps):
            compiled()
        torch.cuda.synchronize()
        return {k: v.detach().double() for k, v in compiled.named_parameters()}

    print(f"case model {name} {kw} float32 vs float64 yardstick", flush=True)
    truth = final_state(torch.float64, False)
    eager = final_state(torch.float32, False)
    fused = final_state(torch.float32, True)
    for k in keys:
        scale = float(truth[k].abs().max())
        err_eager = float((eager[k] - truth[k]).abs().max()) / scale
        err_fused = float((fused[k] - truth[k]).abs().max()) / scale
        assert err_fused <= 1.5 * err_eager + 1e-5, (k, err_fused, err_eager)


def test_shallow_water_float32():
    float32_against_float64_yardstick("swe", 5, ("h", "uh", "vh"))


def test_spring_mass_steps_small():
    c = run("spring", 10, 2e-5, n=8)
    assert float(c.energy) > 0


def test_spring_mass_float32_on_a_large_lattice():
    float32_against_float64_yardstick("spring", 10, ("energy", "force", "vel", "pos"), n=40)


def test_spring_mass_float64():
    run("spring", 10, 1e-10, n=10, dtype=torch.float64)


def test_mesh_components_collector_int64():
    run("swe_parts", 1, 0)


@pytest.mark.parametrize("points", [900, 90000])
def test_geometry_initializer(points):
    c = run("swe_init", 1, 1e-12, points=points)
    assert abs(float(c.area.sum()) - 1.0) < 1e-12


def test_graph_replay_of_a_model_step_matches_eager_launches():
    """One shallow-water step captured as a HIP graph and replayed gives the bits of the same launches
    issued one by one; replays are interleaved with ordinary work and synchronisations."""
    from flexspmv_amd.python_wrapper.graph_replay import capture_step
    print("case graph replay swe", flush=True)
    steps = 6

    def build():
        model = MODELS["swe"](device="cuda", points=40000)
        [compiled] = esr.compile([model], "torch")
        report = accelerate(compiled, prefix="swe", build_if_missing=False)
        assert all(v == "replaced" for v in report.values()), report
        return compiled

    eager = build()
    for _ in range(2 + steps):
        eager()
    torch.cuda.synchronize()
    want = ab_check.save_state(eager)

    replayed = build()
    replay = capture_step(replayed, warmup=2)
    scratch = torch.zeros(1 << 20, device="cuda")
    for i in range(steps):
        replay()
        scratch.add_(1.0)                     # unrelated eager work between replays
        if i % 2 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    got = ab_check.save_state(replayed)
    for k in want:
        assert torch.equal(want[k], got[k]), k
    assert float(scratch[0]) == steps


def test_graph_replay_with_an_unordered_edge_list():
    """The toy model with row ids in random order: the per-step permutation of the streamed edge tensors is
    part of the captured graph; replays equal eager steps bit for bit."""
    from flexspmv_amd.python_wrapper.graph_replay import capture_step
    print("case graph replay system unsorted", flush=True)
    steps = 4

    def build():
        model = MODELS["system"](device="cuda", num_nnz=20000, sorted_rows=False)
        [compiled] = esr.compile([model], "torch")
        report = accelerate(compiled, prefix="system", build_if_missing=False)
        assert all(v == "replaced" for v in report.values()), report
        return compiled

    eager = build()
    for _ in range(2 + steps):
        eager()
    torch.cuda.synchronize()
    want = ab_check.save_state(eager)
    replayed = build()
    replay = capture_step(replayed, warmup=2)
    for i in range(steps):
        replay()
        torch.cuda.synchronize()
    got = ab_check.save_state(replayed)
    for k in want:
        assert torch.equal(want[k], got[k]), k


def test_conjugate_gradients_on_the_fused_poisson_operator():
    """The solver loop around the fused ``A p`` / ``p . A p`` launch converges to the solution of a
    manufactured problem, and launches after the first reuse the tile table."""
    from flexspmv_amd.drivers.poisson_cg import conjugate_gradients, fused_operator
    print("case poisson cg 48^3", flush=True)
    apply, n = fused_operator(48)
    truth = torch.rand(n, dtype=torch.float64, device="cuda", generator=torch.Generator("cuda").manual_seed(1))
    b, _ = apply(truth.clone())
    b = b.clone()
    x, iterations, residual = conjugate_gradients(apply, b, tol=1e-10, maxiter=2000)
    assert residual <= 1e-10 and iterations < 400
    assert float((x - truth).abs().max()) <= 1e-8
