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


def test_system_model_float32():
    run("system", 3, 1e-5, skip=("y_add_2",), dtype=torch.float32)


@pytest.mark.parametrize("points", [900, 40000])
def test_shallow_water_runge_kutta_steps(points):
    c = run("swe", 10, 1e-10, points=points)
    assert float(c.uh.abs().max()) > 0


def test_shallow_water_float32():
    run("swe", 5, 2e-5, dtype=torch.float32)


def test_spring_mass_steps_small():
    c = run("spring", 10, 2e-5, n=8)
    assert float(c.energy) > 0


def test_spring_mass_float32_is_as_accurate_as_torch_float32():
    """On a 40^3 lattice the net force on a node is a small difference of large spring forces and
    positions reach 40: float32 itself is only good to ~1e-4 of the largest force there.  The float64
    model is the yardstick; the generated kernels may not be further from it than torch's float32."""
    steps = 10

    def final_state(dtype, replace):
        model = MODELS["spring"](device="cuda", n=40, dtype=dtype)
        [compiled] = esr.compile([model], "torch")
        if replace:
            report = accelerate(compiled, prefix="spring", build_if_missing=False)
            assert all(v == "replaced" for v in report.values()), report
        for _ in range(steps):
            compiled()
        torch.cuda.synchronize()
        return {k: v.detach().double() for k, v in compiled.named_parameters()}

    print("case model spring n=40 float32 vs float64 yardstick", flush=True)
    truth = final_state(torch.float64, False)
    eager = final_state(torch.float32, False)
    fused = final_state(torch.float32, True)
    for k in ("energy", "force", "vel", "pos"):
        scale = float(truth[k].abs().max())
        err_eager = float((eager[k] - truth[k]).abs().max()) / scale
        err_fused = float((fused[k] - truth[k]).abs().max()) / scale
        assert err_fused <= 1.5 * err_eager + 1e-5, (k, err_fused, err_eager)


def test_spring_mass_float64():
    run("spring", 10, 1e-10, n=10, dtype=torch.float64)
