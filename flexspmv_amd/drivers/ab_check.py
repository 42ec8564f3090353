"""Original-versus-replaced check of a whole model, the flow of the reference's A/B driver
(test_full/easier_full.py:484-578): trace, run the original N steps, generate and build the library of
every fused sub-module, replace them, restore the initial state, run N steps again, compare."""
from __future__ import annotations

from typing import Callable, Dict

import torch

from .. import frontend as esr
from ..python_wrapper.accelerate import accelerate


def save_state(model) -> Dict[str, torch.Tensor]:
    return {k: v.detach().clone() for k, v in model.named_parameters()}


def restore_state(model, state: Dict[str, torch.Tensor]) -> None:
    with torch.no_grad():
        for k, v in model.named_parameters():
            v.copy_(state[k])


def compare_states(original: Dict[str, torch.Tensor], replaced: Dict[str, torch.Tensor], tolerance: float):
    """{name: max |a-b| / max(|a|, tiny)} and whether all are within ``tolerance`` (integers: exact)."""
    worst, ok = {}, True
    for k, a in original.items():
        b = replaced[k]
        if not a.dtype.is_floating_point:
            same = bool(torch.equal(a, b))
            worst[k] = 0.0 if same else float("inf")
            ok = ok and same
            continue
        scale = max(float(a.abs().max()), 1e-300) if a.numel() else 1.0
        err = float((a.double() - b.double()).abs().max()) / scale if a.numel() else 0.0
        worst[k] = err
        ok = ok and err <= tolerance
    return worst, ok


def run_ab(make_model: Callable[[], torch.nn.Module], steps: int = 10, tolerance: float = 1e-10,
           prefix: str = "model", build_if_missing: bool = True, verbose: bool = False):
    """Returns (passed, report of accelerate(), per-tensor relative differences)."""
    model = make_model()
    [compiled] = esr.compile([model], "torch")
    initial = save_state(compiled)
    for _ in range(steps):
        compiled()
    original_final = save_state(compiled)

    report = accelerate(compiled, prefix=prefix, build_if_missing=build_if_missing)
    restore_state(compiled, initial)
    for _ in range(steps):
        compiled()
    if torch.cuda.is_available():
        torch.cuda.synchronize()
    replaced_final = save_state(compiled)
    worst, ok = compare_states(original_final, replaced_final, tolerance)
    if verbose:
        for k, v in report.items():
            print(f"  {k}: {v}")
        for k, v in worst.items():
            print(f"  {k}: max rel diff {v:.3e}")
        print("PASSED" if ok else "FAILED")
    return ok, report, worst


def main(argv=None) -> int:
    """``python -m flexspmv_amd.drivers.ab_check swe --points 200000 --steps 10``: the check above on
    one of the driver models, with the time per step before and after the replacement."""
    import argparse
    import time

    from .prebuilt import MODELS

    ap = argparse.ArgumentParser(description=main.__doc__)
    ap.add_argument("model", choices=sorted(MODELS))
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--tolerance", type=float, default=1e-10)
    ap.add_argument("--device", default="cuda")
    ap.add_argument("--points", type=int, default=None, help="mesh points of the shallow-water model")
    ap.add_argument("--n", type=int, default=None, help="lattice edge of the spring-mass model")
    ap.add_argument("--dt", type=float, default=None, help="time step of the shallow-water model")
    ap.add_argument("--mesh", default=None, help="shallow-water model: read the mesh from this .npz / .hdf5 file "
                                                 "(shallow_water.save_mesh writes one)")
    a = ap.parse_args(argv)
    kw = {k: v for k, v in (("points", a.points), ("n", a.n), ("dt", a.dt), ("mesh", a.mesh)) if v is not None}

    def sync():
        if a.device.startswith("cuda"):
            torch.cuda.synchronize()

    model = MODELS[a.model](device=a.device, **kw)
    [compiled] = esr.compile([model], "torch")
    initial = save_state(compiled)
    compiled()
    restore_state(compiled, initial)
    sync()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        compiled()
    sync()
    t_original = (time.perf_counter() - t0) / a.steps
    original_final = save_state(compiled)
    report = accelerate(compiled, prefix=a.model)
    restore_state(compiled, initial)
    compiled()
    restore_state(compiled, initial)
    sync()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        compiled()
    sync()
    t_replaced = (time.perf_counter() - t0) / a.steps
    worst, ok = compare_states(original_final, save_state(compiled), a.tolerance)
    t_graph = None
    if a.device.startswith("cuda") and all(v == "replaced" for v in report.values()):
        from ..python_wrapper.graph_replay import capture_step
        replay = capture_step(compiled)
        replay()
        sync()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            replay()
        sync()
        t_graph = (time.perf_counter() - t0) / a.steps
    for k, v in report.items():
        print(f"  {k}: {v}")
    for k, v in worst.items():
        print(f"  {k}: max rel diff {v:.3e}")
    print(f"  ms per step: torch sub-modules {t_original * 1e3:.3f}, generated libraries {t_replaced * 1e3:.3f} "
          f"({t_original / t_replaced:.2f}x)"
          + (f", the same replayed as one HIP graph {t_graph * 1e3:.3f} ({t_original / t_graph:.2f}x)" if t_graph else ""))
    print("PASSED" if ok else "FAILED")
    return 0 if ok else 1


if __name__ == "__main__":
    raise SystemExit(main())
