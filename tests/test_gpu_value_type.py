"""The device value type (flexspmv_amd/csrc/flex_tensor.hpp) against the reference-bit fixture.

tests/golden/tensor_kat.json holds the known-answer cases evaluated by the reference's own
data_struct_shared.cuh on a CPU.  The same case list is compiled against the shipped device header
with the flags of the shipped libraries and run on the GPU (tests/device_kat).  Every case whose
result IEEE-754 fixes (single correctly rounded operations, selections, comparisons, integer
arithmetic, the divide-by-zero guards, sign(NaN), int64 pow / exp through double) must give the
reference's bits (a NaN result only has to be a NaN: its sign bit differs between the two machines).  pow / exp come from another math library than the CPU's and a sum of products may
be contracted into fused multiply-adds, so the cases that contain them are held to 2 units in the
last place instead (far inside the 1e-5 / 1e-12 the path is allowed).
"""
import json
import os
import struct
import subprocess

import numpy as np
import pytest

from tests.device_kat.build_device_kat import BINARY, case_labels

pytestmark = pytest.mark.gpu

# cases that evaluate pow / exp in floating point, or a multiply-add chain
ULP_CASES = {"pow_same", "pow_scalar", "scalar_pow", "mixed_int_right_pow", "bcast_pow_6_3", "exp",
             "l2norm_6", "l2norm_3", "chain_spring"}
MAX_ULP = 2


def _ulps(a_hex, b_hex, kind):
    if a_hex == b_hex:
        return 0
    fmt, ifmt = ("<f", "<I") if kind == "f32" else ("<d", "<Q")
    a = struct.unpack(fmt, struct.pack(ifmt, int(a_hex, 16)))[0]
    b = struct.unpack(fmt, struct.pack(ifmt, int(b_hex, 16)))[0]
    if np.isnan(a) and np.isnan(b):
        return 0
    if np.isnan(a) or np.isnan(b) or np.isinf(a) or np.isinf(b) or (a < 0) != (b < 0):
        return 1 << 30
    return abs(int(a_hex, 16) - int(b_hex, 16))


def test_device_value_type_gives_the_reference_bits(golden_dir):
    assert os.path.exists(BINARY), "tests/device_kat is not built (run __graft_entry__.build())"
    with open(os.path.join(golden_dir, "tensor_kat.json")) as f:
        gold = json.load(f)["lines"]
    text = subprocess.run([BINARY], stdout=subprocess.PIPE, check=True, text=True, timeout=120).stdout
    got = {}
    for line in text.splitlines():
        parts = line.split(" ", 2)
        got[parts[0] + " " + parts[1]] = parts[2].strip() if len(parts) > 2 else ""
    expected_keys = {f"{l} {k}" for l in case_labels("tensor_kat_cases.inc") for k in ("f32", "f64")}
    expected_keys |= {f"{l} i64" for l in case_labels("tensor_kat_cases_i64.inc")}
    assert set(got) == expected_keys
    exact = loose = 0
    for key in sorted(got):
        label, kind = key.split(" ")
        g, r = got[key].split(), gold[key].split()
        assert len(g) == len(r), key
        if kind != "i64" and label in ULP_CASES:
            worst = max(_ulps(a, b, kind) for a, b in zip(g, r))
            assert worst <= MAX_ULP, f"{key}: {worst} ulp from the reference ({got[key]} vs {gold[key]})"
            loose += 1
        else:
            # bit for bit, except that a NaN is a NaN: its sign and payload are not fixed by IEEE-754
            # (0 / 0 comes out as 0xffc00000 on the CPU and 0x7fc00000 on the GPU)
            same = all(a == b or (kind != "i64" and _ulps(a, b, kind) == 0) for a, b in zip(g, r))
            assert same, f"{key}: device {got[key]} != reference {gold[key]}"
            exact += 1
    print(f"{exact} cases bit-identical, {loose} cases within {MAX_ULP} ulp")
    assert exact >= 120
