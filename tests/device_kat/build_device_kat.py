"""Build tests/device_kat/tensor_kat_device.hip (the value-type known-answer cases, run on the GPU
against the shipped device header) into tests/device_kat/_build/."""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

SOURCE = os.path.join(HERE, "tensor_kat_device.hip")
BINARY = os.path.join(HERE, "_build", "tensor_kat_device")
ORACLE_DIR = os.path.join(ROOT, "oracle")


def case_labels(inc_file: str, skip_member_compare: bool = True):
    """Labels of a case list in file order (cases inside ``#ifndef KAT_NO_MEMBER_COMPARE`` skipped)."""
    labels, skipping = [], False
    with open(os.path.join(ORACLE_DIR, inc_file)) as f:
        for line in f:
            if line.startswith("#ifndef KAT_NO_MEMBER_COMPARE"):
                skipping = skip_member_compare
            elif line.startswith("#endif"):
                skipping = False
            m = re.match(r'\s*KAT_EMIT(?:_SCALAR)?\("([a-z0-9_]+)"', line)
            if m and not skipping:
                labels.append(m.group(1))
    return labels


def build(force: bool = False) -> str:
    from flexspmv_amd.build import CSRC_DIR, HIPCC_FLAGS, hipcc_path
    deps = [SOURCE, os.path.join(CSRC_DIR, "flex_tensor.hpp"), os.path.join(ORACLE_DIR, "tensor_kat_cases.inc"),
            os.path.join(ORACLE_DIR, "tensor_kat_cases_i64.inc")]
    if not force and os.path.exists(BINARY) and all(os.path.getmtime(BINARY) >= os.path.getmtime(d) for d in deps):
        return BINARY
    os.makedirs(os.path.dirname(BINARY), exist_ok=True)
    quoted = lambda labels: ",".join('"%s"' % l for l in labels)
    # the flags of the shipped libraries (minus -shared / -fPIC): same contraction, same math library
    flags = [f for f in HIPCC_FLAGS if f not in ("-shared", "-fPIC")]
    cmd = [hipcc_path(), *flags, f"-I{CSRC_DIR}", f"-I{ORACLE_DIR}",
           f"-DKAT_FLOAT_LABELS={quoted(case_labels('tensor_kat_cases.inc'))}",
           f"-DKAT_INT_LABELS={quoted(case_labels('tensor_kat_cases_i64.inc'))}", SOURCE, "-o", BINARY]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {SOURCE} failed:\n{' '.join(cmd)}\n{proc.stdout}")
    return BINARY


if __name__ == "__main__":
    print(build(force=True))
