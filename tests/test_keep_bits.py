"""The partial-tile keep bits of the generated-stream kernels (fa_common.hpp: closed forms for causal /
window masks, element loop otherwise) against the element-wise predicate, on the CPU: the header's
integer code is compiled for the host and run over random strips."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
def test_keep_bits_closed_forms_match_the_predicate(tmp_path):
    exe = tmp_path / "keep_bits_check"
    cmd = [HIPCC, "--cuda-host-only", "-x", "hip", "-O1", "-std=c++17", "-Wno-unused-command-line-argument",
           f"-I{ROOT}/include", f"-I{ROOT}/flex_attention_tpu_amd/csrc", os.path.join(ROOT, "tests", "host", "keep_bits_check.cpp"),
           "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert r.stdout.startswith("ok ")
