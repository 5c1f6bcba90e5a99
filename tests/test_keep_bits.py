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


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc")
def test_lds_tile_layout_is_free_of_bank_conflicts(tmp_path):
    """The swizzle of the LDS tiles (tile_io.hpp) under the kernels' two read patterns, row reads of 16 bytes and
    transposing reads of 8 bytes per lane: no LDS cycle puts two different addresses on one of the 64 banks
    (a swizzle that did cost every transposing read a second cycle; the counters showed it as 25-32 % conflict
    cycles)."""
    exe = tmp_path / "lds_banks_check"
    cmd = [HIPCC, "--cuda-host-only", "-x", "hip", "-O1", "-std=c++17", "-Wno-unused-command-line-argument",
           f"-I{ROOT}/include", f"-I{ROOT}/flex_attention_tpu_amd/csrc", os.path.join(ROOT, "tests", "host", "lds_banks_check.cpp"),
           "-o", str(exe)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert r.stdout.startswith("ok ")
