"""The measurement probes under cudanative.jl_amd/examples, whose commands the summaries under
profiles/ give, still compile for gfx950 (device and host code; nothing is run here)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXAMPLES = os.path.join(ROOT, "cudanative.jl_amd", "examples")
PROBES = ["store_patterns.hip", "mfma_lone_wavefront.hip", "mfma_order_power.hip", "valu_issue_rate.hip"]


@pytest.mark.parametrize("name", PROBES)
def test_probe_compiles_for_gfx950(name, tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    out = tmp_path / (name + ".o")
    r = subprocess.run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++20", "-Wno-unused-result", "-c",
                        os.path.join(EXAMPLES, name), "-o", str(out)], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert out.stat().st_size > 0
