"""The C++ ATen-level surface (tc::aten::compile<HipBackend>, prepareOutputs, profile,
ATenAutotuner<HipBackend, GeneticSearch>) exercised by the port of the reference's introductory
example, tc/examples/tensordot.cc:37-90."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "examples", "tensordot")


def test_tensordot_example_runs_and_matches_einsum():
    if not os.path.exists(EXE):
        pytest.fail("examples/tensordot not built (make -C tensorcomprehensions_amd/csrc example)")
    out = subprocess.run([EXE, "2", "8"], capture_output=True, text=True, timeout=300)
    print(out.stdout[-2000:], out.stderr[-2000:], flush=True)
    assert out.returncode == 0
    assert out.stdout.count("ran in:") == 3
    diff = float(re.search(r"max \|diff\| vs at::einsum: ([0-9.e+-]+)", out.stdout).group(1))
    assert diff <= 1e-5 * 4 * 16          # 1e-5 * sqrt(16) * max|ref| (inputs in [0,1): ref <= 16)
    assert "tc::HipMappingOptions::makeNaiveMappingOptions()" in out.stdout
