"""The C++ ATen-level surface (tc::aten::compile<HipBackend>, prepareOutputs, profile,
ATenAutotuner<HipBackend, GeneticSearch>, the options-cache file helpers) exercised by the
reference's examples on the HIP backend: tc/examples/tensordot.cc:37-90,
tc/examples/blockdiagperm.cc:45-152 and tc/examples/group_normalization.cc:45-140."""
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


def test_blockdiagperm_example_reinforces_its_cache_file(tmp_path):
    """Two comprehensions tuned one after the other; the first run starts from the naive options
    and leaves its best options in the cache file, the second run starts from them
    (loadTopKFromCacheFile / appendTopKToCacheFile, tc/autotuner/options_cache-inl.h:337-370)."""
    exe = os.path.join(ROOT, "examples", "blockdiagperm")
    if not os.path.exists(exe):
        pytest.fail("examples/blockdiagperm not built (make -C tensorcomprehensions_amd/csrc example)")
    cache = str(tmp_path / "blockdiagperm.options")
    starts = []
    for _ in range(2):
        out = subprocess.run([exe, "2", "8", cache], capture_output=True, text=True, timeout=300)
        print(out.stdout[-2000:], out.stderr[-2000:], flush=True)
        assert out.returncode == 0 and out.stdout.count("ran in:") == 2
        diff = float(re.search(r"vs at::einsum: ([0-9.e+-]+)", out.stdout).group(1))
        assert diff <= 1e-5 * 8 * 50      # 1e-5 * sqrt(50) * max|ref| (inputs in [0,1): ref <= 50)
        assert "permutation equals at::index_select: yes" in out.stdout
        starts.append(re.search(r"starts from (the naive|cached) options", out.stdout).group(1))
        assert os.path.getsize(cache) > 0
    assert starts == ["the naive", "cached"]


@pytest.mark.parametrize("start", ["naive", "best"])
def test_group_normalization_example_matches_group_norm(start):
    """One comprehension with two reductions and the normalising statement, tuned from the naive
    options or from options written with the fluent C++ builder
    (tc/examples/group_normalization.cc:45-63), against at::group_norm."""
    exe = os.path.join(ROOT, "examples", "group_normalization")
    if not os.path.exists(exe):
        pytest.fail("examples/group_normalization not built (make -C tensorcomprehensions_amd/csrc example)")
    out = subprocess.run([exe, "2", "8", start], capture_output=True, text=True, timeout=300)
    print(out.stdout[-2500:], out.stderr[-2000:], flush=True)
    assert out.returncode == 0 and out.stdout.count("ran in:") == 1
    diff = float(re.search(r"vs at::group_norm: ([0-9.e+-]+)", out.stdout).group(1))
    # sums of 36 864 terms, a variance from a difference of two of them, outputs of a few units
    assert diff <= 1e-4
    assert "tc::HipMappingOptions::makeNaiveMappingOptions()" in out.stdout
    if start == "best":
        microseconds = float(re.search(r"ran in: ([0-9.]+)us", out.stdout).group(1))
        assert microseconds < 80           # the builder-written options or better (they measure 47 us)
