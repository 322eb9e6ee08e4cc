"""HIP backend vs the CPU oracle on identical seeded inputs, through the C ABI."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu


def run_hip(tc_src, entry, inputs_np, options):
    ins = [torch.from_numpy(a).cuda() for a in inputs_np]
    ex = tc.compile(tc_src, entry, ins, options)
    outs = tc.prepare_outputs(tc_src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy() for o in outs], ex


OPTION_SETS = {
    "naive": "naive",
    "single_thread": "single_thread",
    "pointwise": "pointwise",
    "conv": "conv",
    "group_conv": "group_conv",
    "mlp": "mlp",
}

SMALL = {
    "tensordot": (W.TENSORDOT, "tensordot", [(3, 5, 7, 6, 10), (3, 7, 2, 6, 10)], 7),
    "batch_matmul": (W.BATCH_MATMUL, "batch_matmul", [(7, 26, 72), (7, 72, 26)], 72),
    "group_convolution": (W.GROUP_CONVOLUTION, "group_convolution", [(2, 3, 4, 9, 8), (3, 5, 4, 3, 3), (3, 5)], 36),
    "moments": (W.MOMENTS, "moments", [(9, 1000)], 1000),
}


@pytest.mark.parametrize("preset", sorted(OPTION_SETS))
@pytest.mark.parametrize("name", sorted(SMALL))
def test_small_shapes_all_presets(name, preset):
    src, entry, shapes, k = SMALL[name]
    print(f"case {name} preset {preset}", flush=True)
    rng = np.random.Generator(np.random.Philox(1234))
    ins = [rng.standard_normal(s, dtype=np.float32) for s in shapes]
    ref = tc_oracle.run(src, entry, ins)
    got, _ = run_hip(src, entry, ins, OPTION_SETS[preset])
    for g, r in zip(got, ref):
        assert g.shape == r.shape
        assert np.abs(g - r).max() <= W.tolerance(k, r)


@pytest.mark.parametrize("name", sorted(W.CONFIGS))
def test_configs_tuned_options(name):
    src, entry, shapes, _, k = W.CONFIGS[name]
    print(f"config {name} options {W.TUNED[name]}", flush=True)
    ins = W.make_inputs(name)
    ref = tc_oracle.run(src, entry, ins)
    got, ex = run_hip(src, entry, ins, W.TUNED[name])
    for g, r in zip(got, ref):
        assert np.abs(g - r).max() <= W.tolerance(k, r), (name, ex.launch_bounds())


@pytest.mark.parametrize("name", sorted(SMALL))
def test_indexing_bit_exact_with_integer_inputs(name):
    """Small integers make every fp32 product and sum exact, so any mis-indexing shows up as a
    non-zero integer difference regardless of summation order."""
    src, entry, shapes, _ = SMALL[name]
    if name == "moments":
        pytest.skip("divides by N: not exact in fp32")
    rng = np.random.Generator(np.random.Philox(99))
    ins = [rng.integers(-4, 5, size=s).astype(np.float32) for s in shapes]
    ref = tc_oracle.run(src, entry, ins)
    for opts in ("naive", W.TUNED["c2_tensordot"] if name == "tensordot" else "pointwise"):
        got, _ = run_hip(src, entry, ins, opts)
        for g, r in zip(got, ref):
            assert np.array_equal(g, r)
