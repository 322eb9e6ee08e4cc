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
    rng = np.random.Generator(np.random.Philox(99))
    ins = [rng.integers(-4, 5, size=s).astype(np.float32) for s in shapes]
    variants = ("naive", W.TUNED["c2_tensordot"] if name == "tensordot" else "pointwise")
    if name == "moments":
        # Rows of 1024 = 2^10 small integers whose sum is a multiple of 1024: X/N, the mean (an
        # integer), (X - mean)^2 / N and every partial sum of either reduction are exact in fp32.
        half = rng.integers(-4, 5, size=(9, 512))
        rows = np.concatenate([half, -rng.permuted(half, axis=1)], axis=1) + rng.integers(-2, 3, size=(9, 1))
        ins = [rng.permuted(rows, axis=1).astype(np.float32)]
        assert np.all(ins[0].sum(1) % 1024 == 0)
        variants = ("naive", "naive;tile=1;mapToThreads=256;mapToBlocks=9;matchLibraryCalls=1;unroll=4;vectorWidth=4;usePrivateMemory=1")
    ref = tc_oracle.run(src, entry, ins)
    if name == "moments":
        assert np.array_equal(ref[0], ins[0].mean(1, dtype=np.float64).astype(np.float32))
        assert np.array_equal(ref[1], ins[0].var(1, dtype=np.float64).astype(np.float32))
    for opts in variants:
        got, _ = run_hip(src, entry, ins, opts)
        for g, r in zip(got, ref):
            assert np.array_equal(g, r)
