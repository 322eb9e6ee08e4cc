"""Seeded random mapping options (the space the genetic search draws from) on small shapes of the
four workload families and on multi-statement comprehensions of the reference's benchmark suite
(chained matmuls with epilogues, batch normalisation, Kronecker products, the WaveNet layer with
its guarded accesses): whatever the tuner can pick must compute the right values, not only the
hand-picked presets.  Options the mapper refuses (TcError at compile time) are skipped; the
number of accepted sets is asserted so that the test cannot pass vacuously."""
import random

import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import benchmark_tcs as B
from tests import workloads as W

pytestmark = pytest.mark.gpu

SHAPES = {
    "tensordot": (W.TENSORDOT, "tensordot", [(3, 10, 6, 7, 12), (3, 6, 2, 7, 12)], 6, 5),
    "batch_matmul": (W.BATCH_MATMUL, "batch_matmul", [(5, 26, 40), (5, 40, 19)], 40, 3),
    "group_convolution": (W.GROUP_CONVOLUTION, "group_convolution", [(2, 3, 4, 10, 9), (3, 6, 4, 3, 3), (3, 6)], 36, 5),
    "moments": (W.MOMENTS, "moments", [(11, 700)], 700, 2),
}
SUITE = ["2fcrelu", "batchnorm", "kronecker3", "wavenet1"]
SIZES = [1, 2, 3, 4, 5, 7, 8, 13, 16, 32, 64, 128]


def random_options(rng, band):
    tile = [rng.choice(SIZES + [0, 0]) for _ in range(rng.randint(1, band + 1))]
    threads = [rng.choice([1, 2, 4, 7, 8, 16, 32, 64, 128, 256])]
    for _ in range(rng.randint(0, 2)):
        threads.append(rng.choice([1, 2, 3, 4, 8, 16]))
    while np.prod(threads) > 1024:
        threads.pop()
    blocks = [rng.choice([1, 2, 3, 8, 16, 64, 256]) for _ in range(rng.randint(1, 3))]
    parts = ["naive", "tile=" + ",".join(map(str, tile)), "mapToThreads=" + ",".join(map(str, threads)),
             "mapToBlocks=" + ",".join(map(str, blocks)), f"unroll={rng.choice([1, 2, 4, 8, 16, 32, 64, 128, 256])}"]
    for flag in ("useSharedMemory", "usePrivateMemory", "unrollCopyShared", "matchLibraryCalls", "useReadOnlyCache",
                 "collapseContiguous", "useMfma", "prefetchShared", "tileImperfectlyNested"):
        parts.append(f"{flag}={rng.randint(0, 1)}")
    parts.append(f"vectorWidth={rng.choice([1, 1, 2, 4])}")
    parts.append(f"outerScheduleFusionStrategy={rng.choice(['Max', 'Preserve3Coincident', 'Min'])}")
    parts.append(f"intraTileScheduleFusionStrategy={rng.choice(['Max', 'Preserve3Coincident', 'Min'])}")
    if rng.random() < 0.25:
        parts.append(f"reductionBlocks={rng.choice([2, 3, 4, 8, 16])}")
    return ";".join(parts)


@pytest.mark.parametrize("name", sorted(SHAPES) + SUITE)
def test_random_option_sets_compute_the_oracle_values(name):
    if name in SHAPES:
        src, entry, shapes, k, band = SHAPES[name]
        data = np.random.Generator(np.random.Philox(31))
        ins_np = [data.standard_normal(s, dtype=np.float32) for s in shapes]
    else:
        from tests.test_gpu_benchmark_tcs import CHAINED
        src, entry, _, k = B.CASES[name]
        k, band = CHAINED.get(name, k), 4
        ins_np = B.make_inputs(name)
    ref = tc_oracle.run(src, entry, ins_np)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    rng = random.Random(sum(map(ord, name)) + 17)
    accepted = 0
    for trial in range(60):
        options = random_options(rng, band)
        try:
            ex = tc.compile(src, entry, ins, options)
        except tc.TcError:
            continue
        accepted += 1
        print(f"{name} trial {trial}: {options} {ex.launch_bounds()}", flush=True)
        outs = tc.prepare_outputs(src, entry, ins)
        for o in outs:
            o.fill_(float("nan"))
        tc.run(ex, ins, outs)
        torch.cuda.synchronize()
        for o, r in zip(outs, ref):
            err = np.abs(o.cpu().numpy() - r).max()
            # chained reductions: intermediate results may be smaller than their operands
            bound = W.tolerance(k, r) if name in SHAPES else 1e-5 * np.sqrt(k) * max(1.0, float(np.abs(r).max()))
            assert err <= bound, (name, trial, options, ex.launch_bounds(), err)
    assert accepted >= 30
