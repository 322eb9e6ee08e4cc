"""HIP backend vs the CPU oracle on the other workloads of the reference's benchmark suite
(transposed matmul, convolution, fully connected chains, look-up tables with indirect indexing,
batch and group normalisation, Kronecker products, a WaveNet layer), under plain, tiled + LDS,
thread-mapped-reduction and matrix-core mapping options."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import benchmark_tcs as B
from tests.test_benchmark_tcs import OPTION_SETS

pytestmark = pytest.mark.gpu



def chain(*lengths):
    """Effective reduction length of reductions that feed one another: each stage adds its own
    1e-5 * sqrt(K_i) (relative to the common scale), so the bound is 1e-5 * sum(sqrt(K_i)),
    written as the K whose square root that is."""
    return float(sum(np.sqrt(k) for k in lengths)) ** 2


# Reduction lengths at the test sizes of tests/benchmark_tcs.py:CASES.  Chains: the lengths of the
# reductions that feed one another.  The normalisations reduce over everything but the dimension
# they normalise per: batch norm of a 4x6x7x5 input over N*H*W = 4*7*5 per channel, the one-kernel
# group norm of a 3x4x5x6x7 input over D*H*W = 5*6*7 per (n, g).
CHAINED = {"2fcrelu": chain(48, 36), "mlp3": chain(24, 18, 10), "kronecker3": chain(5, 4, 3), "batchnorm": 4 * 7 * 5,
           "wavenet1": chain(16, 8, 8), "wavenet1_skip256": chain(8, 6, 6), "wavenet1_skip256_dilation32": chain(8, 6, 6),
           "group_normalization_single_kernel": 5 * 6 * 7}


@pytest.mark.parametrize("options", sorted(OPTION_SETS))
@pytest.mark.parametrize("name", sorted(B.CASES))
def test_parity_with_oracle(name, options):
    src, entry, _, k = B.CASES[name]
    print(f"case {name} options {options}", flush=True)
    ins_np = B.make_inputs(name)
    ref = tc_oracle.run(src, entry, ins_np)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, OPTION_SETS[options])
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    k = CHAINED.get(name, k)
    for o, r in zip(outs, ref):
        got = o.cpu().numpy()
        assert got.shape == r.shape
        scale = max(float(np.abs(r).max()), 1e-30)
        assert np.abs(got - r).max() <= 1e-5 * np.sqrt(k) * scale, (name, options, ex.launch_bounds())


@pytest.mark.parametrize("name", sorted(B.TUNED_AT_REFERENCE_SIZES))
def test_parity_at_the_reference_sizes_with_the_tuned_options(name):
    src, entry, _, k = B.CASES[name]
    print(f"case {name} at the reference's default size", flush=True)
    ins_np = B.make_inputs(name, reference_sizes=True)
    ref = tc_oracle.run(src, entry, ins_np)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, B.TUNED_AT_REFERENCE_SIZES[name])
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    # reduction lengths at these sizes (chains: see chain()); the group normalisation from given
    # means and variances reduces nothing (1), the one-kernel form and the moments reduce over
    # D*H*W = 16*48*48 elements per (n, g), respectively over a row of 36864
    k = {"tmm": 256, "matmul": 1000, "convolution": 36, "group_convolution": 36, "2fcrelu": chain(2000, 128), "mlp1": 2000, "mlp3": chain(128, 64, 32), "lut": 50,
         "c3": 1000, "2lut": 50, "group_normalization": 1,
         "moments2": 36864, "sum": 36864, "mean": 36864, "sum_squares": 36864, "var": 36864, "sum_and_squares": 36864,
         "kronecker3_1": 16, "kronecker3_2": 16, "kronecker3_3": 16,
         "group_normalization_single_kernel": 16 * 48 * 48, "kronecker3": chain(16, 16, 16),
         "wavenet1": chain(64, 32, 32), "wavenet1_skip256": chain(64, 32, 32), "wavenet1_skip256_dilation32": chain(64, 32, 32)}[name]
    for o, r in zip(outs, ref):
        got = o.cpu().numpy()
        assert got.shape == r.shape
        scale = max(float(np.abs(r).max()), 1e-30)
        assert np.abs(got - r).max() <= 1e-5 * np.sqrt(k) * scale, (name, ex.launch_bounds())


@pytest.mark.parametrize("name", sorted(B.LARGE_CONTRACTIONS) + sorted(B.OTHER_REFERENCE_SIZES))
def test_parity_of_the_large_contractions_and_the_other_reference_sizes(name):
    case, _, options, k = (B.LARGE_CONTRACTIONS if name in B.LARGE_CONTRACTIONS else B.OTHER_REFERENCE_SIZES)[name]
    src, entry, _, _ = B.CASES[case]
    print(f"case {name}", flush=True)
    ins_np = B.make_large_inputs(name)
    if name.startswith("half_"):
        # (the oracle evaluates a converted operand element by element: minutes at these sizes.  The
        # small cases of these two comprehensions pin it to this closed form, the float product of
        # the converted matrices.)
        a, b = (x.astype(np.float32) for x in ins_np)
        ref = [a @ (b.T if case == "half_tmm" else b)]
    else:
        ref = tc_oracle.run(src, entry, ins_np)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, options)
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    for o, r in zip(outs, ref):
        got = o.cpu().numpy()
        assert got.shape == r.shape
        scale = max(float(np.abs(r).max()), 1e-30)
        assert np.abs(got - r).max() <= 1e-5 * np.sqrt(k) * scale, (name, ex.launch_bounds())


def test_autotuning_the_1024_matmul_from_the_naive_options_reaches_the_stored_options():
    """A short, seeded search from the naive options ends within 15 % of the stored options of the
    1024 x 1024 x 1024 product (reduction tiles staged through two LDS copies, loads of several
    tiles in flight), and its winner computes the oracle's values."""
    case, _, stored, k = B.LARGE_CONTRACTIONS["matmul_1024"]
    src, entry, _, _ = B.CASES[case]
    ins_np = B.make_large_inputs("matmul_1024")
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    outs = tc.prepare_outputs(src, entry, ins)

    def kernel_us(options):
        ex = tc.compile(src, entry, ins, options)
        for _ in range(20):
            tc.profile_repeated(ex, ins, outs, 100)
        return min(tc.profile_repeated(ex, ins, outs, 50) / 50 for _ in range(5))

    best = tc.autotune(src, entry, ins, "naive", outputs=outs, generations=3, pop_size=30, threads=16, seed=1)
    t_stored, t_tuned = kernel_us(stored), kernel_us(best[0])
    print(f"matmul_1024: stored {t_stored:.1f} us, tuned from naive {t_tuned:.1f} us with {best[0]}", flush=True)
    assert t_tuned <= 1.15 * t_stored
    ex = tc.compile(src, entry, ins, best[0])
    outs[0].fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    ref = tc_oracle.run(src, entry, ins_np)[0]
    scale = max(float(np.abs(ref).max()), 1e-30)
    assert np.abs(outs[0].cpu().numpy() - ref).max() <= 1e-5 * np.sqrt(k) * scale


def test_lookup_indices_are_exact():
    """Indirect indexing with integer-valued tables: sums are exact, any wrong row shows."""
    rng = np.random.Generator(np.random.Philox(5))
    lut = rng.integers(-8, 9, size=(50, 24)).astype(np.float32)
    idx = rng.integers(0, 50, size=(9, 7)).astype(np.int32)
    ref = tc_oracle.run(B.LUT, "lut", [lut, idx])[0]
    ins = [torch.from_numpy(lut).cuda(), torch.from_numpy(idx).cuda()]
    for options in ("naive", OPTION_SETS["tiled_lds"], OPTION_SETS["library_reductions"]):
        ex = tc.compile(B.LUT, "lut", ins, options)
        (out,) = tc.prepare_outputs(B.LUT, "lut", ins)
        tc.run(ex, ins, [out])
        assert np.array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("options", sorted(OPTION_SETS))
@pytest.mark.parametrize("name", ["2fcrelu", "mlp1", "mlp3", "kronecker3", "matmul", "tmm_odd", "convolution"])
def test_chains_and_contractions_are_exact_on_small_integers(name, options):
    """Inputs in {-2..2}: every product, partial sum and intermediate result is an integer far
    below 2^24, so any order of summation gives the same bits and a dropped or doubled partial
    result cannot hide inside a tolerance."""
    src, entry, _, _ = B.CASES[name]
    rng = np.random.Generator(np.random.Philox(77))
    ins_np = [rng.integers(-2, 3, size=a.shape).astype(a.dtype) for a in B.make_inputs(name)]
    ref = tc_oracle.run(src, entry, ins_np)
    assert all(np.abs(r).max() < 2 ** 22 and np.array_equal(r, np.round(r)) for r in ref)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    ex = tc.compile(src, entry, ins, OPTION_SETS[options])
    outs = tc.prepare_outputs(src, entry, ins)
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    for o, r in zip(outs, ref):
        assert np.array_equal(o.cpu().numpy(), r), (name, options, ex.launch_bounds())
