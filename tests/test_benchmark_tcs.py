"""The other workloads of the reference's benchmark suite (tests/benchmark_tcs.py): the oracle is
pinned against the library routines the reference's own benchmarks check with (at::mm, conv2d,
relu(addmm), embedding sums, group norm; tc/benchmarks/*.cc), and every case must map and JIT for
gfx950 under several mapping options (hipRTC needs no GPU)."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import benchmark_tcs as B

OPTION_SETS = {
    "naive": "naive",
    "tiled_lds": "naive;tile=4,16,8;mapToThreads=16,4;mapToBlocks=64,64;useSharedMemory=1;unroll=16",
    "library_reductions": "naive;tile=1,1;mapToThreads=64;mapToBlocks=128,128;matchLibraryCalls=1;unroll=4",
    "matrix_cores": "naive;tile=32,32,0;mapToThreads=64,4;mapToBlocks=64,64;useMfma=1;useSharedMemory=1",
}


def f64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


def close(got, want, k):
    want = want.numpy() if isinstance(want, torch.Tensor) else want
    scale = max(1.0, float(np.abs(want).max()))
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= 1e-5 * np.sqrt(k) * scale


def test_oracle_matches_library_routines():
    ins = B.make_inputs("tmm")
    close(tc_oracle.run(B.TMM, "tmm", ins)[0], f64(ins[0]) @ f64(ins[1]).T, 256)
    ins = B.make_inputs("matmul")
    close(tc_oracle.run(B.MATMUL, "matmul", ins)[0], f64(ins[0]) @ f64(ins[1]), 60)
    ins = B.make_inputs("convolution")
    ref = torch.nn.functional.conv2d(f64(ins[0]), f64(ins[1]), f64(ins[2]))
    close(tc_oracle.run(B.CONVOLUTION, "convolution", ins)[0], ref, 36)
    I, Wg, Bg = B.make_inputs("group_convolution")
    ref = torch.nn.functional.conv2d(f64(I).reshape(2, 12, 10, 9), f64(Wg).reshape(15, 4, 3, 3), f64(Bg).reshape(15), groups=3)
    close(tc_oracle.run(B.GROUP_CONVOLUTION, "group_convolution", [I, Wg, Bg])[0], ref.reshape(2, 3, 5, 8, 7), 36)
    I, W1, B1, W2, B2 = B.make_inputs("2fcrelu")
    o1 = torch.relu(f64(I) @ f64(W1).T + f64(B1))
    o2 = torch.relu(o1 @ f64(W2).T + f64(B2))
    got = tc_oracle.run(B.FCRELU2, "func_2fcrelu", [I, W1, B1, W2, B2])
    close(got[0], o1, 48)
    close(got[1], o2, 48 * 36)
    I, W1, B1 = B.make_inputs("mlp1")
    close(tc_oracle.run(B.MLP1, "mlp1", [I, W1, B1])[0], torch.relu(f64(I) @ f64(W1) + f64(B1)), 48)
    ins = B.make_inputs("mlp3")
    I, W2, B2, W3, B3, W4, B4 = [f64(a) for a in ins]
    o2 = torch.relu(I @ W2.T + B2)
    o3 = torch.relu(o2 @ W3.T + B3)
    o4 = torch.relu(o3 @ W4.T + B4)
    for got, want, k in zip(tc_oracle.run(B.MLP3, "mlp3", ins), (o2, o3, o4), (24, 24 * 18, 24 * 18 * 10)):
        close(got, want, k)
    lut, idx = B.make_inputs("lut")
    close(tc_oracle.run(B.LUT, "lut", [lut, idx])[0], f64(lut)[torch.from_numpy(idx).long()].sum(1), 7)
    ins = B.make_inputs("c3")
    close(tc_oracle.run(B.C3, "_C3", ins)[0], f64(ins[0]) @ f64(ins[1]).T, 48)
    lut1, idx1, lut2, idx2 = B.make_inputs("2lut")
    got = tc_oracle.run(B.LUT2, "func_2lut", [lut1, idx1, lut2, idx2])
    close(got[0], f64(lut1)[torch.from_numpy(idx1).long()].sum(1), 7)
    close(got[1], f64(lut2)[torch.from_numpy(idx2).long()].sum(1), 5)
    I, gamma, beta, mean, var = B.make_inputs("group_normalization")
    ref = (f64(gamma)[None, :, :, None, None] * (f64(I) - f64(mean)[:, :, None, None, None])
           / torch.sqrt(f64(var)[:, :, None, None, None] + float(np.float32(1e-5))) + f64(beta)[None, :, :, None, None])
    close(tc_oracle.run(B.GROUP_NORMALIZATION, "group_normalization", [I, gamma, beta, mean, var])[0], ref, 1)
    X, = B.make_inputs("moments2")
    mean, var = tc_oracle.run(B.MOMENTS2, "moments2_2D_1D", [X])
    close(mean, f64(X).mean(1), 500)
    close(var, f64(X).var(1, unbiased=False), 500)
    I, gamma, beta = B.make_inputs("group_normalization_single_kernel")
    ref = torch.nn.functional.group_norm(f64(I).reshape(3, 20, 6, 7), 4, eps=1e-5).reshape(3, 4, 5, 6, 7)
    ref = ref * f64(gamma)[None, :, :, None, None] + f64(beta)[None, :, :, None, None]
    got = tc_oracle.run(B.GROUP_NORMALIZATION_SINGLE_KERNEL, "group_normalization_single_kernel", [I, gamma, beta])
    close(got[0], ref, 210)
    close(got[1], f64(I).sum((2, 3, 4)), 210)
    W0, W1k, W2k, X = B.make_inputs("kronecker3")
    ref = torch.einsum("mabc,xa,yb,zc->mxyz", f64(X), f64(W0), f64(W1k), f64(W2k))
    close(tc_oracle.run(B.KRONECKER3, "Kronecker3Full", [W0, W1k, W2k, X])[0], ref, 60)


def test_oracle_batchnorm_and_wavenet_closed_forms():
    momentum, eps, I, rMeanIn, rVarIn = B.make_inputs("batchnorm")
    out = dict(zip(["O", "rMeanOut", "rVarOut", "mean", "centered", "variance", "expectedVariance", "normalizedOut"],
                   tc_oracle.run(B.BATCHNORM, "spatialBatchNorm", [momentum, eps, I, rMeanIn, rVarIn])))
    x = f64(I)
    mean = x.mean((0, 2, 3))
    rmean = (1 - 0.1) * f64(rMeanIn) + float(np.float32(0.1)) * mean
    centered = x - rmean[None, :, None, None]
    ev = (centered * centered + float(np.float32(1e-5))).mean((0, 2, 3))
    rvar = 1.0 / torch.sqrt((1 - 0.1) * f64(rVarIn) + float(np.float32(0.1)) * ev)
    close(out["mean"], mean, 140)
    close(out["rMeanOut"], rmean, 140)
    close(out["expectedVariance"], ev, 140)
    close(out["rVarOut"], rvar, 140)
    close(out["O"], centered * rvar[None, :, None, None], 140)
    assert np.array_equal(out["O"], out["normalizedOut"])
    ins = B.make_inputs("wavenet1")
    data, fw, fb, gw, gb, rw, rb, sw, sb, dil = [f64(a) for a in ins]
    shifted = torch.zeros_like(data)
    shifted[:, :, 2:] = data[:, :, :-2]                  # DILATION_FACTOR = extent of `Dilation` = 2
    filt = fb[None, :, None] + torch.einsum("bcr,dc->bdr", data, fw[:, :, 1]) + torch.einsum("bcr,dc->bdr", shifted, fw[:, :, 0])
    gate = gb[None, :, None] + torch.einsum("bcr,dc->bdr", data, gw[:, :, 1]) + torch.einsum("bcr,dc->bdr", shifted, gw[:, :, 0])
    nonlin = torch.tanh(filt) * torch.sigmoid(gate)
    res = data + rb[None, :, None] + torch.einsum("bdr,cd->bcr", nonlin, rw)
    skip = torch.einsum("bdr,sd->bsr", nonlin, sw) + sb[None, :, None]
    got = tc_oracle.run(B.WAVENET1, "wavenet1", ins)
    for g, want in zip(got, [filt, gate, nonlin, res, skip]):
        close(g, want, 16)


@pytest.mark.parametrize("options", sorted(OPTION_SETS))
@pytest.mark.parametrize("name", sorted(B.CASES))
def test_every_case_maps_and_compiles_for_gfx950(name, options):
    src, entry, _, _ = B.CASES[name]
    shapes = [tc.ShapeOnly(a.shape, str(a.dtype)) for a in B.make_inputs(name)]
    ex = tc.compile(src, entry, shapes, OPTION_SETS[options])
    assert ex.num_kernels >= 1 and "__global__" in ex.compiled_source


@pytest.mark.parametrize("name", sorted(B.TUNED_AT_REFERENCE_SIZES))
def test_tuned_options_compile_at_the_reference_sizes(name):
    """The stored options map and compile (hipRTC, gfx950) at the reference's default sizes: the
    thread block fits the device, LDS stays within 160 KB, every kernel has a launch."""
    src, entry, _, _ = B.CASES[name]
    shapes = [tc.ShapeOnly(s[1], "int32" if s[0] == "int" else "float32") if isinstance(s[0], str) else tc.ShapeOnly(s)
              for s in B.REFERENCE_SIZES[name]]
    ex = tc.compile(src, entry, shapes, B.TUNED_AT_REFERENCE_SIZES[name])
    assert ex.num_kernels >= 1 and ex.lds_bytes() <= 160 * 1024
    for k in range(ex.num_kernels):
        grid, block = ex.launch_bounds(k)
        assert 1 <= block[0] * block[1] * block[2] <= 1024 and min(grid) >= 1


def test_oracle_products_of_converted_halves_are_float_products():
    """`float(A) * float(B)` over float16 operands: the oracle's result is the float matrix product
    of the converted matrices - exactly on small integers, within a float sum on deviates (the
    closed form the GPU test uses at sizes where the oracle's element-wise evaluation takes minutes)."""
    rng = np.random.Generator(np.random.Philox(5))
    for name, transposed in (("half_matmul", False), ("half_tmm", True)):
        src, entry, _, k = B.CASES[name]
        shapes = [spec[1] for spec in B.CASES[name][2]]
        ints = [rng.integers(-4, 5, size=s).astype(np.float16) for s in shapes]
        (got,) = tc_oracle.run(src, entry, ints)
        a, b = (x.astype(np.float32) for x in ints)
        assert got.dtype == np.float32 and np.array_equal(got, a @ (b.T if transposed else b))
        deviates = B.make_inputs(name)
        assert all(x.dtype == np.float16 for x in deviates)
        (got,) = tc_oracle.run(src, entry, deviates)
        a, b = (x.astype(np.float64) for x in deviates)
        exact = a @ (b.T if transposed else b)
        assert np.abs(got - exact).max() <= 1e-6 * np.sqrt(k) * np.abs(exact).max()
