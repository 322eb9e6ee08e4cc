"""Executor contract through the C ABI on the device: checked run errors, profile, unchecked run,
clearing, strides, repeated runs with different base pointers, the autotuner."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle
from tests import workloads as W

pytestmark = pytest.mark.gpu

MM = "def matmul(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }"


def test_run_checks_count_rank_dtype_shape():
    A, B = torch.randn(8, 16, device="cuda"), torch.randn(16, 4, device="cuda")
    ex = tc.compile(MM, "matmul", [A, B], "naive")
    (C,) = tc.prepare_outputs(MM, "matmul", [A, B])
    tc.run(ex, [A, B], [C])
    with pytest.raises(tc.TcError):
        tc.run(ex, [A], [C])
    with pytest.raises(tc.TcError):
        tc.run(ex, [A, B.double()], [C])
    with pytest.raises(tc.TcError):
        tc.run(ex, [A, torch.randn(16, 5, device="cuda")], [C])
    with pytest.raises(tc.TcError):
        tc.run(ex, [A, B], [torch.empty(8, 4, 1, device="cuda")])
    torch.cuda.synchronize()
    assert torch.allclose(C, A @ B, atol=1e-4)


def test_non_contiguous_tensors_are_refused():
    base = torch.randn(64, 128, device="cuda")
    view = base[:, :64]                                     # strides (128, 1)
    src = "def copy(float(M, N) A) -> (B) { B(m, n) = A(m, n) }"
    ex = tc.compile(src, "copy", [view.contiguous()], "naive")
    out = torch.empty(64, 64, device="cuda")
    with pytest.raises(tc.TcError) as e:
        tc.run(ex, [view], [out])
    assert "not contiguous" in str(e.value)
    with pytest.raises(tc.TcError):                          # compile time: stride 1 < 64*... transposed view
        tc.compile(src, "copy", [base.t()], "naive")


def test_profile_reports_kernel_time_and_same_result_for_new_pointers():
    A, B = torch.randn(128, 64, device="cuda"), torch.randn(64, 32, device="cuda")
    ex = tc.compile(MM, "matmul", [A, B], "naive;tile=16,16;mapToThreads=16,16")
    (C,) = tc.prepare_outputs(MM, "matmul", [A, B])
    info = tc.profile(ex, [A, B], [C])
    assert info.kernel_runtime_us > 0 and info.cpu_overhead_us >= 0
    A2, B2, C2 = A.clone() * 2, B.clone(), torch.empty_like(C)
    tc.unchecked_run(ex, [A2, B2], [C2])
    torch.cuda.synchronize()
    assert torch.allclose(C2, 2 * C, atol=1e-4)


def test_clear_runtime_compiled_function_forbids_further_runs():
    A, B = torch.randn(8, 16, device="cuda"), torch.randn(16, 4, device="cuda")
    ex = tc.compile(MM, "matmul", [A, B], "naive")
    (C,) = tc.prepare_outputs(MM, "matmul", [A, B])
    tc.run(ex, [A, B], [C])
    torch.cuda.synchronize()
    ex.clear_runtime_compiled_function()
    with pytest.raises(tc.TcError) as e:
        tc.run(ex, [A, B], [C])
    assert "No rtcFun_" in str(e.value)


def test_runs_on_a_side_stream():
    A, B = torch.randn(64, 64, device="cuda"), torch.randn(64, 64, device="cuda")
    ex = tc.compile(MM, "matmul", [A, B], "naive")
    (C,) = tc.prepare_outputs(MM, "matmul", [A, B])
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        tc.run(ex, [A, B], [C])
    s.synchronize()
    assert torch.allclose(C, A @ B, atol=1e-4)


def test_prepare_outputs_needs_an_input_and_infers_shapes():
    A, B = torch.randn(8, 16, device="cuda"), torch.randn(16, 4, device="cuda")
    (C,) = tc.prepare_outputs(MM, "matmul", [A, B])
    assert C.shape == (8, 4) and C.dtype == torch.float32 and C.is_cuda
    with pytest.raises(tc.TcError):
        tc.prepare_outputs("def f() -> (O) { O(i) = 3 where i in 0:4 }", "f", [])


def test_integer_and_double_tensors():
    src = "def f(int32(N) A, double(N) B) -> (C, D) { C(n) = A(n) * 3 + n \n D(n) = B(n) * B(n) }"
    A = torch.arange(100, dtype=torch.int32, device="cuda")
    B = torch.randn(100, dtype=torch.float64, device="cuda")
    ex = tc.compile(src, "f", [A, B], "naive")
    C, D = tc.prepare_outputs(src, "f", [A, B])
    assert C.dtype == torch.int32 and D.dtype == torch.float64
    tc.run(ex, [A, B], [C, D])
    torch.cuda.synchronize()
    assert torch.equal(C, A * 3 + torch.arange(100, dtype=torch.int32, device="cuda"))
    assert torch.equal(D, B * B)


def test_autotune_small_tensordot_improves_on_naive():
    name = "c1_tensordot_small"
    src, entry, _, _, k = W.CONFIGS[name]
    ins_np = W.make_inputs(name)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    best = tc.autotune(src, entry, ins, "naive", generations=3, pop_size=10, threads=8, seed=7, number_elites=2)
    assert len(best) == 1
    ex = tc.compile(src, entry, ins, best[0])
    outs = tc.prepare_outputs(src, entry, ins)
    t_best = min(tc.profile(ex, ins, outs).kernel_runtime_us for _ in range(5))
    ref = tc_oracle.run(src, entry, ins_np)[0]
    assert np.abs(outs[0].cpu().numpy() - ref).max() <= W.tolerance(k, ref)
    naive = tc.compile(src, entry, ins, "naive")
    t_naive = min(tc.profile(naive, ins, outs).kernel_runtime_us for _ in range(5))
    print(f"naive {t_naive:.1f} us, tuned {t_best:.1f} us: {best[0]}", flush=True)
    assert t_best <= t_naive * 1.05


def test_autotune_survives_unmappable_candidates():
    """A population made mostly of configurations the mapper refuses (fixed huge block) must
    not break the tuner: candidates are marked invalid and the search goes on."""
    A, B = torch.randn(64, 64, device="cuda"), torch.randn(64, 64, device="cuda")
    best = tc.autotune(MM, "matmul", [A, B], "naive", generations=2, pop_size=6, threads=4, seed=3, top_k=2)
    assert 1 <= len(best) <= 2


@pytest.mark.parametrize("resample", [0, 4])
def test_autotune_with_and_without_mutating_duplicates_again(resample):
    """Bred candidates that would repeat a measured mapping are mutated again by default;
    `resample_duplicates=0` is the reference's behaviour.  Both searches return a correct winner."""
    rng = np.random.Generator(np.random.Philox(9))
    A, B = (rng.integers(-3, 4, size=(48, 40)).astype(np.float32) for _ in range(2))
    ins = [torch.from_numpy(A).cuda(), torch.from_numpy(B.T.copy()).cuda()]
    best = tc.autotune(MM, "matmul", ins, "naive", generations=3, pop_size=12, threads=8, seed=5, number_elites=2,
                       resample_duplicates=resample)
    assert len(best) == 1
    ex = tc.compile(MM, "matmul", ins, best[0])
    (out,) = tc.prepare_outputs(MM, "matmul", ins)
    tc.run(ex, ins, [out])
    assert np.array_equal(out.cpu().numpy(), A @ B.T)            # small integers: exact in any order


def test_define_compiles_on_demand_and_memoises():
    defs = """
    def add(float(N) A, float(N) B) -> (C) { C(i) = A(i) + B(i) }
    def scale(float(N) A) -> (C) { C(i) = A(i) * 2.0 }
    """
    T = tc.define(defs, tc.make_naive_options_factory())
    a, b = torch.randn(1000, device="cuda"), torch.randn(1000, device="cuda")
    assert torch.equal(T.add(a, b), a + b)
    assert torch.equal(T.scale(a), a * 2)
    assert len(T._executors) == 2
    out = torch.empty_like(a)
    assert T.add(b, a, outputs=[out]) is out and torch.equal(out, a + b)
    assert len(T._executors) == 2                      # same sizes: no recompilation
    T.add(a[:10].contiguous(), b[:10].contiguous())
    assert len(T._executors) == 3
    tc.assert_almost_equal(T.add(a, b), a + b, a, b, operations=1)


def test_autotune_and_compile_with_cache_round_trip(tmp_path):
    src = "def add(float(N, M) A, float(N, M) B) -> (C) { C(i, j) = A(i, j) + B(i, j) }"
    a, b = torch.randn(64, 300, device="cuda"), torch.randn(64, 300, device="cuda")
    cache = str(tmp_path / "options")
    cfg = tc.TunerConfig().generations(2).pop_size(6).threads(4).seed(3)
    add = tc.autotune_and_compile(src, "add", a, b, starting_options="naive", tuner_config=cfg,
                                  cache_filename=cache, store_to_cache=True)
    assert torch.equal(add(a, b), a + b)
    stored = tc.load_from_cache(src, "add", [a, b], cache, 3)
    assert 1 <= len(stored) <= 3
    T = tc.define(src, tc.make_load_from_cache_options_factory(cache))
    assert torch.equal(T.add(a, b), a + b)
    assert tc.load_from_cache(src, "add", [a[:8].contiguous(), b[:8].contiguous()], cache) == []   # other sizes


@pytest.mark.parametrize("case", ["layernorm", "matmul_3x4x5", "matmul_72x26x72", "matmul_100x400x500"])
def test_autotune_smoke_cases_of_the_reference(case):
    """test/cuda/test_autotuner.cc:86-170 with its smoke-check budget (population 8, few generations):
    the search must return options, and the best ones must compute the right values."""
    import numpy as np
    from oracle import tc_oracle
    layernorm = """def layernorm(float(T, B, C) I) -> (O, mean, centered, var) {
        mean(t, b) +=! I(t, b, c) / C
        centered(t, b, c) = I(t, b, c) - mean(t, b)
        var(t, b) +=! centered(t, b, c) * centered(t, b, c)
        var(t, b) = var(t, b) / C
        O(t, b, c) = centered(t, b, c) / rsqrt(var(t, b)) }"""
    matmul = "def matmul(float(M, N) A, float(N, K) B) -> (output) { output(m, k) +=! A(m, r_n) * B(r_n, k) }"
    src, entry, shapes, k = {
        "layernorm": (layernorm, "layernorm", [(7, 32, 64)], 64),
        "matmul_3x4x5": (matmul, "matmul", [(3, 4), (4, 5)], 4),
        "matmul_72x26x72": (matmul, "matmul", [(72, 26), (26, 72)], 26),
        "matmul_100x400x500": (matmul, "matmul", [(100, 400), (400, 500)], 400),
    }[case]
    rng = np.random.Generator(np.random.Philox(21))
    ins_np = [rng.random(s, dtype=np.float32) for s in shapes]
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    best = tc.autotune(src, entry, ins, "naive", generations=2, pop_size=8, threads=8, number_elites=2, seed=5)
    assert len(best) == 1
    ex = tc.compile(src, entry, ins, best[0])
    outs = tc.prepare_outputs(src, entry, ins)
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    for o, r in zip(outs, tc_oracle.run(src, entry, ins_np)):
        assert np.abs(o.cpu().numpy() - r).max() <= 1e-5 * np.sqrt(k) * max(1.0, float(np.abs(r).max()))


def test_run_can_be_captured_in_a_hip_graph_and_replayed():
    """run() only enqueues kernel launches on the caller's stream, so a caller may capture it into
    a HIP graph (launch-bound TCs such as the batched matmul replay without host launch cost).
    Every replay is checked against an eager run on the same inputs."""
    src, entry, shapes, _, k = W.CONFIGS["c3_batch_matmul"]
    gen = torch.Generator(device="cuda").manual_seed(3)
    ins = [torch.randn(s, device="cuda", generator=gen) for s in shapes]
    ex = tc.compile(src, entry, ins, W.TUNED["c3_batch_matmul"])
    outs = tc.prepare_outputs(src, entry, ins)
    tc.run(ex, ins, outs)                                   # loads the module outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        tc.run(ex, ins, outs)
    eager = tc.prepare_outputs(src, entry, ins)
    for replay in range(3):
        for t in ins:
            t.copy_(torch.randn(t.shape, device="cuda", generator=gen))
        outs[0].fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        tc.run(ex, ins, eager)
        torch.cuda.synchronize()
        assert torch.equal(outs[0], eager[0]), replay
        assert (outs[0] - torch.bmm(ins[0], ins[1])).abs().max().item() <= 1e-5 * 72 ** 0.5 * float(outs[0].abs().max())


@pytest.mark.gpu
def test_device_buffers_stand_in_for_tensors():
    """The package's own device arrays (no tensor library) go through compile, prepare_outputs,
    run and profile like torch tensors and give the oracle's values."""
    from oracle import tc_oracle
    from tests import workloads as W
    name = "c1_tensordot_small"
    src, entry, _, _, k = W.CONFIGS[name]
    ins_np = W.make_inputs(name)
    ins = [tc.DeviceBuffer.from_numpy(a) for a in ins_np]
    ex = tc.compile(src, entry, ins, W.TUNED[name])
    outs = tc.prepare_outputs(src, entry, ins)
    assert isinstance(outs[0], tc.DeviceBuffer) and outs[0].shape == (16, 8, 2, 17, 25)
    tc.run(ex, ins, outs)
    info = tc.profile(ex, ins, outs)
    assert info.kernel_runtime_us > 0
    ref = tc_oracle.run(src, entry, ins_np)[0]
    assert np.abs(outs[0].numpy() - ref).max() <= W.tolerance(k, ref)
    assert "MI3" in tc.device_name() or "AMD" in tc.device_name()


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c2_tensordot", "c3_batch_matmul", "c4_group_convolution", "c5_moments"])
def test_autotune_from_the_naive_options_reaches_the_stored_options(name):
    """What 'after autotuning' means for the benchmark configurations: a short, seeded search that
    starts from the naive options ends within 15 % of the options the benchmark stores, and its
    winner computes the oracle's values (test/cuda/test_autotuner.cc:43-51 tunes and runs;
    tc/autotuner/autotuner-inl.h:418-518)."""
    src, entry, _, _, k = W.CONFIGS[name]
    ins_np = W.make_inputs(name)
    ins = [torch.from_numpy(a).cuda() for a in ins_np]
    outs = tc.prepare_outputs(src, entry, ins)

    def kernel_us(options, warm=200, launches=50, bursts=5):
        ex = tc.compile(src, entry, ins, options)
        tc.profile_repeated(ex, ins, outs, warm)
        return min(tc.profile_repeated(ex, ins, outs, launches) / launches for _ in range(bursts))

    best = tc.autotune(src, entry, ins, "naive", outputs=outs, generations=4, pop_size=30, threads=16, seed=1)
    assert len(best) == 1
    # (a launch under the naive options takes up to 0.2 s: the group convolution on 32 x 8 threads)
    t_stored, t_tuned, t_naive = kernel_us(W.TUNED[name]), kernel_us(best[0]), kernel_us("naive", 1, 2, 1)
    print(f"{name}: naive {t_naive:.1f} us, stored {t_stored:.1f} us, tuned from naive {t_tuned:.1f} us with {best[0]}", flush=True)
    assert t_tuned <= 1.15 * t_stored
    ex = tc.compile(src, entry, ins, best[0])
    for o in outs:
        o.fill_(float("nan"))
    tc.run(ex, ins, outs)
    torch.cuda.synchronize()
    for o, r in zip(outs, tc_oracle.run(src, entry, ins_np)):
        assert np.abs(o.cpu().numpy() - r).max() <= W.tolerance(k, r)


def test_make_autograd_runs_forward_and_backward_comprehensions():
    """The example of tensor_comprehensions/__init__.py:556-600 (a 1x1 convolution and its two
    gradient TCs behind torch.autograd), checked against conv2d's own gradients."""
    conv = """
def convolution(float(N,C,H,W) I, float(M,C,KH,KW) W1) -> (O) {
    O(n, m, h, w) +=! I(n, r_c, h + r_kh, w + r_kw) * W1(m, r_c, r_kh, r_kw)
}
def convolution_igrad(float(M,C,KH,KW) W1, float(N,M,H,W) d_O) -> (d_I) {
    d_I(n, c, h, w) +=! d_O(n, r_m, h - r_kh, w - r_kw) * W1(r_m, c, r_kh, r_kw)
}
def convolution_wgrad(float(N,C,H,W) I, float(N,M,H,W) d_O) -> (d_W1) {
    d_W1(m, c, kh, kw) +=! d_O(r_n, m, r_h - kh, r_w - kw) * I(r_n, c, r_h, r_w)
}
"""
    T = tc.define(conv, tc.make_naive_options_factory())

    def backward(I, W1, d_O):
        return T.convolution_igrad(W1, d_O), T.convolution_wgrad(I, d_O)

    op = tc.make_autograd(T.convolution, backward)
    g = torch.Generator().manual_seed(3)
    I = torch.randint(-3, 4, (2, 3, 9, 8), generator=g).float().cuda().requires_grad_()
    W1 = torch.randint(-3, 4, (4, 3, 1, 1), generator=g).float().cuda().requires_grad_()
    for _ in range(2):                                  # the second pass reuses the compiled kernels
        I.grad = W1.grad = None
        O = op(I, W1)
        seed = torch.randint(-2, 3, O.shape, generator=g).float().cuda()
        O.backward(seed)
        I2, W2 = I.detach().clone().requires_grad_(), W1.detach().clone().requires_grad_()
        O2 = torch.nn.functional.conv2d(I2, W2)
        O2.backward(seed)
        assert torch.equal(O, O2)                       # small integers: exact in any order
        assert torch.equal(I.grad, I2.grad) and torch.equal(W1.grad, W2.grad)
    # no backward function: no gradients flow to the inputs
    I3 = I.detach().clone().requires_grad_()
    tc.make_autograd(T.convolution, None)(I3, W1.detach()).sum().backward()
    assert I3.grad is None
