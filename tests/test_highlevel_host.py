"""Host-side behaviour of the convenience layer (define / factories / TunerConfig / cache lookup)."""
import pytest

import tensorcomprehensions_amd as tc

TWO_DEFS = """
# def commented_out(float(N) A) -> (B) { B(i) = A(i) }
def add(float(N) A, float(N) B) -> (C) { C(i) = A(i) + B(i) }
def scale(float(N) A) -> (C) {
    C(i) = A(i) * 2.0
}
"""


def test_define_exposes_one_method_per_def():
    T = tc.define(TWO_DEFS, tc.make_naive_options_factory())
    assert T.entry_points == ["add", "scale"]
    assert callable(T.add) and callable(T.scale) and not hasattr(T, "commented_out")


def test_tuner_config_is_fluent_and_maps_to_tuner_settings():
    cfg = tc.TunerConfig().generations(3).pop_size(8).threads(4).seed(7).number_elites(2)
    assert cfg.settings() == {"generations": 3, "pop_size": 8, "threads": 4, "seed": 7, "number_elites": 2}


def test_cache_lookup_of_a_missing_file_or_entry_is_empty(tmp_path):
    shapes = [tc.ShapeOnly((100,)), tc.ShapeOnly((100,))]
    assert tc.load_from_cache(TWO_DEFS, "add", shapes, str(tmp_path / "nothing")) == []
    factory = tc.make_load_from_cache_options_factory(str(tmp_path / "nothing"))
    assert factory(TWO_DEFS, "add", *shapes) is None


def test_naive_factory_returns_the_naive_preset():
    assert tc.make_naive_options_factory()("", "f").normalized() == tc.MappingOptions("naive").normalized()


def test_compile_is_reentrant_across_threads():
    """The tuner compiles candidates from several threads at once (front end, mapper and hipRTC
    must be re-entrant): eight threads compiling different TCs and options give the same sources as
    one thread does."""
    import concurrent.futures
    from tests import workloads as W
    jobs = []
    for name, (src, entry, shapes, _, _) in W.CONFIGS.items():
        for options in ("naive", W.TUNED[name]):
            jobs.append((src, entry, [tc.ShapeOnly(s) for s in shapes], options))

    def build(job):
        ex = tc.compile(*job)
        return ex.compiled_source, [ex.launch_bounds(k) for k in range(ex.num_kernels)]

    serial = [build(j) for j in jobs]
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        parallel = list(pool.map(build, jobs * 3))
    assert parallel == serial * 3


def test_make_autograd_wires_forward_and_backward_functions():
    """The autograd helper itself needs no GPU: any two functions on tensors will do."""
    import torch
    calls = []

    def forward(a, b):
        calls.append("f")
        return a * b

    def backward(a, b, g):
        calls.append(("b", g.is_contiguous()))
        return g * b, g * a

    op = tc.make_autograd(forward, backward)
    a = torch.tensor([1.0, 2.0, 3.0], requires_grad=True)
    b = torch.tensor([4.0, 5.0, 6.0], requires_grad=True)
    out = op(a, b)
    out.backward(torch.tensor([1.0, 10.0, 100.0]))
    assert torch.equal(a.grad, torch.tensor([4.0, 50.0, 600.0])) and torch.equal(b.grad, torch.tensor([1.0, 20.0, 300.0]))
    assert calls == ["f", ("b", True)]
    # several outputs, as a list
    two = tc.make_autograd(lambda x: [x + 1, x * 2], lambda x, g1, g2: g1 + 2 * g2)
    x = torch.tensor([1.0, 2.0], requires_grad=True)
    y1, y2 = two(x)
    (y1.sum() + y2.sum()).backward()
    assert torch.equal(x.grad, torch.tensor([3.0, 3.0]))
    # a backward function must answer for every input
    bad = tc.make_autograd(lambda p, q: p + q, lambda p, q, g: g)
    p, q = torch.ones(2, requires_grad=True), torch.ones(2, requires_grad=True)
    with pytest.raises(tc.TcError):
        bad(p, q).sum().backward()
