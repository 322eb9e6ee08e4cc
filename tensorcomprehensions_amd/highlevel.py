"""Convenience layer of the reference's Python package over compile / run / autotune:
`define` with mapping-options factories, `autotune_and_compile`, `TunerConfig`,
`assert_almost_equal` (tensor_comprehensions/__init__.py:47-71, 220-259, 261-327, 329-510).
Pure host logic; every kernel still comes from the JIT behind `compile`."""
import re

import tensorcomprehensions_amd as _tc


class TunerConfig:
    """Fluent tuner settings (tclib.TunerConfig): each setter returns the config."""

    def __init__(self):
        self._settings = {}

    def _set(self, key, value):
        self._settings[key] = value
        return self

    def generations(self, n): return self._set("generations", int(n))
    def pop_size(self, n): return self._set("pop_size", int(n))
    def crossover_rate(self, n): return self._set("crossover_rate", int(n))
    def mutation_rate(self, n): return self._set("mutation_rate", int(n))
    def number_elites(self, n): return self._set("number_elites", int(n))
    def threads(self, n): return self._set("threads", int(n))
    def seed(self, n): return self._set("seed", int(n))
    def tuner_min_launch_total_threads(self, n): return self._set("min_launch_total_threads", int(n))

    def settings(self):
        return dict(self._settings)


def _as_options(options):
    if options is None:
        return _tc.MappingOptions("naive")
    return options if isinstance(options, _tc.MappingOptions) else _tc.MappingOptions(str(options))


def autotune_and_compile(tc, entry_point, *inputs, starting_options=None, tuner_config=None, cache_filename=None,
                         load_from_cache=False, store_to_cache=False):
    """Tune, then compile with the best options found; None when no candidate could be run."""
    best = _autotune(tc, entry_point, inputs, starting_options, tuner_config, cache_filename, load_from_cache,
                     store_to_cache)
    return None if best is None else _tc.compile(tc, entry_point, list(inputs), best)


def _autotune(tc, entry_point, inputs, starting_options, tuner_config, cache_filename, load_from_cache, store_to_cache):
    inputs = list(inputs)
    base = [_as_options(starting_options).to_text()]
    if cache_filename and load_from_cache:
        base = [o.to_text() for o in _tc.load_from_cache(tc, entry_point, inputs, cache_filename, 1)] + base
    settings = (tuner_config or TunerConfig()).settings()
    if cache_filename and store_to_cache:
        settings["cache_file"] = cache_filename
    best = _tc.autotune(tc, entry_point, inputs, "\n".join(base), **settings)
    return best[0] if best else None


def make_naive_options_factory():
    def generate(tc, entry_point, *inputs):
        return _tc.MappingOptions("naive")
    return generate


def make_load_from_cache_options_factory(cache_filename):
    def generate(tc, entry_point, *inputs):
        loaded = _tc.load_from_cache(tc, entry_point, list(inputs), cache_filename, 1)
        return loaded[0] if loaded else None
    return generate


def make_autotuned_options_factory(starting_options=None, tuner_config=None, cache_filename=None, load_from_cache=False,
                                   store_to_cache=False):
    def generate(tc, entry_point, *inputs):
        return _autotune(tc, entry_point, inputs, starting_options, tuner_config, cache_filename, load_from_cache,
                         store_to_cache)
    return generate


class TC:
    """Every def of a TC text as a method; compiles on first use per input sizes and memoises."""

    def __init__(self, tc, mapping_options_factory):
        self.tc = tc
        self.mapping_options_factory = mapping_options_factory
        self._executors = {}
        text = re.sub(r"#[^\n]*", "", tc)
        self.entry_points = re.findall(r"\bdef\s+([A-Za-z_]\w*)\s*\(", text)
        for name in self.entry_points:
            setattr(self, name, self._method(name))

    def _method(self, name):
        def fun(*inputs, outputs=None, unchecked=False):
            return self(name, *inputs, outputs=outputs, unchecked=unchecked)
        return fun

    def __call__(self, entry_point, *inputs, outputs=None, unchecked=False):
        key = (entry_point,) + tuple((tuple(t.shape), str(t.dtype), tuple(t.stride())) for t in inputs)
        ex = self._executors.get(key)
        if ex is None:
            options = self.mapping_options_factory(self.tc, entry_point, *inputs)
            if options is None:
                raise _tc.TcError(f"no mapping options available for {entry_point} at these sizes")
            ex = self._executors[key] = _tc.compile(self.tc, entry_point, list(inputs), options)
        return ex(*inputs, outputs=outputs, unchecked=unchecked)


def define(tc, mapping_options_factory):
    return TC(tc, mapping_options_factory)


def make_autograd(forward_fun, backward_fun):
    """A callable with torch.autograd support from two functions on tensors (typically methods of
    a `define`d TC): `forward_fun(*inputs)` computes the outputs, `backward_fun(*inputs,
    *output_gradients)` the gradients of the inputs, in input order.  Counterpart of the reference's
    helper (tensor_comprehensions/__init__.py:513-576): the inputs are saved for the backward
    pass, incoming gradients are made contiguous, `backward_fun=None` gives no gradients."""
    import torch

    class _Op(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *inputs):
            ctx.save_for_backward(*inputs)
            out = forward_fun(*inputs)
            return tuple(out) if isinstance(out, (list, tuple)) else out

        @staticmethod
        def backward(ctx, *gradients):
            saved = ctx.saved_tensors
            if backward_fun is None:
                return (None,) * len(saved)
            grads = backward_fun(*saved, *[g.contiguous() for g in gradients])
            grads = tuple(grads) if isinstance(grads, (list, tuple)) else (grads,)
            if len(grads) != len(saved):
                raise _tc.TcError(f"backward function returned {len(grads)} gradients for {len(saved)} inputs")
            return grads

    def apply(*inputs):
        return _Op.apply(*inputs)
    return apply


def assert_almost_equal(actual, expected, *inputs, operations=1, precision=1e-7):
    """|actual - expected| <= precision * operations * max|input| elementwise bound of the reference's
    helper (tensor_comprehensions/__init__.py:47-71)."""
    import torch
    diff = (actual.double() - expected.double()).abs().max().item()
    scale = max([float(torch.as_tensor(t).double().abs().max()) for t in inputs] or [1.0])
    bound = precision * operations * max(scale, 1.0)
    if not diff <= bound:
        raise AssertionError(f"max abs difference {diff} exceeds {bound}")
