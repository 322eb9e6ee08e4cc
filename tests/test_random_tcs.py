"""Random comprehensions on a GPU-less host: the front end infers the oracle's output shapes and
types, and the mapper accepts every definition under random mapping options (the generated HIP is
compiled for gfx950 for a sample of them)."""
import random

import numpy as np

import tensorcomprehensions_amd as tc
from tests import random_tcs


def test_front_end_and_mapper_accept_what_the_oracle_accepts():
    rng = random.Random(5)
    compiled = 0
    for n, (src, entry, ins, ref) in enumerate(random_tcs.cases(seed=101, count=60)):
        shapes = [tc.ShapeOnly(a.shape, str(a.dtype)) for a in ins]
        info = tc.infer_output_tensor_info(src, entry, shapes)
        assert [(name, shape) for name, shape, _ in info] == [(str(r.dtype), r.shape) for r in ref], src
        for options in ("naive", random_tcs.random_options(rng), random_tcs.random_options(rng)):
            source, launches = tc.map_only(src, entry, shapes, options)
            assert launches and all(np.prod(block) <= 1024 for _, block in launches), (src, options)
        if n % 10 == 0:
            tc.compile(src, entry, shapes, options)     # hipRTC accepts the generated source
            compiled += 1
    assert compiled == 6


def test_front_end_rejects_what_the_oracle_rejects():
    """Draws the oracle's range inference refuses (unsolved or empty ranges, mostly) are refused by
    the C++ front end as well: acceptance agrees in both directions."""
    from oracle import tc_oracle
    rejected = []
    original = tc_oracle.infer_output_shapes

    def spy(src, name, shapes):
        try:
            return original(src, name, shapes)
        except tc_oracle.TcError:
            rejected.append((src, name, shapes))
            raise

    random_tcs.tc_oracle.infer_output_shapes = spy
    try:
        rng = random.Random(13)
        n = 0
        while len(rejected) < 150:
            n += 1
            random_tcs.generate(rng, f"g{n}")
    finally:
        random_tcs.tc_oracle.infer_output_shapes = original
    for src, name, shapes in rejected:
        dtype = "float64" if "double(" in src else "float32"
        try:
            tc.infer_output_tensor_info(src, name, [tc.ShapeOnly(s, dtype) for s in shapes])
        except tc.TcError:
            continue
        raise AssertionError("accepted although the oracle refuses it:\n" + src)
