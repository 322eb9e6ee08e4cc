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
