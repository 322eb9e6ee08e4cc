"""Seeded generator of random comprehensions for parity tests.

A generated definition has one to three float (sometimes double) inputs of rank one to four and
one to three outputs, each written by a pointwise statement or a reduction (`+=!`, `max=!`,
`min=!`) over a sum or product of accesses, sometimes wrapped in tanh / fmax / fabs / a select on
an index, sometimes with a window access `v + r` or `2 * v + r` (v ranged by that access alone, as
in a convolution), a `where` range for an extra output index, an explicit initialisation followed
by a plain `+=`, or an in-place follow-up statement.  Later statements may read earlier outputs.
Index variables are shared between operands at random, also across dimensions of different size,
so range inference has to intersect.  Definitions the oracle refuses, that read elements no
statement wrote, or whose values overflow are dropped: what remains has one defined answer.

`random_options` draws mapping options from the autotuner's space with wider value sets than the
tuner itself uses."""
import random

import numpy as np

from oracle import tc_oracle

VARS = "ijklmnpq"
EXTENTS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 20, 33, 33, 64, 65, 70, 130]
MAX_POINTS = 2e5            # iteration volume of one statement: bounds every reduction length


def _statement(rng, tensors, sizes, name, scalar):
    """Text of the statement(s) defining output `name` from `tensors` [(name, extents)]."""
    operands = rng.sample(tensors, rng.randint(1, min(3, len(tensors))))
    pool = []              # (index variable, extent it was created for; 0: ranged otherwise)

    def index_for(extent):
        reuse = [v for v in pool if rng.random() < 0.5]
        if reuse and rng.random() < 0.6:
            return rng.choice(reuse)[0]
        if len(pool) == len(VARS):
            return rng.choice(pool)[0]
        pool.append((VARS[len(pool)], extent))
        return pool[-1][0]

    loads = [[t, [index_for(e) for e in extents]] for t, extents in operands]
    variables = [v for v, _ in pool]
    if len(pool) < len(VARS) and len(loads) >= 2 and rng.random() < 0.35:
        first = loads[0]
        pos = rng.randrange(len(first[1]))
        others = [v for ld in loads[1:] for v in ld[1] if v not in first[1]]
        if others:
            fresh = VARS[len(pool)]
            pool.append((fresh, 0))
            variables.append(fresh)
            stride = "" if rng.random() < 0.7 else f"{rng.choice([1, 2])} * "
            first[1][pos] = f"{stride}{fresh} + {rng.choice(others)}"
    lhs = rng.sample(variables, rng.randint(0, len(variables))) or [variables[0]]
    reduced = [v for v in variables if v not in lhs]

    expr = None
    for t, idx in loads:
        term = f"{t}({', '.join(idx)})"
        expr = term if expr is None else f"({expr} {rng.choice(['*', '+', '-'])} {term})"
    w = rng.random()
    if w < 0.15:
        expr = f"tanh({expr})"
    elif w < 0.3:
        expr = f"fmax({expr}, 0)"
    elif w < 0.4:
        expr = f"fabs({expr})"
    elif w < 0.5:
        expr = f"(({lhs[0]} > 1) ? {expr} : {scalar}({lhs[0]}))"
    elif w < 0.55:
        expr = f"{expr} * {rng.choice(sorted(sizes))}"
    op = rng.choice(["+=!", "+=!", "+=!", "max=!", "min=!"]) if reduced else "="

    points = 1
    for _, e in pool:
        points *= max(e, 16)
    if points > MAX_POINTS:
        return None

    where = ""
    if len(pool) < len(VARS) and rng.random() < 0.15:
        extra = VARS[len(pool)]
        pool.append((extra, 0))
        lhs = lhs + [extra]
        where = f" where {extra} in 0:{rng.choice([1, 3, 5, 16])}"
        if rng.random() < 0.5:
            expr = f"({expr} + {extra})"
    target = f"{name}({', '.join(lhs)})"
    lines = []
    if reduced and rng.random() < 0.2:
        ranges = [f"{v} in 0:{e}" for v, e in pool if v in lhs and e > 0]
        clause = ", ".join(([where[len(' where '):]] if where else []) + ranges)
        lines.append(f"    {target} = {scalar}({rng.choice(['0', '1.5', lhs[0]])})"
                     + (f" where {clause}" if clause else ""))
        op = op.replace("!", "")
    lines.append(f"    {target} {op} {expr}{where}")
    if rng.random() < 0.3:
        lines.append(f"    {target} = {target} * 0.5 + 1")
    return lines


def generate(rng, name):
    """(tc text, entry, input shapes, numpy dtype) or None when the draw is not usable."""
    scalar = "double" if rng.random() < 0.15 else "float"
    sizes, tensors, params = {}, [], []
    for t in "ABC"[:rng.randint(1, 3)]:
        dims = []
        for _ in range(rng.choice([1, 2, 2, 3, 3, 4])):
            s = rng.choice(["N", "M", "K", "P", "Q"])
            sizes.setdefault(s, rng.choice(EXTENTS))
            dims.append(s)
        tensors.append((t, [sizes[s] for s in dims]))
        params.append(f"{scalar}({', '.join(dims)}) {t}")
    shapes = [tuple(e) for _, e in tensors]
    lines, outs = [], []
    for si in range(rng.randint(1, 3)):
        out = f"O{si}"
        body = _statement(rng, tensors, sizes, out, scalar)
        if body is None:
            return None
        lines += body
        outs.append(out)
        src = f"def {name}({', '.join(params)}) -> ({', '.join(outs)}) {{\n" + "\n".join(lines) + "\n}\n"
        try:
            extents = tc_oracle.infer_output_shapes(src, name, shapes)[-1][2]
        except tc_oracle.TcError:
            return None
        if any(e <= 0 for e in extents):
            return None
        tensors.append((out, list(extents)))
    return src, name, shapes, np.float64 if scalar == "double" else np.float32


def cases(seed, count):
    """`count` usable definitions with inputs and oracle answers: (src, entry, inputs, outputs)."""
    rng = random.Random(seed)
    data = np.random.Generator(np.random.Philox(seed))
    found = []
    attempt = 0
    while len(found) < count:
        attempt += 1
        g = generate(rng, f"f{attempt}")
        if g is None:
            continue
        src, entry, shapes, dtype = g
        ins = [data.uniform(-1, 1, size=s).astype(dtype) for s in shapes]
        try:
            ref = tc_oracle.run(src, entry, ins)
        except tc_oracle.TcError:
            continue                                      # (a range given empty: nothing to run)
        if not all(np.isfinite(r).all() for r in ref):
            continue
        # an element read before any statement wrote it shows when the outputs start poisoned
        poisoned = tc_oracle.run(src, entry, ins, outputs=[np.full(r.shape, np.nan, r.dtype) for r in ref])
        if not all(np.array_equal(a, b) for a, b in zip(ref, poisoned)):
            continue
        found.append((src, entry, ins, ref))
    return found


SIZES = [0, 0, 1, 2, 3, 4, 5, 7, 8, 9, 13, 16, 17, 24, 32, 33, 64, 100, 128, 256]


def random_options(rng, band=4):
    tile = [rng.choice(SIZES) for _ in range(rng.randint(1, band + 2))]
    threads = [rng.choice([1, 2, 4, 7, 8, 16, 32, 50, 64, 96, 128, 256, 512, 1024])]
    for _ in range(rng.randint(0, 2)):
        threads.append(rng.choice([1, 2, 3, 4, 5, 8, 16, 32]))
    while np.prod(threads) > 1024:
        threads.pop()
    blocks = [rng.choice([1, 2, 3, 5, 8, 16, 64, 256, 1024]) for _ in range(rng.randint(1, 3))]
    parts = ["naive", "tile=" + ",".join(map(str, tile)), "mapToThreads=" + ",".join(map(str, threads)),
             "mapToBlocks=" + ",".join(map(str, blocks)),
             f"unroll={rng.choice([1, 2, 3, 4, 8, 16, 32, 64, 128, 256, 512])}"]
    for flag in ("useSharedMemory", "usePrivateMemory", "unrollCopyShared", "matchLibraryCalls", "useReadOnlyCache",
                 "collapseContiguous", "useMfma", "prefetchShared", "tileImperfectlyNested"):
        parts.append(f"{flag}={rng.randint(0, 1)}")
    parts.append(f"vectorWidth={rng.choice([1, 1, 2, 4])}")
    if rng.random() < 0.3:
        parts.append(f"maxSharedMemory={rng.choice([0, 512, 4096, 16384, 65536])}")
    if rng.random() < 0.3:
        parts.append(f"sharedDepth={rng.randint(0, 5)}")
    if rng.random() < 0.3:
        parts.append(f"privateDepth={rng.randint(0, 5)}")
    parts.append(f"outerScheduleFusionStrategy={rng.choice(['Max', 'Preserve3Coincident', 'Min'])}")
    parts.append(f"intraTileScheduleFusionStrategy={rng.choice(['Max', 'Preserve3Coincident', 'Min'])}")
    return ";".join(parts)
