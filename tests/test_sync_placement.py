"""Barrier placement between the stages of a kernel: the dynamic programme must return a placement
that satisfies every requirement at the minimum (block barriers, wavefront barriers) cost, checked
against exhaustive search over all 3^n assignments.  Role of findBestSyncConfigInSeq,
tc/core/polyhedral/cuda/mapped_scop.cc:580-727."""
import itertools
import random

import tensorcomprehensions_amd as tc


def covered(n, cyclic, need, at):
    for (i, k), lev in need.items():
        if not cyclic and (k == 0 or i + k >= n):
            continue
        length = n if k == 0 else k
        if not any(at[(i + g) % n] >= lev for g in range(length)):
            return False
    return True


def brute_force(n, cyclic, need):
    gaps = n if cyclic else n - 1
    best = None
    for assign in itertools.product((0, 1, 2), repeat=gaps):
        at = list(assign) + [0] * (n - gaps)
        if covered(n, cyclic, need, at):
            cost = (assign.count(2), assign.count(1))
            if best is None or cost < best:
                best = cost
    return best


def solve(n, cyclic, need):
    spec = f"{int(cyclic)};{n};" + ",".join(f"{i}:{k}:{lev}" for (i, k), lev in need.items())
    text = tc.host_query("sync_placement", spec)
    at = [0] * n
    for item in filter(None, text.split(",")):
        p, lev = map(int, item.split(":"))
        assert 0 <= p < (n if cyclic else n - 1)
        at[p] = lev
    return at


def test_no_requirement_no_barrier():
    assert solve(4, False, {}) == [0, 0, 0, 0]
    assert solve(4, True, {}) == [0, 0, 0, 0]


def test_one_barrier_serves_overlapping_pairs():
    # 0->2 and 1->3 both need a block barrier: one barrier after child 1 serves both
    at = solve(4, False, {(0, 2): 2, (1, 2): 2})
    assert at == [0, 2, 0, 0]


def test_block_barrier_also_serves_wave_requirement():
    at = solve(3, False, {(0, 1): 1, (0, 2): 2})
    assert sorted(at) == [0, 0, 2] and at[0] == 2


def test_loop_carried_requirement_uses_any_gap_of_the_cycle():
    # child 2 of one iteration against child 0 of the next, and 0 -> 1 in the same iteration
    at = solve(3, True, {(2, 1): 2, (0, 1): 2})
    assert at.count(2) == 2 and at[0] == 2 and at[2] == 2
    # a self dependence across iterations is satisfied by a barrier anywhere in the body
    at = solve(3, True, {(1, 0): 2, (0, 1): 2})
    assert at == [2, 0, 0]


def test_matches_exhaustive_search_on_random_instances():
    rng = random.Random(1234)
    for trial in range(400):
        n = rng.randint(1, 6)
        cyclic = rng.random() < 0.5
        need = {}
        for i in range(n):
            for k in range(n):
                r = rng.random()
                if r < 0.25:
                    need[(i, k)] = 1 if rng.random() < 0.5 else 2
        at = solve(n, cyclic, need)
        assert covered(n, cyclic, need, at), (n, cyclic, need, at)
        cost = (at.count(2), at.count(1))
        assert cost == brute_force(n, cyclic, need), (n, cyclic, need, at)


def test_dense_random_requirements_as_in_the_reference_test():
    """Same experiment as SyncConfigInSeqOptimalityTest (test/test_cuda_mapper.cc:168-350): every
    entry of the requirement matrix uniform in {0, 1, 2}, 2-4 children, with and without a loop."""
    for cyclic in (False, True):
        for n in range(2, 5):
            for seed in range(50):
                rng = random.Random(seed * 10 + n)
                need = {(i, k): rng.randint(0, 2) for i in range(n) for k in range(n)}
                need = {key: lev for key, lev in need.items() if lev}
                at = solve(n, cyclic, need)
                assert covered(n, cyclic, need, at), (n, cyclic, need, at)
                assert (at.count(2), at.count(1)) == brute_force(n, cyclic, need), (n, cyclic, need, at)
