"""Device-free tuner logic: divisor sets (known answers of test/cuda/test_autotuner_utility.cc:34-50),
the search space built from input shapes, GeneticSearch on a synthetic cost, OptionsCache semantics
(scenarios after test/cuda/test_compilation_cache.cc:133-510), median (tc/core/utils/math.h:23-37)."""
import os
import tempfile

import pytest

import tensorcomprehensions_amd as tc
from tests.scaffolding import scaffold_query


@pytest.mark.parametrize("n,expected", [
    (10, [1, 2, 3, 4, 5, 8, 10, 16]),
    (72, [1, 2, 3, 4, 5, 8, 9, 16, 18, 32, 36, 64, 72, 128]),
    (35, [1, 2, 3, 4, 5, 8, 9, 16, 18, 32, 35, 64]),
    (130, [1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 128, 130, 256]),
])
def test_powers2_and_ceil_divisors(n, expected):
    assert [int(x) for x in tc.host_query("powers2_and_ceil_divisors", n).split(",")] == expected


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_median_of_even_count_is_integer_mean_of_middle_pair():
    assert tc.host_query("median", "3,1,2,10") == "2"
    assert tc.host_query("median", "5,1,9") == "5"
    assert tc.host_query("median", "4") == "4"


def test_search_space_from_shapes():
    fields = dict(kv.split("=") for kv in tc.host_query("search_space", "500x26x72;500x72x26").split(";"))
    tile = [int(x) for x in fields["tile"].split(",")]
    block = [int(x) for x in fields["block"].split(",")]
    assert fields["tile_dims"] == "5"                       # largest rank + 1, + 1 for the slice number of a divided sum
    assert 0 in tile and 0 not in block                     # 0 = "do not tile"; never a block size
    for v in (26, 72, 500, 13, 36, 250, 256, 64):           # divisors of the dims, and of 256
        assert v in tile and v in block
    assert fields["unroll"] == "1,2,4,8,16,32,64,128,256"
    grid = [int(x) for x in fields["grid"].split(",")]      # naive's 64,4 / 256,256 are already members
    # blocks add the thread counts that cover merged trailing dimensions exactly, whole or in lanes
    # of 2 or 4: 26*72 = 1872 -> 936, 468 (72*26 likewise)
    assert sorted(set(block) - set(grid)) == [468, 936] and set(grid) <= set(block)


def test_reduction_tiles_of_the_matrix_members_divide_the_reduction_extent():
    """128 x 1000 times the transpose of 1024 x 1000: the ceiling divisors of 1000 (500, 250, 125, 63, ...)
    hold no usable reduction tile, so the exact divisors that leave at most 16 tiles of whole matrix-core
    steps are candidates too, and the matrix members of generation 0 take the divisor nearest to
    the depth they want (40 for 32, 200 for 256); a power of two stays as it is."""
    fields = dict(kv.split("=") for kv in tc.host_query("search_space", "128x1000;1024x1000").split(";"))
    tile = [int(x) for x in fields["tile"].split(",")]
    assert {100, 200, 500, 250, 125, 63} <= set(tile) and 40 not in tile and 20 not in tile
    seeds = tc.host_query("tuner_seeds", "2,1024,128x1024:128x1000;1024x1000").split("\n")
    staged = [s for s in seeds if "prefetchShared=1" in s and "useMfma=1" in s]
    assert any("tile=16,32,200;" in s and "mapToThreads=64,8" in s for s in staged)
    assert not any("tile=64,64,32;" in s for s in staged)       # 32 does not divide 1000; 40 is no candidate value
    seeds = tc.host_query("tuner_seeds", "2,1024,128x1024:128x1024;1024x1024").split("\n")
    staged = [s for s in seeds if "prefetchShared=1" in s and "useMfma=1" in s]
    for t in ("tile=64,64,32;", "tile=128,128,16;", "tile=64,128,32;", "tile=16,32,256;"):
        assert any(t in s for s in staged), t


def test_base_mapping_outside_the_space_is_refused():
    assert scaffold_query("base_outside_space").startswith("invalid_argument")


def test_genetic_search_is_deterministic_and_monotone_with_elites():
    a = scaffold_query("genetic_search", "seed=5;generations=12;pop_size=24;number_elites=3")
    b = scaffold_query("genetic_search", "seed=5;generations=12;pop_size=24;number_elites=3")
    c = scaffold_query("genetic_search", "seed=6;generations=12;pop_size=24;number_elites=3")
    assert a == b
    best = [float(x) for x in a.split(",")]
    assert all(x >= y for x, y in zip(best, best[1:]))      # elites keep the best alive
    assert best[-1] <= best[0]
    assert len(c.split(",")) == 12


def test_genetic_search_survives_mostly_invalid_generations():
    # only every 6th candidate is valid: with 12 candidates that is 2 < 3 survivors, so every
    # generation takes the re-randomise-around-the-last-best path
    out = scaffold_query("genetic_search", "seed=2;generations=6;pop_size=12;invalid_every=6")
    assert len(out.split(",")) == 6


def test_structured_seeds_are_members_of_the_search_space():
    """Generation 0 holds streaming, row-reduction and matrix-core variants of the first base
    mapping next to it; every seed is expressible in the space built from the same shapes (a seed
    that is not is left out), here for the tensordot, the row moments and the batched matmul."""
    seeds = tc.host_query("tuner_seeds", "5:32x512x8x28x28;32x8x2x28x28").split("\n")
    assert len(seeds) == 18                                   # (3 streaming + 2 reduction) x {256, 196, 392} threads + short rows + 2 mfma
    parsed = [dict(kv.split("=") for kv in tc.MappingOptions(s).normalized().split(";")) for s in seeds]
    assert {p["mapToThreads"] for p in parsed} == {"256", "196", "392", "64,4"}     # 28*28/4, 28*28/2
    assert any(p["tile"] == "1,8,0,0,0" and p["vectorWidth"] == "4" and p["mapToThreads"] == "196" for p in parsed)
    assert sum(p["matchLibraryCalls"] == "1" for p in parsed) == 7 and sum(p["useMfma"] == "1" for p in parsed) == 2
    rows = tc.host_query("tuner_seeds", "1:1024x32768").split("\n")
    assert len(rows) == 8                                     # no merged extent of at most 4096: 256 threads only
    # short rows: four per block along threadIdx.y, a wavefront each
    assert sum(";tile=4,0;" in r and "mapToThreads=64,4" in r and "usePrivateMemory=1" in r for r in rows) == 1
    # row reductions: one row per block (tile 1 on each dimension of the lowest-rank output), the
    # reduction dimension whole, a grid limit that covers all rows
    assert sum(";tile=1,0;" in r and "matchLibraryCalls=1" in r and "mapToBlocks=32768,256" in r for r in rows) == 2


def test_window_seeds_for_convolutions():
    """Outputs of rank three or more with an innermost extent of 8..256 also get the window seeds:
    one image per block, input window in LDS, the innermost output extent along threadIdx.x and a
    power of two of rows along threadIdx.y (group convolution at the benchmark's size: 54 x 16)."""
    seeds = tc.host_query("tuner_seeds", "5,54:32x32x4x56x56;32x4x4x3x3;32x4").split("\n")
    windows = [s for s in seeds if "mapToThreads=54,16" in s]
    assert len(windows) == 2
    assert all(";tile=1,1,0,0,0;" in s and "useSharedMemory=1" in s and "collapseContiguous=0" in s for s in windows)
    assert not any("mapToThreads=54" in s for s in tc.host_query("tuner_seeds", "1,54:1024x54").split("\n"))


def model_tune(settings, name="c5_moments"):
    """The whole tune() on the host against a cost model (tc/autotuner/model_backend.h)."""
    from tests import workloads as W
    text, entry, shapes, _, _ = W.CONFIGS[name]
    arg = settings + "|" + entry + "|" + ";".join("x".join(map(str, s)) for s in shapes) + "|" + text
    fields = dict(line.split("=", 1) for line in scaffold_query("tune_on_model", arg).split("\n"))
    return fields["best"], int(fields["cost_ns"]), int(fields["naive_ns"])


def test_the_tuning_loop_runs_on_the_host_against_a_cost_model():
    """Compile threads, the evaluation thread, duplicate and refused mappings, the refinement
    rounds: the tuner's own machinery on a deterministic cost of the mapping (a charge per launch
    and per statement instance of the busiest thread), with the real front end and mapper."""
    # (one compile thread: with several, the order in which candidates reach the evaluation thread,
    # and with it what is pruned against the best so far, depends on the scheduling of the threads)
    base = "generations=4;pop_size=20;threads=1;seed=3"
    best, cost, naive = model_tune(base)
    assert cost < naive / 10 and tc.MappingOptions(best).normalized() == best
    assert model_tune(base) == (best, cost, naive)                      # a seeded search repeats itself
    # without the structured members of generation 0 and without the refinement the search still leaves the naive options
    _, unseeded, _ = model_tune(base + ";seed_heuristics=0;refinement_rounds=0")
    assert cost <= unseeded < naive
    # mutating repeated mappings again never makes a generation worse informed
    _, plain, _ = model_tune(base + ";seed_heuristics=0;resample_duplicates=0")
    _, resampled, _ = model_tune(base + ";seed_heuristics=0;resample_duplicates=4")
    assert plain < naive and resampled < naive
    for name in ("c2_tensordot", "c3_batch_matmul", "c4_group_convolution"):
        _, c, n = model_tune("generations=3;pop_size=16;threads=8;seed=5", name)
        assert c <= n, name


def test_tuning_on_the_model_reinforces_its_cache_file(tmp_path):
    """cache_file: the first run leaves its best options in `<file>.model` (the backend's suffix,
    as `.cuda` in the reference), a second run starts from them and cannot end worse."""
    cache = str(tmp_path / "tuned.options")
    first = model_tune(f"generations=2;pop_size=10;threads=2;seed=1;seed_heuristics=0;cache_file={cache}")
    assert (tmp_path / "tuned.options.model").stat().st_size > 0
    second = model_tune(f"generations=2;pop_size=10;threads=2;seed=2;seed_heuristics=0;cache_file={cache}")
    assert second[1] <= first[1]


@pytest.mark.parametrize("signal_name,ends", [("SIGINT", "finishes the generation"), ("SIGTERM", "aborts")])
def test_signals_during_tuning(signal_name, ends):
    """SIGINT lets the running generation finish and returns the best found so far, SIGTERM aborts
    the search (tc/autotuner/autotuner-inl.h:418-518: the reference's handlers); here on a search
    far too long to finish, running against the cost model in a child process."""
    import signal
    import subprocess
    import sys
    import time
    child = subprocess.Popen(
        [sys.executable, "-c",
         "import sys; sys.path.insert(0, %r)\n"
         "from tests.test_autotuner_host import model_tune\n"
         "print('started', flush=True)\n"
         "try:\n"
         "    best, cost, naive = model_tune('generations=100000;pop_size=60;threads=4;seed=1;refinement_rounds=0')\n"
         "    print('returned', cost < naive, flush=True)\n"
         "except Exception as e:\n"
         "    print('raised', str(e)[:80], flush=True)\n" % ROOT],
        stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True)
    assert child.stdout.readline().strip() == "started"
    time.sleep(1.5)
    child.send_signal(getattr(signal, signal_name))
    t0 = time.time()
    out, _ = child.communicate(timeout=60)
    assert time.time() - t0 < 30
    if signal_name == "SIGINT":
        assert out.strip() == "returned True", (out, ends)
    else:
        assert out.strip().startswith("raised") and "Abort requested" in out, (out, ends)


def test_fixed_parameters_hold_in_every_candidate_of_a_search():
    """TuningParameterFixer (tc/autotuner/parameters.h:175-220 in the reference): what the caller
    fixes is not searched, so the winner carries it whatever else the search finds."""
    settings = ("generations=3;pop_size=16;threads=1;seed=2;seed_heuristics=0;refinement_rounds=1;"
                "fix_unroll=4;fix_block=128,2;fix_use_shared_memory=1;fix_match_library_calls=0;fix_vector_width=2")
    best, cost, naive = model_tune(settings, "c2_tensordot")
    fields = dict(kv.split("=") for kv in best.split(";"))
    assert fields["unroll"] == "4" and fields["mapToThreads"] == "128,2" and fields["useSharedMemory"] == "1"
    assert fields["matchLibraryCalls"] == "0" and fields["vectorWidth"] == "2" and cost <= naive
    arg_top = settings.replace("generations=3", "generations=2") + ";top_k=3"
    text = scaffold_query("tune_on_model", arg_top + "|moments|64x512|def moments(float(M, N) X) -> (mean) { mean(m) +=! X(m, r_n) / N }")
    assert text.startswith("best=")
