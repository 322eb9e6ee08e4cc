"""Host-side behaviour of the convenience layer (define / factories / TunerConfig / cache lookup)."""
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
