"""The library's host code (front end, range inference, mapper, code generator, option codecs)
built with AddressSanitizer and UndefinedBehaviorSanitizer and run over a corpus through the C ABI:
the five benchmark configurations at full size, every comprehension of the reference's benchmark
suite at its test and default sizes, and seeded random comprehensions, each under seeded random
mapping options (the space the genetic search draws from); every option set also goes through the
wire codec, and damaged copies of its message (truncated, bytes replaced, varints that run on)
are read back; the tuner's host side (value sets, the genetic search on a synthetic cost, the
options cache and 300 damaged copies of a cache file) runs as well, and 100 damaged copies of every
definition go through parser, semantic analysis and mapper (an error report is the only
acceptable outcome; a leak on that path counts as a failure); every fifth definition is tuned
against the cost model of tc/autotuner/model_backend.h (eight compile threads and the evaluation
thread under the sanitizers).  No GPU call is made.  A sanitizer report aborts the driver."""
import os
import random
import re
import subprocess

import numpy as np

from tests import benchmark_tcs as B
from tests import random_tcs
from tests import workloads as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tensorcomprehensions_amd", "csrc")
CODES = {"float32": "2:32", "float64": "2:64", "float16": "2:16", "int32": "0:32", "int64": "0:64", "int8": "0:8",
         "uint8": "1:8"}


def spec(dtype, shape):
    return CODES[str(np.dtype(dtype))] + ":" + "x".join(str(int(e)) for e in shape)


def record(entry, specs, text, options):
    return "\n".join([entry, " ".join(specs), text.strip("\n"), "%%"] + options + ["@@"]) + "\n"


def corpus():
    rng = random.Random(20240607)
    out = []
    for name, (text, entry, shapes, _, _) in W.CONFIGS.items():
        opts = [W.TUNED[name], "naive"] + [random_tcs.random_options(rng, 5) for _ in range(40)]
        out.append(record(entry, [spec("float32", s) for s in shapes], text, opts))
    for name, (text, entry, _, _) in B.CASES.items():
        for reference in (False, True):
            if reference and name not in B.REFERENCE_SIZES:
                continue
            arrays = B.make_inputs(name, reference_sizes=False) if not reference else None
            if reference:
                specs = [spec("int32" if s[0] == "int" else "float32", s[1]) if isinstance(s[0], str) else spec("float32", s)
                         for s in B.REFERENCE_SIZES[name]]
                opts = [B.TUNED_AT_REFERENCE_SIZES.get(name, "naive")]
            else:
                specs = [spec(a.dtype, a.shape) for a in arrays]
                opts = ["naive"]
            opts += [random_tcs.random_options(rng, 4) for _ in range(25)]
            out.append(record(entry, specs, text, opts))
    # sizes at and beyond the 32-bit limits: 2^31 elements and more (64-bit offsets), a single
    # extent of 2^31 (refused), products of extents that only fit 64 bits
    huge = [
        ("copy", "def copy(int8(N, M) I) -> (O) { O(n, m) = I(n, m) }", [("int8", (65544, 32768))]),
        ("copy", "def copy(int8(N) I) -> (O) { O(n) = I(n) }", [("int8", (2 ** 31 + 8,))]),
        ("moments", W.MOMENTS, [("float32", (70000, 40000))]),
        ("mm", "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }",
         [("float32", (2 ** 20, 2 ** 11)), ("float32", (2 ** 11, 2 ** 20))]),
        ("outer", "def outer(float(N) a, float(M) b) -> (O) { O(n, m) = a(n) * b(m) }",
         [("float32", (2 ** 31 - 1,)), ("float32", (3,))]),
    ]
    for entry, text, tensors in huge:
        out.append(record(entry, [spec(d, sh) for d, sh in tensors], text,
                          ["naive"] + [random_tcs.random_options(rng, 3) for _ in range(10)]))
    attempt = 0
    drawn = 0
    while drawn < 100:
        attempt += 1
        g = random_tcs.generate(rng, f"r{attempt}")
        if g is None:
            continue
        text, entry, shapes, dtype = g
        drawn += 1
        out.append(record(entry, [spec(dtype, s) for s in shapes], text,
                          ["naive"] + [random_tcs.random_options(rng, 4) for _ in range(20)]))
    return "".join(out)


def test_host_code_is_clean_under_address_and_undefined_behaviour_sanitizers(tmp_path):
    build = subprocess.run(["make", "-C", CSRC, "-j8", "sanitized"], capture_output=True, text=True)
    assert build.returncode == 0, build.stdout[-3000:] + build.stderr[-3000:]
    path = tmp_path / "corpus.txt"
    path.write_text(corpus())
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([os.path.join(CSRC, "build", "san", "mapper_sanitized"), str(path)], capture_output=True, text=True,
                         env=env, timeout=900)
    print(run.stdout[-500:], run.stderr[-6000:], flush=True)
    assert run.returncode == 0, run.stderr[-6000:]
    assert "ERROR: AddressSanitizer" not in run.stderr and "runtime error:" not in run.stderr
    comprehensions, mappings = (int(x) for x in re.findall(r"(\d+) comprehension\(s\), (\d+) mapping", run.stdout)[0])
    assert comprehensions >= 135 and mappings >= 3000
    assert "and 300 damaged cache file(s) read" in run.stdout
    assert int(re.findall(r"(\d+) damaged definition\(s\) parsed", run.stdout)[0]) >= 13700
    assert int(re.findall(r"(\d+) refused", run.stdout)[0]) >= 1          # the single extent of 2^31
    assert int(re.findall(r"(\d+) tuned on the cost model", run.stdout)[0]) >= 15


def test_the_tuning_loop_is_clean_under_thread_sanitizer():
    """Nine tunings (three definitions, three seeds, eight compile threads each) against the cost
    model, in a build of the library with ThreadSanitizer."""
    build = subprocess.run(["make", "-C", CSRC, "-j8", "tsan"], capture_output=True, text=True)
    assert build.returncode == 0, build.stdout[-3000:] + build.stderr[-3000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1")
    run = subprocess.run([os.path.join(CSRC, "build", "tsan", "tuner_threads")], capture_output=True, text=True, env=env, timeout=600)
    print(run.stdout[-300:], run.stderr[-4000:], flush=True)
    assert run.returncode == 0 and "9 tunings done" in run.stdout
    assert "ThreadSanitizer" not in run.stderr
