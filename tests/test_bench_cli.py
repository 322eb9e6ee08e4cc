"""bench.py's command line, as far as it can be checked without a GPU: one GPU only, and the
probe kernels of --stream / --floor map for gfx950 with the launch shapes their descriptions name."""
import math
import os
import subprocess
import sys

import tensorcomprehensions_amd as tc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0 and "one GPU" in run.stderr


def test_stream_probes_map_with_streaming_loads_and_stores():
    sys.path.insert(0, ROOT)
    import bench
    launches = {}
    for label, src, entry, shapes, options, nbytes in bench.STREAM_PROBES:
        code, launch = tc.map_only(src, entry, [tc.ShapeOnly(s) for s in shapes], options)
        launches[label] = launch
        assert "__builtin_nontemporal_load" in code and "__tc::storeThrough" in code, label
        elements = sum(math.prod(s) for s in shapes)
        assert nbytes >= 4 * elements                           # every input once, plus the output
    assert launches["add4 4:1"] == [((8192, 1, 1), (784, 1, 1))]
    assert launches["add4 4:1, 196 threads x 4 lanes"] == [((8192, 1, 1), (196, 1, 1))]
    assert launches["rowsum 1:0"] == [((1024, 1, 1), (512, 1, 1))]
