"""A tensor of 2^31 elements and more: element offsets are formed in 64 bits (the reference's
generated code indexes with int throughout).  int8 keeps it at 2 GiB per tensor."""
import numpy as np
import pytest
import torch

import tensorcomprehensions_amd as tc
from oracle import tc_oracle

pytestmark = pytest.mark.gpu

BIG = """
def big(int8(M, N) X) -> (s, Y) {
    s(m) +=! int32(X(m, n))
    Y(m, n) = int8(X(m, n) + 1)
}
"""
M, N = 65544, 32768            # 2^31 + 2^18 elements


@pytest.mark.parametrize("options", [
    "naive;tile=1,0;mapToThreads=256;mapToBlocks=65544;matchLibraryCalls=1;vectorWidth=4;unroll=4;outerScheduleFusionStrategy=Min",
    "naive;tile=4,1024;mapToThreads=256;mapToBlocks=256,32;unroll=4;useReadOnlyCache=1",
])
def test_offsets_beyond_32_bits(options):
    rng = np.random.Generator(np.random.Philox(2031))
    X = rng.integers(-100, 100, size=(M, N), dtype=np.int8)
    X[-1, -1], X[M // 2 + 3, 5] = 77, -91           # marked elements on either side of the 2^31 boundary
    ins = [torch.from_numpy(X).cuda()]
    ex = tc.compile(BIG, "big", ins, options)
    assert "(int64)" in ex.compiled_source
    s, Y = tc.prepare_outputs(BIG, "big", ins)
    assert tuple(Y.shape) == (M, N) and Y.dtype == torch.int8 and s.dtype == torch.int32
    Y.fill_(-128)
    tc.run(ex, ins, [s, Y])
    torch.cuda.synchronize()
    ref_s, ref_Y = tc_oracle.run(BIG, "big", [X])
    assert np.array_equal(ref_s, X.sum(1, dtype=np.int32))                  # the oracle itself, past the boundary too
    assert ref_Y[-1, -1] == 78 and ref_Y[M // 2 + 3, 5] == -90
    assert np.array_equal(s.cpu().numpy(), ref_s)
    got = Y.cpu().numpy()
    assert got[-1, -1] == 78 and got[M // 2 + 3, 5] == -90
    assert np.array_equal(got, ref_Y)


def test_a_single_dimension_of_2_to_the_31_is_refused():
    with pytest.raises(tc.TcError) as e:
        tc.compile("def f(int8(N) A) -> (B) { B(i) = A(i) }", "f", [tc.ShapeOnly((2 ** 31 + 8,), "int8")], "naive")
    assert "dimension of 2^31 or more" in str(e.value)
