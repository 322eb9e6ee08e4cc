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


@pytest.mark.parametrize("options", [
    # reduction tiles staged through two LDS copies, loads of four tiles in flight
    "naive;tile=64,64,32;mapToThreads=64,8;mapToBlocks=1024,1;useMfma=1;useSharedMemory=1;prefetchShared=1",
    # operands straight from memory, the reduction of a tile split over four wavefronts
    "naive;tile=16,32;unroll=256;mapToThreads=256,2;mapToBlocks=4096,2;useSharedMemory=1;useReadOnlyCache=1;useMfma=1",
])
def test_matrix_core_product_with_an_operand_of_2_to_the_31_elements(options):
    """A(65536 x 32768) . B(32768 x 64) in fp32: 8 GiB for the first operand, built on the device.
    A(m, k) = ((m + k) mod 3) - 1 and B(k, n) = 1 + (n mod 2) are small integers, so every sum is
    exact in fp32 and has a closed form: the residues of (m + k) mod 3 over k = 0 .. K-1 occur
    c0, c1, c2 times and C(m, n) = (c2 - c0) * (1 + n mod 2)."""
    mm = "def mm(float(M, K) A, float(K, N) B) -> (C) { C(m, n) +=! A(m, r_k) * B(r_k, n) }"
    m_, k_, n_ = 65536, 32768, 64
    rows = torch.arange(m_, device="cuda", dtype=torch.int32).unsqueeze(1)
    cols = torch.arange(k_, device="cuda", dtype=torch.int32).unsqueeze(0)
    A = (((rows + cols) % 3) - 1).to(torch.float32)
    del rows, cols
    B = (1 + (torch.arange(n_, device="cuda") % 2)).to(torch.float32).repeat(k_, 1).contiguous()
    print(f"case {options}", flush=True)
    ex = tc.compile(mm, "mm", [A, B], options)
    assert "(int64)" in ex.compiled_source
    (C,) = tc.prepare_outputs(mm, "mm", [A, B])
    C.fill_(float("nan"))
    tc.run(ex, [A, B], [C])
    torch.cuda.synchronize()
    got = C.cpu().numpy()
    # residue r of (m + k) mod 3 occurs for k = (r - m) mod 3, +3, ...: count = ceil((K - first) / 3)
    mrow = np.arange(m_, dtype=np.int64)
    count = lambda r: (k_ - ((r - mrow) % 3) + 2) // 3
    expected = np.outer(count(2) - count(0), 1 + (np.arange(n_) % 2)).astype(np.float32)
    assert np.array_equal(got, expected)


def test_a_single_dimension_of_2_to_the_31_is_refused():
    with pytest.raises(tc.TcError) as e:
        tc.compile("def f(int8(N) A) -> (B) { B(i) = A(i) }", "f", [tc.ShapeOnly((2 ** 31 + 8,), "int8")], "naive")
    assert "dimension of 2^31 or more" in str(e.value)
