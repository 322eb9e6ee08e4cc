"""The programs of the reference's Python examples through `tc.define` on the GPU
(python/examples/min_distance.py:38-175, tum.py:114-197 and :254-262, masked_conv.py:67-77): tensors
of bytes, sizes written as numbers in a signature, subscripts read from another tensor, scalars and
0-dimensional results, reductions whose right-hand side is a conditional that keeps a subscript out
of bounds from being read.  Every result is compared with the oracle's and with a closed form in
numpy."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
import tensorcomprehensions_amd as tc  # noqa: E402
from oracle import tc_oracle  # noqa: E402

pytestmark = pytest.mark.gpu

OPTION_FACTORIES = {
    "naive": tc.make_naive_options_factory(),
    "rows_of_wavefronts": lambda text, entry, *inputs: tc.MappingOptions(
        "naive;tile=4,16,16;mapToThreads=64,4;mapToBlocks=64,64;matchLibraryCalls=1;unroll=4"),
}


def gpu(*arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays]


def host(t):
    return t.cpu().numpy()


def same_as_oracle(text, entry, inputs, outputs, k):
    ref = tc_oracle.run(text, entry, inputs)
    assert len(ref) == len(outputs)
    for r, o in zip(ref, outputs):
        got = host(o)
        assert got.shape == r.shape and got.dtype == r.dtype, (entry, got.dtype, r.dtype)
        if np.issubdtype(r.dtype, np.integer):
            assert np.array_equal(got, r), entry
        else:
            scale = max(float(np.abs(r).max()), 1e-30)
            assert np.abs(got - r).max() <= 1e-5 * np.sqrt(k) * scale, entry


MIN_DISTANCE = """
def mindis(float(M, 256) L, uint8(N, M) Codes) -> (S, v, min_idx) {
    S(n) +=! L(r_m, int32(Codes(n, r_m)))
    v min=! S(r_n)
    min_idx min=! (S(r_n) == v) ? r_n : N
}
def reduce_codes(float(M, 256) L, uint8(N, M) Codes) -> (S) {
    S(n) +=! L(r_m, int32(Codes(n, r_m)))
}
def min_2d(float(D, NBYD) S) -> (V) {
    V(d) min=! S(d, r_nbyd)
}
def min_1d(float(D) V) -> (v) {
    v min=! V(r_d)
}
def argmin_2d(float(D, NBYD) S, float v) -> (MinIdx) {
    MinIdx(d) min=! (S(d, r_nbyd) == v) ? d * NBYD + r_nbyd : NBYD * D
}
def argmin_1d(float(N) S, int32(D) MinIdx) -> (min_idx) {
    min_idx min=! (MinIdx(r_d) < N) ? r_d : N
}
def mindis_k(float(K, M, 256) L, uint8(N, M) Codes) -> (S, V, MinIdx) {
    S(k, n) +=! L(k, r_m, int32(Codes(n, r_m)))
    V(k) min=! S(k, r_n)
    MinIdx(k) min=! (S(k, r_n) == V(k)) ? r_n : N
}
"""


@pytest.mark.parametrize("factory", sorted(OPTION_FACTORIES))
def test_minimum_distance_over_look_up_tables(factory):
    """Sums of table entries selected by byte codes, their minimum and where it is: as one TC, as
    five with the minimum taken in two steps, and with a leading index over several tables."""
    rng = np.random.Generator(np.random.Philox(61))
    N, D, M, K = 6000, 60, 16, 3
    codes = rng.integers(0, 256, size=(N, M)).astype(np.uint8)
    luts = rng.standard_normal((M, 256)).astype(np.float32)
    T = tc.define(MIN_DISTANCE, OPTION_FACTORIES[factory])
    codes_t, luts_t = gpu(codes, luts)

    S, v, min_idx = T.mindis(luts_t, codes_t)
    same_as_oracle(MIN_DISTANCE, "mindis", [luts, codes], [S, v, min_idx], M)
    sums = luts[np.arange(M)[None, :], codes.astype(np.int64)].astype(np.float64).sum(1)
    np.testing.assert_allclose(host(S), sums, rtol=1e-5, atol=1e-5)
    assert v.dim() == 0 and min_idx.dim() == 0 and min_idx.dtype == torch.int32
    assert float(v) == host(S).min() and int(min_idx) == int(host(S).argmin())

    S2 = T.reduce_codes(luts_t, codes_t)
    assert torch.equal(S2, S)
    V = T.min_2d(S2.view(D, N // D))
    v2 = T.min_1d(V)
    MinIdx = T.argmin_2d(S2.view(D, N // D), v2)
    min_idx2 = T.argmin_1d(S2, MinIdx)
    assert np.array_equal(host(V), host(S).reshape(D, N // D).min(1)) and float(v2) == float(v)
    where = np.where(host(S).reshape(D, N // D) == float(v), np.arange(N).reshape(D, N // D), N).min(1)
    assert np.array_equal(host(MinIdx), where.astype(np.int32))
    # the last step names the first part that holds the minimum
    assert int(min_idx2) == int(min_idx) // (N // D)
    same_as_oracle(MIN_DISTANCE, "argmin_2d", [host(S2).reshape(D, N // D), host(v2)], [MinIdx], 1)
    same_as_oracle(MIN_DISTANCE, "argmin_1d", [host(S2), host(MinIdx)], [min_idx2], 1)

    luts_k = rng.standard_normal((K, M, 256)).astype(np.float32)
    Sk, Vk, Ik = T.mindis_k(gpu(luts_k)[0], codes_t)
    same_as_oracle(MIN_DISTANCE, "mindis_k", [luts_k, codes], [Sk, Vk, Ik], M)
    assert np.array_equal(host(Vk), host(Sk).min(1)) and np.array_equal(host(Ik), host(Sk).argmin(1).astype(np.int32))


def cosine_coherence(pos_dist, neg_dist):
    return """
def make_idx(int32(K) Segments) -> (Idx) {
    Idx(k) +=! (r_k < k) ? Segments(r_k) : 0 where k in 0:K+1
}
def make_alpha(int32(KP1) Idx, int32(MAX_L) SegmentsMetaData) -> (Alpha) {
    Alpha(k, max_l_1, max_l_2) = (max_l_1 >= max_l_2) ? 0.0 :
        ((<pos> == 0 || fabs(float(max_l_1 - max_l_2)) <= float(<pos>)) ? 1.0 :
         (<neg> == 0 && fabs(float(max_l_1 - max_l_2)) >= float(<neg>)) ? -1.0 : 0.0)
        * ((Idx(k) + max_l_1 < Idx(k + 1) && Idx(k) + max_l_2 < Idx(k + 1)) ? 1.0 : 0.0)
        where k in 0:KP1-1, max_l_1 in 0:MAX_L, max_l_2 in 0:MAX_L
}
def make_counts(float(K, MAX_L, MAX_L) Alpha, int32(MAX_L) SegmentsMetaData) -> (PosCount, NegCount, tmpPos, tmpNeg) {
    tmpPos(k, max_l_1) +=! (max_l_1 >= r_max_l_2) ? 0.0 : (Alpha(k, max_l_1, r_max_l_2) > 0.0) ? 1.0 : 0.0
        where k in 0:K, max_l_1 in 0:MAX_L, r_max_l_2 in 0:MAX_L
    PosCount(k) +=! tmpPos(k, max_l_1) where k in 0:K, max_l_1 in 0:MAX_L
    tmpNeg(k, max_l_1) +=! (max_l_1 >= r_max_l_2) ? 0.0 : (Alpha(k, max_l_1, r_max_l_2) < 0.0) ? 1.0 : 0.0
        where k in 0:K, max_l_1 in 0:MAX_L, r_max_l_2 in 0:MAX_L
    NegCount(k) +=! tmpNeg(k, max_l_1) where k in 0:K, max_l_1 in 0:MAX_L
}
def make_beta(float(K, MAX_L, MAX_L) Alpha, float(K) PosCount, float(K) NegCount, int32(MAX_L) SegmentsMetaData) -> (Beta) {
    Beta(k, max_l_1, max_l_2) = (max_l_1 >= max_l_2) ? 0.0 :
        (Alpha(k, max_l_1, max_l_2) == 1.0) ? 1.0 / float(PosCount(k)) :
        (Alpha(k, max_l_1, max_l_2) == -1.0) ? -1.0 / float(NegCount(k)) : 0.0
        where k in 0:K, max_l_1 in 0:MAX_L, max_l_2 in 0:MAX_L
}
def normalize(float(N, C) Input) -> (NormData, Square) {
    Square(n) +=! Input(n, r_c) * Input(n, r_c)
    NormData(n, c) = Input(n, c) / sqrt(Square(n) + 1e-12)
}
def dots(float(N, C) NormData, int32(KP1) Idx, float(K, MAX_L, MAX_L) Beta) -> (Dots) {
    Dots(k, max_l_1, max_l_2) +=! (max_l_1 >= max_l_2) ? 0.0 :
        ((Idx(k) + max_l_1 >= Idx(k + 1) || Idx(k) + max_l_2 >= Idx(k + 1)) ? 0.0 :
          NormData(Idx(k) + max_l_1, r_c) * NormData(Idx(k) + max_l_2, r_c))
        where k in 0:K, max_l_1 in 0:MAX_L, max_l_2 in 0:MAX_L
}
def result(float(K, MAX_L, MAX_L) Beta, float(K, MAX_L, MAX_L) Dots) -> (O, tmpO) {
    tmpO(k, max_l_1) +=! (max_l_1 >= r_max_l_2) ? 0.0 : Dots(k, max_l_1, r_max_l_2) * Beta(k, max_l_1, r_max_l_2)
    O(k) +=! tmpO(k, max_l_1)
}
""".replace("<pos>", str(pos_dist)).replace("<neg>", str(neg_dist))


@pytest.mark.parametrize("factory", sorted(OPTION_FACTORIES))
@pytest.mark.parametrize("pos_dist,neg_dist", [(2, 0), (0, 3), (3, 5)])
def test_cosine_coherence_of_segments(factory, pos_dist, neg_dist):
    """Seven TCs in a row over segments of unequal length: the rows a short segment does not have
    lie beyond the input for the last segment, and the conditional keeps them from being read."""
    rng = np.random.Generator(np.random.Philox(62))
    segments = np.array([5, 3, 12, 1, 9, 12, 4], dtype=np.int32)
    K, N, C, L = len(segments), int(segments.sum()), 24, int(segments.max())
    X = rng.standard_normal((N, C)).astype(np.float32)
    text = cosine_coherence(pos_dist, neg_dist)
    T = tc.define(text, OPTION_FACTORIES[factory])
    X_t, seg_t = gpu(X, segments)
    meta_t = torch.ones(L, dtype=torch.int32, device="cuda")

    Idx = T.make_idx(seg_t)
    Alpha = T.make_alpha(Idx, meta_t)
    PosCount, NegCount, tmpPos, tmpNeg = T.make_counts(Alpha, meta_t)
    Beta = T.make_beta(Alpha, PosCount, NegCount, meta_t)
    NormData, Square = T.normalize(X_t)
    Dots = T.dots(NormData, Idx, Beta)
    O, tmpO = T.result(Beta, Dots)

    start = np.concatenate([[0], np.cumsum(segments)]).astype(np.int32)
    assert np.array_equal(host(Idx), start)
    i, j = np.meshgrid(np.arange(L), np.arange(L), indexing="ij")
    kind = np.where(i >= j, 0.0,
                    np.where((pos_dist == 0) | (np.abs(i - j) <= pos_dist), 1.0,
                             np.where((neg_dist == 0) & (np.abs(i - j) >= neg_dist), -1.0, 0.0)))
    inside = (i[None] < segments[:, None, None]) & (j[None] < segments[:, None, None])
    alpha = (kind[None] * inside).astype(np.float32)
    assert np.array_equal(host(Alpha), alpha)
    pos, neg = (alpha > 0).sum((1, 2)), (alpha < 0).sum((1, 2))
    assert np.array_equal(host(PosCount), pos.astype(np.float32)) and np.array_equal(host(NegCount), neg.astype(np.float32))
    with np.errstate(divide="ignore"):
        beta = np.where(alpha == 1, np.float32(1) / pos[:, None, None].astype(np.float32),
                        np.where(alpha == -1, np.float32(-1) / neg[:, None, None].astype(np.float32), np.float32(0)))
    assert np.array_equal(host(Beta), beta.astype(np.float32))
    norm = X.astype(np.float64) / np.sqrt((X.astype(np.float64) ** 2).sum(1, keepdims=True) + 1e-12)
    np.testing.assert_allclose(host(NormData), norm, rtol=1e-5, atol=1e-6)
    dots = np.zeros((K, L, L))
    for k in range(K):
        rows = norm[start[k]:start[k + 1]]
        dots[k, :len(rows), :len(rows)] = np.triu(rows @ rows.T, 1)
    np.testing.assert_allclose(host(Dots), dots, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(host(O), (dots * beta).sum((1, 2)), rtol=1e-4, atol=1e-5)

    same_as_oracle(text, "make_idx", [segments], [Idx], 1)
    same_as_oracle(text, "make_counts", [host(Alpha), host(meta_t)], [PosCount, NegCount, tmpPos, tmpNeg], L)
    same_as_oracle(text, "dots", [host(NormData), host(Idx), host(Beta)], [Dots], C)
    same_as_oracle(text, "result", [host(Beta), host(Dots)], [O, tmpO], L * L)


MASKED_CONVOLVE = """
def masked_convolve(float(B, C, H, W) Input, float(F, C, K, K) Weights, uint8(F, C) Mask) -> (Output) {
    Output(b, f, h, w) +=! (Mask(f, r_c) == 1) ?
        fmax(0.0, Input(b, r_c, h + r_k1, w + r_k2)) * Weights(f, r_c, r_k1, r_k2) : 0.0
}
"""


@pytest.mark.parametrize("factory", sorted(OPTION_FACTORIES))
@pytest.mark.parametrize("shape", [(3, 12, 5, 14, 14, 1), (2, 6, 4, 9, 11, 3)])
def test_masked_convolution(factory, shape):
    """A convolution over the rectified input whose channels a byte mask switches off per filter
    (the example runs 32 x 128 x 56 x 56 with 1 x 1 windows; here also 3 x 3)."""
    B, C, F, H, W, K = shape
    rng = np.random.Generator(np.random.Philox(63))
    I = rng.standard_normal((B, C, H, W)).astype(np.float32)
    Wt = rng.standard_normal((F, C, K, K)).astype(np.float32)
    mask = rng.integers(0, 3, size=(F, C)).astype(np.uint8)       # 2 is not 1: switched off as well
    T = tc.define(MASKED_CONVOLVE, OPTION_FACTORIES[factory])
    out = T.masked_convolve(*gpu(I, Wt, mask))
    same_as_oracle(MASKED_CONVOLVE, "masked_convolve", [I, Wt, mask], [out], C * K * K)
    relu = np.maximum(I, 0).astype(np.float64)
    w = Wt.astype(np.float64) * (mask == 1)[:, :, None, None]
    ref = np.zeros((B, F, H - K + 1, W - K + 1))
    for k1 in range(K):
        for k2 in range(K):
            ref += np.einsum("bchw,fc->bfhw", relu[:, :, k1:k1 + H - K + 1, k2:k2 + W - K + 1], w[:, :, k1, k2])
    np.testing.assert_allclose(host(out), ref, rtol=1e-4, atol=1e-4)
