"""Pins of oracle/gemm.py (the yardstick of every GEMM gate) that do not go through it:
plain float64 python loops on tiny shapes, exact small-integer cases with hand-computed
values, transposition identities, and hand values of the comparison metrics. Semantics
followed: /root/reference/tests/pytorch/ref/gemm_ref.py:13-41 (per-group loop, rows of an
empty group untouched, variable-K output [G, A, B] zero for an empty group) and
/root/reference/tests/pytorch/test_utils.py:43-45,61-63,76-80 (relative error, cosine, SNR).
Also one order-sensitive pin of ``oracle.quantize.hadamard16`` against a scalar evaluation of
/root/reference/primus_turbo/flydsl/quantization/mxfp4_quant_kernel.py:92-118."""

import math

import numpy as np
import pytest

from oracle import gemm as OG
from oracle import quantize as Q


def _loop_matmul(a, b):
    """a [M, K] x b [K, N] in python floats (float64), the textbook triple loop."""
    M, K = len(a), len(a[0])
    N = len(b[0])
    return [[math.fsum(float(a[m][k]) * float(b[k][n]) for k in range(K)) for n in range(N)] for m in range(M)]


# ---------------------------------------------------------------------------------------------
# dense
# ---------------------------------------------------------------------------------------------
def test_hand_values_all_layouts():
    # op(A) = [[1, 2, 3], [4, 5, 6]], op(B) = [[1, 0], [2, 1], [0, 3]]  ->  [[5, 11], [14, 23]]
    A = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)          # [M, K]
    B_kn = np.array([[1, 0], [2, 1], [0, 3]], dtype=np.float32)     # [K, N]
    want = np.array([[5, 11], [14, 23]], dtype=np.float64)
    for f64 in (False, True):
        assert np.array_equal(OG.gemm_dequantized(A, B_kn.T.copy(), False, True, f64), want)    # NT
        assert np.array_equal(OG.gemm_dequantized(A, B_kn, False, False, f64), want)            # NN
        assert np.array_equal(OG.gemm_dequantized(A.T.copy(), B_kn, True, False, f64), want)    # TN
        assert np.array_equal(OG.gemm_dequantized(A.T.copy(), B_kn.T.copy(), True, True, f64), want)  # TT


@pytest.mark.parametrize("trans_a", [False, True])
@pytest.mark.parametrize("trans_b", [False, True])
def test_dense_against_python_loop(trans_a, trans_b):
    rng = np.random.default_rng(3)
    M, N, K = 5, 7, 9
    a = rng.standard_normal((K, M) if trans_a else (M, K)).astype(np.float32)
    b = rng.standard_normal((N, K) if trans_b else (K, N)).astype(np.float32)
    opa = a.T if trans_a else a
    opb = b.T if trans_b else b
    want = np.array(_loop_matmul(opa.tolist(), opb.tolist()))
    got64 = OG.gemm_dequantized(a, b, trans_a, trans_b, f64=True)
    got32 = OG.gemm_dequantized(a, b, trans_a, trans_b, f64=False)
    assert got64.shape == (M, N) and got32.shape == (M, N)
    assert got32.dtype == np.float32 and got64.dtype == np.float64
    np.testing.assert_allclose(got64, want, rtol=1e-14, atol=1e-14)
    np.testing.assert_allclose(got32, want, rtol=2e-6, atol=2e-6)


def test_small_integers_are_exact_in_fp32():
    """|a|, |b| <= 8 and K = 64: every partial sum is an integer below 2^24, so the fp32
    path has to reproduce the integer result exactly, whatever its summation order."""
    rng = np.random.default_rng(4)
    a = rng.integers(-8, 9, size=(16, 64))
    b = rng.integers(-8, 9, size=(24, 64))
    want = a.astype(np.int64) @ b.astype(np.int64).T
    got = OG.gemm_dequantized(a.astype(np.float32), b.astype(np.float32), False, True)
    assert np.array_equal(got.astype(np.int64), want) and np.array_equal(got, want.astype(np.float32))
    assert not np.array_equal(got, OG.gemm_dequantized(a.astype(np.float32), b.astype(np.float32)[::-1].copy()))


# ---------------------------------------------------------------------------------------------
# grouped forward (gemm_ref.py:13-25)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("f64", [True, False])
def test_grouped_against_python_loop(trans_b, f64):
    rng = np.random.default_rng(5)
    lens = [3, 0, 4, 1, 0]
    G, N, K = len(lens), 6, 5
    rows = sum(lens) + 2                         # two rows past the last group
    a = rng.standard_normal((rows, K)).astype(np.float32)
    b = rng.standard_normal((G, N, K) if trans_b else (G, K, N)).astype(np.float32)
    got = OG.grouped_gemm_dequantized(a, b, lens, trans_b=trans_b, f64=f64)
    assert got.shape == (rows, N)
    s = 0
    for g, n in enumerate(lens):
        rhs = b[g].T if trans_b else b[g]
        for r in range(s, s + n):
            want = _loop_matmul([a[r].tolist()], rhs.tolist())[0]
            np.testing.assert_allclose(got[r], want, rtol=1e-13 if f64 else 2e-6, atol=1e-13 if f64 else 2e-6)
        s += n
    assert np.all(got[s:] == 0), "rows past sum(group_lens) must be zero"


def test_grouped_hand_values_and_group_boundaries():
    # group 0 = rows 0-1 times W0 = 2 I, group 1 empty, group 2 = row 2 times W2 = [[0, 1], [1, 0]]
    a = np.array([[1, 2], [3, 4], [5, 6], [7, 8]], dtype=np.float32)
    w = np.stack([2 * np.eye(2), 9 * np.ones((2, 2)), np.array([[0, 1], [1, 0]])]).astype(np.float32)
    got = OG.grouped_gemm_dequantized(a, w, [2, 0, 1], trans_b=True)
    assert np.array_equal(got, np.array([[2, 4], [6, 8], [6, 5], [0, 0]], dtype=np.float32))
    # a non-symmetric weight tells trans_b apart: row [1, 2] x [[0, 1], [0, 0]] (stored [N, K])
    w2 = np.array([[[0, 1], [0, 0]]], dtype=np.float32)
    assert np.array_equal(OG.grouped_gemm_dequantized(a[:1], w2, [1], trans_b=True), [[2, 0]])
    assert np.array_equal(OG.grouped_gemm_dequantized(a[:1], w2, [1], trans_b=False), [[0, 1]])


# ---------------------------------------------------------------------------------------------
# grouped variable-K (gemm_ref.py:28-41)
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("f64", [True, False])
def test_variable_k_against_python_loop(f64):
    rng = np.random.default_rng(6)
    lens = [0, 5, 2, 0, 3]
    A, B = 4, 3
    lhs = rng.standard_normal((sum(lens), A)).astype(np.float32)
    rhs = rng.standard_normal((sum(lens), B)).astype(np.float32)
    got = OG.grouped_gemm_variable_k_dequantized(lhs, rhs, lens, f64=f64)
    assert got.shape == (len(lens), A, B)
    s = 0
    for g, n in enumerate(lens):
        if n == 0:
            assert np.all(got[g] == 0), "an empty group gives exactly zero"
        else:
            lt = [[float(lhs[s + r][i]) for r in range(n)] for i in range(A)]   # lhs_g^T [A, n]
            want = _loop_matmul(lt, rhs[s : s + n].tolist())
            np.testing.assert_allclose(got[g], want, rtol=1e-13 if f64 else 2e-6, atol=1e-13 if f64 else 2e-6)
        s += n


def test_variable_k_hand_values():
    lhs = np.array([[1, 2], [3, 4], [5, 6]], dtype=np.float32)
    rhs = np.array([[1, 0, 2], [0, 1, 0], [1, 1, 1]], dtype=np.float32)
    got = OG.grouped_gemm_variable_k_dequantized(lhs, rhs, [2, 0, 1])
    want = np.zeros((3, 2, 3))
    want[0] = [[1, 3, 2], [2, 4, 4]]          # [[1,3],[2,4]] @ [[1,0,2],[0,1,0]]
    want[2] = [[5, 5, 5], [6, 6, 6]]          # outer([5,6], [1,1,1])
    assert np.array_equal(got, want)
    # the variable-K product of a group is the transpose of the swapped product
    swapped = OG.grouped_gemm_variable_k_dequantized(rhs, lhs, [2, 0, 1])
    assert np.array_equal(swapped, np.swapaxes(want, 1, 2))


def test_grouped_forward_and_variable_k_are_adjoint():
    """<grouped(A, W), dY> == <W, variable_k(dY, A)>: the two oracles describe one bilinear form."""
    rng = np.random.default_rng(7)
    lens = [4, 0, 3, 6]
    G, N, K = len(lens), 5, 8
    a = rng.standard_normal((sum(lens), K)).astype(np.float32)
    w = rng.standard_normal((G, N, K)).astype(np.float32)
    dy = rng.standard_normal((sum(lens), N)).astype(np.float32)
    y = OG.grouped_gemm_dequantized(a, w, lens, trans_b=True, f64=True)
    dw = OG.grouped_gemm_variable_k_dequantized(dy, a, lens, f64=True)    # [G, N, K]
    assert math.isclose(float(np.sum(y * dy)), float(np.sum(dw * w)), rel_tol=1e-12)


# ---------------------------------------------------------------------------------------------
# metrics (test_utils.py:43-45, 61-63, 76-80)
# ---------------------------------------------------------------------------------------------
def test_metric_hand_values():
    assert OG.cosine([1, 0], [0, 1]) == 0.0
    assert math.isclose(OG.cosine([1, 2, 3], [2, 4, 6]), 1.0, rel_tol=0, abs_tol=1e-15)
    assert math.isclose(OG.cosine([1, 0], [1, 1]), 1 / math.sqrt(2), rel_tol=1e-15)
    assert math.isclose(OG.cosine([1, 2], [-1, -2]), -1.0, abs_tol=1e-15)
    assert OG.cosine([0, 0], [0, 0]) == 1.0

    # max |y - ref| / max |ref|: relative to the output's dynamic range, NOT element-wise
    ref = np.array([10.0, -20.0, 0.5])
    y = np.array([10.5, -20.0, 0.0])
    assert OG.max_rel_err(ref, y) == 0.5 / 20.0
    assert OG.max_rel_err(ref, ref) == 0.0
    assert OG.max_rel_err(np.zeros(3), np.array([0.0, 3.0, -1.0])) == 3.0
    assert OG.max_rel_err(y, ref) == 0.5 / 20.0 and OG.max_rel_err(2 * ref, 2 * y) == 0.5 / 20.0

    # |y - ref|_F / |ref|_F: ref (3, 4), error (0.3, 0.4) -> 0.5 / 5
    assert math.isclose(OG.rel_fro([3.0, 4.0], [3.3, 4.4]), 0.1, rel_tol=1e-12)
    assert OG.rel_fro([3.0, 4.0], [3.0, 4.0]) == 0.0 and OG.rel_fro([0.0, 0.0], [3.0, 4.0]) == 5.0
    assert math.isclose(OG.rel_fro(ref, y), math.sqrt(0.5) / math.sqrt(100 + 400 + 0.25), rel_tol=1e-12)

    # element-wise bound |err| <= r |ref| + r rms(row): row (3, 4) has rms sqrt(12.5)
    r = 2.0 ** -7
    rms = math.sqrt(12.5)
    assert math.isclose(OG.elementwise_excess([3.0, 4.0], [3.0, 4.0 + 0.01]), 0.01 / (r * 4 + r * rms), rel_tol=1e-12)
    assert OG.elementwise_excess([3.0, 4.0], [3.0, 4.0]) == 0.0
    # rows are judged on their own: the same 0.05 error passes in a row of large values and fails in a small one
    big_small = np.array([[100.0, -100.0, 100.0], [0.1, -0.1, 0.1]])
    e1, e2 = big_small.copy(), big_small.copy()
    e1[0, 1] += 0.05
    e2[1, 1] += 0.05
    assert OG.elementwise_excess(big_small, e1) < 1 < OG.elementwise_excess(big_small, e2)
    # what the range-relative gate cannot see: both read 5e-4 there
    assert math.isclose(OG.max_rel_err(big_small, e1), 5e-4, rel_tol=1e-9) and math.isclose(OG.max_rel_err(big_small, e2), 5e-4, rel_tol=1e-9)
    assert OG.elementwise_excess(np.zeros((2, 2)), np.zeros((2, 2))) == 0.0
    assert OG.elementwise_excess(np.zeros((2, 2)), np.array([[0.0, 1e-30], [0.0, 0.0]])) == math.inf

    # 10 log10(|ref|^2 / |ref - y|^2): ref (3, 4), noise (0.3, 0.4) -> 25 / 0.25 = 100 -> 20 dB
    assert math.isclose(OG.snr_db([3.0, 4.0], [3.3, 4.4]), 20.0, abs_tol=1e-9)
    assert math.isclose(OG.snr_db([3.0, 4.0], [3.0 + 3, 4.0 + 4]), 0.0, abs_tol=1e-9)
    # a tenfold smaller error is 20 dB more; the 1e-12 guard keeps identical inputs finite
    assert math.isclose(OG.snr_db([3.0, 4.0], [3.03, 4.04]), 40.0, abs_tol=1e-6)
    assert math.isclose(OG.snr_db([3.0, 4.0], [3.0, 4.0]), 10 * math.log10(25 / 1e-12), rel_tol=1e-12)


def test_metrics_against_torch_formulas():
    """The same three formulas evaluated as the reference's helpers state them, in torch."""
    import torch

    rng = np.random.default_rng(8)
    ref = rng.standard_normal((33, 17)).astype(np.float32)
    y = (ref + 0.01 * rng.standard_normal(ref.shape)).astype(np.float32)
    tr, ty = torch.from_numpy(ref), torch.from_numpy(y)
    cos = torch.nn.functional.cosine_similarity(tr.flatten().float(), ty.flatten().float(), dim=0).item()
    snr = (10 * torch.log10(torch.norm(tr).pow(2) / (torch.norm(tr - ty).pow(2) + 1e-12))).item()
    assert math.isclose(OG.cosine(ref, y), cos, abs_tol=2e-6)
    assert math.isclose(OG.snr_db(ref, y), snr, abs_tol=1e-3)
    assert math.isclose(OG.max_rel_err(ref, y), (tr - ty).abs().max().item() / tr.abs().max().item(), rel_tol=1e-6)
    assert math.isclose(OG.rel_fro(ref, y), (torch.norm(tr - ty) / torch.norm(tr)).item(), rel_tol=1e-5)


# ---------------------------------------------------------------------------------------------
# the 16-point Hadamard transform: summation order on data where the order matters
# ---------------------------------------------------------------------------------------------
def _rht16_scalar(v):
    """mxfp4_quant_kernel.py:92-118 evaluated one fp32 operation at a time."""
    f = np.float32

    def h4(v0, v1, v2, v3):
        a0, a1, a2, a3 = f(v0 + v1), f(v0 - v1), f(v2 + v3), f(v2 - v3)
        return f(a0 + a2), f(a1 + a3), f(a0 - a2), f(a1 - a3)

    o = [None] * 16
    for b in range(4):
        o[4 * b : 4 * b + 4] = h4(*[f(x) for x in v[4 * b : 4 * b + 4]])
    r = [None] * 16
    for lc in range(4):
        ys = h4(o[lc], o[4 + lc], o[8 + lc], o[12 + lc])
        for blk in range(4):
            r[4 * blk + lc] = f(ys[blk] * f(0.25))
    return np.array(r, dtype=np.float32)


def test_hadamard16_rounding_order_on_non_integer_data():
    rng = np.random.default_rng(9)
    # wide dynamic range so that fp32 additions round and the order of the butterflies shows
    x = (rng.standard_normal((64, 48)) * np.exp2(rng.integers(-12, 12, size=(64, 48)))).astype(np.float32)
    got = Q.hadamard16(x)
    want = np.stack([np.concatenate([_rht16_scalar(row[16 * g : 16 * g + 16]) for g in range(3)]) for row in x])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the data is order-sensitive: the other butterfly order (across the runs first, then
    # inside them) gives the same values in exact arithmetic and different fp32 bits here
    g = x.reshape(64, 3, 4, 4)
    other = np.swapaxes(Q.hadamard16(np.ascontiguousarray(np.swapaxes(g, -1, -2)).reshape(64, 48)).reshape(64, 3, 4, 4), -1, -2)
    np.testing.assert_allclose(other.reshape(64, 48), got, rtol=1e-4, atol=1e-4 * np.abs(x).max())
    assert not np.array_equal(other.reshape(64, 48).view(np.uint32), got.view(np.uint32))
