"""CPU oracles for the scaled GEMMs (TEST INFRASTRUCTURE ONLY; see oracle/formats.py).

Every scaled GEMM of the path is linear in its block products, so its exact value
is the matmul of the de-quantized operands; kernels may differ from it only by
fp32 summation order and the final rounding to the output dtype:

* tensorwise / rowwise  C = (A_q . B_q) * sA[m] * sB[n]
  (/root/reference/primus_turbo/triton/gemm/gemm_fp8_kernel.py:123-243,446-565)
* 128-blockwise         C = sum_kb (A_kb . B_kb) * sA[m, kb] * sB[n/128, kb]
  (/root/reference/primus_turbo/triton/gemm/gemm_fp8_kernel.py:871-1013)
* MX                    C = sum_kb 2^(sa[m,kb]-127) 2^(sb[n,kb]-127) (A_kb . B_kb)
  (/root/reference/primus_turbo/pytorch/kernels/gemm/gemm_fp8_impl.py:341-393)
* grouped forward / variable-K
  (/root/reference/tests/pytorch/ref/gemm_ref.py:13-41)

Pinned by (tests/test_oracle_gemm.py): float64 python-loop evaluation on tiny shapes in all
four operand layouts, hand-computed values, exact small-integer cases where fp32 accumulation
is exact, grouped cases with empty groups and rows past the last group, the adjoint identity
between the grouped forward and the variable-K product, and hand values of the metrics
(cosine, range-relative maximum, Frobenius-relative error, element-wise bound, SNR).
"""

from __future__ import annotations

import numpy as np
import torch


def matmul_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """a [M, K] @ b [K, N] with fp32 operands and accumulation (torch CPU kernel)."""
    ta = torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))
    tb = torch.from_numpy(np.ascontiguousarray(b, dtype=np.float32))
    return (ta @ tb).numpy()


def matmul_f64(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    return np.asarray(a, dtype=np.float64) @ np.asarray(b, dtype=np.float64)


def gemm_dequantized(a_deq: np.ndarray, b_deq: np.ndarray, trans_a=False, trans_b=True, f64=False):
    """C = op(A) op(B) from de-quantized operands; ``trans_b`` means B is stored [N, K]."""
    a = a_deq.T if trans_a else a_deq
    b = b_deq.T if trans_b else b_deq
    return matmul_f64(a, b) if f64 else matmul_f32(a, b)


def grouped_gemm_dequantized(a_deq, b_deq, group_lens, trans_b=True, f64=False):
    """out[offs[g]:offs[g+1]] = A_g @ op(B[g]); rows past sum(group_lens) are zero."""
    gl = np.asarray(group_lens, dtype=np.int64)
    N = b_deq.shape[1] if trans_b else b_deq.shape[2]
    out = np.zeros((a_deq.shape[0], N), dtype=np.float64 if f64 else np.float32)
    s = 0
    for g, n in enumerate(gl):
        n = int(n)
        if n:
            rhs = b_deq[g].T if trans_b else b_deq[g]
            out[s : s + n] = (matmul_f64 if f64 else matmul_f32)(a_deq[s : s + n], rhs)
        s += n
    return out


def grouped_gemm_variable_k_dequantized(lhs_deq, rhs_deq, group_lens, f64=False):
    """dW[g] = lhs_g^T @ rhs_g over the rows of group g (zero for an empty group).

    lhs [M_total, A], rhs [M_total, B] -> [G, A, B]."""
    gl = np.asarray(group_lens, dtype=np.int64)
    out = np.zeros((len(gl), lhs_deq.shape[1], rhs_deq.shape[1]), dtype=np.float64 if f64 else np.float32)
    s = 0
    for g, n in enumerate(gl):
        n = int(n)
        if n:
            out[g] = (matmul_f64 if f64 else matmul_f32)(lhs_deq[s : s + n].T, rhs_deq[s : s + n])
        s += n
    return out


# ---------------------------------------------------------------------------
# comparison metrics used by the GEMM gates
# ---------------------------------------------------------------------------
def cosine(x: np.ndarray, y: np.ndarray) -> float:
    x = np.asarray(x, dtype=np.float64).ravel()
    y = np.asarray(y, dtype=np.float64).ravel()
    den = np.linalg.norm(x) * np.linalg.norm(y)
    return float(x @ y / den) if den > 0 else 1.0


def max_rel_err(ref: np.ndarray, y: np.ndarray) -> float:
    """max |y - ref| / max |ref| (error relative to the output's dynamic range)."""
    ref = np.asarray(ref, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    den = np.max(np.abs(ref))
    return float(np.max(np.abs(y - ref)) / den) if den > 0 else float(np.max(np.abs(y)))


def rel_fro(ref: np.ndarray, y: np.ndarray) -> float:
    """|y - ref|_F / |ref|_F, the reference tests' relative error
    (/root/reference/tests/pytorch/test_utils.py:43-45)."""
    ref = np.asarray(ref, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    den = np.linalg.norm(ref)
    return float(np.linalg.norm(y - ref) / den) if den > 0 else float(np.linalg.norm(y))


def elementwise_excess(ref: np.ndarray, y: np.ndarray, rtol: float = 2.0 ** -7) -> float:
    """max over elements of |y - ref| / (rtol |ref| + rtol rms(ref's row)); a result is inside the
    element-wise bound when this is <= 1. Unlike the range-relative maximum, an error of a few
    per cent of ONE small element (a wrong scale on one row block) fails it: every element is
    held to its own size plus a share of its row's typical size (1-D input: one row)."""
    ref = np.atleast_2d(np.asarray(ref, dtype=np.float64))
    y = np.atleast_2d(np.asarray(y, dtype=np.float64))
    ref2, y2 = ref.reshape(-1, ref.shape[-1]), y.reshape(-1, y.shape[-1])
    rms = np.sqrt(np.mean(ref2 * ref2, axis=1, keepdims=True))
    bound = rtol * np.abs(ref2) + rtol * rms
    err = np.abs(y2 - ref2)
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(bound > 0, err / bound, np.where(err > 0, np.inf, 0.0))
    return float(ratio.max()) if ratio.size else 0.0


def snr_db(ref: np.ndarray, y: np.ndarray) -> float:
    """10 log10(|ref|^2 / |ref - y|^2) (/root/reference/tests/pytorch/test_utils.py:76-80)."""
    ref = np.asarray(ref, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    return float(10 * np.log10(np.sum(ref * ref) / (np.sum((ref - y) ** 2) + 1e-12)))
