"""Pins for oracle/activation.py: the gradients against central finite differences of the forward
formula, closed-form values, and PyTorch's own silu / gelu on the CPU."""

import numpy as np
import pytest
import torch

from oracle import activation as A


@pytest.mark.parametrize("kind", ["silu", "gelu"])
def test_forward_matches_torch_and_closed_forms(kind):
    g = np.linspace(-8, 8, 401)
    ref = (torch.nn.functional.silu if kind == "silu" else torch.nn.functional.gelu)(torch.from_numpy(g)).numpy()
    assert np.allclose(A.act(g, kind), ref, rtol=1e-12, atol=1e-14)
    assert A.act(np.array([0.0]), kind)[0] == 0.0
    assert abs(A.act_grad(np.array([0.0]), kind)[0] - 0.5) < 1e-15
    big = A.act(np.array([30.0, -30.0]), kind)
    assert abs(big[0] - 30.0) < 1e-9 and abs(big[1]) < 1e-9


@pytest.mark.parametrize("kind", ["silu", "gelu"])
def test_gradients_by_finite_differences(kind):
    rng = np.random.default_rng(3)
    T, H = 5, 7
    x, p, go = rng.standard_normal((T, 2 * H)), rng.random(T) + 0.1, rng.standard_normal((T, H))
    mask = np.array([1, 1, 0, 1, 1])
    gx, gp = A.glu_with_probs_grad(go, x, p, kind, mask)
    f = lambda xx, pp: float((A.glu_with_probs(xx, pp, kind, mask) * go).sum())  # noqa: E731
    eps = 1e-6
    for t, c in [(0, 0), (1, 3), (3, H + 2), (4, 2 * H - 1), (2, 1)]:
        d = np.zeros_like(x)
        d[t, c] = eps
        assert abs((f(x + d, p) - f(x - d, p)) / (2 * eps) - gx[t, c]) < 1e-7
    for t in range(T):
        d = np.zeros_like(p)
        d[t] = eps
        assert abs((f(x, p + d) - f(x, p - d)) / (2 * eps) - gp[t]) < 1e-7
    assert not gx[2].any() and gp[2] == 0  # masked row
