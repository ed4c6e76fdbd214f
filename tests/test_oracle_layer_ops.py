"""Pins of the oracle's RMSNorm and SiLU-gate restatements (third-party functions the reference reaches through the
model forward): closed forms and the library's own routines."""
import numpy as np
import torch

from oracle import blockrank_oracle as orc


def test_rms_norm_closed_forms():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 64)) * rng.uniform(0.1, 30.0, size=(5, 1))
    y = orc.rms_norm(x, np.ones(64), 0.0)
    np.testing.assert_allclose((y * y).mean(axis=-1), 1.0, rtol=1e-12)               # unit mean square
    np.testing.assert_allclose(orc.rms_norm(7.5 * x, np.ones(64), 0.0), y, rtol=1e-12)  # scale invariance
    w = rng.standard_normal(64)
    np.testing.assert_allclose(orc.rms_norm(np.full((1, 64), -3.0), w, 0.0), -w[None], rtol=1e-12)   # constant row
    # eps enters under the root: a zero row stays zero, a tiny row is damped
    assert (orc.rms_norm(np.zeros((1, 64)), w, 1e-6) == 0).all()
    np.testing.assert_allclose(orc.rms_norm(np.full((1, 64), 1e-3), np.ones(64), 1e-6), 1e-3 / np.sqrt(2e-6), rtol=1e-12)


def test_rms_norm_matches_the_published_expression_in_torch():
    rng = np.random.default_rng(1)
    x, w = rng.standard_normal((3, 7, 32)), rng.standard_normal(32)
    t = torch.from_numpy(x)
    want = torch.from_numpy(w) * (t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-5))
    np.testing.assert_allclose(orc.rms_norm(x, w, 1e-5), want.numpy(), rtol=1e-12)


def test_silu_mul():
    g = np.linspace(-20, 20, 401)
    u = np.ones_like(g)
    s = orc.silu_mul(g, u)
    assert s[200] == 0.0                                                     # silu(0) = 0
    np.testing.assert_allclose(s - s[::-1], g, atol=1e-12)                   # silu(g) - silu(-g) = g
    assert abs(s[-1] - 20.0) < 1e-7                                          # -> g for large g
    np.testing.assert_allclose(s, torch.nn.functional.silu(torch.from_numpy(g)).numpy(), rtol=1e-12, atol=1e-15)
    rng = np.random.default_rng(2)
    a, b = rng.standard_normal(50), rng.standard_normal(50)
    np.testing.assert_allclose(orc.silu_mul(a, b), orc.silu_mul(a, np.ones(50)) * b, rtol=1e-15)
