"""Pins of the oracle's closed-form attention gradients: central finite differences of the float64 brute-force
forward (catches a dropped term or a wrong sign), torch autograd through the library-SDPA restatement of the
reference's three-call algorithm (catches a transposed operand or a wrong head reduction), and the
log-sum-exp against the dense logits."""
import numpy as np
import torch

from oracle import blockrank_oracle as orc


def _case(seed, lengths, H, Nq, Nkv, D):
    rng = np.random.default_rng(seed)
    valid = orc.left_padded_valid(lengths, H)
    B, M, _ = valid.shape
    S = M * H
    q = rng.standard_normal((B, Nq, S, D))
    k = rng.standard_normal((B, Nkv, S, D))
    v = rng.standard_normal((B, Nkv, S, D))
    dout = rng.standard_normal((B, S, Nq, D))
    return valid, q, k, v, dout


def _loss(q, k, v, dout, valid, scale):
    out, _ = orc.dense_attention(q, k, v, valid, scale)
    rows = valid.reshape(valid.shape[0], -1)
    return float((out[rows] * dout[rows]).sum())


def test_gradients_match_finite_differences():
    valid, q, k, v, dout = _case(0, [[3, 4, 2, 3], [1, 0, 4, 2]], 4, 4, 2, 3)
    scale = 0.7
    dq, dk, dv, _ = orc.dense_attention_backward(q, k, v, dout, valid, scale)
    rng = np.random.default_rng(1)
    eps = 1e-5
    for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for _ in range(40):
            idx = tuple(rng.integers(0, n) for n in x.shape)
            old = x[idx]
            x[idx] = old + eps
            up = _loss(q, k, v, dout, valid, scale)
            x[idx] = old - eps
            dn = _loss(q, k, v, dout, valid, scale)
            x[idx] = old
            fd = (up - dn) / (2 * eps)
            assert abs(fd - g[idx]) <= 1e-6 * max(1.0, abs(fd)), f"d{name}{idx}: finite difference {fd}, closed form {g[idx]}"


def test_gradients_match_autograd_through_library_sdpa():
    valid, q, k, v, dout = _case(2, [[5, 8, 3, 0, 6], [2, 7, 8, 1, 4]], 8, 6, 2, 4)
    scale = 0.5
    dq, dk, dv, _ = orc.dense_attention_backward(q, k, v, dout, valid, scale)
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    m5 = orc.additive_mask(torch.from_numpy(valid), torch.float64)
    out, _ = orc.sdpa_blockrank_forward(tq, tk, tv, m5, scale)
    rows = torch.from_numpy(valid.reshape(valid.shape[0], -1))
    (out[rows] * torch.from_numpy(dout)[rows]).sum().backward()
    real = valid.reshape(valid.shape[0], 1, -1, 1)
    # padded query rows: the reference's uniform average there feeds nothing (their dout is excluded above)
    np.testing.assert_allclose(dq * real, tq.grad.numpy() * real, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(dk * real, tk.grad.numpy() * real, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(dv * real, tv.grad.numpy() * real, rtol=1e-9, atol=1e-10)
    # and padded keys receive nothing at all
    assert (dk * ~real == 0).all() and (dv * ~real == 0).all() and (dq * ~real == 0).all()


def test_log_sum_exp_against_dense_logits():
    valid, q, k, v, dout = _case(3, [[2, 5, 4]], 5, 2, 1, 4)
    scale = 0.3
    *_, lse = orc.dense_attention_backward(q, k, v, dout, valid, scale)
    _, logits = orc.dense_attention(q, k, v, valid, scale)
    ok = orc.allowed(valid)
    want = torch.logsumexp(torch.from_numpy(np.where(ok[:, None], logits, -np.inf)), dim=-1).numpy()
    rows = valid.reshape(1, 1, -1).repeat(2, axis=1)
    np.testing.assert_allclose(lse[rows], want[rows], rtol=1e-12)
    assert np.isnan(lse[~rows]).all()
