"""Pins for the oracle's attention: the SDPA three-call restatement against (1) the float64 dense
brute force, (2) torch's own causal SDPA on the concatenated real tokens with no mask tensor at all,
(3) invariants that a dropped term, wrong index or transposed operand would break."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import blockrank_oracle as orc


def make(lens, H, Nq, Nkv, D, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    lens = np.asarray(lens)
    B, M = lens.shape
    S = M * H
    q = torch.randn(B, Nq, S, D, generator=g).to(dtype)
    k = torch.randn(B, Nkv, S, D, generator=g).to(dtype)
    v = torch.randn(B, Nkv, S, D, generator=g).to(dtype)
    valid = orc.left_padded_valid(lens, H)
    return q, k, v, valid


def run_sdpa(q, k, v, valid, scale, **kw):
    m5 = orc.additive_mask(torch.as_tensor(valid), q.dtype)
    return orc.sdpa_blockrank_forward(q, k, v, m5, scale, **kw)


CASES = [
    ([[3, 4, 2, 3]], 4, 4, 2, 8),
    ([[5, 1, 8, 3, 2], [8, 8, 0, 4, 1]], 8, 6, 2, 4),
    ([[4]], 4, 2, 2, 8),
    ([[2, 3]], 4, 2, 1, 8),
    ([[7, 7, 7]], 7, 3, 3, 5),
]


@pytest.mark.parametrize("lens,H,Nq,Nkv,D", CASES)
def test_sdpa_restatement_vs_dense_bruteforce(lens, H, Nq, Nkv, D):
    q, k, v, valid = make(lens, H, Nq, Nkv, D)
    scale = D ** -0.5
    out, _ = run_sdpa(q, k, v, valid, scale)
    ref, _ = orc.dense_attention(q, k, v, valid, scale)
    rows = valid.reshape(valid.shape[0], -1)
    np.testing.assert_allclose(out.numpy()[rows], ref[rows], atol=2e-6, rtol=1e-5)
    assert np.isnan(ref[~rows]).all()


def test_segments_reduce_to_library_causal_sdpa():
    # no mask tensor anywhere on the right-hand side: concatenate the real tokens and use is_causal
    lens = [[5, 3, 8, 2, 4]]
    H, Nq, Nkv, D = 8, 4, 2, 16
    q, k, v, valid = make(lens, H, Nq, Nkv, D, seed=3)
    scale = 0.3
    out, _ = run_sdpa(q, k, v, valid, scale)
    out = out[0].transpose(0, 1)                       # (Nq, S, D)
    kk, vv = orc.repeat_kv(k, 2)[0], orc.repeat_kv(v, 2)[0]
    M = len(lens[0])

    def real(m):
        L = lens[0][m]
        return slice(m * H + H - L, (m + 1) * H)

    # prefix: plain causal over its real tokens
    r0 = real(0)
    exp = F.scaled_dot_product_attention(q[0][:, r0], kk[:, r0], vv[:, r0], is_causal=True, scale=scale)
    torch.testing.assert_close(out[:, r0], exp, atol=2e-6, rtol=1e-5)
    # document m: last d rows of causal attention over [prefix real ; doc real]
    for m in range(1, M - 1):
        rm = real(m)
        idx = list(range(r0.start, r0.stop)) + list(range(rm.start, rm.stop))
        exp = F.scaled_dot_product_attention(q[0][:, idx], kk[:, idx], vv[:, idx], is_causal=True, scale=scale)
        torch.testing.assert_close(out[:, rm], exp[:, -lens[0][m]:], atol=2e-6, rtol=1e-5)
    # query block: last rows of causal attention over every real token in order
    idx = [i for m in range(M) for i in range(real(m).start, real(m).stop)]
    exp = F.scaled_dot_product_attention(q[0][:, idx], kk[:, idx], vv[:, idx], is_causal=True, scale=scale)
    torch.testing.assert_close(out[:, real(M - 1)], exp[:, -lens[0][-1]:], atol=2e-6, rtol=1e-5)


def test_value_of_ones_gives_ones():
    q, k, v, valid = make([[3, 6, 2, 5]], 6, 4, 2, 8, seed=1)
    out, _ = run_sdpa(q, k, torch.ones_like(v), valid, 0.5)
    rows = torch.as_tensor(valid.reshape(1, -1))
    torch.testing.assert_close(out[rows], torch.ones_like(out[rows]))


def test_document_permutation_equivariance():
    lens = [[4, 3, 6, 2, 5]]
    H = 6
    q, k, v, valid = make(lens, H, 4, 2, 8, seed=2)
    out, _ = run_sdpa(q, k, v, valid, 0.4)
    perm = [0, 3, 1, 2, 4]                              # shuffle the three documents
    M = 5

    def shuffle(x):
        B, N, S, D = x.shape
        return x.view(B, N, M, H, D)[:, :, perm].reshape(B, N, S, D)

    valid_p = valid[:, perm]
    out_p, _ = run_sdpa(shuffle(q), shuffle(k), shuffle(v), valid_p, 0.4)
    out_b = out.view(1, M, H, 4, 8)[:, perm]
    rows = torch.as_tensor(valid_p)
    torch.testing.assert_close(out_p.view(1, M, H, 4, 8)[rows], out_b[rows], atol=2e-6, rtol=1e-5)


def test_gqa_equals_explicit_expansion():
    q, k, v, valid = make([[3, 4, 4, 2]], 4, 6, 2, 8, seed=4)
    a, _ = run_sdpa(q, k, v, valid, 0.35)
    b, _ = run_sdpa(q, orc.repeat_kv(k, 3), orc.repeat_kv(v, 3), valid, 0.35)
    torch.testing.assert_close(a, b)
    # head n must read kv head n // G, not n % Nkv: make kv heads very different and check one head
    ref, _ = orc.dense_attention(q, k, v, valid, 0.35)
    rows = valid.reshape(1, -1)
    np.testing.assert_allclose(a.numpy()[rows], ref[rows], atol=2e-6, rtol=1e-5)


def test_padding_content_is_never_read():
    lens = [[2, 5, 3, 4]]
    H = 6
    q, k, v, valid = make(lens, H, 2, 2, 8, seed=5)
    a, _ = run_sdpa(q, k, v, valid, 0.5)
    pad = torch.as_tensor(~valid.reshape(1, 1, -1, 1))
    q2 = torch.where(pad, torch.full_like(q, 37.0), q)
    k2 = torch.where(pad, torch.full_like(k, -51.0), k)
    v2 = torch.where(pad, torch.full_like(v, 1e4), v)
    b, _ = run_sdpa(q2, k2, v2, valid, 0.5)
    rows = torch.as_tensor(valid.reshape(1, -1))
    torch.testing.assert_close(a[rows], b[rows])


def test_single_block_is_plain_causal():
    q, k, v, valid = make([[6]], 6, 2, 2, 8, seed=6)
    out, s = run_sdpa(q, k, v, valid, 0.5, return_scores=True)
    assert s is None
    exp = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.5).transpose(1, 2)
    torch.testing.assert_close(out, exp, atol=2e-6, rtol=1e-5)


def test_last_block_logits_closed_form_and_scaling_variants():
    lens = [[3, 4, 2, 4]]
    H, D = 4, 8
    q, k, v, valid = make(lens, H, 4, 2, D, seed=7)
    scale = 0.25
    _, s_scaled = run_sdpa(q, k, v, valid, scale, return_scores=True, num_last_queries=3)
    _, s_raw = run_sdpa(q, k, v, valid, scale, return_scores=True, num_last_queries=3, scaled_scores=False)
    cf = orc.last_block_logits(q, k, valid, scale, 3)
    _, dense_logits = orc.dense_attention(q, k, v, valid, scale)
    ok = orc.allowed(valid)[:, -3:, :]
    assert s_scaled.shape == (1, 4, 3, 16)
    # allowed entries: the plain scaled dot product; the rest: pushed to about NEG
    np.testing.assert_allclose(s_scaled.numpy()[:, :, ok[0]], dense_logits[:, :, -3:, :][:, :, ok[0]], atol=1e-5)
    np.testing.assert_allclose(s_raw.numpy()[:, :, ok[0]] * scale, dense_logits[:, :, -3:, :][:, :, ok[0]], atol=1e-5)
    np.testing.assert_allclose(cf[:, :, ok[0]], dense_logits[:, :, -3:, :][:, :, ok[0]], atol=1e-12)
    assert (s_scaled.numpy()[:, :, ~ok[0]] < -1e37).all() and (cf[:, :, ~ok[0]] < -1e37).all()
    # num_last_queries larger than H falls back to the whole block (blockrank_std_attention.py:642)
    _, s_all = run_sdpa(q, k, v, valid, scale, return_scores=True, num_last_queries=16)
    assert s_all.shape[2] == H


def test_bf16_runs_and_is_close_to_float64():
    q, k, v, valid = make([[5, 8, 3, 6]], 8, 4, 2, 16, seed=8, dtype=torch.bfloat16)
    out, _ = run_sdpa(q, k, v, valid, 0.25)
    ref, _ = orc.dense_attention(q.float(), k.float(), v.float(), valid, 0.25)
    rows = valid.reshape(1, -1)
    assert np.abs(out.float().numpy()[rows] - ref[rows]).max() < 2e-2
