"""Pins for the oracle's per-document score (losses.py:37-78) and top-k."""
import numpy as np
import pytest
import torch

from oracle import blockrank_oracle as orc


def layout(lens, H):
    valid = orc.left_padded_valid(lens, H)
    return valid, orc.eval_labels(valid)


def test_zero_query_gives_length_shares():
    # q = 0 => every real document token has the same logit => document i gets len_i / sum(len)
    lens = [[3, 2, 5, 1, 4]]
    H = 5
    valid, labels = layout(lens, H)
    B, M = 1, 5
    k = np.random.default_rng(0).normal(size=(B, 2, M * H, 8))
    q = np.zeros((B, 4, M * H, 8))
    tau = 0.05
    s = orc.doc_scores(q, k, valid, labels, 0.3, temperature=tau)
    np.testing.assert_allclose(s[0] * tau, np.array([2, 5, 1]) / 8.0, rtol=1e-12)


def test_scores_sum_to_one_over_tau_and_are_nonnegative():
    lens = [[4, 3, 6, 2, 5], [6, 6, 1, 4, 3]]
    H = 6
    valid, labels = layout(lens, H)
    rng = np.random.default_rng(1)
    q = rng.normal(size=(2, 4, 5 * H, 8))
    k = rng.normal(size=(2, 2, 5 * H, 8))
    s = orc.doc_scores(q, k, valid, labels, 0.35, temperature=0.05)
    assert (s >= 0).all()
    np.testing.assert_allclose(s.sum(-1) * 0.05, 1.0, rtol=1e-12)


def test_hand_computed_two_documents():
    # one head, D=1, H=2, M=4; real tokens: prefix 1, doc A 2 tokens, doc B 1 token, query 2 tokens.
    H, M = 2, 4
    valid, labels = layout([[1, 2, 1, 2]], H)
    q = np.zeros((1, 1, M * H, 1))
    k = np.zeros((1, 1, M * H, 1))
    q[0, 0, 6, 0], q[0, 0, 7, 0] = 1.0, 2.0            # rows bracket-1 and bracket
    k[0, 0, 2, 0], k[0, 0, 3, 0] = np.log(2.0), np.log(3.0)   # doc A keys
    k[0, 0, 4, 0] = 100.0                              # padding slot of doc B: must be ignored
    k[0, 0, 5, 0] = np.log(5.0)                        # doc B key
    s = orc.doc_scores(q, k, valid, labels, 1.0, temperature=1.0, num_last_queries=2)
    # row 6: weights 2,3 | 5 -> A = 5/10 ; row 7: weights 4,9 | 25 -> A = 13/38 ; mean over the two rows
    np.testing.assert_allclose(s[0], [(0.5 + 13 / 38) / 2, (0.5 + 25 / 38) / 2], rtol=1e-12)


def test_document_permutation_equivariance():
    lens = [[3, 4, 2, 6, 3]]
    H = 6
    valid, labels = layout(lens, H)
    rng = np.random.default_rng(2)
    q = rng.normal(size=(1, 2, 5 * H, 4))
    k = rng.normal(size=(1, 2, 5 * H, 4))
    s = orc.doc_scores(q, k, valid, labels, 0.5)
    perm = [0, 2, 3, 1, 4]
    kp = k.reshape(1, 2, 5, H, 4)[:, :, perm].reshape(1, 2, 5 * H, 4)
    sp = orc.doc_scores(q, kp, valid[:, perm], labels, 0.5)
    np.testing.assert_allclose(sp[0], s[0][[1, 2, 0]], rtol=1e-10)


def test_bracket_rows_follow_labels():
    H, M = 8, 3
    labels = np.full((2, M * H), -100)
    labels[0, -1] = 7                    # eval: "[" is the last token -> rows (h1-2, h1-1)
    labels[1, -5:] = 3                   # training: "[" followed by 4 answer tokens
    rows = orc.bracket_rows(labels, 8)
    assert rows.tolist() == [[6, 7], [2, 3]]
    labels[1, -8:] = 3                   # bracket at index 0 -> the row before it does not exist
    with pytest.raises(AssertionError):
        orc.bracket_rows(labels, 8)


def test_from_logits_matches_torch_formula_on_full_tensor():
    # the same reduction written with torch ops on a random (B,N,h1,S) tensor
    rng = np.random.default_rng(3)
    B, N, h1, M, H = 2, 3, 4, 5, 4
    s = rng.normal(size=(B, N, h1, M * H))
    valid = np.ones((B, M, H), dtype=bool)
    labels = np.full((B, M * H), -100)
    labels[0, -1] = 1
    labels[1, -2:] = 1
    got = orc.doc_scores_from_logits(s, labels, valid, 0.1)
    t = torch.as_tensor(s)
    rows = torch.as_tensor(orc.bracket_rows(labels, h1))
    x = t.take_along_dim(rows[:, None, :, None], dim=2)[..., H:-H]
    p = torch.softmax(x, -1).reshape(B, N, 2, M - 2, H)
    exp = (p.mean(dim=(1, 2)).sum(-1) / 0.1).numpy()
    np.testing.assert_allclose(got, exp, rtol=1e-12)


def test_topk_is_stable_descending():
    s = np.array([[0.1, 0.9, 0.9, 0.3], [3.0, 1.0, 2.0, 2.0]])
    assert orc.topk_indices(s, 3).tolist() == [[1, 2, 3], [0, 2, 3]]
    assert orc.topk_indices(s, 10).shape == (2, 4)


def test_fp8_quantiser_pins():
    """quantize_fp8_e4m3: values with at most four significant bits survive, the relative round-trip error of
    normal values is at most 2^-4, a power-of-two factor passes through, padded positions come back as zero."""
    import torch
    from oracle import blockrank_oracle as orc
    valid = torch.ones(1, 2, 4, dtype=torch.bool)
    valid[0, 0, 0] = False
    # four significant bits, the largest (240) sets the scale 2^0; 2^-6 is e4m3's smallest normal value
    vals = torch.tensor([0.0, 240.0, -208.0, 1.0, 0.875, 2.0 ** -6, 3.5, -120.0])
    for factor in (1.0, 2.0 ** -11, 2.0 ** 5):        # any power-of-two factor must cancel
        x = torch.zeros(1, 1, 8, 4)
        x[0, 0, :, 0] = vals * factor
        x[0, 0, 0, :] = 1e6                           # padded position: must not set the scale
        got = orc.quantize_fp8_e4m3(x, valid)
        assert torch.equal(got[0, 0, 0], torch.zeros(4))
        assert torch.equal(got[0, 0, 1:, 0], x[0, 0, 1:, 0])
    # five significant bits are rounded to four, ties to even: 17 -> 16, 19 -> 20, 18.5 -> 18
    x = torch.zeros(1, 1, 8, 4)
    x[0, 0, 1:5, 0] = torch.tensor([128.0, 17.0, 19.0, 18.5])
    got = orc.quantize_fp8_e4m3(x, valid)
    assert got[0, 0, 1:5, 0].tolist() == [128.0, 16.0, 20.0, 18.0]
    g = torch.Generator().manual_seed(0)
    y = torch.randn(2, 3, 8, 16, generator=g)
    v2 = torch.ones(2, 2, 4, dtype=torch.bool)
    for per_row in (False, True):
        r = orc.quantize_fp8_e4m3(y, v2, per_row=per_row)
        amax = y.abs().amax(dim=(3,) if per_row else (2, 3), keepdim=True)
        normal = y.abs() >= amax * 2.0 ** -13          # max / 2^7 >= 1 = 2^6 times the smallest normal value
        rel = ((r - y).abs() / y.abs())[normal.expand_as(y)]
        assert rel.max().item() <= 2.0 ** -4 + 1e-6
        assert torch.equal(orc.quantize_fp8_e4m3(y * 2.0 ** -9, v2, per_row=per_row) * 2.0 ** 9, r)
    # one scale per row: a row of tiny values keeps its relative precision
    tiny = y.clone()
    tiny[:, :, 3] *= 2.0 ** -14
    rt = orc.quantize_fp8_e4m3(tiny, v2, per_row=True)
    assert torch.equal(rt[:, :, 3] * 2.0 ** 14, orc.quantize_fp8_e4m3(y, v2, per_row=True)[:, :, 3])
