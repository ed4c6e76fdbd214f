"""Pins for the oracle's mask: the reference states the mask twice (additive builder + segment
composition, blockrank_std_attention.py:293-309/:581-588/:607-614, and the flex predicate, :344-399);
both restatements must agree, and both must agree with a hand-written tiny case."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import blockrank_oracle as orc


@st.composite
def layouts(draw):
    B = draw(st.integers(1, 3))
    M = draw(st.integers(1, 6))
    H = draw(st.integers(1, 9))
    lens = [[draw(st.integers(0, H)) for _ in range(M)] for _ in range(B)]
    return np.array(lens), H


@settings(max_examples=60, deadline=None)
@given(layouts())
def test_predicate_equals_segment_composition(lay):
    lens, H = lay
    valid = orc.left_padded_valid(lens, H)
    np.testing.assert_array_equal(orc.allowed(valid), orc.allowed_from_segments(valid))


@settings(max_examples=30, deadline=None)
@given(layouts(), st.integers(0, 2**31 - 1))
def test_predicate_equals_segments_arbitrary_validity(lay, seed):
    # the reference's mask builder does not require left padding; neither restatement may
    lens, H = lay
    rng = np.random.default_rng(seed)
    valid = rng.random((lens.shape[0], lens.shape[1], H)) < 0.7
    # rows of real tokens only: on a padded query slot that follows a real key the additive mask
    # keeps the key visible while the predicate hides it; nothing consumes such rows
    rows = valid.reshape(valid.shape[0], -1)
    np.testing.assert_array_equal(orc.allowed(valid)[rows], orc.allowed_from_segments(valid)[rows])


def test_hand_written_case():
    # M=3, H=2: prefix len 1 (slot 1), doc len 2, query len 1 (slot 5).  Tokens: 1 | 2 3 | 5
    valid = orc.left_padded_valid([[1, 2, 1]], 2)
    a = orc.allowed(valid)[0]
    expect = np.zeros((6, 6), dtype=bool)
    expect[1, 1] = True                      # prefix token sees itself
    expect[2, [1, 2]] = True                 # doc token 0: prefix + itself
    expect[3, [1, 2, 3]] = True              # doc token 1: prefix + doc causal
    expect[5, [1, 2, 3, 5]] = True           # query: everything real before + itself
    np.testing.assert_array_equal(a, expect)


def test_additive_mask_values():
    valid = torch.as_tensor(orc.left_padded_valid([[2, 3]], 3))
    for dt in (torch.float32, torch.bfloat16):
        m = orc.additive_mask(valid, dt)
        assert m.shape == (1, 1, 2, 3, 3) and m.dtype == dt
        neg = 0.7 * torch.finfo(dt).min
        assert torch.isfinite(m).all()
        assert set(m.float().unique().tolist()) == {0.0, float(torch.tensor(neg, dtype=dt))}
        # block 0 has slots 1,2 real: row 2 sees keys 1,2; row 0 (padding) sees nothing
        assert (m[0, 0, 0, 2] == 0).tolist() == [False, True, True]
        assert (m[0, 0, 0, 0] == 0).tolist() == [False, False, False]


@pytest.mark.parametrize("M", [1, 2, 3, 5])
def test_block_counts(M):
    H = 4
    valid = orc.left_padded_valid([[H] * M], H)
    a = orc.allowed(valid)[0]
    S = M * H
    tri = H * (H + 1) // 2
    if M == 1:
        assert a.sum() == tri
    else:
        # prefix causal + docs (prefix + causal) + query (all earlier + causal)
        assert a.sum() == tri + (M - 2) * (H * H + tri) + (H * (M - 1) * H + tri)
    assert not a[:, :][np.triu_indices(S, 1)].any()      # never looks ahead in sequence order
