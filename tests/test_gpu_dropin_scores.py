"""The attention hook called the way the reference's callers call it (scripts/eval_attn.py:139: no extra keyword,
labels not visible to the hook) and its result consumed the way they consume it (losses.py:37-78).

  * the hook guesses the score rows (the last two positions, what losses.py:43-48 yields in evaluation) and reduces
    their scores inside the attention call; the loss function confirms the guess with the labels and returns them;
  * a wrong guess (answers after the "[") still gives the oracle's scores;
  * the handle in place of the s_last tensor behaves as that tensor for a consumer that knows nothing of this
    package: the reference's formula, restated here, runs on it unchanged."""
import pytest
import torch
import torch.nn.functional as F

import blockrank_amd as br
from blockrank_amd import attention as att, losses, synthetic
from tests._util import assert_scores_close, oracle_doc_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class Mod:
    layer_idx = 20
    num_key_value_groups = 4
    training = False


def _setup(seed, bracket_from_end):
    lay = synthetic.random_layout(3, 24, 9, 10, 120, 30, seed=seed)
    lay.labels[:] = -100
    lay.labels[:, -bracket_from_end:] = 7            # "[" sits bracket_from_end tokens before the end
    q, k, v = synthetic.random_qkv(lay, 8, 2, 128, torch.bfloat16, DEV, seed=seed)
    mask = br.blockrank_attention_mask(batch_size=lay.B, attention_mask=lay.valid.to(DEV), dtype=torch.bfloat16)
    return lay, q, k, v, mask, 128 ** -0.5


def stranger_loss(attention_scores, labels, attention_mask, temperature=0.05):
    """The formula of losses.py:37-78, written against nothing but the tensor protocol."""
    B, M, H = attention_mask.shape
    _, N, h1, MH = attention_scores.shape
    assert MH == M * H
    first = (labels[:, -h1:] > -100).int().argmax(dim=-1)[:, None]
    idx = torch.hstack([first - 1, first])
    assert torch.all(idx >= 0)
    x = attention_scores.take_along_dim(idx[:, None, :, None], dim=2)
    x = x[..., H:-H]
    p = F.softmax(x, dim=-1).reshape(B, N, -1, M - 2, H)
    return p.mean(dim=(1, 2)).sum(dim=-1) / temperature


def test_right_guess_returns_the_scores_of_the_attention_call():
    lay, q, k, v, mask, scale = _setup(1, 1)
    out, handle = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[20])
    assert handle.speculative and handle.ranked is not None
    got = losses.compute_auxiliary_attention_loss(handle, lay.labels.to(DEV), lay.valid.to(DEV), return_logits=True)
    assert got is handle.ranked[2], "a confirmed guess must not cost another launch"
    assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
    # same values as the route that never guesses
    _, plain = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[20], speculate_score_rows=False)
    assert not plain.speculative and plain.ranked is None
    want = losses.compute_auxiliary_attention_loss(plain, lay.labels.to(DEV), lay.valid.to(DEV), return_logits=True)
    assert torch.equal(got, want)
    # asking the handle directly with a rows tensor of its own: compared once, then remembered
    rows = torch.tensor([[14, 15]] * lay.B, dtype=torch.int32, device=DEV)
    assert handle.doc_scores_window(rows) is handle.ranked[2]
    rows[0, 0] = 3                                   # changed in place: no longer the guess
    other = handle.doc_scores_window(rows)
    assert other is not handle.ranked[2] and not torch.equal(other, got)


def test_wrong_guess_still_gives_the_oracles_scores():
    lay, q, k, v, mask, scale = _setup(2, 4)         # answers follow the "[": the rows are not the last two
    out, handle = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[20])
    assert handle.speculative
    got = losses.compute_auxiliary_attention_loss(handle, lay.labels.to(DEV), lay.valid.to(DEV), return_logits=True)
    assert got is not handle.ranked[2]
    assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
    # and the guess did not disturb the attention output
    out2, _ = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[20], speculate_score_rows=False)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("bracket_from_end", [1, 5])
def test_handle_serves_a_consumer_that_only_knows_tensors(bracket_from_end):
    lay, q, k, v, mask, scale = _setup(3, bracket_from_end)
    _, handle = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[20])
    got = stranger_loss(handle, lay.labels.to(DEV), lay.valid.to(DEV))
    assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
    assert handle._dense is None, "take_along_dim over the rows must not have materialised all sixteen"
    # the rest of the protocol: shape, indexing, methods, torch functions - all on the (B, Nq, 16, S) fp32 logits
    dense = handle.dense()
    assert tuple(handle.shape) == tuple(dense.shape) and handle.dim() == 4 and handle.size(2) == 16 and handle.dtype == dense.dtype
    assert torch.equal(handle[..., 5:9], dense[..., 5:9])
    assert torch.equal(handle.float().cpu(), dense.cpu())
    assert torch.equal(torch.softmax(handle, dim=-1), torch.softmax(dense, dim=-1))
    assert torch.equal(handle + 1.0, dense + 1.0)
    assert torch.equal(stranger_loss(dense, lay.labels.to(DEV), lay.valid.to(DEV)), got)
