"""The benchmark configurations with ragged documents at their full size, through the attention hook and the
loss API, against the CPU oracle: attention output within 2e-2 max-abs on rows of real tokens, per-document
scores within 1e-3 relative with the same top-10 (reference: sdpa_blockrank_attention_forward,
src/blockrank/blockrank_std_attention.py:472-650, and compute_auxiliary_attention_loss, src/blockrank/losses.py:37-78).

  * ranking batch of the end-to-end configuration: B = 8, 64-token prefix + 20 documents U[96, 224] + 32-token
    query, one Mistral-7B-shaped attention layer (projections + RoPE with the BlockRank position ids);
  * long list: B = 1, 64-token prefix + 100 documents U[64, 384] + 48-token query, scores over all 100 documents
    (the reduction path for more than 64 documents, a query walk of about 360 key tiles split into chunks).
"""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc
from tests._util import assert_scores_close, max_abs_on_real_rows, oracle_attention, oracle_doc_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NQ, NKV, D, HIDDEN = 32, 8, 128, 4096


class _Layer:
    layer_idx = 20
    num_key_value_groups = NQ // NKV
    training = False


def _hook_step(lay):
    q, k, v = synthetic.attention_layer_inputs(lay, NQ, NKV, D, HIDDEN, torch.bfloat16, DEV)
    valid = lay.valid.to(DEV)
    mask = br.blockrank_attention_mask(batch_size=lay.B, attention_mask=valid, dtype=torch.bfloat16)
    out, handle = br.blockrank_attention_forward(_Layer(), q, k, v, mask, D ** -0.5, layers_to_return_scores=[20])
    assert handle.partials is not None, "bf16 inputs take the fused score path"
    scores = br.compute_auxiliary_attention_loss(handle, lay.labels.to(DEV), valid, answer_ids=None, return_logits=True)
    torch.cuda.synchronize()
    return q, k, v, out, scores


def test_ranking_batch_of_ragged_documents_full_size():
    lay = synthetic.random_layout(8, 64, 20, 96, 224, 32, seed=0)
    assert (lay.B, lay.M, lay.H) == (8, 22, 224) and lay.lengths[:, 1:-1].min() >= 96
    q, k, v, out, scores = _hook_step(lay)
    want = oracle_attention(q, k, v, lay, D ** -0.5)
    assert max_abs_on_real_rows(out, want, lay) <= 2e-2
    want_s = oracle_doc_scores(q, k, lay, D ** -0.5)
    assert scores.shape == (8, 20)
    assert_scores_close(scores, want_s)
    np.testing.assert_array_equal(br.rank_documents(scores).cpu().numpy(), orc.topk_indices(want_s, 10))


def test_long_list_scores_and_output_full_size():
    lay = synthetic.random_layout(1, 64, 100, 64, 384, 48, seed=0)
    assert (lay.M, lay.H, lay.S) == (102, 384, 39168) and lay.valid_tokens == 22804
    q, k, v, out, scores = _hook_step(lay)
    want_s = oracle_doc_scores(q, k, lay, D ** -0.5)
    assert scores.shape == (1, 100)
    assert_scores_close(scores, want_s)
    np.testing.assert_array_equal(br.rank_documents(scores).cpu().numpy(), orc.topk_indices(want_s, 10))
    np.testing.assert_allclose(scores.sum(-1).cpu().numpy() * 0.05, 1.0, rtol=1e-4)
    want = oracle_attention(q, k, v, lay, D ** -0.5)
    assert max_abs_on_real_rows(out, want, lay) <= 2e-2
