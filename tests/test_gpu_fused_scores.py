"""Score partials left by the prefill kernel: per-document scores from them must equal the stand-alone
score kernels and the float64 oracle (src/blockrank/losses.py:37-78) to 1e-3 relative with the same
top-10, and asking for them must not change the attention output."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import attention as att, losses, synthetic
from tests._util import assert_scores_close, oracle_doc_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _lay(kind):
    if kind == "small":
        return synthetic.random_layout(2, 20, 4, 1, 96, 24, seed=0), 8, 2, 64
    if kind == "headline":
        return synthetic.uniform_layout(4, 64, 20, 160, 32), 32, 8, 128
    if kind == "many_docs":          # more than 64 documents: the general reduction path
        return synthetic.random_layout(1, 30, 70, 5, 64, 20, seed=2), 8, 8, 128
    if kind == "long_blocks":        # blocks longer than 8 tiles: the general reduction path
        return synthetic.random_layout(2, 100, 3, 200, 600, 40, seed=3), 4, 1, 64
    if kind == "one_doc":
        return synthetic.random_layout(3, 7, 1, 3, 40, 17, seed=4), 6, 2, 64
    if kind == "empty_doc":
        return synthetic.make_layout([[5, 17, 0, 300, 33, 19], [40, 1, 65, 31, 2, 70]]), 8, 2, 128
    raise KeyError(kind)


@pytest.mark.parametrize("kind", ["small", "headline", "many_docs", "long_blocks", "one_doc", "empty_doc"])
def test_partials_match_standalone_kernels_and_oracle(kind):
    lay, Nq, Nkv, D = _lay(kind)
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=7)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    scale = D ** -0.5
    H, B, M = lay.H, lay.B, lay.M
    R = min(16, H)
    out_plain = br.blockrank_attention(q, k, v, mask, scale)
    out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R)
    assert torch.equal(out, out_plain), "asking for score partials must not change the attention output"
    # the rows the eval recipe uses: the last two positions
    rows = torch.tensor([[R - 2, R - 1]] * B, dtype=torch.int32, device=DEV)
    got, got_p = br.doc_scores_from_partials(part, mask, rows, R, Nq, Nkv, return_probs=True)
    want, want_p = br.doc_scores(q, k, mask, rows + (H - R), scale, return_probs=True)
    torch.testing.assert_close(got_p, want_p, rtol=1e-3, atol=1e-6)
    torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-5)
    assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
    # any other pair of rows inside the window
    g = torch.Generator().manual_seed(1)
    rows2 = torch.stack([torch.randperm(R, generator=g)[:2] for _ in range(B)]).to(torch.int32).to(DEV)
    got2 = br.doc_scores_from_partials(part, mask, rows2, R, Nq, Nkv)
    want2 = br.doc_scores(q, k, mask, rows2 + (H - R), scale)
    torch.testing.assert_close(got2, want2, rtol=1e-3, atol=1e-5)


def test_hook_takes_fused_path_and_loss_api_agrees():
    lay = synthetic.random_layout(2, 16, 6, 8, 80, 30, seed=11)
    lay.labels[:] = -100
    lay.labels[:, -3:] = 5                     # "[" sits three from the end
    Nq, Nkv, D = 8, 2, 64
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=11)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    scale = D ** -0.5

    class Mod:
        layer_idx = 3
        num_key_value_groups = Nq // Nkv
        training = False

    out, handle = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[3])
    assert handle.partials is not None, "the hook must take the fused path for bf16"
    got = losses.compute_auxiliary_attention_loss(handle, lay.labels.to(DEV), lay.valid.to(DEV), return_logits=True)
    assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
    dense = losses.compute_auxiliary_attention_loss(handle.dense(), lay.labels.to(DEV), lay.valid.to(DEV), return_logits=True)
    torch.testing.assert_close(got, dense, rtol=1e-3, atol=1e-5)
    # a layer that is not asked for scores returns none and the same output
    out2, none = att.blockrank_attention_forward(Mod(), q, k, v, mask, scale, layers_to_return_scores=[4])
    assert none is None and torch.equal(out, out2)
    # fp32 inputs keep the stand-alone kernels
    _, h32 = att.blockrank_attention_forward(Mod(), q.float(), k.float(), v.float(), br.BlockMask(lay.valid.to(DEV)), scale,
                                             layers_to_return_scores=[3])
    assert h32.partials is None
    got32 = losses.compute_auxiliary_attention_loss(h32, lay.labels.to(DEV), lay.valid.to(DEV), return_logits=True)
    assert_scores_close(got32, oracle_doc_scores(q, k, lay, scale))


def test_window_rows_on_padding_give_uniform():
    # query block of 5 real tokens: most of the 16-row window is padding
    lay = synthetic.make_layout([[10, 30, 64, 7, 5], [3, 64, 1, 20, 40]])
    Nq, Nkv, D = 4, 2, 64
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=5)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    scale = D ** -0.5
    H, M = lay.H, lay.M
    _, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=16)
    rows = torch.tensor([[0, 15], [14, 15]], dtype=torch.int32, device=DEV)
    got, got_p = br.doc_scores_from_partials(part, mask, rows, 16, Nq, Nkv, return_probs=True)
    want, want_p = br.doc_scores(q, k, mask, rows + (H - 16), scale, return_probs=True)
    torch.testing.assert_close(got_p, want_p, rtol=1e-3, atol=1e-6)
    torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-5)
    assert torch.allclose(got_p[0, :, 0], torch.full_like(got_p[0, :, 0], 1.0 / (M - 2)))


def test_partials_argument_errors():
    lay = synthetic.uniform_layout(1, 8, 2, 64, 16)
    q, k, v = synthetic.random_qkv(lay, 4, 2, 64, torch.bfloat16, DEV)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    with pytest.raises(Exception, match="bf16"):
        br.blockrank_attention(q.float(), k.float(), v.float(), br.BlockMask(lay.valid.to(DEV)), 0.125, score_rows=16)
    with pytest.raises(Exception, match="score_rows"):
        br.blockrank_attention(q, k, v, mask, 0.125, score_rows=lay.H + 1)
