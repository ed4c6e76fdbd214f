"""The hooks inside a Hugging Face model: a small random Mistral / Qwen2 runs with
attn_implementation="sdpa_blockrank" (HIP path) and is compared with the same weights run through the
library's own eager attention under an explicit 4-D additive mask built from the oracle's predicate."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def build(kind, dtype):
    from transformers import MistralConfig, MistralForCausalLM, Qwen2Config, Qwen2ForCausalLM
    common = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=3, max_position_embeddings=32768,
                  rope_theta=1e6)
    torch.manual_seed(0)
    if kind == "mistral":
        cfg = MistralConfig(num_attention_heads=4, num_key_value_heads=2, head_dim=64, sliding_window=None, **common)
        model = MistralForCausalLM(cfg)
    else:
        cfg = Qwen2Config(num_attention_heads=14, num_key_value_heads=2, **{**common, "hidden_size": 14 * 64})
        model = Qwen2ForCausalLM(cfg)
    return model.to(DEV, dtype).eval()


@pytest.mark.parametrize("kind,dtype,tol", [("mistral", torch.float32, 2e-4), ("mistral", torch.bfloat16, 6e-2), ("qwen2", torch.bfloat16, 6e-2)])
def test_model_forward_matches_eager_with_dense_mask(kind, dtype, tol):
    br.register_blockrank_attention()
    br.register_triton_blockrank_attention()
    model = build(kind, dtype)
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    B, S = lay.B, lay.S
    ids = torch.randint(0, 512, (B, S), generator=torch.Generator().manual_seed(1)).to(DEV)
    pos = lay.position_ids.to(DEV)

    model.set_attn_implementation("sdpa_blockrank")
    with torch.no_grad():
        ours = model(input_ids=ids, position_ids=pos, attention_mask=lay.valid.to(DEV), output_attentions=True,
                     layers_to_return_scores=[1], output_hidden_states=True, use_cache=False)
    assert len(ours.attentions) == 1 and isinstance(ours.attentions[0], br.LastBlockScores)

    ok = torch.as_tensor(orc.allowed(lay.valid.numpy()))
    ok = ok | torch.eye(S, dtype=torch.bool)[None]              # padded rows: keep softmax finite
    add = torch.zeros(B, 1, S, S, dtype=dtype)
    add.masked_fill_(~ok[:, None], torch.finfo(dtype).min)
    model.set_attn_implementation("eager")
    with torch.no_grad():
        ref = model(input_ids=ids, position_ids=pos, attention_mask=add.to(DEV), output_hidden_states=True, use_cache=False)
    rows = lay.valid.reshape(B, S).to(DEV)
    # compare the hidden state after layer 2 (index 2): it went through two block-sparse attentions
    a = ours.hidden_states[2][rows].float()
    b = ref.hidden_states[2][rows].float()
    assert torch.isfinite(a).all()
    err = (a - b).abs().max().item()
    assert err <= tol * max(1.0, b.abs().max().item()), f"hidden state differs by {err}"

    # layer-score API end to end: scores from the handle vs the oracle fed with the same model's q/k
    logits = br.compute_auxiliary_attention_loss(ours.attentions[0], lay.labels.to(DEV), lay.valid.to(DEV), answer_ids=None,
                                                 return_logits=True)
    h = ours.attentions[0]
    want = orc.doc_scores(h.query.float().cpu().numpy(), h.key.float().cpu().numpy(), lay.valid.numpy(), lay.labels.numpy(),
                          h.scaling, 0.05, 16)
    np.testing.assert_allclose(logits.cpu().numpy(), want, rtol=1e-3)
    assert torch.equal(br.rank_documents(logits).cpu(), torch.as_tensor(orc.topk_indices(want, 10)))


def test_every_reference_impl_name_is_registered():
    from transformers import AttentionInterface, AttentionMaskInterface
    br.register_blockrank_attention()
    br.register_triton_blockrank_attention()
    for name in ["default_blockrank", "max-autotune_blockrank", "eager_blockrank", "flex_blockrank", "sdpa_blockrank",
                 "sdpa_compiled_blockrank", "triton_blockrank", "triton_blockrank_compiled"]:
        assert AttentionInterface()[name] is br.blockrank_attention_forward
        assert AttentionMaskInterface()[name] is br.blockrank_attention_mask


@pytest.mark.parametrize("kind,dtype", [("mistral", torch.float32), ("mistral", torch.bfloat16), ("qwen2", torch.bfloat16)])
def test_truncated_ranker_matches_full_forward(kind, dtype):
    """The layer-truncated driver (scripts/eval_attn.py:102-151 counterpart) returns the scores of the full
    forward + compute_auxiliary_attention_loss, for the scoring layer in the middle and at the start."""
    br.register_triton_blockrank_attention()
    model = build(kind, dtype)
    model.set_attn_implementation("triton_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    lay.labels[:] = -100
    lay.labels[:, -2:] = 7                                   # "[" is the second to last token
    B, S = lay.B, lay.S
    ids = torch.randint(0, 512, (B, S), generator=torch.Generator().manual_seed(3)).to(DEV)
    pos = lay.position_ids.to(DEV)
    valid = lay.valid.to(DEV)
    for layer_idx in (1, 0, 2):
        with torch.no_grad():
            full = model(input_ids=ids, position_ids=pos, attention_mask=valid, output_attentions=True,
                         layers_to_return_scores=[layer_idx], use_cache=False)
        want = br.compute_auxiliary_attention_loss(full.attentions[0], lay.labels.to(DEV), valid, answer_ids=None, return_logits=True)
        ranker = br.TruncatedRanker(model, layer_idx)
        got = ranker(ids, valid, pos, labels=lay.labels.to(DEV))
        assert got.shape == (B, lay.M - 2)
        torch.testing.assert_close(got, want, rtol=2e-3 if dtype == torch.bfloat16 else 1e-4, atol=1e-5)
        assert torch.equal(ranker.rank(ids, valid, pos, labels=lay.labels.to(DEV), k=3), br.rank_documents(want, 3))
