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


def test_training_step_gradients_match_eager_autograd():
    """A training step through the hooks (trainer.py:79-101: language-model loss + auxiliary attention loss on the
    scoring layer's logits): parameter gradients from the HIP backward against torch autograd through the
    library's eager attention under the dense mask.  The yardstick is the same step in fp32: the HIP path (bf16)
    must be about as close to it as the eager path is in bf16 (at most 1.5 times its relative error, and the
    same direction)."""
    import copy
    br.register_blockrank_attention()
    model = build("mistral", torch.bfloat16)
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    lay.labels[:] = -100
    lay.labels[:, -2:] = 7
    B, S, M, H = lay.B, lay.S, lay.M, lay.H
    ids = torch.randint(0, 512, (B, S), generator=torch.Generator().manual_seed(5)).to(DEV)
    pos = lay.position_ids.to(DEV)
    valid = lay.valid.to(DEV)
    labels = lay.labels.to(DEV)
    answer_ids = torch.tensor([[1], [2]], device=DEV)
    rows_real = valid.reshape(B, S)
    probe = torch.randn((B, S, 256), generator=torch.Generator().manual_seed(6)).to(DEV)
    picked = ("layers.0.self_attn", "layers.1.self_attn.q_proj", "embed_tokens")

    def losses(out, aux_logits):
        lm = (out.hidden_states[-1].float() * probe)[rows_real].sum() / rows_real.sum()
        aux = torch.nn.functional.cross_entropy(aux_logits.float(), answer_ids[:, 0])
        return lm + aux

    def grads(mdl):
        return {n: p.grad.detach().float().clone() for n, p in mdl.named_parameters() if any(k in n for k in picked)}

    model.set_attn_implementation("default_blockrank")
    model.zero_grad()
    out = model(input_ids=ids, position_ids=pos, attention_mask=valid, output_attentions=True, layers_to_return_scores=[1],
                output_hidden_states=True, use_cache=False)
    s_last = out.attentions[0]
    assert isinstance(s_last, torch.Tensor) and s_last.requires_grad, "training returns the differentiable logits tensor"
    aux_logits = br.compute_auxiliary_attention_loss(s_last, labels, valid, answer_ids=None, return_logits=True)
    losses(out, aux_logits).backward()
    ours = grads(model)

    def eager_step(mdl, dtype):
        ok = torch.as_tensor(orc.allowed(lay.valid.numpy())) | torch.eye(S, dtype=torch.bool)[None]
        add = torch.zeros(B, 1, S, S, dtype=dtype).masked_fill_(~ok[:, None], torch.finfo(dtype).min).to(DEV)
        mdl.set_attn_implementation("eager")
        mdl.zero_grad()
        ref = mdl(input_ids=ids, position_ids=pos, attention_mask=add, output_attentions=True, output_hidden_states=True, use_cache=False)
        # the per-document score from the eager probabilities: a softmax restricted to the document columns is the
        # probabilities renormalised over them (losses.py:56-68)
        p = ref.attentions[1][:, :, S - 3:S - 1, H:S - H].float()          # rows {bracket - 1, bracket}: the bracket is the first labelled token
        p = p / p.sum(dim=-1, keepdim=True)
        logits = p.reshape(B, p.shape[1], 2, M - 2, H).sum(-1).mean(dim=(1, 2)) / 0.05
        losses(ref, logits).backward()
        return logits.detach(), grads(mdl)

    logits16, eager16 = eager_step(model, torch.bfloat16)
    logits32, exact = eager_step(copy.deepcopy(model).float(), torch.float32)
    assert (aux_logits.float() - logits32).abs().max() <= max(1.5 * (logits16 - logits32).abs().max().item(), 1e-3)
    for n, w in exact.items():
        rel = ((ours[n] - w).norm() / w.norm()).item()
        rel16 = ((eager16[n] - w).norm() / w.norm()).item()
        cos = torch.nn.functional.cosine_similarity(ours[n].flatten(), w.flatten(), dim=0).item()
        assert rel <= max(1.5 * rel16, 2e-2) and cos >= 0.99, f"{n}: relative gradient error {rel:.3e} (eager bf16: {rel16:.3e}), cosine {cos:.5f}"


def _eager_scores(mdl, dtype, lay, ids, pos, layer_idx, bracket_from_end=1):
    """Per-document scores of scripts/eval_attn.py:139-151 from the library's own eager attention: the model under the
    dense additive mask of the oracle's predicate, the scoring layer's probabilities on rows {bracket - 1, bracket},
    renormalised over the document columns (a softmax restricted to them, losses.py:56-59), summed per document,
    mean over heads and the two rows, divided by the temperature (losses.py:64-74)."""
    B, S, M, H = lay.B, lay.S, lay.M, lay.H
    ok = torch.as_tensor(orc.allowed(lay.valid.numpy())) | torch.eye(S, dtype=torch.bool)[None]
    add = torch.zeros(B, 1, S, S, dtype=dtype).masked_fill_(~ok[:, None], torch.finfo(dtype).min).to(DEV)
    mdl.set_attn_implementation("eager")
    with torch.no_grad():
        ref = mdl(input_ids=ids, position_ids=pos, attention_mask=add, output_attentions=True, use_cache=False)
    br_row = S - 1 - bracket_from_end
    p = ref.attentions[layer_idx][:, :, br_row - 1:br_row + 1, H:S - H].double()
    p = p / p.sum(dim=-1, keepdim=True)
    return (p.reshape(B, p.shape[1], 2, M - 2, H).sum(-1).mean(dim=(1, 2)) / 0.05).cpu()


def _ranker_inputs(lay, vocab, seed):
    lay.labels[:] = -100
    lay.labels[:, -2:] = 7                                   # "[" is the second to last token
    ids = torch.randint(0, vocab, (lay.B, lay.S), generator=torch.Generator().manual_seed(seed)).to(DEV)
    return ids, lay.position_ids.to(DEV), lay.valid.to(DEV), lay.labels.to(DEV)


def _packed_call(ranker, lay, ids, pos):
    keep = lay.valid.reshape(-1).to(DEV)
    lens = torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV)
    h1 = min(16, lay.H)
    rows = torch.tensor([[h1 - 3, h1 - 2]] * lay.B, dtype=torch.int32, device=DEV)       # bracket = second to last token
    return ranker.forward_packed(ids.reshape(-1)[keep][None], pos.reshape(-1)[keep][None], lens, rows, H=lay.H)


@pytest.mark.parametrize("kind", ["mistral", "qwen2"])
def test_truncated_ranker_against_eager_model_under_the_oracle_mask(kind):
    """The layer-truncated driver, padded and packed entry, against scores computed without any of this package's
    kernels: fp32 weights, so the comparison is tight (1e-3 relative, same order)."""
    import copy
    br.register_triton_blockrank_attention()
    model = build(kind, torch.float32)
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    ids, pos, valid, labels = _ranker_inputs(lay, 512, 3)
    for layer_idx in (1, 2):
        want = _eager_scores(model, torch.float32, lay, ids, pos, layer_idx).numpy()
        model.set_attn_implementation("triton_blockrank")
        ranker = br.TruncatedRanker(model, layer_idx)
        got = ranker(ids, valid, pos, labels=labels)
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-3)
        got_p = _packed_call(ranker, lay, ids, pos)
        np.testing.assert_allclose(got_p.cpu().numpy(), want, rtol=1e-3)
        assert (orc.topk_indices(got.cpu().numpy(), 3) == orc.topk_indices(want, 3)).all()
    # bf16 weights (what ranking runs in): as close to the fp32 result as the eager bf16 model is
    m16 = copy.deepcopy(model).to(torch.bfloat16)
    e16 = _eager_scores(m16, torch.bfloat16, lay, ids, pos, 2).numpy()
    m16.set_attn_implementation("triton_blockrank")
    r16 = br.TruncatedRanker(m16, 2)
    yard = np.abs(e16 - want).max()
    for got in (r16(ids, valid, pos, labels=labels), _packed_call(r16, lay, ids, pos)):
        assert np.abs(got.cpu().numpy() - want).max() <= max(1.5 * yard, 1e-3 * np.abs(want).max())


def test_truncated_ranker_at_7b_width():
    """Mistral-7B layer shapes (hidden 4096, 32 / 8 heads of 128, MLP 14336), three layers, one ranking request of the
    end-to-end benchmark configuration (64-token prefix, 20 documents U[96, 224], 32-token query), bf16 through the
    truncated driver against the fp32 eager model under the oracle's mask; the yardstick is the eager model in bf16."""
    import copy
    from transformers import MistralConfig, MistralForCausalLM
    br.register_triton_blockrank_attention()
    torch.manual_seed(0)
    cfg = MistralConfig(vocab_size=2048, hidden_size=4096, intermediate_size=14336, num_hidden_layers=3, num_attention_heads=32,
                        num_key_value_heads=8, head_dim=128, max_position_embeddings=32768, rope_theta=1e6, sliding_window=None)
    model = MistralForCausalLM(cfg).to(DEV, torch.bfloat16).eval()
    lay = synthetic.random_layout(1, 64, 20, 96, 224, 32, seed=0)
    ids, pos, valid, labels = _ranker_inputs(lay, 2048, 4)
    want = _eager_scores(copy.deepcopy(model).float(), torch.float32, lay, ids, pos, 2).numpy()
    e16 = _eager_scores(model, torch.bfloat16, lay, ids, pos, 2).numpy()
    model.set_attn_implementation("triton_blockrank")
    ranker = br.TruncatedRanker(model, 2)
    yard = np.abs(e16 - want).max()
    assert yard <= 0.05 * np.abs(want).max(), "the bf16 eager model itself should be within a few percent"
    for got in (ranker(ids, valid, pos, labels=labels), _packed_call(ranker, lay, ids, pos)):
        g = got.cpu().numpy()
        assert g.shape == (1, 20)
        assert np.abs(g - want).max() <= max(1.5 * yard, 1e-3 * np.abs(want).max()), (np.abs(g - want).max(), yard)
        np.testing.assert_allclose(g.sum(-1) * 0.05, 1.0, rtol=1e-3)


def test_fp8_logits_through_several_layers_against_eager_model():
    """BASELINE config 5's variant end to end: a small Qwen2-shaped model (head dim 128) through the truncated driver with
    Q K^T of layers 0..2 in fp8 e4m3 (``qk_fp8=True`` reaches every layer's attention hook), scored at layer 3.  The
    single-layer test cannot see the fp8 logits (the scores are read from rows the kernel computes in bf16); here
    their error reaches the scores through the documents' hidden states.  Measured: against the fp32 eager model under
    the oracle's mask the bf16 eager model is off by 3-7 % (its own rounding through four layers), this package's
    bf16 path by the same, and the fp8 variant by the same again - so the bound is the bf16 yardstick (1.1 times), and,
    which isolates what fp8 adds, the fp8 scores stay within 5e-3 relative of the bf16 path's with the same top-10."""
    import copy
    from transformers import Qwen2Config, Qwen2ForCausalLM
    br.register_triton_blockrank_attention()
    torch.manual_seed(0)
    cfg = Qwen2Config(vocab_size=512, hidden_size=4 * 128, intermediate_size=1024, num_hidden_layers=4, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=32768, rope_theta=1e6)
    model = Qwen2ForCausalLM(cfg).to(DEV, torch.float32).eval()
    for seed in (0, 1, 2):
        lay = synthetic.random_layout(2, 24, 12, 20, 150, 24, seed=seed)
        ids, pos, valid, labels = _ranker_inputs(lay, 512, 3 + seed)
        want = _eager_scores(model, torch.float32, lay, ids, pos, 3).numpy()
        m16 = copy.deepcopy(model).to(torch.bfloat16)
        e16 = _eager_scores(m16, torch.bfloat16, lay, ids, pos, 3).numpy()
        m16.set_attn_implementation("triton_blockrank")
        r16 = br.TruncatedRanker(m16, 3)
        g16 = r16(ids, valid, pos, labels=labels).cpu().numpy()
        g8 = r16(ids, valid, pos, labels=labels, qk_fp8=True).cpu().numpy()
        assert not np.array_equal(g8, g16), "the fp8 variant must actually have run"
        rel = lambda a, ref: (np.abs(a - ref) / np.abs(ref)).max()
        yard = rel(e16, want)
        assert rel(g16, want) <= 1.1 * yard and rel(g8, want) <= 1.1 * yard, (rel(g16, want), rel(g8, want), yard)
        assert rel(g8, g16) <= 5e-3, rel(g8, g16)
        t8, t16 = orc.topk_indices(g8, 10), orc.topk_indices(g16, 10)
        for b in range(lay.B):
            if (t8[b] != t16[b]).any():                      # only a near tie may reorder
                s = np.sort(g16[b])[::-1][:11]
                assert (np.abs(np.diff(s)) / s[:-1]).min() < 2 * rel(g8, g16)


def test_full_depth_config3_forward_properties():
    """BASELINE config 3 at full size: the 21 layers of a random-initialised Mistral-7B-shaped decoder (hidden 4096,
    32 / 8 heads, MLP 14336, vocabulary 32768), B = 8, 64-token prefix + 20 documents U[96, 224] + 32-token query, bf16,
    through the truncated driver's padded and packed entries.  No oracle run fits a test at this size; what the score
    formula fixes does: finite scores, the documents' shares sum to one (sum of scores x temperature = 1), and the
    two token layouts agree - measured 7e-3 relative after twenty layers of different GEMM shapes - with the same
    top-10 wherever the scores are not tied at that precision."""
    from transformers import MistralConfig, MistralModel
    br.register_triton_blockrank_attention()
    cfg = MistralConfig(vocab_size=32768, hidden_size=4096, intermediate_size=14336, num_hidden_layers=21, num_attention_heads=32,
                        num_key_value_heads=8, head_dim=128, rope_theta=1e6, sliding_window=None, max_position_embeddings=32768)
    torch.manual_seed(0)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(DEV):
            model = MistralModel(cfg)
    finally:
        torch.set_default_dtype(old)
    model.eval()
    model.set_attn_implementation("triton_blockrank")
    lay = synthetic.random_layout(8, 64, 20, 96, 224, 32, seed=0)
    ids, pos, valid, labels = _ranker_inputs(lay, 32768, 1)
    ranker = br.TruncatedRanker(model, 20)
    a = ranker(ids, valid, pos, labels=labels).float().cpu().numpy()
    b = _packed_call(ranker, lay, ids, pos).float().cpu().numpy()
    assert a.shape == b.shape == (8, 20) and np.isfinite(a).all() and np.isfinite(b).all()
    np.testing.assert_allclose(a.sum(-1) * 0.05, 1.0, rtol=1e-3)
    np.testing.assert_allclose(b.sum(-1) * 0.05, 1.0, rtol=1e-3)
    diff = (np.abs(a - b) / np.abs(a)).max()
    assert diff <= 2e-2, diff
    ta, tb = orc.topk_indices(a, 10), orc.topk_indices(b, 10)
    for i in range(8):
        if (ta[i] != tb[i]).any():
            s = np.sort(a[i])[::-1][:11]
            assert (np.abs(np.diff(s)) / s[:-1]).min() < 2 * diff, f"sequence {i}: top-10 differs without a near tie"
    del model
    torch.cuda.empty_cache()
