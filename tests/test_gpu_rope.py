"""The one-pass rotary embedding kernel: against the float64 oracle on the same inputs (fp32: 1e-6; bf16:
the rounding of the result, 2^-8 relative), closer to it than the eager bf16 expression it replaces, and
swapped into a small Hugging Face model without changing what the model computes."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(B, Nq, Nkv, S, D, dtype, seed, batch_table=True):
    g = torch.Generator().manual_seed(seed)
    # head-transposed views of (B, S, heads, D) projections, as the decoder layers hand them over
    q = torch.randn(B, S, Nq, D, generator=g).to(DEV, dtype).transpose(1, 2)
    k = torch.randn(B, S, Nkv, D, generator=g).to(DEV, dtype).transpose(1, 2)
    ang = torch.rand(B if batch_table else 1, S, D // 2, generator=g) * 6.28
    ang = torch.cat([ang, ang], dim=-1)
    return q, k, ang.cos().to(DEV, dtype), ang.sin().to(DEV, dtype)


def _eager(q, k, cos, sin):
    def rot(x):
        h = x.shape[-1] // 2
        return torch.cat((-x[..., h:], x[..., :h]), dim=-1)
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    return q * c + rot(q) * s, k * c + rot(k) * s


@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.float32, 128), (torch.bfloat16, 64), (torch.bfloat16, 128)])
@pytest.mark.parametrize("batch_table", [True, False])
def test_kernel_matches_the_oracle(dtype, D, batch_table):
    B, Nq, Nkv, S = 2, 6, 2, 37
    q, k, cos, sin = _inputs(B, Nq, Nkv, S, D, dtype, seed=D, batch_table=batch_table)
    qo, ko = br.apply_rotary_pos_emb(q, k, cos, sin)
    assert qo.shape == q.shape and ko.shape == k.shape and qo.dtype == dtype
    assert qo.transpose(1, 2).is_contiguous() and ko.transpose(1, 2).is_contiguous()       # stored (B, S, heads, D)
    c64, s64 = cos.double().cpu().numpy(), sin.double().cpu().numpy()
    eq, ek = _eager(q, k, cos, sin)
    for got, x, eager in ((qo, q, eq), (ko, k, ek)):
        want = orc.rotary_embedding(x.double().cpu().numpy(), c64, s64)
        err = np.abs(got.double().cpu().numpy() - want)
        if dtype == torch.float32:
            assert err.max() <= 1e-6
        else:
            assert (err <= 2.0 ** -8 * np.maximum(np.abs(want), 1e-2)).all(), err.max()
            # one rounding instead of three: on average nearer the exact value than the eager expression
            assert err.mean() <= np.abs(eager.double().cpu().numpy() - want).mean()


def test_argument_errors():
    q, k, cos, sin = _inputs(1, 2, 1, 8, 64, torch.bfloat16, seed=1)
    with pytest.raises(AssertionError):
        br.apply_rotary_pos_emb(q, k, cos.float(), sin.float())
    with pytest.raises(AssertionError):
        br.apply_rotary_pos_emb(q, k, cos[:, :4], sin[:, :4])
    q96 = torch.randn(1, 2, 8, 96, device=DEV, dtype=torch.bfloat16)
    c96 = torch.ones(1, 8, 96, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        br.apply_rotary_pos_emb(q96, q96, c96, c96)


@pytest.mark.parametrize("kind", ["mistral", "qwen2"])
def test_patched_model_and_ranker_agree_with_unpatched(kind):
    from tests.test_gpu_hf_model import build
    br.register_blockrank_attention()
    model = build(kind, torch.bfloat16)
    model.set_attn_implementation("sdpa_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    ids = torch.randint(0, 512, (lay.B, lay.S), generator=torch.Generator().manual_seed(1)).to(DEV)
    pos, valid, labels = lay.position_ids.to(DEV), lay.valid.to(DEV), lay.labels.to(DEV)
    ranker = br.TruncatedRanker(model, layer_idx=2)
    with torch.no_grad():
        ref_h = model(input_ids=ids, position_ids=pos, attention_mask=valid, output_hidden_states=True, use_cache=False).hidden_states[-1]
        ref_s = ranker(ids, valid, pos, labels)
    names = br.patch_rotary(model)
    try:
        assert names and all(kind in n for n in names)
        with torch.no_grad():
            got_h = model(input_ids=ids, position_ids=pos, attention_mask=valid, output_hidden_states=True, use_cache=False).hidden_states[-1]
            got_s = ranker(ids, valid, pos, labels)
    finally:
        br.unpatch_rotary(model)
    rows = lay.valid.reshape(lay.B, lay.S).to(DEV)
    assert (got_h.float() - ref_h.float())[rows].abs().max().item() <= 6e-2
    torch.testing.assert_close(got_s, ref_s, rtol=2e-2, atol=2e-2)
    import sys
    mod = sys.modules[type(model.model.layers[0].self_attn).__module__]
    assert mod.apply_rotary_pos_emb.__module__ != "blockrank_amd.rope", "unpatch_rotary must restore the model's own function"


def test_gradients_match_the_eager_expression():
    """The rotation is differentiable in q and k: its backward (the same kernel on the gradients) against autograd
    through the model file's expression in float64, with tables whose two halves differ."""
    B, Nq, Nkv, S, D = 2, 4, 2, 19, 64
    g = torch.Generator().manual_seed(3)
    q, k, _, _ = _inputs(B, Nq, Nkv, S, D, torch.float32, seed=7)
    ang = torch.rand(B, S, D, generator=g) * 6.28                       # halves not equal
    cos, sin = ang.cos().to(DEV), (ang * 1.3).sin().to(DEV)
    wq, wk = torch.randn(q.shape, generator=g).to(DEV), torch.randn(k.shape, generator=g).to(DEV)
    q1, k1 = q.clone().requires_grad_(), k.clone().requires_grad_()
    qo, ko = br.apply_rotary_pos_emb(q1, k1, cos, sin)
    assert qo.requires_grad and ko.requires_grad
    ((qo * wq).sum() + (ko * wk).sum()).backward()
    q2, k2 = q.double().requires_grad_(), k.double().requires_grad_()
    eq, ek = _eager(q2, k2, cos.double(), sin.double())
    ((eq * wq.double()).sum() + (ek * wk.double()).sum()).backward()
    assert (q1.grad.double() - q2.grad).abs().max().item() <= 1e-5
    assert (k1.grad.double() - k2.grad).abs().max().item() <= 1e-5


def test_patched_model_trains_through_the_rotation():
    """After patch_rotary the projections in front of the rotation still get their gradients: q_proj / k_proj of a
    small Mistral, patched against unpatched, same loss."""
    from tests.test_gpu_hf_model import build
    br.register_blockrank_attention()
    model = build("mistral", torch.float32)
    model.set_attn_implementation("default_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    ids = torch.randint(0, 512, (lay.B, lay.S), generator=torch.Generator().manual_seed(1)).to(DEV)
    pos, valid = lay.position_ids.to(DEV), lay.valid.to(DEV)
    rows = lay.valid.reshape(lay.B, lay.S).to(DEV)
    probe = torch.randn((lay.B, lay.S, 256), generator=torch.Generator().manual_seed(2)).to(DEV)

    def step():
        model.zero_grad()
        # fp32 inputs have no attention backward here: the eager library attention under a dense mask carries the graph
        ok = torch.as_tensor(orc.allowed(lay.valid.numpy())) | torch.eye(lay.S, dtype=torch.bool)[None]
        add = torch.zeros(lay.B, 1, lay.S, lay.S).masked_fill_(~ok[:, None], torch.finfo(torch.float32).min).to(DEV)
        model.set_attn_implementation("eager")
        out = model(input_ids=ids, position_ids=pos, attention_mask=add, output_hidden_states=True, use_cache=False)
        (out.hidden_states[-1] * probe)[rows].sum().backward()
        return {n: p.grad.clone() for n, p in model.named_parameters() if "q_proj" in n or "k_proj" in n}

    ref = step()
    br.patch_rotary(model)
    try:
        got = step()
    finally:
        br.unpatch_rotary(model)
    assert ref.keys() == got.keys() and len(ref) == 6
    for n in ref:
        assert got[n].abs().max().item() > 0
        torch.testing.assert_close(got[n], ref[n], rtol=1e-3, atol=1e-5 * ref[n].abs().max().item() + 1e-7)


@pytest.mark.parametrize("Nq,Nkv,D", [(8, 2, 128), (4, 4, 64), (14, 2, 128)])
def test_attention_kernel_rotates_q_rows_itself(Nq, Nkv, D):
    """blockrank_attention(..., q_rope=(cos, sin)) on the unrotated Q against the oracle's rotation followed by the
    oracle's attention, and against the two-kernel path (stand-alone rotation, then attention): same result to a
    bf16 rounding of a Q element here and there."""
    from tests._util import max_abs_on_real_rows, oracle_attention, oracle_doc_scores, assert_scores_close
    from blockrank_amd.rope import rotate_k
    lay = synthetic.make_layout([[40, 100, 7, 160, 33, 20], [64, 0, 150, 90, 65, 31]])
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=11)
    g = torch.Generator().manual_seed(5)
    ang = torch.rand(lay.B, lay.S, D // 2, generator=g) * 6.28
    ang = torch.cat([ang, ang * 1.1], dim=-1)                          # halves that differ: nothing may rely on their equality
    cos, sin = ang.cos().to(DEV, torch.bfloat16), ang.sin().to(DEV, torch.bfloat16)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    scale = D ** -0.5
    k_rot = rotate_k(k, cos, sin)
    out, part = br.blockrank_attention(q, k_rot, v, mask, scale, score_rows=16, q_rope=(cos, sin))
    # oracle: rotation in float64, rounded to bf16 like the tensors the attention oracle is given elsewhere
    c64, s64 = cos.double().cpu().numpy(), sin.double().cpu().numpy()
    q_ref = torch.as_tensor(orc.rotary_embedding(q.double().cpu().numpy(), c64, s64)).to(torch.bfloat16)
    k_ref = torch.as_tensor(orc.rotary_embedding(k.double().cpu().numpy(), c64, s64)).to(torch.bfloat16)
    assert max_abs_on_real_rows(out, oracle_attention(q_ref, k_ref, v, lay, scale), lay) <= 2e-2
    rows = torch.tensor([[14, 15]] * lay.B, dtype=torch.int32, device=DEV)
    scores = br.doc_scores_from_partials(part, mask, rows, 16, Nq, Nkv)
    assert_scores_close(scores, oracle_doc_scores(q_ref, k_ref, lay, scale), rel=2e-3)
    q_rot, _ = br.apply_rotary_pos_emb(q, k, cos, sin)
    two = br.blockrank_attention(q_rot, k_rot, v, mask, scale)
    real = lay.valid.reshape(lay.B, lay.S).to(DEV)
    assert (out[real].float() - two[real].float()).abs().max().item() <= 4e-3
    # one table for the whole batch, and the packed layout
    cos1, sin1 = cos[:1].contiguous(), sin[:1].contiguous()
    k1 = rotate_k(k, cos1, sin1)
    a = br.blockrank_attention(q, k1, v, mask, scale, q_rope=(cos1, sin1))
    b = br.blockrank_attention(br.apply_rotary_pos_emb(q, k, cos1, sin1)[0], k1, v, mask, scale)
    assert (a[real].float() - b[real].float()).abs().max().item() <= 4e-3
    with pytest.raises(NotImplementedError):
        br.blockrank_attention(q, k_rot, v, mask, scale, q_rope=(cos, sin), qk_fp8=True)


@pytest.mark.parametrize("kind", ["mistral", "qwen2"])
def test_model_with_q_rotation_left_to_the_attention_kernel(kind):
    """patch_rotary(model, fuse_q=True): hidden states and ranking scores of a small model as with the model file's own
    rotary function; a layer that returns scores, and a training step, rotate Q before the hook uses it."""
    from tests.test_gpu_hf_model import build
    br.register_blockrank_attention()
    model = build(kind, torch.bfloat16)
    model.set_attn_implementation("sdpa_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    ids = torch.randint(0, 512, (lay.B, lay.S), generator=torch.Generator().manual_seed(1)).to(DEV)
    pos, valid, labels = lay.position_ids.to(DEV), lay.valid.to(DEV), lay.labels.to(DEV)
    ranker = br.TruncatedRanker(model, layer_idx=2)
    rows = lay.valid.reshape(lay.B, lay.S).to(DEV)

    def run():
        with torch.no_grad():
            o = model(input_ids=ids, position_ids=pos, attention_mask=valid, output_hidden_states=True, output_attentions=True,
                      layers_to_return_scores=[1], use_cache=False)
            s1 = br.compute_auxiliary_attention_loss(o.attentions[0], labels, valid, answer_ids=None, return_logits=True)
            return o.hidden_states[-1], s1, ranker(ids, valid, pos, labels)

    ref_h, ref_s1, ref_s = run()
    br.patch_rotary(model, fuse_q=True)
    try:
        got_h, got_s1, got_s = run()
    finally:
        br.unpatch_rotary(model)
    assert (got_h.float() - ref_h.float())[rows].abs().max().item() <= 6e-2
    torch.testing.assert_close(got_s1, ref_s1, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got_s, ref_s, rtol=2e-2, atol=2e-2)
