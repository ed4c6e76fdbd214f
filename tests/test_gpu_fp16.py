"""fp16 inputs (the reference runs in whatever dtype the model has, blockrank_std_attention.py:527): the 16-bit MFMA
kernels instantiated for _Float16.  Same oracle, same cases as bf16; bound 4e-3 max-abs on the attention output (fp16
carries three more mantissa bits than bf16, whose bound is 2e-2) and the 1e-3 relative bound on the scores."""
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc
from tests._util import assert_scores_close, eval_rows, max_abs_on_real_rows, oracle_attention, oracle_doc_scores, real_rows

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F16 = torch.float16


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("lens,Nq,Nkv", [([[5, 17, 0, 64, 33, 9], [40, 1, 65, 31, 2, 70]], 8, 2), ([[20, 70, 45, 130, 37]], 14, 2),
                                         ([[100]], 4, 4), ([[32] + [40] * 60 + [16]], 8, 2)])
def test_attention_output_and_fused_scores(D, lens, Nq, Nkv):
    lay = synthetic.make_layout(lens)
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, F16, DEV, seed=4)
    mask = br.BlockMask(lay.valid.to(DEV), F16)
    scale = D ** -0.5
    M = lay.lengths.shape[1]
    if M >= 3:
        R = min(16, lay.H)
        out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R)
    else:
        out = br.blockrank_attention(q, k, v, mask, scale)
    assert out.dtype == F16 and out.shape == (lay.B, lay.S, Nq, D)
    err = max_abs_on_real_rows(out, oracle_attention(q, k, v, lay, scale), lay)
    assert err <= 4e-3, err
    assert (out.cpu()[~real_rows(lay)] == 0).all()
    if M >= 3:
        rows = eval_rows(lay, DEV)
        want = oracle_doc_scores(q, k, lay, scale)
        got = br.doc_scores_from_partials(part, mask, rows - (lay.H - R), R, Nq, Nkv)
        assert_scores_close(got, want)
        assert_scores_close(br.doc_scores(q, k, mask, rows, scale), want)               # the stand-alone kernels


def test_config2_shape_full_size():
    lay = synthetic.uniform_layout(4, 64, 20, 160, 32)
    q, k, v = synthetic.attention_layer_inputs(lay, 32, 8, 128, 4096, F16, DEV)
    scale = 128 ** -0.5
    out, part = br.blockrank_attention(q, k, v, br.BlockMask(lay.valid.to(DEV), F16), scale, score_rows=16)
    assert max_abs_on_real_rows(out, oracle_attention(q, k, v, lay, scale), lay) <= 4e-3
    got = br.doc_scores_from_partials(part, br.BlockMask(lay.valid.to(DEV), F16), eval_rows(lay, DEV) - (lay.H - 16), 16, 32, 8)
    assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))


def test_rotary_kernel_and_rotation_inside_the_attention_kernel():
    lay = synthetic.make_layout([[40, 100, 7, 160, 33, 20]])
    Nq, Nkv, D = 8, 2, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, F16, DEV, seed=11)
    ang = torch.rand(1, lay.S, D // 2, generator=torch.Generator().manual_seed(5)) * 6.28
    ang = torch.cat([ang, ang], dim=-1)
    cos, sin = ang.cos().to(DEV, F16), ang.sin().to(DEV, F16)
    q_rot, k_rot = br.apply_rotary_pos_emb(q, k, cos, sin)
    c64, s64 = cos.double().cpu().numpy(), sin.double().cpu().numpy()
    want_q = torch.as_tensor(orc.rotary_embedding(q.double().cpu().numpy(), c64, s64))
    assert (q_rot.double().cpu() - want_q).abs().max().item() <= 4e-3
    mask = br.BlockMask(lay.valid.to(DEV), F16)
    a = br.blockrank_attention(q, k_rot, v, mask, D ** -0.5, q_rope=(cos, sin))
    b = br.blockrank_attention(q_rot, k_rot, v, mask, D ** -0.5)
    real = lay.valid.reshape(lay.B, lay.S).to(DEV)
    assert (a[real].float() - b[real].float()).abs().max().item() <= 1e-3


def test_last_block_logits_and_what_fp16_does_not_have():
    lay = synthetic.make_layout([[9, 30, 0, 17, 20]])
    q, k, v = synthetic.random_qkv(lay, 8, 2, 64, F16, DEV, seed=5)
    mask = br.BlockMask(lay.valid.to(DEV), F16)
    rows = torch.arange(lay.H - 16, lay.H, dtype=torch.int32, device=DEV)[None]
    got = br.last_block_logits(q, k, mask, rows, 0.17).cpu().double().numpy()
    want = orc.last_block_logits(q.float().cpu().numpy(), k.float().cpu().numpy(), lay.valid.numpy(), 0.17, 16, neg=0.7 * torch.finfo(F16).min)
    ok = orc.allowed(lay.valid.numpy())[:, lay.S - 16:, :][:, None].repeat(8, axis=1)
    assert abs(got[ok] - want[ok]).max() <= 1e-4
    with pytest.raises(NotImplementedError):                      # no backward kernels for fp16
        br.blockrank_attention(q.clone().requires_grad_(True), k, v, mask, 0.125)
    with pytest.raises(NotImplementedError):                      # the fp8 variant takes bf16
        br.blockrank_attention(q, k, v, mask, 0.125, qk_fp8=True)


def test_small_model_in_fp16():
    """A small Mistral in fp16 through the hooks against its own eager attention under the oracle's mask."""
    from tests.test_gpu_hf_model import build
    br.register_blockrank_attention()
    model = build("mistral", F16)
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    B, S = lay.B, lay.S
    ids = torch.randint(0, 512, (B, S), generator=torch.Generator().manual_seed(1)).to(DEV)
    pos, valid, labels = lay.position_ids.to(DEV), lay.valid.to(DEV), lay.labels.to(DEV)
    model.set_attn_implementation("sdpa_blockrank")
    with torch.no_grad():
        ours = model(input_ids=ids, position_ids=pos, attention_mask=valid, output_attentions=True, layers_to_return_scores=[1],
                     output_hidden_states=True, use_cache=False)
    ok = torch.as_tensor(orc.allowed(lay.valid.numpy())) | torch.eye(S, dtype=torch.bool)[None]
    add = torch.zeros(B, 1, S, S, dtype=F16)
    add.masked_fill_(~ok[:, None], torch.finfo(F16).min)
    model.set_attn_implementation("eager")
    with torch.no_grad():
        ref = model(input_ids=ids, position_ids=pos, attention_mask=add.to(DEV), output_hidden_states=True, use_cache=False)
    rows = lay.valid.reshape(B, S).to(DEV)
    a, b = ours.hidden_states[2][rows].float(), ref.hidden_states[2][rows].float()
    assert torch.isfinite(a).all() and (a - b).abs().max().item() <= 1e-2 * max(1.0, b.abs().max().item())
    h = ours.attentions[0]
    logits = br.compute_auxiliary_attention_loss(h, labels, valid, answer_ids=None, return_logits=True)
    want = orc.doc_scores(h.query.float().cpu().numpy(), h.key.float().cpu().numpy(), lay.valid.numpy(), lay.labels.numpy(), h.scaling, 0.05, 16)
    assert_scores_close(logits, want)
