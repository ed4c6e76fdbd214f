"""Parity of the fused per-document score kernel and of the materialised last-block logits with the
float64 oracle.  Tolerance (from the target statement): 1e-3 relative per score, identical top-10."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc
from tests._util import assert_scores_close, eval_rows, oracle_doc_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
R_MIN = 16


def fused(q, k, lay, scale, rows=None, **kw):
    rows = eval_rows(lay, DEV) if rows is None else rows
    return br.doc_scores(q, k, lay.valid.to(DEV), rows, scale, **kw)


def test_config1_scores_fp32():
    lay = synthetic.uniform_layout(1, 32, 8, 64, 16)
    q, k, _ = synthetic.random_qkv(lay, 8, 2, 64, torch.float32, DEV)
    got = fused(q, k, lay, 64 ** -0.5)
    want = oracle_doc_scores(q, k, lay, 64 ** -0.5)
    assert got.shape == (1, 8)
    assert_scores_close(got, want)


def test_config2_scores_bf16_full_size():
    lay = synthetic.uniform_layout(4, 64, 20, 160, 32)
    q, k, _ = synthetic.attention_layer_inputs(lay, 32, 8, 128, 4096, torch.bfloat16, DEV)
    got = fused(q, k, lay, 128 ** -0.5)
    want = oracle_doc_scores(q, k, lay, 128 ** -0.5)
    assert got.shape == (4, 20)
    assert_scores_close(got, want)
    np.testing.assert_allclose(got.sum(-1).cpu().numpy() * 0.05, 1.0, rtol=1e-4)


@pytest.mark.parametrize("Nq,Nkv,D,dtype", [(8, 2, 128, torch.bfloat16), (28, 4, 128, torch.bfloat16), (6, 2, 64, torch.float32),
                                            (16, 1, 64, torch.bfloat16)])
def test_ragged_documents(Nq, Nkv, D, dtype):
    lay = synthetic.make_layout([[5, 17, 0, 300, 33, 9], [40, 1, 65, 31, 2, 70]])
    q, k, _ = synthetic.random_qkv(lay, Nq, Nkv, D, dtype, DEV, seed=2, pad_fill=float("nan"))
    fill = lambda t: torch.where(~lay.valid.view(lay.B, 1, lay.S, 1).to(DEV), torch.zeros_like(t), t)
    got, probs = fused(q, k, lay, 0.11, return_probs=True)
    want = oracle_doc_scores(fill(q), fill(k), lay, 0.11)
    assert_scores_close(got, want)
    assert got[0, 1].item() == 0.0                         # the empty document gets no mass
    np.testing.assert_allclose(probs.sum(-1).cpu().numpy(), 1.0, rtol=1e-5)
    assert probs.shape == (2, Nq, 2, 4)


def test_training_style_rows_and_reductions():
    # bracket not at the end (answers follow it): rows come from the labels
    lay = synthetic.make_layout([[10, 40, 50, 24], [10, 30, 20, 24]])
    lay.labels[:] = -100
    lay.labels[0, -5:] = 1
    lay.labels[1, -9:] = 1
    q, k, _ = synthetic.random_qkv(lay, 4, 2, 64, torch.float32, DEV, seed=3)
    h1 = 16
    rows = torch.as_tensor(orc.bracket_rows(lay.labels.numpy(), h1)) + (lay.H - h1)
    got = fused(q, k, lay, 0.2, rows=rows.to(DEV, torch.int32), temperature=0.1)
    want = oracle_doc_scores(q, k, lay, 0.2, temperature=0.1, num_last=h1)
    assert_scores_close(got, want)
    summed = fused(q, k, lay, 0.2, rows=rows.to(DEV, torch.int32), temperature=0.1, head_reduce="sum", row_reduce="sum")
    np.testing.assert_allclose(summed.cpu().numpy(), got.cpu().numpy() * 8, rtol=1e-6)


def test_padded_row_gives_the_uniform_answer():
    # a chosen row that is padding sees nothing: the reference's softmax over equal values is uniform
    lay = synthetic.make_layout([[8, 20, 30, 40, 1]], H=48)
    q, k, _ = synthetic.random_qkv(lay, 4, 2, 64, torch.float32, DEV, seed=4)
    rows = torch.tensor([[lay.H - 2, lay.H - 2]], dtype=torch.int32, device=DEV)     # H-2 is padding (query has 1 token)
    got = fused(q, k, lay, 0.3, rows=rows, temperature=1.0)
    np.testing.assert_allclose(got.cpu().numpy(), np.full((1, 3), 1 / 3), rtol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_last_block_logits_match_closed_form(dtype):
    lay = synthetic.make_layout([[9, 30, 0, 17, 20], [12, 5, 33, 8, 3]])
    Nq, Nkv, D, R = 8, 2, 64, 16
    q, k, _ = synthetic.random_qkv(lay, Nq, Nkv, D, dtype, DEV, seed=5)
    rows = torch.arange(lay.H - R, lay.H, dtype=torch.int32, device=DEV)[None].expand(2, R).contiguous()
    got = br.last_block_logits(q, k, lay.valid.to(DEV), rows, 0.17).cpu().double().numpy()
    neg = 0.7 * torch.finfo(dtype).min
    want = orc.last_block_logits(q.float().cpu().numpy(), k.float().cpu().numpy(), lay.valid.numpy(), 0.17, R, neg=neg)
    assert got.shape == (2, Nq, R, lay.S)
    ok = orc.allowed(lay.valid.numpy())[:, lay.S - R:, :]
    okb = np.broadcast_to(ok[:, None], got.shape)
    np.testing.assert_allclose(got[okb], want[okb], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[~okb], want[~okb], rtol=1e-5)      # masked: NEG plus a negligible logit


def test_loss_api_handle_and_tensor_paths_agree():
    lay = synthetic.uniform_layout(2, 16, 6, 48, 20)
    Nq, Nkv, D = 8, 2, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=6)

    class Mod:
        layer_idx = 3
        num_key_value_groups = 4
        training = False

    mask = br.blockrank_attention_mask(batch_size=2, attention_mask=lay.valid.to(DEV), dtype=torch.bfloat16)
    out, h = br.blockrank_attention_forward(Mod(), q, k, v, mask, D ** -0.5, layers_to_return_scores=[3])
    assert isinstance(h, br.LastBlockScores) and h.shape == (2, Nq, 16, lay.S)
    _, none = br.blockrank_attention_forward(Mod(), q, k, v, mask, D ** -0.5, layers_to_return_scores=[4])
    assert none is None
    labels = lay.labels.to(DEV)
    fused = br.compute_auxiliary_attention_loss(h, labels, lay.valid.to(DEV), answer_ids=None, return_logits=True)
    dense = br.compute_auxiliary_attention_loss(h.dense(), labels, lay.valid.to(DEV), answer_ids=None, return_logits=True)
    want = oracle_doc_scores(q, k, lay, D ** -0.5)
    assert_scores_close(fused, want)
    assert_scores_close(dense, want)
    top = br.rank_documents(fused)
    assert top.shape == (2, 6)
    np.testing.assert_array_equal(top.cpu().numpy(), orc.topk_indices(want, 10))
    # materialised tensor straight from the hook, and the literal-SDPA unscaled variant
    _, t = br.blockrank_attention_forward(Mod(), q, k, v, mask, D ** -0.5, return_last_block_attn_scores=True, materialize_scores=True)
    assert torch.is_tensor(t) and t.dtype == torch.float32 and t.shape == (2, Nq, 16, lay.S)
    _, u = br.blockrank_attention_forward(Mod(), q, k, v, mask, D ** -0.5, return_last_block_attn_scores=True, materialize_scores=True,
                                          unscaled_scores=True)
    okcol = t > -1e30
    torch.testing.assert_close(u[okcol] * D ** -0.5, t[okcol], rtol=1e-5, atol=1e-5)
    with pytest.raises(AssertionError):
        br.compute_auxiliary_attention_loss(h, labels, lay.valid.to(DEV), answer_ids=None, return_logits=False)
    loss, acc, lg = br.compute_auxiliary_attention_loss(h, labels, lay.valid.to(DEV), answer_ids=torch.tensor([[0, -1], [2, 3]], device=DEV),
                                                        return_logits=True)
    assert torch.isfinite(loss) and 0 <= acc.item() <= 1 and torch.equal(lg, fused)


def test_more_than_sixteen_score_rows_materialised():
    """num_last_queries above 16 (the reference accepts any value, blockrank_std_attention.py:637-645): the dense
    logits tensor is assembled from groups of 16 rows and equals the closed form row by row."""
    lay = synthetic.uniform_layout(1, 16, 3, 48, 40)
    Nq, Nkv, D = 4, 2, 64
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.float32, DEV, seed=8)

    class Mod:
        layer_idx = 0
        num_key_value_groups = 2
        training = False

    mask = br.blockrank_attention_mask(batch_size=1, attention_mask=lay.valid.to(DEV), dtype=torch.float32)
    _, t = br.blockrank_attention_forward(Mod(), q, k, v, mask, D ** -0.5, return_last_block_attn_scores=True, num_last_queries=37,
                                          materialize_scores=True)
    assert t.shape == (1, Nq, 37, lay.S)
    _, t16 = br.blockrank_attention_forward(Mod(), q, k, v, mask, D ** -0.5, return_last_block_attn_scores=True, materialize_scores=True)
    assert torch.equal(t[:, :, -16:], t16)
    qq = q[:, :, -37:].double().cpu()
    kk = k.double().cpu().repeat_interleave(2, dim=1)
    want = torch.einsum("bnrd,bnsd->bnrs", qq, kk) * D ** -0.5
    vis = lay.valid.reshape(1, 1, 1, lay.S).expand_as(want).clone()
    for r in range(37):                              # causal inside the query block
        vis[..., r, lay.S - 37 + r + 1:] = False
    torch.testing.assert_close(t.double().cpu()[vis], want[vis], rtol=1e-5, atol=1e-5)
    assert (t.cpu()[~vis] < -1e30).all()


def test_dropout_in_training_is_refused():
    lay = synthetic.uniform_layout(1, 16, 2, 32, 16)
    q, k, v = synthetic.random_qkv(lay, 4, 2, 64, torch.bfloat16, DEV, seed=9)

    class Mod:
        layer_idx = 0
        num_key_value_groups = 2
        training = True

    mask = br.blockrank_attention_mask(batch_size=1, attention_mask=lay.valid.to(DEV), dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="dropout"):
        br.blockrank_attention_forward(Mod(), q, k, v, mask, 0.125, dropout=0.1)
    Mod.training = False
    out, _ = br.blockrank_attention_forward(Mod(), q, k, v, mask, 0.125, dropout=0.1)      # evaluation: dropout is off anyway
    assert out.shape == (1, lay.S, 4, 64)


@pytest.mark.parametrize("docs,H", [(20, 160), (100, 96), (300, 40)])
@pytest.mark.parametrize("qk_fp8", [False, True])
def test_scores_reduced_inside_the_attention_call(docs, H, qk_fp8):
    """rank_rows: the per-document scores come out of the launch that merges the split partials - bit-identical to
    the separate reduction of the same partials (one-document-per-lane, four-per-lane and general paths), the
    attention output untouched; through the hook with score_rows_hint, and two calls in a row (LDS and partials of
    the first must not leak into the second)."""
    g = torch.Generator().manual_seed(docs)
    lens = [[int(x) for x in torch.randint(1, H + 1, (docs + 2,), generator=g)] for _ in range(2)]
    lens[1][3] = 0                                                    # an empty document
    lens[0][-1] = H
    lens[1][-1] = max(R_MIN, H - 3)
    lay = synthetic.make_layout(lens, H=H)
    Nq, Nkv, D = 8, 2, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=3)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    scale = D ** -0.5
    R = min(16, H)
    rows = torch.tensor([[R - 2, R - 1], [R - 5, R - 1]], dtype=torch.int32, device=DEV)
    out_scale = 1.0 / (0.05 * Nq * 2)
    out0, part0 = br.blockrank_attention(q, k, v, mask, scale, score_rows=R, qk_fp8=qk_fp8)
    want = br.doc_scores_from_partials(part0, mask, rows, R, Nq, Nkv)
    for _ in range(2):
        out1, part1, got = br.blockrank_attention(q, k, v, mask, scale, score_rows=R, qk_fp8=qk_fp8, rank_rows=rows, rank_scale=out_scale)
        assert torch.equal(got, want)
        assert torch.equal(out1, out0)                       # (the partials buffer has slots no kernel writes: not compared)

    class Layer:
        layer_idx = 3
        num_key_value_groups = Nq // Nkv
        training = False
    out2, handle = br.blockrank_attention_forward(Layer(), q, k, v, mask, scale, layers_to_return_scores=[3], score_rows_hint=rows,
                                                   qk_fp8=qk_fp8)
    assert torch.equal(out2, out0)
    assert handle.ranked is not None and handle.doc_scores_window(rows, temperature=0.05) is handle.ranked[2]
    assert torch.equal(handle.doc_scores_window(rows, temperature=0.05), want)
    other = rows.clone()
    assert torch.equal(handle.doc_scores_window(other, temperature=0.05), want)          # another tensor object: from the partials
    assert torch.allclose(handle.doc_scores_window(rows, temperature=0.1), want * 0.5, rtol=1e-6)
    labels = lay.labels.to(DEV)
    l1 = br.compute_auxiliary_attention_loss(handle, labels, lay.valid.to(DEV), return_logits=True)
    hint = br.bracket_rows(labels, R)
    _, h2 = br.blockrank_attention_forward(Layer(), q, k, v, mask, scale, layers_to_return_scores=[3], score_rows_hint=hint, qk_fp8=qk_fp8)
    l2 = br.compute_auxiliary_attention_loss(h2, labels, lay.valid.to(DEV), return_logits=True, rows=hint)
    assert l2 is h2.ranked[2] and torch.equal(l1, l2)


def test_score_reduction_in_the_attention_call_argument_errors():
    lay = synthetic.make_layout([[20, 30, 25, 18]])
    q, k, v = synthetic.random_qkv(lay, 4, 2, 64, torch.bfloat16, DEV, seed=1)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    rows = torch.zeros((1, 2), dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError):
        br.blockrank_attention(q, k, v, mask, 0.125, rank_rows=rows)
    with pytest.raises(AssertionError, match="rows not supported"):
        br.blockrank_attention(q, k, v, mask, 0.125, score_rows=16, rank_rows=torch.zeros((1, 17), dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("dtype,Nq,Nkv,D,tol", [(torch.float32, 8, 2, 64, 2e-5), (torch.bfloat16, 8, 2, 128, 1.2e-2), (torch.float32, 6, 6, 128, 2e-5)])
def test_gradient_of_the_last_block_logits(dtype, Nq, Nkv, D, tol):
    """LastBlockScores.dense() with gradients: dq and dk from the HIP kernels against torch autograd of the closed form
    s = scale * q_row . k over real rows and real keys (fp32: to rounding; bf16: to the rounding of the stored result),
    padded and packed layouts, 16 default rows; a loss through compute_auxiliary_attention_loss on top."""
    lay = synthetic.make_layout([[9, 30, 0, 17, 20], [12, 5, 33, 8, 13]])
    R, scale = 16, 0.17
    q0, k0, _ = synthetic.random_qkv(lay, Nq, Nkv, D, dtype, DEV, seed=5)
    valid = lay.valid.to(DEV)
    B, S, H, M = lay.B, lay.S, lay.H, lay.lengths.shape[1]
    G = Nq // Nkv
    g = torch.Generator().manual_seed(2)
    ds = torch.randn(B, Nq, R, S, generator=g).to(DEV)

    # closed form in float64 on the padded layout
    qr = q0.double().clone().requires_grad_(True)
    kr = k0.double().clone().requires_grad_(True)
    vrow = valid.reshape(B, S)
    rows_tok = torch.arange(S - R, S, device=DEV)
    row_real = vrow[:, rows_tok]                                            # (B, R)
    s_ref = scale * torch.einsum("bnrd,bnsd->bnrs", qr[:, :, rows_tok], kr.repeat_interleave(G, dim=1))
    s_ref = s_ref * (row_real[:, None, :, None] & vrow[:, None, None, :])   # padded rows / empty slots: constants
    (s_ref * ds.double()).sum().backward()

    def run(bm, q, k):
        q = q.clone().requires_grad_(True)
        k = k.clone().requires_grad_(True)
        h = br.LastBlockScores(q, k, bm, scale, R)
        assert h.needs_grad()
        out = h.dense()
        assert out.shape == (B, Nq, R, S) and out.requires_grad
        (out * ds).sum().backward()
        return q.grad, k.grad

    dq, dk = run(br.BlockMask(valid, dtype), q0, k0)
    real = vrow[:, None, :, None]
    for got, want, name in ((dq, qr.grad, "dq"), (dk, kr.grad, "dk")):
        want = want * real                                                   # (the closed form has zeros there already)
        err = (got.double() - want).abs().max().item() / max(want.abs().max().item(), 1e-9)
        assert err <= tol, f"{name}: {err}"
        assert (got * ~real).abs().max().item() == 0.0, f"{name}: padded slots must be zero"

    # packed layout: the same numbers on the real tokens
    from tests.test_gpu_packed import _pack
    lengths = torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV)
    packed = br.BlockMask.from_lengths(lengths, H=H, packed=True, dtype=dtype)
    dqp, dkp = run(packed, _pack(q0, lay.valid), _pack(k0, lay.valid))
    assert torch.equal(dqp, _pack(dq, lay.valid)) and torch.equal(dkp, _pack(dk, lay.valid))

    # through the loss API (the training path of trainer.py:91-101)
    q = q0.clone().requires_grad_(True)
    k = k0.clone().requires_grad_(True)
    h = br.LastBlockScores(q, k, br.BlockMask(valid, dtype), scale, R)
    loss, acc = br.compute_auxiliary_attention_loss(h, lay.labels.to(DEV), valid, answer_ids=torch.tensor([[1], [0]], device=DEV))
    loss.backward()
    assert torch.isfinite(q.grad).all() and torch.isfinite(k.grad).all() and q.grad.abs().max() > 0 and k.grad.abs().max() > 0


def test_gradient_of_the_logits_rows_named_twice():
    """The C entry with a row given twice: its two gradient rows add up in dq (one row of the tensor)."""
    from blockrank_amd import _lib
    from blockrank_amd.attention import _stream_ptr
    lay = synthetic.make_layout([[8, 20, 12, 16]])
    Nq, Nkv, D, scale = 4, 2, 64, 0.2
    q, k, _ = synthetic.random_qkv(lay, Nq, Nkv, D, torch.float32, DEV, seed=1)
    bm = br.BlockMask(lay.valid.to(DEV), torch.float32)
    rows = torch.tensor([[lay.H - 3, lay.H - 1, lay.H - 3]], dtype=torch.int32, device=DEV)   # real positions of the query block
    ds = torch.randn(1, Nq, 3, lay.S, generator=torch.Generator().manual_seed(3)).to(DEV)
    lib = _lib.load()
    plan = bm.plan(Nq, Nkv)
    dq = torch.zeros(1, lay.S, Nq, D, device=DEV)
    dk = torch.empty(1, lay.S, Nkv, D, device=DEV)
    _lib.check(lib.br_last_block_logits_bwd(ds.data_ptr(), q.data_ptr(), k.data_ptr(), plan.data_ptr(), rows.data_ptr(), 3, 1, Nq, Nkv, bm.M, bm.H, D,
                                            _lib.strides3(q), _lib.strides3(k), scale, 0, dq.data_ptr(), _lib.strides3(dq.transpose(1, 2)),
                                            dk.data_ptr(), _lib.strides3(dk.transpose(1, 2)), _stream_ptr(torch.device(DEV))))
    vrow = lay.valid.reshape(1, lay.S).to(DEV)
    kk = (k * vrow[:, None, :, None]).repeat_interleave(Nq // Nkv, dim=1)
    per_row = scale * torch.einsum("bnrs,bnsd->bnrd", ds, kk)                 # (1, Nq, 3, D)
    tok = 3 * lay.H + rows[0].long()
    want = torch.zeros_like(dq)
    want[0, tok[0]] = per_row[0, :, 0] + per_row[0, :, 2]
    want[0, tok[1]] = per_row[0, :, 1]
    torch.testing.assert_close(dq, want, rtol=1e-5, atol=1e-5)
