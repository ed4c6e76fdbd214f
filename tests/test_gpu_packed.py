"""Packed token layout (no padded slots): same kernels, same plan items, tokens addressed through the
plan's token table.  Everything must equal the padded layout on the real tokens."""
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _pack(t, valid):            # (B, heads, S, D) -> (1, heads, T, D)
    B, Hh, S, D = t.shape
    keep = valid.reshape(B * S).to(t.device)
    return t.permute(1, 0, 2, 3).reshape(Hh, B * S, D)[:, keep][None].contiguous()


@pytest.mark.parametrize("dtype,Nq,Nkv,D", [(torch.bfloat16, 8, 2, 128), (torch.float32, 4, 2, 64), (torch.bfloat16, 14, 2, 64)])
def test_packed_equals_padded(dtype, Nq, Nkv, D):
    lay = synthetic.make_layout([[5, 17, 0, 300, 33, 19], [40, 1, 65, 31, 2, 70], [64, 64, 64, 64, 64, 16]])
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, dtype, DEV, seed=3)
    scale = D ** -0.5
    padded = br.BlockMask(lay.valid.to(DEV), dtype)
    lengths = torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV)
    packed = br.BlockMask.from_lengths(lengths, H=lay.H, packed=True, dtype=dtype)
    assert packed.total_tokens == int(lay.lengths.sum())
    qp, kp, vp = (_pack(t, lay.valid) for t in (q, k, v))
    R = 16
    if dtype == torch.bfloat16:
        out, part = br.blockrank_attention(q, k, v, padded, scale, score_rows=R)
        outp, partp = br.blockrank_attention(qp, kp, vp, packed, scale, score_rows=R)
    else:
        out = br.blockrank_attention(q, k, v, padded, scale)
        outp = br.blockrank_attention(qp, kp, vp, packed, scale)
    assert outp.shape == (1, packed.total_tokens, Nq, D)
    rows_real = lay.valid.reshape(lay.B, lay.S).to(DEV)
    assert torch.equal(out[rows_real], outp[0]), "packed and padded attention outputs differ on real tokens"
    rows = torch.tensor([[14, 15], [3, 15], [0, 1]], dtype=torch.int32, device=DEV)
    pos = rows + (lay.H - R)
    want = br.doc_scores(q, k, padded, pos, scale)
    got = br.doc_scores(qp, kp, packed, pos, scale)
    assert torch.equal(got, want)
    if dtype == torch.bfloat16:
        f_pad = br.doc_scores_from_partials(part, padded, rows, R, Nq, Nkv)
        f_pack = br.doc_scores_from_partials(partp, packed, rows, R, Nq, Nkv)
        assert torch.equal(f_pack, f_pad)
        torch.testing.assert_close(f_pack, want, rtol=1e-3, atol=1e-5)
    lp = br.last_block_logits(q, k, padded, pos, scale)
    lk = br.last_block_logits(qp, kp, packed, pos, scale)
    assert lk.shape == lp.shape == (lay.B, Nq, 2, lay.S)
    assert torch.equal(lk, lp)
    neg = 0.7 * torch.finfo(dtype).min
    assert torch.all(lk[(~rows_real)[:, None, None, :].expand_as(lk)] == neg)


def test_plan_from_lengths_equals_plan_from_mask():
    lay = synthetic.random_layout(3, 20, 7, 1, 90, 24, seed=5)
    q, k, v = synthetic.random_qkv(lay, 8, 2, 64, torch.bfloat16, DEV, seed=5)
    a = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    b = br.BlockMask.from_lengths(torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV), H=lay.H, packed=False)
    pa, pb = a.plan(8, 2), b.plan(8, 2)
    n = 96 + 3 * lay.B * lay.M                      # header, block starts, lengths and token table
    assert torch.equal(pa[:n], pb[:n])
    assert torch.equal(br.blockrank_attention(q, k, v, a, 0.125), br.blockrank_attention(q, k, v, b, 0.125))
    assert torch.equal(b.dense(torch.bfloat16), a.dense(torch.bfloat16))


def test_packed_ranker_equals_padded_ranker():
    from tests.test_gpu_hf_model import build
    br.register_triton_blockrank_attention()
    model = build("mistral", torch.bfloat16)
    model.set_attn_implementation("triton_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    lay.labels[:] = -100
    lay.labels[:, -2:] = 7
    ids = torch.randint(0, 512, (lay.B, lay.S), generator=torch.Generator().manual_seed(3))
    batch = dict(input_ids=ids, position_ids=lay.position_ids, attention_mask=lay.valid, labels=lay.labels)
    pk = br.pack_padded_batch(batch)
    assert pk["input_ids"].shape == (1, int(lay.lengths.sum()))
    ranker = br.TruncatedRanker(model, 1)
    want = ranker(ids.to(DEV), lay.valid.to(DEV), lay.position_ids.to(DEV), labels=lay.labels.to(DEV))
    got = ranker.forward_packed(pk["input_ids"].to(DEV), pk["position_ids"].to(DEV), pk["block_lengths"].to(DEV),
                                pk["score_rows"].to(DEV), H=pk["H"])
    # the dense layers see the same tokens in both layouts; only the GEMM shapes differ
    torch.testing.assert_close(got, want, rtol=2e-2, atol=1e-3)
    assert torch.equal(br.rank_documents(got, 3), br.rank_documents(want, 3))
