"""Q K^T in fp8 e4m3, P V in bf16 (the benchmark configuration with Qwen2.5-7B attention shapes: 28 query
heads / 4 kv heads, D = 128).  K carries one power-of-two scale per (sequence, kv head), every query row its own
scale (applied in registers by the attention kernel); the query block's rows - the ones the scores
are read from - are computed on the bf16 Q and K.  Two checks:
  * against the oracle fed with the same quantised Q and K (oracle.quantize_fp8_e4m3) for the prefix and
    document rows and with the unquantised ones for the query block: the kernel's own arithmetic, to the
    usual bf16 bar (outputs 2e-2 max-abs, scores 1e-3 relative);
  * against the unquantised fp32 oracle, the variant as a whole, at the bound that benchmark configuration states:
    every score within 5e-3 relative, identical top-10."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc
from tests._util import assert_scores_close, max_abs_on_real_rows, oracle_attention, oracle_doc_scores

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run(lay, Nq, Nkv, seed, hidden=None):
    D = 128
    if hidden:
        q, k, v = synthetic.attention_layer_inputs(lay, Nq, Nkv, D, hidden, torch.bfloat16, DEV)
    else:
        q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=seed)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    scale = D ** -0.5
    R = min(16, lay.H)
    out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R, qk_fp8=True)
    rows = torch.tensor([[R - 2, R - 1]] * lay.B, dtype=torch.int32, device=DEV)
    scores = br.doc_scores_from_partials(part, mask, rows, R, Nq, Nkv)
    return q, k, v, out, scores, scale


@pytest.mark.parametrize("Nq,Nkv,kind", [(28, 4, "qwen"), (32, 8, "mistral"), (8, 8, "mha")])
def test_fp8_kernel_matches_oracle_on_quantised_inputs(Nq, Nkv, kind):
    lay = synthetic.lognormal_layout(2, 32, 12, 120, 0.6, 16, 512, 24, seed=1) if kind == "qwen" else \
        synthetic.random_layout(2, 40, 6, 10, 200, 30, seed=2)
    q, k, v, out, scores, scale = _run(lay, Nq, Nkv, 4)
    qd = orc.quantize_fp8_e4m3(q.cpu(), lay.valid, per_row=True)
    kd = orc.quantize_fp8_e4m3(k.cpu(), lay.valid)
    want = oracle_attention(qd, kd, v, lay, scale)
    want16 = oracle_attention(q, k, v, lay, scale)
    last = slice((lay.M - 1) * lay.H, lay.M * lay.H)
    want[:, last] = want16[:, last]                  # the query block runs in bf16
    assert max_abs_on_real_rows(out, want, lay) <= 2e-2
    assert_scores_close(scores, oracle_doc_scores(q, k, lay, scale))
    # the fp8 logits are really used: the document rows differ from the bf16 kernel's
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    out16 = br.blockrank_attention(q, k, v, mask, scale)
    assert not torch.equal(out[:, :last.start], out16[:, :last.start])
    real_last = lay.valid.reshape(lay.B, lay.S)[:, last].to(DEV)
    assert torch.equal(out[:, last][real_last], out16[:, last][real_last])


def test_config5_scores_against_fp32_oracle():
    # that configuration at full size: B=4, 50 lognormal documents, projection + RoPE inputs
    lay = synthetic.lognormal_layout(4, 32, 50, 120, 0.6, 16, 512, 24, seed=0)
    q, k, v, out, scores, scale = _run(lay, 28, 4, 0, hidden=3584)
    want = oracle_doc_scores(q, k, lay, scale)                    # unquantised, float64 arithmetic
    assert_scores_close(scores, want, rel=5e-3)
    got = scores.cpu().double().numpy()
    assert (orc.topk_indices(got, 10) == orc.topk_indices(want, 10)).all()
    np.testing.assert_allclose(scores.sum(-1).cpu().numpy() * 0.05, 1.0, rtol=1e-4)
    # outputs against the fp32 oracle on the unquantised inputs: rows of the prefix and the documents carry the
    # e4m3 error of their logits (three mantissa bits), a sanity bound only; the query block's rows meet the bf16 bar
    want_o = oracle_attention(q, k, v, lay, scale)
    rows = lay.valid.reshape(lay.B, lay.S)
    diff = (out.float().cpu() - want_o).abs()
    assert diff[rows].mean().item() <= 2e-2 and diff[rows].max().item() <= 0.5, (diff[rows].mean().item(), diff[rows].max().item())
    last = slice((lay.M - 1) * lay.H, lay.M * lay.H)
    assert diff[:, last][rows[:, last]].max().item() <= 2e-2


def test_fp8_packed_equals_padded_and_errors():
    lay = synthetic.make_layout([[5, 17, 0, 300, 33, 19], [40, 1, 65, 31, 2, 70]])
    q, k, v = synthetic.random_qkv(lay, 8, 2, 128, torch.bfloat16, DEV, seed=3)
    padded = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    packed = br.BlockMask.from_lengths(torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV), H=lay.H, packed=True)
    keep = lay.valid.reshape(-1).to(DEV)
    pk = lambda t: t.permute(1, 0, 2, 3).reshape(t.shape[1], -1, t.shape[3])[:, keep][None].contiguous()
    a = br.blockrank_attention(q, k, v, padded, 0.1, qk_fp8=True)
    b = br.blockrank_attention(pk(q), pk(k), pk(v), packed, 0.1, qk_fp8=True)
    assert torch.equal(a[lay.valid.reshape(lay.B, lay.S).to(DEV)], b[0])
    with pytest.raises(NotImplementedError):
        br.blockrank_attention(q.float(), k.float(), v.float(), br.BlockMask(lay.valid.to(DEV)), 0.1, qk_fp8=True)
    q64, k64, v64 = synthetic.random_qkv(lay, 8, 2, 64, torch.bfloat16, DEV, seed=3)
    with pytest.raises(NotImplementedError):
        br.blockrank_attention(q64, k64, v64, padded, 0.1, qk_fp8=True)
