"""RMSNorm and SiLU-gate kernels against the oracle (float64) and against the model file's own expressions.

Tolerances: fp32 within 2e-6 relative of the float64 result; bf16 within one rounding step of it per rounding the
model file performs (two: 2 * 2^-8 relative), and no further from it than the model file's own bf16 expression."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from oracle import blockrank_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("dtype,hidden", [(torch.bfloat16, 4096), (torch.bfloat16, 3584), (torch.bfloat16, 256), (torch.float32, 4096),
                                          (torch.bfloat16, 8192), (torch.float32, 4100)])
def test_rms_norm(dtype, hidden):
    g = torch.Generator().manual_seed(hidden)
    x = (torch.randn((3, 37, hidden), generator=g) * torch.rand((3, 37, 1), generator=g) * 4).to(dtype).to(DEV)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype).to(DEV)
    got = br.rms_norm(x, w, 1e-5)
    assert got.shape == x.shape and got.dtype == dtype
    want = orc.rms_norm(x.float().cpu().numpy(), w.float().cpu().numpy(), 1e-5)
    tol = 2e-6 if dtype == torch.float32 else 2 * 2.0 ** -8
    err = np.abs(got.float().cpu().numpy() - want) / np.maximum(np.abs(want), 1e-3)
    assert err.max() <= tol, f"max relative error {err.max():.3e}"
    # the model file's expression (transformers MistralRMSNorm.forward)
    h = x.float()
    ref = w * (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-5)).to(dtype)
    ref_err = np.abs(ref.float().cpu().numpy() - want) / np.maximum(np.abs(want), 1e-3)
    assert err.mean() <= ref_err.mean() * 1.5 + 1e-9          # (fp32: both are at the last bit; the summation order differs)
    # a strided view (rows further apart than hidden)
    big = torch.zeros((5, hidden + 64), dtype=dtype, device=DEV)
    big[:, :hidden] = x[0, :5]
    assert torch.equal(br.rms_norm(big[:, :hidden], w, 1e-5), got[0, :5])


def test_rms_norm_rejects_rows_it_cannot_hold():
    x = torch.zeros((2, 8196), dtype=torch.float32, device=DEV)          # 2049 16-byte pieces: one more than the kernel keeps
    with pytest.raises(AssertionError, match="too large"):
        br.rms_norm(x, torch.ones(8196, device=DEV), 1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_silu_mul(dtype):
    g = torch.Generator().manual_seed(3)
    a = (torch.randn((2, 19, 14336), generator=g) * 3).to(dtype).to(DEV)
    b = torch.randn((2, 19, 14336), generator=g).to(dtype).to(DEV)
    got = br.silu_mul(a, b)
    want = orc.silu_mul(a.float().cpu().numpy(), b.float().cpu().numpy())
    tol = 2e-6 if dtype == torch.float32 else 2 * 2.0 ** -8
    err = np.abs(got.float().cpu().numpy() - want) / np.maximum(np.abs(want), 1e-3)
    assert err.max() <= tol, f"max relative error {err.max():.3e}"
    ref = torch.nn.functional.silu(a) * b
    ref_err = np.abs(ref.float().cpu().numpy() - want) / np.maximum(np.abs(want), 1e-3)
    assert err.mean() <= ref_err.mean() * 1.5 + 1e-9          # (fp32: both are at the last bit; the summation order differs)


@pytest.mark.parametrize("kind", ["mistral", "qwen2"])
def test_patched_model_matches_unpatched(kind):
    from tests.test_gpu_hf_model import build
    from blockrank_amd import synthetic
    br.register_blockrank_attention()
    model = build(kind, torch.bfloat16)
    model.set_attn_implementation("sdpa_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    ids = torch.randint(0, 512, (lay.B, lay.S), generator=torch.Generator().manual_seed(1)).to(DEV)
    kw = dict(input_ids=ids, position_ids=lay.position_ids.to(DEV), attention_mask=lay.valid.to(DEV), output_hidden_states=True, use_cache=False)
    with torch.no_grad():
        ref = model(**kw).hidden_states[-1].float()
        n = br.patch_layer_ops(model)
        assert n == 3 * 2 + 1 + 3, "two norms and an MLP per layer, and the final norm"
        got = model(**kw).hidden_states[-1].float()
        br.unpatch_layer_ops(model)
        again = model(**kw).hidden_states[-1].float()
    rows = lay.valid.reshape(lay.B, lay.S).to(DEV)
    assert torch.equal(again, ref), "unpatching restores the model's own forward"
    err = (got[rows] - ref[rows]).abs().max().item()
    assert err <= 3e-2 * max(1.0, ref[rows].abs().max().item()), f"hidden state differs by {err}"
    # with gradients enabled the modules' own forwards run (the kernels have no backward)
    br.patch_layer_ops(model)
    out = model(**kw).hidden_states[-1]
    assert out.requires_grad
    br.unpatch_layer_ops(model)


@pytest.mark.parametrize("kind", ["mistral", "qwen2"])
def test_stacked_qkv_projection(kind):
    """patch_qkv: one GEMM for the three projections of a decoder layer.  A GEMM over the stacked weight may round its
    sums in another order than three separate ones, so hidden states are compared to the bf16 bar; the ranking path
    (TruncatedRanker, which projects K of all tokens and Q of the query block separately at the scoring layer) must
    keep working on the patched model."""
    from tests.test_gpu_hf_model import build
    from blockrank_amd import synthetic
    br.register_blockrank_attention()
    model = build(kind, torch.bfloat16)          # qwen2 has projection biases
    model.set_attn_implementation("sdpa_blockrank")
    lay = synthetic.make_layout([[12, 30, 17, 25, 9], [10, 22, 31, 8, 11]])
    lay.labels[:] = -100
    lay.labels[:, -2:] = 7
    ids = torch.randint(0, 512, (lay.B, lay.S), generator=torch.Generator().manual_seed(1)).to(DEV)
    pos, valid, labels = lay.position_ids.to(DEV), lay.valid.to(DEV), lay.labels.to(DEV)
    kw = dict(input_ids=ids, position_ids=pos, attention_mask=valid, output_hidden_states=True, use_cache=False)
    ranker = br.TruncatedRanker(model, 1)
    with torch.no_grad():
        ref = model(**kw).hidden_states[-1].float()
        ref_scores = ranker(ids, valid, pos, labels=labels)
        assert br.patch_qkv(model) == 3
        got = model(**kw).hidden_states[-1].float()
        got_scores = ranker(ids, valid, pos, labels=labels)
        br.unpatch_qkv(model)
        again = model(**kw).hidden_states[-1].float()
    rows = valid.reshape(lay.B, lay.S)
    assert torch.equal(again, ref), "unpatching restores the model's own projections"
    err = (got[rows] - ref[rows]).abs().max().item()
    assert err <= 3e-2 * max(1.0, ref[rows].abs().max().item()), f"hidden state differs by {err}"
    torch.testing.assert_close(got_scores, ref_scores, rtol=2e-2, atol=1e-3)
