"""Helpers shared by the GPU parity tests: run the HIP path through the package (which calls the
C ABI) and the CPU oracle on the same tensors."""
import numpy as np
import torch

from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc


def oracle_attention(q, k, v, layout, scale):
    """fp32 oracle output (B, S, Nq, D) for tensors living on any device (values taken as they are)."""
    qc, kc, vc = (t.detach().float().cpu() for t in (q, k, v))
    m5 = orc.additive_mask(layout.valid, torch.float32)
    out, _ = orc.sdpa_blockrank_forward(qc.contiguous(), kc.contiguous(), vc.contiguous(), m5, scale)
    return out


def real_rows(layout):
    return layout.valid.reshape(layout.B, layout.S)


def max_abs_on_real_rows(got, want, layout):
    rows = real_rows(layout)
    g = got.detach().float().cpu()[rows]
    w = want.detach().float().cpu()[rows]
    assert torch.isfinite(g).all(), "non-finite values in the output rows of real tokens"
    return (g - w).abs().max().item() if g.numel() else 0.0


def eval_rows(layout, device):
    """(B, 2) positions of the last two tokens of the query block (the rows the eval recipe uses)."""
    H = layout.H
    return torch.tensor([[H - 2, H - 1]] * layout.B, dtype=torch.int32, device=device)


def oracle_doc_scores(q, k, layout, scale, temperature=0.05, num_last=16):
    qc, kc = (t.detach().float().cpu().numpy() for t in (q, k))
    return orc.doc_scores(qc, kc, layout.valid.numpy(), layout.labels.numpy(), scale, temperature, num_last)


def assert_scores_close(got, want, rel=1e-3, k=10):
    got = got.detach().cpu().double().numpy()
    denom = np.maximum(np.abs(want), 1e-30)
    err = np.abs(got - want) / denom
    # a relative bound on each score, with an absolute floor for documents of vanishing mass
    floor = np.abs(got - want) <= 1e-6 * np.abs(want).max(axis=-1, keepdims=True)
    assert (err <= rel)[~floor].all(), f"max relative score error {err[~floor].max():.3e} > {rel}"
    top_w = orc.topk_indices(want, k)
    top_g = orc.topk_indices(got, k)
    # identical order unless the oracle itself has a near tie (then order is not defined at this precision)
    for b in range(want.shape[0]):
        if (top_w[b] != top_g[b]).any():
            s = want[b][top_w[b]]
            gaps = np.abs(np.diff(s)) / np.abs(s[:-1])
            assert gaps.min() < 2 * rel, f"top-{k} order differs without a near tie: {top_w[b]} vs {top_g[b]}"
