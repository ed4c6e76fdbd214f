"""The committed known-answer case (tests/golden/kat_small.npz, written by tests/golden/make_fixtures.py from
the oracle): the oracle must still reproduce it, and the HIP path must match it through the C ABI - fp32 to
1e-5 on the attention output, bf16 to 2e-2, scores to 1e-3 relative with the same order."""
import os

import numpy as np
import pytest
import torch

from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc

KAT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat_small.npz")


def _load():
    d = np.load(KAT, allow_pickle=False)
    lay = synthetic.make_layout(d["lengths"].tolist(), H=int(d["H"]))
    return d, lay


def test_oracle_reproduces_the_fixture():
    d, lay = _load()
    assert (lay.labels.numpy() == d["labels"]).all()
    q, k, v = (torch.from_numpy(d[n]) for n in ("q", "k", "v"))
    out, _ = orc.sdpa_blockrank_forward(q, k, v, orc.additive_mask(lay.valid, torch.float32), float(d["scale"]))
    rows = lay.valid.reshape(lay.B, lay.S)
    np.testing.assert_allclose(out.numpy()[rows], d["out"][rows], rtol=0, atol=1e-6)
    scores = orc.doc_scores(d["q"], d["k"], lay.valid.numpy(), d["labels"], float(d["scale"]), 0.05, 16)
    np.testing.assert_allclose(scores, d["scores"], rtol=1e-9, atol=1e-12)
    assert (orc.topk_indices(scores, 10) == d["top"]).all()
    # an empty document gets no attention mass at all, and every row of scores sums to 1 / temperature
    assert d["scores"][0, 1] == 0.0
    np.testing.assert_allclose(d["scores"].sum(-1), 1 / 0.05, rtol=1e-9)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_hip_path_matches_the_fixture(dtype, tol):
    import blockrank_amd as br
    d, lay = _load()
    dev = "cuda:0"
    q, k, v = (torch.from_numpy(d[n]).to(dev, dtype) for n in ("q", "k", "v"))
    scale = float(d["scale"])
    mask = br.BlockMask(lay.valid.to(dev), dtype)
    out = br.blockrank_attention(q, k, v, mask, scale)
    rows = lay.valid.reshape(lay.B, lay.S)
    want = torch.from_numpy(d["out"])
    if dtype == torch.bfloat16:      # the fixture is the fp32 result of fp32 inputs: compare against it with the inputs' rounding in the bound
        q32, k32, v32 = (t.float().cpu() for t in (q, k, v))
        want, _ = orc.sdpa_blockrank_forward(q32, k32, v32, orc.additive_mask(lay.valid, torch.float32), scale)
    err = (out.float().cpu()[rows] - want[rows]).abs().max().item()
    assert err <= tol, f"max abs error {err:.3e}"
    assert (out.cpu()[~rows] == 0).all()
    pos = torch.tensor([[lay.H - 2, lay.H - 1]] * lay.B, dtype=torch.int32, device=dev)
    scores = br.doc_scores(q, k, mask, pos, scale, temperature=0.05).cpu().double().numpy()
    if dtype == torch.float32:
        np.testing.assert_allclose(scores, d["scores"], rtol=1e-3, atol=1e-6)
        assert (orc.topk_indices(scores, 10) == d["top"]).all()
    else:
        np.testing.assert_allclose(scores, d["scores"], rtol=5e-2, atol=5e-2)     # bf16-rounded inputs against the fp32 fixture
