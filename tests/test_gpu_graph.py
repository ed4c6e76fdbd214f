"""The attention + score step captured in a HIP graph: every replay must give the eager result, also with
eager launches of the same library (which use and re-arm the same plan's ticket counters) in between.
The library allocates nothing and records no memset: the plan's counters are re-armed by the last
workgroup of each launch."""
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_graph_replays_equal_eager():
    lay = synthetic.make_layout([[40, 100, 160, 33, 192, 20], [64, 7, 150, 90, 0, 31]])
    Nq, Nkv, D = 8, 2, 128
    scale = D ** -0.5
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=5)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    R = 16
    rows = torch.tensor([[R - 2, R - 1]] * lay.B, dtype=torch.int32, device=DEV)

    def step():
        out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R)
        return out, br.doc_scores_from_partials(part, mask, rows, R, Nq, Nkv)

    want_out, want_scores = step()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()                                   # warm-up on the capture stream
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            g_out, g_scores = step()
    torch.cuda.synchronize()
    for i in range(4):
        g_out.fill_(float("nan"))
        g_scores.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_out, want_out), f"replay {i}: attention output differs from the eager result"
        assert torch.equal(g_scores, want_scores), f"replay {i}: scores differ from the eager result"
        e_out, e_scores = step()                 # eager work of the same kind between the replays
        torch.cuda.synchronize()
        assert torch.equal(e_out, want_out) and torch.equal(e_scores, want_scores)


def test_training_step_in_a_graph():
    """Forward with saved log-sum-exp + backward captured in a HIP graph (the backward clears its fp32 sum buffers with
    a fill kernel, not a memset node): replays give the eager gradients, eager steps in between.  The fp32 atomic
    sums of shared rows may differ in the last bit between runs, so gradients are compared to 1e-2 of their largest
    magnitude rather than bit for bit."""
    lay = synthetic.make_layout([[40, 100, 160, 33, 192, 20], [64, 7, 150, 90, 0, 31]])
    Nq, Nkv, D = 8, 2, 128
    scale = D ** -0.5
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=9)
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    dout = torch.randn((lay.B, lay.S, Nq, D), generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).to(DEV)
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))

    def step():
        for t in (qq, kk, vv):
            t.grad = None
        br.blockrank_attention(qq, kk, vv, mask, scale).backward(dout)
        return [t.grad for t in (qq, kk, vv)]

    want = [g.clone() for g in step()]
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            grads = step()
    torch.cuda.synchronize()
    for i in range(3):
        for t in grads:
            t.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("dq", "dk", "dv"), grads, want):
            err = (a.float() - b.float()).abs().max().item()
            assert err <= 1e-2 * b.float().abs().max().item(), f"replay {i}: {name} differs from the eager result by {err}"
        eager = br.blockrank_attention(q, k, v, mask, scale)          # eager work of the same library between the replays
        torch.cuda.synchronize()
        assert torch.isfinite(eager[lay.valid.reshape(lay.B, lay.S).to(DEV)].float()).all()
