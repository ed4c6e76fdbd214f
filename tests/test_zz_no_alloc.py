"""br_prefill_fwd_noalloc (the entry point for callers that cannot allocate device memory) against br_prefill_fwd,
through the C ABI: same plan, same inputs, outputs must be identical bit for bit (same kernels, the split-KV
partials in the library's own device array instead of a caller workspace).  Two calls in a row, the second on a
smaller request, so that whatever the first left in the array is there when the second runs."""
import numpy as np
import pytest
import torch

from blockrank_amd import _lib, synthetic
from blockrank_amd.attention import BlockMask, _stream_ptr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(lay, Nq, Nkv, D, seed):
    lib = _lib.load()
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=seed)
    mask = BlockMask(lay.valid.to(DEV), torch.bfloat16)
    plan = mask.plan(Nq, Nkv)
    B, M, H, S = lay.B, lay.M, lay.H, lay.S
    ws_bytes = lib.br_prefill_workspace_bytes(B, Nq, Nkv, D)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    outs = [torch.full((B, S, Nq, D), float("nan"), dtype=torch.bfloat16, device=DEV) for _ in range(2)]
    so = _lib._I64x3(S * Nq * D, D, Nq * D)
    args = lambda o: (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), plan.data_ptr(), B, Nq, Nkv, M, H, D,
                      _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), so, D ** -0.5, _lib.BR_DTYPE_BF16)
    _lib.check(lib.br_prefill_fwd(*args(outs[0]), ws.data_ptr(), ws_bytes, _stream_ptr(torch.device(DEV))))
    _lib.check(lib.br_prefill_fwd_noalloc(*args(outs[1]), _stream_ptr(torch.device(DEV))))
    torch.cuda.synchronize()
    return outs


def test_noalloc_entry_matches_workspace_entry_twice():
    # first call: a long query block (its key walk is split: partials are used), B = 3
    big = synthetic.random_layout(3, 64, 30, 60, 200, 48, seed=5)
    a, b = _both(big, 32, 8, 128, 1)
    assert not torch.isnan(a.float()).any()
    assert torch.equal(a, b)
    # second call, smaller request, other head layout: the array still holds the first call's partials
    small = synthetic.random_layout(1, 40, 12, 20, 130, 24, seed=6)
    a, b = _both(small, 8, 2, 64, 2)
    assert not torch.isnan(a.float()).any()
    assert torch.equal(a, b)


def test_noalloc_entry_serves_the_config3_batch():
    # BASELINE config 3's batch: B = 8 at Mistral heads, 20 documents of U[96, 224] tokens (the partial pool does not
    # grow with the batch, so the built-in array holds it)
    rng = np.random.default_rng(0)
    lay = synthetic.make_layout([[64] + [int(x) for x in rng.integers(96, 225, 20)] + [32] for _ in range(8)])
    lib = _lib.load()
    assert lib.br_prefill_workspace_bytes(8, 32, 8, 128) <= lib.br_prefill_noalloc_max_workspace_bytes()
    a, b = _both(lay, 32, 8, 128, 3)
    assert not torch.isnan(a.float()).any()
    assert torch.equal(a, b)


def test_noalloc_entry_under_graph_capture():
    # the callers this entry is for: captured once (after the plan was built, which is what looks the array up),
    # replayed several times with eager work in between; every replay must reproduce the eager result
    lib = _lib.load()
    lay = synthetic.random_layout(2, 64, 12, 60, 200, 40, seed=9)
    Nq, Nkv, D = 32, 8, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=4)
    mask = BlockMask(lay.valid.to(DEV), torch.bfloat16)
    plan = mask.plan(Nq, Nkv)
    B, M, H, S = lay.B, lay.M, lay.H, lay.S
    so = _lib._I64x3(S * Nq * D, D, Nq * D)
    sq, sk, sv = _lib.strides3(q), _lib.strides3(k), _lib.strides3(v)

    def call(o, stream):
        _lib.check(lib.br_prefill_fwd_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), plan.data_ptr(), B, Nq, Nkv, M, H, D,
                                              sq, sk, sv, so, D ** -0.5, _lib.BR_DTYPE_BF16, stream))

    eager = torch.empty((B, S, Nq, D), dtype=torch.bfloat16, device=DEV)
    call(eager, _stream_ptr(torch.device(DEV)))
    torch.cuda.synchronize()
    out = torch.empty_like(eager)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(out, torch.cuda.current_stream().cuda_stream)
    for i in range(3):
        out.fill_(float("nan"))
        junk = torch.randn(1 << 20, device=DEV).sum()          # the program's own eager work between replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"
        del junk


def test_noalloc_entry_refuses_what_does_not_fit():
    lib = _lib.load()
    cap = lib.br_prefill_noalloc_max_workspace_bytes()
    assert cap == 32 << 20
    # the partial pool follows the head layout, not the batch: only an absurd one (1024 kv heads) exceeds the array
    assert lib.br_prefill_workspace_bytes(1, 1024, 1024, 128) > cap
    rc = lib.br_prefill_fwd_noalloc(None, None, None, None, None, 1, 1024, 1024, 3, 64, 128, None, None, None, None, 1.0, 1, None)
    assert rc == _lib.BR_ERR_SPACE and b"built-in scratch" in lib.br_last_error()
