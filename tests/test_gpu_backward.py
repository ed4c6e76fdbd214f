"""Backward of the block-sparse attention (bf16): dq, dk, dv of the HIP kernel, reached through the autograd
function and the C ABI, against the oracle's closed-form float64 gradients on the same bf16 inputs.

Tolerance: the kernel rounds P, dS, O and the results to bf16 and sums in fp32, so every gradient tensor must
be within 2e-2 of its own largest magnitude (max-abs, the same bar as the forward's outputs, scaled because
gradients are not O(1)); the saved log-sum-exp within 2e-3 absolute.  Rows of padded slots must be zero."""
import math

import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from oracle import blockrank_oracle as orc
from tests._util import real_rows

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check(lay, Nq, Nkv, D, seed=0, packed=False):
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=seed)
    scale = D ** -0.5
    gen = torch.Generator().manual_seed(seed + 1000)
    dout = torch.randn((lay.B, lay.S, Nq, D), generator=gen).to(torch.bfloat16).to(DEV)
    want = orc.dense_attention_backward(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                        dout.float().cpu().numpy(), lay.valid.numpy(), scale)
    rows = real_rows(lay)                                                   # (B, S)
    if packed:
        from tests.test_gpu_packed import _pack
        lengths = torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV)
        mask = br.BlockMask.from_lengths(lengths, H=lay.H, packed=True, dtype=torch.bfloat16)
        qq, kk, vv = (_pack(t, lay.valid).requires_grad_(True) for t in (q, k, v))
        out = br.blockrank_attention(qq, kk, vv, mask, scale)
        out.backward(dout[rows.to(DEV)][None])
        grads = []
        for t, heads in ((qq, Nq), (kk, Nkv), (vv, Nkv)):
            full = torch.zeros((lay.B, heads, lay.S, D), dtype=torch.float32)
            full.transpose(1, 2)[rows] = t.grad.float().cpu()[0].transpose(0, 1)
            grads.append(full)
    else:
        mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = br.blockrank_attention(qq, kk, vv, mask, scale)
        out.backward(dout)
        grads = [t.grad.float().cpu() for t in (qq, kk, vv)]
    torch.cuda.synchronize()
    for name, got, ref in zip(("dq", "dk", "dv"), grads, want[:3]):
        got = got.numpy().astype(np.float64)
        assert np.isfinite(got).all(), f"{name} has non-finite values"
        real = rows.numpy()[:, None, :, None]
        assert (got * ~real == 0).all(), f"{name}: rows of padded slots must be zero"
        err = np.abs(got - ref).max()
        bound = 2e-2 * max(np.abs(ref).max(), 1e-6)
        assert err <= bound, f"{name}: max abs error {err:.3e} > {bound:.3e} (largest gradient {np.abs(ref).max():.3e})"
    return want[3]


def test_saved_log_sum_exp_matches_oracle():
    lay = synthetic.make_layout([[40, 100, 160, 33, 192, 20], [64, 7, 150, 90, 0, 31]])
    Nq, Nkv, D = 8, 2, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=3)
    qq = q.clone().requires_grad_(True)
    out = br.blockrank_attention(qq, k, v, br.BlockMask(lay.valid.to(DEV), torch.bfloat16), D ** -0.5)
    lse = out.grad_fn.saved_tensors[4].cpu().double().numpy() * math.log(2.0)
    *_, want = orc.dense_attention_backward(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                            np.zeros((lay.B, lay.S, Nq, D)), lay.valid.numpy(), D ** -0.5)
    rows = np.broadcast_to(real_rows(lay).numpy()[:, None, :], want.shape)
    assert np.abs(lse[rows] - want[rows]).max() <= 2e-3


def test_log_sum_exp_of_split_rows_is_exact_too():
    # one request with many documents: the query block's key walk is cut into several items and its rows' log-sum-exp
    # comes from the merge of their partials.  Peaked rows (large logits: one key carries the mass, so the sum of the
    # bf16-rounded probabilities that normalises the output is off from the exact one by up to 2^-9) must come out as
    # exact as the rows a single item finishes: 1e-4 in natural-log units.
    lay = synthetic.random_layout(1, 48, 40, 30, 96, 24, seed=8)
    Nq, Nkv, D = 8, 2, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=5)
    q = (q * 6).contiguous()
    qq = q.clone().requires_grad_(True)
    out = br.blockrank_attention(qq, k, v, br.BlockMask(lay.valid.to(DEV), torch.bfloat16), D ** -0.5)
    lse = out.grad_fn.saved_tensors[4].cpu().double().numpy() * math.log(2.0)
    *_, want = orc.dense_attention_backward(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                            np.zeros((lay.B, lay.S, Nq, D)), lay.valid.numpy(), D ** -0.5)
    rows = np.broadcast_to(real_rows(lay).numpy()[:, None, :], want.shape)
    err = np.abs(lse - want)
    assert err[rows].max() <= 1e-4
    last = np.zeros_like(rows)
    last[:, :, -lay.H:] = rows[:, :, -lay.H:]                    # the query block's rows: the split ones
    assert last.any() and err[last].max() <= 1e-4


def test_ragged_blocks_four_heads_per_group():
    _check(synthetic.make_layout([[40, 100, 160, 33, 192, 20], [64, 7, 150, 90, 0, 31]]), 8, 2, 128)


@pytest.mark.parametrize("G", [1, 2, 3, 7, 8])
def test_head_group_sizes(G):
    _check(synthetic.make_layout([[20, 70, 45, 130, 37]]), 2 * G, 2, 128, seed=G)


def test_head_dim_64():
    _check(synthetic.make_layout([[5, 17, 0, 64, 33, 9], [40, 1, 65, 31, 2, 70]]), 8, 2, 64, seed=11)


def test_single_block_and_no_documents():
    _check(synthetic.make_layout([[100]]), 4, 2, 128, seed=12)
    _check(synthetic.make_layout([[100, 50]]), 4, 2, 128, seed=13)
    _check(synthetic.make_layout([[0, 30, 0, 40, 5]]), 4, 1, 128, seed=14)


def test_long_document_list_splits_the_query_walk():
    # 30 documents of up to 96 tokens: the query block's key walk is cut into several items whose dq partial
    # sums meet in the accumulation buffer
    lay = synthetic.random_layout(1, 48, 30, 30, 96, 24, seed=4)
    _check(lay, 8, 2, 128, seed=15)


def test_packed_layout():
    _check(synthetic.make_layout([[40, 100, 160, 33, 192, 20], [64, 7, 150, 90, 0, 31]]), 8, 2, 128, seed=16, packed=True)


def test_random_layouts():
    """Seeded random block layouts (empty, one-token, tile-edge and long blocks; every head grouping; both head
    dims), the same generator as the forward's randomised test."""
    from tests.test_gpu_random_layouts import _cases
    for it, lens, G, Nkv, D in _cases(seed=23, n=16):
        lay = synthetic.make_layout(lens)
        if lay.S > 2600:                                   # keep the dense float64 oracle within seconds
            continue
        try:
            _check(lay, G * Nkv, Nkv, D, seed=100 + it)
        except AssertionError as e:
            raise AssertionError(f"case {it}: lengths {lens}, {G} heads per kv head, {Nkv} kv heads, D={D}: {e}") from e
