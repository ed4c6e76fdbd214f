"""Parity of the HIP prefill attention with the CPU oracle, on rows of real tokens.
Tolerances (from the target statement): max-abs 1e-5 for fp32, 2e-2 for bf16."""
import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from tests._util import max_abs_on_real_rows, oracle_attention, real_rows

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def check(layout, Nq, Nkv, D, dtype, seed=0, pad_fill=None, scale=None):
    q, k, v = synthetic.random_qkv(layout, Nq, Nkv, D, dtype, DEV, seed=seed, pad_fill=pad_fill)
    scale = scale if scale is not None else D ** -0.5
    out = br.blockrank_attention(q, k, v, layout.valid.to(DEV), scale)
    torch.cuda.synchronize()
    assert out.shape == (layout.B, layout.S, Nq, D) and out.is_contiguous() and out.dtype == dtype
    if pad_fill is not None:
        fill = lambda t: torch.where(~layout.valid.view(layout.B, 1, layout.S, 1).to(DEV), torch.zeros_like(t), t)
        q, k, v = fill(q), fill(k), fill(v)
    want = oracle_attention(q, k, v, layout, scale)
    err = max_abs_on_real_rows(out, want, layout)
    assert err <= TOL[dtype], f"max abs error {err:.3e} > {TOL[dtype]}"
    pad = ~real_rows(layout)
    assert (out.cpu()[pad] == 0).all(), "rows of padded slots must be zero"
    return out


def test_config1_fp32_reference_case():
    # batch 1, fp32, 8 query / 2 kv heads, D=64, 32-token prefix + 8 docs x 64 + 16-token query
    lay = synthetic.uniform_layout(1, 32, 8, 64, 16)
    assert (lay.M, lay.H, lay.S, lay.valid_tokens) == (10, 64, 640, 560)
    assert lay.unmasked_pairs() == 42392
    check(lay, 8, 2, 64, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
def test_ragged_small(dtype, D):
    lay = synthetic.make_layout([[5, 17, 0, 64, 33, 9], [40, 1, 65, 31, 2, 70]])
    check(lay, 8, 2, D, dtype, seed=1)


@pytest.mark.parametrize("G", [1, 2, 3, 4, 5, 6, 7, 8, 16])
def test_head_group_sizes(G):
    # every workgroup shape: G = 7 is Qwen2.5-7B's 28/4, G = 16 splits into two groups of 8
    lay = synthetic.make_layout([[20, 70, 45, 130, 37]])
    check(lay, 2 * G, 2, 128, torch.bfloat16, seed=G)


@pytest.mark.parametrize("G", [1, 3, 7])
def test_head_group_sizes_fp32(G):
    lay = synthetic.make_layout([[20, 70, 45, 37]])
    check(lay, G, 1, 64, torch.float32, seed=G)


def test_single_block_and_two_blocks():
    check(synthetic.make_layout([[100]]), 4, 2, 128, torch.bfloat16)
    check(synthetic.make_layout([[100, 50]]), 4, 2, 128, torch.bfloat16)
    check(synthetic.make_layout([[7]]), 4, 2, 64, torch.float32)
    check(synthetic.make_layout([[0, 9]]), 4, 2, 64, torch.float32)


def test_empty_prefix_empty_docs_empty_query():
    check(synthetic.make_layout([[0, 30, 0, 40, 5]]), 4, 1, 128, torch.bfloat16)
    check(synthetic.make_layout([[12, 0, 0, 0, 3]]), 4, 1, 128, torch.bfloat16)
    check(synthetic.make_layout([[12, 30, 10, 0]], H=32), 4, 1, 128, torch.bfloat16)


def test_long_query_block_many_tiles_and_splits():
    # query block longer than one tile and a key walk long enough to be split many ways
    lay = synthetic.make_layout([[64] + [200] * 12 + [150]])
    check(lay, 8, 2, 128, torch.bfloat16, seed=3)
    check(lay, 4, 2, 64, torch.float32, seed=3)


def test_query_block_longer_than_slot_budget():
    # more query tiles than split slots: the query block falls back to unsplit items
    lay = synthetic.make_layout([[16, 40, 1200]])
    check(lay, 8, 1, 64, torch.bfloat16, seed=4)


def test_garbage_in_padding_is_never_read():
    lay = synthetic.make_layout([[5, 17, 64, 33, 9], [40, 1, 65, 31, 2]])
    check(lay, 8, 2, 128, torch.bfloat16, seed=5, pad_fill=float("nan"))
    check(lay, 4, 2, 64, torch.float32, seed=5, pad_fill=float("inf"))


def test_right_padded_blocks():
    lay = synthetic.make_layout([[20, 50, 33, 10]])
    valid = torch.flip(lay.valid, dims=[-1])            # real tokens at the start of each block
    q, k, v = synthetic.random_qkv(lay, 4, 2, 128, torch.bfloat16, DEV, seed=6)
    out = br.blockrank_attention(q, k, v, valid.to(DEV), 0.1)
    lay2 = synthetic.BlockLayout(lay.lengths, lay.H, valid, lay.position_ids, lay.labels)
    want = oracle_attention(q, k, v, lay2, 0.1)
    assert max_abs_on_real_rows(out, want, lay2) <= 2e-2


def test_reference_dense_mask_and_hf_strides():
    # the reference's (B,1,M,H,H) additive tensor as mask, and q/k/v as head-transposed views of
    # (B,S,heads,D) projections, which is how the attention hook receives them
    lay = synthetic.make_layout([[30, 64, 100, 20]])
    B, S, Nq, Nkv, D = lay.B, lay.S, 8, 2, 128
    g = torch.Generator().manual_seed(7)
    q = torch.randn(B, S, Nq, D, generator=g).to(DEV, torch.bfloat16).transpose(1, 2)
    k = torch.randn(B, S, Nkv, D, generator=g).to(DEV, torch.bfloat16).transpose(1, 2)
    v = torch.randn(B, S, Nkv, D, generator=g).to(DEV, torch.bfloat16).transpose(1, 2)
    assert not q.is_contiguous()
    m5 = br.BlockMask(lay.valid.to(DEV), torch.bfloat16).dense()
    assert m5.shape == (B, 1, lay.M, lay.H, lay.H)
    out = br.blockrank_attention(q, k, v, m5, D ** -0.5)
    want = oracle_attention(q, k, v, lay, D ** -0.5)
    assert max_abs_on_real_rows(out, want, lay) <= 2e-2


def test_repeated_calls_reuse_the_plan():
    lay = synthetic.make_layout([[64] + [100] * 6 + [40]] * 2)
    q, k, v = synthetic.random_qkv(lay, 8, 2, 128, torch.bfloat16, DEV, seed=8)
    bm = br.BlockMask(lay.valid.to(DEV))
    outs = [br.blockrank_attention(q, k, v, bm, 0.09) for _ in range(4)]
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    plan = bm.plan(8, 2)
    assert plan[48].item() == 0 and (plan[32:41] == 0).all()     # done and ticket counters re-armed


def test_plan_left_by_an_unfinished_launch_is_detected_and_rearmed():
    lay = synthetic.make_layout([[64] + [100] * 6 + [40]] * 2)
    q, k, v = synthetic.random_qkv(lay, 8, 2, 128, torch.bfloat16, DEV, seed=8)
    bm = br.BlockMask(lay.valid.to(DEV))
    want = br.blockrank_attention(q, k, v, bm, 0.09)
    assert bm.plans_at_rest()
    plan = bm.plan(8, 2)
    plan[33] = 7                      # what a launch that never finished leaves behind: tickets handed out, nobody home
    plan[48] = 3
    assert not bm.plans_at_rest()
    bm.rearm_plans()
    assert bm.plans_at_rest()
    assert torch.equal(br.blockrank_attention(q, k, v, bm, 0.09), want)


@pytest.mark.parametrize("B", [600, 2100])
def test_more_sequences_than_plan_threads(B):
    # the plan kernel walks one sequence per thread; a batch beyond its 512 threads takes the looping path (the
    # sequences whose blocks straddle two queues' runs have their query block's walk cut in two: partial slots and
    # merges come from both rounds of the loop)
    # (2100 sequences of four blocks are also more blocks than the plan kernel stages in LDS)
    rng = np.random.default_rng(7)
    blocks = [[int(rng.integers(0, 20)), int(rng.integers(0, 40)), int(rng.integers(1, 40)), int(rng.integers(1, 33))] for _ in range(B)]
    lay = synthetic.make_layout(blocks)
    check(lay, 4, 2, 64, torch.bfloat16, seed=11)


def test_config2_full_size():
    # Mistral-7B-shaped layer: B=4, 32/8 heads, D=128, 64 + 20 x 160 + 32 tokens, projections + RoPE
    lay = synthetic.uniform_layout(4, 64, 20, 160, 32)
    assert (lay.M, lay.H, lay.S, lay.valid_tokens) == (22, 160, 3520, 4 * 3296)
    assert lay.unmasked_pairs() == 4 * 569456
    q, k, v = synthetic.attention_layer_inputs(lay, 32, 8, 128, 4096, torch.bfloat16, DEV)
    out = br.blockrank_attention(q, k, v, lay.valid.to(DEV), 128 ** -0.5)
    want = oracle_attention(q, k, v, lay, 128 ** -0.5)
    assert max_abs_on_real_rows(out, want, lay) <= 2e-2


def test_long_list_properties_at_full_size():
    # 100 documents of 64..384 tokens (about 23k tokens): too slow for the dense oracle, so check
    # size-independent properties.  (1) V = 1 gives 1 on every real row; (2) the query block's
    # output does not depend on the order of the documents.
    lay = synthetic.random_layout(1, 64, 100, 64, 384, 48, seed=0)
    Nq, Nkv, D = 32, 8, 128
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=9)
    bm = br.BlockMask(lay.valid.to(DEV))
    ones = br.blockrank_attention(q, k, torch.ones_like(v), bm, D ** -0.5)
    rows = real_rows(lay)
    assert (ones.float().cpu()[rows] - 1).abs().max() <= 1e-2
    out = br.blockrank_attention(q, k, v, bm, D ** -0.5)
    M, H = lay.M, lay.H
    perm = torch.cat([torch.tensor([0]), 1 + torch.randperm(M - 2, generator=torch.Generator().manual_seed(1)), torch.tensor([M - 1])])

    def shuffle(x):
        B, N, S, Dd = x.shape
        return x.view(B, N, M, H, Dd)[:, :, perm.to(x.device)].reshape(B, N, S, Dd)

    lay_p = synthetic.make_layout(lay.lengths[:, perm.numpy()], H=H)
    out_p = br.blockrank_attention(shuffle(q), shuffle(k), shuffle(v), lay_p.valid.to(DEV), D ** -0.5)
    a = out.view(1, M, H, Nq, D)[:, perm.to(DEV)]
    b = out_p.view(1, M, H, Nq, D)
    real = lay_p.valid.to(DEV)
    # documents: identical inputs, identical tile walk -> bitwise equal; query block: same keys in
    # another order -> equal up to bf16 rounding of the output
    assert torch.equal(a[:, 1:-1][real[:, 1:-1]], b[:, 1:-1][real[:, 1:-1]])
    assert (a[:, -1][real[:, -1]].float() - b[:, -1][real[:, -1]].float()).abs().max() <= 2e-2


def test_error_behaviour():
    lay = synthetic.make_layout([[8, 8, 8]])
    q, k, v = synthetic.random_qkv(lay, 4, 2, 128, torch.bfloat16, DEV)
    with pytest.raises(AssertionError):
        br.blockrank_attention_forward(None, q, k, v, None, 0.1)
    with pytest.raises(AssertionError):
        br.blockrank_attention_forward(None, q, k, v, torch.zeros(1, 1, 3, 8, device=DEV), 0.1)
    with pytest.raises(AssertionError):   # H != S // M
        br.blockrank_attention(q, k, v, torch.ones(1, 2, 8, dtype=torch.bool, device=DEV), 0.1)
    with pytest.raises(NotImplementedError):   # a dtype without kernels
        br.blockrank_attention(q.double(), k.double(), v.double(), lay.valid.to(DEV), 0.1)
    # gradients: bf16 attention has a backward; fp32 inputs and the fused score partials do not
    # (the reference's kernelised path refuses every backward, blockrank_triton_kernel_attention.py:759-761)
    with pytest.raises(NotImplementedError):
        br.blockrank_attention(q.float().requires_grad_(), k.float(), v.float(), lay.valid.to(DEV), 0.1)
    with pytest.raises(NotImplementedError):
        br.blockrank_attention(q.clone().requires_grad_(), k, v, lay.valid.to(DEV), 0.1, score_rows=8)
    assert br.blockrank_attention(q.clone().requires_grad_(), k, v, lay.valid.to(DEV), 0.1).requires_grad
    with pytest.raises(RuntimeError):
        br.blockrank_attention(q.cpu(), k.cpu(), v.cpu(), br.BlockMask(lay.valid.to(DEV)), 0.1)
    # head dim the kernels do not cover
    q3, k3, v3 = synthetic.random_qkv(lay, 4, 2, 96, torch.bfloat16, DEV)
    with pytest.raises(AssertionError):
        br.blockrank_attention(q3, k3, v3, lay.valid.to(DEV), 0.1)
