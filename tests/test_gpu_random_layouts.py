"""Randomised (seeded) block layouts - empty, one-token, tile-edge and long blocks, every head grouping,
both head dims: attention output against the
oracle to 2e-2 on real rows, zeros on padded rows, scores to 1e-3 relative with the same top-10."""
import random

import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from tests._util import assert_scores_close, max_abs_on_real_rows, oracle_attention, oracle_doc_scores, real_rows

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cases(seed, n):
    rng = random.Random(seed)
    for it in range(n):
        B = rng.choice([1, 2, 3])
        M = rng.choice([2, 3, 4, 6, 9, 14])
        style = rng.choice(["short", "mixed", "long"])

        def doc_len():
            if style == "short":
                return rng.choice([0, 1, 7, 31, 32, 33, 63, 64, 65, 100, 128, 160, 192])
            if style == "mixed":
                return rng.choice([0, 5, 64, 150, 192, 193, 300])
            return rng.choice([10, 200, 400, 600])

        lens = [[rng.choice([0, 3, 32, 64, 65, 100])] + [doc_len() for _ in range(M - 2)] + [rng.choice([1, 5, 16, 31, 32, 33, 48, 64, 65, 90])]
                for _ in range(B)]
        yield it, lens, rng.choice([1, 2, 3, 4, 7, 8]), rng.choice([1, 2]), rng.choice([64, 128])


@pytest.mark.parametrize("seed", [11, 12])
def test_random_layouts_match_the_oracle(seed):
    for it, lens, G, Nkv, D in _cases(seed=seed, n=24):
        lay = synthetic.make_layout(lens)
        q, k, v = synthetic.random_qkv(lay, G * Nkv, Nkv, D, torch.bfloat16, DEV, seed=it)
        scale = D ** -0.5
        mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
        R = min(16, lay.H)
        tag = f"case {it}: lengths {lens}, {G} heads per kv head, {Nkv} kv heads, D={D}"
        if lay.M >= 3:
            out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R)
        else:
            out = br.blockrank_attention(q, k, v, mask, scale)
        err = max_abs_on_real_rows(out, oracle_attention(q, k, v, lay, scale), lay)
        assert err <= 2e-2, f"{tag}: max abs error {err:.3e}"
        assert (out.cpu()[~real_rows(lay)] == 0).all(), f"{tag}: rows of padded slots must be zero"
        if lay.M >= 3:
            rows = torch.tensor([[R - 2, R - 1]] * lay.B, dtype=torch.int32, device=DEV)
            got = br.doc_scores_from_partials(part, mask, rows, R, G * Nkv, Nkv)
            assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))


def test_larger_batches_fp16_and_scores_reduced_in_the_attention_call():
    """Batches large enough that the query block's key walk is cut into splits longer than the minimum (the split
    length follows the batch's work per workgroup), groups of 4, 7 and 8 heads, bf16 and fp16 alternating, every other
    case with the per-document scores reduced inside the attention call: same bounds as above."""
    rng = random.Random(99)
    for it in range(10):
        B = rng.choice([6, 8, 12])
        M = rng.choice([8, 12, 22])
        lens = [[rng.choice([16, 64, 100])] + [rng.choice([20, 64, 100, 160, 200]) for _ in range(M - 2)] + [rng.choice([16, 32, 48, 70])]
                for _ in range(B)]
        G, Nkv, D = rng.choice([(4, 2, 128), (7, 1, 128), (4, 4, 64), (8, 1, 128)])
        dtype = torch.bfloat16 if it % 2 else torch.float16
        lay = synthetic.make_layout(lens)
        q, k, v = synthetic.random_qkv(lay, G * Nkv, Nkv, D, dtype, DEV, seed=it)
        scale = D ** -0.5
        mask = br.BlockMask(lay.valid.to(DEV), dtype)
        R = min(16, lay.H)
        rows = torch.tensor([[R - 2, R - 1]] * lay.B, dtype=torch.int32, device=DEV)
        tag = f"case {it}: B={B}, M={M}, {G} heads per kv head, {Nkv} kv heads, D={D}, {dtype}"
        scores = None
        if it % 2:
            out, part, scores = br.blockrank_attention(q, k, v, mask, scale, score_rows=R, rank_rows=rows, rank_scale=1.0 / (0.05 * G * Nkv * 2))
        else:
            out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R)
        err = max_abs_on_real_rows(out, oracle_attention(q, k, v, lay, scale), lay)
        assert err <= (2e-2 if dtype == torch.bfloat16 else 4e-3), f"{tag}: max abs error {err:.3e}"
        assert (out.cpu()[~real_rows(lay)] == 0).all(), f"{tag}: rows of padded slots must be zero"
        got = br.doc_scores_from_partials(part, mask, rows, R, G * Nkv, Nkv)
        assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
        if scores is not None:
            assert torch.equal(scores, got), f"{tag}: scores reduced inside the call differ"
