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
