"""The opt-in resident path (BLOCKRANK_AMD_RESIDENT=1): sequences whose blocks are short enough for
LDS go to the resident kernel, which also computes the query block's rows against every block and
leaves their partials - and the score partials - to the same merge kernels as the streaming path.
Same oracle, same tolerances as the default path (2e-2 max-abs on bf16 outputs, 1e-3 relative on
scores with the same top-10); and the two paths must agree with each other."""
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import synthetic
from tests._util import assert_scores_close, max_abs_on_real_rows, oracle_attention, oracle_doc_scores, real_rows

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NRES = 3          # plan header word: number of resident items


@pytest.fixture(autouse=True)
def resident_on(monkeypatch):
    monkeypatch.setenv("BLOCKRANK_AMD_RESIDENT", "1")


def _run(lay, Nq, Nkv, D, seed=0, fused_sequences=None, scores=True):
    q, k, v = synthetic.random_qkv(lay, Nq, Nkv, D, torch.bfloat16, DEV, seed=seed)
    scale = D ** -0.5
    mask = br.BlockMask(lay.valid.to(DEV), torch.bfloat16)
    if fused_sequences is not None:
        nres = int(mask.plan(Nq, Nkv)[NRES].item())
        assert nres == fused_sequences * lay.M, f"{nres} resident items, expected {fused_sequences} fused sequences of {lay.M} blocks"
    R = min(16, lay.H)
    want_scores = scores and lay.M >= 3
    if want_scores:
        out, part = br.blockrank_attention(q, k, v, mask, scale, score_rows=R)
    else:
        out = br.blockrank_attention(q, k, v, mask, scale)
    torch.cuda.synchronize()
    err = max_abs_on_real_rows(out, oracle_attention(q, k, v, lay, scale), lay)
    assert err <= 2e-2, f"max abs error {err:.3e}"
    assert (out.cpu()[~real_rows(lay)] == 0).all(), "rows of padded slots must be zero"
    if want_scores:
        rows = torch.tensor([[R - 2, R - 1]] * lay.B, dtype=torch.int32, device=DEV)
        got = br.doc_scores_from_partials(part, mask, rows, R, Nq, Nkv)
        assert_scores_close(got, oracle_doc_scores(q, k, lay, scale))
    return out


def test_headline_shape_is_fused_and_matches_oracle_and_streaming_path(monkeypatch):
    lay = synthetic.uniform_layout(4, 64, 20, 160, 32)
    out = _run(lay, 32, 8, 128, fused_sequences=4)
    monkeypatch.setenv("BLOCKRANK_AMD_RESIDENT", "0")
    q, k, v = synthetic.random_qkv(lay, 32, 8, 128, torch.bfloat16, DEV, seed=0)
    ref = br.blockrank_attention(q, k, v, lay.valid.to(DEV), 128 ** -0.5)
    rows = real_rows(lay).to(DEV)
    diff = (out.float() - ref.float())[rows].abs().max().item()
    assert diff <= 2e-2, f"resident and streaming outputs differ by {diff:.3e}"


@pytest.mark.parametrize("G", [1, 2, 3, 4, 7, 8, 16])
def test_head_group_sizes(G):
    lay = synthetic.make_layout([[20, 70, 45, 130, 37]])
    _run(lay, 2 * G, 2, 128, seed=G, fused_sequences=1)


def test_head_dim_64_and_ragged_blocks():
    lay = synthetic.make_layout([[5, 17, 0, 64, 33, 9], [40, 1, 65, 31, 2, 70]])
    _run(lay, 8, 2, 64, seed=1, fused_sequences=None)
    _run(lay, 8, 2, 128, seed=2, fused_sequences=None)


def test_mixed_batch_one_long_document():
    # the second sequence has a 300-token document: it stays with the streaming kernel, the first is fused
    lay = synthetic.make_layout([[30, 100, 60, 192, 20], [30, 100, 300, 64, 20]])
    _run(lay, 8, 2, 128, seed=3, fused_sequences=1)


def test_query_block_of_two_tiles_and_too_long():
    # 8 query / 2 kv heads: 4 heads per workgroup, 32 tokens per query tile
    _run(synthetic.make_layout([[40, 90, 120, 33]]), 8, 2, 128, seed=4, fused_sequences=1)      # two query tiles, one ragged
    _run(synthetic.make_layout([[40, 90, 120, 64]]), 8, 2, 128, seed=5, fused_sequences=1)      # two full query tiles
    _run(synthetic.make_layout([[40, 90, 120, 65]]), 8, 2, 128, seed=6, fused_sequences=0)      # three: not fused


def test_empty_blocks_and_limits():
    _run(synthetic.make_layout([[0, 30, 0, 40, 5]]), 4, 1, 128, seed=7, fused_sequences=1)        # no prefix, an empty document
    _run(synthetic.make_layout([[12, 0, 0, 0, 3]]), 4, 1, 128, seed=8, fused_sequences=1)         # every document empty
    _run(synthetic.make_layout([[64, 192, 1, 192, 7]]), 4, 1, 128, seed=9, fused_sequences=1)     # exactly four tiles per block
    _run(synthetic.make_layout([[65, 192, 1, 192, 7]]), 4, 1, 128, seed=10, fused_sequences=0)    # five: not fused
    _run(synthetic.make_layout([[100, 50]]), 4, 2, 128, seed=11, fused_sequences=1, scores=False)  # prefix and query block only
    _run(synthetic.make_layout([[100]]), 4, 2, 128, seed=12, fused_sequences=0, scores=False)      # a single block: not fused


def test_packed_layout_and_many_documents():
    lay = synthetic.random_layout(2, 30, 70, 5, 64, 20, seed=2)            # 70 documents: 2 * M partial slots per sequence
    _run(lay, 8, 8, 128, seed=13, fused_sequences=2)
    from tests.test_gpu_packed import _pack
    q, k, v = synthetic.random_qkv(lay, 8, 2, 128, torch.bfloat16, DEV, seed=14)
    padded = br.blockrank_attention(q, k, v, lay.valid.to(DEV), 128 ** -0.5)
    lengths = torch.as_tensor(lay.lengths, dtype=torch.int32, device=DEV)
    mask = br.BlockMask.from_lengths(lengths, H=lay.H, packed=True, dtype=torch.bfloat16)
    assert int(mask.plan(8, 2)[NRES].item()) == 2 * lay.M
    out = br.blockrank_attention(_pack(q, lay.valid), _pack(k, lay.valid), _pack(v, lay.valid), mask, 128 ** -0.5)
    assert torch.equal(out[0], padded[real_rows(lay).to(DEV)]), "packed and padded layouts must give the same rows"
