"""The packed collate function against a padded batch built by the reference's rules
(src/blockrank/dataset.py:191-276: left padding to a multiple of 16, completion merged into the last
block, labels only on the completion, permutation-invariant position ids)."""
import torch

from blockrank_amd.collate import block_icr_collate_packed, pack_padded_batch


def _items(seed=0, B=3, M=5):
    g = torch.Generator().manual_seed(seed)
    items = []
    for _ in range(B):
        bl = torch.randint(3, 40, (M,), generator=g)
        comp = torch.randint(2, 6, (1,), generator=g)
        lens = torch.cat([bl, comp])
        items.append(dict(input_ids=torch.randint(5, 500, (int(lens.sum()),), generator=g), block_lengths=lens,
                          answer_ids=torch.randint(0, M - 2, (2,), generator=g)))
    return items


def _padded_by_reference_rules(items, pad_id=0, multiple=16, max_block_length=None):
    B, M = len(items), len(items[0]["block_lengths"]) - 1
    merged = []
    for it in items:
        bl = it["block_lengths"].clone()
        last_prompt = int(bl[-2])
        bl = bl[:-1]
        bl[-1] += it["block_lengths"][-1]
        merged.append((bl, last_prompt))
    H = min(max(int(bl.max()) for bl, _ in merged), max_block_length or 10 ** 9)          # dataset.py:205-208
    H = (H + multiple - 1) // multiple * multiple                                          # :210-211
    ids = torch.full((B, M, H), pad_id, dtype=torch.long)
    for b, (it, (bl, _)) in enumerate(zip(items, merged)):
        ptr = torch.cumsum(torch.cat([torch.zeros(1, dtype=torch.long), bl]), 0)
        for m in range(M):
            tok = it["input_ids"][ptr[m]:ptr[m + 1]][:H]                                   # :216 (truncation)
            ids[b, m, H - len(tok):] = tok                                                 # left padding (:219-226)
    mask = ids != pad_id
    labels = ids.clone()
    labels[~mask] = -100
    labels[:, :-1] = -100                                                                  # :231
    for b, (bl, last_prompt) in enumerate(merged):
        adj = last_prompt + (H - min(int(bl[-1]), H))                                      # :238-241
        labels[b, -1, :adj] = -100                                                         # :246-249
    pos = mask.cumsum(-1)                                                                  # :253
    pos[:, 1:-1] += pos[:, 0].max(dim=-1).values[:, None, None]
    pos[:, -1] += 16384
    pos = torch.clamp_min(pos - 1, 0)
    pos[~mask] = 0
    return dict(input_ids=ids.view(B, -1), position_ids=pos.view(B, -1), attention_mask=mask, labels=labels.view(B, -1))


def test_packed_collate_matches_padded_rules():
    for seed, cap in [(0, None), (1, 32), (2, None)]:
        items = _items(seed)
        padded = _padded_by_reference_rules([dict(x) for x in items], max_block_length=cap)
        want = pack_padded_batch(padded)
        got = block_icr_collate_packed([dict(x) for x in items], max_block_length=cap)
        assert got["H"] == want["H"]
        for key in ("input_ids", "position_ids", "labels", "block_lengths", "score_rows"):
            assert torch.equal(got[key].long(), want[key].long()), key
        assert got["answer_ids"].shape == (len(items), 2)
        assert got["input_ids"].shape[1] == int(got["block_lengths"].sum())


def test_completion_removed_by_truncation_is_refused():
    """A last block so long that truncation to H cuts the completion off has no bracket token left: the reference's
    score routine fails on such a batch (losses.py:46-48), and so does the packed collate function."""
    import pytest
    items = _items(seed=3, B=2, M=4)
    long = dict(items[0])
    lens = long["block_lengths"].clone()
    lens[-2] = 40                                    # last prompt block alone reaches the cap
    long["block_lengths"] = lens
    long["input_ids"] = torch.randint(5, 500, (int(lens.sum()),))
    with pytest.raises(AssertionError, match="Bracket token not found"):
        block_icr_collate_packed([long, dict(items[1])], max_block_length=32)
