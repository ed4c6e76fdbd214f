"""Packed (unpadded) batches for the BlockRank path.

The reference's collate function (src/blockrank/dataset.py:191-276) pads every block of every
sequence to a common length H, so the model's dense layers and the attention run over B*M*H slots of
which a third to two thirds are padding in realistic batches.  The attention kernels here never read
padded slots, and with a packed plan (``BlockMask.from_lengths(..., packed=True)``) they do not need
them to exist: all real tokens follow each other on one token axis, ``input_ids`` is (1, T).

Two entry points:
  * ``pack_padded_batch``  turns a batch the reference's collate function produced into the packed form;
  * ``block_icr_collate_packed``  builds the packed form directly from the same per-example items the
    reference's collate function takes, with the same truncation, label and position-id rules.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .losses import bracket_rows


def pack_padded_batch(batch: Dict[str, torch.Tensor], num_last_queries: int = 16) -> Dict[str, torch.Tensor]:
    """batch: 'input_ids' (B, M*H), 'position_ids' (B, M*H), 'attention_mask' (B, M, H) and optionally
    'labels' (B, M*H), as block_icr_collate_fn returns them (dataset.py:269-276).  Returns
    'input_ids', 'position_ids' (and 'labels') of shape (1, T) holding the real tokens in order
    (sequence, block, position), 'block_lengths' (B, M) int32, 'H', and - when labels are given -
    'score_rows' (B, 2): the bracket row and the one before it as indices into the last
    ``num_last_queries`` positions of the query block (losses.py:43-48)."""
    mask = batch["attention_mask"].bool()
    B, M, H = mask.shape
    keep = mask.reshape(-1)
    out = {
        "input_ids": batch["input_ids"].reshape(-1)[keep][None],
        "position_ids": batch["position_ids"].reshape(-1)[keep][None],
        "block_lengths": mask.sum(-1, dtype=torch.int32),
        "H": H,
    }
    if "labels" in batch:
        labels = batch["labels"].reshape(B, M * H)
        out["labels"] = labels.reshape(-1)[keep][None]
        h1 = num_last_queries if H >= num_last_queries else H
        out["score_rows"] = bracket_rows(labels, h1)
    if "answer_ids" in batch:
        out["answer_ids"] = batch["answer_ids"]
    return out


def block_icr_collate_packed(batch: List[dict], pad_to_multiple_of: Optional[int] = 16, max_block_length: Optional[int] = None,
                             num_last_queries: int = 16) -> Dict[str, torch.Tensor]:
    """Counterpart of block_icr_collate_fn (dataset.py:191-276) that pads nothing.

    batch: items with 'input_ids' (1-D tensor: all blocks, then the completion), 'block_lengths'
    (1-D tensor: the M prompt blocks, then the completion) and optionally 'answer_ids'.  As in the
    reference the completion is merged into the last prompt block, blocks longer than
    max_block_length are truncated, labels are -100 except on the completion, and position ids are
    permutation invariant: 0.. inside the prefix, every document continues after the prefix, the last
    block starts at 16384 (dataset.py:252-257)."""
    B = len(batch)
    M = len(batch[0]["block_lengths"]) - 1
    ids, pos, lab, lens, rows = [], [], [], [], []
    merged = []
    for item in batch:
        bl = torch.as_tensor(item["block_lengths"]).clone().long()
        assert len(bl) == M + 1, "Number of blocks mismatch"
        last_prompt, completion = int(bl[-2]), int(bl[-1])
        bl = bl[:-1]
        bl[-1] += completion
        assert int(bl.sum()) == item["input_ids"].numel(), "Block lengths do not sum to input_ids length"
        merged.append((bl, last_prompt))
    longest = max(int(bl.max()) for bl, _ in merged)
    cap = min(longest, max_block_length or int(1e9))
    H = cap if pad_to_multiple_of is None else (cap + pad_to_multiple_of - 1) // pad_to_multiple_of * pad_to_multiple_of
    h1 = num_last_queries if H >= num_last_queries else H
    for item, (bl, last_prompt) in zip(batch, merged):
        start = torch.cumsum(torch.cat([torch.zeros(1, dtype=torch.long), bl]), 0)
        kept = torch.clamp(bl, max=H)                     # the reference truncates to the padded length
        prefix_len = int(kept[0])
        for m in range(M):
            n = int(kept[m])
            tok = item["input_ids"][start[m]: start[m] + n]
            ids.append(tok)
            base = 0 if m == 0 else (16384 if m == M - 1 else prefix_len)
            pos.append(torch.arange(n) + base)
            l = torch.full((n,), -100, dtype=torch.long)
            if m == M - 1:
                l[min(last_prompt, n):] = tok[min(last_prompt, n):]
            lab.append(l)
        lens.append(kept.to(torch.int32))
        # the completion starts at position last_prompt of the last block; in a block of H slots
        # whose tokens sit at the end that is slot H - n + last_prompt, i.e. this index into the last h1
        bracket = h1 - int(kept[-1]) + min(last_prompt, int(kept[-1]))
        # (a completion that truncation removed altogether has no bracket row: the reference fails the same way,
        # losses.py:46-48)
        assert 1 <= bracket <= h1 - 1 and last_prompt < int(kept[-1]), "Bracket token not found in last h1 positions."
        rows.append([bracket - 1, bracket])
    out = {
        "input_ids": torch.cat(ids)[None],
        "position_ids": torch.cat(pos)[None],
        "labels": torch.cat(lab)[None],
        "block_lengths": torch.stack(lens),
        "H": H,
        "score_rows": torch.tensor(rows, dtype=torch.long),
        "num_blocks": torch.tensor(M, dtype=torch.long),
    }
    if all("answer_ids" in item for item in batch):
        out["answer_ids"] = torch.nn.utils.rnn.pad_sequence([torch.as_tensor(item["answer_ids"]) for item in batch],
                                                            batch_first=True, padding_value=-1)
    return out
