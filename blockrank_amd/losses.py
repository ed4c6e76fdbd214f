"""Per-document relevance scores from the query block's attention (the reference's layer-score API).

Drop-in for src/blockrank/losses.py::compute_auxiliary_attention_loss: same name, arguments and
return values.  When ``attention_scores`` is the LastBlockScores handle this package's attention hook
returns, the scores come from the fused HIP kernel; a plain (B, N, h1, M*H) tensor (for instance from
``LastBlockScores.dense()`` or from the reference's own attention) is reduced with the same formula in
torch.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from .attention import LastBlockScores


def bracket_rows(labels: torch.Tensor, h1: int, guess: torch.Tensor | None = None, return_match: bool = False):
    """(B, S) labels -> (B, 2) indices into the last h1 positions: the first label > -100 (the "["
    token) and the position before it (losses.py:43-48).  With ``guess`` (B, 2) and ``return_match`` also whether the
    rows equal it, found out in the same host synchronisation as the reference's bracket check."""
    last = labels[:, -h1:] > -100
    br = last.int().argmax(dim=-1)[:, None]
    rows = torch.hstack([br - 1, br])
    if guess is None or not return_match:
        assert torch.all(rows >= 0), "Bracket token not found in last h1 positions."
        return (rows, False) if return_match else rows
    same = (rows == guess.to(rows.device)).all() if rows.shape == guess.shape else torch.zeros((), dtype=torch.bool, device=rows.device)
    ok, match = torch.stack([torch.all(rows >= 0), same]).tolist()
    assert ok, "Bracket token not found in last h1 positions."
    return rows, bool(match)


def _infonce(logits: torch.Tensor, answer_ids: torch.Tensor, return_logits: bool):
    # losses.py:80-93; forward values only - the HIP path has no backward
    B, num_docs = logits.shape
    pos_mask = torch.zeros(B, num_docs + 1, dtype=torch.bool, device=logits.device)
    safe = torch.where(answer_ids >= 0, answer_ids, num_docs)
    pos_mask.scatter_(1, safe, True)
    pos_mask = pos_mask[:, :-1]
    pos_lse = torch.logsumexp(logits.masked_fill(~pos_mask, float("-inf")), dim=1)
    all_lse = torch.logsumexp(logits, dim=1)
    loss = -(pos_lse - all_lse).mean()
    accuracy = pos_mask.gather(1, logits.argmax(dim=1, keepdim=True)).float().mean()
    return (loss, accuracy, logits) if return_logits else (loss, accuracy)


def compute_auxiliary_attention_loss(
    attention_scores,
    labels: torch.Tensor,
    attention_mask: torch.Tensor,
    answer_ids: torch.Tensor | None = None,
    temperature: float = 0.05,
    return_logits=False,
    rows: torch.Tensor | None = None,
):
    """(B, M-2) per-document logits (and, with ``answer_ids``, the InfoNCE loss and accuracy).

    attention_scores: LastBlockScores handle or (B, N, h1, M*H) tensor; labels (B, M*H) with -100 on
    everything but the completion; attention_mask (B, M, H).  Follows losses.py:37-78: rows =
    {bracket-1, bracket}; softmax over all document tokens jointly; sum per document; mean over heads
    and the two rows; divide by temperature.  ``rows``: the result of ``bracket_rows(labels, h1)`` if the caller
    already has it (the tensor given to the model call as ``score_rows_hint``: the handle then holds the scores).
    """
    B, M, H = attention_mask.shape
    _, N, h1, MH = attention_scores.shape
    assert MH == M * H, "Attention scores last dimension must match M*H"
    if rows is None:
        guess = attention_scores.speculated_rows() if isinstance(attention_scores, LastBlockScores) else None
        rows, match = bracket_rows(labels, h1, guess, return_match=True)     # (B, 2) in [0, h1)
        if match:
            attention_scores.confirm_rows(rows)              # the attention call's own guess holds: its scores are these rows'
    if isinstance(attention_scores, LastBlockScores) and attention_scores.needs_grad():
        attention_scores = attention_scores.dense()          # training: the differentiable logits tensor
    if isinstance(attention_scores, LastBlockScores):
        logits = attention_scores.doc_scores_window(rows, temperature=temperature)
    else:
        x = attention_scores.take_along_dim(rows[:, None, :, None], dim=2)[..., H:-H]
        p = F.softmax(x, dim=-1).reshape(B, N, -1, M - 2, H)
        logits = p.mean(dim=(1, 2)).sum(dim=-1) / temperature
    if answer_ids is None:
        assert return_logits, "If answer_ids is None, return_logits must be True."
        return logits
    return _infonce(logits, answer_ids, return_logits)


def rank_documents(logits: torch.Tensor, k: int = 10) -> torch.Tensor:
    """Top-k document indices per sequence, as scripts/eval_attn.py:150-151 takes them."""
    return torch.topk(logits, k=min(k, logits.shape[-1]), dim=-1).indices
