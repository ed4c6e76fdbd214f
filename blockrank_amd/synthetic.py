"""Synthetic ranking requests in the reference's block layout, for benchmarks and tests.

The layout rules follow block_icr_collate_fn (src/blockrank/dataset.py:191-276): every block is padded
on the left to a common H that is a multiple of 16; position ids restart at the prefix length for
every document and the query block is offset by 16384 (dataset.py:252-257); labels are -100 except on
the completion, which in the eval recipe is the single "[" token ending the query block.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Sequence

import numpy as np
import torch


@dataclass
class BlockLayout:
    lengths: np.ndarray          # (B, M) real tokens per block
    H: int
    valid: torch.Tensor          # (B, M, H) bool, left padded
    position_ids: torch.Tensor   # (B, M*H) int64
    labels: torch.Tensor         # (B, M*H) int64

    @property
    def B(self) -> int:
        return self.lengths.shape[0]

    @property
    def M(self) -> int:
        return self.lengths.shape[1]

    @property
    def S(self) -> int:
        return self.M * self.H

    @property
    def valid_tokens(self) -> int:
        return int(self.lengths.sum())

    def unmasked_pairs(self) -> int:
        """Number of (query, key) pairs the attention evaluates: p(p+1)/2 + sum_i [d_i p + d_i(d_i+1)/2]
        + q (p + sum d_i) + q(q+1)/2 per sequence."""
        total = 0
        for row in self.lengths:
            p, docs, q = int(row[0]), row[1:-1].astype(np.int64), int(row[-1])
            if len(row) == 1:
                total += p * (p + 1) // 2
                continue
            total += p * (p + 1) // 2 + int((docs * p + docs * (docs + 1) // 2).sum())
            total += q * (p + int(docs.sum())) + q * (q + 1) // 2
        return total


def make_layout(lengths: Sequence[Sequence[int]], pad_to_multiple_of: int = 16, H: int | None = None) -> BlockLayout:
    lengths = np.asarray(lengths, dtype=np.int64)
    B, M = lengths.shape
    if H is None:
        H = int(lengths.max())
        if pad_to_multiple_of:
            H = ((H + pad_to_multiple_of - 1) // pad_to_multiple_of) * pad_to_multiple_of
    j = torch.arange(H)[None, None, :]
    valid = j >= (H - torch.as_tensor(lengths)[:, :, None])
    pos = valid.cumsum(-1)
    if M > 2:
        pos[:, 1:-1] += pos[:, 0].max(dim=-1).values[:, None, None]
    if M > 1:
        pos[:, -1] += 16384
    pos = torch.clamp_min(pos - 1, 0)
    pos[~valid] = 0
    labels = torch.full((B, M * H), -100, dtype=torch.long)
    labels[:, -1] = 1
    return BlockLayout(lengths, H, valid, pos.view(B, M * H), labels)


def uniform_layout(B: int, prefix: int, docs: int, doc_len: int, query: int) -> BlockLayout:
    return make_layout([[prefix] + [doc_len] * docs + [query]] * B)


def random_layout(B: int, prefix: int, docs: int, lo: int, hi: int, query: int, seed: int = 0) -> BlockLayout:
    rng = np.random.default_rng(seed)
    rows = [[prefix] + rng.integers(lo, hi + 1, size=docs).tolist() + [query] for _ in range(B)]
    return make_layout(rows)


def lognormal_layout(B: int, prefix: int, docs: int, median: float, sigma: float, lo: int, hi: int, query: int,
                     seed: int = 0) -> BlockLayout:
    rng = np.random.default_rng(seed)
    rows = []
    for _ in range(B):
        d = np.clip(np.rint(rng.lognormal(math.log(median), sigma, size=docs)), lo, hi).astype(int).tolist()
        rows.append([prefix] + d + [query])
    return make_layout(rows)


def rope_cos_sin(position_ids: torch.Tensor, D: int, theta: float, dtype: torch.dtype, device) -> tuple[torch.Tensor, torch.Tensor]:
    inv = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float32, device=device) / D))
    f = position_ids.to(device=device, dtype=torch.float32)[:, :, None] * inv[None, None, :]
    emb = torch.cat([f, f], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x (B, heads, S, D); cos/sin (B, S, D); the half-rotation convention of Llama/Mistral/Qwen."""
    D = x.shape[-1]
    x1, x2 = x[..., : D // 2], x[..., D // 2:]
    rot = torch.cat([-x2, x1], dim=-1)
    return x * cos[:, None] + rot * sin[:, None]


def attention_layer_inputs(layout: BlockLayout, Nq: int, Nkv: int, D: int, hidden: int, dtype: torch.dtype, device,
                           rope_theta: float = 1e6, seed: int = 0):
    """Hidden states ~ N(0,1), projection weights ~ N(0, 0.02), RoPE with the layout's position ids:
    returns (q (B,Nq,S,D), k, v (B,Nkv,S,D)) as the attention hook of a Mistral/Qwen layer receives
    them, i.e. head-transposed views of (B, S, heads, D) projections."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    B, S = layout.B, layout.S
    x = torch.randn(B, S, hidden, generator=g, dtype=torch.float32).to(device=device, dtype=dtype)
    wq = (torch.randn(Nq * D, hidden, generator=g) * 0.02).to(device=device, dtype=dtype)
    wk = (torch.randn(Nkv * D, hidden, generator=g) * 0.02).to(device=device, dtype=dtype)
    wv = (torch.randn(Nkv * D, hidden, generator=g) * 0.02).to(device=device, dtype=dtype)
    q = (x @ wq.T).view(B, S, Nq, D).transpose(1, 2)
    k = (x @ wk.T).view(B, S, Nkv, D).transpose(1, 2)
    v = (x @ wv.T).view(B, S, Nkv, D).transpose(1, 2)
    cos, sin = rope_cos_sin(layout.position_ids, D, rope_theta, dtype, device)
    return apply_rope(q, cos, sin), apply_rope(k, cos, sin), v


def random_qkv(layout: BlockLayout, Nq: int, Nkv: int, D: int, dtype: torch.dtype, device, seed: int = 0, pad_fill: float | None = None):
    """Q, K, V ~ N(0,1) drawn directly in (B, heads, S, D).  pad_fill overwrites the padded slots
    (to show that nothing there is read)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    B, S = layout.B, layout.S
    q = torch.randn(B, Nq, S, D, generator=g, dtype=torch.float32)
    k = torch.randn(B, Nkv, S, D, generator=g, dtype=torch.float32)
    v = torch.randn(B, Nkv, S, D, generator=g, dtype=torch.float32)
    if pad_fill is not None:
        pad = ~layout.valid.view(B, 1, S, 1)
        q = torch.where(pad, torch.full_like(q, pad_fill), q)
        k = torch.where(pad, torch.full_like(k, pad_fill), k)
        v = torch.where(pad, torch.full_like(v, pad_fill), v)
    return q.to(device=device, dtype=dtype), k.to(device=device, dtype=dtype), v.to(device=device, dtype=dtype)
