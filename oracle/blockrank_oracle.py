"""CPU oracle for the BlockRank block-sparse prefill attention + attention-score ranking path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module: it exists so
that tests, the smoke check and the bench's CPU-baseline leg have an independent statement of what
the HIP kernels must compute.  It is a from-scratch restatement (numpy float64 for the brute-force
forms, torch CPU for the library-SDPA form) of the algorithm in the reference repository
nilesh2797/BlockRank; each function cites the reference lines it follows.

Notation: B batch, Nq query heads, Nkv key/value heads, G = Nq // Nkv, D head dim, M blocks,
H padded block length, S = M*H, ``valid`` = the (B, M, H) boolean block mask (True = real token).

How each function is pinned (see tests/test_oracle_*.py):
  additive_mask / allowed          two independent statements of the mask in the reference (the
                                   additive builder + segment composition, and the flex
                                   predicate); asserted equal on random masks.
  dense_attention                  textbook softmax(scale*QK^T + mask) V in float64 over the full
                                   S x S predicate; the anchor for everything else.
  sdpa_blockrank_forward           checked against dense_attention, against torch's own causal
                                   SDPA on the concatenated valid tokens (no mask tensor at all),
                                   and by invariants (V = 1, document permutation, GQA expansion,
                                   garbage in padding).
  dense_attention_backward         closed-form gradients; checked against central finite differences of
                                   dense_attention in float64 and against torch autograd through
                                   sdpa_blockrank_forward (library SDPA calls only); the log-sum-exp against
                                   the rows of dense logits.
  last_block_logits                closed form scale*q.k + {0 | NEG}; checked against the rows of
                                   dense logits.
  doc_scores_from_logits           closed forms: q = 0 gives len_i / sum(len); scores * tau sum to
                                   1; permutation equivariance; hand-computed 2-document case.
  topk_indices                     definition (stable descending order).
  rotary_embedding                 restates a third-party function the reference calls through the model
                                   forward (transformers >= 4.30 per the reference's requirements.txt:3;
                                   the installed 5.x has the same definition): pinned by the plane-rotation
                                   closed form (angle 0 = identity, pair norms preserved, angle then minus
                                   angle = identity, the vector (1, 0) goes to (cos, sin)) and against
                                   complex multiplication.
  rms_norm, silu_mul               restate third-party functions the reference calls through the model forward
                                   (same transformers files): pinned by closed forms - with unit weight and eps = 0
                                   every output row has mean square 1, scaling a row leaves its output unchanged,
                                   a constant row c gives sign(c) * weight; silu(0) = 0, silu(g) -> g for large g,
                                   silu(g) - silu(-g) = g, and against torch.nn.functional.silu / the published formula
                                   written with torch ops.
No golden vectors exist in the reference (it ships no tests); none of the functions above needed
an import of the reference to be pinned, so the reference was only read, never run.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------
# Mask (reference: src/blockrank/blockrank_std_attention.py:264-309, 344-399)
# --------------------------------------------------------------------------------------------

def neg_value(dtype: torch.dtype) -> float:
    """The finite "minus infinity" of the reference: 0.7 * finfo(dtype).min
    (blockrank_std_attention.py:306)."""
    return 0.7 * torch.finfo(dtype).min


def additive_mask(valid: torch.Tensor, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """(B, M, H) bool -> (B, 1, M, H, H) additive mask: 0 where key j is valid and j <= i, else NEG.

    Follows eager_blockrank_attention_mask, blockrank_std_attention.py:293-309.
    """
    B, M, H = valid.shape
    keep = valid.bool().view(B, 1, M, 1, H) & torch.tril(torch.ones(H, H, dtype=torch.bool))[None, None, None]
    out = torch.full((B, 1, M, H, H), neg_value(dtype), dtype=dtype)
    out[keep] = 0.0
    return out


def allowed(valid: np.ndarray, first_row: int = 0) -> np.ndarray:
    """(B, M, H) bool -> (B, S - first_row, S) bool, the element-wise predicate "query token may see key
    token" for the query tokens first_row .. S-1 (all of them by default; the score rows are the last few,
    and a long request's full S x S table would be gigabytes).

    Follows blockrank_mask_fn, blockrank_std_attention.py:344-399: both tokens valid, and
      block 0      : same block, causal
      middle block : key in block 0 (a different block), or same block and causal
      last block   : same block and causal, or key block earlier than the query block.
    """
    valid = np.asarray(valid, dtype=bool)
    B, M, H = valid.shape
    S = M * H
    idx = np.arange(S)
    blk, pos = idx // H, idx % H
    qb, kb = blk[first_row:, None], blk[None, :]
    qp, kp = pos[first_row:, None], pos[None, :]
    same = qb == kb
    causal = qp >= kp
    is0 = qb == 0
    last = qb == (M - 1)
    mid = ~is0 & ~last
    pat0 = is0 & same & causal
    patm = mid & (((kb == 0) & ~same) | (same & causal))
    patl = last & ((same & causal) | (~same & (kb < qb)))
    pattern = pat0 | patm | patl
    flat = valid.reshape(B, S)
    return flat[:, first_row:, None] & flat[:, None, :] & pattern[None]


def segment_masks(mask5: torch.Tensor) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Compose the three additive masks the reference's forward builds from the 5-D mask.

    Returns (m0 (B,1,H,H), m_mid (B,1,M-2,H,2H) or None, m_last (B,1,H,M*H) or None).
    Follows blockrank_std_attention.py:547 (block 0), :581-588 (documents), :607-614 (last block).
    """
    B, _, M, H, _ = mask5.shape
    m0 = mask5[:, :, 0]
    m_mid = None
    m_last = None
    if M > 2:
        key_ok0 = mask5[:, :, 0, -1, :]                       # (B,1,H): last row of block 0 = key validity
        first = key_ok0[:, :, None, None, :].expand(B, 1, M - 2, H, H)
        self_m = mask5[:, :, 1:M - 1]                         # (B,1,M-2,H,H)
        q_ok = self_m[:, :, :, -1, :, None]                   # validity of each query row of the doc
        first = torch.minimum(first, q_ok)
        m_mid = torch.cat([first, self_m], dim=-1)
    if M > 1:
        others = mask5[:, :, :M - 1, -1, :].reshape(B, 1, (M - 1) * H)
        others = others[:, :, None, :].expand(B, 1, H, (M - 1) * H)
        self_l = mask5[:, :, M - 1]
        others = torch.minimum(others, self_l[:, :, -1, :, None])
        m_last = torch.cat([others, self_l], dim=-1)
    return m0, m_mid, m_last


def allowed_from_segments(valid: np.ndarray) -> np.ndarray:
    """Same (B, S, S) predicate as ``allowed`` but derived from the additive masks and their
    segment composition (the other statement of the mask in the reference)."""
    v = torch.as_tensor(np.asarray(valid, dtype=bool))
    B, M, H = v.shape
    S = M * H
    m5 = additive_mask(v, torch.float32)
    m0, m_mid, m_last = segment_masks(m5)
    out = np.zeros((B, S, S), dtype=bool)
    out[:, :H, :H] = (m0[:, 0] == 0).numpy()
    if M > 1:
        if M > 2:
            mm = (m_mid[:, 0] == 0).numpy()                   # (B, M-2, H, 2H)
            for d in range(M - 2):
                r = slice((d + 1) * H, (d + 2) * H)
                out[:, r, :H] = mm[:, d, :, :H]
                out[:, r, r] = mm[:, d, :, H:]
        out[:, (M - 1) * H:, :] = (m_last[:, 0] == 0).numpy()
    return out


# --------------------------------------------------------------------------------------------
# Attention (reference: src/blockrank/blockrank_std_attention.py:472-650 and eager twin :96-262)
# --------------------------------------------------------------------------------------------

def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, Nkv, S, D) -> (B, Nkv*n_rep, S, D); query head n reads kv head n // n_rep.
    Same expansion the reference gets from transformers' repeat_kv (blockrank_std_attention.py:518)."""
    if n_rep == 1:
        return x
    B, Nkv, S, D = x.shape
    return x[:, :, None].expand(B, Nkv, n_rep, S, D).reshape(B, Nkv * n_rep, S, D)


def dense_attention(q, k, v, valid, scale: float) -> Tuple[np.ndarray, np.ndarray]:
    """Brute force in float64: softmax over allowed keys of scale*q.k, times V.

    q (B,Nq,S,D), k/v (B,Nkv,S,D) array-likes; valid (B,M,H) bool.  Returns
    (out (B,S,Nq,D) float64, logits (B,Nq,S,S) float64 scaled, not masked).  Rows whose query token
    is padding have no allowed key; their output is returned as NaN (the reference leaves an
    unspecified uniform average there and never consumes it).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, Nq, S, D = q.shape
    Nkv = k.shape[1]
    G = Nq // Nkv
    ok = allowed(valid)                                       # (B,S,S)
    out = np.full((B, S, Nq, D), np.nan)
    logits = np.empty((B, Nq, S, S))
    for b in range(B):
        for n in range(Nq):
            kk, vv = k[b, n // G], v[b, n // G]
            s = scale * (q[b, n] @ kk.T)
            logits[b, n] = s
            sm = np.where(ok[b], s, -np.inf)
            rows = ok[b].any(axis=1)
            mx = np.max(sm[rows], axis=1, keepdims=True)
            e = np.exp(sm[rows] - mx)
            p = e / e.sum(axis=1, keepdims=True)
            out[b, rows, n] = p @ vv
    return out, logits


def dense_attention_backward(q, k, v, dout, valid, scale: float) -> Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
    """Gradients of dense_attention in float64, in closed form, plus the log-sum-exp of every real row.

    The reference has no hand-written backward: its trainable path (the "default"/"eager"/"sdpa" hooks,
    blockrank_std_attention.py:96-262, :472-650, used by trainer.py:79-101) is differentiated by torch
    autograd, and its Triton path refuses (blockrank_triton_kernel_attention.py:759-761).  This is the
    derivative of softmax(scale*QK^T over allowed keys) V that autograd would produce:
        P = softmax(S),  dV = P^T dO,  dP = dO V^T,  dS = P * (dP - rowsum(dP * P)),
        dQ = scale * dS K,  dK = scale * dS^T Q,
    with dK and dV summed over the query heads that share a kv head (the transpose of repeat_kv).
    Rows of padded query tokens take part in nothing (their dout is ignored, their dq is zero).

    q (B,Nq,S,D), k/v (B,Nkv,S,D), dout (B,S,Nq,D); returns dq (B,Nq,S,D), dk, dv (B,Nkv,S,D) and
    lse (B,Nq,S) = log sum_j exp(scale*q.k_j) over allowed keys (NaN on padded rows).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    dout = np.asarray(dout, dtype=np.float64)
    B, Nq, S, D = q.shape
    Nkv = k.shape[1]
    G = Nq // Nkv
    ok = allowed(valid)
    dq = np.zeros_like(q)
    dk = np.zeros_like(k)
    dv = np.zeros_like(v)
    lse = np.full((B, Nq, S), np.nan)
    for b in range(B):
        rows = ok[b].any(axis=1)
        for n in range(Nq):
            kk, vv = k[b, n // G], v[b, n // G]
            s = np.where(ok[b][rows], scale * (q[b, n, rows] @ kk.T), -np.inf)
            mx = s.max(axis=1, keepdims=True)
            e = np.exp(s - mx)
            den = e.sum(axis=1, keepdims=True)
            p = e / den
            lse[b, n, rows] = (mx + np.log(den))[:, 0]
            do = dout[b, rows, n]
            dv[b, n // G] += p.T @ do
            dp = do @ vv.T
            ds = p * (dp - (dp * p).sum(axis=1, keepdims=True))
            dq[b, n, rows] = scale * (ds @ kk)
            dk[b, n // G] += scale * (ds.T @ q[b, n, rows])
    return dq, dk, dv, lse


def sdpa_blockrank_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask5: torch.Tensor,
    scaling: float,
    *,
    return_scores: bool = False,
    num_last_queries: int = 16,
    scaled_scores: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """The reference's three-call SDPA algorithm restated on torch CPU (also the timed CPU baseline).

    q (B,Nq,S,D), k/v (B,Nkv,S,D), mask5 (B,1,M,H,H) additive.  Returns (out (B,S,Nq,D) contiguous,
    s_last (B,Nq,R,S) or None).  Follows sdpa_blockrank_attention_forward,
    blockrank_std_attention.py:503-650: GQA expansion (:518-519), block view (:522-525), block 0
    (:544-554), documents over [K0 | K_self] (:565-596), last block over every key (:602-621), raw
    logits of the last R rows plus the additive mask (:639-645), final transpose copy (:648).

    ``scaled_scores``: the literal SDPA function leaves s_last unscaled (:537, :643) whereas the
    eager twin (:154, :233) and the Triton kernel (blockrank_triton_kernel_attention.py:499) scale it;
    True (the eager/Triton convention, which the published recipe trains and evaluates with) is
    the default here.
    """
    B, Nq, S, D = q.shape
    Nkv = k.shape[1]
    _, _, M, H, _ = mask5.shape
    assert H == S // M
    G = Nq // Nkv
    k = repeat_kv(k, G)
    v = repeat_kv(v, G)
    Q = q.reshape(B, Nq, M, H, D)
    K = k.reshape(B, Nq, M, H, D)
    V = v.reshape(B, Nq, M, H, D)
    m0, m_mid, m_last = segment_masks(mask5)
    out = torch.empty((B, Nq, M, H, D), dtype=q.dtype)
    K0, V0 = K[:, :, 0], V[:, :, 0]
    out[:, :, 0] = F.scaled_dot_product_attention(Q[:, :, 0], K0, V0, attn_mask=m0, scale=scaling)
    if M == 1:
        return out.view(B, Nq, S, D).transpose(1, 2).contiguous(), None
    if M > 2:
        K_mid = torch.cat([K0[:, :, None].expand(B, Nq, M - 2, H, D), K[:, :, 1:M - 1]], dim=-2)
        V_mid = torch.cat([V0[:, :, None].expand(B, Nq, M - 2, H, D), V[:, :, 1:M - 1]], dim=-2)
        out[:, :, 1:M - 1] = F.scaled_dot_product_attention(Q[:, :, 1:M - 1], K_mid, V_mid, attn_mask=m_mid, scale=scaling)
    K_all = K.reshape(B, Nq, S, D)
    V_all = V.reshape(B, Nq, S, D)
    Q_last = Q[:, :, M - 1]
    out[:, :, M - 1] = F.scaled_dot_product_attention(Q_last, K_all, V_all, attn_mask=m_last, scale=scaling)
    s_last = None
    if return_scores:
        R = num_last_queries if H >= num_last_queries else H
        qs = Q_last[:, :, -R:]
        if scaled_scores:
            qs = qs * scaling
        s_last = torch.matmul(qs, K_all.transpose(-2, -1)) + m_last[:, :, -R:]
    return out.view(B, Nq, S, D).transpose(1, 2).contiguous(), s_last


def last_block_logits(q, k, valid, scale: float, num_last_queries: int = 16, neg: float = None) -> np.ndarray:
    """Closed form of s_last in float64: scale*q.k + (0 if allowed else NEG) for the last R rows of
    the last block against all S keys.  (blockrank_std_attention.py:233,259 / :639-645.)"""
    valid = np.asarray(valid, dtype=bool)
    B, Nq, S, D = np.shape(q)
    _, M, H = valid.shape
    R = num_last_queries if H >= num_last_queries else H
    q = np.asarray(np.asarray(q)[:, :, S - R:], dtype=np.float64)      # only these rows are used
    k = np.asarray(k, dtype=np.float64)
    Nkv = k.shape[1]
    G = Nq // Nkv
    if neg is None:
        neg = neg_value(torch.float32)
    ok = allowed(valid, first_row=S - R)                      # (B,R,S)
    out = np.empty((B, Nq, R, S))
    for b in range(B):
        for n in range(Nq):
            s = scale * (q[b, n] @ k[b, n // G].T)
            out[b, n] = s + np.where(ok[b], 0.0, neg)
    return out


# --------------------------------------------------------------------------------------------
# Per-document score (reference: src/blockrank/losses.py:37-78) and top-k (scripts/eval_attn.py:150-151)
# --------------------------------------------------------------------------------------------

def bracket_rows(labels: np.ndarray, h1: int) -> np.ndarray:
    """(B, S) labels -> (B, 2) row indices into the last h1 rows: [bracket-1, bracket], where
    bracket = first position among the last h1 labels that is > -100 (losses.py:43-48)."""
    last = np.asarray(labels)[:, -h1:] > -100
    br = last.astype(np.int64).argmax(axis=1)
    rows = np.stack([br - 1, br], axis=1)
    assert (rows >= 0).all(), "Bracket token not found in last h1 positions."
    return rows


def doc_scores_from_logits(s_last, labels, valid, temperature: float = 0.05) -> np.ndarray:
    """(B,Nq,h1,S) logits -> (B, M-2) per-document logits, float64.

    Follows compute_auxiliary_attention_loss(answer_ids=None, return_logits=True), losses.py:37-78:
    pick rows {bracket-1, bracket} (:43-53); keep document columns H:S-H (:56); softmax jointly over
    all document tokens (:59); reshape to (docs, H) (:64); mean over heads and the two rows, sum over
    tokens (:68); divide by temperature (:74).
    """
    s = np.asarray(s_last, dtype=np.float64)
    valid = np.asarray(valid, dtype=bool)
    B, M, H = valid.shape
    _, N, h1, S = s.shape
    assert S == M * H
    rows = bracket_rows(labels, h1)
    out = np.empty((B, M - 2))
    for b in range(B):
        x = s[b][:, rows[b], H:S - H]                         # (N,2,(M-2)H)
        x = x - x.max(axis=-1, keepdims=True)
        e = np.exp(x)
        p = e / e.sum(axis=-1, keepdims=True)
        p = p.reshape(N, 2, M - 2, H)
        out[b] = p.mean(axis=(0, 1)).sum(axis=-1) / temperature
    return out


def doc_scores(q, k, valid, labels, scale: float, temperature: float = 0.05, num_last_queries: int = 16) -> np.ndarray:
    """End-to-end float64 oracle for the per-document score: logits of the last rows (scaled), then
    doc_scores_from_logits."""
    H = np.asarray(valid).shape[2]
    R = num_last_queries if H >= num_last_queries else H
    s = last_block_logits(q, k, valid, scale, R)
    return doc_scores_from_logits(s, labels, valid, temperature)


def topk_indices(scores: np.ndarray, k: int = 10) -> np.ndarray:
    """Indices of the k largest scores per row, descending, ties to the lower index
    (scripts/eval_attn.py:150-151 uses torch.topk(k=min(10, docs)))."""
    scores = np.asarray(scores)
    k = min(k, scores.shape[-1])
    return np.argsort(-scores, axis=-1, kind="stable")[..., :k]


# --------------------------------------------------------------------------------------------
# Synthetic layout helpers used by the tests (reference: src/blockrank/dataset.py:219-257)
# --------------------------------------------------------------------------------------------

def left_padded_valid(lengths: Sequence[Sequence[int]], H: int) -> np.ndarray:
    """Per-sequence block lengths -> (B, M, H) bool with each block's tokens right-aligned
    (left padding, the tokenizer side the reference's eval recipe uses)."""
    lengths = np.asarray(lengths)
    B, M = lengths.shape
    j = np.arange(H)[None, None, :]
    return j >= (H - lengths[:, :, None])


def eval_labels(valid: np.ndarray) -> np.ndarray:
    """Labels as the eval collate leaves them when the completion is the single "[" token: every
    position is -100 except the final token of the last block (dataset.py:229-249)."""
    B, M, H = np.asarray(valid).shape
    labels = np.full((B, M * H), -100, dtype=np.int64)
    labels[:, -1] = 1
    return labels


def quantize_fp8_e4m3(x: torch.Tensor, valid: torch.Tensor, per_row: bool = False) -> torch.Tensor:
    """Quantisation to fp8 e4m3 and back, as the fp8 Q K^T variant defines it (no reference counterpart; the
    Qwen2.5-7B-shaped benchmark configuration).  One power-of-two scale per group, 2^(floor(log2(max |x|)) - 7),
    which puts the group's largest magnitude into [128, 256) of e4m3's range (largest value 448); the group is the
    sequence's real tokens of one head (per_row=False: how K is quantised) or one token of one head
    (per_row=True: how the query rows are).  x / scale is rounded to the nearest e4m3 value (torch.float8_e4m3fn,
    round to nearest even, the same format the gfx950 conversion instruction produces) and returned dequantised,
    in float32.  A power-of-two scale makes the division exact: 16-bit inputs land on exact ties of the e4m3 grid
    often (one element in a thousand), and an inexact scale would break them differently from one implementation
    to the next.  A group whose maximum is below 2^-119 counts as zero.
    x (B, heads, S, D); valid (B, M, H) with M*H = S.  Pinned by: values with at most four significant bits
    within 2^9 of the group's maximum survive unchanged; the round trip error is at most 2^-4 relative for normal
    values; multiplying a group by a power of two multiplies its result by the same."""
    B, Hh, S, D = x.shape
    keep = valid.reshape(B, 1, S, 1).to(x.device)
    xf = x.float()
    amax = torch.where(keep, xf.abs(), torch.zeros((), dtype=torch.float32)).amax(dim=(3,) if per_row else (2, 3), keepdim=True)
    amax = amax.clamp(max=3.0e38).contiguous()
    ebits = amax.view(torch.int32) & 0x7F800000
    ok = ebits >= (8 << 23)
    sbits = torch.where(ok, ebits - (7 << 23), torch.full_like(ebits, 127 << 23))
    scale = torch.where(ok, sbits.view(torch.float32), torch.zeros_like(amax))
    inv = torch.where(ok, ((254 << 23) - sbits).view(torch.float32), torch.zeros_like(amax))
    q = (xf * inv).to(torch.float8_e4m3fn).float()
    return torch.where(keep, q * scale, torch.zeros((), dtype=torch.float32))


# --------------------------------------------------------------------------------------------
# the step in front of attention: rotary position embedding
# --------------------------------------------------------------------------------------------

def rotary_embedding(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x (B, N, S, D); cos, sin (B or 1, S, D).  out = x * cos + rotate_half(x) * sin with
    rotate_half(x) = concat(-x[..., D/2:], x[..., :D/2]) - the published definition in transformers
    models/mistral/modeling_mistral.py (rotate_half, apply_rotary_pos_emb; identical in the Llama and Qwen2
    files), which the reference applies through the Hugging Face model forward (scripts/eval_attn.py:139-151).
    float64."""
    x = np.asarray(x, dtype=np.float64)
    c = np.asarray(cos, dtype=np.float64)[:, None]
    s_ = np.asarray(sin, dtype=np.float64)[:, None]
    h = x.shape[-1] // 2
    rot = np.concatenate([-x[..., h:], x[..., :h]], axis=-1)
    return x * c + rot * s_


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """weight * x / sqrt(mean(x^2, -1) + eps) in float64: the RMSNorm of the Hugging Face decoder classes
    (transformers models/mistral/modeling_mistral.py, MistralRMSNorm.forward; the same class in the Llama and
    Qwen2 files), which the reference reaches through the model forward of scripts/eval_attn.py:139-151."""
    x = np.asarray(x, dtype=np.float64)
    return np.asarray(weight, dtype=np.float64) * x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """silu(gate) * up with silu(g) = g / (1 + exp(-g)) in float64: the gated product of MistralMLP.forward
    (same model files)."""
    g = np.asarray(gate, dtype=np.float64)
    return g / (1.0 + np.exp(-g)) * np.asarray(up, dtype=np.float64)
