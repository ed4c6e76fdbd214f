"""Hugging Face attention-interface hooks for BlockRank attention on MI355X.

Mirrors the reference's plugin surface for this path:
  * ``register_blockrank_attention()``          (src/blockrank/blockrank_std_attention.py:652-665)
  * ``register_triton_blockrank_attention()``   (src/blockrank/blockrank_triton_kernel_attention.py:938-965)
  * the attention hook ``fwd(module, query, key, value, attention_mask, scaling, dropout=0.0, **kwargs)
    -> (attn_output (B, S, Nq, D), scores_or_None)`` (blockrank_std_attention.py:472-481, 648-650)
  * the mask hook that turns the collate's (B, M, H) block mask into what the attention hook receives
    as ``attention_mask`` (blockrank_std_attention.py:264-309).

Every implementation name the reference registers is routed to the one HIP path; there is no eager,
SDPA, flex or Triton code here and no fallback when the HIP library is absent.
"""
from __future__ import annotations

import os
import warnings
from typing import Optional

import torch

from . import _lib

# Names the reference registers (blockrank_std_attention.py:654-665).
STD_IMPL_NAMES = (
    "default_blockrank",
    "max-autotune_blockrank",
    "eager_blockrank",
    "flex_blockrank",
    "sdpa_blockrank",
    "sdpa_compiled_blockrank",
)
# blockrank_triton_kernel_attention.py:960-965
TRITON_IMPL_NAMES = ("triton_blockrank", "triton_blockrank_compiled")

_DTYPE_CODE = {torch.float32: _lib.BR_DTYPE_F32, torch.bfloat16: _lib.BR_DTYPE_BF16, torch.float16: _lib.BR_DTYPE_F16}
_HALF = (torch.bfloat16, torch.float16)      # the MFMA kernels' input types


def _env_flag(name: str) -> bool:
    return os.environ.get(name, "0") not in ("", "0", "false", "False")


def _stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class BlockMask:
    """What the mask hook hands to the attention hook: the (B, M, H) real-token mask plus the device
    plan built from it.

    It stands where the reference passes a (B, 1, M, H, H) additive tensor
    (blockrank_std_attention.py:293-309) and reports that shape, but holds B*M*H bytes instead of
    B*M*H*H values; ``dense()`` materialises the reference tensor for callers that want it.  Plans
    are built lazily per head layout and shared by every layer of a forward pass.
    """

    def __init__(self, valid: torch.Tensor, dtype: torch.dtype = torch.float32):
        assert valid.dim() == 3, "block attention mask must be (B, M, H)"
        if not valid.is_cuda:
            raise RuntimeError("blockrank_amd runs on a GPU only: the block attention mask must be a CUDA/HIP tensor")
        self.valid = valid.bool().contiguous()
        self.lengths = None
        self.packed = False
        self.left_padded = True
        self.total_tokens = None
        self.dtype = dtype
        self.B, self.M, self.H = valid.shape
        self._plans: dict[tuple[int, int], torch.Tensor] = {}

    @classmethod
    def from_lengths(cls, lengths: torch.Tensor, H: Optional[int] = None, packed: bool = False, left_padded: bool = True,
                     dtype: torch.dtype = torch.float32) -> "BlockMask":
        """From per-block real-token counts (B, M) instead of a padded mask.

        packed=False describes the reference's padded layout (every block in H slots, its tokens at the
        left or right end of them).  packed=True describes tensors with no padded slots at all: the
        tokens of all blocks of all sequences follow each other on one token axis, q/k/v are
        (1, heads, T, D) with T = lengths.sum(); H is then only an upper bound of the block lengths
        (default: the maximum rounded up to 16) and the coordinate system of score rows."""
        assert lengths.dim() == 2, "lengths must be (B, M)"
        if not lengths.is_cuda:
            raise RuntimeError("blockrank_amd runs on a GPU only: the block lengths must be a CUDA/HIP tensor")
        self = cls.__new__(cls)
        self.valid = None
        self.lengths = lengths.to(torch.int32).contiguous()
        self.packed = bool(packed)
        self.left_padded = bool(left_padded)
        host = None
        if H is None or packed:
            host = lengths.cpu()
        if H is None:
            H = (int(host.max()) + 15) // 16 * 16
        self.total_tokens = int(host.sum()) if packed else None
        self.dtype = dtype
        self.B, self.M = lengths.shape
        self.H = int(H)
        self._plans = {}
        return self

    def _valid_mask(self) -> torch.Tensor:
        if self.valid is None:
            j = torch.arange(self.H, device=self.lengths.device)[None, None, :]
            ln = self.lengths[:, :, None]
            self.valid = (j >= self.H - ln) if self.left_padded else (j < ln)
        return self.valid

    # -- what the reference's 5-D tensor would answer ------------------------------------------
    @property
    def shape(self):
        return torch.Size((self.B, 1, self.M, self.H, self.H))

    @property
    def device(self):
        return self.valid.device if self.valid is not None else self.lengths.device

    def dim(self) -> int:
        return 5

    def size(self, i: Optional[int] = None):
        return self.shape if i is None else self.shape[i]

    def to(self, *args, **kwargs):
        return self

    def dense(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """The reference's additive mask: 0 where key j of the block is real and j <= i, else
        0.7 * finfo(dtype).min (blockrank_std_attention.py:297-307)."""
        dtype = dtype or self.dtype
        B, M, H = self.B, self.M, self.H
        if self.packed:
            raise NotImplementedError("a packed layout has no padded (B, 1, M, H, H) mask tensor")
        valid = self._valid_mask()
        keep = valid.view(B, 1, M, 1, H) & torch.tril(torch.ones(H, H, dtype=torch.bool, device=valid.device))
        neg = 0.7 * torch.finfo(dtype).min
        return torch.where(keep, torch.zeros((), dtype=dtype, device=keep.device), torch.full((), neg, dtype=dtype, device=keep.device))

    @classmethod
    def from_dense(cls, mask5: torch.Tensor) -> "BlockMask":
        """Recover the block mask from a reference-style (B, 1, M, H, H) additive tensor: the last
        row of each H x H tile is zero exactly at the block's real keys."""
        assert mask5.dim() == 5, "Attention mask must be 5D for BlockRank attention"
        return cls(mask5[:, 0, :, -1, :] == 0, mask5.dtype)

    # -- device plan --------------------------------------------------------------------------
    def plan(self, Nq: int, Nkv: int) -> torch.Tensor:
        key = (Nq, Nkv)
        plan = self._plans.get(key)
        if plan is None:
            lib = _lib.load()
            n = lib.br_plan_ints(self.B, self.M, self.H, Nq, Nkv)
            assert n > 0, f"unsupported head layout: {Nq} query heads, {Nkv} kv heads"
            dev = self.device
            with torch.cuda.device(dev):
                plan = torch.empty(n, dtype=torch.int32, device=dev)
                if self.lengths is None:
                    _lib.check(lib.br_plan_build(self.valid.data_ptr(), self.B, self.M, self.H, Nq, Nkv, plan.data_ptr(), n,
                                                 _stream_ptr(dev)))
                elif self.packed:
                    _lib.check(lib.br_plan_build_packed(self.lengths.data_ptr(), self.B, self.M, self.H, Nq, Nkv,
                                                        plan.data_ptr(), n, _stream_ptr(dev)))
                else:
                    _lib.check(lib.br_plan_build_from_lengths(self.lengths.data_ptr(), int(self.left_padded), self.B, self.M,
                                                              self.H, Nq, Nkv, plan.data_ptr(), n, _stream_ptr(dev)))
            if _env_flag("BLOCKRANK_AMD_DEBUG"):
                # same role as the reference's _DEBUG left-padding check (blockrank_std_attention.py:146-148)
                assert int(plan[4].item()) == 0, "Attention mask is not one contiguous span of real tokens per block"
            self._plans[key] = plan
        return plan

    def plans_at_rest(self) -> bool:
        """Whether every plan built for this mask is ready for a launch (waits for the device).  A launch that did not
        run to its end leaves a plan's ticket counters counting; ``rearm_plans`` puts them back."""
        lib = _lib.load()
        for plan in self._plans.values():
            rc = lib.br_plan_check(plan.data_ptr(), _stream_ptr(self.device))
            if rc == _lib.BR_ERR_PLAN:
                return False
            _lib.check(rc)
        return True

    def rearm_plans(self) -> None:
        lib = _lib.load()
        with torch.cuda.device(self.device):
            for plan in self._plans.values():
                _lib.check(lib.br_plan_rearm(plan.data_ptr(), _stream_ptr(self.device)))

    def block_lengths(self) -> torch.Tensor:
        """(B, M) int32 number of real tokens per block."""
        return self.lengths if self.lengths is not None else self.valid.sum(-1, dtype=torch.int32)


def blockrank_attention_mask(
    batch_size=None,
    cache_position=None,
    kv_length=None,
    kv_offset=0,
    mask_function=None,
    attention_mask: Optional[torch.Tensor] = None,
    dtype: torch.dtype = torch.float32,
    **kwargs,
):
    """Mask hook (AttentionMaskInterface).  Accepts both calling conventions of the transformers
    library - the older positional ``cache_position`` one the reference is written against
    (blockrank_std_attention.py:264-273) and the newer keyword one (``q_length``, ``q_offset``, ...),
    and like the reference ignores everything except ``attention_mask`` (B, M, H) and ``dtype``.

    Returns a BlockMask.  With BLOCKRANK_AMD_DENSE_MASK=1 it returns the reference's dense
    (B, 1, M, H, H) tensor instead, which the attention hook also accepts."""
    assert attention_mask is not None, "attention_mask must be provided for BlockRank attention"
    assert attention_mask.dim() == 3, "BlockRank attention mask must be (B, M, H)"
    bm = BlockMask(attention_mask, dtype)
    if _env_flag("BLOCKRANK_AMD_DENSE_MASK"):
        return bm.dense()
    return bm


def _as_block_mask(attention_mask) -> BlockMask:
    assert attention_mask is not None, "BlockRank attention requires an attention mask"
    if isinstance(attention_mask, BlockMask):
        return attention_mask
    assert len(attention_mask.shape) == 5, "Attention mask must be 5D for BlockRank attention"
    cached = getattr(attention_mask, "_blockrank_block_mask", None)
    if cached is None:
        cached = BlockMask.from_dense(attention_mask)
        try:
            attention_mask._blockrank_block_mask = cached   # every layer of the forward reuses the plan
        except Exception:
            pass
    return cached


def _dense_last_dim(t: torch.Tensor, per16: int) -> torch.Tensor:
    """The kernels read 16-byte pieces along the head dim: make it dense and the strides/pointer
    16-byte multiples (a copy only if the caller's view is not already so)."""
    if t.stride(-1) != 1 or any(s % per16 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


class _AttentionWithGrad(torch.autograd.Function):
    """bf16 attention whose backward is the HIP kernel: the role of the reference's autograd-differentiated
    hooks (blockrank_std_attention.py:96-262, :472-650, as trainer.py:79-101 uses them).  The forward saves
    the log-sum-exp of every row; the backward rebuilds the probabilities from it."""

    @staticmethod
    def forward(ctx, query, key, value, bm, scaling):
        lib = _lib.load()
        Bt, Nq, S, D = query.shape
        Nkv = key.shape[1]
        M, H, B, packed = bm.M, bm.H, bm.B, bm.packed
        q, k, v = (_dense_last_dim(t.detach(), 8) for t in (query, key, value))
        dev = query.device
        with torch.cuda.device(dev):
            plan = bm.plan(Nq, Nkv)
            out = torch.empty((Bt, S, Nq, D), dtype=query.dtype, device=dev)
            lse = torch.empty((Bt, Nq, S), dtype=torch.float32, device=dev)
            ws_bytes = lib.br_prefill_workspace_bytes(B, Nq, Nkv, D)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
            _lib.check(lib.br_prefill_fwd_lse(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), plan.data_ptr(), B, Nq, Nkv, M, H, D,
                _lib.strides3(q, packed), _lib.strides3(k, packed), _lib.strides3(v, packed),
                _lib._I64x3(0 if packed else S * Nq * D, D, Nq * D), scaling, ws.data_ptr(), ws_bytes, lse.data_ptr(),
                _lib._I64x3(0 if packed else Nq * S, S, 1), _stream_ptr(dev)))
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.bm, ctx.scaling = bm, scaling
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        bm = ctx.bm
        lib = _lib.load()
        Bt, Nq, S, D = q.shape
        Nkv = k.shape[1]
        M, H, B, packed = bm.M, bm.H, bm.B, bm.packed
        g = _dense_last_dim(dout.transpose(1, 2), 8)                     # logical (B, Nq, S, D)
        dev = q.device
        with torch.cuda.device(dev):
            plan = bm.plan(Nq, Nkv)
            dq = torch.empty((Bt, S, Nq, D), dtype=q.dtype, device=dev)
            dk = torch.empty((Bt, S, Nkv, D), dtype=q.dtype, device=dev)
            dv = torch.empty((Bt, S, Nkv, D), dtype=q.dtype, device=dev)
            slots = Bt * S
            ws_bytes = lib.br_prefill_bwd_workspace_bytes(B, Nq, Nkv, H, D, slots)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            bs = 0 if packed else 1
            _lib.check(lib.br_prefill_bwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), g.data_ptr(), lse.data_ptr(), plan.data_ptr(),
                B, Nq, Nkv, M, H, D,
                _lib.strides3(q, packed), _lib.strides3(k, packed), _lib.strides3(v, packed),
                _lib._I64x3(bs * S * Nq * D, D, Nq * D), _lib.strides3(g, packed), _lib._I64x3(bs * Nq * S, S, 1),
                dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                _lib._I64x3(bs * S * Nq * D, D, Nq * D), _lib._I64x3(bs * S * Nkv * D, D, Nkv * D),
                _lib._I64x3(bs * S * Nkv * D, D, Nkv * D), ctx.scaling, slots, ws.data_ptr(), ws_bytes, _stream_ptr(dev)))
        return dq.transpose(1, 2), dk.transpose(1, 2), dv.transpose(1, 2), None, None


def blockrank_attention(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    block_mask,
    scaling: float,
    *,
    kernel_events=None,
    score_rows: int = 0,
    qk_fp8: bool = False,
    q_rope=None,
    rank_rows: Optional[torch.Tensor] = None,
    rank_scale: float = 1.0,
):
    """Block-sparse prefill attention.  query (B, Nq, S, D), key/value (B, Nkv, S, D) with any
    (batch, head, token) strides; block_mask a BlockMask, a (B, M, H) bool tensor, or the reference's
    (B, 1, M, H, H) additive tensor.  Returns (B, S, Nq, D) contiguous, rows of padded slots zero.

    Same result as sdpa_blockrank_attention_forward (blockrank_std_attention.py:503-650) on rows of
    real tokens.  kernel_events: optional pair of raw hipEvent_t handles recorded right before and
    after the main attention kernel (see blockrank_amd.profiling).

    score_rows > 0 (bf16, at least one document block): the same kernel pass also leaves the per-tile
    score partials of the query block's last score_rows positions, and the call returns
    (out, partials); ``doc_scores_from_partials`` turns them into per-document scores.

    qk_fp8 (bf16 inputs, head dim 128): Q K^T of the prefix and document blocks is computed in fp8 e4m3
    (K with one power-of-two scale per (sequence, kv head), every query row with its own), P V
    stays bf16; the query block's rows, from which the scores are read, are computed in bf16 - the
    reduced-precision variant for ranking (scores as accurate as the bf16 kernel's).

    q_rope=(cos, sin) (bf16, tables (B or 1, S, D) on query's token axis): ``query`` is the projection's output
    without its rotary position embedding, and the kernel rotates every Q row when it loads it; ``key`` must come
    rotated (``blockrank_amd.rope.rotate_k``).

    rank_rows (B, R) with score_rows > 0: indices 0..score_rows-1 into the last score_rows positions of the query
    block, known before the layer runs (the reference derives them from the labels, losses.py:43-48).  The
    per-document scores of those rows - ``doc_scores_from_partials`` with out_scale = rank_scale - are then reduced
    in the launch that merges the attention's split partials, and the call returns (out, partials, scores)."""
    if rank_rows is not None and score_rows <= 0:
        raise ValueError("rank_rows needs score_rows > 0")
    if isinstance(block_mask, torch.Tensor) and block_mask.dim() == 3:
        block_mask = BlockMask(block_mask, query.dtype)
    bm = _as_block_mask(block_mask)
    if not query.is_cuda:
        raise RuntimeError("blockrank_amd runs on a GPU only (got CPU tensors); it has no CPU fallback")
    Bt, Nq, S, D = query.shape
    Nkv = key.shape[1]
    M, H, B, packed = bm.M, bm.H, bm.B, bm.packed
    if packed:
        assert Bt == 1 and S == bm.total_tokens, "a packed layout takes (1, heads, T, D) tensors with T = sum of block lengths"
    else:
        assert H == S // M and M * H == S, f"Block size H={H} does not match MH // M = {S // M}"
        assert Bt == B, "attention mask batch size does not match query"
    assert key.shape == (Bt, Nkv, S, D) and value.shape == (Bt, Nkv, S, D), "key/value must be (B, Nkv, S, D)"
    if query.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"dtype {query.dtype} not supported by the HIP kernels (bfloat16, float16 and float32 are)")
    assert key.dtype == query.dtype and value.dtype == query.dtype, "query, key and value must share a dtype"
    if q_rope is not None and (query.dtype not in _HALF or qk_fp8):
        raise NotImplementedError("the rotary embedding inside the attention kernel takes 16-bit inputs and not the fp8 variant")
    if torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad):
        if query.dtype != torch.bfloat16 or qk_fp8 or score_rows > 0 or q_rope is not None:
            # same contract as the reference's kernelised path (blockrank_triton_kernel_attention.py:759-761)
            raise NotImplementedError("Backward pass not implemented yet (bfloat16 attention without fused score partials has one)")
        return _AttentionWithGrad.apply(query, key, value, bm, float(scaling))
    lib = _lib.load()
    per16 = 16 // query.element_size()
    q = _dense_last_dim(query, per16)
    k = _dense_last_dim(key, per16)
    v = _dense_last_dim(value, per16)
    dev = query.device
    with torch.cuda.device(dev):
        plan = bm.plan(Nq, Nkv)
        out = torch.empty((Bt, S, Nq, D), dtype=query.dtype, device=dev)
        ws_bytes = lib.br_prefill_workspace_bytes(B, Nq, Nkv, D)
        out_strides = _lib._I64x3(0 if packed else S * Nq * D, D, Nq * D)
        opt = _lib.BrPrefillOptions()
        opt.struct_bytes = _lib.ctypes.sizeof(opt)
        if kernel_events is not None:
            opt.ev_start, opt.ev_stop = kernel_events
        keep = []                                     # what the option structure points to, alive until the call returns
        if qk_fp8:
            if query.dtype != torch.bfloat16 or D != 128:
                raise NotImplementedError("the fp8 Q K^T variant takes bfloat16 inputs with head dim 128")
            opt.fp8_tokens = S if packed else B * S
            ws_bytes = lib.br_prefill_fp8qk_workspace_bytes(B, Nq, Nkv, D, M, opt.fp8_tokens)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        if q_rope is not None:
            cos, sin = q_rope
            assert cos.dim() == 3 and cos.shape == sin.shape and cos.shape[-2:] == (S, D) and cos.shape[0] in (1, Bt), \
                "cos / sin must be (B or 1, S, D) on the token axis of query"
            assert cos.dtype == query.dtype and sin.dtype == query.dtype and cos.is_cuda and sin.is_cuda
            if cos.stride(-1) != 1 or cos.stride(0) % 8 or cos.stride(1) % 8 or cos.stride() != sin.stride():
                cos, sin = cos.contiguous(), sin.contiguous()
            cs = (_lib.c_int64 * 2)(0 if cos.shape[0] == 1 else cos.stride(0), cos.stride(1))
            keep += [cos, sin, cs]
            opt.rope_cos, opt.rope_sin = cos.data_ptr(), sin.data_ptr()
            opt.rope_strides = _lib.ctypes.cast(cs, _lib.c_void_p)
        part = scores = None
        if score_rows > 0:
            opt.score_rows = score_rows
            opt.score_part_bytes = lib.br_score_partials_bytes(B, Nq, M, H, score_rows)
            part = torch.empty(max(opt.score_part_bytes // 4, 4), dtype=torch.float32, device=dev)
            opt.score_part = part.data_ptr()
        if rank_rows is not None:
            assert M >= 3, "per-document scores need at least one document block"
            assert rank_rows.shape[0] == B and rank_rows.dim() == 2, "rank_rows must be (B, R)"
            rr = rank_rows.to(device=dev, dtype=torch.int32).contiguous()
            scores = torch.empty((B, M - 2), dtype=torch.float32, device=dev)
            keep.append(rr)
            opt.rank_rows, opt.rank_R, opt.rank_scale, opt.rank_scores = rr.data_ptr(), rr.shape[1], float(rank_scale), scores.data_ptr()
        _lib.check(lib.br_prefill_fwd_ex(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), plan.data_ptr(), B, Nq, Nkv, M, H, D,
            _lib.strides3(q, packed), _lib.strides3(k, packed), _lib.strides3(v, packed), out_strides, float(scaling),
            _DTYPE_CODE[query.dtype], ws.data_ptr(), ws_bytes, _lib.ctypes.byref(opt), _stream_ptr(dev)))
        del keep
    if rank_rows is not None:
        return out, part, scores
    return (out, part) if score_rows > 0 else out


def fused_scores_supported(query: torch.Tensor, block_mask) -> bool:
    """Whether blockrank_attention(..., score_rows=R) can produce score partials for these inputs."""
    return query.dtype in _HALF and block_mask.M >= 3


def doc_scores_from_partials(partials: torch.Tensor, block_mask, rows: torch.Tensor, score_rows: int, num_heads: int,
                             num_kv_heads: int, temperature: float = 0.05, head_reduce: str = "mean",
                             row_reduce: str = "mean", return_probs: bool = False):
    """Per-document scores (B, M-2) from the partials of blockrank_attention(..., score_rows=...).
    rows: (B, R) indices 0..score_rows-1 into the last score_rows positions of the query block, as
    losses.py:43-48 computes them.  Same value as ``doc_scores`` for those rows."""
    bm = _as_block_mask(block_mask)
    assert bm.M >= 3, "per-document scores need at least one document block"
    assert head_reduce in ("mean", "sum") and row_reduce in ("mean", "sum")
    assert rows.dim() == 2 and rows.shape[0] == bm.B, "rows must be (B, R)"
    B, R = rows.shape
    out_scale = 1.0 / temperature
    if head_reduce == "mean":
        out_scale /= num_heads
    if row_reduce == "mean":
        out_scale /= R
    lib = _lib.load()
    dev = partials.device
    rows = rows.to(device=dev, dtype=torch.int32).contiguous()
    with torch.cuda.device(dev):
        plan = bm.plan(num_heads, num_kv_heads)
        scores = torch.empty((B, bm.M - 2), dtype=torch.float32, device=dev)
        probs = torch.empty((B, num_heads, R, bm.M - 2), dtype=torch.float32, device=dev) if return_probs else None
        _lib.check(lib.br_doc_scores_from_partials(
            partials.data_ptr(), plan.data_ptr(), rows.data_ptr(), R, score_rows, B, num_heads, bm.M, bm.H,
            float(out_scale), scores.data_ptr(), probs.data_ptr() if probs is not None else None, _stream_ptr(dev)))
    return (scores, probs) if return_probs else scores


_SPEC_ROWS: dict = {}
# rows tensors found equal to a guess: id -> (weak reference, tensor version, id of the guess).  Kept outside the
# handles: a serving loop asks every new handle with the same rows tensor, and the comparison costs a host
# synchronisation.
_CONFIRMED_ROWS: dict = {}


def _is_confirmed(rows: torch.Tensor, spec: torch.Tensor) -> bool:
    hit = _CONFIRMED_ROWS.get(id(rows))
    return hit is not None and hit[0]() is rows and hit[1] == rows._version and hit[2] == id(spec)


def _confirm(rows: torch.Tensor, spec: torch.Tensor) -> None:
    import weakref
    if len(_CONFIRMED_ROWS) > 256:
        for key in [k for k, v in _CONFIRMED_ROWS.items() if v[0]() is None]:
            del _CONFIRMED_ROWS[key]
    _CONFIRMED_ROWS[id(rows)] = (weakref.ref(rows), rows._version, id(spec))


def _speculated_rows(B: int, R: int, device) -> torch.Tensor:
    """(B, 2) indices {R-2, R-1} into the last R positions of the query block: the rows losses.py:43-48 arrives at
    whenever the completion is the single "[" token (evaluation: dataset.py:229-249 puts nothing after it), which the
    attention hook reduces the scores of before anybody has told it the rows.  One tensor per (B, R, device)."""
    key = (B, R, str(device))
    t = _SPEC_ROWS.get(key)
    if t is None:
        t = torch.tensor([[R - 2, R - 1]] * B, dtype=torch.int32, device=device)
        _SPEC_ROWS[key] = t
    return t


class LastBlockScores:
    """What the attention hook returns in place of the reference's s_last tensor (B, Nq, R, S)
    (blockrank_std_attention.py:639-645).  It keeps the layer's query/key tensors, the block mask and what the
    attention kernel already left (score partials, and the per-document scores of the rows it was told or guessed),
    so that ``compute_auxiliary_attention_loss`` of this package gets the scores without the logits ever being
    written.

    To everything else it behaves as the tensor: shape / dim / size / dtype / device, indexing, any method of
    torch.Tensor and any torch function (``torch.softmax(h, -1)``, ``h.take_along_dim(...)``, ``h[..., H:-H]``,
    ``h.float().cpu()``) work on it - the logits are computed when first asked for (``dense()``, fp32) and kept.  The
    reference's own ``compute_auxiliary_attention_loss`` (losses.py:37-78) therefore runs on it unchanged;
    ``take_along_dim`` over the row dimension, the first thing that function does, computes just the rows it asks for."""

    def __init__(self, query, key, block_mask: BlockMask, scaling: float, num_rows: int, scaled: bool = True, partials=None,
                 ranked=None, speculative: bool = False):
        self.query, self.key, self.block_mask = query, key, block_mask
        self.scaling, self.R, self.scaled = float(scaling), int(num_rows), scaled
        self.partials = partials if scaled else None    # per-tile (max, sum) pairs left by the attention kernel
        # (rows, temperature, scores): per-document scores the attention call already reduced for these rows;
        # speculative: nobody named the rows, they are the hook's guess (_speculated_rows) and have to be compared
        self.ranked = ranked if scaled else None
        self.speculative = bool(speculative) and self.ranked is not None
        self._dense = None
        _, Nq, _, D = query.shape
        self.shape = torch.Size((block_mask.B, Nq, self.R, block_mask.M * block_mask.H))
        self.device, self.dtype = query.device, torch.float32

    # -- the tensor it stands for -----------------------------------------------------------------
    def dim(self) -> int:
        return 4

    @property
    def ndim(self) -> int:
        return 4

    def size(self, i=None):
        return self.shape if i is None else self.shape[i]

    def __len__(self):
        return self.shape[0]

    def __getitem__(self, idx):
        return self.dense()[idx]

    def __getattr__(self, name):
        # (reached only for what the handle itself does not define: every other attribute or method of torch.Tensor)
        if name.startswith("__") or name in ("query", "key", "block_mask", "_dense"):
            raise AttributeError(name)
        return getattr(self.dense(), name)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        def unwrap(x):
            if isinstance(x, LastBlockScores):
                return x.dense()
            if isinstance(x, (list, tuple)):
                return type(x)(unwrap(y) for y in x)
            return x
        return func(*unwrap(args), **{k: unwrap(v) for k, v in (kwargs or {}).items()})

    def take_along_dim(self, indices, dim=None):
        """Tensor.take_along_dim; the pattern of losses.py:53 - (B, 1, R', 1) row indices over dim 2 - is served by
        computing those rows' logits alone."""
        if (dim in (2, -2) and torch.is_tensor(indices) and indices.dim() == 4 and indices.shape[1] == 1 and indices.shape[3] == 1
                and indices.shape[0] == self.shape[0] and indices.shape[2] <= 16 and self._dense is None and not self.needs_grad()):
            rows = indices[:, 0, :, 0]
            # negative indices count from the end, as in torch
            pos = torch.where(rows < 0, rows + self.R, rows) + (self.block_mask.H - self.R)
            return last_block_logits(self.query, self.key, self.block_mask, pos.to(torch.int32), self.scaling if self.scaled else 1.0,
                                     neg=0.7 * torch.finfo(self.query.dtype).min)
        return self.dense().take_along_dim(indices, dim)

    def _rows_default(self) -> torch.Tensor:
        H = self.block_mask.H
        return (torch.arange(H - self.R, H, dtype=torch.int32, device=self.device)[None]).expand(self.shape[0], self.R).contiguous()

    def needs_grad(self) -> bool:
        return torch.is_grad_enabled() and (self.query.requires_grad or self.key.requires_grad)

    def dense(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """(B, Nq, R, S) logits + additive mask, fp32 unless ``dtype`` is given.  Differentiable with respect
        to the layer's query and key when they require gradients (the auxiliary attention loss of
        trainer.py:79-101 trains through this tensor)."""
        if self._dense is None:
            scale = self.scaling if self.scaled else 1.0
            neg = 0.7 * torch.finfo(self.query.dtype).min
            if self.needs_grad():
                self._dense = _LastLogitsWithGrad.apply(self.query, self.key, self.block_mask, self._rows_default(), scale, neg)
            else:
                self._dense = last_block_logits(self.query, self.key, self.block_mask, self._rows_default(), scale, neg=neg)
        out = self._dense
        return out if dtype is None else out.to(dtype)

    # -- the scores -------------------------------------------------------------------------------
    def doc_scores(self, rows: torch.Tensor, temperature: float = 0.05, head_reduce: str = "mean", row_reduce: str = "mean",
                   return_probs: bool = False):
        """Per-document scores for ``rows`` (B, R') positions inside the query block (0..H-1)."""
        return doc_scores(self.query, self.key, self.block_mask, rows, self.scaling if self.scaled else 1.0,
                          temperature=temperature, head_reduce=head_reduce, row_reduce=row_reduce, return_probs=return_probs)

    def speculated_rows(self) -> Optional[torch.Tensor]:
        """The rows whose scores the attention call reduced on its own guess, or None."""
        return self.ranked[0] if self.speculative else None

    def confirm_rows(self, rows: torch.Tensor) -> None:
        """Tell the handle that ``rows`` was compared with ``speculated_rows()`` and found equal (the caller did
        the comparison together with a check of its own, see losses.compute_auxiliary_attention_loss)."""
        _confirm(rows, self.ranked[0])

    def _ranked_for(self, rows: torch.Tensor) -> bool:
        if self.ranked is None:
            return False
        if rows is self.ranked[0]:
            return True
        if not self.speculative:
            return False
        if _is_confirmed(rows, self.ranked[0]):
            return True
        # the guess has to be checked against what the caller's labels gave: one small comparison, one host
        # synchronisation (the reference's own bracket check, losses.py:48, is one too), once per rows tensor
        spec = self.ranked[0]
        same = rows.shape == spec.shape and bool((rows.to(device=spec.device, dtype=spec.dtype) == spec).all())
        if same:
            _confirm(rows, spec)
        return same

    def doc_scores_window(self, rows: torch.Tensor, temperature: float = 0.05, head_reduce: str = "mean",
                          row_reduce: str = "mean", return_probs: bool = False):
        """Same for ``rows`` (B, R') given as indices 0..R-1 into the handle's own R rows (the last R
        positions of the query block).  Uses the scores themselves when the attention call already reduced them for
        these very rows (it was told them, or guessed them and the guess holds), else the partials the attention
        kernel left, else the stand-alone score kernels."""
        if (self.ranked is not None and temperature == self.ranked[1] and head_reduce == "mean" and row_reduce == "mean"
                and not return_probs and self._ranked_for(rows)):
            return self.ranked[2]
        if self.partials is not None:
            return doc_scores_from_partials(self.partials, self.block_mask, rows, self.R, self.query.shape[1],
                                            self.key.shape[1], temperature=temperature, head_reduce=head_reduce,
                                            row_reduce=row_reduce, return_probs=return_probs)
        pos = (rows + (self.block_mask.H - self.R)).to(torch.int32)
        return self.doc_scores(pos, temperature=temperature, head_reduce=head_reduce, row_reduce=row_reduce,
                               return_probs=return_probs)


def _delegate_operator(name):
    def op(self, *args, **kwargs):
        return getattr(self.dense(), name)(*args, **kwargs)
    op.__name__ = name
    return op


# arithmetic and ordering operators are looked up on the type, not through __getattr__: give the handle the tensor's
# (== and != keep Python's identity semantics, so that a handle stays hashable)
for _name in ("add", "radd", "sub", "rsub", "mul", "rmul", "truediv", "rtruediv", "pow", "rpow", "matmul", "rmatmul", "neg", "abs",
              "lt", "le", "gt", "ge", "float", "iter"):
    setattr(LastBlockScores, f"__{_name}__", _delegate_operator(f"__{_name}__"))
del _name


def _score_args(query, key, block_mask, rows, query_block_only=False):
    if isinstance(block_mask, torch.Tensor) and block_mask.dim() == 3:
        block_mask = BlockMask(block_mask, query.dtype)
    bm = _as_block_mask(block_mask)
    if not query.is_cuda:
        raise RuntimeError("blockrank_amd runs on a GPU only (got CPU tensors); it has no CPU fallback")
    _, Nq, Sq, D = query.shape
    Nkv, S = key.shape[1], key.shape[2]
    B = bm.B
    if bm.packed:
        assert key.shape[0] == 1 and S == bm.total_tokens, "a packed layout takes (1, heads, T, D) tensors"
        assert not query_block_only and Sq == S, "a packed layout takes the query tensor over all T tokens"
    else:
        assert bm.M * bm.H == S, "attention mask does not match the sequence length"
        assert Sq == (bm.H if query_block_only else S), "query must cover the query block only" if query_block_only else \
            "query and key must cover the same tokens"
    if query.dtype not in _DTYPE_CODE:
        raise NotImplementedError(f"dtype {query.dtype} not supported by the HIP kernels (bfloat16, float16 and float32 are)")
    assert rows.dim() == 2 and rows.shape[0] == B, "rows must be (B, R)"
    per16 = 16 // query.element_size()
    q = _dense_last_dim(query, per16)
    k = _dense_last_dim(key, per16)
    rows = rows.to(device=query.device, dtype=torch.int32).contiguous()
    return bm, q, k, rows, (B, Nq, Nkv, S, D)


def doc_scores(query, key, block_mask, rows, scaling: float, temperature: float = 0.05, head_reduce: str = "mean",
               row_reduce: str = "mean", return_probs: bool = False, query_block_only: bool = False):
    """Fused per-document relevance: for every (head, chosen query-block row) a softmax of
    scaling*q.k over all real document tokens, summed per document, reduced over heads and rows and
    divided by the temperature.  Equals compute_auxiliary_attention_loss(s_last, ..., answer_ids=None,
    return_logits=True) (src/blockrank/losses.py:37-78) with rows = the bracket row and the one before.

    rows: (B, R) positions inside the query block (0..H-1), R <= 16.  Returns (B, M-2) fp32, and the
    (B, Nq, R, M-2) per-head probabilities too if return_probs.

    query_block_only: ``query`` holds the query block's H tokens only, (B, Nq, H, D) - for callers that
    never project the other tokens' queries (the kernels read no other query rows)."""
    bm, q, k, rows, (B, Nq, Nkv, S, D) = _score_args(query, key, block_mask, rows, query_block_only)
    R = rows.shape[1]
    assert bm.M >= 3, "per-document scores need at least one document block"
    assert head_reduce in ("mean", "sum") and row_reduce in ("mean", "sum")
    out_scale = 1.0 / temperature
    if head_reduce == "mean":
        out_scale /= Nq
    if row_reduce == "mean":
        out_scale /= R
    lib = _lib.load()
    dev = query.device
    with torch.cuda.device(dev):
        plan = bm.plan(Nq, Nkv)
        scores = torch.empty((B, bm.M - 2), dtype=torch.float32, device=dev)
        probs = torch.empty((B, Nq, R, bm.M - 2), dtype=torch.float32, device=dev) if return_probs else None
        ws_bytes = lib.br_doc_scores_workspace_bytes(B, Nq, bm.M, R)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        # the kernels address query rows as token (M-1)*H + position: shift the base accordingly
        q_ptr = q.data_ptr() - ((bm.M - 1) * bm.H * q.stride(2) * q.element_size() if query_block_only else 0)
        _lib.check(lib.br_doc_scores(
            q_ptr, k.data_ptr(), plan.data_ptr(), rows.data_ptr(), R, B, Nq, Nkv, bm.M, bm.H, D,
            _lib.strides3(q, bm.packed), _lib.strides3(k, bm.packed), float(scaling), float(out_scale), _DTYPE_CODE[query.dtype],
            scores.data_ptr(), probs.data_ptr() if probs is not None else None, ws.data_ptr(), ws_bytes, _stream_ptr(dev)))
    return (scores, probs) if return_probs else scores


def last_block_logits(query, key, block_mask, rows, scaling: float, neg: Optional[float] = None) -> torch.Tensor:
    """The reference's s_last: (B, Nq, R, S) fp32 = scaling*q.k + (0 | neg) for the given query-block
    rows against every key slot (blockrank_std_attention.py:233, 259, 639-645)."""
    bm, q, k, rows, (B, Nq, Nkv, S, D) = _score_args(query, key, block_mask, rows)
    R = rows.shape[1]
    if neg is None:
        neg = 0.7 * torch.finfo(query.dtype).min
    lib = _lib.load()
    dev = query.device
    MH = bm.M * bm.H
    with torch.cuda.device(dev):
        plan = bm.plan(Nq, Nkv)
        # (for a packed layout too the result is laid out over the M*H padded key slots, like the reference's)
        if R <= 16:
            out = torch.empty((B, Nq, R, MH), dtype=torch.float32, device=dev)
            chunks = [(rows, out)]
        else:
            # the kernel takes up to 16 rows per call (the reference's default num_last_queries); more rows go in
            # groups of 16, each into its own buffer, joined at the end
            chunks = [(rows[:, r0:r0 + 16].contiguous(), torch.empty((B, Nq, min(16, R - r0), MH), dtype=torch.float32, device=dev))
                      for r0 in range(0, R, 16)]
        for rws, dst in chunks:
            _lib.check(lib.br_last_block_logits(
                q.data_ptr(), k.data_ptr(), plan.data_ptr(), rws.data_ptr(), rws.shape[1], B, Nq, Nkv, bm.M, bm.H, D,
                _lib.strides3(q, bm.packed), _lib.strides3(k, bm.packed), float(scaling), float(neg), _DTYPE_CODE[query.dtype],
                dst.data_ptr(), _stream_ptr(dev)))
        if R > 16:
            out = torch.cat([d for _, d in chunks], dim=2)
    return out


class _LastLogitsWithGrad(torch.autograd.Function):
    """last_block_logits with a backward: s[b,n,r,k] = scaling * q[b,n,row_r] . k[b,n//G,k] + constant, so
    dq[row_r] = scaling * sum_k ds k and dk[k] = scaling * sum_{n in group, r} ds q[row_r] - two small products
    over the R score rows (br_last_block_logits_bwd; padded and packed layouts)."""

    @staticmethod
    def forward(ctx, query, key, bm, rows, scaling, neg):
        ctx.save_for_backward(query, key, rows)
        ctx.bm, ctx.scaling = bm, float(scaling)
        return last_block_logits(query.detach(), key.detach(), bm, rows, scaling, neg=neg)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, ds):
        query, key, rows = ctx.saved_tensors
        bm = ctx.bm
        _, q, k, rows, (B, Nq, Nkv, S, D) = _score_args(query.detach(), key.detach(), bm, rows)
        R = rows.shape[1]
        lib = _lib.load()
        dev = query.device
        ds = ds.float().contiguous()
        Bt = q.shape[0]
        with torch.cuda.device(dev):
            plan = bm.plan(Nq, Nkv)
            # gradients in the (B, S, heads, D) layout the projections' outputs have, returned as head-transposed views
            dq = torch.zeros((Bt, S, Nq, D), dtype=q.dtype, device=dev)
            dk = None
            for r0 in range(0, R, 16):                                  # the kernels take up to 16 rows per call
                rws = rows[:, r0:r0 + 16].contiguous()
                dsc = ds if R <= 16 else ds[:, :, r0:r0 + 16].contiguous()
                dki = torch.empty((Bt, S, Nkv, D), dtype=k.dtype, device=dev)
                dqi = dq if r0 == 0 else torch.zeros_like(dq)
                _lib.check(lib.br_last_block_logits_bwd(
                    dsc.data_ptr(), q.data_ptr(), k.data_ptr(), plan.data_ptr(), rws.data_ptr(), rws.shape[1], B, Nq, Nkv, bm.M, bm.H, D,
                    _lib.strides3(q, bm.packed), _lib.strides3(k, bm.packed), ctx.scaling, _DTYPE_CODE[q.dtype],
                    dqi.data_ptr(), _lib.strides3(dqi.transpose(1, 2), bm.packed), dki.data_ptr(), _lib.strides3(dki.transpose(1, 2), bm.packed),
                    _stream_ptr(dev)))
                if r0 > 0:
                    dq += dqi
                dk = dki if dk is None else dk + dki
        return dq.transpose(1, 2), dk.transpose(1, 2), None, None, None, None


def blockrank_attention_forward(
    module,
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    attention_mask,
    scaling: float,
    dropout: float = 0.0,
    **kwargs,
):
    """Attention hook (AttentionInterface).  Same contract as the reference's forwards
    (blockrank_std_attention.py:472-650, blockrank_triton_kernel_attention.py:798-884):

      query (B, Nq, S, D), key/value (B, Nkv, S, D), attention_mask from the mask hook (a BlockMask, or
      the reference's (B, 1, M, H, H) tensor); returns (attn_output (B, S, Nq, D), scores or None).

    Scores are returned when ``layers_to_return_scores`` contains ``module.layer_idx`` or, without
    that list, when ``return_last_block_attn_scores`` is true (:625-635), for the last
    ``num_last_queries`` (default 16) rows of the query block (:637-645).  They come back as a
    LastBlockScores handle (scaled logits, the eager/Triton convention); pass
    ``materialize_scores=True`` or set BLOCKRANK_AMD_DENSE_SCORES=1 for the fp32 tensor itself, and
    ``unscaled_scores=True`` for the literal SDPA function's unscaled variant (:537, :643).
    ``qk_fp8=True`` (or BLOCKRANK_AMD_QK_FP8=1) computes Q K^T in fp8 e4m3 (see blockrank_attention).
    ``score_rows_hint`` (B, R') int tensor with ``score_temperature`` (default 0.05): the rows (indices into the last
    ``num_last_queries`` positions) the caller is going to ask the handle's ``doc_scores_window`` for with that
    temperature and the default reductions; their scores are then reduced inside the attention call's second launch
    and the handle returns them when asked with that same tensor object.  Without a hint the hook guesses the last
    two positions (what losses.py:43-48 yields in evaluation) and the handle checks the guess against the rows it is
    asked for, falling back to the partials if it was wrong; ``speculate_score_rows=False`` or
    BLOCKRANK_AMD_NO_SPECULATION=1 switch the guess off.
    """
    assert attention_mask is not None, "BlockRank attention requires an attention mask"
    bm = _as_block_mask(attention_mask)
    B, Nq, S, D = query.shape
    if not bm.packed:
        assert bm.H == S // bm.M, f"Block size H={bm.H} does not match MH // M = {S // bm.M}"
    groups = getattr(module, "num_key_value_groups", None)
    if groups is not None:
        assert key.shape[1] * groups == Nq, "num_key_value_groups does not match the query/key head counts"
    if dropout > 0.0 and getattr(module, "training", False):
        # the reference's trainable hooks apply attention dropout in training (blockrank_std_attention.py:168-169, :551);
        # its kernelised hook ignores it with a warning (blockrank_triton_kernel_attention.py:844-846).  Ignoring it
        # silently changes what is trained, so refuse.
        raise NotImplementedError("attention dropout > 0 in training is not supported by the HIP attention (set attention_dropout=0)")

    layers = kwargs.get("layers_to_return_scores", None)
    if layers is not None:
        layer_idx = getattr(module, "layer_idx", None)
        want = layer_idx is not None and layer_idx in layers
    else:
        want = kwargs.get("return_last_block_attn_scores", False)
    want = want and bm.M > 1
    num_last = kwargs.get("num_last_queries", 16)
    R = num_last if bm.H >= num_last else bm.H
    scaled = not kwargs.get("unscaled_scores", False)
    # training (gradients wanted): the attention runs through its autograd function and the scores come back
    # as the dense, differentiable logits tensor the reference returns
    needs_grad = torch.is_grad_enabled() and (query.requires_grad or key.requires_grad or value.requires_grad)
    fuse = (want and scaled and not needs_grad and fused_scores_supported(query, bm)
            and not _env_flag("BLOCKRANK_AMD_SEPARATE_SCORES"))

    qk_fp8 = bool(kwargs.get("qk_fp8", False)) or _env_flag("BLOCKRANK_AMD_QK_FP8")
    # A query that came through rope.apply_rotary_pos_emb_fused is still unrotated and carries its cos / sin tables:
    # the attention kernel rotates the rows it loads.  Where something else reads the query as well (the scoring
    # layer's logits, the fp8 variant's quantiser, a backward pass), it is rotated here instead.
    deferred = getattr(query, "_blockrank_rope", None)
    q_rope = None
    if deferred is not None:
        if want or qk_fp8 or needs_grad or query.dtype not in _HALF:
            from .rope import rotate_q
            query = rotate_q(query, deferred.cos, deferred.sin)
        else:
            q_rope = (deferred.cos, deferred.sin)
    hint = kwargs.get("score_rows_hint", None) if fuse and bm.M >= 3 else None
    temperature = float(kwargs.get("score_temperature", 0.05))
    if hint is not None and not 1 <= hint.shape[-1] <= 16:
        hint = None
    # Nobody named the rows (the reference's callers do not: scripts/eval_attn.py:139): guess the ones losses.py:43-48
    # yields whenever the completion is the "[" token alone - the last two positions -, reduce their scores in the
    # attention call's second launch, and let the handle compare the guess with the rows it is later asked for.
    speculative = False
    if (hint is None and fuse and bm.M >= 3 and R >= 2 and kwargs.get("speculate_score_rows", True)
            and not _env_flag("BLOCKRANK_AMD_NO_SPECULATION")):
        hint = _speculated_rows(bm.B, R, query.device)
        speculative = True
    out = blockrank_attention(query, key, value, bm, scaling, kernel_events=kwargs.get("kernel_events", None),
                              score_rows=R if fuse else 0, qk_fp8=qk_fp8, q_rope=q_rope, rank_rows=hint,
                              rank_scale=1.0 / (temperature * Nq * hint.shape[-1]) if hint is not None else 1.0)
    partials = ranked = None
    if hint is not None:
        out, partials, scores = out
        ranked = (hint, temperature, scores)
    elif fuse:
        out, partials = out
    if not want:
        return out, None
    handle = LastBlockScores(query, key, bm, scaling, R, scaled=scaled, partials=partials, ranked=ranked, speculative=speculative)
    if needs_grad or kwargs.get("materialize_scores", False) or _env_flag("BLOCKRANK_AMD_DENSE_SCORES"):
        return out, handle.dense()
    return out, handle


def _register(names) -> None:
    try:
        from transformers import AttentionInterface, AttentionMaskInterface
    except ImportError as e:  # same failure mode as blockrank_triton_kernel_attention.py:951-955
        raise ImportError("Transformers is not available. Please install it with: pip install transformers") from e
    for name in names:
        AttentionInterface.register(name, blockrank_attention_forward)
        AttentionMaskInterface.register(name, blockrank_attention_mask)


def register_blockrank_attention() -> None:
    """Register the implementation names of blockrank_std_attention.py:652-665, all served by the
    HIP path."""
    _register(STD_IMPL_NAMES)


def register_triton_blockrank_attention() -> None:
    """Register the implementation names of blockrank_triton_kernel_attention.py:938-965, served by
    the HIP path (nothing here uses Triton)."""
    _register(TRITON_IMPL_NAMES)
