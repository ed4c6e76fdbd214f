"""Rotary position embedding of Q and K in one HIP pass.

``apply_rotary_pos_emb`` has the signature and the result layout of the function of the same name in the
Hugging Face model files (transformers models/mistral/modeling_mistral.py, and the Llama / Qwen2 copies),
which every decoder layer of the models BlockRank ranks with calls on the projected Q and K right before
the attention interface.  There it is eight elementwise passes per layer (measured at the Mistral-7B
shape: 9 % of a ranking forward); here Q and K are read once and written once.  ``patch_rotary`` swaps
it into the module a model's attention class was defined in; ``TruncatedRanker`` then uses it as well.
"""
from __future__ import annotations

import sys

import torch

from . import _lib
from .attention import _DTYPE_CODE, _dense_last_dim, _stream_ptr

_I64x2 = _lib.ctypes.c_int64 * 2


class _RotaryWithGrad(torch.autograd.Function):
    """The rotation with its backward.  With x = (x1, x2) the two halves of the head dim, y1 = x1 c1 - x2 s1 and
    y2 = x2 c2 + x1 s2, so dx1 = g1 c1 + g2 s2 and dx2 = g2 c2 - g1 s1: the same kernel applied to the incoming
    gradient with the sine table's halves exchanged and negated (no assumption that the two halves of cos / sin
    are equal).  cos and sin are position tables, not parameters: they get no gradient."""

    @staticmethod
    def forward(ctx, q, k, cos, sin):
        ctx.save_for_backward(cos, sin)
        return _rotate(q, k, cos, sin)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, gq, gk):
        cos, sin = ctx.saved_tensors
        sin_t = -torch.roll(sin, sin.shape[-1] // 2, dims=-1)
        dq, dk = _rotate(gq, gk, cos, sin_t)
        return dq, dk, None, None


def apply_rotary_pos_emb(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, unsqueeze_dim: int = 1):
    """q (B, Nq, S, D), k (B, Nkv, S, D) (any strides with a dense last dim, e.g. the head-transposed views of
    the projections), cos / sin (B or 1, S, D).  Returns (q_embed, k_embed) with the same logical shapes, stored
    as (B, S, heads, D) - what the attention hook takes without a copy.  bf16 or fp32, D 64 or 128, CUDA tensors.
    Differentiable with respect to q and k (the backward is the same kernel on the gradients)."""
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad):
        if cos.requires_grad or sin.requires_grad:
            raise NotImplementedError("gradients with respect to the cos / sin tables are not implemented")
        return _RotaryWithGrad.apply(q, k, cos, sin)
    return _rotate(q, k, cos, sin, unsqueeze_dim)


class DeferredRotary:
    """What ``apply_rotary_pos_emb_fused`` leaves on the query tensor: the tables the attention kernel rotates its
    Q rows with."""

    def __init__(self, cos: torch.Tensor, sin: torch.Tensor):
        self.cos, self.sin = cos, sin


def rotate_k(k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """The rotary embedding of K alone (same kernel, no query heads): (B, Nkv, S, D) in, the same logical shape out,
    stored as (B, S, Nkv, D)."""
    return _rotate(None, k, cos, sin)[1]


def rotate_q(q: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """The rotary embedding of a query tensor alone (the kernel takes a key tensor along: its first head goes twice)."""
    return _rotate_impl(q, q[:, :1], cos, sin)[0]


def apply_rotary_pos_emb_fused(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, unsqueeze_dim: int = 1):
    """Signature of the model files' ``apply_rotary_pos_emb``; K is rotated here, Q is returned as it came with the
    tables attached (``q._blockrank_rope``): the BlockRank attention hook of this package hands them to the attention
    kernel, which rotates every Q row in registers when it loads it - two passes over the largest tensor of the layer
    less.  Only for inference through that hook (bf16): any other consumer of the returned q would see it unrotated, so
    with gradients enabled, or dtypes the fused path does not take, both tensors are rotated here as usual."""
    fused_ok = (q.dtype in (torch.bfloat16, torch.float16) and q.is_cuda and cos.dim() == 3
                and not (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad)))
    if not fused_ok:
        return apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim)
    assert unsqueeze_dim == 1, "only the (batch, heads, tokens, dim) convention of the decoder layers is supported"
    k_out = rotate_k(k, cos, sin)
    q._blockrank_rope = DeferredRotary(cos, sin)
    return q, k_out


apply_rotary_pos_emb_fused._blockrank_fused_q = True


def _rotate(q, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, unsqueeze_dim: int = 1):
    if q is None:                      # K alone
        return None, _rotate_impl(None, k, cos, sin)[1]
    return _rotate_impl(q, k, cos, sin, unsqueeze_dim)


def _rotate_impl(q, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, unsqueeze_dim: int = 1):
    k_only = q is None
    if k_only:
        q = k
    assert unsqueeze_dim == 1, "only the (batch, heads, tokens, dim) convention of the decoder layers is supported"
    assert q.is_cuda and k.is_cuda and cos.is_cuda and sin.is_cuda, "the rotary embedding kernel needs device tensors"
    assert q.dtype == k.dtype == cos.dtype == sin.dtype and q.dtype in _DTYPE_CODE, "q, k, cos and sin must share a dtype (bf16, fp16 or fp32)"
    B, Nq, S, D = q.shape
    Nkv = k.shape[1]
    assert k.shape == (B, Nkv, S, D) and cos.shape[-2:] == (S, D) and sin.shape == cos.shape and cos.dim() == 3
    assert cos.shape[0] in (1, B), "cos/sin must have the batch size of q or 1"
    lib = _lib.load()
    per16 = 16 // q.element_size()
    q = _dense_last_dim(q, per16)
    k = _dense_last_dim(k, per16)
    if cos.stride(-1) != 1 or cos.stride(0) % per16 or cos.stride(1) % per16 or cos.stride() != sin.stride():
        cos, sin = cos.contiguous(), sin.contiguous()
    with torch.cuda.device(q.device):
        k_out = torch.empty((B, S, Nkv, D), dtype=q.dtype, device=q.device)
        cs = _I64x2(0 if cos.shape[0] == 1 else cos.stride(0), cos.stride(1))
        if k_only:
            _lib.check(lib.br_rope_qk(None, k.data_ptr(), cos.data_ptr(), sin.data_ptr(), None, k_out.data_ptr(), B, 0, Nkv,
                                      S, D, None, _lib.strides3(k), cs, _DTYPE_CODE[q.dtype], _stream_ptr(q.device)))
            return None, k_out.transpose(1, 2)
        q_out = torch.empty((B, S, Nq, D), dtype=q.dtype, device=q.device)
        _lib.check(lib.br_rope_qk(q.data_ptr(), k.data_ptr(), cos.data_ptr(), sin.data_ptr(), q_out.data_ptr(), k_out.data_ptr(), B, Nq, Nkv,
                                  S, D, _lib.strides3(q), _lib.strides3(k), cs, _DTYPE_CODE[q.dtype], _stream_ptr(q.device)))
    return q_out.transpose(1, 2), k_out.transpose(1, 2)


def patch_rotary(model, fuse_q: bool = False) -> list[str]:
    """Replace ``apply_rotary_pos_emb`` in the module(s) that define the attention classes of ``model`` (a
    Hugging Face decoder).  Returns the names of the patched modules; ``unpatch_rotary`` restores them.
    ``fuse_q=True`` installs ``apply_rotary_pos_emb_fused`` instead: K is rotated by the kernel here, Q by the
    attention kernel: the model's attention implementation must be one of this package's BlockRank names (checked here;
    call ``unpatch_rotary`` before switching the model to another implementation)."""
    fn = apply_rotary_pos_emb_fused if fuse_q else apply_rotary_pos_emb
    if fuse_q:
        # the unrotated Q the fused function returns is only completed by this package's attention hook: under any
        # other attention implementation it would be consumed as it is, silently wrong
        from .attention import STD_IMPL_NAMES, TRITON_IMPL_NAMES
        impl = getattr(getattr(model, "config", None), "_attn_implementation", None)
        if impl not in STD_IMPL_NAMES + TRITON_IMPL_NAMES:
            raise ValueError(f"patch_rotary(fuse_q=True) needs one of the BlockRank attention implementations, the model uses {impl!r}; "
                             "set it first (and call unpatch_rotary before switching to another one)")
    done = []
    for m in model.modules():
        mod = sys.modules.get(type(m).__module__)
        if mod is None or mod.__name__ in done or not hasattr(mod, "apply_rotary_pos_emb") or not type(m).__name__.endswith("Attention"):
            continue
        if getattr(mod.apply_rotary_pos_emb, "__module__", "") != __name__:
            mod._blockrank_amd_saved_rotary = mod.apply_rotary_pos_emb
        mod.apply_rotary_pos_emb = fn
        done.append(mod.__name__)
    return done


def unpatch_rotary(model) -> None:
    for m in model.modules():
        mod = sys.modules.get(type(m).__module__)
        if mod is not None and hasattr(mod, "_blockrank_amd_saved_rotary"):
            mod.apply_rotary_pos_emb = mod._blockrank_amd_saved_rotary
            del mod._blockrank_amd_saved_rotary
