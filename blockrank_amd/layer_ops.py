"""RMSNorm and the SiLU-gated product of a decoder layer, each in one HIP pass.

The Hugging Face model classes the reference's models are instances of (transformers
models/mistral/modeling_mistral.py: ``MistralRMSNorm.forward`` and ``MistralMLP.forward``; the same classes in the
Llama and Qwen2 model files) express them as eight and two elementwise passes over the activations; the
ranking forward of scripts/eval_attn.py:139-151 runs them in every decoder layer (measured at the Mistral-7B
shape: 17 % of the GPU time of a forward pass).  ``patch_layer_ops(model)`` gives the model's norm and MLP
modules a forward that calls the kernels; with gradients enabled, or on tensors the kernels do not take, the
module's own forward runs as before.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import _lib
from .attention import _DTYPE_CODE as _ALL_DTYPES, _stream_ptr

# the norm / gate kernels are built for fp32 and bf16
_DTYPE_CODE = {t: c for t, c in _ALL_DTYPES.items() if t in (torch.float32, torch.bfloat16)}


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """weight * (x * rsqrt(mean(x^2, -1) + eps)) for x (..., hidden); fp32 arithmetic, the model file's rounding."""
    assert x.is_cuda and x.dtype in _DTYPE_CODE and weight.dtype == x.dtype, "rms_norm takes bf16 or fp32 device tensors of one dtype"
    hidden = x.shape[-1]
    assert weight.shape == (hidden,), "weight must have the size of the last dim"
    per16 = 16 // x.element_size()
    x2 = x.reshape(-1, hidden)
    if x2.stride(-1) != 1 or x2.stride(0) % per16 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    w = weight if weight.is_contiguous() and weight.data_ptr() % 16 == 0 else weight.contiguous()
    lib = _lib.load()
    with torch.cuda.device(x.device):
        out = torch.empty((x2.shape[0], hidden), dtype=x.dtype, device=x.device)
        _lib.check(lib.br_rmsnorm(x2.data_ptr(), w.data_ptr(), out.data_ptr(), x2.shape[0], hidden, x2.stride(0), hidden, float(eps),
                                  _DTYPE_CODE[x.dtype], _stream_ptr(x.device)))
    return out.view(x.shape)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up, elementwise, tensors of one shape and dtype (bf16 or fp32)."""
    assert gate.is_cuda and gate.dtype in _DTYPE_CODE and up.dtype == gate.dtype and up.shape == gate.shape
    g, u = gate.contiguous(), up.contiguous()
    lib = _lib.load()
    with torch.cuda.device(gate.device):
        out = torch.empty_like(g)
        _lib.check(lib.br_silu_mul(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _DTYPE_CODE[g.dtype], _stream_ptr(g.device)))
    return out


def _kernel_ok(x: torch.Tensor, *params: torch.Tensor) -> bool:
    if not x.is_cuda or x.dtype not in _DTYPE_CODE or (x.shape[-1] * x.element_size()) % 16:
        return False
    if any(p.dtype != x.dtype for p in params):
        return False
    return not (torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in params)))


def patch_layer_ops(model) -> int:
    """Give every ``*RMSNorm`` module (``weight``, ``variance_epsilon``) and every gated ``*MLP`` module
    (``gate_proj``, ``up_proj``, ``down_proj``, SiLU activation) of ``model`` a forward that uses the kernels.
    Returns the number of modules patched; ``unpatch_layer_ops`` restores them."""
    n = 0
    for m in model.modules():
        if "_blockrank_amd_saved_forward" in m.__dict__:
            continue
        name = type(m).__name__
        if name.endswith("RMSNorm") and hasattr(m, "weight") and hasattr(m, "variance_epsilon"):
            orig = m.forward

            def norm_forward(hidden_states, _m=m, _orig=orig):
                if not _kernel_ok(hidden_states, _m.weight):
                    return _orig(hidden_states)
                return rms_norm(hidden_states, _m.weight, _m.variance_epsilon)

            m.__dict__["_blockrank_amd_saved_forward"] = orig
            m.forward = norm_forward
            n += 1
        elif name.endswith("MLP") and all(hasattr(m, a) for a in ("gate_proj", "up_proj", "down_proj", "act_fn")) and \
                "silu" in type(m.act_fn).__name__.lower():
            orig = m.forward

            def mlp_forward(x, _m=m, _orig=orig):
                if not _kernel_ok(x, _m.gate_proj.weight):
                    return _orig(x)
                return _m.down_proj(silu_mul(_m.gate_proj(x), _m.up_proj(x)))

            m.__dict__["_blockrank_amd_saved_forward"] = orig
            m.forward = mlp_forward
            n += 1
    return n


def unpatch_layer_ops(model) -> None:
    for m in model.modules():
        if "_blockrank_amd_saved_forward" in m.__dict__:
            del m.__dict__["_blockrank_amd_saved_forward"]
            if "forward" in m.__dict__:
                del m.__dict__["forward"]


class _FusedQKV:
    """One GEMM for the Q, K and V projections of an attention module: the three weight matrices stacked once; the
    result of the stacked product is kept until the three projections of the same input tensor have taken their
    slices."""

    def __init__(self, attn):
        mods = (attn.q_proj, attn.k_proj, attn.v_proj)
        self.sizes = [m.out_features for m in mods]
        self.weight = torch.cat([m.weight.detach() for m in mods], dim=0).contiguous()
        self.bias = None
        if any(m.bias is not None for m in mods):
            self.bias = torch.cat([m.bias.detach() if m.bias is not None else m.weight.new_zeros(m.out_features) for m in mods]).contiguous()
        self.x = None
        self.y = None
        self.taken = 0

    def part(self, index: int, x: torch.Tensor):
        """Slice ``index`` of the stacked projection of ``x``, or None if ``x`` is not the tensor the cached product
        belongs to and this is not the first projection (the caller then runs its own GEMM)."""
        if self.x is not x:
            if index != 0:
                return None
            self.x, self.y, self.taken = x, F.linear(x, self.weight, self.bias), 0
        lo = sum(self.sizes[:index])
        out = self.y[..., lo:lo + self.sizes[index]]
        self.taken |= 1 << index
        if self.taken == 7:
            self.x = self.y = None
        return out


def patch_qkv(model) -> int:
    """Give the ``q_proj`` / ``k_proj`` / ``v_proj`` linears of every attention module of ``model`` forwards that share
    one stacked GEMM when they are applied to the same tensor (what the decoder layers do), and run their own GEMM
    otherwise (and whenever gradients are enabled: the stacked weight is a detached copy).  Measured at the Mistral-7B
    shape with 26.8k tokens: 917 us for the stacked product against 1089 us for the three.  Returns the number of
    attention modules patched; ``unpatch_qkv`` restores them.  Call again after the weights change."""
    n = 0
    for m in model.modules():
        if not type(m).__name__.endswith("Attention") or not all(isinstance(getattr(m, a, None), torch.nn.Linear) for a in ("q_proj", "k_proj", "v_proj")):
            continue
        if "_blockrank_amd_fused_qkv" in m.__dict__:
            continue
        fused = _FusedQKV(m)
        m.__dict__["_blockrank_amd_fused_qkv"] = fused
        for index, name in enumerate(("q_proj", "k_proj", "v_proj")):
            lin = getattr(m, name)
            orig = lin.forward

            def forward(x, _index=index, _orig=orig, _fused=fused, _lin=lin):
                if torch.is_grad_enabled() and (x.requires_grad or _lin.weight.requires_grad):
                    return _orig(x)
                out = _fused.part(_index, x)
                return _orig(x) if out is None else out

            lin.__dict__["_blockrank_amd_saved_linear_forward"] = orig
            lin.forward = forward
        n += 1
    return n


def unpatch_qkv(model) -> None:
    for m in model.modules():
        if "_blockrank_amd_fused_qkv" in m.__dict__:
            del m.__dict__["_blockrank_amd_fused_qkv"]
            for name in ("q_proj", "k_proj", "v_proj"):
                lin = getattr(m, name)
                if "_blockrank_amd_saved_linear_forward" in lin.__dict__:
                    del lin.__dict__["_blockrank_amd_saved_linear_forward"]
                    if "forward" in lin.__dict__:
                        del lin.__dict__["forward"]
