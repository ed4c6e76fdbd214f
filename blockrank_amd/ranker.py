"""Layer-truncated prefill for attention-based ranking.

The reference's evaluation (scripts/eval_attn.py:102-151) runs a full Hugging Face forward with every
decoder layer after the scoring layer and the LM head monkey-patched to identity, and still pays for
the scoring layer's whole attention output, output projection and MLP although nothing consumes
them.  ``TruncatedRanker`` drives the same decoder stack directly:

  * layers 0 .. l*-1 run in full (the model's own layer modules, with this package's attention hook);
  * of layer l* only what the per-document scores need is computed: the input norm, the key
    projection of all tokens, the query projection of the query block only, RoPE on both, and the
    fused score kernels.  No V projection, no attention output, no o_proj, no MLP, no final norm,
    no LM head, no KV cache.

The scores are those of ``compute_auxiliary_attention_loss(out.attentions[0], ...)`` of the full
forward (src/blockrank/losses.py:37-78), and ``rank`` returns the top-k document indices as
scripts/eval_attn.py:150-151 does.
"""
from __future__ import annotations

import sys
from typing import Optional

import torch

from .attention import BlockMask, blockrank_attention_mask, doc_scores
from .losses import bracket_rows, rank_documents


def _decoder(model):
    base = model.model if hasattr(model, "model") and hasattr(model.model, "layers") else model
    if not hasattr(base, "layers"):
        raise TypeError("cannot find the decoder layer list (expected .model.layers or .layers)")
    return base


def _module_rotary(attn):
    """The rotary function of the file the attention class lives in - unless it is this package's variant that leaves
    Q to the attention kernel: the scoring layer's queries go to the score kernels, which take them rotated."""
    fn = sys.modules[type(attn).__module__].apply_rotary_pos_emb
    if getattr(fn, "_blockrank_fused_q", False):
        from .rope import apply_rotary_pos_emb
        return apply_rotary_pos_emb
    return fn


class TruncatedRanker:
    """scores = TruncatedRanker(model, layer_idx)(input_ids, attention_mask, position_ids, labels)

    ``model``: a Hugging Face decoder (MistralForCausalLM / LlamaForCausalLM / Qwen2ForCausalLM or the
    bare ``*Model``) whose attention implementation is one of the BlockRank names this package
    registers.  ``layer_idx``: the scoring layer (``eval.aux_layer_idx`` of the reference's configs).
    """

    def __init__(self, model, layer_idx: int, temperature: float = 0.05, num_last_queries: int = 16):
        self.base = _decoder(model)
        if not 0 <= layer_idx < len(self.base.layers):
            raise ValueError(f"layer_idx {layer_idx} outside 0..{len(self.base.layers) - 1}")
        self.layer_idx = int(layer_idx)
        self.temperature = float(temperature)
        self.num_last_queries = int(num_last_queries)

    @torch.no_grad()
    def __call__(self, input_ids: torch.Tensor, attention_mask: torch.Tensor, position_ids: torch.Tensor,
                 labels: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None, **layer_kwargs) -> torch.Tensor:
        """input_ids, position_ids (B, M*H) or (B, M, H); attention_mask (B, M, H) as the collate function
        of the reference builds them (src/blockrank/dataset.py:219-257).  The rows whose attention is
        scored are the bracket token and the one before it, found from ``labels`` (B, M*H) exactly as
        losses.py:43-48 does, or given directly as ``rows`` (B, R) indices into the last
        ``num_last_queries`` positions.  Further keyword arguments go to every decoder layer (and from
        there to the attention hook).  Returns (B, M-2) fp32 scores."""
        base = self.base
        B, M, H = attention_mask.shape
        S = M * H
        assert M >= 3, "ranking needs a prefix, at least one document and a query block"
        input_ids = input_ids.reshape(B, S)
        position_ids = position_ids.reshape(B, S)
        h1 = self.num_last_queries if H >= self.num_last_queries else H
        if rows is None:
            assert labels is not None, "either labels or rows must be given"
            rows = bracket_rows(labels.reshape(B, S), h1)
        pos = (rows + (H - h1)).to(torch.int32)                       # positions inside the query block

        hidden = base.embed_tokens(input_ids)
        mask = blockrank_attention_mask(batch_size=B, attention_mask=attention_mask, dtype=hidden.dtype)
        if not isinstance(mask, BlockMask):                             # the dense-mask debugging switch is on
            mask = BlockMask(attention_mask, hidden.dtype)
        cos_sin = base.rotary_emb(hidden, position_ids=position_ids)
        for layer in base.layers[: self.layer_idx]:
            hidden = layer(hidden, attention_mask=mask, position_ids=position_ids, past_key_values=None, use_cache=False,
                           position_embeddings=cos_sin, **layer_kwargs)
            if isinstance(hidden, tuple):                               # older decoder layers return a tuple
                hidden = hidden[0]

        # the scoring layer: keys of all tokens, queries of the query block only
        layer = base.layers[self.layer_idx]
        attn = layer.self_attn
        rope = _module_rotary(attn)
        D = attn.head_dim
        x = layer.input_layernorm(hidden)
        k = attn.k_proj(x).view(B, S, -1, D).transpose(1, 2)           # (B, Nkv, S, D)
        q = attn.q_proj(x[:, S - H:]).view(B, H, -1, D).transpose(1, 2)  # (B, Nq, H, D): the query block
        for name in ("q_norm", "k_norm"):                               # per-head norms of newer model families
            if hasattr(attn, name):
                raise NotImplementedError(f"attention modules with {name} are not supported by the truncated driver")
        cos, sin = cos_sin
        _, k = rope(k, k, cos, sin)
        q, _ = rope(q, q, cos[:, S - H:], sin[:, S - H:])
        return doc_scores(q, k, mask, pos, attn.scaling, temperature=self.temperature, query_block_only=True)

    def prepare_packed(self, block_lengths: torch.Tensor, H: Optional[int] = None, dtype: torch.dtype = torch.bfloat16) -> dict:
        """Everything about a packed batch that depends on the block lengths alone and needs the host to look at
        them: the block mask with its device plan and the positions of the query blocks' tokens on the token axis.
        ``forward_packed(..., prepared=...)`` then runs without a host synchronisation, so it can be captured in a
        HIP graph and replayed for every batch of that shape."""
        B, M = block_lengths.shape
        dev = block_lengths.device
        mask = BlockMask.from_lengths(block_lengths, H=H, packed=True, dtype=dtype)
        cfg = self.base.config
        mask.plan(cfg.num_attention_heads, cfg.num_key_value_heads)
        flat = block_lengths.reshape(-1).long()
        block_of = torch.repeat_interleave(torch.arange(B * M, device=dev), flat, output_size=mask.total_tokens)
        idx_q = ((block_of % M) == M - 1).nonzero().squeeze(-1)
        return dict(mask=mask, idx_q=idx_q)

    @torch.no_grad()
    def forward_packed(self, input_ids: torch.Tensor, position_ids: torch.Tensor, block_lengths: torch.Tensor, rows: torch.Tensor,
                       H: Optional[int] = None, prepared: Optional[dict] = None, **layer_kwargs) -> torch.Tensor:
        """The same forward on a packed batch (see blockrank_amd.collate): input_ids, position_ids (1, T)
        hold the real tokens only, block_lengths (B, M) says how they split into blocks, rows (B, R)
        are indices into the last ``num_last_queries`` positions of the query block.  The dense layers
        then run over T tokens instead of B*M*H slots.  ``prepared``: the result of ``prepare_packed`` for these
        block lengths (the call then never waits for the device).  Returns (B, M-2) fp32 scores."""
        base = self.base
        B, M = block_lengths.shape
        assert M >= 3, "ranking needs a prefix, at least one document and a query block"
        dev = input_ids.device
        T = input_ids.shape[-1]
        input_ids = input_ids.reshape(1, T)
        position_ids = position_ids.reshape(1, T)
        hidden = base.embed_tokens(input_ids)
        if prepared is None:
            prepared = self.prepare_packed(block_lengths.to(dev), H, hidden.dtype)
        mask = prepared["mask"]
        assert mask.total_tokens == T, "block_lengths do not sum to the number of tokens"
        Hs = mask.H
        h1 = self.num_last_queries if Hs >= self.num_last_queries else Hs
        pos = (rows.to(dev) + (Hs - h1)).to(torch.int32)
        cos_sin = base.rotary_emb(hidden, position_ids=position_ids)
        for layer in base.layers[: self.layer_idx]:
            hidden = layer(hidden, attention_mask=mask, position_ids=position_ids, past_key_values=None, use_cache=False,
                           position_embeddings=cos_sin, **layer_kwargs)
            if isinstance(hidden, tuple):
                hidden = hidden[0]
        layer = base.layers[self.layer_idx]
        attn = layer.self_attn
        rope = _module_rotary(attn)
        D = attn.head_dim
        for name in ("q_norm", "k_norm"):
            if hasattr(attn, name):
                raise NotImplementedError(f"attention modules with {name} are not supported by the truncated driver")
        x = layer.input_layernorm(hidden)
        cos, sin = cos_sin
        k = attn.k_proj(x).view(1, T, -1, D).transpose(1, 2)
        _, k = rope(k, k, cos, sin)
        # queries of the query blocks only, scattered to their places on the token axis (the score
        # kernels read no other query rows, so the rest of that buffer stays unwritten)
        idx_q = prepared["idx_q"]
        qc = attn.q_proj(x[:, idx_q]).view(1, idx_q.numel(), -1, D).transpose(1, 2)
        qc, _ = rope(qc, qc, cos[:, idx_q], sin[:, idx_q])
        Nq = qc.shape[1]
        q_full = torch.empty((1, T, Nq, D), dtype=qc.dtype, device=dev)
        q_full[:, idx_q] = qc.transpose(1, 2)
        return doc_scores(q_full.transpose(1, 2), k, mask, pos, attn.scaling, temperature=self.temperature)

    def rank(self, *args, k: int = 10, **kwargs) -> torch.Tensor:
        """Top-k document indices (B, min(k, docs)), as scripts/eval_attn.py:150-151 takes them."""
        return rank_documents(self(*args, **kwargs), k)
