"""blockrank_amd: BlockRank block-sparse prefill attention and attention-score ranking on MI355X.

Public surface (same names as the reference package exports for this path,
src/blockrank/__init__.py:19-33):

    register_blockrank_attention, register_triton_blockrank_attention   attention-interface hooks
    compute_auxiliary_attention_loss                                    per-document scores

``TruncatedRanker`` (the evaluation script's layer-truncated forward, scripts/eval_attn.py:102-151),
plus the functional entry points ``blockrank_attention``, ``doc_scores``, ``last_block_logits`` and
the ``BlockMask`` / ``LastBlockScores`` objects the hooks exchange.  Everything computes in
hand-written HIP kernels (libblockrank_hip.so); there is no fallback implementation.
"""
from .attention import (
    BlockMask,
    LastBlockScores,
    blockrank_attention,
    blockrank_attention_forward,
    blockrank_attention_mask,
    doc_scores,
    doc_scores_from_partials,
    last_block_logits,
    register_blockrank_attention,
    register_triton_blockrank_attention,
)
from .losses import bracket_rows, compute_auxiliary_attention_loss, rank_documents
from .ranker import TruncatedRanker
from .collate import block_icr_collate_packed, pack_padded_batch
from .rope import apply_rotary_pos_emb, apply_rotary_pos_emb_fused, patch_rotary, rotate_k, rotate_q, unpatch_rotary
from .layer_ops import patch_layer_ops, patch_qkv, rms_norm, silu_mul, unpatch_layer_ops, unpatch_qkv

__all__ = [
    "apply_rotary_pos_emb",
    "apply_rotary_pos_emb_fused",
    "rotate_k",
    "rotate_q",
    "patch_rotary",
    "unpatch_rotary",
    "rms_norm",
    "silu_mul",
    "patch_layer_ops",
    "unpatch_layer_ops",
    "patch_qkv",
    "unpatch_qkv",
    "BlockMask",
    "LastBlockScores",
    "blockrank_attention",
    "blockrank_attention_forward",
    "blockrank_attention_mask",
    "doc_scores",
    "doc_scores_from_partials",
    "last_block_logits",
    "register_blockrank_attention",
    "register_triton_blockrank_attention",
    "compute_auxiliary_attention_loss",
    "bracket_rows",
    "rank_documents",
    "TruncatedRanker",
    "block_icr_collate_packed",
    "pack_padded_batch",
]
__version__ = "0.1.0"
