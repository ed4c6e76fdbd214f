"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, pure host
entry points behave, the Python hooks keep the reference's error conventions, and the synthetic layout
follows the reference's collate rules.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import blockrank_amd as br
from blockrank_amd import _lib, synthetic

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "blockrank_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(br_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 10
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/blockrank_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes signatures and header are out of step"
    assert lib.br_version() >= 100
    assert lib.br_last_error() == b""


def test_pure_host_entry_points():
    lib = _lib.load()
    assert lib.br_tile_tokens(32, 8) == 32        # 4 heads x 32 tokens per workgroup
    assert lib.br_tile_tokens(28, 4) == 32        # 7 heads x 32 tokens
    assert lib.br_tile_tokens(8, 8) == 128        # 1 head x 128 tokens
    assert lib.br_tile_tokens(6, 2) == 64
    assert lib.br_tile_tokens(7, 2) == 0          # not a whole number of query heads per kv head
    assert lib.br_plan_ints(4, 22, 160, 32, 8) > 4 * 22 * 5 * 8
    assert lib.br_plan_ints(0, 22, 160, 32, 8) == 0
    # the split partials' pool follows the head layout and the device's compute units, not the batch (0: no device here)
    ws = lib.br_prefill_workspace_bytes(4, 32, 8, 128)
    assert ws == lib.br_prefill_workspace_bytes(64, 32, 8, 128)
    assert ws == 0 or 4 << 20 < ws < 32 << 20
    assert lib.br_doc_scores_workspace_bytes(4, 32, 22, 2) == 4 * 32 * 2 * 20 * 2 * 4
    assert ws == 0 or lib.br_prefill_fp8qk_workspace_bytes(4, 32, 8, 128, 22, 4 * 3520) > ws
    # backward: fp32 sums of the query block's dQ rows and of the prefix keys' dK / dV, rounded up to 256 bytes, then one
    # float per token slot and query head (delta)
    assert lib.br_prefill_bwd_workspace_bytes(4, 32, 8, 160, 128, 4 * 3520) == 4 * (32 + 16) * 160 * 128 * 4 + 4 * 3520 * 32 * 4
    assert lib.br_prefill_bwd_workspace_bytes(0, 32, 8, 160, 128, 10) == 0
    rc = lib.br_prefill_bwd(None, None, None, None, None, None, None, 1, 4, 2, 3, 8, 96, None, None, None, None, None, None,
                            None, None, None, None, None, None, 1.0, 24, None, 0, None)
    assert rc == _lib.BR_ERR_ARG and b"head dim" in lib.br_last_error()
    # the entry point that allocates nothing refuses a request beyond its built-in scratch, before any device call
    # (without a device the size of the request cannot be worked out: that is refused as well)
    assert lib.br_prefill_noalloc_max_workspace_bytes() == 32 << 20
    rc = lib.br_prefill_fwd_noalloc(None, None, None, None, None, 1, 1024, 1024, 3, 64, 128, None, None, None, None, 1.0, 1, None)
    assert (rc == _lib.BR_ERR_SPACE and b"built-in scratch" in lib.br_last_error()) or (rc == _lib.BR_ERR_HIP and b"device" in lib.br_last_error())
    # argument errors come back as codes with a message, before anything touches a device
    rc = lib.br_prefill_fwd(None, None, None, None, None, 1, 4, 2, 3, 8, 96, None, None, None, None, 1.0, 1, None, 0, None)
    assert rc == _lib.BR_ERR_ARG and b"head dim" in lib.br_last_error()
    rc = lib.br_plan_build(None, 1, 3, 8, 4, 2, None, 0, None)
    assert rc == _lib.BR_ERR_ARG and b"mask" in lib.br_last_error()
    with pytest.raises(AssertionError):
        _lib.check(rc)


def test_hooks_fail_loudly_without_gpu_tensors():
    valid = torch.ones(1, 3, 8, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="GPU"):
        br.blockrank_attention_mask(batch_size=1, attention_mask=valid)
    with pytest.raises(AssertionError):
        br.blockrank_attention_mask(batch_size=1, attention_mask=None)
    with pytest.raises(AssertionError):
        br.blockrank_attention_forward(None, torch.zeros(1, 2, 24, 64), torch.zeros(1, 2, 24, 64), torch.zeros(1, 2, 24, 64), None, 0.1)


def test_no_fallback_when_library_is_missing(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libblockrank_hip.so")
    with pytest.raises(_lib.BlockRankLibraryError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_registration_uses_reference_names():
    from transformers import AttentionInterface, AttentionMaskInterface
    br.register_blockrank_attention()
    br.register_triton_blockrank_attention()
    for name in br.attention.STD_IMPL_NAMES + br.attention.TRITON_IMPL_NAMES:
        assert AttentionInterface()[name] is br.blockrank_attention_forward
        assert AttentionMaskInterface()[name] is br.blockrank_attention_mask
    # a model config accepts the name
    from transformers import MistralConfig, MistralForCausalLM
    cfg = MistralConfig(vocab_size=64, hidden_size=64, intermediate_size=64, num_hidden_layers=1, num_attention_heads=2,
                        num_key_value_heads=1, head_dim=64)
    model = MistralForCausalLM(cfg)
    model.set_attn_implementation("triton_blockrank")
    assert model.config._attn_implementation == "triton_blockrank"


def test_layout_follows_collate_rules():
    lay = synthetic.make_layout([[3, 5, 2, 4]])
    assert lay.H == 16 and lay.S == 64                       # padded to a multiple of 16
    v = lay.valid[0]
    assert v[0].tolist() == [False] * 13 + [True] * 3         # left padding
    pos = lay.position_ids.view(1, 4, 16)[0]
    assert pos[0, -3:].tolist() == [0, 1, 2]                  # prefix 0..p-1
    assert pos[1, -5:].tolist() == [3, 4, 5, 6, 7]            # every document restarts at p
    assert pos[2, -2:].tolist() == [3, 4]
    assert pos[3, -4:].tolist() == [16384, 16385, 16386, 16387]
    assert (pos[~v] == 0).all()
    assert (lay.labels[0, :-1] == -100).all() and lay.labels[0, -1] != -100
    assert lay.unmasked_pairs() == 6 + (5 * 3 + 15) + (2 * 3 + 3) + 4 * 10 + 10


def test_baseline_pair_counts():
    assert synthetic.uniform_layout(1, 32, 8, 64, 16).unmasked_pairs() == 42392
    assert synthetic.uniform_layout(1, 64, 20, 160, 32).unmasked_pairs() == 569456


def test_bracket_rows_match_reference_rule():
    labels = torch.full((2, 48), -100)
    labels[0, -1] = 5
    labels[1, -4:] = 5
    rows = br.losses.bracket_rows(labels, 16)
    assert rows.tolist() == [[14, 15], [11, 12]]
    labels[1, -16:] = 5
    with pytest.raises(AssertionError):
        br.losses.bracket_rows(labels, 16)


def test_tensor_path_of_loss_matches_oracle_on_cpu():
    from oracle import blockrank_oracle as orc
    rng = np.random.default_rng(0)
    B, N, h1, M, H = 2, 3, 8, 4, 8
    s = torch.as_tensor(rng.normal(size=(B, N, h1, M * H)))
    valid = torch.ones(B, M, H, dtype=torch.bool)
    labels = torch.full((B, M * H), -100)
    labels[:, -1] = 1
    got = br.compute_auxiliary_attention_loss(s, labels, valid, answer_ids=None, return_logits=True)
    want = orc.doc_scores_from_logits(s.numpy(), labels.numpy(), valid.numpy(), 0.05)
    np.testing.assert_allclose(got.numpy(), want, rtol=1e-10)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_scores_handle_is_a_tensor_to_strangers(monkeypatch):
    """LastBlockScores in place of the reference's s_last tensor: torch functions, methods and indexing reach the
    logits (here a stub of the logits kernel, so that the protocol itself is checked without a GPU)."""
    import types
    from blockrank_amd import attention as att
    B, Nq, R, M, H, D = 2, 4, 16, 5, 32, 64
    g = torch.Generator().manual_seed(0)
    full = torch.randn(B, Nq, H, M * H, generator=g)                       # logits of every query-block position

    def fake_logits(query, key, bm, rows, scaling, neg=None):
        return full.take_along_dim(rows.long()[:, None, :, None], dim=2)

    monkeypatch.setattr(att, "last_block_logits", fake_logits)
    bm = types.SimpleNamespace(B=B, M=M, H=H)
    h = att.LastBlockScores(torch.zeros(B, Nq, M * H, D), torch.zeros(B, 2, M * H, D), bm, 0.125, R)
    want = full[:, :, H - R:]
    idx = torch.tensor([[14, 15], [3, 4]])[:, None, :, None]
    got = h.take_along_dim(idx, dim=2)
    assert h._dense is None and torch.equal(got, want.take_along_dim(idx, dim=2))
    assert torch.equal(h.take_along_dim(torch.tensor([[-1, -2], [0, 1]])[:, None, :, None], dim=2),
                       want.take_along_dim(torch.tensor([[15, 14], [0, 1]])[:, None, :, None], dim=2))
    assert tuple(h.shape) == (B, Nq, R, M * H) and h.dim() == 4 and h.size(-1) == M * H and len(h) == B
    assert torch.equal(h[..., H:-H], want[..., H:-H])
    assert torch.equal(torch.softmax(h, dim=-1), torch.softmax(want, dim=-1))
    assert torch.equal(torch.nn.functional.softmax(h[..., H:-H], dim=-1), torch.softmax(want[..., H:-H], dim=-1))
    assert torch.equal(h * 2, want * 2) and torch.equal(h.double(), want.double()) and torch.allclose(h.mean(dim=(1, 2)), want.mean(dim=(1, 2)), atol=1e-6)
    with pytest.raises(AttributeError):
        h.no_such_attribute
