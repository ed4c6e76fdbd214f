#!/usr/bin/env python3
"""Benchmark of the BlockRank attention + per-document score path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg4|cfg5shape|cfg1] [--qk-fp8] [--backward] [--no-cpu-baseline] [--no-e2e]

A step is one pass of the hot path over one batch already resident in HBM: the attention hook
(block-sparse prefill attention of one layer, query/key/value as a Mistral layer hands them over)
followed by the fused per-document score extraction.  The request plan (block table + work items) is
built once per forward pass by the mask hook and shared by every layer, so it is built outside the
timed region and its cost is reported separately (``plan_build_ms``).

``--workload cfg3`` is the end-to-end case instead: a random-initialised
Mistral-7B-shaped decoder run by the layer-truncated ranking driver (layers 0..19 in full, of layer 20
only what the scores need), B=8; its line reports requests/s of the whole forward and, from HIP events
around each layer's attention kernel, that kernel's roofline fraction at this layout.

Prints ONE JSON line: requests/s for the batch, plus
  roofline      the main attention kernel against the bf16 MFMA peak (FLOPs of unmasked
                (query, key) pairs only), its duration measured live with HIP events recorded
                around the kernel on its own stream inside the timed region;
  roofline_hbm  the same kernel against the HBM peak (algorithmic bytes: Q, K, V read once, O
                written once) - the op sits below the machine ridge, so this roof co-binds;
  cpu_baseline  the CPU restatement of the reference's three-call SDPA algorithm + score formula,
                timed on this machine's host cores on a bounded sample (one sequence of the batch);
  e2e           (default workload) the whole ranking request measured in the same run: the --workload cfg3 forward,
                five batches - requests/s, ms per batch, the attention launches' share and roofline fraction, the
                plan's cost, one request alone, the share of the time the GPU idles between launches.

Order of the default run: W warm-up + K timed steps as the process's first GPU work (reported as ``first_launches``:
the GPU raises its clocks over the first tenths of a second of load, so these are the slowest the step ever is), the
end-to-end forward, then W warm-up + K timed steps again - the headline (``clock_state`` says which of the two
conditions a line's figures belong to), then the CPU baseline.  With ``--no-e2e`` there is one pass, as found.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E


def workloads():
    from blockrank_amd import synthetic
    return {
        # the configuration the headline metric is quoted on
        "cfg2": dict(desc="Mistral-7B-shaped attention layer, B=4, 32q/8kv heads, D=128, 64-token prefix + 20 docs x 160 + 32-token query (3296 tokens/seq), bf16, proj+RoPE inputs",
                     layout=lambda: synthetic.uniform_layout(4, 64, 20, 160, 32), Nq=32, Nkv=8, D=128, hidden=4096, dtype=torch.bfloat16),
        # long document list
        "cfg4": dict(desc="Mistral-7B attention shapes, B=1, 64-token prefix + 100 docs U[64,384] + 48-token query, bf16",
                     layout=lambda: synthetic.random_layout(1, 64, 100, 64, 384, 48, seed=0), Nq=32, Nkv=8, D=128, hidden=4096, dtype=torch.bfloat16),
        # Qwen2.5-7B head layout and a long-tailed document length distribution (bf16; --qk-fp8 computes Q K^T in fp8)
        "cfg5shape": dict(desc="Qwen2.5-7B attention shapes, B=4, 28q/4kv heads, D=128, 32-token prefix + 50 lognormal docs + 24-token query, bf16",
                          layout=lambda: synthetic.lognormal_layout(4, 32, 50, 120, 0.6, 16, 512, 24, seed=0), Nq=28, Nkv=4, D=128, hidden=3584, dtype=torch.bfloat16),
        "cfg2d64": dict(desc="cfg2 layout with head dim 64", layout=lambda: synthetic.uniform_layout(4, 64, 20, 160, 32), Nq=32, Nkv=8, D=64, hidden=None, dtype=torch.bfloat16),
        "cfg2_b1": dict(desc="cfg2 with B=1", layout=lambda: synthetic.uniform_layout(1, 64, 20, 160, 32), Nq=32, Nkv=8, D=128, hidden=4096, dtype=torch.bfloat16),
        "cfg2_b16": dict(desc="cfg2 with B=16", layout=lambda: synthetic.uniform_layout(16, 64, 20, 160, 32), Nq=32, Nkv=8, D=128, hidden=4096, dtype=torch.bfloat16),
        # one long causal block per sequence: many key tiles per work item (steady-state tile throughput)
        "causal4k": dict(desc="single block of 4096 tokens per sequence (plain causal), B=8, 32q/8kv heads, D=128, bf16",
                         layout=lambda: synthetic.make_layout([[4096]] * 8), Nq=32, Nkv=8, D=128, hidden=None, dtype=torch.bfloat16),
        # the headline layout with eight query heads per kv head (Llama-3-70B-like grouping)
        "cfg2g8": dict(desc="cfg2 layout with 32q/4kv heads (8 per group), D=128, bf16", layout=lambda: synthetic.uniform_layout(4, 64, 20, 160, 32),
                       Nq=32, Nkv=4, D=128, hidden=None, dtype=torch.bfloat16),
        # the ragged layout of the end-to-end request (BASELINE config 3), one attention layer of it
        "cfg3layout": dict(desc="Mistral-7B attention shapes, B=8, 64-token prefix + 20 docs U[96,224] + 32-token query, bf16 (the end-to-end request's layout)",
                           layout=lambda: synthetic.random_layout(8, 64, 20, 96, 224, 32, seed=0), Nq=32, Nkv=8, D=128, hidden=None, dtype=torch.bfloat16),
        # the small fp32 case that also runs on a CPU in seconds
        "cfg1": dict(desc="fp32, B=1, 8q/2kv heads, D=64, 32-token prefix + 8 docs x 64 + 16-token query", layout=lambda: synthetic.uniform_layout(1, 32, 8, 64, 16),
                     Nq=8, Nkv=2, D=64, hidden=None, dtype=torch.float32),
    }


class _Module:
    """What the attention hook reads from the Hugging Face attention module."""
    training = False

    def __init__(self, layer_idx, groups):
        self.layer_idx, self.num_key_value_groups = layer_idx, groups


def cpu_baseline(layout, q, k, v, scale, dtype, budget_s=12.0):
    """Time the oracle's restatement of the reference algorithm (three SDPA calls with dense additive
    masks, GQA expansion, K0 concatenation, final transpose, 16-row logits, score formula) on the host
    cores, for the first sequence of the batch."""
    from oracle import blockrank_oracle as orc
    import numpy as np
    torch.set_num_threads(os.cpu_count() if "OMP_NUM_THREADS" not in os.environ else int(os.environ["OMP_NUM_THREADS"]))
    q1, k1, v1 = (t[:1].detach().to("cpu", dtype).contiguous() for t in (q, k, v))
    valid1 = layout.valid[:1]
    labels1 = layout.labels[:1].numpy()
    m5 = orc.additive_mask(valid1, dtype)

    def one():
        out, s_last = orc.sdpa_blockrank_forward(q1, k1, v1, m5, scale, return_scores=True)
        return out, orc.doc_scores_from_logits(s_last.float().numpy(), labels1, valid1.numpy(), 0.05)

    one()
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return dict(value=1.0 / med, unit="requests/s", cores=torch.get_num_threads(), kind="port",
                sample=f"first sequence of the batch ({int(layout.lengths[0].sum())} tokens), {str(dtype).replace('torch.', '')}, "
                       f"median of {len(times)} runs, {med * 1e3:.1f} ms per request",
                ms_per_request=med * 1e3)


def cpu_baseline_backward(layout, q, k, v, dout, scale, dtype, budget_s=12.0):
    """The same for the training step: forward of the oracle's restatement of the reference's three-call SDPA
    algorithm plus torch autograd through it (how the reference's trainable hooks are differentiated), on the
    host cores, for the first sequence of the batch."""
    from oracle import blockrank_oracle as orc
    import numpy as np
    torch.set_num_threads(os.cpu_count() if "OMP_NUM_THREADS" not in os.environ else int(os.environ["OMP_NUM_THREADS"]))
    q1, k1, v1 = (t[:1].detach().to("cpu", dtype).contiguous().requires_grad_(True) for t in (q, k, v))
    g1 = dout[:1].detach().to("cpu", dtype).contiguous()
    m5 = orc.additive_mask(layout.valid[:1], dtype)

    def one():
        for t in (q1, k1, v1):
            t.grad = None
        out, _ = orc.sdpa_blockrank_forward(q1, k1, v1, m5, scale)
        out.backward(g1)

    one()
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    return dict(value=1.0 / med, unit="sequences/s", cores=torch.get_num_threads(), kind="port",
                sample=f"first sequence of the batch ({int(layout.lengths[0].sum())} tokens), {str(dtype).replace('torch.', '')}, forward + "
                       f"autograd backward, median of {len(times)} runs, {med * 1e3:.1f} ms per sequence",
                ms_per_sequence=med * 1e3)


def run_model(args, steps, warmup):
    """cfg3: the truncated ranking forward of a Mistral-7B-shaped model with random weights.  Returns the result
    line as a dict."""
    import blockrank_amd as br
    from blockrank_amd import profiling, synthetic
    from transformers import MistralConfig, MistralModel
    dev = torch.device("cuda:0")
    layer_idx = 20
    cfg = MistralConfig(vocab_size=32768, hidden_size=4096, intermediate_size=14336, num_hidden_layers=layer_idx + 1,
                        num_attention_heads=32, num_key_value_heads=8, head_dim=128, rope_theta=1e6, sliding_window=None,
                        max_position_embeddings=32768)
    br.register_triton_blockrank_attention()
    torch.manual_seed(0)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            model = MistralModel(cfg)          # only the layers the driver runs are built: 0 .. layer_idx
    finally:
        torch.set_default_dtype(old)
    model.eval()
    model.set_attn_implementation("triton_blockrank")
    layout = synthetic.random_layout(8, 64, 20, 96, 224, 32, seed=0)
    B, S = layout.B, layout.S
    ids = torch.randint(0, cfg.vocab_size, (B, S), generator=torch.Generator().manual_seed(1)).to(dev)
    pos = layout.position_ids.to(dev)
    valid = layout.valid.to(dev)
    R = min(16, layout.H)
    rows = torch.tensor([[R - 2, R - 1]] * B, dtype=torch.int32, device=dev)
    ranker = br.TruncatedRanker(model, layer_idx)
    if not args.hf_rope:
        # Q and K through the one-pass rotary kernel (--fused-rope: K alone, Q rotated by the attention kernel as it
        # loads its rows - measured the same time per batch: what the rotary kernel saves, the attention kernel pays)
        br.patch_rotary(model, fuse_q=args.fused_rope)
    if not args.hf_layer_ops:
        br.patch_layer_ops(model)        # one-pass RMSNorm and SiLU-gate kernels instead of the model file's eager expressions
        br.patch_qkv(model)              # one GEMM for the Q, K and V projections of a layer
    extra = {}
    if args.padded:
        def forward(**kw):
            return ranker(ids, valid, pos, rows=rows, **kw)

        def build_plan():
            br.blockrank_attention_mask(batch_size=B, attention_mask=valid, dtype=torch.bfloat16).plan(32, 8)
    else:
        pk = br.pack_padded_batch(dict(input_ids=ids, position_ids=pos, attention_mask=valid))
        lens_dev = pk["block_lengths"]

        def forward(**kw):
            return ranker.forward_packed(pk["input_ids"], pk["position_ids"], lens_dev, rows, H=layout.H, **kw)

        def build_plan():
            br.BlockMask.from_lengths(lens_dev, H=layout.H, packed=True, dtype=torch.bfloat16).plan(32, 8)
    # the request plan is built once per forward pass (inside the timed forward); its cost alone, second call
    build_plan()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    build_plan()
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(warmup):
        scores = forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        scores = forward()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    assert torch.isfinite(scores).all()

    def timed_each(fn, n):
        """Median of n calls, each waited for: what one caller sees from call to result."""
        ts = []
        for _ in range(n):
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t1) * 1e3)
        ts.sort()
        return ts[len(ts) // 2]

    def graph_of(fn):
        """The forward captured in a HIP graph (everything the host would have to look at is prepared beforehand);
        returns (replay, result) or None where the capture does not go through."""
        try:
            g = torch.cuda.CUDAGraph()
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                fn()
                torch.cuda.synchronize()
                with torch.cuda.graph(g, stream=s):
                    out = fn()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            return g.replay, out
        except Exception as e:          # a library call inside the model that cannot be captured: report, do not fail the run
            sys.stderr.write(f"HIP graph capture of the forward failed: {e}\n")
            torch.cuda.synchronize()
            return None

    # Ranking latency: one request (the first sequence of the batch) through the same layers, call to result; and the
    # share of the eager forward's wall time that replaying the very same kernels from a HIP graph does not need (the
    # GPU idling between eager launches).
    if not args.padded:
        prep = ranker.prepare_packed(lens_dev, layout.H)
        lay1 = synthetic.make_layout([list(layout.lengths[0])], H=layout.H)
        keep1 = lay1.valid.reshape(-1)
        ids1 = ids[:1].reshape(-1)[keep1.to(dev)][None]
        pos1 = lay1.position_ids.reshape(-1)[keep1][None].to(dev)
        lens1 = torch.as_tensor(lay1.lengths, dtype=torch.int32, device=dev)
        prep1 = ranker.prepare_packed(lens1, layout.H)
        rows1 = rows[:1].contiguous()

        def forward1(**kw):
            return ranker.forward_packed(ids1, pos1, lens1, rows1, H=layout.H, prepared=prep1, **kw)

        for _ in range(3):
            forward1()
        extra["latency_ms_b1"] = timed_each(forward1, 15)
        extra["ms_per_batch_each"] = timed_each(lambda: forward(prepared=prep), 5)
        g8 = graph_of(lambda: forward(prepared=prep))
        if g8 is not None:
            replay8, out8 = g8
            assert torch.allclose(out8, scores, rtol=1e-3, atol=1e-5), "graph replay changed the scores"
            extra["ms_per_batch_graph"] = timed_each(replay8, 5)
            extra["gpu_idle_frac"] = max(0.0, 1.0 - extra["ms_per_batch_graph"] / extra["ms_per_batch_each"])
            del g8, replay8, out8
        g1 = graph_of(forward1)
        if g1 is not None:
            extra["latency_ms_b1_graph"] = timed_each(g1[0], 15)
            extra["gpu_idle_frac_b1"] = max(0.0, 1.0 - extra["latency_ms_b1_graph"] / extra["latency_ms_b1"])
            del g1
    # the attention kernel of every layer of one more forward, from HIP events around it
    pairs = []

    class _Events:
        def __iter__(self):
            pairs.append(profiling.EventPair())
            return iter(pairs[-1].handles)

    forward(kernel_events=_Events())
    torch.cuda.synchronize()
    kern_ms = [p.elapsed_ms() for p in pairs]
    kern_avg_ms = sum(kern_ms) / len(kern_ms)
    pairs_n = layout.unmasked_pairs()
    flops = 4.0 * 128 * pairs_n * 32
    alg_bytes = float(layout.valid_tokens) * 128 * 2 * (2 * 32 + 2 * 8)
    tflops = flops / (kern_avg_ms * 1e-3) / 1e12
    gbs = alg_bytes / (kern_avg_ms * 1e-3) / 1e9
    dense_flops = 2.0 * 218103808 * layout.valid_tokens * layer_idx      # the projections and MLPs of layers 0..19 (real tokens)
    res = {
        "metric": "ranking requests/sec (Mistral-7B-shaped decoder, layers 0-20, layer-truncated forward, 20 docs)",
        "value": B / (ms_per_step * 1e-3), "unit": "requests/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Mistral-7B-shaped decoder (random init), B=8, 64-token prefix + 20 docs U[96,224] + 32-token query, "
                               "layers 0..19 in full and the score part of layer 20, bf16",
                   "name": "cfg3", "batch": B, "blocks": layout.M, "block_len": layout.H, "valid_tokens": layout.valid_tokens,
                   "padded_tokens": B * S, "unmasked_pairs": pairs_n, "launch": "eager",
                   "token_layout": "padded (B, M, H)" if args.padded else "packed (real tokens only)",
                   "rotary": "model's eager expression" if args.hf_rope else ("K: one-pass HIP kernel; Q: inside the attention kernel" if args.fused_rope
                                                                               else "one-pass HIP kernel"),
                   "norm_and_gate": "model's eager expressions" if args.hf_layer_ops else "one-pass HIP kernels",
                   "qkv_projection": "three GEMMs" if args.hf_layer_ops else "one stacked GEMM"},
        "prefill_tok_per_s": layout.valid_tokens / (ms_per_step * 1e-3),
        "plan_build_ms": plan_ms,
        "attention_ms_per_step": sum(kern_ms),
        "attention_share": sum(kern_ms) / ms_per_step,
        "dense_tflops": dense_flops / (ms_per_step * 1e-3) / 1e12,
        "kernel_us": {"prefill_avg": kern_avg_ms * 1e3, "prefill_min": min(kern_ms) * 1e3, "prefill_max": max(kern_ms) * 1e3,
                      "launches": len(kern_ms)},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tflops / PEAK_BF16_TFLOPS,
                     "traffic": None, "kernel": "br_prefill_mfma_kernel", "flops_per_launch": flops},
        "roofline_hbm": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "bytes_per_launch": alg_bytes},
    }
    res.update(extra)
    return res


def bench_model(args):
    print(json.dumps(run_model(args, args.steps if args.steps is not None else 10, args.warmup if args.warmup is not None else 2)))


def bench_backward(args, br, layout, wl, q, k, v, mask, scale):
    """Attention training step (bf16): forward + saved log-sum-exp, then dq, dk, dv.  One JSON line; the roofline
    object prices the backward launches (dQ kernel + dK/dV kernel + their small helpers) at 2.5 times the forward's
    algorithmic FLOPs: five products per visible pair instead of two."""
    Nq, D = wl["Nq"], wl["D"]
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    dout = torch.randn((layout.B, layout.S, Nq, D), device=q.device, dtype=q.dtype)

    def step(ev=None):
        for t in (qq, kk, vv):
            t.grad = None
        if ev:
            ev[0].record()
        out = br.blockrank_attention(qq, kk, vv, mask, scale)
        if ev:
            ev[1].record()
        out.backward(dout)
        if ev:
            ev[2].record()

    for _ in range(args.warmup):
        step()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(evs[i])
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / args.steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / args.steps
    pairs_n = layout.unmasked_pairs()
    flops_bwd = 10.0 * D * pairs_n * Nq
    tflops = flops_bwd / (bwd_ms * 1e-3) / 1e12
    res = {
        "metric": f"attention training steps: sequences/sec through forward + backward ({args.workload})",
        "value": layout.B / (ms_per_step * 1e-3), "unit": "sequences/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": wl["desc"], "name": args.workload, "batch": layout.B, "blocks": layout.M, "block_len": layout.H,
                   "valid_tokens": layout.valid_tokens, "unmasked_pairs": pairs_n, "pass": "forward + backward"},
        "forward_us": fwd_ms * 1e3, "backward_us": bwd_ms * 1e3,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tflops / PEAK_BF16_TFLOPS,
                     "traffic": None, "kernel": "br_bwd_dq_kernel + br_bwd_dkv_kernel", "flops_per_launch": flops_bwd},
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_backward(layout, q, k, v, dout, scale, q.dtype)
        res["cpu_baseline"]["gpu_over_cpu"] = res["value"] / res["cpu_baseline"]["value"]
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="cfg2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-e2e", action="store_true",
                    help="cfg2: leave out the end-to-end leg (the Mistral-7B-shaped ranking forward of --workload cfg3, five batches)")
    ap.add_argument("--graph", action="store_true", help="also time the step replayed from a HIP graph")
    ap.add_argument("--qk-fp8", action="store_true",
                    help="compute Q K^T in fp8 e4m3 (bf16 workloads with head dim 128; includes the quantisation pass)")
    ap.add_argument("--backward", action="store_true",
                    help="time the training step of the attention instead: forward that saves the log-sum-exp, then the backward kernels")
    ap.add_argument("--hf-rope", action="store_true", help="cfg3: keep the model file's own rotary embedding (eight elementwise passes per layer)")
    ap.add_argument("--hinted", action="store_true", help="name the score rows to the hook beforehand (score_rows_hint) instead of letting it guess")
    ap.add_argument("--separate-scores", action="store_true",
                    help="reduce the per-document scores in a launch of their own instead of inside the launch that merges the split partials")
    ap.add_argument("--fused-rope", action="store_true", help="cfg3: rotate Q inside the attention kernel instead of in the stand-alone rotary kernel")
    ap.add_argument("--hf-layer-ops", action="store_true",
                    help="cfg3: keep the model file's own RMSNorm and SiLU-gate expressions (ten elementwise passes per layer)")
    ap.add_argument("--padded", action="store_true",
                    help="cfg3: feed the reference's padded (B, M, H) batch instead of the packed one")
    ap.add_argument("--packed-layout", action="store_true",
                    help="single-layer workloads: feed the packed token layout (real tokens only) instead of the padded (B, M, H) one")
    ap.add_argument("--alias-kv", action="store_true",
                    help="measurement aid (results are wrong): K and V with a token stride of 0, so that every key row is the same 256 cached "
                         "bytes - what is left of the kernel's HBM traffic is the Q and output streams")
    ap.add_argument("--alias-q", action="store_true", help="measurement aid (results are wrong): Q with a token stride of 0 - what is left of the "
                                                           "HBM reads is the K/V stream")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times, so that a profiler's HBM byte counters can be "
                         "scaled against a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: ranking requests are independent and this build uses a single MI355X "
                 "(run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    if args.workload == "cfg3":
        return bench_model(args)
    args.steps = 200 if args.steps is None else args.steps
    args.warmup = 20 if args.warmup is None else args.warmup

    import blockrank_amd as br
    from blockrank_amd import profiling, synthetic

    wl = workloads()[args.workload]
    dev = torch.device("cuda:0")
    layout = wl["layout"]()
    Nq, Nkv, D, dtype = wl["Nq"], wl["Nkv"], wl["D"], wl["dtype"]
    scale = D ** -0.5
    if wl["hidden"]:
        q, k, v = synthetic.attention_layer_inputs(layout, Nq, Nkv, D, wl["hidden"], dtype, dev)
    else:
        q, k, v = synthetic.random_qkv(layout, Nq, Nkv, D, dtype, dev)
    valid = layout.valid.to(dev)
    R = min(16, layout.H)
    rows16 = torch.tensor([[R - 2, R - 1]] * layout.B, dtype=torch.int32, device=dev)   # "[" and the token before it, in the last 16 positions
    module = _Module(20, Nq // Nkv)
    if args.packed_layout:
        # real tokens only, all blocks of all sequences one after the other on one token axis: (1, heads, T, D)
        q, k, v = (t.transpose(1, 2)[valid.reshape(layout.B, layout.S)][None].transpose(1, 2) for t in (q, k, v))
        lens_dev = torch.as_tensor(layout.lengths, dtype=torch.int32, device=dev)
    if args.alias_kv:
        k, v = k[:, :, :1].expand_as(k), v[:, :, :1].expand_as(v)
    if args.alias_q:
        q = q[:, :, :1].expand_as(q)

    # once per forward pass: mask hook -> plan (timed on the second build: the first also loads the library's code)
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if args.packed_layout:
            mask = br.BlockMask.from_lengths(lens_dev, H=layout.H, packed=True, dtype=dtype)
        else:
            mask = br.blockrank_attention_mask(batch_size=layout.B, attention_mask=valid, dtype=dtype)
        mask.plan(Nq, Nkv)
        torch.cuda.synchronize()
        plan_ms = (time.perf_counter() - t0) * 1e3

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.backward:
        return bench_backward(args, br, layout, wl, q, k, v, mask, scale)

    def step(events=None):
        # the hook as the reference's callers call it (scripts/eval_attn.py:139: no extra keyword): it guesses the score
        # rows, the handle confirms the guess against rows16 (once: the tensor is remembered) and returns the scores
        # the attention call already reduced.  --hinted names the rows beforehand, --separate-scores switches the
        # guess off (the scores then take a launch of their own).
        extra = {}
        if args.separate_scores:
            extra["speculate_score_rows"] = False
        elif args.hinted:
            extra["score_rows_hint"] = rows16
        if events is not None:
            extra["kernel_events"] = events
        if args.qk_fp8:
            extra["qk_fp8"] = True
        out, handle = br.blockrank_attention_forward(module, q, k, v, mask, scale, layers_to_return_scores=[20], **extra)
        scores = handle.doc_scores_window(rows16, temperature=0.05) if handle is not None else None
        return out, scores

    def timed_pass():
        for _ in range(args.warmup):
            step()
        pairs = [profiling.EventPair() for _ in range(args.steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            o_, s_ = step(pairs[i].handles)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        return elapsed / args.steps * 1e3, sorted(p.elapsed_ms() for p in pairs), o_, s_

    # The GPU raises its clocks over the first tenths of a second of load: the same 20 steps take 8 % less after a
    # second of work than as the first launches of a process.  The default run therefore times the step twice: once
    # as the process's first GPU work ("first_launches" in the output) and once - the headline - after the end-to-end
    # forward below, which a ranking service would be running anyway, has brought the GPU to its sustained state.
    e2e_model = None
    first = None
    run_e2e = args.workload == "cfg2" and not args.no_e2e and not args.qk_fp8 and not args.backward
    if run_e2e:
        ms_c, kern_c, _, _ = timed_pass()
        first = {"ms_per_step": ms_c, "kernel_us_avg": sum(kern_c) / len(kern_c) * 1e3}
        try:
            e2e_model = run_model(args, steps=5, warmup=2)
        except Exception as exc:      # the headline below does not depend on it
            e2e_model = {"error": f"{type(exc).__name__}: {exc}"}
        torch.cuda.empty_cache()
    ms_per_step, kern_ms, out, scores = timed_pass()
    kern_avg_ms = sum(kern_ms) / len(kern_ms)

    graph_ms = None
    if args.graph:
        g = torch.cuda.CUDAGraph()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            step()
            torch.cuda.synchronize()
            with torch.cuda.graph(g, stream=s):
                g_out, g_scores = step()
        torch.cuda.synchronize()
        for _ in range(5):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            g.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) / args.steps * 1e3
        assert torch.equal(g_out, out), "graph replay changed the attention output"
        assert scores is None or torch.equal(g_scores, scores), "graph replay changed the scores"

    pairs_n = layout.unmasked_pairs()
    flops = 4.0 * D * pairs_n * Nq
    esize = torch.tensor([], dtype=dtype).element_size()
    alg_bytes = float(layout.valid_tokens) * D * esize * (2 * Nq + 2 * Nkv)
    tflops = flops / (kern_avg_ms * 1e-3) / 1e12
    gbs = alg_bytes / (kern_avg_ms * 1e-3) / 1e9
    # HBM bytes per launch are not measured by this run: they come from the profiler's FETCH_SIZE / WRITE_SIZE counters,
    # recorded with the command and the commit they were taken at
    traffic, traffic_from = None, None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        try:
            rec = json.load(open(tpath)).get(args.workload)
            if rec:
                traffic, traffic_from = rec["bytes_per_launch"], f"{rec['source']} (rocprofv3 counters, taken at commit {rec['commit']})"
        except Exception:
            traffic = None

    best_ms = ms_per_step if graph_ms is None else min(ms_per_step, graph_ms)
    res = {
        "metric": "ranking requests/sec (one Mistral-7B-shaped attention layer + per-document score extraction, 20 docs)"
        if args.workload == "cfg2" else f"ranking requests/sec ({args.workload})",
        "value": layout.B / (best_ms * 1e-3),
        "unit": "requests/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": best_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("fp8 e4m3 Q K^T (power-of-two scales: one per (sequence, kv head) for K, one per row for Q; the query block's rows stay bf16) + bf16 P V"
                  if args.qk_fp8 else "bf16") if dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {"workload": wl["desc"], "name": args.workload, "batch": layout.B, "blocks": layout.M, "block_len": layout.H,
                   "valid_tokens": layout.valid_tokens, "unmasked_pairs": pairs_n, "launch": "graph" if graph_ms is not None and graph_ms < ms_per_step else "eager",
                   "token_layout": "packed (real tokens only)" if args.packed_layout else "padded (B, M, H)",
                   "score_rows": "named beforehand (score_rows_hint)" if args.hinted else ("reduced in a launch of their own" if args.separate_scores
                                                                                       else "guessed by the hook, confirmed by the handle"),
                   **({"aliased": "K/V" if args.alias_kv else "Q"} if (args.alias_kv or args.alias_q) else {})},
        "prefill_tok_per_s": layout.valid_tokens / (best_ms * 1e-3),
        "ms_per_step_eager": ms_per_step,
        "ms_per_step_graph": graph_ms,
        "plan_build_ms": plan_ms,
        "kernel_us": {"prefill_avg": kern_avg_ms * 1e3, "prefill_p10": kern_ms[len(kern_ms) // 10] * 1e3,
                      "prefill_p50": kern_ms[len(kern_ms) // 2] * 1e3, "prefill_p90": kern_ms[(len(kern_ms) * 9) // 10] * 1e3},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tflops / PEAK_BF16_TFLOPS,
                     "traffic": traffic, "traffic_from": traffic_from, "kernel": "br_prefill_mfma_kernel", "flops_per_launch": flops},
        "roofline_hbm": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "bytes_per_launch": alg_bytes},
    }
    if dtype == torch.float32:
        res["roofline"].update(bound="mfma", peak=157.3, frac=tflops / 157.3, kernel="br_prefill_f32_kernel")
    if not args.no_cpu_baseline and not (args.packed_layout or args.alias_kv or args.alias_q):
        res["cpu_baseline"] = cpu_baseline(layout, q, k, v, scale, dtype)
        res["cpu_baseline"]["gpu_over_cpu"] = res["value"] / res["cpu_baseline"]["value"]
        if args.workload == "cfg2" and dtype == torch.bfloat16:
            # the same request in fp32 (the dtype the reference's CPU path is quoted in) and BASELINE config 1, both bounded
            res["cpu_baseline"]["fp32"] = cpu_baseline(layout, q, k, v, scale, torch.float32, budget_s=5.0)
            w1 = workloads()["cfg1"]
            lay1 = w1["layout"]()
            q1, k1, v1 = synthetic.random_qkv(lay1, w1["Nq"], w1["Nkv"], w1["D"], torch.float32, dev)
            res["cpu_baseline"]["cfg1_fp32"] = cpu_baseline(lay1, q1, k1, v1, w1["D"] ** -0.5, torch.float32, budget_s=2.0)
    if first is not None:
        first["roofline_frac"] = flops / (first["kernel_us_avg"] * 1e-6) / 1e12 / PEAK_BF16_TFLOPS
        res["first_launches"] = first
    res["clock_state"] = ("sustained: timed after the end-to-end forward of the same run" if run_e2e
                          else "as found: the step is this process's first GPU work")
    if run_e2e:
        # the ranking request end to end: what the headline layer is one twenty-first of
        m = e2e_model
        if "error" in m:
            res["e2e"] = m
            print(json.dumps(res))
            return
        res["e2e"] = {
            "workload": m["config"]["workload"], "name": "cfg3", "requests_per_s": m["value"], "ms_per_batch": m["ms_per_step"],
            "batch": m["config"]["batch"], "steps": 5, "warmup": 2, "prefill_tok_per_s": m["prefill_tok_per_s"],
            "token_layout": m["config"]["token_layout"], "plan_build_ms": m["plan_build_ms"],
            "attention_ms_per_batch": m["attention_ms_per_step"], "attention_share": m["attention_share"],
            "attention_kernel_us_per_layer": m["kernel_us"]["prefill_avg"], "attention_launches": m["kernel_us"]["launches"],
            "attention_roofline_frac_mfma": m["roofline"]["frac"], "attention_roofline_frac_hbm": m["roofline_hbm"]["frac"],
            "dense_tflops": m["dense_tflops"],
        }
        for key in ("latency_ms_b1", "latency_ms_b1_graph", "ms_per_batch_each", "ms_per_batch_graph", "gpu_idle_frac", "gpu_idle_frac_b1"):
            if key in m:
                res["e2e"][key] = m[key]
    print(json.dumps(res))


if __name__ == "__main__":
    main()
