#!/usr/bin/env python3
"""Mekevik beside Mixtral at equal layer sizes: engine prefill / decode
throughput and per-kernel roofline fractions (random weights).

Run through `python bench.py --arch-compare --arch mekevik [--arch-size
NAME]`; prints one JSON object.  Same two measurements as
tools/bench_hybrid.py: the LLMEngine loop for both models (eager decode
for both), and each new kernel next to the like kernel of the Llama /
Mixtral path, priced against the MI355X roofline (2.5 PFLOP/s dense bf16,
8 TB/s HBM).
"""
from __future__ import annotations

import json
import sys
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
sys.path.insert(0, str(Path(__file__).resolve().parent))

from bench_hybrid import _engine_run, _entry, _time  # noqa: E402

# Mixtral-8x7B's layer shape, and a half-width one.  Both models: 4
# layers of attention + 8 experts (top 2); grouped key/value heads 4:1.
SIZES = {
    "4k": dict(width=4096, heads=32, kv_heads=8, dim=128, vdim=128,
               window=4096, ff=14336, experts=8, top=2, expert_ff=14336,
               vocab=32000, layers=4, bias_rows=64, bias_far=4096.0),
    "2k": dict(width=2048, heads=16, kv_heads=4, dim=128, vdim=128,
               window=1024, ff=8192, experts=8, top=2, expert_ff=4096,
               vocab=32000, layers=4, bias_rows=32, bias_far=1024.0),
}


def _configs(sz):
    from inference_gateway_amd.engine.config import (ModelConfig,
                                                     mekevik_preset)

    mek = mekevik_preset(
        "mekevik-bench", width=sz["width"], vocab=sz["vocab"],
        pattern=" ".join("m" for _ in range(sz["layers"])),
        heads=sz["heads"], kv_heads=sz["kv_heads"], dim=sz["dim"],
        vdim=sz["vdim"], window=sz["window"], ff=sz["ff"],
        experts=sz["experts"], top=sz["top"], expert_ff=sz["expert_ff"],
        bias_rows=sz["bias_rows"], bias_far=sz["bias_far"])
    mix = ModelConfig(
        name="mixtral-bench", hidden_size=sz["width"],
        num_layers=sz["layers"], num_heads=sz["heads"],
        num_kv_heads=sz["kv_heads"], head_dim=128,
        intermediate_size=sz["expert_ff"], vocab_size=sz["vocab"],
        rope_base=1e6, num_experts=sz["experts"],
        num_experts_per_tok=sz["top"])
    return mek, mix


def _kernels(sz):
    from inference_gateway_amd import ops

    dev, bf = "cuda", torch.bfloat16
    D, H, G = sz["width"], sz["heads"], sz["kv_heads"]
    dk, dv = sz["dim"], sz["vdim"]
    out = {}
    bs = 16

    def paged(nseq, ctx):
        nb = nseq * (ctx // bs) + 1
        kc = torch.randn(nb, G, bs, dk, device=dev, dtype=bf)
        vc = torch.randn(nb, G, dv, bs, device=dev, dtype=bf)
        bt = (torch.arange(nseq * (ctx // bs), dtype=torch.int32,
                           device=dev) + 1).view(nseq, ctx // bs)
        return kc, vc, bt

    nd = min(int(sz["bias_far"]) + 1, sz["window"] or 1 << 30)
    bias = torch.randn(nd, H, device=dev) - 4.0
    talk = torch.eye(H, device=dev) + 0.05 * torch.randn(H, H, device=dev)

    # ---- prompt attention: 4 x 2048 tokens, window as configured ----
    nseq, L = 4, 2048
    T = nseq * L
    W = min(sz["window"], L) if sz["window"] else L
    kc, vc, bt = paged(nseq, L)
    q = torch.randn(T, H * dk, device=dev, dtype=bf)
    gate = torch.randn(T, H * dv, device=dev, dtype=bf)
    row_seq = torch.arange(nseq, dtype=torch.int32,
                           device=dev).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=dev).repeat(nseq)
    keys = sum(min(p + 1, W) for p in range(L)) * nseq     # (row, key) pairs
    t = _time(lambda: ops.sigmoid_attention(
        q, kc, vc, bt, row_seq, pos, bias, talk, gate, 0.09, sz["window"], T,
        [L] * nseq, L), 5)
    out["sigmoid_attention_prompt"] = _entry(
        t, flops=2.0 * keys * H * (dk + dv + H))
    hd = 128
    q3 = torch.randn(T, H, hd, device=dev, dtype=bf)
    k3 = torch.randn(T, G, hd, device=dev, dtype=bf)
    v3 = torch.randn(T, G, hd, device=dev, dtype=bf)
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.flash_prefill(q3, k3, v3, cu, [L] * nseq, 0.09), 5)
    out["flash_prefill"] = _entry(
        t, flops=4.0 * nseq * (L * (L + 1) / 2) * H * hd)

    # ---- decode attention: 256 sequences at 2048 tokens ----
    B, ctx = 256, 2048
    kc, vc, bt = paged(B, ctx)
    q = torch.randn(B, H * dk, device=dev, dtype=bf)
    gate = torch.randn(B, H * dv, device=dev, dtype=bf)
    row_seq = torch.arange(B, dtype=torch.int32, device=dev)
    pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=dev)
    Wd = min(sz["window"], ctx) if sz["window"] else ctx
    t = _time(lambda: ops.sigmoid_attention(
        q, kc, vc, bt, row_seq, pos, bias, talk, gate, 0.09, sz["window"],
        0, None, ctx))
    out["sigmoid_attention_decode"] = _entry(
        t, flops=2.0 * B * Wd * H * (dk + dv + H),
        bytes_=2.0 * B * Wd * G * (dk + dv))
    kc2 = torch.randn(B * (ctx // bs) + 1, G, bs, hd, device=dev, dtype=bf)
    vc2 = torch.randn_like(kc2)
    ctx_lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q3 = torch.randn(B, H, hd, device=dev, dtype=bf)
    t = _time(lambda: ops.paged_attn_decode(q3, kc2, vc2, bt, ctx_lens, 0.09))
    out["paged_attn_decode"] = _entry(
        t, flops=4.0 * B * ctx * H * hd, bytes_=4.0 * B * ctx * G * hd)
    del kc, vc, kc2, vc2

    # ---- norms on 8192 rows ----
    T = 8192
    res = torch.randn(T, D, device=dev)
    da = torch.randn(T, D, device=dev, dtype=bf)
    db = torch.randn(T, D, device=dev, dtype=bf)
    w1, w2 = torch.ones(D, device=dev), torch.ones(D, device=dev)
    t = _time(lambda: ops.add_rmsnorm_pair(res, da, db, w1, w2, 1e-6, bf))
    # residual read + write, two deltas in, two normed outputs
    out["add_rmsnorm_pair"] = _entry(t, bytes_=T * D * (8 + 4 + 4.0))
    x = torch.randn(T, D, device=dev, dtype=bf)
    rs = torch.randn(T, D, device=dev, dtype=bf)
    wb = torch.ones(D, device=dev, dtype=bf)
    t = _time(lambda: ops.fused_add_rmsnorm(x, rs, wb, 1e-5))
    out["fused_add_rmsnorm"] = _entry(t, bytes_=T * D * 8.0)

    # ---- projection post-processing on 8192 rows ----
    nq, nk, nv = H * dk, G * dk, G * dv
    proj = torch.randn(T, nq + nk + nv + H * dv, device=dev, dtype=bf)
    vf = torch.randn(T, nv, device=dev, dtype=bf)
    kc = torch.zeros(T // bs + 1, G, bs, dk, device=dev, dtype=bf)
    vc = torch.zeros(T // bs + 1, G, dv, bs, device=dev, dtype=bf)
    slots = torch.arange(bs, T + bs, dtype=torch.int32, device=dev)
    wq, wk = torch.ones(nq, device=dev), torch.ones(nk, device=dev)
    t = _time(lambda: ops.qk_norm_append(proj, slots, kc, vc, wq, wk, vf,
                                         0.5, 1e-6, H, G, dk, dv))
    out["qk_norm_append"] = _entry(
        t, bytes_=T * 2.0 * (2 * nq + 2 * nk + 3 * nv))
    cs = ops.build_cos_sin_cache(hd, 4096, 1e6, dev) if hasattr(
        ops, "build_cos_sin_cache") else None
    pos8 = torch.arange(T, dtype=torch.int32, device=dev) % 4096
    qf = torch.randn(T, H * hd, device=dev, dtype=bf)
    kf = torch.randn(T, G * hd, device=dev, dtype=bf)
    vf2 = torch.randn(T, G * hd, device=dev, dtype=bf)
    kc2 = torch.zeros(T // bs + 1, G, bs, hd, device=dev, dtype=bf)
    vc2 = torch.zeros_like(kc2)
    try:
        def rope_append():
            ops.rotary_embedding(pos8, qf, kf, hd, cs)
            ops.append_kv_cache(kf.view(T, G, hd), vf2.view(T, G, hd), kc2,
                                vc2, slots)
        t = _time(rope_append)
        out["rotary_plus_append"] = _entry(
            t, bytes_=T * 2.0 * (2 * H * hd + 3 * G * hd + 2 * G * hd))
    except Exception as e:       # a signature the harness guessed wrong
        out["rotary_plus_append"] = {"error": type(e).__name__}

    # ---- activations on [8192, ff] ----
    F_ = sz["ff"]
    gu = torch.randn(T, 2 * F_, device=dev, dtype=bf)
    t = _time(lambda: ops.gated_act(gu, ops.GATED_ACT_CLAMPED, 7.0, 1.702))
    out["gated_act_clamped"] = _entry(t, bytes_=T * F_ * 6.0)
    t = _time(lambda: ops.gated_act(gu, ops.GATED_ACT_SILU))
    out["gated_act_silu"] = _entry(t, bytes_=T * F_ * 6.0)
    t = _time(lambda: ops.silu_mul(gu))
    out["silu_mul"] = _entry(t, bytes_=T * F_ * 6.0)

    # ---- routing, 256 rows ----
    lg = torch.randn(256, sz["experts"], device=dev)
    t = _time(lambda: ops.moe_topk_route(lg, sz["top"], 256, 2.0))
    out["moe_topk_route"] = _entry(t)
    t = _time(lambda: ops.moe_route(lg, sz["top"], 256))
    out["moe_route"] = _entry(t)
    return out


def run(size: str = "2k", batch: int = 64, prompt_len: int = 1024,
        steps: int = 32, warmup: int = 4) -> dict:
    sz = SIZES[size]
    mek, mix = _configs(sz)
    res = {"size": size, "shape": sz, "batch": batch,
           "prompt_len": prompt_len, "steps": steps, "dtype": "bf16",
           "data": "synthetic (random weights and tokens)"}
    res["kernels"] = _kernels(sz)
    res["mekevik"] = _engine_run(mek, batch, prompt_len, steps, warmup)
    res["mixtral"] = _engine_run(mix, batch, prompt_len, steps, warmup)
    return res


if __name__ == "__main__":
    print(json.dumps(run(*(sys.argv[1:2] or ["2k"]))))
