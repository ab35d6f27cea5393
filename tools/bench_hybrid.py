#!/usr/bin/env python3
"""Fedatar beside Mixtral at equal layer sizes: engine prefill / decode
throughput and per-kernel roofline fractions (random weights).

Run through `python bench.py --arch-compare [--arch-size NAME]`; prints
one JSON object.  Two measurements:

* engine level — the same LLMEngine loop for both models (eager decode
  for both: the hybrid model has no captured decode graph), a burst of
  equal prompts then decode steps; tokens/s for each phase.
* kernel level — each hybrid kernel and the like kernel of the Llama /
  Mixtral path on the shapes of that layer, timed with device events and
  priced against the MI355X roofline (2.5 PFLOP/s dense bf16, 8 TB/s
  HBM): `frac` is achieved / peak of whichever bound applies.
"""
from __future__ import annotations

import json
import math
import sys
import time
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

PEAK_FLOPS = 2.5e15
PEAK_BW = 8.0e12

# width, heads, (dim, rot, vdim, kv_rank, q_rank), window, ff, experts,
# top, expert_ff — Mixtral-8x7B's layer shape, and a half-width one
SIZES = {
    "4k": dict(width=4096, heads=32, dim=128, rot_dim=64, vdim=128,
               kv_rank=512, q_rank=1536, window=4096, ff=14336, experts=8,
               top=2, expert_ff=14336, vocab=32000, layers=4),
    "2k": dict(width=2048, heads=16, dim=128, rot_dim=64, vdim=128,
               kv_rank=256, q_rank=768, window=1024, ff=8192, experts=8,
               top=2, expert_ff=4096, vocab=32000, layers=4),
}


def _configs(sz):
    from inference_gateway_amd.engine.config import (ModelConfig,
                                                     fedatar_preset)

    pat = " ".join(["gd", "am", "gm", "am"][i % 4]
                   for i in range(sz["layers"]))
    fed = fedatar_preset(
        "fedatar-bench", width=sz["width"], vocab=sz["vocab"], pattern=pat,
        heads=sz["heads"], dim=sz["dim"], rot_dim=sz["rot_dim"],
        vdim=sz["vdim"], kv_rank=sz["kv_rank"], q_rank=sz["q_rank"],
        window=sz["window"], ff=sz["ff"], experts=sz["experts"],
        top=sz["top"], expert_ff=sz["expert_ff"], shared_ff=0)
    mix = ModelConfig(
        name="mixtral-bench", hidden_size=sz["width"],
        num_layers=sz["layers"], num_heads=sz["heads"],
        num_kv_heads=max(1, sz["heads"] // 4), head_dim=128,
        intermediate_size=sz["expert_ff"], vocab_size=sz["vocab"],
        rope_base=1e6, num_experts=sz["experts"],
        num_experts_per_tok=sz["top"])
    return fed, mix


def _engine_run(model_cfg, batch, prompt_len, steps, warmup):
    from inference_gateway_amd.engine.config import (EngineConfig,
                                                     SamplingParams)
    from inference_gateway_amd.engine.engine import LLMEngine

    cfg = EngineConfig(
        model=model_cfg, max_num_seqs=batch,
        max_batched_tokens=max(8192, prompt_len * 4),
        max_model_len=prompt_len + steps + warmup + 64,
        num_gpu_blocks=batch * ((prompt_len + steps + warmup) // 16 + 4) + 8,
        use_hip_graphs=False, enforce_eager=True)
    eng = LLMEngine(cfg, device="cuda:0")
    gen = torch.Generator().manual_seed(7)

    def burst():
        for _ in range(batch):
            eng.add_request(
                torch.randint(0, model_cfg.vocab_size, (prompt_len,),
                              generator=gen).tolist(),
                SamplingParams(max_new_tokens=10 ** 9, temperature=0.0,
                               ignore_eos=True))

    # warm the prefill path once (library GEMM selection), then time it
    burst()
    while eng.scheduler.waiting:
        eng.step()
    for s in list(eng.scheduler.running):
        eng.abort_request(s.seq_id)
    torch.cuda.synchronize()
    burst()
    t0 = time.perf_counter()
    while eng.scheduler.waiting:
        eng.step()
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    for _ in range(warmup):
        eng.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    torch.cuda.synchronize()
    t_decode = time.perf_counter() - t0
    del eng
    torch.cuda.empty_cache()
    return {"prefill_tok_s": round(batch * prompt_len / t_prefill),
            "decode_tok_s": round(batch * steps / t_decode),
            "decode_ms_per_step": round(1e3 * t_decode / steps, 3)}


def _time(fn, iters=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(True), torch.cuda.Event(True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def _entry(seconds, flops=0.0, bytes_=0.0):
    t_roof = max(flops / PEAK_FLOPS, bytes_ / PEAK_BW)
    return {"us": round(seconds * 1e6, 1),
            "tflops": round(flops / seconds / 1e12, 1),
            "gbps": round(bytes_ / seconds / 1e9),
            "bound": "flops" if flops / PEAK_FLOPS > bytes_ / PEAK_BW
            else "bytes",
            "frac": round(t_roof / seconds, 4)}


def _kernels(sz):
    from inference_gateway_amd import ops

    dev, bf = "cuda", torch.bfloat16
    D, H, R, RD = sz["width"], sz["heads"], sz["kv_rank"], sz["rot_dim"]
    out = {}
    bs = 16

    def paged(nseq, ctx, width):
        nb = nseq * (ctx // bs) + 1
        cache = torch.randn(nb, bs, width, device=dev, dtype=bf)
        bt = (torch.arange(nseq * (ctx // bs), dtype=torch.int32,
                           device=dev) + 1).view(nseq, ctx // bs)
        return cache, bt

    # ---- prompt attention: 4 x 2048 tokens, window as configured ----
    nseq, L = 4, 2048
    T = nseq * L
    W = min(sz["window"], L) if sz["window"] else L
    cache, bt = paged(nseq, L, R + RD)
    qa = torch.randn(T, H, R, device=dev, dtype=bf)
    qr = torch.randn(T, H, RD, device=dev, dtype=bf)
    row_seq = torch.arange(nseq, dtype=torch.int32,
                           device=dev).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=dev).repeat(nseq)
    sink = torch.zeros(H, device=dev)
    keys = sum(min(p + 1, W) for p in range(L)) * nseq     # (row, key) pairs
    t = _time(lambda: ops.latent_attention(
        qa, qr, cache, bt, row_seq, pos, sink, 0.05, sz["window"], T,
        [L] * nseq), 5)
    out["latent_attention_prompt"] = _entry(
        t, flops=2.0 * keys * H * (R + RD + R))
    hd, nkv = 128, max(1, H // 4)
    q = torch.randn(T, H, hd, device=dev, dtype=bf)
    k = torch.randn(T, nkv, hd, device=dev, dtype=bf)
    v = torch.randn(T, nkv, hd, device=dev, dtype=bf)
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.flash_prefill(q, k, v, cu, [L] * nseq, 0.09), 5)
    out["flash_prefill"] = _entry(
        t, flops=4.0 * nseq * (L * (L + 1) / 2) * H * hd)

    # ---- decode attention: 256 sequences at 2048 tokens ----
    B, ctx = 256, 2048
    cache, bt = paged(B, ctx, R + RD)
    qa = torch.randn(B, H, R, device=dev, dtype=bf)
    qr = torch.randn(B, H, RD, device=dev, dtype=bf)
    row_seq = torch.arange(B, dtype=torch.int32, device=dev)
    pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=dev)
    Wd = min(sz["window"], ctx) if sz["window"] else ctx
    t = _time(lambda: ops.latent_attention(
        qa, qr, cache, bt, row_seq, pos, sink, 0.05, sz["window"]))
    out["latent_attention_decode"] = _entry(
        t, flops=2.0 * B * Wd * H * (2 * R + RD),
        bytes_=2.0 * B * Wd * (R + RD))
    kc = torch.randn(B * (ctx // bs) + 1, nkv, bs, hd, device=dev, dtype=bf)
    vc = torch.randn_like(kc)
    ctx_lens = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q = torch.randn(B, H, hd, device=dev, dtype=bf)
    t = _time(lambda: ops.paged_attn_decode(q, kc, vc, bt, ctx_lens, 0.09))
    out["paged_attn_decode"] = _entry(
        t, flops=4.0 * B * ctx * H * hd, bytes_=4.0 * B * ctx * nkv * hd)

    # ---- norms on 8192 rows ----
    T = 8192
    res = torch.randn(T, D, device=dev)
    dl = torch.randn(T, D, device=dev, dtype=bf)
    w, b = torch.ones(D, device=dev), torch.zeros(D, device=dev)
    t = _time(lambda: ops.add_layernorm(res, dl, w, b, 1e-5, bf))
    out["add_layernorm"] = _entry(t, bytes_=T * D * (4 + 4 + 2 + 2.0))
    x = torch.randn(T, D, device=dev, dtype=bf)
    rs = torch.randn(T, D, device=dev, dtype=bf)
    wb = torch.ones(D, device=dev, dtype=bf)
    t = _time(lambda: ops.fused_add_rmsnorm(x, rs, wb, 1e-5))
    out["fused_add_rmsnorm"] = _entry(t, bytes_=T * D * 8.0)

    # ---- activations on [8192, ff] ----
    F_ = sz["ff"]
    z = torch.randn(T, F_, device=dev, dtype=bf)
    pq = torch.zeros(2, device=dev)
    t = _time(lambda: ops.xielu(z, pq))
    out["xielu"] = _entry(t, bytes_=T * F_ * 4.0)
    t = _time(lambda: ops.relu2(z))
    out["relu2"] = _entry(t, bytes_=T * F_ * 4.0)
    gu = torch.randn(T, 2 * F_, device=dev, dtype=bf)
    t = _time(lambda: ops.silu_mul(gu))
    out["silu_mul"] = _entry(t, bytes_=T * F_ * 6.0)

    # ---- recurrence: a prompt burst (chunked scan) and a decode batch ----
    nseq, L = 4, 2048
    T = nseq * L
    zug = torch.randn(T, 3 * D, device=dev, dtype=bf)
    state = torch.zeros(nseq, D, device=dev)
    cu = torch.arange(0, T + 1, L, dtype=torch.int32, device=dev)
    st = torch.zeros(nseq, dtype=torch.int32, device=dev)
    sl = torch.arange(nseq, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.mingru_scan(zug, state, cu, st, sl, [L] * nseq))
    # chunked: the projection is read twice, y written once
    out["mingru_scan_prompt"] = _entry(t, bytes_=T * D * (2 * 6 + 2.0))
    B = 256
    zug = torch.randn(B, 3 * D, device=dev, dtype=bf)
    state = torch.zeros(B, D, device=dev)
    cu = torch.arange(0, B + 1, dtype=torch.int32, device=dev)
    st = torch.ones(B, dtype=torch.int32, device=dev)
    sl = torch.arange(B, dtype=torch.int32, device=dev)
    t = _time(lambda: ops.mingru_scan(zug, state, cu, st, sl, [1] * B))
    out["mingru_scan_decode"] = _entry(t, bytes_=B * D * (6 + 2 + 8.0))

    # ---- routing, 256 rows ----
    lg = torch.randn(256, sz["experts"], device=dev)
    t = _time(lambda: ops.moe_topk_route(lg, sz["top"], 256))
    out["moe_topk_route"] = _entry(t)
    t = _time(lambda: ops.moe_route(lg, sz["top"], 256))
    out["moe_route"] = _entry(t)
    return out


def run(size: str = "2k", batch: int = 64, prompt_len: int = 1024,
        steps: int = 32, warmup: int = 4) -> dict:
    sz = SIZES[size]
    fed, mix = _configs(sz)
    res = {"size": size, "shape": sz, "batch": batch,
           "prompt_len": prompt_len, "steps": steps, "dtype": "bf16",
           "data": "synthetic (random weights and tokens)"}
    res["kernels"] = _kernels(sz)
    res["fedatar"] = _engine_run(fed, batch, prompt_len, steps, warmup)
    res["mixtral"] = _engine_run(mix, batch, prompt_len, steps, warmup)
    return res


if __name__ == "__main__":
    print(json.dumps(run(*(sys.argv[1:2] or ["2k"]))))
