"""Mekevik (parallel-block decoder with windowed sigmoid attention)
against a plain float64 model written from the equations
(tests/mekevik_oracle.py).

Every test builds its own small configuration and random checkpoint; the
engine reads it through the product loader.  Device-parametrized: the CPU
cases run the reference ops, the GPU cases the HIP kernels, both through
the same engine, cache manager and scheduler.
"""
import json
import math
import os
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import mekevik_oracle as oracle
from inference_gateway_amd import ops
from inference_gateway_amd.engine.config import (EngineConfig,
                                                 MekevikConfig,
                                                 SamplingParams,
                                                 distance_bucket)
from inference_gateway_amd.engine.engine import LLMEngine
from inference_gateway_amd.engine.models.registry import \
    model_config_from_dir

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64


def _dev(device):
    return "cuda:0" if device == "cuda" else "cpu"


def make_engine(tmp_path, cfg, W, device, dtype="float32", blocks=40,
                block=4, slots=4, **kw):
    path = oracle.save_checkpoint(Path(tmp_path) / "ckpt", cfg, W)
    ecfg = EngineConfig(
        model=model_config_from_dir(path), block_size=block,
        num_gpu_blocks=blocks, max_num_seqs=slots,
        max_batched_tokens=kw.pop("max_batched_tokens", 4096),
        max_model_len=4096, use_hip_graphs=False, weights_path=path,
        dtype=dtype, **kw)
    return LLMEngine(ecfg, device=_dev(device))


def close(got, ref, tol):
    """Mean-free relative RMS difference per row, like a logit check."""
    got, ref = got.double().cpu(), ref.double().cpu()
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()
    assert float(err.max()) < tol, f"rel err {float(err.max()):.3e}"


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay_all(engine, tokens, cuts):
    """Feed one request in portions `cuts`; returns logits of every
    position [T, vocab]."""
    sid = engine.open_stream()
    out, at = [], 0
    for n in cuts:
        part = tokens[at:at + n]
        out.append(engine.replay_step([(sid, part)],
                                      {sid: list(range(len(part)))}))
        at += n
    assert at == len(tokens)
    engine.close_stream(sid)
    return torch.cat(out)


# ---------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,far", [(32, 128), (10, 30), (2, 5), (64, 512),
                                      (12, 40.0), (6, 1000)])
def test_distance_buckets(rows, far):
    """Identity below rows/2, monotone, last row from `far` on, and the
    same rows as the plain formula."""
    got = [distance_bucket(n, rows, far) for n in range(int(far) + 40)]
    assert got == [oracle.distance_bucket(n, rows, far)
                   for n in range(int(far) + 40)]
    assert got[:rows // 2] == list(range(rows // 2))
    assert all(a <= b for a, b in zip(got, got[1:]))
    assert all(g == rows - 1 for g in got[int(math.ceil(far)):])
    assert max(got) == rows - 1


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("D", [48, 257, 1024])
def test_add_rmsnorm_pair(device, D):
    """residual += a + b once; both outputs from the same statistic;
    eps inside the root."""
    dev = _dev(device)
    g = torch.Generator().manual_seed(D)
    T, eps = 5, 1e-3
    res = torch.randn(T, D, generator=g) * 3
    a = torch.randn(T, D, generator=g)
    b = torch.randn(T, D, generator=g)
    w1 = torch.randn(D, generator=g)
    w2 = torch.randn(D, generator=g)
    x = res.to(F64) + a.to(F64) + b.to(F64)
    n1 = oracle.rms_norm(x, w1.to(F64), eps)
    n2 = oracle.rms_norm(x, w2.to(F64), eps)
    r = res.clone().to(dev)
    o1, o2 = ops.add_rmsnorm_pair(r, a.to(dev), b.to(dev), w1.to(dev),
                                  w2.to(dev), eps, torch.float32)
    assert torch.allclose(r.cpu().double(), x, atol=1e-5)
    assert torch.allclose(o1.cpu().double(), n1, atol=2e-5)
    assert torch.allclose(o2.cpu().double(), n2, atol=2e-5)
    # one delta, no delta, one output
    r = res.clone().to(dev)
    o1, o2 = ops.add_rmsnorm_pair(r, None, b.to(dev), w1.to(dev), None,
                                  eps, torch.float32)
    assert o2 is None
    assert torch.allclose(o1.cpu().double(), oracle.rms_norm(
        res.to(F64) + b.to(F64), w1.to(F64), eps), atol=2e-5)
    r = res.clone().to(dev)
    o1, _ = ops.add_rmsnorm_pair(r, None, None, w1.to(dev), None, eps,
                                 torch.float32)
    assert torch.equal(r.cpu(), res)
    assert torch.allclose(o1.cpu().double(), oracle.rms_norm(
        res.to(F64), w1.to(F64), eps), atol=2e-5)


def _paged_layout(T, bs, seed, extra=3):
    """A shuffled page order for T tokens: (block table row, slots)."""
    nb = (T + bs - 1) // bs
    g = torch.Generator().manual_seed(seed)
    pages = (torch.randperm(nb + extra, generator=g)[:nb] + 1).tolist()
    slots = [pages[j // bs] * bs + j % bs for j in range(T)]
    return pages, slots, nb + extra + 1


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 12, 10), (1, 1, 5, 7),
                                       (6, 6, 8, 8), (3, 1, 70, 33),
                                       (4, 2, 16, 8)])
def test_qk_norm_append(device, H, G, dk, dv):
    """Norm statistics span ALL heads of q (and of k); values are blended
    before they are paged; extra projection columns are left alone."""
    dev = _dev(device)
    g = torch.Generator().manual_seed(H * 100 + dk)
    T, bs, eps, lam = 7, 4, 1e-4, 0.3125
    nq, nk, nv = H * dk, G * dk, G * dv
    # the last case keeps rows 16-byte aligned (the vector path)
    proj = torch.randn(T, nq + nk + nv + (4 if dk == 16 else 5),
                       generator=g) * 2
    wq = torch.randn(nq, generator=g)
    wk = torch.randn(nk, generator=g)
    vf = torch.randn(T, nv + 3, generator=g)[:, 1:1 + nv]   # strided rows
    pages, slots, nblocks = _paged_layout(T, bs, 5)
    P = proj.to(F64)
    q_ref = oracle.rms_norm(P[:, :nq], wq.to(F64), eps)
    k_ref = oracle.rms_norm(P[:, nq:nq + nk], wk.to(F64), eps)
    v_raw = P[:, nq + nk:nq + nk + nv]
    for blend in (False, True):
        v_ref = ((1 - lam) * v_raw + lam * vf.to(F64)) if blend else v_raw
        kc = torch.zeros(nblocks, G, bs, dk, device=dev)
        vc = torch.zeros(nblocks, G, dv, bs, device=dev)
        q = ops.qk_norm_append(
            proj.to(dev), torch.tensor(slots, dtype=torch.int32, device=dev),
            kc, vc, wq.to(dev), wk.to(dev),
            vf.to(dev) if blend else None, lam, eps, H, G, dk, dv)
        assert torch.allclose(q.cpu().double(), q_ref, atol=3e-5)
        for t, s in enumerate(slots):
            kk = kc[s // bs, :, s % bs].reshape(-1).cpu().double()
            vv = vc[s // bs, :, :, s % bs].reshape(-1).cpu().double()
            assert torch.allclose(kk, k_ref[t], atol=3e-5)
            assert torch.allclose(vv, v_ref[t], atol=3e-5)
        # nothing else was written
        written = torch.zeros(nblocks * bs, dtype=torch.bool)
        written[slots] = True
        flat = kc.permute(0, 2, 1, 3).reshape(nblocks * bs, -1).cpu()
        assert float(flat[~written].abs().max()) == 0.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_qk_norm_append_many_rows(device, dtype):
    """A prompt-sized batch: runs of consecutive slots that start on and
    off 8-token boundaries, a run cut by the end of the batch, and
    scattered slots, all land in the right place of the transposed
    value pages."""
    dev = _dev(device)
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(77)
    H, G, dk, dv, bs, eps, lam = 8, 8, 16, 136, 16, 1e-5, 0.25
    T = 1030
    nq, nk, nv = H * dk, G * dk, G * dv     # nv wide enough for the
    #                                         staged-store path on the GPU
    proj = (torch.randn(T, nq + nk + nv + 8, generator=g) * 2).to(dt)
    vf = torch.randn(T, nv, generator=g).to(dt)
    wq = torch.randn(nq, generator=g)
    wk = torch.randn(nk, generator=g)
    nblocks = 200
    slots = list(range(16, 16 + 600))                  # aligned run
    slots += list(range(16 * 60 + 3, 16 * 60 + 3 + 200))   # off by three
    free = torch.randperm(16 * 100, generator=g)[:T - 800] + 16 * 90
    slots += free.tolist()                             # scattered
    assert len(slots) == T and len(set(slots)) == T
    P = proj.to(F64)
    qn = P[:, :nq]
    q_ref = qn / torch.sqrt((qn ** 2).mean(-1, keepdim=True) + eps) * wq
    kn = P[:, nq:nq + nk]
    k_ref = kn / torch.sqrt((kn ** 2).mean(-1, keepdim=True) + eps) * wk
    v_ref = (1 - lam) * P[:, nq + nk:nq + nk + nv] + lam * vf.to(F64)
    kc = torch.zeros(nblocks, G, bs, dk, device=dev, dtype=dt)
    vc = torch.zeros(nblocks, G, dv, bs, device=dev, dtype=dt)
    q = ops.qk_norm_append(
        proj.to(dev), torch.tensor(slots, dtype=torch.int32, device=dev), kc,
        vc, wq.to(dev), wk.to(dev), vf.to(dev), lam, eps, H, G, dk, dv)
    tol = 3e-5 if dtype == "float32" else 4e-2
    st = torch.tensor(slots)
    got_k = kc.cpu()[st // bs, :, st % bs].reshape(T, nk).double()
    got_v = vc.cpu()[st // bs, :, :, st % bs].reshape(T, nv).double()
    assert float((q.cpu().double() - q_ref).abs().max()) < tol
    assert float((got_k - k_ref).abs().max()) < tol
    assert float((got_v - v_ref).abs().max()) < tol
    # nothing else was written
    mask = torch.ones(nblocks * bs, dtype=torch.bool)
    mask[st] = False
    flat = vc.cpu().permute(0, 3, 1, 2).reshape(nblocks * bs, -1)
    assert float(flat[mask].abs().max()) == 0.0


def _attention_case(H, G, dk, dv, T, bs, window, rows, far, seed, dev,
                    dtype=torch.float32):
    """Random q/k/v of one sequence, paged in shuffled order.  Returns the
    op's arguments and the float64 inputs for the plain model."""
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(T, H, dk, generator=g)).to(dtype)
    k = (torch.randn(T, G, dk, generator=g)).to(dtype)
    v = (torch.randn(T, G, dv, generator=g)).to(dtype)
    gate = (torch.randn(T, H * dv + 2, generator=g) * 2).to(dtype)
    rel = torch.randn(rows, H, generator=g)
    pb = torch.randn(H, generator=g) - 1.0
    talk = torch.eye(H) * 0.7 + torch.randn(H, H, generator=g) * 0.3
    pages, slots, nblocks = _paged_layout(T, bs, seed + 1)
    kc = torch.zeros(nblocks, G, bs, dk, dtype=dtype)
    vc = torch.zeros(nblocks, G, dv, bs, dtype=dtype)
    for j, s in enumerate(slots):
        kc[s // bs, :, s % bs] = k[j]
        vc[s // bs, :, :, s % bs] = v[j]
    nd = int(math.ceil(far)) + 1
    nd = min(nd, window) if window else nd
    bias = torch.stack([rel[distance_bucket(n, rows, far)] + pb
                        for n in range(nd)])
    args = dict(
        q=q.reshape(T, H * dk).to(dev), kcache=kc.to(dev),
        vcache=vc.to(dev),
        block_table=torch.tensor([[0] * len(pages), pages],
                                 dtype=torch.int32, device=dev),
        row_seq=torch.ones(T, dtype=torch.int32, device=dev),
        positions=torch.arange(T, dtype=torch.int32, device=dev),
        dist_bias=bias.to(dev), talk=talk.to(dev),
        gate=gate.to(dev)[:, 1:1 + H * dv])
    plain = dict(q=q.to(F64), k=k.to(F64), v=v.to(F64),
                 gate=gate.to(F64)[:, 1:1 + H * dv], rel=rel.to(F64),
                 pb=pb.to(F64), talk=talk.to(F64))
    return args, plain


def _attention_plain(p, rows_at, window, far, scale):
    out = []
    for t in rows_at:
        o = oracle.attention_row(p["q"][t], p["k"], p["v"], t, window,
                                 p["rel"], far, p["pb"], p["talk"], scale)
        out.append(o.reshape(-1) * oracle.logistic(p["gate"][t]))
    return torch.stack(out)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,dk,dv,window,rows,far", [
    (4, 2, 12, 10, 9, 10, 30),      # window shorter than the table
    (1, 1, 5, 7, 1, 2, 3),          # sees only itself
    (6, 6, 8, 8, 0, 8, 20),         # no window: distances clamp at far
    (3, 1, 70, 33, 37, 6, 11),      # one kv head, window over the clamp
    (8, 2, 16, 16, 50, 24, 200),
])
def test_sigmoid_attention_op(device, H, G, dk, dv, window, rows, far):
    """Every row of a 45-token sequence (a whole prompt to the op) and
    the same rows one by one (decoding), pages in shuffled order."""
    dev = _dev(device)
    T, bs, scale = 45, 4, 1.3 / math.sqrt(dk)
    a, p = _attention_case(H, G, dk, dv, T, bs, window, rows, far,
                           7 * H + dk, dev)
    ref = _attention_plain(p, range(T), window, far, scale)
    got = ops.sigmoid_attention(
        a["q"], a["kcache"], a["vcache"], a["block_table"], a["row_seq"],
        a["positions"], a["dist_bias"], a["talk"], a["gate"], scale, window,
        T, [T])
    assert torch.allclose(got.cpu().double(), ref, atol=5e-5, rtol=1e-5)
    for t in (0, 1, window, T - 1):
        t = min(t, T - 1)
        got1 = ops.sigmoid_attention(
            a["q"][t:t + 1], a["kcache"], a["vcache"], a["block_table"],
            a["row_seq"][t:t + 1], a["positions"][t:t + 1], a["dist_bias"],
            a["talk"], a["gate"][t:t + 1], scale, window)
        assert torch.allclose(got1.cpu().double(), ref[t:t + 1], atol=5e-5,
                              rtol=1e-5)


CRAFTED = [("cpu", "float32", w) for w in ("prompt", "decode")] + [
    pytest.param("cuda", t, w, marks=pytest.mark.gpu)
    for t in ("float32", "bfloat16") for w in ("prompt", "decode")]


@pytest.mark.parametrize("device,dtype,where", CRAFTED)
def test_sigmoid_attention_far_key_window_and_page_edges(device, dtype,
                                                         where):
    """All weights are pushed to ~0 by a large negative offset except
    ONE key whose score is boosted; the output is then that key's value
    (through the head mixing) if the key is visible and ~0 if not.  Keys:
    far back among hundreds (no window), the last one inside and the
    first one outside a window, the first token, and both sides of a
    page border."""
    dev = _dev(device)
    dt = getattr(torch, dtype)
    H, G, dk, dv, bs = 4, 2, 16, 8, 16
    T = 700
    tol = 2e-2 if dtype == "bfloat16" else 1e-3
    for window, target, qpos, visible in [
            (0, 3, 699, True),          # far key, everything visible
            (0, 0, 650, True),          # the very first token
            (64, 400 - 63, 400, True),  # last key inside the window
            (64, 400 - 64, 400, False),  # first key outside it
            (33, 207, 239, True),       # window edge at a page's end
            (33, 208, 240, True),       # ... and at a page's start
            (33, 207, 240, False),
            (1, 300, 300, True),        # sees only itself
            (1, 299, 300, False)]:
        a, p = _attention_case(H, G, dk, dv, T, bs, window, 8, 50, 99, dev,
                               dt)
        # offset -18 everywhere; the boosted pair scores +28, every
        # other key 0 (entry 5 of all other keys is cleared)
        a["dist_bias"] = torch.full_like(a["dist_bias"], -18.0)
        a["kcache"][..., 5] = 0
        qd = torch.zeros(H, dk)
        qd[:, 5] = 7.0
        kd = torch.zeros(G, dk)
        kd[:, 5] = 4.0
        a["q"][qpos] = qd.reshape(-1).to(dt)
        slot_row = a["block_table"][1, target // bs].item()
        a["kcache"][slot_row, :, target % bs] = kd.to(dt).to(dev)
        talk = a["talk"].double().cpu()
        v_t = a["vcache"][slot_row, :, :, target % bs].double().cpu()
        per = H // G
        want = torch.stack([talk[h].sum() * v_t[h // per] for h in range(H)])
        want = want.reshape(-1) * oracle.logistic(
            a["gate"][qpos].double().cpu())
        if not visible:
            want = torch.zeros_like(want)
        if where == "prompt":
            lo = max(0, qpos - 20)
            rows = slice(lo, qpos + 1)
            got = ops.sigmoid_attention(
                a["q"][rows], a["kcache"], a["vcache"], a["block_table"],
                a["row_seq"][rows], a["positions"][rows], a["dist_bias"],
                a["talk"], a["gate"][rows], 1.0, window, qpos + 1 - lo,
                [qpos + 1 - lo])[-1]
        else:
            rows = slice(qpos, qpos + 1)
            got = ops.sigmoid_attention(
                a["q"][rows], a["kcache"], a["vcache"], a["block_table"],
                a["row_seq"][rows], a["positions"][rows], a["dist_bias"],
                a["talk"], a["gate"][rows], 1.0, window)[0]
        err = float((got.double().cpu() - want).abs().max())
        assert err < tol, (window, target, qpos, visible, err)
        if visible:
            assert float(want.abs().max()) > 0.05


@pytest.mark.parametrize("device", DEVICES)
def test_gated_activations_and_route(device):
    dev = _dev(device)
    g = torch.Generator().manual_seed(3)
    for f in (7, 64):
        z = torch.randn(9, 2 * f, generator=g) * 3
        gate, up = z[:, :f].to(F64), z[:, f:].to(F64)
        silu = gate * oracle.logistic(gate) * up
        got = ops.gated_act(z.to(dev), ops.GATED_ACT_SILU)
        assert torch.allclose(got.cpu().double(), silu, atol=1e-5)
        lim, alpha = 1.25, 1.702
        gc = torch.clamp(gate, max=lim)
        uc = torch.clamp(up, -lim, lim)
        ref = gc * oracle.logistic(alpha * gc) * (uc + 1)
        got = ops.gated_act(z.to(dev), ops.GATED_ACT_CLAMPED, lim, alpha)
        assert torch.allclose(got.cpu().double(), ref, atol=1e-5)
        # the clamp is one-sided for the gate: a very negative gate stays
        assert float(got.min()) < -0.1 or f == 7
    # routing: softmax over ALL experts, top-k renormalised, scaled
    T, E = 33, 7
    logits = torch.randn(T, E, generator=g) * 2
    for K in (1, 3, 7):
        w, idx, _ = ops.moe_topk_route(logits.to(dev), K, 0, 2.5)
        s = torch.softmax(logits.to(F64), -1)
        for t in range(T):
            order = sorted(range(E), key=lambda e: -float(s[t, e]))[:K]
            assert sorted(idx[t].tolist()) == sorted(order)
            tot = sum(float(s[t, e]) for e in order) + 1e-20
            for k in range(K):
                e = int(idx[t, k])
                assert abs(float(w[t, k]) - float(s[t, e]) / tot * 2.5) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [7, 300])
def test_feed_forward_modules(tmp_path, device, T):
    """The dense unit and the routed experts as the engine's modules
    (both dispatch routes of the experts) against the plain functions."""
    cfg = oracle.make_config(pattern=("d", "m"))
    W = oracle.make_weights(cfg, seed=5)
    eng = make_engine(tmp_path, cfg, W, device)
    W64 = {k: v.to(F64) for k, v in W.items()}
    g = torch.Generator().manual_seed(T)
    h = torch.randn(T, cfg["width"], generator=g)
    hd = h.to(_dev(device))
    with torch.inference_mode():
        dense = eng.model.layers[0].mlp(hd, None)
        routed = eng.model.layers[1].mlp(hd, None)
    close(dense, oracle.clamped_glu_ff(h.to(F64), W64, "l0.mlp.",
                                       cfg["layers"][0]["mlp"]), 2e-5)
    close(routed, oracle.routed_ff(h.to(F64), W64, "l1.mlp.",
                                   cfg["layers"][1]["mlp"]), 2e-5)


# ---------------------------------------------------------------------------
# whole model through the engine
# ---------------------------------------------------------------------------
CONFIGS = {
    # all feed-forward kinds, sizes all different, every layer blends
    "mixed": dict(),
    # values that happen to be 1 or equal elsewhere: one head, one kv
    # head, top = all experts, window of one token, two-row bias table,
    # blending starts at the second layer, scales of one
    "ones": dict(width=32, vocab=50, pattern=("m", "d", "-", "m"), heads=1,
                 kv_heads=1, dim=6, vdim=5, window=1, ff=20, experts=3,
                 top=3, expert_ff=8, bias_rows=2, bias_max=4,
                 v_mix=(False, True, False, True), embed_scale=1.0,
                 logit_scale=1.0, router_scale=1.0),
    # full attention (no window) past the last bias row, kv heads = heads,
    # one expert chosen of many, no blending at all, dim == vdim
    "full": dict(width=40, vocab=61, pattern=("-", "m", "d"), heads=2,
                 kv_heads=2, dim=8, vdim=8, window=0, ff=24, experts=9,
                 top=1, expert_ff=10, bias_rows=6, bias_max=13,
                 v_mix=(False,)),
    # window longer than the table's reach, many heads on one kv head
    "wide": dict(width=64, vocab=70, pattern=("d", "d"), heads=6,
                 kv_heads=1, dim=10, vdim=12, window=30, bias_rows=8,
                 bias_max=12, v_mix=(True, True)),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_decode_and_portions(tmp_path, device, name):
    """One request four ways — whole, token by token, ragged portions
    down to two tokens — all equal to the plain model at every
    position."""
    cfg = oracle.make_config(**CONFIGS[name])
    W = oracle.make_weights(cfg, seed=11)
    T = 41
    tokens = toks(T, cfg["vocab"], 12)
    ref = oracle.forward(cfg, W, tokens)
    eng = make_engine(tmp_path, cfg, W, device)
    close(replay_all(eng, tokens, [T]), ref, 2e-5)
    close(replay_all(eng, tokens, [1] * T), ref, 2e-5)
    close(replay_all(eng, tokens, [2, 3, 1, 7, 2, 9, 5, 2, 10]), ref, 2e-5)
    close(replay_all(eng, tokens, [16, 1, 1, 1, 8, 14]), ref, 2e-5)
    # every page and slot went back to the pools
    assert eng.block_manager.num_free == eng.block_manager.num_blocks - 1
    assert len(eng.scheduler._free_slots) == eng.cfg.max_num_seqs


@pytest.mark.parametrize("device", DEVICES)
def test_layer_taps_match(tmp_path, device):
    """The residual stream after every layer, not just the logits."""
    cfg = oracle.make_config()
    W = oracle.make_weights(cfg, seed=13)
    tokens = toks(17, cfg["vocab"], 14)
    taps_ref, taps = [], []
    oracle.forward(cfg, W, tokens, taps_ref)
    eng = make_engine(tmp_path, cfg, W, device)
    eng.model.tap = lambda i, x: taps.append(x.clone())
    replay_all(eng, tokens, [len(tokens)])
    assert len(taps) == len(taps_ref) == len(cfg["layers"])
    for a, b in zip(taps, taps_ref):
        close(a, b, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_passes_window_and_pages(tmp_path, device):
    """A short prompt, then 70 single tokens: the window (9) slides over
    decoded tokens only, across many 4-token pages."""
    cfg = oracle.make_config()
    W = oracle.make_weights(cfg, seed=15)
    tokens = toks(76, cfg["vocab"], 16)
    ref = oracle.forward(cfg, W, tokens)
    eng = make_engine(tmp_path, cfg, W, device)
    close(replay_all(eng, tokens, [6] + [1] * 70), ref, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_reuse_pages_and_slots(tmp_path, device):
    """Five unequal requests over four slots and a pool too small for
    all of them at once: portions of some beside single tokens of
    others, requests ending and new ones taking their pages and slots.
    Each must equal itself alone."""
    cfg = oracle.make_config()
    W = oracle.make_weights(cfg, seed=17)
    lens = {"a": 30, "b": 9, "c": 23, "d": 2, "e": 26}
    reqs = {k: toks(n, cfg["vocab"], 20 + i)
            for i, (k, n) in enumerate(lens.items())}
    refs = {k: oracle.forward(cfg, W, v) for k, v in reqs.items()}
    # 4-token pages; live at most a+b+c+d = 8+3+6+1 = 18 pages
    eng = make_engine(tmp_path, cfg, W, device, blocks=20, slots=4)
    schedule = [
        [("a", 7), ("b", 1)],
        [("a", 1), ("b", 3), ("c", 11)],
        [("b", 1), ("c", 2), ("d", 2)],           # d ends
        [("a", 13), ("b", 4), ("c", 1)],          # b ends
        [("a", 1), ("c", 1), ("e", 5)],           # e: b's or d's slot
        [("e", 1), ("a", 8), ("c", 8)],           # a, c end
        [("e", 19)],
        [("e", 1)],
    ]
    sids, at, got = {}, {k: 0 for k in reqs}, {k: [] for k in reqs}
    seen_slots, seen_pages = {}, {}
    for step in schedule:
        feeds, want = [], {}
        for k, n in step:
            if k not in sids:
                sids[k] = eng.open_stream()
            part = reqs[k][at[k]:at[k] + n]
            feeds.append((sids[k], part))
            want[sids[k]] = list(range(n))
            at[k] += n
        out = eng.replay_step(feeds, want)
        row = 0
        for k, n in step:
            got[k].append(out[row:row + n])
            row += n
            seen_slots.setdefault(k, eng._seqs[sids[k]].slot)
            seen_pages.setdefault(k, set()).update(
                eng._seqs[sids[k]].block_ids)
        for k, _n in step:
            if at[k] == lens[k] and k in sids:
                eng.close_stream(sids.pop(k))
    assert at == lens
    assert seen_slots["e"] in (seen_slots["b"], seen_slots["d"])
    assert seen_pages["e"] & (seen_pages["a"] | seen_pages["b"]
                              | seen_pages["c"] | seen_pages["d"])
    for k in reqs:
        close(torch.cat(got[k]), refs[k], 2e-5)
    assert eng.block_manager.num_free == eng.block_manager.num_blocks - 1


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_serving_precision(tmp_path, device):
    """The bf16 mode keeps the residual, norms, scores and weights in
    fp32: whole prompt, portions and decoding stay within bf16 rounding
    of the plain model and of each other.  (No routed layer here: a
    rounding that flips a near-tie between two experts is a different,
    legitimate answer and not a precision fault.)"""
    cfg = oracle.make_config(pattern=("d", "-", "d"))
    W = oracle.make_weights(cfg, seed=21)
    tokens = toks(37, cfg["vocab"], 22)
    ref = oracle.forward(cfg, W, tokens)
    eng = make_engine(tmp_path, cfg, W, device, dtype="bfloat16")
    whole = replay_all(eng, tokens, [37])
    close(whole, ref, 4e-2)
    close(replay_all(eng, tokens, [5, 2, 9, 1, 1, 19]), ref, 4e-2)
    close(replay_all(eng, tokens, [1] * 37), ref, 4e-2)


def _greedy_ref(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(oracle.forward(cfg, W, seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode", ["plain", "chunked_mixed"])
def test_greedy_generation(tmp_path, device, mode):
    """Greedy decoding through add_request / step — the engine's own
    scheduler, batching and sampler — equals argmax of the plain model
    re-run from scratch at every token."""
    cfg = oracle.make_config()
    W = oracle.make_weights(cfg, seed=23)
    kw = {}
    if mode == "chunked_mixed":
        kw = dict(enable_chunked_prefill=True, enable_mixed_batches=True,
                  max_batched_tokens=8)
    eng = make_engine(tmp_path, cfg, W, device, blocks=60, **kw)
    prompts = [toks(n, cfg["vocab"], 30 + n) for n in (5, 19, 11)]
    n_new = 7
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=n_new,
                                             temperature=0.0))
           for p in prompts]
    steps = 0
    while not eng.is_finished() and steps < 400:
        eng.step()
        steps += 1
    assert eng.is_finished()
    for sid, p in zip(ids, prompts):
        assert eng.get_output(sid).token_ids == _greedy_ref(cfg, W, p, n_new)
    assert eng.block_manager.num_free == eng.block_manager.num_blocks - 1


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_recomputes_the_cache(tmp_path, device):
    """A pool too small for both requests' decoding: one is preempted,
    its pages go back, and its folded prompt is run again; the tokens
    are still the plain model's."""
    cfg = oracle.make_config(pattern=("d", "m"))
    W = oracle.make_weights(cfg, seed=25)
    eng = make_engine(tmp_path, cfg, W, device, blocks=9, slots=2)
    prompts = [toks(9, cfg["vocab"], 41), toks(10, cfg["vocab"], 42)]
    n_new = 8
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=n_new,
                                             temperature=0.0))
           for p in prompts]
    steps = 0
    while not eng.is_finished() and steps < 400:
        eng.step()
        steps += 1
    assert eng.is_finished()
    for sid, p in zip(ids, prompts):
        assert eng.get_output(sid).token_ids == _greedy_ref(cfg, W, p, n_new)


@pytest.mark.parametrize("device", DEVICES)
def test_prefix_cache_reuses_blended_values(tmp_path, device):
    """Nothing is kept per sequence outside the pages (the cached values
    are already blended), so a shared prompt prefix can be served from
    another request's pages."""
    cfg = oracle.make_config(pattern=("d", "m"))
    W = oracle.make_weights(cfg, seed=27)
    eng = make_engine(tmp_path, cfg, W, device, blocks=40,
                      enable_prefix_caching=True)
    shared = toks(12, cfg["vocab"], 51)
    prompts = [shared + toks(3, cfg["vocab"], 52),
               shared + toks(5, cfg["vocab"], 53)]
    outs = []
    for p in prompts:
        sid = eng.add_request(p, SamplingParams(max_new_tokens=4,
                                                temperature=0.0))
        steps = 0
        while not eng.is_finished() and steps < 100:
            eng.step()
            steps += 1
        outs.append(eng.get_output(sid).token_ids)
    for p, o in zip(prompts, outs):
        assert o == _greedy_ref(cfg, W, p, 4)


def test_config_reader_and_registry(tmp_path):
    cfg = oracle.make_config(**CONFIGS["ones"])
    W = oracle.make_weights(cfg, seed=1)
    path = oracle.save_checkpoint(Path(tmp_path) / "m", cfg, W)
    mc = model_config_from_dir(path)
    assert isinstance(mc, MekevikConfig)
    a = mc.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window) == (1, 1, 6, 5, 1)
    assert a.bias_rows == 2 and a.bias_far == 4 and a.v_mix is False
    assert mc.layers[1].mixer.v_mix is True
    assert mc.layers[2].mlp is None
    assert mc.layers[0].mlp.top == 3 and mc.layers[0].mlp.scale == 1.0
    assert mc.layers[1].mlp.limit == 0.8
    assert (mc.embed_scale, mc.logit_scale) == (1.0, 1.0)
    # no mask entry: full attention
    full = oracle.make_config(**CONFIGS["full"])
    p2 = oracle.save_checkpoint(Path(tmp_path) / "f", full,
                                oracle.make_weights(full, seed=2))
    m2 = model_config_from_dir(p2)
    assert m2.layers[0].mixer.window == 0
    assert m2.layers[0].mixer.bias_distances() == 14
    bad = dict(full, layers=[dict(full["layers"][0], type="conv")])
    with pytest.raises(ValueError):
        MekevikConfig.from_dict(bad)


def test_loader_rejects_wrong_shapes(tmp_path):
    cfg = oracle.make_config(pattern=("d",))
    W = oracle.make_weights(cfg, seed=3)
    W["l0.mix.talk"] = W["l0.mix.talk"][:, :-1]
    with pytest.raises(ValueError):
        make_engine(tmp_path, cfg, W, "cpu")


def test_trace_runner_command(tmp_path):
    """bin/trace_run end to end on a small checkpoint: chooses the model
    by config.json, answers every step, writes logits in entry order."""
    cfg = oracle.make_config(pattern=("d", "m"))
    W = oracle.make_weights(cfg, seed=29)
    path = oracle.save_checkpoint(Path(tmp_path) / "ckpt", cfg, W)
    a, b = toks(21, cfg["vocab"], 61), toks(6, cfg["vocab"], 62)
    ra, rb = oracle.forward(cfg, W, a), oracle.forward(cfg, W, b)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:9],
                                 "want": [0, 8]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]},
                                {"id": "b", "tokens": b[:4], "want": [3]}],
         "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[4:], "want": []}],
         "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[10:],
                                 "want": [10]}], "end": ["a"]},
    ]
    out = Path(tmp_path) / "out"
    root = Path(__file__).resolve().parent.parent
    env = dict(os.environ, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    r = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", path,
         "--dtype", "float32", "--out", str(out), "--max-tokens", "128"],
        input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
        capture_output=True, env=env, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [
        f"done {i}" for i in range(4)]
    import numpy as np

    V = cfg["vocab"]
    s0 = torch.from_numpy(np.fromfile(out / "0.f32", "<f4").reshape(-1, V))
    close(s0, ra[[0, 8]], 2e-5)
    s1 = torch.from_numpy(np.fromfile(out / "1.f32", "<f4").reshape(-1, V))
    close(s1, torch.stack([ra[9], rb[3]]), 2e-5)
    assert not (out / "2.f32").exists()
    s3 = torch.from_numpy(np.fromfile(out / "3.f32", "<f4").reshape(-1, V))
    close(s3, ra[20:21], 2e-5)


# ---------------------------------------------------------------------------
# the bf16 matrix-core attention kernel (GPU only; pages of 8 or 16)
# ---------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,dk,dv,window,bs,T", [
    (4, 2, 16, 16, 9, 8, 70),        # one head per wave, waves idle
    (8, 4, 40, 24, 37, 16, 150),     # dk not a multiple of 32
    (6, 3, 24, 40, 0, 16, 100),      # no window, dv not a multiple of 16
    (1, 1, 8, 8, 1, 8, 40),          # sees only itself
    (16, 4, 64, 64, 33, 16, 120),    # two heads per wave
    (32, 8, 128, 128, 50, 16, 90),   # four heads per wave, value split
    (24, 24, 32, 96, 64, 16, 130),   # three heads per wave, kv = heads
])
def test_sigmoid_attention_mfma(H, G, dk, dv, window, bs, T):
    """Prompt portions with a cached prefix, whole prompts and decoded
    rows in ONE launch, against the plain model on the same bf16 inputs."""
    dev = "cuda:0"
    rows_tab, far = 12, 45
    scale = 1.3 / math.sqrt(dk)
    a, p = _attention_case(H, G, dk, dv, T, bs, window, rows_tab, far,
                           3 * H + dk, dev, torch.bfloat16)
    start = 21                       # portion = positions [21, T-4)
    dec = [T - 4, T - 1, 5]          # decoded rows, any order
    rows = list(range(start, T - 4)) + dec
    idx = torch.tensor(rows, device=dev)
    ref = _attention_plain(p, rows, window, far, scale)
    got = ops.sigmoid_attention(
        a["q"][idx], a["kcache"], a["vcache"], a["block_table"],
        a["row_seq"][idx], a["positions"][idx], a["dist_bias"], a["talk"],
        a["gate"][idx], scale, window, T - 4 - start, [T - 4 - start], T)
    err = (got.double().cpu() - ref).pow(2).mean().sqrt() / \
        ref.pow(2).mean().sqrt()
    assert float(err) < 1.2e-2, float(err)
    worst = (got.double().cpu() - ref).abs().max() / ref.abs().max()
    assert float(worst) < 4e-2, float(worst)
    # the same rows through the block-per-row kernel agree as well
    ops.SIGMOID_ATTENTION_MFMA = False
    try:
        slow = ops.sigmoid_attention(
            a["q"][idx], a["kcache"], a["vcache"], a["block_table"],
            a["row_seq"][idx], a["positions"][idx], a["dist_bias"],
            a["talk"], a["gate"][idx], scale, window)
    finally:
        ops.SIGMOID_ATTENTION_MFMA = True
    err = (slow.double().cpu() - ref).pow(2).mean().sqrt() / \
        ref.pow(2).mean().sqrt()
    assert float(err) < 6e-3, float(err)


@pytest.mark.gpu
def test_sigmoid_attention_mfma_key_splits():
    """Few rows and many keys: the keys are split over workgroups and
    summed; a long prompt in one launch crosses many tiles."""
    dev = "cuda:0"
    H, G, dk, dv, bs, T = 8, 4, 32, 32, 16, 900
    for window in (0, 700):
        scale = 1.0 / math.sqrt(dk)
        a, p = _attention_case(H, G, dk, dv, T, bs, window, 16, 300, 5, dev,
                               torch.bfloat16)
        a["dist_bias"] = a["dist_bias"] - 3.0   # keep 900-key sums small
        p["pb"] = p["pb"] - 3.0
        rows = [T - 1, 640, 31, 32]
        idx = torch.tensor(rows, device=dev)
        ref = _attention_plain(p, rows, window, 300, scale)
        got = ops.sigmoid_attention(
            a["q"][idx], a["kcache"], a["vcache"], a["block_table"],
            a["row_seq"][idx], a["positions"][idx], a["dist_bias"],
            a["talk"], a["gate"][idx], scale, window, 0, None, T)
        err = (got.double().cpu() - ref).pow(2).mean().sqrt() / \
            ref.pow(2).mean().sqrt()
        assert float(err) < 1.2e-2, (window, float(err))


@pytest.mark.gpu
@pytest.mark.parametrize("block", [8, 16])
def test_bfloat16_engine_on_matrix_cores(tmp_path, block):
    """The bf16 engine with pages the matrix-core kernel accepts: whole
    prompt, ragged portions, decoding and a mixed batch agree with the
    plain model and with each other."""
    cfg = oracle.make_config(pattern=("d", "-", "d"), dim=16, vdim=24,
                             window=19)
    W = oracle.make_weights(cfg, seed=31)
    tokens = toks(75, cfg["vocab"], 32)
    ref = oracle.forward(cfg, W, tokens)
    eng = make_engine(tmp_path, cfg, W, "cuda", dtype="bfloat16",
                      block=block, blocks=40)
    close(replay_all(eng, tokens, [75]), ref, 4e-2)
    close(replay_all(eng, tokens, [5, 2, 30, 1, 1, 17, 19]), ref, 4e-2)
    close(replay_all(eng, tokens, [40] + [1] * 35), ref, 4e-2)
    # two requests side by side: a portion next to single tokens
    a, b = eng.open_stream(), eng.open_stream()
    outs = []
    eng.replay_step([(a, tokens[:30])], {})
    for n in range(5):
        outs.append(eng.replay_step(
            [(b, tokens[9 * n:9 * n + 9]), (a, tokens[30 + n:31 + n])],
            {a: [0]}))
    close(torch.cat(outs), ref[30:35], 4e-2)
    eng.close_stream(a)
    eng.close_stream(b)


def test_local_provider_serves_a_checkpoint_directory(tmp_path):
    """The gateway's local provider with LOCAL_MODEL=hf picks the
    architecture from the directory's config.json and generates through
    the async engine; the preset name works the same way."""
    import asyncio

    from inference_gateway_amd.config import LocalConfig
    from inference_gateway_amd.providers.local import LocalProvider

    cfg = oracle.make_config(vocab=300, pattern=("d", "m"))
    W = oracle.make_weights(cfg, seed=35)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    lc = LocalConfig(enabled=True, model="hf", max_num_seqs=4,
                     max_model_len=128)
    lc.num_gpu_blocks = 64
    lc.weights_path = path
    provider = LocalProvider(lc, device="cpu")
    try:
        assert isinstance(provider.engine.engine.cfg.model, MekevikConfig)

        async def go():
            return await provider.chat_completions({
                "model": "local/hf",
                "messages": [{"role": "user", "content": "hi"}],
                "max_tokens": 3, "temperature": 0})

        body = asyncio.run(go())
        assert body["usage"]["completion_tokens"] == 3
    finally:
        provider.engine.shutdown()


def test_preset_generates():
    eng = LLMEngine(EngineConfig.tiny_mekevik(), device="cpu")
    sid = eng.add_request(list(range(1, 30)),
                          SamplingParams(max_new_tokens=5, temperature=0.0))
    steps = 0
    while not eng.is_finished() and steps < 50:
        eng.step()
        steps += 1
    assert len(eng.get_output(sid).token_ids) == 5
