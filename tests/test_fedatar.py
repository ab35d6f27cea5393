"""Fedatar (hybrid minGRU / latent-attention decoder) against a plain
float64 model written from the equations (tests/fedatar_oracle.py).

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

import fedatar_oracle as oracle
from inference_gateway_amd import ops
from inference_gateway_amd.engine.config import (EngineConfig,
                                                 FedatarConfig,
                                                 SamplingParams)
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
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("D", [48, 257])
def test_layernorm_residual(device, D):
    g = torch.Generator().manual_seed(1)
    res = torch.randn(7, D, generator=g) * 3 + 1
    delta = torch.randn(7, D, generator=g)
    w, b = torch.randn(D, generator=g), torch.randn(D, generator=g)
    ref = oracle.layer_norm((res + delta).to(F64), w.to(F64), b.to(F64),
                            1e-5)
    r = res.clone().to(device)
    out = ops.add_layernorm(r, delta.to(device), w.to(device),
                            b.to(device), 1e-5, torch.float32)
    torch.testing.assert_close(out.cpu().double(), ref, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(r.cpu(), res + delta)
    # no delta: the stream is normed as it is
    out = ops.add_layernorm(r, None, w.to(device), b.to(device), 1e-5,
                            torch.float32)
    torch.testing.assert_close(out.cpu().double(), ref, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("rows", [[5, 1, 9, 1], [300, 2], [1, 1, 1]])
@pytest.mark.parametrize("W", [37, 40])
def test_mingru_scan(device, rows, W):
    """Ragged batch: fresh sequences (stale slot content must be
    ignored), continued ones (slot state is the start), and a segment
    long enough for the chunked scan; widths with and without the
    4-channel vector path."""
    g = torch.Generator().manual_seed(2)
    T, S = sum(rows), len(rows)
    zug = torch.randn(T, 3 * W, generator=g) * 2
    state = torch.randn(S + 2, W, generator=g)
    slots = list(range(S + 1, 1, -1))[:S]
    starts = [0 if i % 2 == 0 else 7 for i in range(S)]
    cu = [0]
    for n in rows:
        cu.append(cu[-1] + n)
    eye = torch.eye(W, dtype=F64)
    zero = torch.zeros(W, dtype=F64)
    st = state.clone().to(device)
    y = ops.mingru_scan(
        zug.to(device), st,
        torch.tensor(cu, dtype=torch.int32, device=device),
        torch.tensor(starts, dtype=torch.int32, device=device),
        torch.tensor(slots, dtype=torch.int32, device=device), rows)
    for s in range(S):
        seg = zug[cu[s]:cu[s + 1]].to(F64)
        S0 = state[slots[s]].to(F64) if starts[s] > 0 else None
        # identity projections turn the oracle's mixer into the bare scan
        ref_rows, ref_S = [], (zero.clone() if S0 is None else S0)
        for t in range(seg.shape[0]):
            # feed pre-activations straight through identity weights
            z = oracle.logistic(seg[t, :W])
            u = seg[t, W:2 * W]
            cand = torch.where(u >= 0, u + 0.5, oracle.logistic(u))
            ref_S = (1 - z) * ref_S + z * cand
            gg = seg[t, 2 * W:]
            ref_rows.append(ref_S * gg * oracle.logistic(gg))
        torch.testing.assert_close(y[cu[s]:cu[s + 1]].cpu().double(),
                                   torch.stack(ref_rows), atol=3e-5,
                                   rtol=3e-5)
        torch.testing.assert_close(st[slots[s]].cpu().double(), ref_S,
                                   atol=3e-5, rtol=3e-5)
    # untouched slots keep their content
    torch.testing.assert_close(st[0].cpu(), state[0])
    del eye


def test_mingru_oracle_matches_its_own_chunks():
    """The oracle's mixer carried over a cut equals the uncut run (the
    state hand-over the engine tests rely on)."""
    g = torch.Generator().manual_seed(3)
    D, W = 6, 5
    m = [torch.randn(W, D, generator=g).double() for _ in range(3)]
    bz, bx = torch.randn(W).double(), torch.randn(W).double()
    Wo = torch.randn(D, W, generator=g).double()
    h = torch.randn(9, D, generator=g).double()
    full, _ = oracle.mingru(h, m[0], bz, m[1], bx, m[2], Wo)
    a, S = oracle.mingru(h[:4], m[0], bz, m[1], bx, m[2], Wo)
    b, _ = oracle.mingru(h[4:], m[0], bz, m[1], bx, m[2], Wo, S)
    torch.testing.assert_close(torch.cat([a, b]), full)


@pytest.mark.parametrize("device", DEVICES)
def test_latent_down_post_and_rope(device):
    QR, R, RD, H, bs = 11, 13, 6, 3, 4
    g = torch.Generator().manual_seed(4)
    T = 6
    down = torch.randn(T, QR + R + RD + H, generator=g)
    pos = [0, 1, 5, 63, 64, 4097]
    slots = [9, 2, 30, 17, 4, 5]
    wq, wc = torch.randn(QR, generator=g), torch.randn(R, generator=g)
    inv = ops.rotary_inv_freq(321.0, RD)
    cache = torch.zeros(8, bs, R + RD)
    c = cache.clone().to(device)
    cq, gate = ops.latent_down_post(
        down.to(device), torch.tensor(pos, dtype=torch.int32, device=device),
        torch.tensor(slots, dtype=torch.int32, device=device), c,
        wq.to(device), wc.to(device), inv.to(device), 1e-5, QR, R, RD, H)
    d64 = down.to(F64)
    torch.testing.assert_close(
        cq.cpu().double(), oracle.rms_norm(d64[:, :QR], wq.to(F64), 1e-5),
        atol=2e-5, rtol=2e-5)
    lat = oracle.rms_norm(d64[:, QR:QR + R], wc.to(F64), 1e-5)
    flat = c.cpu().double().view(-1, R + RD)
    for t in range(T):
        torch.testing.assert_close(flat[slots[t], :R], lat[t], atol=2e-5,
                                   rtol=2e-5)
        kr = oracle.rotate(d64[t, QR + R:QR + R + RD], pos[t], 321.0, RD)
        torch.testing.assert_close(flat[slots[t], R:], kr, atol=5e-4,
                                   rtol=1e-4)
    torch.testing.assert_close(
        gate.cpu().double(), oracle.logistic(d64[:, QR + R + RD:]),
        atol=1e-6, rtol=1e-6)
    # rows that were not addressed stay zero
    used = torch.zeros(8 * bs, dtype=torch.bool)
    used[slots] = True
    assert float(flat[~used].abs().max()) == 0.0
    # the query side: a slice of every head is turned in place
    x = torch.randn(T, H, 5 + RD, generator=g)
    xr = ops.rope_pairs_(x.clone().to(device),
                         torch.tensor(pos, dtype=torch.int32, device=device),
                         inv.to(device), 5).cpu().double()
    for t in range(T):
        for h in range(H):
            torch.testing.assert_close(xr[t, h, :5], x[t, h, :5].double())
            torch.testing.assert_close(
                xr[t, h, 5:], oracle.rotate(x[t, h, 5:].double(), pos[t],
                                            321.0, RD),
                atol=5e-4, rtol=1e-4)


def _paged(c, kr, bs, order_seed):
    """Scatter rows (c | kr) of one sequence into shuffled pages."""
    n = c.shape[0]
    nb = (n + bs - 1) // bs
    g = torch.Generator().manual_seed(order_seed)
    pages = (torch.randperm(nb + 3, generator=g)[:nb] + 1).tolist()
    cache = torch.randn(nb + 5, bs, c.shape[1] + kr.shape[1], generator=g)
    flat = cache.view(-1, cache.shape[-1])
    for j in range(n):
        flat[pages[j // bs] * bs + j % bs] = torch.cat([c[j], kr[j]])
    return cache, pages


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R,RD,H", [(20, 6, 3), (70, 2, 1), (130, 8, 2)])
def test_latent_attention_op(device, R, RD, H):
    g = torch.Generator().manual_seed(5)
    n, bs = 45, 4
    c = torch.randn(n, R, generator=g)
    kr = torch.randn(n, RD, generator=g)
    cache, pages = _paged(c, kr, bs, 6)
    rows = [0, 1, 3, 4, 8, 9, 31, 44]
    T = len(rows)
    qa = torch.randn(T, H, R, generator=g) * 0.5
    qr = torch.randn(T, H, RD, generator=g)
    sink = torch.randn(H, generator=g)
    bt = torch.tensor([pages], dtype=torch.int32)
    for window in (0, 1, 9):
        out = ops.latent_attention(
            qa.to(device), qr.to(device), cache.to(device), bt.to(device),
            torch.zeros(T, dtype=torch.int32, device=device),
            torch.tensor(rows, dtype=torch.int32, device=device),
            sink.to(device), 0.4, window).cpu().double()
        for i, p in enumerate(rows):
            for h in range(H):
                ref = oracle.absorbed_row(
                    qa[i, h].double(), qr[i, h].double(), c.double(),
                    kr.double(), p, window, sink[h], 0.4)
                torch.testing.assert_close(out[i, h], ref, atol=3e-5,
                                           rtol=3e-5)


CRAFTED = [("cpu", "float32", "decode"), ("cpu", "float32", "prompt"),
           pytest.param("cuda", "float32", "decode", marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", "decode", marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", "prompt", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("device,dtype,where", CRAFTED)
def test_latent_attention_far_key_window_edges_and_sink(device, dtype,
                                                        where):
    """Inputs shaped so that ONE key decides the result: a far key among
    hundreds (full attention), the oldest key a window still holds, and
    the first key it has dropped; and a dominant sink empties the
    output.  The deciding query is either a lone decoded row or the last
    row of a five-row prompt portion."""
    R, RD, bs, n = 16, 8, 16, 330
    dt = getattr(torch, dtype)
    tol = 1e-3 if dt == torch.float32 else 5e-2
    g = torch.Generator().manual_seed(7)
    c = torch.randn(n, R, generator=g) * 0.1
    kr = torch.randn(n, RD, generator=g) * 0.1
    marks = {17: 0, 330 - 40: 1, 330 - 41: 2, 255: 3, 256: 4}
    for j, axis in marks.items():      # distinctive keys on page borders
        c[j] = 0
        c[j, axis] = 6.0               # and just inside/outside a window
    c, kr = c.to(dt).float(), kr.to(dt).float()
    cache, pages = _paged(c, kr, bs, 8)
    bt = torch.tensor([pages], dtype=torch.int32)
    pos = n - 1
    nq = 1 if where == "decode" else 5

    def run(qvec, window, sink):
        qa = torch.randn(nq, 1, R, generator=g) * 0.1
        qa[-1, 0] = qvec
        out = ops.latent_attention(
            qa.to(dt).to(device),
            torch.zeros(nq, 1, RD, dtype=dt, device=device),
            cache.to(dt).to(device), bt.to(device),
            torch.zeros(nq, dtype=torch.int32, device=device),
            torch.arange(pos - nq + 1, pos + 1, dtype=torch.int32,
                         device=device),
            torch.tensor([sink], device=device), 1.0, window,
            nq if where == "prompt" else 0,
            [nq] if where == "prompt" else None)
        return out[-1, 0].float().cpu().double()

    def unit(axis):
        v = torch.zeros(R)
        v[axis] = 6.0
        return v

    def ref(axis, window, sink):
        return oracle.absorbed_row(
            unit(axis).double(), torch.zeros(RD).double(), c.double(),
            kr.double(), pos, window, sink, 1.0)

    # far key, full attention: the output IS that latent
    torch.testing.assert_close(run(unit(0), 0, -30.0), c[17].double(),
                               atol=tol, rtol=tol)
    # window 40 ends at position 290 = n - 40: seen
    torch.testing.assert_close(run(unit(1), 40, -30.0), c[290].double(),
                               atol=tol, rtol=tol)
    # position 289 is one too old: the marked key must be invisible
    out = run(unit(2), 40, -30.0)
    torch.testing.assert_close(out, ref(2, 40, -30.0), atol=tol, rtol=tol)
    assert float(out[2]) < 1.0
    # keys on both sides of a page border
    torch.testing.assert_close(run(unit(3), 0, -30.0), c[255].double(),
                               atol=tol, rtol=tol)
    torch.testing.assert_close(run(unit(4), 0, -30.0), c[256].double(),
                               atol=tol, rtol=tol)
    # a huge sink takes all the mass and carries no value
    assert float(run(unit(0), 0, 80.0).abs().max()) < 1e-6
    # a moderate sink: exact share (the sink is not scaled, counts once)
    torch.testing.assert_close(run(unit(0), 0, 30.0), ref(0, 0, 30.0),
                               atol=tol, rtol=tol)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [7, 300])
def test_feed_forward_modules(device, T):
    """Dense xIELU and routed relu^2 feed-forwards alone, through the
    padded (few rows) and the sorted (many rows) expert dispatch."""
    from inference_gateway_amd.engine.config import DenseFFSpec, MoEFFSpec
    from inference_gateway_amd.engine.models.fedatar import (Relu2MoE,
                                                             XieluMLP)

    D = 24
    cfg = oracle.make_config(width=D, pattern=("gd", "gm"), ff=20,
                             experts=5, top=2, expert_ff=9, shared_ff=7)
    W = {k: v.float() for k, v in oracle.make_weights(cfg, seed=37).items()}
    h = torch.randn(T, D, generator=torch.Generator().manual_seed(38))
    dev = _dev(device)
    mlp = XieluMLP(D, DenseFFSpec(ff=20), "x", dev, torch.float32)
    mlp.up.data.copy_(W["l0.mlp.up"])
    mlp.down.data.copy_(W["l0.mlp.down"])
    mlp.act.data.copy_(W["l0.mlp.act"])
    W64 = {k: v.double() for k, v in W.items()}
    close(mlp(h.to(dev), None), oracle.dense_ff(h.double(), W64, "l0.mlp."),
          2e-5)
    moe = Relu2MoE(D, MoEFFSpec(experts=5, top=2, expert_ff=9, shared_ff=7),
                   "m", dev, torch.float32)
    moe.router_w.data.copy_(W["l1.mlp.router"])
    moe.router_b.data.copy_(W["l1.mlp.router.b"])
    moe.up_t.data.copy_(torch.stack(
        [W[f"l1.mlp.e{e}.up"].t() for e in range(5)]))
    moe.down_t.data.copy_(torch.stack(
        [W[f"l1.mlp.e{e}.down"].t() for e in range(5)]))
    moe.shared_up.data.copy_(W["l1.mlp.shared.up"])
    moe.shared_down.data.copy_(W["l1.mlp.shared.down"])
    close(moe(h.to(dev), None),
          oracle.moe_ff(h.double(), W64, "l1.mlp.", cfg["layers"][1]["mlp"]),
          2e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_activations_and_route(device):
    g = torch.Generator().manual_seed(9)
    z = torch.randn(33, 21, generator=g) * 3
    for p, q in ((0.3, -0.7), (-2.0, 1.5)):
        pq = torch.tensor([p, q])
        torch.testing.assert_close(
            ops.xielu(z.to(device), pq.to(device)).cpu().double(),
            oracle.xielu(z.double(), p, q), atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(
        ops.relu2(z.to(device)).cpu().double(),
        torch.clamp(z.double(), min=0) ** 2, atol=1e-5, rtol=1e-5)
    for E, K in ((5, 3), (12, 12), (7, 1)):
        lg = torch.randn(19, E, generator=g)
        w, idx, dst = ops.moe_topk_route(lg.to(device), K, 64)
        w, idx = w.cpu(), idx.cpu()
        if dst is not None:
            # padded rows: distinct, inside the chosen expert's segment
            d = dst.cpu().view(19, K)
            assert len(set(d.flatten().tolist())) == 19 * K
            assert torch.equal(d // 64, idx.long())
        for t in range(19):
            order = sorted(range(E), key=lambda e: -float(lg[t, e]))[:K]
            assert idx[t].tolist() == order
            zz = lg[t, order].double()
            ref = torch.exp(zz - zz.max())
            torch.testing.assert_close(w[t].double(), ref / ref.sum(),
                                       atol=1e-6, rtol=1e-5)


# ---------------------------------------------------------------------------
# the whole model through the engine
# ---------------------------------------------------------------------------
CONFIGS = {
    # both mixers, all feed-forward kinds, sizes all different
    "mixed": dict(),
    # values that happen to be 1 or equal elsewhere: one head, top = all
    # experts, window of one token, no shared expert, gru wider than D
    "ones": dict(width=32, vocab=50, pattern=("am", "gd", "a-", "gm"),
                 heads=1, dim=6, rot_dim=2, vdim=5, kv_rank=7, q_rank=9,
                 window=1, ff=20, experts=3, top=3, expert_ff=8,
                 shared_ff=0, gru_width=40),
    # full attention (no window), one expert chosen of many
    "full": dict(width=40, vocab=61, pattern=("a-", "gm", "ad"),
                 heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8, q_rank=8,
                 window=0, ff=24, experts=9, top=1, expert_ff=10,
                 shared_ff=6),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_decode_and_portions(tmp_path, device, name):
    """One request three ways — whole, token by token, ragged portions
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
    seen_slots = {}
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
        for k, _n in step:
            if at[k] == lens[k] and k in sids:
                eng.close_stream(sids.pop(k))
    assert at == lens
    assert seen_slots["e"] in (seen_slots["b"], seen_slots["d"])
    for k in reqs:
        close(torch.cat(got[k]), refs[k], 2e-5)
    assert eng.block_manager.num_free == eng.block_manager.num_blocks - 1


@pytest.mark.parametrize("device", DEVICES)
def test_forced_step_errors(tmp_path, device):
    cfg = oracle.make_config(pattern=("gd", "a-"))
    W = oracle.make_weights(cfg, seed=19)
    eng = make_engine(tmp_path, cfg, W, device, blocks=4, slots=1)
    a, b = eng.open_stream(), eng.open_stream()
    eng.replay_step([(a, [1, 2, 3])], {})
    with pytest.raises(RuntimeError):          # no second slot
        eng.replay_step([(b, [1])], {})
    with pytest.raises(RuntimeError):          # 3 usable pages of 4 tokens
        eng.replay_step([(a, list(range(20)))], {})


@pytest.mark.parametrize("device", DEVICES)
def test_bfloat16_serving_precision(tmp_path, device):
    """bf16 weights/activations with fp32 norms, state and softmax stay
    within rounding of the plain model, cut or uncut."""
    cfg = oracle.make_config()
    W = oracle.make_weights(cfg, seed=21)
    tokens = toks(33, cfg["vocab"], 22)
    ref = oracle.forward(cfg, W, tokens)
    eng = make_engine(tmp_path, cfg, W, device, dtype="bfloat16")
    close(replay_all(eng, tokens, [33]), ref, 4e-2)
    close(replay_all(eng, tokens, [5, 2, 1, 1, 24]), ref, 4e-2)


# ---------------------------------------------------------------------------
# generation through the engine's own entry point and scheduler
# ---------------------------------------------------------------------------
def _greedy_ref(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(oracle.forward(cfg, W, seq)[-1].argmax()))
    return seq[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode", ["plain", "chunked_mixed"])
def test_greedy_generation(tmp_path, device, mode):
    cfg = oracle.make_config(width=32, vocab=40, pattern=("gd", "am", "g-"),
                             heads=2, dim=6, rot_dim=4, vdim=6, kv_rank=10,
                             q_rank=8, window=7, ff=24, experts=4, top=2,
                             expert_ff=8, shared_ff=8)
    W = oracle.make_weights(cfg, seed=23)
    prompts = [toks(n, cfg["vocab"], 30 + n) for n in (11, 3, 18)]
    refs = [_greedy_ref(cfg, W, p, 6) for p in prompts]
    kw = {}
    if mode == "chunked_mixed":
        # prompts are cut at 5 tokens and ride beside running decodes
        kw = dict(enable_chunked_prefill=True, enable_mixed_batches=True,
                  max_batched_tokens=5)
    eng = make_engine(tmp_path, cfg, W, device, blocks=64, **kw)
    sp = SamplingParams(max_new_tokens=6, temperature=0.0)
    ids = [eng.add_request(p, sp) for p in prompts]
    steps = 0
    while not eng.is_finished() and steps < 200:
        eng.step()
        steps += 1
    for i, r in zip(ids, refs):
        assert eng.get_output(i).token_ids == r
    assert eng.block_manager.num_free == eng.block_manager.num_blocks - 1


@pytest.mark.parametrize("device", DEVICES)
def test_preemption_rebuilds_state(tmp_path, device):
    """A pool too small for both requests: the newer one is preempted,
    its state dropped, and it resumes by re-running its folded prompt."""
    cfg = oracle.make_config(width=32, vocab=40, pattern=("gd", "a-"),
                             heads=2, dim=6, rot_dim=4, vdim=6, kv_rank=10,
                             q_rank=8, window=0, ff=24)
    W = oracle.make_weights(cfg, seed=25)
    prompts = [toks(7, 40, 41), toks(6, 40, 42)]
    refs = [_greedy_ref(cfg, W, p, 10) for p in prompts]
    eng = make_engine(tmp_path, cfg, W, device, blocks=8, block=4)
    sp = SamplingParams(max_new_tokens=10, temperature=0.0)
    ids = [eng.add_request(p, sp) for p in prompts]
    steps = 0
    while not eng.is_finished() and steps < 300:
        eng.step()
        steps += 1
    assert eng.scheduler.num_preemptions > 0
    for i, r in zip(ids, refs):
        assert eng.get_output(i).token_ids == r


@pytest.mark.parametrize("device", DEVICES)
def test_forked_group_copies_state(tmp_path, device):
    """n=2 from one prefill: the branch shares the prompt's pages and
    starts from a COPY of the parent's recurrent state."""
    cfg = oracle.make_config(width=32, vocab=40, pattern=("gd", "a-"),
                             heads=2, dim=6, rot_dim=4, vdim=6, kv_rank=10,
                             q_rank=8, window=0, ff=24)
    W = oracle.make_weights(cfg, seed=27)
    prompt = toks(10, 40, 43)          # 2 full pages + a partial one
    ref = _greedy_ref(cfg, W, prompt, 5)
    eng = make_engine(tmp_path, cfg, W, device, blocks=32)
    ids = eng.add_request_group(
        prompt, SamplingParams(max_new_tokens=5, temperature=0.0), n=2)
    while not eng.is_finished():
        eng.step()
    assert eng.num_forks == 1
    for i in ids:
        assert eng.get_output(i).token_ids == ref


# ---------------------------------------------------------------------------
# configuration, registry, loader, command line
# ---------------------------------------------------------------------------
def test_config_reader_and_registry(tmp_path):
    cfg = oracle.make_config(**CONFIGS["full"])
    del cfg["layers"][0]["mixer"]["q_rank"]     # left to the tensor shape
    W = oracle.make_weights(oracle.make_config(**CONFIGS["full"]), seed=1)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    mc = model_config_from_dir(path)
    assert isinstance(mc, FedatarConfig) and mc.num_layers == 3
    a = mc.layers[0].mixer
    assert (a.q_rank, a.window, a.rot.dims) == (8, 0, 4)
    assert mc.layers[0].mlp is None and mc.layers[1].mlp.top == 1
    assert mc.kv_bytes_per_token() == 2 * (8 + 4) * 2
    with pytest.raises(ValueError):
        FedatarConfig.from_dict({"width": 4, "vocab": 4, "layers": [
            {"type": "conv", "mixer": {}, "mlp": None}]})


def test_loader_rejects_wrong_shapes(tmp_path):
    cfg = oracle.make_config(pattern=("gd",))
    W = oracle.make_weights(cfg, seed=2)
    W["l0.mix.o"] = W["l0.mix.o"][:, :-1]
    with pytest.raises(ValueError):
        make_engine(tmp_path, cfg, W, "cpu")


def test_prefix_caching_refused_for_recurrent_layers(tmp_path):
    cfg = oracle.make_config(pattern=("gd",))
    W = oracle.make_weights(cfg, seed=3)
    with pytest.raises(ValueError):
        make_engine(tmp_path, cfg, W, "cpu", enable_prefix_caching=True)


def test_trace_runner_command(tmp_path):
    """bin/trace_run end to end on the CPU: steps in, logit files and
    'done' lines out, slots and pages recycled over five requests."""
    cfg = oracle.make_config(pattern=("gd", "am"))
    W = oracle.make_weights(cfg, seed=29)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    reqs = {f"r{i}": toks(9 + i, cfg["vocab"], 50 + i) for i in range(5)}
    lines = []
    for n, (k, t) in enumerate(reqs.items()):
        lines.append({"step": 2 * n, "entries": [
            {"id": k, "tokens": t[:-1], "want": [0, len(t) - 2]}],
            "end": []})
        lines.append({"step": 2 * n + 1, "entries": [
            {"id": k, "tokens": t[-1:], "want": [0]}], "end": [k]})
    lines.append({"step": 10, "entries": [], "end": []})
    root = Path(__file__).resolve().parent.parent
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", CUDA_VISIBLE_DEVICES="")
    p = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", path,
         "--dtype", "float32", "--out", str(tmp_path / "out"),
         "--max-tokens", "64"],
        input="\n".join(json.dumps(x) for x in lines) + "\n", text=True,
        capture_output=True, env=env, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    done = [x for x in p.stdout.splitlines() if x.startswith("done ")]
    assert done == [f"done {i}" for i in range(11)]
    import numpy as np

    V = cfg["vocab"]
    for n, (k, t) in enumerate(reqs.items()):
        ref = oracle.forward(cfg, W, t)
        a = np.fromfile(tmp_path / "out" / f"{2 * n}.f32", dtype="<f4")
        b = np.fromfile(tmp_path / "out" / f"{2 * n + 1}.f32", dtype="<f4")
        close(torch.tensor(a).view(2, V), ref[[0, len(t) - 2]], 2e-5)
        close(torch.tensor(b).view(1, V), ref[[len(t) - 1]], 2e-5)
    assert not (tmp_path / "out" / "10.f32").exists()


# ---------------------------------------------------------------------------
# GPU only: the bf16 matrix-core attention kernel against the plain
# float64 rows, over its register-tile instantiations, both staging
# paths, partial tiles, several head groups and ragged batches
# ---------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("R,RD,H,window", [
    (20, 6, 3, 9),        # scalar staging, odd head count
    (48, 16, 6, 0),       # vector staging, smallest tile set, key splits
    (48, 16, 6, 37),
    (136, 24, 100, 50),   # two head groups, middle tile set
    (512, 64, 16, 70),    # largest tile set (LDS above 64 KiB)
])
def test_latent_attention_mfma(R, RD, H, window):
    g = torch.Generator().manual_seed(31)
    bs = 16
    lens = [75, 130]                       # cached tokens per sequence
    caches, tables = [], []
    c_all, kr_all = [], []
    nb_total = 1
    for n in lens:
        c = (torch.randn(n, R, generator=g) * 0.5).bfloat16().float()
        kr = (torch.randn(n, RD, generator=g) * 0.5).bfloat16().float()
        c_all.append(c)
        kr_all.append(kr)
    # interleave the two sequences' pages in one pool
    nblk = [(n + bs - 1) // bs for n in lens]
    perm = (torch.randperm(sum(nblk) + 2, generator=g) + 1).tolist()
    cache = torch.randn(sum(nblk) + 4, bs, R + RD, generator=g)
    flat = cache.view(-1, R + RD)
    maxb = max(nblk)
    bt = torch.zeros(2, maxb, dtype=torch.int32)
    at = 0
    for s, n in enumerate(lens):
        pages = perm[at:at + nblk[s]]
        at += nblk[s]
        bt[s, :nblk[s]] = torch.tensor(pages, dtype=torch.int32)
        for j in range(n):
            flat[pages[j // bs] * bs + j % bs] = torch.cat(
                [c_all[s][j], kr_all[s][j]])
    # rows: a 23-row portion of seq 0 ending at its last token, a
    # 41-row portion of seq 1 from position 60, then decoded rows
    segs = [(0, 75 - 23, 23), (1, 60, 41)]
    dec = [(1, 129), (0, 74)]
    row_seq, pos = [], []
    for s, p0, n in segs:
        row_seq += [s] * n
        pos += list(range(p0, p0 + n))
    for s, p in dec:
        row_seq.append(s)
        pos.append(p)
    T = len(pos)
    qa = (torch.randn(T, H, R, generator=g) * 0.3).bfloat16()
    qr = (torch.randn(T, H, RD, generator=g) * 0.3).bfloat16()
    sink = torch.randn(H, generator=g)
    scale = 0.7 / math.sqrt(R)
    dev = "cuda"
    out = ops.latent_attention(
        qa.to(dev), qr.to(dev), cache.bfloat16().to(dev), bt.to(dev),
        torch.tensor(row_seq, dtype=torch.int32, device=dev),
        torch.tensor(pos, dtype=torch.int32, device=dev), sink.to(dev),
        scale, window, 64, [23, 41]).float().cpu()
    check_rows = [0, 1, 22, 23, 40, 63, 64, 65]
    heads = sorted({0, H // 2, H - 1})
    for t in check_rows:
        s = row_seq[t]
        for h in heads:
            ref = oracle.absorbed_row(
                qa[t, h].double(), qr[t, h].double(), c_all[s].double(),
                kr_all[s].double(), pos[t], window, sink[h], scale)
            torch.testing.assert_close(out[t, h].double(), ref, atol=2e-2,
                                       rtol=2e-2)
    # and the whole output against the fp32 one-wave-per-row kernel
    ops.LATENT_ATTENTION_MFMA = False
    try:
        slow = ops.latent_attention(
            qa.to(dev), qr.to(dev), cache.bfloat16().to(dev), bt.to(dev),
            torch.tensor(row_seq, dtype=torch.int32, device=dev),
            torch.tensor(pos, dtype=torch.int32, device=dev), sink.to(dev),
            scale, window).float().cpu()
    finally:
        ops.LATENT_ATTENTION_MFMA = True
    torch.testing.assert_close(out, slow, atol=2e-2, rtol=2e-2)


@pytest.mark.gpu
def test_latent_attention_mfma_many_tiles():
    """Thousands of single-row tiles: the launch shape that neither
    splits keys nor prefetches through registers."""
    g = torch.Generator().manual_seed(33)
    R, RD, H, bs, n = 56, 8, 5, 16, 200
    T = 2200
    cache = (torch.randn(n // bs + 2, bs, R + RD, generator=g) * 0.5)
    bt = (torch.randperm(n // bs + 1, generator=g) + 1).to(
        torch.int32).view(1, -1)
    pos = torch.randint(0, n, (T,), generator=g).to(torch.int32)
    qa = (torch.randn(T, H, R, generator=g) * 0.3).bfloat16()
    qr = (torch.randn(T, H, RD, generator=g) * 0.3).bfloat16()
    sink = torch.randn(H, generator=g)
    args = (qa.cuda(), qr.cuda(), cache.bfloat16().cuda(), bt.cuda(),
            torch.zeros(T, dtype=torch.int32, device="cuda"), pos.cuda(),
            sink.cuda(), 0.1, 70)
    fast = ops.latent_attention(*args).float().cpu()
    ops.LATENT_ATTENTION_MFMA = False
    try:
        slow = ops.latent_attention(*args).float().cpu()
    finally:
        ops.LATENT_ATTENTION_MFMA = True
    torch.testing.assert_close(fast, slow, atol=2e-2, rtol=2e-2)


def test_local_provider_serves_a_checkpoint_directory(tmp_path):
    """The gateway's local provider with LOCAL_MODEL=hf picks the
    architecture from the directory's config.json and generates through
    the async engine."""
    import asyncio

    from inference_gateway_amd.config import LocalConfig
    from inference_gateway_amd.providers.local import LocalProvider

    cfg = oracle.make_config(vocab=300, pattern=("gd", "am"))
    W = oracle.make_weights(cfg, seed=35)
    path = oracle.save_checkpoint(tmp_path / "m", cfg, W)
    lc = LocalConfig(enabled=True, model="hf", max_num_seqs=4,
                     max_model_len=128)
    lc.num_gpu_blocks = 64
    lc.weights_path = path
    provider = LocalProvider(lc, device="cpu")
    try:
        assert isinstance(provider.engine.engine.cfg.model, FedatarConfig)

        async def go():
            return await provider.chat_completions({
                "model": "local/hf",
                "messages": [{"role": "user", "content": "hi"}],
                "max_tokens": 3, "temperature": 0})

        body = asyncio.run(go())
        assert body["usage"]["completion_tokens"] == 3
    finally:
        provider.engine.shutdown()
