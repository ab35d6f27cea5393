"""Plain, slow float64 model of the Mekevik design, one function per
mechanism, written from the equations (no code shared with the engine).

It works on a dict of named tensors in the checkpoint's naming plus the
config dict, so a test can hand the SAME tensors to the engine's loader
(through a safetensors file) and to this file.

Notation: h is a [T, D] block holding ALL rows of one sequence from
position 0; everything is recomputed from scratch (no cache).
"""
import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        out[t] = x[t] / math.sqrt((x[t] ** 2).sum() / x.shape[1] + eps) * w
    return out


def logistic(x):
    return 1.0 / (1.0 + torch.exp(-x))


def distance_bucket(n, rows, far):
    """Row of the distance table for a key n tokens back: one row per
    distance below rows/2, then logarithmic steps that reach the last
    row at distance `far`."""
    half = rows // 2
    if n < half:
        return n
    step = math.log(n / half) / math.log(far / half) * (rows - half)
    return min(rows - 1, half + int(math.floor(step)))


def sigmoid_attention(h, W, pre, m, eps, v_first=None):
    """Returns (mixer output [T, D], the values this layer keeps
    [T, G*vd]).  v_first: the first value-mixing layer's values, or None
    when this layer does not mix (or is that first layer)."""
    T = h.shape[0]
    H, G = m["heads"], m["kv_heads"]
    dk, dv = m["dim"], m["vdim"]
    window = (m.get("mask") or {}).get("size")
    q = rms_norm(h @ W[pre + "q"].T, W[pre + "q.norm"], eps)   # whole row
    k = rms_norm(h @ W[pre + "k"].T, W[pre + "k.norm"], eps)
    v = h @ W[pre + "v"].T
    if v_first is not None:
        lam = float(W[pre + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    rel, pb, talk = W[pre + "rel"], W[pre + "pb"], W[pre + "talk"]
    B = rel.shape[0]
    q = q.view(T, H, dk)
    k = k.view(T, G, dk)
    vh = v.view(T, G, dv)
    per = H // G
    heads = torch.zeros((T, H, dv), dtype=F64)
    for i in range(T):
        lo = 0 if not window else max(0, i - window + 1)
        for j in range(lo, i + 1):
            b = distance_bucket(i - j, B, m["bias_max"])
            wts = torch.empty(H, dtype=F64)
            for g in range(H):
                s = float(q[i, g] @ k[j, g // per]) * m["scale"]
                s = s + float(rel[b, g]) + float(pb[g])
                wts[g] = 1.0 / (1.0 + math.exp(-s))
            mixed = talk @ wts                      # head h: sum_g T[h,g] w_g
            for hh in range(H):
                heads[i, hh] += mixed[hh] * vh[j, hh // per]
    gate = logistic(h @ W[pre + "g"].T)
    out = (heads.reshape(T, H * dv) * gate) @ W[pre + "o"].T
    return out, v


def clamped_glu_ff(h, W, pre, f):
    lim = f["limit"]
    g = torch.clamp(h @ W[pre + "gate"].T, max=lim)
    u = torch.clamp(h @ W[pre + "up"].T, min=-lim, max=lim)
    return (g * logistic(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def routed_ff(h, W, pre, f):
    E, top = f["router"]["experts"], f["router"]["top"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        z = W[pre + "router"] @ h[t]
        s = torch.exp(z - z.max())
        s = s / s.sum()
        chosen = sorted(range(E), key=lambda e: -float(s[e]))[:top]
        tot = sum(float(s[e]) for e in chosen) + 1e-20
        for e in chosen:
            a = W[pre + f"e{e}.gate"] @ h[t]
            u = W[pre + f"e{e}.up"] @ h[t]
            y = W[pre + f"e{e}.down"] @ (a * logistic(a) * u)
            out[t] += float(s[e]) / tot * f["router"]["scale"] * y
    return out


def forward(cfg, W, tokens, taps=None):
    """Logits [T, vocab] of one sequence from position 0; taps (a list)
    receives the residual stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    v_first = None
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert l["type"] == "attention"
        m = l["mixer"]
        mixes = bool(m.get("v_mix"))
        y, v = sigmoid_attention(rms_norm(x, W[p + "norm1"], eps), W,
                                 p + "mix.", m, eps,
                                 v_first if mixes else None)
        if mixes and v_first is None:
            v_first = v
        f = l.get("mlp")
        if f is not None:
            h2 = rms_norm(x, W[p + "norm2"], eps)
            if f["kind"] == "dense":
                y = y + clamped_glu_ff(h2, W, p + "mlp.", f)
            else:
                y = y + routed_ff(h2, W, p + "mlp.", f)
        x = x + y
        if taps is not None:
            taps.append(x.clone())
    xn = rms_norm(x, W["final.norm"], eps)
    return xn @ W["head"].T * cfg["logit_scale"]


def attention_row(qrow, keys, vals, pos, window, rel, far, pb, talk, scale):
    """One query row of all heads against cached keys [n, G, dk] and
    values [n, G, dv] (row j = position j): sum_j mixed weights * values,
    [H, dv], before the gate.  Plain loops, float64."""
    H, dk = qrow.shape
    G = keys.shape[1]
    per = H // G
    lo = 0 if not window else max(0, pos - window + 1)
    out = torch.zeros((H, vals.shape[2]), dtype=F64)
    for j in range(lo, pos + 1):
        b = distance_bucket(pos - j, rel.shape[0], far)
        w = torch.tensor([
            1.0 / (1.0 + math.exp(-(float(qrow[g] @ keys[j, g // per])
                                    * scale + float(rel[b, g])
                                    + float(pb[g]))))
            for g in range(H)], dtype=F64)
        mixed = talk @ w
        for h in range(H):
            out[h] += mixed[h] * vals[j, h // per]
    return out


def make_config(width=48, vocab=97, pattern=("d", "m", "-", "m"), heads=4,
                kv_heads=2, dim=12, vdim=10, window=9, ff=40, experts=5,
                top=2, expert_ff=14, bias_rows=10, bias_max=30,
                limit=0.8, router_scale=1.7, v_mix=(True, True, True, True),
                embed_scale=0.7, logit_scale=0.4, eps=1e-5):
    """pattern: one letter per layer for its feed-forward — d dense,
    m mixture, - none.  v_mix: per layer."""
    layers = []
    for i, tok in enumerate(pattern):
        mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                 "vdim": vdim, "bias_max": bias_max,
                 "scale": 1.6 / math.sqrt(dim),
                 "v_mix": bool(v_mix[i % len(v_mix)])}
        if window:
            mixer["mask"] = {"size": window}
        L = {"type": "attention", "mixer": mixer}
        if tok == "d":
            L["mlp"] = {"kind": "dense", "ff": ff, "limit": limit}
        elif tok == "m":
            L["mlp"] = {"kind": "moe", "expert": {"ff": expert_ff},
                        "router": {"experts": experts, "top": top,
                                   "scale": router_scale}}
        else:
            L["mlp"] = None
        layers.append(L)
    return {"architecture": "Mekevik", "layers": layers,
            "embedding": {"scale": embed_scale}, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "vocab": vocab, "width": width,
            "_bias_rows": bias_rows}


def make_weights(cfg, seed=0):
    """bf16-representable random tensors in the checkpoint's naming."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]
    W = {}

    def rnd(name, *shape, scale=1.0, shift=0.0):
        t = torch.randn(*shape, generator=g) * scale + shift
        W[name] = t.to(torch.bfloat16)

    def lin(name, out, inn, gain=1.0):
        rnd(name, out, inn, scale=gain / math.sqrt(inn))

    rnd("embed", cfg["vocab"], D)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        rnd(p + "norm1", D, scale=0.2, shift=1.0)
        m = L["mixer"]
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        lin(p + "mix.q", H * dk, D, 2.0)
        lin(p + "mix.k", G * dk, D, 2.0)
        lin(p + "mix.v", G * dv, D)
        rnd(p + "mix.q.norm", H * dk, scale=0.2, shift=1.0)
        rnd(p + "mix.k.norm", G * dk, scale=0.2, shift=1.0)
        rnd(p + "mix.rel", cfg["_bias_rows"], H, scale=1.0)
        rnd(p + "mix.pb", H, scale=0.5, shift=-1.5)
        W[p + "mix.talk"] = (torch.eye(H) * 0.7 + torch.randn(
            H, H, generator=g) * 0.25).to(torch.bfloat16)
        W[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.6
                             + 0.2).to(torch.bfloat16)
        lin(p + "mix.g", H * dv, D, 2.0)
        lin(p + "mix.o", D, H * dv)
        f = L["mlp"]
        if f is None:
            continue
        rnd(p + "norm2", D, scale=0.2, shift=1.0)
        if f["kind"] == "dense":
            lin(p + "mlp.gate", f["ff"], D, 2.0)
            lin(p + "mlp.up", f["ff"], D, 2.0)
            lin(p + "mlp.down", D, f["ff"])
        else:
            E = f["router"]["experts"]
            lin(p + "mlp.router", E, D, 3.0)
            for e in range(E):
                lin(p + f"mlp.e{e}.gate", f["expert"]["ff"], D, 2.0)
                lin(p + f"mlp.e{e}.up", f["expert"]["ff"], D)
                lin(p + f"mlp.e{e}.down", D, f["expert"]["ff"])
    rnd("final.norm", D, scale=0.2, shift=1.0)
    lin("head", cfg["vocab"], D)
    return W


def save_checkpoint(path, cfg, W):
    import json

    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    public = {k: v for k, v in cfg.items() if not k.startswith("_")}
    (path / "config.json").write_text(json.dumps(public))
    save_file({k: v.contiguous() for k, v in W.items()},
              str(path / "model.safetensors"))
    return str(path)
