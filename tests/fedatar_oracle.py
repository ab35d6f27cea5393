"""Plain, slow float64 model of the Fedatar design, one function per
mechanism, written from the equations (no code shared with the engine).

It works on a dict of named tensors in the checkpoint's naming plus the
config dict, so a test can hand the SAME tensors to the engine's loader
(through a safetensors file) and to this file.

Notation: h is a [T, D] block of one sequence's rows starting at
position p0; everything is recomputed from scratch (no cache).
"""
import math

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        mu = x[t].sum() / x.shape[1]
        var = ((x[t] - mu) ** 2).sum() / x.shape[1]
        out[t] = (x[t] - mu) / math.sqrt(var + eps) * w + b
    return out


def rms_norm(x, w, eps):
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        out[t] = x[t] / math.sqrt((x[t] ** 2).sum() / x.shape[1] + eps) * w
    return out


def logistic(x):
    return 1.0 / (1.0 + torch.exp(-x))


def mingru(h, Wz, bz, Wx, bx, Wg, Wo, S0=None):
    """Returns (output [T, D], end state)."""
    T = h.shape[0]
    S = torch.zeros(Wz.shape[0], dtype=F64) if S0 is None else S0.clone()
    rows = []
    for t in range(T):
        z = logistic(Wz @ h[t] + bz)
        u = Wx @ h[t] + bx
        cand = torch.where(u >= 0, u + 0.5, logistic(u))
        S = (1 - z) * S + z * cand
        g = Wg @ h[t]
        rows.append(Wo @ (S * (g * logistic(g))))
    return torch.stack(rows), S


def rotate(vec, pos, base, dims):
    """Pairs (2i, 2i+1), i < dims/2, of a 1-d vector turned by
    pos * base**(-2i/dims); entries from `dims` on are untouched."""
    out = vec.clone()
    for i in range(dims // 2):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(ang), math.sin(ang)
        u, v = vec[2 * i], vec[2 * i + 1]
        out[2 * i] = u * c - v * s
        out[2 * i + 1] = v * c + u * s
    return out


def latent_attention(h, W, pre, m, eps):
    """h [T, D]: ALL rows of the sequence from position 0.  W: tensor
    dict, pre: name prefix ('l3.mix.'), m: the layer's mixer config."""
    T = h.shape[0]
    H, dn, rd = m["heads"], m["dim"], m["rot_dim"]
    vd, R = m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    window = (m.get("mask") or {}).get("size")
    scale = m["scale"]
    cq = rms_norm(h @ W[pre + "dq"].T, W[pre + "dq.norm"], eps)
    q = cq @ W[pre + "uq"].T                       # [T, H*(dn+rd)]
    dkv = h @ W[pre + "dkv"].T
    c = rms_norm(dkv[:, :R], W[pre + "dkv.norm"], eps)
    kr = torch.stack([rotate(dkv[t, R:], t, base, dims) for t in range(T)])
    kn = c @ W[pre + "uk"].T                       # [T, H*dn]
    v = c @ W[pre + "uv"].T                        # [T, H*vd]
    gate = logistic(h @ W[pre + "g"].T)            # [T, H]
    out = torch.zeros(T, H * vd, dtype=F64)
    for t in range(T):
        lo = 0 if not window else max(0, t - window + 1)
        for hh in range(H):
            qh = q[t, hh * (dn + rd):(hh + 1) * (dn + rd)]
            qn, qr = qh[:dn], rotate(qh[dn:], t, base, dims)
            sc = torch.stack([
                (qn @ kn[j, hh * dn:(hh + 1) * dn] + qr @ kr[j]) * scale
                for j in range(lo, t + 1)])
            sink = W[pre + "sink"][hh]
            mx = max(float(sc.max()), float(sink))
            e = torch.exp(sc - mx)
            den = e.sum() + math.exp(float(sink) - mx)
            o = torch.zeros(vd, dtype=F64)
            for n, j in enumerate(range(lo, t + 1)):
                o += e[n] / den * v[j, hh * vd:(hh + 1) * vd]
            out[t, hh * vd:(hh + 1) * vd] = o * gate[t, hh]
    return out @ W[pre + "o"].T


def softplus(x):
    return math.log1p(math.exp(x))


def xielu(z, p, q):
    ap, an = softplus(float(p)), 0.5 + softplus(float(q))
    pos = ap * z * z + z / 2
    neg = an * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ff(h, W, pre):
    a = W[pre + "act"]
    return xielu(h @ W[pre + "up"].T, a[0], a[1]) @ W[pre + "down"].T


def moe_ff(h, W, pre, m):
    E, K = m["router"]["experts"], m["router"]["top"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        z = W[pre + "router"] @ h[t] + W[pre + "router.b"]
        chosen = sorted(range(E), key=lambda e: -float(z[e]))[:K]
        zz = torch.stack([z[e] for e in chosen])
        w = torch.exp(zz - zz.max())
        w = w / w.sum()
        for k, e in enumerate(chosen):
            a = torch.clamp(W[pre + f"e{e}.up"] @ h[t], min=0.0) ** 2
            out[t] += w[k] * (W[pre + f"e{e}.down"] @ a)
        if m.get("shared"):
            a = torch.clamp(W[pre + "shared.up"] @ h[t], min=0.0) ** 2
            out[t] += W[pre + "shared.down"] @ a
    return out


def forward(cfg, W, tokens, taps=None):
    """Logits [T, vocab] (float64) of one whole sequence."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        if L["type"] == "mingru":
            y, _ = mingru(h, W[p + "mix.z"], W[p + "mix.z.b"],
                          W[p + "mix.x"], W[p + "mix.x.b"], W[p + "mix.g"],
                          W[p + "mix.o"])
        else:
            y = latent_attention(h, W, p + "mix.", L["mixer"], eps)
        x = x + y
        if L["mlp"] is not None:
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            if L["mlp"]["kind"] == "dense":
                x = x + dense_ff(h, W, p + "mlp.")
            else:
                x = x + moe_ff(h, W, p + "mlp.", L["mlp"])
        if taps is not None:
            taps.append(x.clone())
    x = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return x @ W["head"].T


# ---------------------------------------------------------------------------
# random checkpoints
# ---------------------------------------------------------------------------
def make_config(width=48, vocab=97, pattern=("gd", "am", "gm", "a-"),
                heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=20, q_rank=18,
                window=9, ff=40, experts=5, top=3, expert_ff=12,
                shared_ff=20, gru_width=None, rot_base=777.0, eps=1e-5):
    layers = []
    for tok in pattern:
        if tok[0] == "g":
            L = {"type": "mingru",
                 "mixer": {"width": gru_width or width}}
        else:
            mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim,
                     "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                     "rot": {"base": rot_base, "dims": rot_dim},
                     "scale": 1.3 / math.sqrt(dim + rot_dim)}
            if window:
                mixer["mask"] = {"size": window}
            L = {"type": "latent_attention", "mixer": mixer}
        if tok[1] == "d":
            L["mlp"] = {"kind": "dense", "ff": ff}
        elif tok[1] == "m":
            L["mlp"] = {"kind": "moe", "expert": {"ff": expert_ff},
                        "router": {"experts": experts, "top": top}}
            if shared_ff:
                L["mlp"]["shared"] = {"ff": shared_ff}
        else:
            L["mlp"] = None
        layers.append(L)
    return {"architecture": "Fedatar", "layers": layers,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


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

    def norm(name):
        rnd(name, D, scale=0.2, shift=1.0)
        rnd(name + ".b", D, scale=0.1)

    rnd("embed", cfg["vocab"], D)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        norm(p + "norm1")
        m = L["mixer"]
        if L["type"] == "mingru":
            Wd = m["width"]
            lin(p + "mix.z", Wd, D, 2.0)
            rnd(p + "mix.z.b", Wd, scale=0.5)
            lin(p + "mix.x", Wd, D, 2.0)
            rnd(p + "mix.x.b", Wd, scale=0.5)
            lin(p + "mix.g", Wd, D, 2.0)
            lin(p + "mix.o", D, Wd)
        else:
            H, dn, rd = m["heads"], m["dim"], m["rot_dim"]
            lin(p + "mix.dq", m["q_rank"], D)
            rnd(p + "mix.dq.norm", m["q_rank"], scale=0.2, shift=1.0)
            lin(p + "mix.uq", H * (dn + rd), m["q_rank"], 2.0)
            lin(p + "mix.dkv", m["kv_rank"] + rd, D, 2.0)
            rnd(p + "mix.dkv.norm", m["kv_rank"], scale=0.2, shift=1.0)
            lin(p + "mix.uk", H * dn, m["kv_rank"], 2.0)
            lin(p + "mix.uv", H * m["vdim"], m["kv_rank"])
            rnd(p + "mix.sink", H, scale=1.0)
            lin(p + "mix.g", H, D, 2.0)
            lin(p + "mix.o", D, H * m["vdim"])
        f = L["mlp"]
        if f is None:
            continue
        norm(p + "norm2")
        if f["kind"] == "dense":
            lin(p + "mlp.up", f["ff"], D)
            lin(p + "mlp.down", D, f["ff"])
            rnd(p + "mlp.act", 2, scale=0.7)
        else:
            E = f["router"]["experts"]
            lin(p + "mlp.router", E, D, 3.0)
            rnd(p + "mlp.router.b", E, scale=0.5)
            for e in range(E):
                lin(p + f"mlp.e{e}.up", f["expert"]["ff"], D)
                lin(p + f"mlp.e{e}.down", D, f["expert"]["ff"])
            if f.get("shared"):
                lin(p + "mlp.shared.up", f["shared"]["ff"], D)
                lin(p + "mlp.shared.down", D, f["shared"]["ff"])
    norm("final.norm")
    lin("head", cfg["vocab"], D)
    return W


def save_checkpoint(path, cfg, W):
    import json

    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()},
              str(path / "model.safetensors"))
    return str(path)


def absorbed_row(qa, qr, c, kr, pos, window, sink, scale):
    """One query row of one head against cached rows c [n, R], kr [n, rd]
    (row j = position j): the probability-weighted sum of latents, with
    the sink in the denominator.  Plain loops, float64."""
    lo = 0 if not window else max(0, pos - window + 1)
    sc = [float((qa @ c[j] + qr @ kr[j]) * scale) for j in range(lo, pos + 1)]
    mx = max(max(sc), float(sink))
    e = [math.exp(s - mx) for s in sc]
    den = sum(e) + math.exp(float(sink) - mx)
    out = torch.zeros(c.shape[1], dtype=F64)
    for n, j in enumerate(range(lo, pos + 1)):
        out += e[n] / den * c[j]
    return out
