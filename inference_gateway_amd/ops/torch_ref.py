"""Plain-PyTorch fp32 reference implementations of every HIP kernel.

These are the *numerics oracle* for the gfx950 kernels (the
rebuild adds a GPU-kernel test tier comparing hand-written kernels against
a PyTorch fp32 reference) and the CPU execution path for the engine so the
full request flow is testable without a GPU. On a GPU box the engine uses
the _kernels extension and refuses to fall back silently.
"""
from __future__ import annotations

import torch


def rmsnorm_ref(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    inv = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * inv * weight.float()).to(x.dtype)


def fused_add_rmsnorm_ref(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> tuple[torch.Tensor, torch.Tensor]:
    """Returns (normed, new_residual); matches the in-place HIP op."""
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return rmsnorm_ref(new_residual, weight, eps), new_residual


def rope_ref(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    head_dim: int,
    cos_sin_cache: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor]:
    """NeoX-style rotate-half RoPE. q: [T, NQ*HD], k: [T, NKV*HD]."""
    half = head_dim // 2
    cs = cos_sin_cache[positions.long()].float()  # [T, HD]
    cos, sin = cs[:, :half], cs[:, half:]

    def rot(x: torch.Tensor) -> torch.Tensor:
        T = x.shape[0]
        xs = x.float().view(T, -1, head_dim)
        x1, x2 = xs[..., :half], xs[..., half:]
        c = cos.unsqueeze(1)
        s = sin.unsqueeze(1)
        out = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)
        return out.view(x.shape).to(x.dtype)

    return rot(q), rot(k)


def build_cos_sin_cache(
    head_dim: int, max_pos: int, base: float = 10000.0, device="cpu",
    rope_scaling: dict = None,
) -> torch.Tensor:
    """[max_pos, HD] fp32 — cos in [0, HD/2), sin in [HD/2, HD).

    rope_scaling: HF `rope_scaling` dict.  Supported: the Llama-3.1
    "llama3" scheme (wavelength-banded frequency rescale: short
    wavelengths untouched, long wavelengths divided by `factor`, a
    smooth ramp between — the published long-context extension) and
    "linear" (all frequencies divided by `factor`).  None/unknown-less
    configs keep plain RoPE; an unsupported rope_type raises (silent
    wrong positions would corrupt every long-context generation)."""
    half = head_dim // 2
    inv_freq = 1.0 / (
        base ** (torch.arange(0, half, dtype=torch.float64, device=device) / half)
    )
    if rope_scaling:
        rtype = (rope_scaling.get("rope_type")
                 or rope_scaling.get("type") or "llama3")
        factor = float(rope_scaling.get("factor", 8.0))
        if rtype == "llama3":
            lo = float(rope_scaling.get("low_freq_factor", 1.0))
            hi = float(rope_scaling.get("high_freq_factor", 4.0))
            orig = float(rope_scaling.get(
                "original_max_position_embeddings", 8192))
            import math

            wavelen = 2 * math.pi / inv_freq
            low_wl = orig / lo            # longest untouched band edge
            high_wl = orig / hi           # shortest scaled band edge
            smooth = (orig / wavelen - lo) / (hi - lo)
            scaled = torch.where(
                wavelen > low_wl, inv_freq / factor, inv_freq)
            ramp = ((1 - smooth) * inv_freq / factor
                    + smooth * inv_freq)
            inv_freq = torch.where(
                (wavelen <= low_wl) & (wavelen >= high_wl), ramp, scaled)
        elif rtype == "linear":
            inv_freq = inv_freq / factor
        else:
            raise ValueError(
                f"unsupported rope_scaling type {rtype!r} (supported: "
                "llama3, linear)")
    t = torch.arange(max_pos, dtype=torch.float64, device=device)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()


def append_kv_cache_ref(k, v, kcache, vcache, slot_mapping):
    """kcache/vcache: [NB, NKV, BS, HD]; k/v: [T, NKV, HD]."""
    bs = kcache.shape[2]
    for t in range(k.shape[0]):
        slot = int(slot_mapping[t])
        if slot < 0:
            continue
        blk, off = slot // bs, slot % bs
        kcache[blk, :, off, :] = k[t]
        vcache[blk, :, off, :] = v[t]


def paged_attn_decode_ref(q, kcache, vcache, block_table, ctx_lens, scale):
    """q: [B, NQ, HD] -> out [B, NQ, HD]; fp32 math."""
    B, NQ, HD = q.shape
    NKV, BS = kcache.shape[1], kcache.shape[2]
    G = NQ // NKV
    out = torch.empty_like(q)
    for b in range(B):
        ctx = int(ctx_lens[b])
        nblk = (ctx + BS - 1) // BS
        blocks = block_table[b, :nblk].long()
        # gather [ctx, NKV, HD]
        keys = kcache[blocks].permute(0, 2, 1, 3).reshape(-1, NKV, HD)[:ctx]
        vals = vcache[blocks].permute(0, 2, 1, 3).reshape(-1, NKV, HD)[:ctx]
        for h in range(NQ):
            kvh = h // G
            s = (keys[:, kvh].float() @ q[b, h].float()) * scale
            p = torch.softmax(s, dim=-1)
            out[b, h] = (p @ vals[:, kvh].float()).to(q.dtype)
    return out


def flash_prefill_ref(q, k, v, cu_seqlens, scale):
    """Varlen causal attention. q: [T, NQ, HD], k/v: [T, NKV, HD]."""
    T, NQ, HD = q.shape
    NKV = k.shape[1]
    G = NQ // NKV
    out = torch.empty_like(q)
    for s in range(cu_seqlens.shape[0] - 1):
        a, b = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        L = b - a
        mask = torch.tril(torch.ones(L, L, dtype=torch.bool, device=q.device))
        for h in range(NQ):
            kvh = h // G
            sc = (q[a:b, h].float() @ k[a:b, kvh].float().T) * scale
            sc = sc.masked_fill(~mask, float("-inf"))
            p = torch.softmax(sc, dim=-1)
            out[a:b, h] = (p @ v[a:b, kvh].float()).to(q.dtype)
    return out


def flash_prefill_paged_ref(q, kcache, vcache, block_table, prefix_lens,
                            cu_seqlens, scale):
    """Reference for the paged-extend prefill: gather each sequence's
    full K/V (prefix + chunk) from the cache via its block table, then
    run offset-causal attention for the chunk's q rows."""
    Tq, NQ, HD = q.shape
    NKV = kcache.shape[1]
    BS = kcache.shape[2]
    G = NQ // NKV
    out = torch.empty_like(q)
    for s in range(cu_seqlens.shape[0] - 1):
        a, b = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        Lq = b - a
        P = int(prefix_lens[s])
        KVL = P + Lq
        nblk = (KVL + BS - 1) // BS
        blocks = block_table[s, :nblk].long()
        # [nblk*BS, NKV, HD] gathered then trimmed
        keys = kcache[blocks].permute(0, 2, 1, 3).reshape(
            nblk * BS, NKV, HD)[:KVL]
        vals = vcache[blocks].permute(0, 2, 1, 3).reshape(
            nblk * BS, NKV, HD)[:KVL]
        qpos = torch.arange(P, KVL, device=q.device)
        kpos = torch.arange(KVL, device=q.device)
        mask = kpos.unsqueeze(0) <= qpos.unsqueeze(1)     # [Lq, KVL]
        for h in range(NQ):
            kvh = h // G
            sc = (q[a:b, h].float() @ keys[:, kvh].float().T) * scale
            sc = sc.masked_fill(~mask, float("-inf"))
            p = torch.softmax(sc, dim=-1)
            out[a:b, h] = (p @ vals[:, kvh].float()).to(q.dtype)
    return out


def make_prefill_tiles(seq_lens, tile_m: int = 64, device="cpu"):
    """Host-side tile map for flash_prefill: (tile_seq, tile_off) int32."""
    tseq, toff = [], []
    for i, L in enumerate(seq_lens):
        for off in range(0, int(L), tile_m):
            tseq.append(i)
            toff.append(off)
    return (
        torch.tensor(tseq, dtype=torch.int32, device=device),
        torch.tensor(toff, dtype=torch.int32, device=device),
    )


def silu_mul_ref(gate_up: torch.Tensor) -> torch.Tensor:
    inter = gate_up.shape[-1] // 2
    g = gate_up[..., :inter].float()
    u = gate_up[..., inter:].float()
    return (torch.nn.functional.silu(g) * u).to(gate_up.dtype)


def _f32_key(x: torch.Tensor) -> torch.Tensor:
    u = x.float().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    neg = (u & 0x80000000) != 0
    return torch.where(neg, u ^ 0xFFFFFFFF, u | 0x80000000)


def sample_ref(logits, temperature, top_k, top_p, uniforms):
    """Reference with the kernel's exact semantics (see sampling.hip):

    value-threshold top-k (keeps ties), value-threshold nucleus (smallest
    top set with mass >= p), inverse CDF over kept tokens in index order.
    """
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int32)
    for i in range(B):
        row = logits[i].float()
        temp = float(temperature[i])
        if temp <= 0.0:
            out[i] = int(torch.argmax(row))
            continue
        # thresholds live in the UNSCALED value domain (temperature > 0
        # preserves order; the bf16 kernel walks unscaled bf16 keys), the
        # exp-weights use the temperature
        inv_t = 1.0 / temp
        m = float(row.max())
        probs = torch.exp((row - m) * inv_t)
        Z = float(probs.sum())
        sorted_vals, _ = torch.sort(row, descending=True)
        k = int(top_k[i])
        tau_k = float("-inf")
        if 0 < k < V:
            tau_k = float(sorted_vals[k - 1])
        p = float(top_p[i])
        tau_p = float("-inf")
        if p < 1.0:
            sp = torch.exp((sorted_vals - m) * inv_t)
            cum = torch.cumsum(sp, 0)
            idx = int(torch.searchsorted(cum, p * Z))
            idx = min(idx, V - 1)
            tau_p = float(sorted_vals[idx])
        tau = max(tau_k, tau_p)
        keep = row >= tau
        masked = torch.where(keep, probs, torch.zeros(()))
        zf = float(masked.sum())
        target = float(uniforms[i]) * zf
        cdf = torch.cumsum(masked, 0)
        chosen = int(torch.searchsorted(cdf, target, right=True))
        chosen = min(chosen, V - 1)
        while masked[chosen] == 0 and chosen > 0:
            chosen -= 1
        out[i] = chosen
    return out


def moe_route_ref(logits: torch.Tensor, top_k: int, capacity: int):
    """Reference for the fused MoE routing kernel (moe_route.hip).

    Returns (weights [T,K] fp32, dst [T*K] int32, topk_idx [T,K] int32).
    dst = expert * capacity + rank; rank order within an expert is NOT
    part of the contract (the kernel uses atomic counters) — tests check
    validity, not order.
    """
    T, E = logits.shape
    vals, idx = torch.topk(logits.float(), top_k, dim=-1)
    weights = torch.softmax(vals, dim=-1)
    flat = idx.reshape(-1)
    onehot = torch.nn.functional.one_hot(flat, E)
    rank = (torch.cumsum(onehot, 0) - onehot).mul(onehot).sum(-1)
    dst = (flat * capacity + rank).to(torch.int32)
    counts = torch.bincount(flat, minlength=E).to(torch.int32)
    return weights, dst, idx.to(torch.int32), counts


def moe_grouped_gemm_ref(a, w, counts, capacity):
    """Per-expert GEMM reference: only rows < counts[e] are computed;
    padded rows of the output stay zero."""
    E, N, K = w.shape
    out = torch.zeros((a.shape[0], N), dtype=a.dtype)
    for e in range(E):
        c = int(counts[e])
        if c == 0:
            continue
        rows = a[e * capacity:e * capacity + c].float()
        out[e * capacity:e * capacity + c] = (
            rows @ w[e].float().T).to(a.dtype)
    return out


def silu_mul_grouped_ref(gate_up, counts, capacity):
    inter = gate_up.shape[-1] // 2
    out = torch.zeros((*gate_up.shape[:-1], inter), dtype=gate_up.dtype)
    E = counts.shape[0]
    for e in range(E):
        c = int(counts[e])
        if c:
            seg = gate_up[e * capacity:e * capacity + c]
            out[e * capacity:e * capacity + c] = silu_mul_ref(seg)
    return out


# ---------------------------------------------------------------------------
# Hybrid-decoder mechanisms (layer norm on an fp32 residual, minGRU scan,
# windowed latent attention with a softmax sink, xIELU / relu^2).  These are
# the CPU implementations behind ops.*; the GPU path runs the HIP kernels.
# Everything the recurrences, norms, angles and softmax touch is fp32.
# ---------------------------------------------------------------------------
def add_layernorm_ref(residual, delta, w, b, eps, out_dtype):
    """residual (fp32, in place) += delta; returns LayerNorm(residual)
    with weight/bias, variance = mean squared deviation."""
    if delta is not None:
        residual.add_(delta.float())
    mean = residual.mean(-1, keepdim=True)
    dev = residual - mean
    var = (dev * dev).mean(-1, keepdim=True)
    return (dev * torch.rsqrt(var + eps) * w + b).to(out_dtype)


def mingru_scan_ref(zug, state, seq_cu, seq_start, seq_slots):
    """zug [T, 3W] = (gate pre-activation | candidate pre-activation |
    output-gate pre-activation).  Per sequence and channel:
    S <- (1 - z) S + z * cand, y = S * silu(g).  state [slots, W] fp32
    carries S between steps; a sequence that starts at position 0 starts
    from zero whatever its slot held."""
    T, W3 = zug.shape
    W = W3 // 3
    x = zug.float()
    z = torch.sigmoid(x[:, :W])
    u = x[:, W:2 * W]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    a, bb = 1.0 - z, z * cand
    g = x[:, 2 * W:]
    out = torch.empty((T, W), dtype=torch.float32, device=zug.device)
    cu = seq_cu.tolist()
    starts = seq_start.tolist()
    slots = seq_slots.tolist()
    for s, slot in enumerate(slots):
        S = (state[slot].clone() if starts[s] > 0
             else torch.zeros(W, dtype=torch.float32, device=zug.device))
        for t in range(cu[s], cu[s + 1]):
            S = a[t] * S + bb[t]
            out[t] = S
        state[slot] = S
    return (out * (g * torch.sigmoid(g))).to(zug.dtype)


def _rope_pairs(x, positions, inv_freq):
    """Interleaved pairs (2i, 2i+1) of the last dim of x [T, ..., 2n]
    turned by positions * inv_freq[i]; fp32 in, fp32 out."""
    ang = positions.float().unsqueeze(-1) * inv_freq.float()   # [T, n]
    while ang.dim() < x.dim():
        ang = ang.unsqueeze(1)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0::2], x[..., 1::2]
    return torch.stack((u * c - v * s, v * c + u * s), -1).flatten(-2)


def rope_pairs_ref(x, positions, inv_freq, offset):
    """In place on x[..., offset : offset + 2*len(inv_freq)]."""
    n2 = 2 * inv_freq.numel()
    part = x[..., offset:offset + n2]
    part.copy_(_rope_pairs(part.float(), positions, inv_freq).to(x.dtype))
    return x


def latent_down_post_ref(down, positions, slot_mapping, cache, qnorm_w,
                         kvnorm_w, inv_freq, eps, q_rank, kv_rank, rot_dim,
                         heads):
    """Everything between the fused down projection and the up
    projections: RMS-norm the query latent, RMS-norm the key/value
    latent and write it with the rotated shared key into the paged
    cache, and squash the per-head output gate."""
    x = down.float()
    cq = x[:, :q_rank]
    cq = cq * torch.rsqrt((cq * cq).mean(-1, keepdim=True) + eps) * qnorm_w
    c = x[:, q_rank:q_rank + kv_rank]
    c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * kvnorm_w
    kr = x[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim].clone()
    n2 = 2 * inv_freq.numel()
    kr[:, :n2] = _rope_pairs(kr[:, :n2], positions, inv_freq)
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping.long()] = torch.cat([c, kr], -1).to(cache.dtype)
    gate = torch.sigmoid(x[:, q_rank + kv_rank + rot_dim:
                           q_rank + kv_rank + rot_dim + heads])
    return cq.to(down.dtype), gate


def latent_attention_ref(q_abs, q_rot, cache, block_table, row_seq,
                         positions, sink, scale, window):
    """Absorbed latent attention over the paged cache.  Row t of head h
    scores key j as (q_abs[t,h] . c_j + q_rot[t,h] . kr_j) * scale for
    pos-window < j <= pos; the softmax denominator also holds exp(sink_h).
    Returns the probability-weighted sum of latents [T, H, kv_rank]."""
    T, H, R = q_abs.shape
    bs = cache.shape[1]
    out = torch.zeros((T, H, R), dtype=torch.float32, device=q_abs.device)
    pos = positions.tolist()
    seqs = row_seq.tolist()
    flat = cache.view(-1, cache.shape[-1])
    qa, qr = q_abs.float(), q_rot.float()
    for t in range(T):
        p = pos[t]
        lo = max(0, p - window + 1) if window > 0 else 0
        j = torch.arange(lo, p + 1, device=q_abs.device)
        bt = block_table[seqs[t]].long()
        rows = flat[bt[j // bs] * bs + j % bs].float()        # [n, R+rd]
        sc = (qa[t] @ rows[:, :R].t() + qr[t] @ rows[:, R:].t()) * scale
        m = torch.maximum(sc.max(-1).values, sink)            # [H]
        e = torch.exp(sc - m[:, None])
        den = e.sum(-1) + torch.exp(sink - m)
        out[t] = (e @ rows[:, :R]) / den[:, None]
    return out.to(q_abs.dtype)


def xielu_ref(z, pq):
    """xIELU: softplus(p) z^2 + z/2 for z > 0, else
    (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    x = z.float()
    ap = torch.nn.functional.softplus(pq[0].float())
    an = 0.5 + torch.nn.functional.softplus(pq[1].float())
    neg = torch.clamp(x, max=0.0)
    y = torch.where(x > 0, ap * x * x + 0.5 * x,
                    an * (torch.expm1(neg) - neg) + 0.5 * x)
    return y.to(z.dtype)


def relu2_ref(z):
    r = torch.relu(z.float())
    return (r * r).to(z.dtype)


def gate_heads_ref(v, gate):
    """v [H, T, vd] per-head values, gate [T, H] fp32 -> [T, H*vd]."""
    H, T, vd = v.shape
    return (v.float().transpose(0, 1) * gate[:, :, None]).reshape(
        T, H * vd).to(v.dtype)


def moe_topk_route_ref(logits, top_k):
    """Top-k experts by logit and the softmax over just those k."""
    w, idx = torch.topk(logits, top_k, dim=-1)
    return torch.softmax(w, dim=-1), idx.to(torch.int32)


def rotary_inv_freq(base: float, dims: int, device="cpu"):
    """f_i = base**(-2i/dims), i < dims/2, evaluated in float64 and
    rounded once to fp32 (the angle position * f_i is an fp32 product)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / dims)).to(torch.float32).to(device)


# ---------------------------------------------------------------------------
# Parallel-block / sigmoid-attention mechanisms: one RMS statistic feeding
# two norms, whole-projection query/key norm with value blending and paged
# append, windowed sigmoid attention with a per-distance bias and mixing of
# the weights across heads, gated feed-forward activations.  CPU
# implementations behind ops.*; all arithmetic fp32.
# ---------------------------------------------------------------------------
def add_rmsnorm_pair_ref(residual, delta_a, delta_b, w1, w2, eps,
                         out_dtype):
    """residual (fp32, in place) += delta_a + delta_b (either may be
    None); returns (x/rms(x) * w1, x/rms(x) * w2) — the second is None
    when w2 is."""
    if delta_a is not None and delta_b is not None:
        residual.add_(delta_a.float() + delta_b.float())
    elif delta_a is not None:
        residual.add_(delta_a.float())
    elif delta_b is not None:
        residual.add_(delta_b.float())
    n = residual * torch.rsqrt(
        (residual * residual).mean(-1, keepdim=True) + eps)
    return ((n * w1).to(out_dtype),
            None if w2 is None else (n * w2).to(out_dtype))


def qk_norm_append_ref(proj, slot_mapping, kcache, vcache, qnorm_w,
                       knorm_w, v_first, lam, eps, H, G, dk, dv):
    """proj [T, H*dk | G*dk | G*dv | ...]: RMS-norm the WHOLE query
    block and the whole key block (one statistic each, over all heads),
    blend the values with v_first (v <- (1-lam) v + lam v_first) when
    given, append keys to [blocks, G, block, dk] and values to the
    page-transposed [blocks, G, dv, block]; returns the normed queries
    [T, H*dk]."""
    T = proj.shape[0]
    x = proj.float()
    nq, nk, nv = H * dk, G * dk, G * dv
    q = x[:, :nq]
    q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * qnorm_w
    k = x[:, nq:nq + nk]
    k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * knorm_w
    v = x[:, nq + nk:nq + nk + nv]
    if v_first is not None:
        v = (1.0 - lam) * v + lam * v_first.float()
    bs = kcache.shape[2]
    sm = slot_mapping.long()
    blk, off = sm // bs, sm % bs
    kcache[blk, :, off] = k.view(T, G, dk).to(kcache.dtype)
    vcache[blk, :, :, off] = v.view(T, G, dv).to(vcache.dtype)
    return q.to(proj.dtype)


def sigmoid_attention_ref(q, kcache, vcache, block_table, row_seq,
                          positions, dist_bias, talk, gate, scale, window):
    """Row t (position p) of head g weighs key j, max(0, p-window+1) <= j
    <= p, with sigmoid((q . k_j) * scale + dist_bias[min(p-j, last), g]);
    head h then uses sum_g talk[h, g] * weight_g on the values of its own
    key/value head.  The result, times sigmoid(gate), is [T, H*dv]."""
    T = q.shape[0]
    H = talk.shape[0]
    G, bs, dk = kcache.shape[1], kcache.shape[2], kcache.shape[3]
    dv = vcache.shape[2]            # values are [blocks, G, dv, block]
    per = H // G
    last = dist_bias.shape[0] - 1
    out = torch.zeros((T, H, dv), dtype=torch.float32, device=q.device)
    qf = q.float().view(T, G, per, dk)
    pos = positions.tolist()
    seqs = row_seq.tolist()
    talk = talk.float()
    for t in range(T):
        p = pos[t]
        lo = max(0, p - window + 1) if window > 0 else 0
        j = torch.arange(lo, p + 1, device=q.device)
        bt = block_table[seqs[t]].long()
        blk, off = bt[j // bs], j % bs
        kk = kcache[blk, :, off].float()                 # [n, G, dk]
        vv = vcache[blk, :, :, off].float()              # [n, G, dv]
        sc = torch.einsum("gpd,ngd->gpn", qf[t], kk).reshape(H, -1) * scale
        bias = dist_bias[torch.clamp(p - j, max=last)]   # [n, H]
        w = torch.sigmoid(sc + bias.t())
        mixed = (talk @ w).view(G, per, -1)
        out[t] = torch.einsum("gpn,ngd->gpd", mixed, vv).reshape(H, dv)
    out = out.view(T, H * dv) * torch.sigmoid(gate.float())
    return out.to(q.dtype)


GATED_ACT_SILU = 0       # silu(g) * u
GATED_ACT_CLAMPED = 1    # min(g, L) * sigmoid(alpha * min(g, L))
                         #   * (clamp(u, -L, L) + 1)


def gated_act_ref(gate_up, mode, limit=0.0, alpha=1.0):
    """gate_up [..., 2f] = (gate | up) -> [..., f]."""
    f = gate_up.shape[-1] // 2
    g, u = gate_up[..., :f].float(), gate_up[..., f:].float()
    if mode == GATED_ACT_SILU:
        y = g * torch.sigmoid(g) * u
    else:
        g = torch.clamp(g, max=limit)
        u = torch.clamp(u, min=-limit, max=limit)
        y = g * torch.sigmoid(alpha * g) * (u + 1.0)
    return y.to(gate_up.dtype)
