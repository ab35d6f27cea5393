"""Op dispatch for the MI355X engine.

On a GPU box the hand-written gfx950 HIP kernels (_kernels extension) are
REQUIRED — if a CUDA/HIP device is visible and the extension is missing,
every op raises instead of silently falling back to eager PyTorch (the
round-end harness records which .so files the GPU processes load). On CPU
the fp32 torch references (torch_ref) run so the whole engine and gateway
are testable without a GPU.
"""
from __future__ import annotations

import torch

from . import torch_ref

try:
    from . import _kernels  # compiled by setup.py build_ext --inplace

    HAS_KERNELS = True
except ImportError:  # pragma: no cover - absent only before first build
    _kernels = None
    HAS_KERNELS = False


try:
    from . import _hybrid  # recurrent / latent-attention mechanisms

    HAS_HYBRID = True
except ImportError:  # pragma: no cover - absent only before first build
    _hybrid = None
    HAS_HYBRID = False


def _require_hybrid() -> None:
    if not HAS_HYBRID:
        raise RuntimeError(
            "inference_gateway_amd.ops._hybrid is not built but a GPU "
            "tensor was passed. Build it in-tree with: IGW_BUILD_EXT=hybrid "
            "PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace"
        )


def _require_kernels() -> None:
    if not HAS_KERNELS:
        raise RuntimeError(
            "inference_gateway_amd.ops._kernels is not built but a GPU tensor "
            "was passed. Build it in-tree with: "
            "PYTORCH_ROCM_ARCH=gfx950 python setup.py build_ext --inplace"
        )


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda:
        _require_kernels()
        out = torch.empty_like(x)
        _kernels.rmsnorm(out, x, weight, eps)
        return out
    return torch_ref.rmsnorm_ref(x, weight, eps)


def fused_add_rmsnorm(x, residual, weight, eps: float):
    """In-place: residual += x; x = rmsnorm(residual) * w. Returns (x, residual)."""
    if x.is_cuda:
        _require_kernels()
        _kernels.fused_add_rmsnorm(x, residual, weight, eps)
        return x, residual
    nx, nres = torch_ref.fused_add_rmsnorm_ref(x, residual, weight, eps)
    x.copy_(nx)
    residual.copy_(nres)
    return x, residual


def rotary_embedding(positions, q, k, head_dim: int, cos_sin_cache):
    """In-place NeoX RoPE on q [T, NQ*HD] and k [T, NKV*HD]."""
    if q.is_cuda:
        _require_kernels()
        _kernels.rotary_embedding(positions, q, k, head_dim, cos_sin_cache)
        return q, k
    nq, nk = torch_ref.rope_ref(positions, q, k, head_dim, cos_sin_cache)
    q.copy_(nq)
    k.copy_(nk)
    return q, k


def append_kv_cache(k, v, kcache, vcache, slot_mapping):
    if k.is_cuda:
        _require_kernels()
        _kernels.append_kv_cache(k, v, kcache, vcache, slot_mapping)
        return
    torch_ref.append_kv_cache_ref(k, v, kcache, vcache, slot_mapping)


def paged_attn_decode(q, kcache, vcache, block_table, ctx_lens, scale: float):
    if q.is_cuda:
        _require_kernels()
        out = torch.empty_like(q)
        _kernels.paged_attn_decode(
            out, q, kcache, vcache, block_table, ctx_lens, scale
        )
        return out
    return torch_ref.paged_attn_decode_ref(
        q, kcache, vcache, block_table, ctx_lens, scale
    )


def flash_prefill(q, k, v, cu_seqlens, seq_lens, scale: float):
    """Varlen causal prefill attention. seq_lens: python list of ints."""
    if q.is_cuda:
        _require_kernels()
        out = torch.empty_like(q)
        tile_seq, tile_off = torch_ref.make_prefill_tiles(
            seq_lens, tile_m=64, device=q.device
        )
        _kernels.flash_prefill(
            out, q, k, v, cu_seqlens, tile_seq, tile_off, scale
        )
        return out
    return torch_ref.flash_prefill_ref(q, k, v, cu_seqlens, scale)


def flash_prefill_paged(q, kcache, vcache, block_table, prefix_lens,
                        cu_seqlens, seq_lens, scale: float):
    """Paged-EXTEND prefill (chunked-prefill / prefix-cache enabler):
    q rows are a per-seq CHUNK whose own K/V plus `prefix_lens` cached
    tokens before it are all in the paged cache; each q row attends over
    cache positions [0, prefix + row].  seq_lens: python ints (q rows
    per sequence)."""
    if q.is_cuda:
        _require_kernels()
        out = torch.empty_like(q)
        tile_seq, tile_off = torch_ref.make_prefill_tiles(
            seq_lens, tile_m=64, device=q.device
        )
        _kernels.flash_prefill_paged(
            out, q, kcache, vcache, block_table, prefix_lens, cu_seqlens,
            tile_seq, tile_off, scale
        )
        return out
    return torch_ref.flash_prefill_paged_ref(
        q, kcache, vcache, block_table, prefix_lens, cu_seqlens, scale
    )


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    if gate_up.is_cuda:
        _require_kernels()
        inter = gate_up.shape[-1] // 2
        out = torch.empty(
            (*gate_up.shape[:-1], inter),
            dtype=gate_up.dtype,
            device=gate_up.device,
        )
        _kernels.silu_mul(out, gate_up)
        return out
    return torch_ref.silu_mul_ref(gate_up)


def sample(logits, temperature, top_k, top_p, uniforms):
    """logits [B, V] fp32 -> sampled token ids [B] int32."""
    if logits.is_cuda:
        _require_kernels()
        out = torch.empty(
            logits.shape[0], dtype=torch.int32, device=logits.device
        )
        _kernels.sample(out, logits, temperature, top_k, top_p, uniforms)
        return out
    return torch_ref.sample_ref(logits, temperature, top_k, top_p, uniforms)


build_cos_sin_cache = torch_ref.build_cos_sin_cache
rotary_inv_freq = torch_ref.rotary_inv_freq
make_prefill_tiles = torch_ref.make_prefill_tiles


def moe_route(router_logits: torch.Tensor, top_k: int, capacity: int):
    """Fused MoE routing: top-k + softmax + padded-dispatch row indices.

    router_logits: [T, E] fp32. Returns (weights [T,K] fp32,
    dst [T*K] int32, topk_idx [T,K] int32, counts [E] int32)."""
    if router_logits.is_cuda:
        _require_kernels()
        T, E = router_logits.shape
        weights = torch.empty((T, top_k), dtype=torch.float32,
                              device=router_logits.device)
        dst = torch.empty(T * top_k, dtype=torch.int32,
                          device=router_logits.device)
        topk_idx = torch.empty((T, top_k), dtype=torch.int32,
                               device=router_logits.device)
        counts = torch.empty(E, dtype=torch.int32,
                             device=router_logits.device)
        _kernels.moe_route(weights, dst, topk_idx, counts, router_logits,
                           capacity)
        return weights, dst, topk_idx, counts
    return torch_ref.moe_route_ref(router_logits, top_k, capacity)


def moe_grouped_gemm(a: torch.Tensor, w: torch.Tensor,
                     counts: torch.Tensor, capacity: int) -> torch.Tensor:
    """Per-expert GEMM over the padded dispatch buffer.

    a: [E*C, K] bf16 (rows >= counts[e] in each expert segment are
    ignored), w: [E, N, K] bf16 -> out [E*C, N] bf16 (only real rows
    written)."""
    if a.is_cuda:
        _require_kernels()
        E, N, _K = w.shape
        out = torch.empty((a.shape[0], N), dtype=a.dtype, device=a.device)
        _kernels.moe_grouped_gemm(out, a, w, counts, capacity)
        return out
    return torch_ref.moe_grouped_gemm_ref(a, w, counts, capacity)


def silu_mul_grouped(gate_up: torch.Tensor, counts: torch.Tensor,
                     capacity: int) -> torch.Tensor:
    """SwiGLU over only the real rows of the padded dispatch buffer."""
    if gate_up.is_cuda:
        _require_kernels()
        inter = gate_up.shape[-1] // 2
        out = torch.empty((*gate_up.shape[:-1], inter), dtype=gate_up.dtype,
                          device=gate_up.device)
        _kernels.silu_mul_grouped(out, gate_up, counts, capacity)
        return out
    return torch_ref.silu_mul_grouped_ref(gate_up, counts, capacity)


def fused_gemm_tn(x: torch.Tensor, w: torch.Tensor, swiglu: bool = False,
                  nt_weights: bool = False) -> torch.Tensor:
    """TN bf16 GEMM out = x @ w.T with an optional fused SwiGLU
    epilogue (w = [gate; up] rows, out = silu(g)*u).  Decode
    weight-streaming shapes (M%128==0, N%64==0, K%32==0); callers fall
    back to the library GEMM otherwise (ops/csrc/fused_gemm.hip)."""
    if x.is_cuda:
        _require_kernels()
        N = w.shape[0] // 2 if swiglu else w.shape[0]
        out = torch.empty((x.shape[0], N), dtype=x.dtype, device=x.device)
        _kernels.fused_gemm_tn(out, x, w, swiglu, nt_weights)
        return out
    y = x.float() @ w.float().t()
    if swiglu:
        N = w.shape[0] // 2
        g, u = y[:, :N], y[:, N:]
        y = torch.nn.functional.silu(g) * u
    return y.to(x.dtype)


def fused_gemm_tn_supported(M: int, N_rows: int, K: int,
                            swiglu: bool) -> bool:
    N = N_rows // 2 if swiglu else N_rows
    return M % 128 == 0 and N % 64 == 0 and K % 32 == 0


# ---------------------------------------------------------------------------
# Hybrid-decoder mechanisms: fp32-residual LayerNorm, minGRU scan, windowed
# latent attention with a softmax sink, xIELU / relu^2 activations.  The
# kernels are typed for bf16 AND fp32 activations (true 32-bit serving);
# norms, recurrent state, angles and softmax are fp32 in both.
# ---------------------------------------------------------------------------
def add_layernorm(residual, delta, weight, bias, eps: float, out_dtype):
    """residual [T, D] fp32 += delta (in place; delta may be None);
    returns LayerNorm(residual) * weight + bias in out_dtype."""
    if residual.is_cuda:
        _require_hybrid()
        out = torch.empty(residual.shape, dtype=out_dtype,
                          device=residual.device)
        _hybrid.add_layernorm(out, residual, delta, weight, bias, eps)
        return out
    return torch_ref.add_layernorm_ref(residual, delta, weight, bias, eps,
                                       out_dtype)


# rows per chunk of the chunked minGRU scan, and the segment length from
# which it replaces the one-thread-per-channel walk
MINGRU_CHUNK = 16
MINGRU_CHUNKED_FROM = 256


def mingru_scan(zug, state, seq_cu, seq_start, seq_slots, seq_rows):
    """minGRU recurrence + output gate over a ragged batch.  zug [T, 3W]
    (z | x | g pre-activations), state [slots, W] fp32 (read when the
    sequence's first row is not position 0, always written back).
    seq_rows: python row counts per sequence (host side; picks the
    sequential or the chunked-scan schedule and lays out its chunks)."""
    if zug.is_cuda:
        _require_hybrid()
        W = zug.shape[1] // 3
        out = torch.empty((zug.shape[0], W), dtype=zug.dtype,
                          device=zug.device)
        if max(seq_rows) < MINGRU_CHUNKED_FROM:
            _hybrid.mingru_scan(out, zug, state, seq_cu, seq_start,
                                seq_slots)
            return out
        tab, ccu_t = _scan_chunks(tuple(seq_rows), MINGRU_CHUNK, zug.device)
        work = torch.empty((2, tab.shape[1], W), dtype=torch.float32,
                           device=zug.device)
        _hybrid.mingru_scan_chunked(out, zug, state, seq_start, seq_slots,
                                    tab[0], tab[1], ccu_t, work)
        return out
    return torch_ref.mingru_scan_ref(zug, state, seq_cu, seq_start,
                                     seq_slots)


def rope_pairs_(x, positions, inv_freq, offset: int):
    """In-place interleaved-pair rotation of x[T, H, hd][..., offset :
    offset + 2*len(inv_freq)] by positions * inv_freq (fp32 angles)."""
    if x.is_cuda:
        _require_hybrid()
        _hybrid.rope_pairs(x, positions, inv_freq, offset)
        return x
    return torch_ref.rope_pairs_ref(x, positions, inv_freq, offset)


def latent_down_post(down, positions, slot_mapping, cache, qnorm_w,
                     kvnorm_w, inv_freq, eps: float, q_rank: int,
                     kv_rank: int, rot_dim: int, heads: int):
    """Post-processing of the fused down projection [T, q_rank + kv_rank
    + rot_dim + heads]: returns (normed query latent [T, q_rank],
    sigmoid head gates [T, heads] fp32) and appends (normed latent |
    rotated shared key) to the paged cache at slot_mapping."""
    if down.is_cuda:
        _require_hybrid()
        T = down.shape[0]
        cq = torch.empty((T, q_rank), dtype=down.dtype, device=down.device)
        gate = torch.empty((T, heads), dtype=torch.float32,
                           device=down.device)
        _hybrid.latent_down_post(cq, gate, down, positions, slot_mapping,
                                  cache, qnorm_w, kvnorm_w, inv_freq, eps,
                                  q_rank, kv_rank, rot_dim, heads)
        return cq, gate
    return torch_ref.latent_down_post_ref(
        down, positions, slot_mapping, cache, qnorm_w, kvnorm_w, inv_freq,
        eps, q_rank, kv_rank, rot_dim, heads)


import functools


@functools.lru_cache(maxsize=256)
def _attention_tiles(tq: int, num_prefill_rows: int, seq_lens: tuple,
                     T: int, device):
    """[2, ntiles] int32 (first row, row count) of the attention tiles:
    prompt portions cut into runs of tq rows, decoded rows one each.
    Cached: serving repeats the same batch shapes."""
    row0, nrows, row = [], [], 0
    for n in seq_lens:
        for a in range(0, n, tq):
            row0.append(row + a)
            nrows.append(min(tq, n - a))
        row += n
    assert row == num_prefill_rows
    row0.extend(range(num_prefill_rows, T))
    nrows.extend([1] * (T - num_prefill_rows))
    return torch.tensor([row0, nrows], dtype=torch.int32).to(device)


@functools.lru_cache(maxsize=256)
def _scan_chunks(seq_rows: tuple, chunk: int, device):
    """Chunk table of the chunked minGRU scan: ([2, NC] row ranges,
    [S+1] chunk offsets per sequence), cached per batch shape."""
    r0, r1, ccu, row = [], [], [0], 0
    for n in seq_rows:
        for a in range(0, n, chunk):
            r0.append(row + a)
            r1.append(row + min(n, a + chunk))
        row += n
        ccu.append(len(r0))
    return (torch.tensor([r0, r1], dtype=torch.int32).to(device),
            torch.tensor(ccu, dtype=torch.int32).to(device))


# bf16 batches run the MFMA tile kernel; off = the one-wave-per-row kernel
# (any dtype, any sizes) for everything
LATENT_ATTENTION_MFMA = True


def latent_attention(q_abs, q_rot, cache, block_table, row_seq, positions,
                     sink, scale: float, window: int,
                     num_prefill_rows: int = 0, prefill_seq_lens=None,
                     max_context: int = 0):
    """Absorbed latent attention (all heads share one cached latent per
    token) with a sliding window and a per-head softmax sink.
    q_abs [T, H, kv_rank], q_rot [T, H, rot_dim] (strided views ok),
    cache [blocks, block, kv_rank + rot_dim].  Rows [0, num_prefill_rows)
    are prompt portions (prefill_seq_lens = python row counts per
    sequence), the rest are single decoded tokens; max_context is a host
    hint (longest sequence in the batch) for splitting keys over
    workgroups."""
    if q_abs.is_cuda:
        _require_hybrid()
        T, H, R = q_abs.shape
        out = torch.empty((T, H, R), dtype=q_abs.dtype, device=q_abs.device)
        if q_abs.dtype == torch.bfloat16 and LATENT_ATTENTION_MFMA:
            tiles = _attention_tiles(
                _hybrid.latent_attention_tile_rows(H), num_prefill_rows,
                tuple(prefill_seq_lens or ()) if num_prefill_rows else (),
                T, q_abs.device)
            ctx = max_context or 4096
            max_keys = min(window, ctx) if window > 0 else ctx
            if _hybrid.latent_attention_mfma(
                    out, q_abs, q_rot, cache, block_table, row_seq,
                    positions, tiles[0], tiles[1], sink, scale, window,
                    max_keys):
                return out
        _hybrid.latent_attention(out, q_abs, q_rot, cache, block_table,
                                 row_seq, positions, sink, scale, window)
        return out
    return torch_ref.latent_attention_ref(
        q_abs, q_rot, cache, block_table, row_seq, positions, sink, scale,
        window)


def xielu(z, pq):
    if z.is_cuda:
        _require_hybrid()
        out = torch.empty_like(z)
        _hybrid.xielu(out, z, pq)
        return out
    return torch_ref.xielu_ref(z, pq)


def relu2(z):
    if z.is_cuda:
        _require_hybrid()
        out = torch.empty_like(z)
        _hybrid.relu2(out, z)
        return out
    return torch_ref.relu2_ref(z)


def gate_heads(v, gate):
    """v [H, T, vd] (strided ok), gate [T, H] fp32 -> [T, H*vd]."""
    if v.is_cuda:
        _require_hybrid()
        H, T, vd = v.shape
        out = torch.empty((T, H * vd), dtype=v.dtype, device=v.device)
        _hybrid.gate_heads(out, v, gate)
        return out
    return torch_ref.gate_heads_ref(v, gate)


def moe_topk_route(logits, top_k: int, capacity: int = 0,
                   scale: float = 1.0):
    """logits [T, E] fp32 -> (softmax-over-chosen weights [T, K] fp32
    times `scale`,
    expert ids [T, K] int32, padded rows [T*K] int64 or None).  With
    capacity > 0 (>= T) the padded-dispatch row of every assignment,
    expert * capacity + rank, comes from the same launch.  Any K <= E <=
    64 on the GPU kernel, wider routers take the library top-k."""
    if logits.is_cuda and logits.shape[1] <= 64:
        _require_hybrid()
        T, E = logits.shape
        w = torch.empty((T, top_k), dtype=torch.float32,
                        device=logits.device)
        idx = torch.empty((T, top_k), dtype=torch.int32,
                          device=logits.device)
        dst = counts = None
        if capacity > 0:
            dst = torch.empty(T * top_k, dtype=torch.int64,
                              device=logits.device)
            counts = torch.zeros(E, dtype=torch.int32, device=logits.device)
        _hybrid.moe_topk_route(w, idx, logits, dst, counts, capacity,
                               scale)
        return w, idx, dst
    w, idx = torch_ref.moe_topk_route_ref(logits, top_k)
    return (w * scale if scale != 1.0 else w), idx, None


# ---------------------------------------------------------------------------
# Parallel-block / sigmoid-attention mechanisms (same extension, same
# typing rules: bf16 or fp32 activations, fp32 arithmetic).
# ---------------------------------------------------------------------------
GATED_ACT_SILU = torch_ref.GATED_ACT_SILU
GATED_ACT_CLAMPED = torch_ref.GATED_ACT_CLAMPED


def add_rmsnorm_pair(residual, delta_a, delta_b, w1, w2, eps: float,
                     out_dtype):
    """residual [T, D] fp32 += delta_a + delta_b (in place; either may
    be None).  Returns (rmsnorm(residual) * w1, rmsnorm(residual) * w2)
    from ONE pass and one statistic; w2 None gives (out, None)."""
    if residual.is_cuda:
        _require_hybrid()
        out1 = torch.empty(residual.shape, dtype=out_dtype,
                           device=residual.device)
        out2 = None if w2 is None else torch.empty_like(out1)
        _hybrid.add_rmsnorm_pair(out1, out2, residual, delta_a, delta_b,
                                 w1, w2, eps)
        return out1, out2
    return torch_ref.add_rmsnorm_pair_ref(residual, delta_a, delta_b, w1,
                                          w2, eps, out_dtype)


def qk_norm_append(proj, slot_mapping, kcache, vcache, qnorm_w, knorm_w,
                   v_first, lam: float, eps: float, heads: int,
                   kv_heads: int, dim: int, vdim: int):
    """Post-processing of a fused projection [T, H*dim | G*dim | G*vdim |
    ...]: RMS norm over the whole query block and over the whole key
    block, optional value blend (1-lam) v + lam v_first (v_first [T,
    G*vdim], strided rows ok), keys and values appended to the paged
    caches (keys [blocks, G, block, dim], values page-transposed
    [blocks, G, vdim, block]).  Returns the normed queries."""
    if proj.is_cuda:
        _require_hybrid()
        q = torch.empty((proj.shape[0], heads * dim), dtype=proj.dtype,
                        device=proj.device)
        _hybrid.qk_norm_append(q, proj, slot_mapping, kcache, vcache,
                               qnorm_w, knorm_w, v_first, lam, eps, heads,
                               kv_heads, dim, vdim)
        return q
    return torch_ref.qk_norm_append_ref(
        proj, slot_mapping, kcache, vcache, qnorm_w, knorm_w, v_first, lam,
        eps, heads, kv_heads, dim, vdim)


# bf16 batches run the MFMA tile kernel; off = the block-per-row kernel
# (any dtype, any sizes) for everything
SIGMOID_ATTENTION_MFMA = True


def sigmoid_attention(q, kcache, vcache, block_table, row_seq, positions,
                      dist_bias, talk, gate, scale: float, window: int,
                      num_prefill_rows: int = 0, prefill_seq_lens=None,
                      max_context: int = 0):
    """Windowed sigmoid attention over the paged cache with a bias per
    (distance, head) (dist_bias [ND, H] fp32, distances from ND-1 on
    share the last row), the heads' weights mixed by talk [H, H], grouped
    key/value heads, and a sigmoid output gate (gate [T, H*vdim]
    pre-activations, strided rows ok).  q [T, H*dim]; returns [T,
    H*vdim].  Rows [0, num_prefill_rows) are prompt portions
    (prefill_seq_lens = python row counts per sequence), the rest single
    decoded tokens; every row reads its keys from the cache.
    max_context is a host hint (longest sequence in the batch) for
    splitting keys over workgroups."""
    if q.is_cuda:
        _require_hybrid()
        T = q.shape[0]
        H = talk.shape[0]
        out = torch.empty((T, H * vcache.shape[2]), dtype=q.dtype,
                          device=q.device)
        if q.dtype == torch.bfloat16 and SIGMOID_ATTENTION_MFMA:
            tq = _hybrid.sigmoid_attention_tile_rows()
            tiles = _attention_tiles(
                tq, num_prefill_rows,
                tuple(prefill_seq_lens or ()) if num_prefill_rows else (),
                T, q.device)
            ctx = max_context or 4096
            max_keys = min(window, ctx) if window > 0 else ctx
            if _hybrid.sigmoid_attention_mfma(
                    out, q, kcache, vcache, block_table, row_seq, positions,
                    tiles[0], tiles[1], dist_bias, talk, gate, scale,
                    window, max_keys, num_prefill_rows):
                return out
        _hybrid.sigmoid_attention(out, q, kcache, vcache, block_table,
                                  row_seq, positions, dist_bias, talk, gate,
                                  scale, window)
        return out
    return torch_ref.sigmoid_attention_ref(
        q, kcache, vcache, block_table, row_seq, positions, dist_bias, talk,
        gate, scale, window)


def gated_act(gate_up, mode: int, limit: float = 0.0, alpha: float = 1.0):
    """(gate | up) halves of the last dim -> one activation:
    GATED_ACT_SILU silu(g) * u; GATED_ACT_CLAMPED with g' = min(g, limit),
    u' = clamp(u, -limit, limit): g' * sigmoid(alpha g') * (u' + 1)."""
    if gate_up.is_cuda:
        _require_hybrid()
        f = gate_up.shape[-1] // 2
        out = torch.empty((*gate_up.shape[:-1], f), dtype=gate_up.dtype,
                          device=gate_up.device)
        _hybrid.gated_act(out, gate_up, mode, limit, alpha)
        return out
    return torch_ref.gated_act_ref(gate_up, mode, limit, alpha)
