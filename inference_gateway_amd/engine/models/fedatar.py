"""Fedatar: a per-layer hybrid decoder for the MI355X engine.

Each layer is pre-norm (LayerNorm with bias on an fp32 residual stream)
around one MIXER and, optionally, one FEED-FORWARD, both chosen per layer
by the configuration:

  mixers         MinGRUMixer      gated linear recurrence, one fp32 state
                                  vector per sequence slot
                 LatentAttention  low-rank (latent) queries and keys/values,
                                  one rotated key part shared by all heads,
                                  sliding window, per-head softmax sink,
                                  per-head sigmoid output gate; only the
                                  latent and the rotated key are paged
  feed-forwards  XieluMLP         dense, xIELU activation
                 Relu2MoE         top-k routed relu^2 experts (+ optional
                                  always-on shared expert)

The mechanisms are separate modules with their constants as arguments so
other designs can assemble them differently.  GEMMs go through
F.linear/bmm (hipBLASLt / rocBLAS); everything between them is a gfx950
kernel from ops (fp32 math for norms, angles, softmax, gates and the
recurrence; bf16 or fp32 activations).
"""
from __future__ import annotations

from typing import List

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import ops
from ...parallel.comm import tp_world_size
from ...parallel.layers import _init_weight
from ..config import (DenseFFSpec, FedatarConfig, LatentAttentionSpec,
                      MinGRUSpec, MoEFFSpec)
from . import moe_common
from .batch import ForwardBatch
from .llama import _seed


def _param(t: torch.Tensor) -> nn.Parameter:
    return nn.Parameter(t.contiguous(), requires_grad=False)


def _rand(shape, device, dtype, name: str, scale: float = 1.0):
    return _init_weight(shape, device, torch.float32, _seed(name)).mul_(
        scale).to(dtype)


class LayerNormParams(nn.Module):
    """Weight and bias of a LayerNorm, held in fp32 (the norm runs in
    fp32 on the fp32 residual — ops.add_layernorm)."""

    def __init__(self, n: int, device, name: str):
        super().__init__()
        self.weight = _param(1.0 + _rand((n,), device, torch.float32,
                                         name + ".w", 2.0))
        self.bias = _param(_rand((n,), device, torch.float32, name + ".b"))


class MinGRUMixer(nn.Module):
    """S_t = (1 - z_t) S_{t-1} + z_t c_t with z = sigmoid(W_z h + b_z),
    c = cand(W_x h + b_x), cand(u) = u + 1/2 (u >= 0) | sigmoid(u);
    out = W_o (S_t * silu(W_g h)).  The three input projections are one
    fused GEMM; the recurrence, gates and the state are fp32."""

    cache_kind = "state"

    def __init__(self, hidden: int, spec: MinGRUSpec, name: str, device,
                 dtype):
        super().__init__()
        W = self.width = spec.width
        s = hidden ** -0.5 / 0.02
        self.zxg = _param(_rand((3 * W, hidden), device, dtype,
                                name + ".zxg", s))
        b = _rand((3 * W,), device, dtype, name + ".zxg_b", 25.0)
        b[2 * W:] = 0          # the output gate has no bias
        self.zxg_b = _param(b)
        self.o = _param(_rand((hidden, W), device, dtype, name + ".o",
                              W ** -0.5 / 0.02))

    def cache_width(self) -> int:
        return self.width

    def forward(self, h: torch.Tensor, fb: ForwardBatch,
                state: torch.Tensor) -> torch.Tensor:
        zxg = F.linear(h, self.zxg, self.zxg_b)
        y = ops.mingru_scan(zxg, state, fb.seq_cu, fb.seq_start,
                            fb.seq_slots, fb.seq_rows)
        return F.linear(y, self.o)


class LatentAttention(nn.Module):
    """Attention through low-rank latents, computed in ABSORBED form:
    the per-head key up-projection is folded into the query
    (q_abs = W_uk^T q_unrotated) and the value up-projection is applied
    after the probability-weighted sum of latents, so every head reads
    the same cached row (latent | rotated key) — prefill portions and
    decoded tokens both attend straight out of the paged cache."""

    cache_kind = "latent"

    def __init__(self, hidden: int, spec: LatentAttentionSpec, eps: float,
                 name: str, device, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        H, dn, rd = spec.heads, spec.dim, spec.rot_dim
        R, vd, qr = spec.kv_rank, spec.vdim, spec.q_rank
        s = hidden ** -0.5 / 0.02
        # fused down projection: query latent | kv latent | rotated key
        # | per-head output-gate logits
        self.down = _param(_rand((qr + R + rd + H, hidden), device, dtype,
                                 name + ".down", s))
        self.qnorm_w = _param(1.0 + _rand((qr,), device, torch.float32,
                                          name + ".qn", 2.0))
        self.kvnorm_w = _param(1.0 + _rand((R,), device, torch.float32,
                                           name + ".kvn", 2.0))
        self.uq = _param(_rand((H * (dn + rd), qr), device, dtype,
                               name + ".uq", qr ** -0.5 / 0.02))
        # absorbed forms, per head: uk [H, dn, R] maps an unrotated query
        # to latent space; uv_t [H, R, vd] maps a latent sum to values
        self.uk = _param(_rand((H, dn, R), device, dtype, name + ".uk",
                               R ** -0.5 / 0.02))
        self.uv_t = _param(_rand((H, R, vd), device, dtype, name + ".uv",
                                 R ** -0.5 / 0.02))
        self.sink = _param(_rand((H,), device, torch.float32,
                                 name + ".sink", 25.0))
        self.o = _param(_rand((hidden, H * vd), device, dtype, name + ".o",
                              (H * vd) ** -0.5 / 0.02))
        self.inv_freq = _param(ops.rotary_inv_freq(
            spec.rot.base, spec.rot.dims, device))

    def cache_width(self) -> int:
        return self.spec.cache_width

    def forward(self, h: torch.Tensor, fb: ForwardBatch,
                cache: torch.Tensor) -> torch.Tensor:
        sp = self.spec
        T = h.shape[0]
        H, dn, rd = sp.heads, sp.dim, sp.rot_dim
        down = F.linear(h, self.down)
        cq, gate = ops.latent_down_post(
            down, fb.positions, fb.slot_mapping, cache, self.qnorm_w,
            self.kvnorm_w, self.inv_freq, self.eps, sp.q_rank, sp.kv_rank,
            rd, H)
        q = F.linear(cq, self.uq).view(T, H, dn + rd)
        ops.rope_pairs_(q, fb.positions, self.inv_freq, dn)
        q_abs = torch.bmm(q[:, :, :dn].transpose(0, 1), self.uk)  # [H,T,R]
        o_lat = ops.latent_attention(
            q_abs.transpose(0, 1), q[:, :, dn:], cache, fb.seq_block_table,
            fb.row_seq, fb.positions, self.sink, sp.scale, sp.window,
            fb.num_chunk_rows, fb.seq_lens, fb.max_context)
        v = torch.bmm(o_lat.transpose(0, 1), self.uv_t)           # [H,T,vd]
        return F.linear(ops.gate_heads(v, gate), self.o)


class XieluMLP(nn.Module):
    """W_down xielu(W_up h); the activation's two shape numbers are
    learned per layer and kept in fp32."""

    def __init__(self, hidden: int, spec: DenseFFSpec, name: str, device,
                 dtype):
        super().__init__()
        self.up = _param(_rand((spec.ff, hidden), device, dtype,
                               name + ".up", hidden ** -0.5 / 0.02))
        self.down = _param(_rand((hidden, spec.ff), device, dtype,
                                 name + ".down", spec.ff ** -0.5 / 0.02))
        self.act = _param(_rand((2,), device, torch.float32,
                                name + ".act", 25.0))

    def forward(self, h: torch.Tensor, fb: ForwardBatch) -> torch.Tensor:
        return F.linear(ops.xielu(F.linear(h, self.up), self.act),
                        self.down)


class Relu2MoE(nn.Module):
    """Top-k routed experts W_down relu(W_up h)^2, mixed with the
    softmax over the k chosen router logits (fp32 router with bias),
    plus an optional shared expert of the same form for every token.
    Expert weights are stored K-major ([E, in, out]) for the batched
    GEMMs, as the Mixtral experts are."""

    # above this many rows the sorted per-expert route replaces the
    # padded batched route (engine/models/moe_common.py)
    PADDED_MAX_ROWS = 256

    def __init__(self, hidden: int, spec: MoEFFSpec, name: str, device,
                 dtype):
        super().__init__()
        self.spec = spec
        E, f = spec.experts, spec.expert_ff
        self.router_w = _param(_rand((E, hidden), device, torch.float32,
                                     name + ".router",
                                     hidden ** -0.5 / 0.02))
        self.router_b = _param(_rand((E,), device, torch.float32,
                                     name + ".router_b", 5.0))
        self.up_t = _param(_rand((E, hidden, f), device, dtype,
                                 name + ".up", hidden ** -0.5 / 0.02))
        self.down_t = _param(_rand((E, f, hidden), device, dtype,
                                   name + ".down", f ** -0.5 / 0.02))
        if spec.shared_ff:
            sf = spec.shared_ff
            self.shared_up = _param(_rand((sf, hidden), device, dtype,
                                          name + ".sup",
                                          hidden ** -0.5 / 0.02))
            self.shared_down = _param(_rand((hidden, sf), device, dtype,
                                            name + ".sdown",
                                            sf ** -0.5 / 0.02))
        else:
            self.shared_up = self.shared_down = None

    def forward(self, h: torch.Tensor, fb: ForwardBatch) -> torch.Tensor:
        T = h.shape[0]
        E, K = self.spec.experts, self.spec.top
        logits = F.linear(h.float(), self.router_w, self.router_b)
        padded = T <= self.PADDED_MAX_ROWS
        C = (T + 63) // 64 * 64
        weights, idx, dst = ops.moe_topk_route(logits, K, C if padded else 0)
        if padded:
            if dst is None:
                dst = moe_common.padded_rows(idx, E, C)
            out = moe_common.experts_padded(h, weights, dst, self.up_t,
                                            self.down_t, C, ops.relu2)
        else:
            out = moe_common.experts_sorted(h, weights, idx, self.up_t,
                                            self.down_t, ops.relu2)
        if self.shared_up is not None:
            out = out + F.linear(ops.relu2(F.linear(h, self.shared_up)),
                                 self.shared_down)
        return out


class FedatarLayer(nn.Module):
    def __init__(self, cfg: FedatarConfig, i: int, device, dtype):
        super().__init__()
        spec = cfg.layers[i]
        D = cfg.hidden_size
        self.eps = cfg.norm_eps
        self.dtype = dtype
        self.norm1 = LayerNormParams(D, device, f"l{i}.norm1")
        if spec.type == "mingru":
            self.mixer = MinGRUMixer(D, spec.mixer, f"l{i}.mix", device,
                                     dtype)
        else:
            self.mixer = LatentAttention(D, spec.mixer, cfg.norm_eps,
                                         f"l{i}.mix", device, dtype)
        if spec.mlp is None:
            self.norm2 = self.mlp = None
        else:
            self.norm2 = LayerNormParams(D, device, f"l{i}.norm2")
            if isinstance(spec.mlp, DenseFFSpec):
                self.mlp = XieluMLP(D, spec.mlp, f"l{i}.mlp", device, dtype)
            else:
                self.mlp = Relu2MoE(D, spec.mlp, f"l{i}.mlp", device, dtype)

    def forward(self, residual, delta, fb, cache):
        """residual: fp32 stream, updated in place with the PREVIOUS
        sub-block's output `delta` inside the fused add+norm; returns
        this layer's last un-added output."""
        h = ops.add_layernorm(residual, delta, self.norm1.weight,
                              self.norm1.bias, self.eps, self.dtype)
        delta = self.mixer(h, fb, cache)
        if self.mlp is not None:
            h = ops.add_layernorm(residual, delta, self.norm2.weight,
                                  self.norm2.bias, self.eps, self.dtype)
            delta = self.mlp(h, fb)
        return delta


class FedatarForCausalLM(nn.Module):
    needs_seq_meta = True          # ForwardBatch.seq_* / row_seq fields
    supports_decode_graph = False  # decode runs eagerly
    supported_dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, cfg: FedatarConfig, device, dtype=torch.bfloat16):
        super().__init__()
        if tp_world_size() != 1:
            raise ValueError("Fedatar runs unsharded (tensor parallel "
                             "degree 1)")
        self.cfg = cfg
        self.device = device
        self.dtype = dtype
        self.embed = _param(_rand((cfg.vocab_size, cfg.hidden_size),
                                  device, dtype, "embed", 50.0))
        self.layers = nn.ModuleList(
            FedatarLayer(cfg, i, device, dtype)
            for i in range(cfg.num_layers))
        self.final_norm = LayerNormParams(cfg.hidden_size, device,
                                          "final.norm")
        self.head = _param(_rand((cfg.vocab_size, cfg.hidden_size), device,
                                 dtype, "head",
                                 cfg.hidden_size ** -0.5 / 0.02))
        self.tap = None    # debugging hook: called with (layer, residual)

    def cache_specs(self) -> List[tuple]:
        """Per layer: ("latent", row width) paged rows in the compute
        dtype, or ("state", width) one fp32 vector per sequence slot."""
        return [(l.mixer.cache_kind, l.mixer.cache_width())
                for l in self.layers]

    def forward(self, fb: ForwardBatch, caches) -> torch.Tensor:
        residual = F.embedding(fb.token_ids, self.embed).float()
        delta = None
        for i, layer in enumerate(self.layers):
            delta = layer(residual, delta, fb, caches[i])
            if self.tap is not None:
                self.tap(i, residual + delta.float())
        return ops.add_layernorm(residual, delta, self.final_norm.weight,
                                 self.final_norm.bias, self.cfg.norm_eps,
                                 self.dtype)

    def compute_logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden_last, self.head).float()
