"""Mekevik: a parallel-block decoder with windowed sigmoid attention.

Every layer reads the fp32 residual stream through TWO RMS norms that
share one statistic; the mixer takes the first, the feed-forward the
second, and both results are added back together:

    x <- x + mixer(norm1(x)) + ff(norm2(x))

  mixer          SigmoidWindowAttention  per-key logistic weights (no
                                 softmax), a learned bias per (distance
                                 bucket, head), the heads' weights mixed
                                 by an [H, H] matrix, grouped key/value
                                 heads with a value width of their own,
                                 RMS norm over the whole query and key
                                 projections, values optionally blended
                                 with the first layer's, sigmoid output
                                 gate; keys and (blended) values paged
  feed-forwards  ClampedGLUMLP   gate clamped above, linear part clamped
                                 both sides and shifted by one
                 RoutedGLUMoE    softmax router over all experts, top-k
                                 renormalised and scaled, SwiGLU experts

The mechanisms are separate modules with their constants as arguments.
GEMMs go through F.linear/bmm (hipBLASLt / rocBLAS); everything between
them is a gfx950 kernel from ops (fp32 math for norms, scores, weights,
router; bf16 or fp32 activations).
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ... import ops
from ...parallel.comm import tp_world_size
from ..config import (ClampedGLUSpec, MekevikConfig, RoutedGLUSpec,
                      SigmoidAttentionSpec, distance_bucket)
from . import moe_common
from .batch import ForwardBatch
from .fedatar import _param, _rand


class SigmoidWindowAttention(nn.Module):
    """weight_g(i, j) = sigmoid(q_g(i) . k_c(j) * scale + rel[bucket(i-j),
    g] + pb[g]) for the keys j of the window, c = g // (H/G);
    out_h(i) = sum_j (sum_g talk[h, g] weight_g(i, j)) v_c'(j), c' = h //
    (H/G); then * sigmoid(W_g x) and the output projection.

    Queries, keys, values and the gate come from one fused GEMM.  The
    bucketed table and the per-head offset are expanded once into a
    per-distance table (`dist_bias`), so the kernel's inner loop does one
    indexed add."""

    cache_kind = "paged_k_vt"

    def __init__(self, hidden: int, spec: SigmoidAttentionSpec, eps: float,
                 name: str, device, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        H, G, dk, dv = spec.heads, spec.kv_heads, spec.dim, spec.vdim
        self.nq, self.nk, self.nv = H * dk, G * dk, G * dv
        s = hidden ** -0.5 / 0.02
        # fused projection rows: queries | keys | values | output gate
        self.qkvg = _param(_rand((self.nq + self.nk + self.nv + H * dv,
                                  hidden), device, dtype, name + ".qkvg", s))
        self.qnorm_w = _param(1.0 + _rand((self.nq,), device, torch.float32,
                                          name + ".qn", 2.0))
        self.knorm_w = _param(1.0 + _rand((self.nk,), device, torch.float32,
                                          name + ".kn", 2.0))
        self.rel = _param(_rand((spec.bias_rows, H), device, torch.float32,
                                name + ".rel", 25.0))
        self.pb = _param(_rand((H,), device, torch.float32, name + ".pb",
                               25.0) - 2.0)
        self.talk = _param(torch.eye(H, device=device) * 0.8 + _rand(
            (H, H), device, torch.float32, name + ".talk", 5.0))
        self.vmix = _param(0.5 + _rand((1,), device, torch.float32,
                                       name + ".vmix", 5.0))
        self.o = _param(_rand((hidden, H * dv), device, dtype, name + ".o",
                              (H * dv) ** -0.5 / 0.02))
        self.register_buffer("dist_bias", torch.zeros(
            (spec.bias_distances(), H), dtype=torch.float32, device=device),
            persistent=False)
        self.lam = 0.0
        self.rebuild_tables()

    def rebuild_tables(self) -> None:
        """Derived constants (after init and after a checkpoint load):
        dist_bias[n, h] = rel[bucket(n), h] + pb[h] for every distance
        that can occur or differs from its successor, and the value
        blend factor as a host number."""
        sp = self.spec
        rows = torch.tensor(
            [distance_bucket(n, sp.bias_rows, sp.bias_far)
             for n in range(self.dist_bias.shape[0])],
            dtype=torch.int64, device=self.rel.device)
        self.dist_bias.copy_(self.rel[rows] + self.pb)
        self.lam = float(self.vmix.reshape(-1)[0])

    def cache_spec(self) -> tuple:
        sp = self.spec
        return ("paged_k_vt", sp.kv_heads, sp.dim, sp.vdim)

    def forward(self, h: torch.Tensor, fb: ForwardBatch, cache,
                v_first: Optional[torch.Tensor]):
        """Returns (mixer output, this layer's own unblended values as a
        view of the projection — what later layers blend with when this
        is the first blending layer)."""
        sp = self.spec
        kcache, vcache = cache
        proj = F.linear(h, self.qkvg)
        q = ops.qk_norm_append(
            proj, fb.slot_mapping, kcache, vcache, self.qnorm_w,
            self.knorm_w, v_first, self.lam, self.eps, sp.heads,
            sp.kv_heads, sp.dim, sp.vdim)
        v0 = self.nq + self.nk
        o = ops.sigmoid_attention(
            q, kcache, vcache, fb.seq_block_table, fb.row_seq, fb.positions,
            self.dist_bias, self.talk, proj[:, v0 + self.nv:], sp.scale,
            sp.window, fb.num_chunk_rows, fb.seq_lens, fb.max_context)
        return F.linear(o, self.o), proj[:, v0:v0 + self.nv]


class ClampedGLUMLP(nn.Module):
    """W_down (g' * sigmoid(ALPHA g') * (u' + 1)), g' = min(W_gate h, L),
    u' = clamp(W_up h, -L, L); gate and up are one fused GEMM."""

    ALPHA = 1.702

    def __init__(self, hidden: int, spec: ClampedGLUSpec, name: str, device,
                 dtype):
        super().__init__()
        self.limit = spec.limit
        self.gate_up = _param(_rand((2 * spec.ff, hidden), device, dtype,
                                    name + ".gate_up",
                                    hidden ** -0.5 / 0.02))
        self.down = _param(_rand((hidden, spec.ff), device, dtype,
                                 name + ".down", spec.ff ** -0.5 / 0.02))

    def forward(self, h: torch.Tensor, fb: ForwardBatch) -> torch.Tensor:
        a = ops.gated_act(F.linear(h, self.gate_up), ops.GATED_ACT_CLAMPED,
                          self.limit, self.ALPHA)
        return F.linear(a, self.down)


class RoutedGLUMoE(nn.Module):
    """Router scores = softmax over ALL experts (fp32); the top-k scores,
    divided by their sum and multiplied by `scale`, weigh the chosen
    SwiGLU experts W_down (silu(W_gate h) * W_up h).  Renormalising the
    top-k of a softmax equals the softmax over the chosen logits, which
    is what the routing kernel evaluates.  Expert weights are stored
    K-major ([E, in, out]) for the batched GEMMs, gate and up stacked."""

    PADDED_MAX_ROWS = 256

    def __init__(self, hidden: int, spec: RoutedGLUSpec, name: str, device,
                 dtype):
        super().__init__()
        self.spec = spec
        E, f = spec.experts, spec.expert_ff
        self.router_w = _param(_rand((E, hidden), device, torch.float32,
                                     name + ".router",
                                     hidden ** -0.5 / 0.02))
        self.up_t = _param(_rand((E, hidden, 2 * f), device, dtype,
                                 name + ".up", hidden ** -0.5 / 0.02))
        self.down_t = _param(_rand((E, f, hidden), device, dtype,
                                   name + ".down", f ** -0.5 / 0.02))

    @staticmethod
    def _act(z: torch.Tensor) -> torch.Tensor:
        return ops.gated_act(z, ops.GATED_ACT_SILU)

    def forward(self, h: torch.Tensor, fb: ForwardBatch) -> torch.Tensor:
        T = h.shape[0]
        E, K = self.spec.experts, self.spec.top
        logits = F.linear(h.float(), self.router_w)
        padded = T <= self.PADDED_MAX_ROWS
        C = (T + 63) // 64 * 64
        weights, idx, dst = ops.moe_topk_route(
            logits, K, C if padded else 0, self.spec.scale)
        if padded:
            if dst is None:
                dst = moe_common.padded_rows(idx, E, C)
            return moe_common.experts_padded(h, weights, dst, self.up_t,
                                             self.down_t, C, self._act)
        return moe_common.experts_sorted(h, weights, idx, self.up_t,
                                         self.down_t, self._act)


class ParallelLayer(nn.Module):
    """x <- x + mixer(norm1(x)) + ff(norm2(x)).  The add of the PREVIOUS
    layer's two results is fused into this layer's norm kernel, which
    evaluates the RMS statistic once for both norms."""

    def __init__(self, cfg: MekevikConfig, i: int, device, dtype):
        super().__init__()
        spec = cfg.layers[i]
        D = cfg.hidden_size
        self.eps = cfg.norm_eps
        self.dtype = dtype
        self.v_mix = spec.mixer.v_mix
        self.norm1_w = _param(1.0 + _rand((D,), device, torch.float32,
                                          f"l{i}.norm1", 2.0))
        self.mixer = SigmoidWindowAttention(D, spec.mixer, cfg.norm_eps,
                                            f"l{i}.mix", device, dtype)
        if spec.mlp is None:
            self.norm2_w = self.mlp = None
        else:
            self.norm2_w = _param(1.0 + _rand((D,), device, torch.float32,
                                              f"l{i}.norm2", 2.0))
            if isinstance(spec.mlp, ClampedGLUSpec):
                self.mlp = ClampedGLUMLP(D, spec.mlp, f"l{i}.mlp", device,
                                         dtype)
            else:
                self.mlp = RoutedGLUMoE(D, spec.mlp, f"l{i}.mlp", device,
                                        dtype)

    def forward(self, residual, delta_a, delta_b, fb, cache, v_first):
        h1, h2 = ops.add_rmsnorm_pair(residual, delta_a, delta_b,
                                      self.norm1_w, self.norm2_w, self.eps,
                                      self.dtype)
        a, v_own = self.mixer(h1, fb, cache, v_first)
        b = self.mlp(h2, fb) if self.mlp is not None else None
        return a, b, v_own


class MekevikForCausalLM(nn.Module):
    needs_seq_meta = True          # ForwardBatch.seq_* / row_seq fields
    supports_decode_graph = False  # decode runs eagerly
    supported_dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, cfg: MekevikConfig, device, dtype=torch.bfloat16):
        super().__init__()
        if tp_world_size() != 1:
            raise ValueError("Mekevik runs unsharded (tensor parallel "
                             "degree 1)")
        self.cfg = cfg
        self.device = device
        self.dtype = dtype
        self.embed = _param(_rand((cfg.vocab_size, cfg.hidden_size),
                                  device, dtype, "embed", 50.0))
        self.layers = nn.ModuleList(
            ParallelLayer(cfg, i, device, dtype)
            for i in range(cfg.num_layers))
        self.final_norm_w = _param(1.0 + _rand(
            (cfg.hidden_size,), device, torch.float32, "final.norm", 2.0))
        self.head = _param(_rand((cfg.vocab_size, cfg.hidden_size), device,
                                 dtype, "head",
                                 cfg.hidden_size ** -0.5 / 0.02))
        self.tap = None    # debugging hook: called with (layer, residual)

    def cache_specs(self) -> List[tuple]:
        return [l.mixer.cache_spec() for l in self.layers]

    def rebuild_tables(self) -> None:
        for l in self.layers:
            l.mixer.rebuild_tables()

    def forward(self, fb: ForwardBatch, caches) -> torch.Tensor:
        residual = F.embedding(fb.token_ids, self.embed).float()
        if self.cfg.embed_scale != 1.0:
            residual.mul_(self.cfg.embed_scale)
        a = b = v_first = None
        for i, layer in enumerate(self.layers):
            blend = v_first if layer.v_mix else None
            a, b, v_own = layer(residual, a, b, fb, caches[i], blend)
            if layer.v_mix and v_first is None:
                v_first = v_own
            if self.tap is not None:
                self.tap(i, residual + a.float()
                         + (b.float() if b is not None else 0.0))
        h, _ = ops.add_rmsnorm_pair(residual, a, b, self.final_norm_w, None,
                                    self.cfg.norm_eps, self.dtype)
        return h

    def compute_logits(self, hidden_last: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden_last, self.head).float()
        if self.cfg.logit_scale != 1.0:
            logits.mul_(self.cfg.logit_scale)
        return logits
