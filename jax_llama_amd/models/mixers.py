"""Building blocks of layer-list decoders (``models/zavevik.py``): each block is a thin view over one layer's weights
that issues the ``ops.hybrid`` kernels, like ``models/modules.py`` does for LLaMA. Every constant is a constructor
argument (taken from the layer's ``MixerSpec`` / ``MoESpec``), so another architecture of the registry can assemble
the same mechanisms with other values.

  BiasedAttention : fused q|k|v projection, per-head RMS-normed q / k / v, query temperature, cache write; soft-capped
                    scores + learned distance bias + causal softmax; o projection. May read another layer's keys and
                    values (``kv_from``) -- then it projects queries only.
  GatedDeltaMixer : fused q|k|v|gate|b|a projection, short causal convolutions + SiLU, unit-length q / k, the gated
                    delta-rule recurrence over a carried fp32 state, gated RMS norm, o projection.
  TableMoE        : mixture of SwiGLU experts chosen by a token-id table (no router), averaged.
  TokenSide       : per-layer token-side input: gelu_tanh(gate x) * (slice of a second embedding), projected back,
                    RMS-normed with a vector gain, added to the residual.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..ops import hybrid as hy


@dataclass
class StepContext:
    """What one forward step hands to every block: the tokens, where they sit, and the cache."""

    ids: torch.Tensor        # int32 [B * S]
    positions: torch.Tensor  # int32 [B * S]
    b: int
    s: int
    cache: object            # HybridCache (or a row view)
    slot0: object            # int, or device int32[1] (graph-capturable)


class BiasedAttention:
    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, w_o: torch.Tensor,
                 bias_by_distance: Optional[torch.Tensor]):
        self.i = layer_idx
        self.spec = spec
        self.eps = eps
        self.w_in = w_in            # [H dim (+ G dim + G vdim), D]
        self.w_o = w_o              # [D, H vdim]
        self.bias = bias_by_distance  # fp32 [bias_max + 1, H] or None

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        proj = hy.linear(x, self.w_in)
        kc, vc = ctx.cache.layer(self.i)
        own = sp.kv_from is None
        q = hy.attn_prep(proj, ctx.positions, ctx.slot0, ctx.b, ctx.s, sp.heads, sp.kv_heads, sp.dim, sp.vdim,
                         kc if own else None, vc if own else None, self.eps, sp.q_temp_coef, sp.q_temp_every)
        a = hy.attn_bias(q, kc, vc, ctx.slot0, sp.scale, sp.softcap, self.bias)
        return hy.linear(a, self.w_o)


class GatedDeltaMixer:
    def __init__(self, layer_idx: int, spec, eps: float, w_in: torch.Tensor, conv_w: torch.Tensor,
                 a_log: torch.Tensor, dt_bias: torch.Tensor, norm_w: torch.Tensor, w_o: torch.Tensor):
        self.i = layer_idx
        self.spec = spec
        self.eps = eps
        self.w_in = w_in      # [2 G dim + 2 H vdim + 2 H, D]: q | k | v | gate | b | a
        self.conv_w = conv_w  # fp32 [2 G dim + H vdim, taps]
        self.a_log, self.dt_bias, self.norm_w = a_log, dt_bias, norm_w
        self.w_o = w_o

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        sp = self.spec
        proj = hy.linear(x, self.w_in)
        state, tail = ctx.cache.recurrent(self.i)
        q, k, v, beta, decay = hy.delta_prep(proj, ctx.b, ctx.s, sp.heads, sp.kv_heads, sp.dim, sp.vdim, self.conv_w,
                                             tail, self.a_log, self.dt_bias)
        o = hy.delta_scan(q, k, v, beta, decay, state, ctx.b, ctx.s)
        c = 2 * sp.kv_heads * sp.dim + sp.heads * sp.vdim
        gate = proj[:, c:c + sp.heads * sp.vdim]
        return hy.linear(hy.gated_rmsnorm(o, gate, self.norm_w, self.eps), self.w_o)


class TableMoE:
    def __init__(self, spec, table: torch.Tensor, w_gu: torch.Tensor, w_down: torch.Tensor):
        self.spec = spec
        self.table = table    # int32 [vocab, top]
        self.w_gu = w_gu      # [E, 2 ff, D] gate rows then up rows
        self.w_down = w_down  # [E, D, ff]

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        """The chosen experts' outputs ``[M * top, D]``; the caller's output norm averages them."""
        return hy.moe_table(x, ctx.ids, self.table, self.w_gu, self.w_down)


class TokenSide:
    def __init__(self, table: torch.Tensor, col0: int, w_gate: torch.Tensor, w_proj: torch.Tensor, norm_w: torch.Tensor,
                 eps: float):
        self.table, self.col0 = table, col0
        self.w_gate, self.w_proj, self.norm_w, self.eps = w_gate, w_proj, norm_w, eps

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> None:
        g = hy.gelu_gate_rows(hy.linear(x, self.w_gate), ctx.ids, self.table, self.col0)
        hy.norm_residual_(x, hy.linear(g, self.w_proj), self.norm_w, self.eps)


class OutputNormBlock:
    """``x += norm1(mixer(x)); x += norm2(ff(x)); x += side(x)``: the norm sits on each sublayer's OUTPUT (a scalar
    gain), the sublayers read the residual itself."""

    def __init__(self, mixer, norm1: torch.Tensor, mlp: Optional[TableMoE], norm2: Optional[torch.Tensor],
                 side: Optional[TokenSide], eps: float):
        self.mixer, self.norm1, self.mlp, self.norm2, self.side, self.eps = mixer, norm1, mlp, norm2, side, eps

    def __call__(self, x: torch.Tensor, ctx: StepContext) -> None:
        hy.norm_residual_(x, self.mixer(x, ctx), self.norm1, self.eps)
        if self.mlp is not None:
            top = self.mlp.spec.top
            hy.norm_residual_(x, self.mlp(x, ctx), self.norm2, self.eps, nsum=top, ysc=1.0 / top)
        if self.side is not None:
            self.side(x, ctx)
