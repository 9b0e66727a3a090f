"""Ops of the hybrid sequence-mixer stack (``csrc/hybrid`` -> ``jax_llama_amd._C_hybrid``).

Same dispatch rule as the rest of ``ops``: GPU tensors run the hand-written gfx950 kernels (a missing extension
raises), CPU tensors run the PyTorch implementation below (the test / oracle path of the framework).

Conventions: activations between ops are fp32 in both number formats. A weight (or cache) tensor's dtype selects the
arithmetic: bf16 weights -> operands rounded to bf16, fp32 accumulation; fp32 weights -> exact fp32 products.

Mechanisms (each with its constants as arguments, usable by any model of the registry):
  * ``linear`` / ``moe_table``: row-major weights of any shape; a token-id -> experts table routes a mixture of SwiGLU
    experts without a router (expert-grouped GEMM over a counting-sorted batch, or per-row GEMVs for decode);
  * ``norm_residual_``: RMS norm on a sublayer's OUTPUT (scalar or vector gain) fused with the residual add;
  * ``attn_prep`` / ``attn_bias``: per-head RMS-normed q / k / v, position-dependent query temperature, soft-capped
    scores, learned per-distance bias (any bucketing: the table is expanded by distance on the host), causal softmax;
  * ``delta_prep`` / ``delta_scan`` / ``gated_rmsnorm``: the gated delta rule with short causal convolutions.
"""
from __future__ import annotations

import importlib
import math
import os
from typing import Optional, Tuple

import torch

BF16 = torch.bfloat16
F32 = torch.float32

_EXT = None
_ERR: Optional[BaseException] = None
# bf16 prefill attention on the MFMA flash kernel where its shapes apply (JLA_HY_MMA_PREFILL=0: the plain kernel, A/B)
MMA_PREFILL = os.environ.get("JLA_HY_MMA_PREFILL", "1") != "0"


def ext():
    """The native module, or a loud error saying how to build it."""
    global _EXT, _ERR
    if _EXT is None and _ERR is None:
        try:
            _EXT = importlib.import_module("jax_llama_amd._C_hybrid")
        except BaseException as e:  # ImportError, OSError (undefined symbol), ...
            _ERR = e
    if _EXT is None:
        raise RuntimeError("jax_llama_amd hybrid HIP extension is not available "
                           f"({type(_ERR).__name__}: {_ERR}). Build it with `python build.py --only hybrid` "
                           "(requires hipcc, targets gfx950). GPU tensors are never run on a fallback path.")
    return _EXT


def ext_available() -> bool:
    try:
        ext()
        return True
    except RuntimeError:
        return False


def so_path() -> Optional[str]:
    return getattr(ext(), "__file__", None) if ext_available() else None


def _gpu(t: torch.Tensor) -> bool:
    return t.device.type == "cuda"


def _slot_tensor(slot, device) -> torch.Tensor:
    if torch.is_tensor(slot):
        return slot
    return torch.tensor([int(slot)], dtype=torch.int32, device=device)


def _slot_int(slot) -> int:
    return int(slot.reshape(-1)[0].item()) if torch.is_tensor(slot) else int(slot)


def _round_like(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """The operand rounding of a product with weight ``w`` (CPU path)."""
    return x.to(BF16).float() if w.dtype == BF16 else x.float()


# ------------------------------------------------------------------------------------------------ rows
def embed_rows(ids: torch.Tensor, table: torch.Tensor, col0: int = 0, ncols: Optional[int] = None) -> torch.Tensor:
    """fp32 ``[M, ncols]`` = ``table[ids, col0 : col0 + ncols]``."""
    ncols = table.shape[1] - col0 if ncols is None else ncols
    ids = ids.reshape(-1)
    if not _gpu(table):
        return table[ids.long(), col0:col0 + ncols].float()
    out = torch.empty(ids.numel(), ncols, dtype=F32, device=table.device)
    ext().embed_rows(ids.to(torch.int32).contiguous(), table, int(col0), out)
    return out


# Dense bf16 linears of a prompt-sized batch run on the framework's tuned MFMA GEMM (ops.linear over the fragment-
# packed weight layout, csrc/kernels/gemm.hip) when the main extension is built and the shape fits its layout
# (N % 16 == 0, K % 32 == 0); the row-major kernel here serves every other case. JLA_HY_PACKED_GEMM=0: never.
PACKED_GEMM = os.environ.get("JLA_HY_PACKED_GEMM", "1") != "0"
PACKED_GEMM_MIN_M = 256
GROUPED_GEMV_MAX_R = 64  # rows up to which an expert-sorted batch runs the expert-grouped GEMV (csrc: HY_GROUPED_GEMV_MAX_R)
_PACKED = {}


def _packed_weight(w: torch.Tensor):
    """The fragment-packed copy of a dense ``[N, K]`` bf16 weight (made once, kept beside the row-major one)."""
    key = (w.data_ptr(), tuple(w.shape))
    pw = _PACKED.get(key)
    if pw is None or pw[0] is not w:
        from ..models.weights import PackedLinear
        pw = _PACKED[key] = (w, PackedLinear.from_dense(w, w.device))
    return pw[1]


def _use_packed_gemm(x: torch.Tensor, w: torch.Tensor) -> bool:
    if not PACKED_GEMM or w.dtype != BF16 or w.dim() != 2 or x.shape[0] < PACKED_GEMM_MIN_M:
        return False
    if w.shape[0] % 16 or w.shape[1] % 32 or not x.is_contiguous():
        return False
    from . import ext_available as core_available
    return core_available()


def linear(x: torch.Tensor, w: torch.Tensor, swiglu: bool = False) -> torch.Tensor:
    """``x [M, K] (fp32) @ w [N, K]^T`` -> fp32 ``[M, N]``; ``swiglu``: ``w`` is ``[2N, K]`` (gate rows, then up rows)
    and the result is ``silu(x Wg^T) * (x Wu^T)``. ``x`` may be a column-contiguous view with strided rows."""
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    if not _gpu(x):
        y = _round_like(x, w) @ w.float().t()
        return torch.nn.functional.silu(y[:, :n]) * y[:, n:] if swiglu else y
    if not swiglu and _use_packed_gemm(x, w):
        from . import linear as packed_linear
        xb = torch.empty(x.shape, dtype=BF16, device=x.device)
        ext().cast_bf16(x, xb)
        return packed_linear(xb, _packed_weight(w), out_dtype=F32)
    out = torch.empty(x.shape[0], n, dtype=F32, device=x.device)
    ext().linear_rows(x, None, w, out, None, None, None, x.shape[0], bool(swiglu))
    return out


def moe_table(x: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, w_gu: torch.Tensor,
              w_down: torch.Tensor) -> torch.Tensor:
    """Mixture of SwiGLU experts chosen by a ``[vocab, top]`` int32 table of the token id (no router).

    ``w_gu [E, 2F, K]`` (gate rows then up rows), ``w_down [E, D, F]``. Returns the chosen experts' outputs, fp32
    ``[M * top, D]`` in (token, choice) order; the caller averages them (``norm_residual_(nsum=top, ysc=1/top)``)."""
    m, top, e_n = x.shape[0], table.shape[1], w_gu.shape[0]
    r = m * top
    ids = ids.reshape(-1)
    if not _gpu(x):
        ex = table[ids.long()].reshape(-1).long()  # [R]
        xr = _round_like(x, w_gu).repeat_interleave(top, 0)
        y = torch.empty(r, w_down.shape[1], dtype=F32)
        f = w_gu.shape[1] // 2
        for e in ex.unique().tolist():
            sel = (ex == e).nonzero().squeeze(1)
            gu = xr[sel] @ w_gu[e].float().t()
            h = torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]
            y[sel] = _round_like(h, w_down) @ w_down[e].float().t()
        return y
    dev = x.device
    e = ext()
    idx = torch.empty(4 * r + e_n + 1, dtype=torch.int32, device=dev)
    row_expert, row_tok, sort_tok, sort_dst, offs = idx[:r], idx[r:2 * r], idx[2 * r:3 * r], idx[3 * r:4 * r], idx[4 * r:]
    e.route_table(ids.to(torch.int32).contiguous(), table, e_n, row_expert, row_tok, sort_tok, sort_dst, offs)
    y = torch.empty(r, w_down.shape[1], dtype=F32, device=dev)
    bf16_pair = w_gu.dtype == BF16 and r > GROUPED_GEMV_MAX_R and x.is_contiguous() and x.shape[1] % 8 == 0
    h = None if bf16_pair else torch.empty(r, w_gu.shape[1] // 2, dtype=F32, device=dev)
    if r <= e.GEMV_MAX_R:  # decode: one GEMV per (token, choice) row, expert read on the device
        e.linear_rows(x, row_tok, w_gu, h, None, None, row_expert, r, True)
        e.linear_rows(h, None, w_down, y, None, None, row_expert, r, False)
    elif bf16_pair:
        # prompt-sized, bf16: the tiles read a bf16 copy of x and keep the hidden activation bf16 (the operands they
        # would round to anyway), which halves the activation traffic of both products
        xb = torch.empty(x.shape, dtype=BF16, device=dev)
        e.cast_bf16(x, xb)
        hb = torch.empty(r, w_gu.shape[1] // 2, dtype=BF16, device=dev)
        e.linear_rows(xb, sort_tok, w_gu, hb, None, offs, None, r, True)
        e.linear_rows(hb, None, w_down, y, sort_dst, offs, None, r, False)
    else:  # expert-grouped tiles over the sorted rows; the down projection scatters back to (token, choice) order
        e.linear_rows(x, sort_tok, w_gu, h, None, offs, None, r, True)
        e.linear_rows(h, None, w_down, y, sort_dst, offs, None, r, False)
    return y


def norm_residual_(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float, nsum: int = 1,
                   ysc: float = 1.0) -> torch.Tensor:
    """``x += rms_norm(ysc * sum of each token's nsum rows of y) * w`` in place; ``w`` one number or ``[D]``."""
    if not _gpu(x):
        v = y.float().reshape(x.shape[0], nsum, -1).sum(1) * ysc
        x.add_(v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float().reshape(-1))
        return x
    ext().norm_residual(y, int(nsum), float(ysc), w.reshape(-1), float(eps), x, None)
    return x


def rms_rows(y: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``y / sqrt(mean(y^2) + eps) * w`` (fp32), ``w`` one number or ``[D]``."""
    if not _gpu(y):
        v = y.float()
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float().reshape(-1)
    out = torch.empty_like(y)
    ext().norm_residual(y, 1, 1.0, w.reshape(-1), float(eps), None, out)
    return out


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def gelu_gate_rows(gp: torch.Tensor, ids: torch.Tensor, table: torch.Tensor, col0: int) -> torch.Tensor:
    """``gelu_tanh(gp) * table[ids, col0 : col0 + D]``."""
    ids = ids.reshape(-1)
    if not _gpu(gp):
        return gelu_tanh(gp.float()) * table[ids.long(), col0:col0 + gp.shape[1]].float()
    g = torch.empty_like(gp)
    ext().gelu_gate_rows(gp, ids.to(torch.int32).contiguous(), table, int(col0), g)
    return g


# ------------------------------------------------------------------------------------------------ attention
def distance_bias_table(rel: torch.Tensor, bias_max: int) -> torch.Tensor:
    """Expand a bucketed ``[buckets, H]`` bias into a per-distance table ``[bias_max + 1, H]`` (fp32; distances past
    the end use the last row). Buckets: the first half one per distance, the second half log-spaced up to
    ``bias_max``: ``bucket(n) = n`` for ``n < B/2``, else ``min(B - 1, B/2 + floor(ln(n / (B/2)) / ln(D / (B/2)) * (B - B/2)))``."""
    nb = rel.shape[0]
    half = nb // 2
    rows = []
    for n in range(int(bias_max) + 1):
        if n < half:
            rows.append(n)
        elif half == 0 or bias_max <= half:
            rows.append(nb - 1)
        else:
            rows.append(min(nb - 1, half + int(math.floor(math.log(n / half) / math.log(bias_max / half) * (nb - half)))))
    idx = torch.tensor(rows, dtype=torch.long, device=rel.device)
    return rel.float()[idx].contiguous()


def attn_prep(proj: torch.Tensor, positions: torch.Tensor, slot, b: int, s: int, heads: int, kv_heads: int, dim: int,
              vdim: int, kc: Optional[torch.Tensor], vc: Optional[torch.Tensor], eps: float, temp_coef: float = 0.0,
              temp_every: int = 1) -> torch.Tensor:
    """From the fused projection ``proj [B*S, H*dim (+ G*dim + G*vdim)]``: q / k divided by their per-head RMS over
    ``dim`` (v over ``vdim``), q scaled by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)``, k / v written into
    the caches ``[B, G, T, .]`` at ``slot + s``. ``kc is None``: the layer reads another layer's cache (q only).
    Returns q ``[B, S, H, dim]`` fp32."""
    m = b * s
    if not _gpu(proj):
        s0 = _slot_int(slot)
        q = proj[:, :heads * dim].float().reshape(m, heads, dim)
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
        if temp_coef:
            p = positions.reshape(-1).to(torch.int64)
            q = q * (1.0 + temp_coef * torch.log(torch.div(p + 1, temp_every, rounding_mode="floor").float() + 1.0)
                     )[:, None, None]
        if kc is not None:
            k = proj[:, heads * dim:(heads + kv_heads) * dim].float().reshape(b, s, kv_heads, dim)
            v = proj[:, (heads + kv_heads) * dim:(heads + kv_heads) * dim + kv_heads * vdim].float().reshape(
                b, s, kv_heads, vdim)
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
            kc[:, :, s0:s0 + s] = k.permute(0, 2, 1, 3).to(kc.dtype)
            vc[:, :, s0:s0 + s] = v.permute(0, 2, 1, 3).to(vc.dtype)
        return q.reshape(b, s, heads, dim)
    q = torch.empty(b, s, heads, dim, dtype=F32, device=proj.device)
    ext().attn_prep(proj, positions.reshape(-1).to(torch.int32).contiguous(), _slot_tensor(slot, proj.device), b, s,
                    heads, kv_heads, dim, vdim, kc, vc, q, float(eps), float(temp_coef), int(temp_every))
    return q


def attn_bias(q: torch.Tensor, kc: torch.Tensor, vc: torch.Tensor, slot, scale: float, softcap: float = 0.0,
              bias: Optional[torch.Tensor] = None, max_kv: Optional[int] = None) -> torch.Tensor:
    """Causal attention of ``q [B, S, H, dim]`` (queries at cache slots ``slot + s``) over ``[B, G, T, .]`` caches:
    ``score = q.k * scale``; ``softcap * tanh(score / softcap)`` if ``softcap > 0``; ``+ bias[min(i - j, last), h]``;
    softmax over ``j <= i``. Returns fp32 ``[B*S, H*vdim]``."""
    b, s, h, dim = q.shape
    g, vdim = kc.shape[1], vc.shape[3]
    if not _gpu(q):
        s0 = _slot_int(slot)
        t = s0 + s
        k = kc[:, :, :t].float().repeat_interleave(h // g, 1)  # [B, H, t, dim]
        v = vc[:, :, :t].float().repeat_interleave(h // g, 1)
        sc = torch.einsum("bshd,bhtd->bhst", q.float(), k) * scale
        if softcap and softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        qi = torch.arange(s0, t)[:, None]
        kj = torch.arange(t)[None, :]
        dist = qi - kj
        if bias is not None:
            bt = bias.float()[dist.clamp(0, bias.shape[0] - 1)]  # [s, t, H]
            sc = sc + bt.permute(2, 0, 1)[None]
        sc = sc.masked_fill((dist < 0)[None, None], float("-inf"))
        o = torch.einsum("bhst,bhtv->bshv", torch.softmax(sc, -1), v)
        return o.reshape(b * s, h * vdim)
    out = torch.empty(b * s, h * vdim, dtype=F32, device=q.device)
    e = ext()
    t_cap = int(max_kv) if max_kv is not None else kc.shape[2]
    ws, splits, vt = None, 1, None
    if s == 1:
        splits = int(e.attn_decode_splits(b, h, t_cap))
        ws = torch.empty(b * h * splits * (vdim + 2), dtype=F32, device=q.device)
    elif MMA_PREFILL:
        nb = int(e.attn_prefill_ws_bytes(b, s, g, dim, vdim, kc.shape[2], kc.dtype == BF16))
        if nb:  # bf16 caches at the MFMA shapes: the flash kernel over a transposed copy of the values
            vt = torch.empty(nb // 2, dtype=BF16, device=q.device)
    e.attn_bias(q.contiguous(), kc, vc, _slot_tensor(slot, q.device), float(scale), float(softcap or 0.0), bias, out,
                t_cap, ws, splits, vt)
    return out


# ------------------------------------------------------------------------------------------------ gated delta rule
def delta_prep(proj: torch.Tensor, b: int, s: int, heads: int, kv_heads: int, dim: int, vdim: int,
               conv_w: torch.Tensor, conv_state: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor
               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """From ``proj [B*S, q (G*dim) | k (G*dim) | v (H*vdim) | gate (H*vdim) | b (H) | a (H)]``: the short causal
    convolution (``conv_w [channels, taps]``, last tap = current token; earlier inputs from ``conv_state
    [B, channels, taps-1]``, which is advanced) + SiLU on q, k, v; q, k to unit length per head (``1e-6`` inside the
    root; q also times ``dim^-1/2``); ``beta = sigmoid(b)``; ``decay = exp(-exp(a_log) * softplus(a + dt_bias))``.
    Returns ``(q [M,G,dim], k [M,G,dim], v [M,H,vdim], beta [M,H], decay [M,H])`` fp32."""
    m = b * s
    qk, vv = kv_heads * dim, heads * vdim
    c = 2 * qk + vv
    if not _gpu(proj):
        taps = conv_w.shape[1]
        x = proj[:, :c].float().reshape(b, s, c)
        full = torch.cat([conv_state.float().permute(0, 2, 1), x], 1)  # [B, taps-1+S, C]
        y = torch.zeros(b, s, c)
        for tap in range(taps):
            y = y + full[:, tap:tap + s] * conv_w.float()[:, tap]
        if taps > 1:
            conv_state.copy_(full[:, -(taps - 1):].permute(0, 2, 1))
        y = torch.nn.functional.silu(y).reshape(m, c)
        q = y[:, :qk].reshape(m, kv_heads, dim)
        k = y[:, qk:2 * qk].reshape(m, kv_heads, dim)
        v = y[:, 2 * qk:].reshape(m, heads, vdim)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        gates = proj[:, c + vv:c + vv + 2 * heads].float()
        beta = torch.sigmoid(gates[:, :heads])
        decay = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(gates[:, heads:] + dt_bias.float()))
        return q.contiguous(), k.contiguous(), v.contiguous(), beta.contiguous(), decay.contiguous()
    dev = proj.device
    q = torch.empty(m, kv_heads, dim, dtype=F32, device=dev)
    k = torch.empty(m, kv_heads, dim, dtype=F32, device=dev)
    v = torch.empty(m, heads, vdim, dtype=F32, device=dev)
    beta = torch.empty(m, heads, dtype=F32, device=dev)
    decay = torch.empty(m, heads, dtype=F32, device=dev)
    e = ext()
    e.delta_prep(proj, b, s, heads, kv_heads, dim, vdim, conv_w, conv_state, a_log, dt_bias, q, k, v, beta, decay)
    e.conv_state_update(proj, b, s, heads, kv_heads, dim, vdim, conv_w, conv_state)
    return q, k, v, beta, decay


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor,
               state: torch.Tensor, b: int, s: int) -> torch.Tensor:
    """The recurrence per head over ``s`` tokens, ``state [B, H, dim, vdim]`` (fp32) read and advanced in place:
    ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``. Returns ``o [M, H, vdim]``."""
    m, g, dim = q.shape
    h, vdim = v.shape[1], v.shape[2]
    if not _gpu(q):
        rep = h // g
        qq = q.reshape(b, s, g, dim).repeat_interleave(rep, 2)
        kk = k.reshape(b, s, g, dim).repeat_interleave(rep, 2)
        vv = v.reshape(b, s, h, vdim)
        be, de = beta.reshape(b, s, h), decay.reshape(b, s, h)
        o = torch.empty(b, s, h, vdim)
        st = state
        for t in range(s):
            st.mul_(de[:, t, :, None, None])
            u = be[:, t, :, None] * (vv[:, t] - torch.einsum("bhdv,bhd->bhv", st, kk[:, t]))
            st.add_(kk[:, t, :, :, None] * u[:, :, None, :])
            o[:, t] = torch.einsum("bhdv,bhd->bhv", st, qq[:, t])
        return o.reshape(m, h, vdim)
    o = torch.empty(m, h, vdim, dtype=F32, device=q.device)
    ext().delta_scan(q, k, v, beta, decay, state, o, b, s, h, g, dim, vdim)
    return o


def gated_rmsnorm(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``o [M, H, vdim] / rms(o) * w [vdim] * silu(gate [M, H*vdim])`` -> fp32 ``[M, H*vdim]``."""
    m, h, vdim = o.shape
    if not _gpu(o):
        x = o.float()
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        return x.reshape(m, h * vdim) * torch.nn.functional.silu(gate.float())
    out = torch.empty(m, h * vdim, dtype=F32, device=o.device)
    ext().gated_rmsnorm(o, gate, w, float(eps), out, h, vdim)
    return out
