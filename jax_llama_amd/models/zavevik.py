"""Zavevik: a layer-list decoder that interleaves gated-delta-rule layers with biased softmax attention.

Per layer (``models/mixers.OutputNormBlock``): ``x += g1 * rms_norm(mixer(x))``, ``x += g2 * rms_norm(moe(x))`` with
scalar gains on the sublayer OUTPUTS, then a token-side input. Mixers: ``attention`` (RMS-normed q / k / v, query
temperature, soft-capped scores, bucketed distance bias, optional cross-layer key / value sharing) and ``delta`` (gated
delta rule with short convolutions). Feed-forward: a table-routed mixture of SwiGLU experts. Logits: scalar-gain RMS
norm, then the head.

Checkpoint: ``config.json`` + ``model.safetensors`` with tensors ``embed``, ``side.embed``, ``l<i>.norm1|norm2``,
``l<i>.mix.*``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.table``, ``l<i>.side.gate|proj|norm``, ``final.norm``,
``head`` (linear weights ``[out, in]``). Loading fuses each mixer's input projections into one matrix, stacks the
experts, expands the distance-bias buckets by distance and keeps the small recurrence constants in fp32.

Number formats: ``dtype=bfloat16`` (serving: bf16 matrix operands and caches, fp32 accumulation, and fp32 residual,
norms, scores, recurrent state) or ``dtype=float32`` (everything exact fp32). The model runs on the framework's step
interface -- ``forward_tokens(ids, positions, cache, slot0, ...)`` over an ``init_cache`` object -- so the generation
engine (``runtime/engine.py``) and the request stepper (``runtime/stepper.py``) drive it like LLaMA.
"""
from __future__ import annotations

import os
from typing import Dict, List, Optional

import torch

from ..config import MixerSpec, ZavevikConfig
from ..ops import hybrid as hy
from ..parallel.comm import NO_COMM
from .kv_cache import HybridCache
from .mixers import BiasedAttention, GatedDeltaMixer, OutputNormBlock, StepContext, TableMoE, TokenSide

BF16 = torch.bfloat16
F32 = torch.float32


def cache_specs(config: ZavevikConfig) -> list:
    out = []
    for ls in config.layers:
        m = ls.mixer
        if m.type == "delta":
            out.append(("delta", m.heads, m.kv_heads, m.dim, m.vdim, m.conv))
        elif m.kv_from is not None:
            out.append(("kv_from", m.kv_from))
        else:
            out.append(("kv", m.kv_heads, m.dim, m.vdim))
    return out


def bias_buckets(spec: MixerSpec) -> int:
    """Rows of a random-init distance-bias table for ``spec`` (a checkpoint's own table decides when loading)."""
    return 32 if spec.bias_max else 0


def random_state_dict(config: ZavevikConfig, seed: int = 0, buckets: Optional[int] = None) -> Dict[str, torch.Tensor]:
    """A random checkpoint of ``config`` with the checkpoint's tensor names (bf16 matrices, int32 tables): synthetic
    benchmarks and tests. Scales keep every sublayer's output O(1)."""
    g = torch.Generator().manual_seed(seed)
    d, v = config.hidden_size, config.vocab_size

    def mat(n, k, std=None):
        return (torch.randn(n, k, generator=g) * (std if std is not None else k ** -0.5)).to(BF16)

    def vec(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).to(BF16)

    sd: Dict[str, torch.Tensor] = {"embed": mat(v, d, 1.0), "head": mat(v, d), "final.norm": vec(1, 0.8, 1.2).reshape(())}
    if config.side_dim:
        sd["side.embed"] = mat(v, config.side_dim * len(config.layers), 1.0)
    for i, ls in enumerate(config.layers):
        p, m = f"l{i}.", ls.mixer
        sd[p + "norm1"] = vec(1, 0.5, 1.0).reshape(())
        if m.type == "attention":
            sd[p + "mix.q"] = mat(m.heads * m.dim, d)
            if m.kv_from is None:
                sd[p + "mix.k"] = mat(m.kv_heads * m.dim, d)
                sd[p + "mix.v"] = mat(m.kv_heads * m.vdim, d)
            nb = buckets if buckets is not None else bias_buckets(m)
            if m.bias_max and nb:
                sd[p + "mix.rel"] = mat(nb, m.heads, 1.0)
            sd[p + "mix.o"] = mat(d, m.heads * m.vdim)
        else:
            for n, rows in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
                sd[p + f"mix.{n}"] = mat(rows, d)
                sd[p + f"mix.{n}.conv"] = mat(rows, m.conv, 0.7)
            sd[p + "mix.b"] = mat(m.heads, d)
            sd[p + "mix.a"] = mat(m.heads, d)
            sd[p + "mix.g"] = mat(m.heads * m.vdim, d)
            sd[p + "mix.A_log"] = vec(m.heads, -2.0, 0.5)
            sd[p + "mix.dt_bias"] = vec(m.heads, -1.0, 1.0)
            sd[p + "mix.norm"] = vec(m.vdim, 0.5, 1.5)
            sd[p + "mix.o"] = mat(d, m.heads * m.vdim)
        if ls.mlp is not None:
            f = ls.mlp
            sd[p + "norm2"] = vec(1, 0.5, 1.0).reshape(())
            for e in range(f.experts):
                sd[p + f"mlp.e{e}.gate"] = mat(f.ff, d)
                sd[p + f"mlp.e{e}.up"] = mat(f.ff, d)
                sd[p + f"mlp.e{e}.down"] = mat(d, f.ff)
            sd[p + "mlp.table"] = torch.stack([torch.randperm(f.experts, generator=g)[:f.top] for _ in range(v)]
                                              ).to(torch.int32)
        if config.side_dim:
            sd[p + "side.gate"] = mat(config.side_dim, d)
            sd[p + "side.proj"] = mat(d, config.side_dim)
            sd[p + "side.norm"] = vec(d, 0.2, 0.6)
    return sd


class ZavevikForCausalLM:
    """Causal LM over the hybrid op layer (inference)."""

    config_class = ZavevikConfig

    def __init__(self, config: ZavevikConfig, device="cpu", dtype=BF16, seed: int = 0, _do_init: bool = True):
        if dtype not in (BF16, F32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype}")
        self.config = config
        self.device = torch.device(device)
        self.param_dtype = dtype  # matrix operand / cache element type
        self.dtype = F32          # logits
        self.comm = NO_COMM
        self.vocab_local = config.vocab_size
        self.eps = config.norm_eps
        self.blocks: List[OutputNormBlock] = []
        self.embed: Optional[torch.Tensor] = None
        self.side_embed: Optional[torch.Tensor] = None
        self.final_norm: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        if _do_init:
            self.load_state_dict(random_state_dict(config, seed))

    # ------------------------------------------------------------------ weights
    def load_state_dict(self, sd: Dict[str, torch.Tensor]) -> "ZavevikForCausalLM":
        c, dev, wdt, eps = self.config, self.device, self.param_dtype, self.eps

        def mat(*names):  # one matrix, or several stacked along the rows
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            return t.to(dev, wdt).contiguous()

        def f32(name):
            return sd[name].to(dev, F32).reshape(-1).contiguous()

        self.embed = mat("embed")
        self.side_embed = mat("side.embed") if c.side_dim else None
        self.final_norm = f32("final.norm")
        self.head = mat("head")
        self.blocks = []
        for i, ls in enumerate(c.layers):
            p, m = f"l{i}.", ls.mixer
            if m.type == "attention":
                names = [p + "mix.q"] + ([p + "mix.k", p + "mix.v"] if m.kv_from is None else [])
                rel = sd.get(p + "mix.rel")
                if rel is not None and not m.bias_max:
                    raise ValueError(f"layer {i}: a distance-bias table without bias_max")
                bias = hy.distance_bias_table(rel.to(dev, F32), m.bias_max) if rel is not None else None
                mixer = BiasedAttention(i, m, eps, mat(*names), mat(p + "mix.o"), bias)
            else:
                w_in = mat(*(p + "mix." + n for n in ("q", "k", "v", "g", "b", "a")))
                conv = torch.cat([sd[p + f"mix.{n}.conv"] for n in ("q", "k", "v")], 0).to(dev, F32).contiguous()
                mixer = GatedDeltaMixer(i, m, eps, w_in, conv, f32(p + "mix.A_log"), f32(p + "mix.dt_bias"),
                                        f32(p + "mix.norm"), mat(p + "mix.o"))
            mlp = norm2 = None
            if ls.mlp is not None:
                f = ls.mlp
                w_gu = torch.stack([torch.cat([sd[p + f"mlp.e{e}.gate"], sd[p + f"mlp.e{e}.up"]], 0)
                                    for e in range(f.experts)]).to(dev, wdt).contiguous()
                w_down = torch.stack([sd[p + f"mlp.e{e}.down"] for e in range(f.experts)]).to(dev, wdt).contiguous()
                table = sd[p + "mlp.table"].to(dev, torch.int32).contiguous()
                if table.shape != (c.vocab_size, f.top):
                    raise ValueError(f"layer {i}: expert table of shape {tuple(table.shape)}")
                mlp, norm2 = TableMoE(f, table, w_gu, w_down), f32(p + "norm2")
            side = None
            if c.side_dim:
                side = TokenSide(self.side_embed, i * c.side_dim, mat(p + "side.gate"), mat(p + "side.proj"),
                                 f32(p + "side.norm"), eps)
            self.blocks.append(OutputNormBlock(mixer, f32(p + "norm1"), mlp, norm2, side, eps))
        return self

    @classmethod
    def from_pretrained(cls, directory: str, device="cpu", dtype=BF16) -> "ZavevikForCausalLM":
        from safetensors import safe_open
        config = ZavevikConfig.from_pretrained(directory)
        model = cls(config, device=device, dtype=dtype, _do_init=False)
        sd = {}
        with safe_open(os.path.join(directory, "model.safetensors"), framework="pt", device="cpu") as f:
            for k in f.keys():
                sd[k] = f.get_tensor(k)
        return model.load_state_dict(sd)

    def save_pretrained(self, directory: str, state_dict: Dict[str, torch.Tensor]) -> None:
        """Write ``config.json`` + ``model.safetensors`` (checkpoint names) from a checkpoint-named state dict."""
        from safetensors.torch import save_file
        self.config.save_pretrained(directory)
        save_file({k: v.contiguous() for k, v in state_dict.items()}, os.path.join(directory, "model.safetensors"))

    def weight_bytes(self) -> int:
        seen, n = set(), 0
        stack = [self.embed, self.side_embed, self.head]
        for blk in self.blocks:
            for obj in (blk.mixer, blk.mlp, blk.side):
                if obj is not None:
                    stack += [t for t in vars(obj).values() if torch.is_tensor(t)]
        for t in stack:
            if t is not None and t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ cache
    def init_cache(self, batch_size: int, max_length: int) -> HybridCache:
        return HybridCache(cache_specs(self.config), batch_size, max_length, self.device, self.param_dtype)

    def cache_nbytes(self, batch_size: int, max_length: int) -> int:
        return HybridCache.bytes_per(cache_specs(self.config), batch_size, max_length, self.param_dtype)

    # ------------------------------------------------------------------ forward
    def forward_tokens(self, ids: torch.Tensor, positions: torch.Tensor, cache, slot0, kv_start=None, key_mask=None,
                       logits_mode: str = "last", collect_hidden: bool = False, collect_attn: bool = False,
                       logit_rows: Optional[torch.Tensor] = None):
        """Run all layers for ``ids [B, S]`` placed at cache slots ``slot0 .. slot0 + S - 1`` (``slot0``: int or a
        device int32[1]); keys / values and recurrent state of ``cache`` advance. Returns ``(logits, x, hidden, [])``:
        fp32 logits ``[B, V]`` ("last" / "argmax": the sampler reduces them), ``[B*S, V]`` ("all"), the rows
        ``logit_rows`` of the flattened ``[B*S]`` tokens ("rows"), or None ("none"). ``hidden`` (``collect_hidden``):
        the residual stream after every layer. Recurrent layers carry no padding mask: every row's tokens must be
        real (``kv_start`` all zero, no ``key_mask``)."""
        if key_mask is not None or collect_attn:
            raise NotImplementedError("Zavevik: key masks / attention maps are not supported")
        b, s = ids.shape
        d = self.config.hidden_size
        idf = ids.reshape(-1).to(self.device, torch.int32).contiguous()
        ctx = StepContext(idf, positions.reshape(-1).to(self.device, torch.int32).contiguous(), b, s, cache, slot0)
        x = hy.embed_rows(idf, self.embed)
        hidden = []
        for blk in self.blocks:
            blk(x, ctx)
            if collect_hidden:
                hidden.append(x.reshape(b, s, d).clone())
        if logits_mode == "none":
            return None, x, hidden, []
        if logits_mode in ("last", "argmax"):
            xl = x.reshape(b, s, d)[:, -1].contiguous()
        elif logits_mode == "rows":
            xl = x.index_select(0, logit_rows.to(self.device, torch.long))
        elif logits_mode == "all":
            xl = x
        else:
            raise ValueError(f"unknown logits_mode {logits_mode!r}")
        logits = hy.linear(hy.rms_rows(xl, self.final_norm, self.eps), self.head)
        return logits, x, hidden, []

    def gather_logits(self, logits_local: torch.Tensor) -> torch.Tensor:
        return logits_local

    def __call__(self, input_ids, position_ids=None, past_key_values: Optional[HybridCache] = None,
                 output_hidden_states: bool = False):
        """Logits for every position ``[B, S, V]`` (fp32); ``past_key_values`` (an ``init_cache`` object) is advanced in
        place when given. Returns ``CausalLMOutput``."""
        from .llama import CausalLMOutput
        ids = torch.as_tensor(input_ids).to(self.device, torch.int32)
        b, s = ids.shape
        cache = past_key_values if past_key_values is not None else self.init_cache(b, s)
        slot0 = cache.index
        if slot0 + s > cache.max_length:
            raise ValueError(f"cache overflow: {slot0}+{s} > {cache.max_length}")
        if position_ids is None:
            position_ids = torch.arange(slot0, slot0 + s, dtype=torch.int32).expand(b, s)
        pos = torch.as_tensor(position_ids).to(self.device, torch.int32).reshape(b, s).contiguous()
        logits, _, hidden, _ = self.forward_tokens(ids, pos, cache, slot0, logits_mode="all",
                                                   collect_hidden=output_hidden_states)
        if past_key_values is not None:
            cache.advance(s)
        return CausalLMOutput(logits=logits.reshape(b, s, -1), past_key_values=past_key_values,
                              hidden_states=tuple(hidden) if output_hidden_states else None)

    def generate(self, input_ids, attention_mask=None, generation_config=None, prng_key=None, **kwargs):
        """Greedy / sampled generation on the framework's decode engine (``runtime/engine.py``)."""
        from ..runtime.engine import generate as _generate
        if attention_mask is not None and not bool(torch.as_tensor(attention_mask).bool().all()):
            raise NotImplementedError("Zavevik: padded batches are not supported (recurrent layers carry no mask)")
        return _generate(self, input_ids, None, generation_config, prng_key=prng_key, **kwargs)
