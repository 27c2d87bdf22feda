"""Vodinex: a layer-list decoder whose layers mix tokens either with a gated
delta rule alone or with chunked softmax attention and a gated delta rule
side by side, optionally followed by a tanh-GELU gated feed-forward.

Residual form (m = residual_mult, n = scalar-gain RMS norm of the result):
    x <- x + m * n(sigmoid(R1 x + r1) * mixer(x))
    x <- x + m * n(sigmoid(R2 x + r2) * ff(x))        (if the layer has one)
Sublayers read x itself; the residual stream, norms and everything the
recurrence consumes are fp32, GEMM operands are the engine's activation type.

Per sublayer the work is: one merged input GEMM (all projections of x and the
residual gate), the mixer kernels (sutro_amd/ops/hybrid.py), one output GEMM
over the concatenated heads of all mixers of the layer, and one fused
gate + norm + residual kernel.
"""

from __future__ import annotations

import math
import zlib
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.batch import ForwardBatch
from ..engine.kv_cache import PagedKVCache
from ..ops import hybrid as hops
from ..parallel.tp import TPContext
from .hybrid_spec import (AttnMixerSpec, DeltaMixerSpec, HybridLayerSpec,
                          HybridSpec, ParallelMixerSpec)
from .layers import GatedDeltaRule, LocalAttention, SectionedLinear, _pad


class HybridBlock(nn.Module):
    def __init__(self, spec: HybridSpec, layer: HybridLayerSpec, idx: int,
                 dtype: torch.dtype):
        super().__init__()
        W = spec.hidden_size
        self.idx = idx
        self.eps = spec.norm_eps
        self.mult = spec.residual_mult
        m = layer.mixer
        mixers = []           # (tag, module, out_scale, checkpoint prefix)
        ck = f"l{idx}.mix"
        if isinstance(m, ParallelMixerSpec):
            mixers.append(("L.", LocalAttention(m.left, spec.norm_eps, idx),
                           m.left_scale, ck + ".left"))
            mixers.append(("R.", GatedDeltaRule(m.right, spec.norm_eps, idx),
                           m.right_scale, ck + ".right"))
        elif isinstance(m, DeltaMixerSpec):
            mixers.append(("", GatedDeltaRule(m, spec.norm_eps, idx), 1.0, ck))
        else:
            mixers.append(("", LocalAttention(m, spec.norm_eps, idx), 1.0, ck))
        self.mixers = nn.ModuleList([mod for _, mod, _, _ in mixers])
        self._mix_meta = [(tag, scale, pre) for tag, _, scale, pre in mixers]
        sections = []
        for tag, mod, _, _ in mixers:
            sections += mod.in_sections(tag)
        sections.append(("rg", W, True))
        self.in_proj = SectionedLinear(W, sections, dtype)
        self.out_offsets: List[int] = []
        k_total = 0
        for _, mod, _, _ in mixers:
            self.out_offsets.append(k_total)
            k_total += _pad(mod.out_width)
        self.out_padded = any(_pad(mod.out_width) != mod.out_width
                              for _, mod, _, _ in mixers)
        has_bias = any(isinstance(mod, LocalAttention) and mod.spec.bias
                       for _, mod, _, _ in mixers)
        self.out_proj = nn.Linear(k_total, W, bias=has_bias, dtype=dtype)
        self.norm1 = nn.Parameter(torch.ones((), dtype=torch.float32))
        self.ff = layer.ff
        if layer.ff:
            self.ff_in = SectionedLinear(
                W, [("gate", layer.ff, False), ("up", layer.ff, False),
                    ("rg", W, True)], dtype)
            self.ff_out = nn.Linear(layer.ff, W, bias=False, dtype=dtype)
            self.norm2 = nn.Parameter(torch.ones((), dtype=torch.float32))

    # ---- cache layout ----

    def kv_shape(self):
        for mod in self.mixers:
            if isinstance(mod, LocalAttention):
                return mod.kv_shape()
        return None

    def state_shape(self):
        for mod in self.mixers:
            if isinstance(mod, GatedDeltaRule):
                return mod.state_shape()
        return None

    # ---- checkpoint layout ----

    def checkpoint_targets(self, prefix: str) -> Dict[str, tuple]:
        t: Dict[str, tuple] = {}
        lp = f"l{self.idx}"
        names = {"rg": lp + ".rg1"}
        for (tag, scale, ck), mod, o_off in zip(self._mix_meta, self.mixers,
                                                self.out_offsets):
            mp = f"{prefix}mixers.{list(self.mixers).index(mod)}."
            if isinstance(mod, LocalAttention):
                names.update({tag + "q": ck + ".q", tag + "k": ck + ".k",
                              tag + "v": ck + ".v"})
                if mod.spec.out_gate:
                    names[tag + "g"] = ck + ".g"
                if mod.spec.qk_norm:
                    t[ck + ".q.norm"] = (mp + "q_norm", 0, 0, mod.spec.dim, 1.0)
                    t[ck + ".k.norm"] = (mp + "k_norm", 0, 0, mod.spec.dim, 1.0)
                if mod.spec.bias:
                    t[ck + ".o.b"] = (prefix + "out_proj.bias", 0, 0,
                                      self.out_proj.out_features, scale)
            else:
                names.update({tag + k: ck + "." + k
                              for k in ("q", "k", "v", "b", "a1", "g1")})
                t.update(mod.param_targets(mp, ck))
            t[ck + ".o"] = (prefix + "out_proj.weight", 1, o_off,
                            mod.out_width, 1.0)
        t.update(self.in_proj.section_targets(prefix + "in_proj.", names))
        t[lp + ".norm1"] = (prefix + "norm1", None, 0, 0, 1.0)
        if self.ff:
            t.update(self.ff_in.section_targets(
                prefix + "ff_in.", {"gate": lp + ".mlp.gate",
                                    "up": lp + ".mlp.up", "rg": lp + ".rg2"}))
            t[lp + ".mlp.down"] = (prefix + "ff_out.weight", 1, 0, self.ff, 1.0)
            t[lp + ".norm2"] = (prefix + "norm2", None, 0, 0, 1.0)
        return t

    # ---- compute ----

    def forward(self, x: torch.Tensor, h: torch.Tensor, fb: ForwardBatch,
                kv: PagedKVCache) -> None:
        """x: fp32 residual stream [T, W], updated in place. h: x in the
        activation type (the same tensor when that is fp32), updated too."""
        h_out = None if h is x else h
        proj = self.in_proj(h)
        off = self.in_proj.offsets
        T = x.shape[0]
        alloc = torch.zeros if self.out_padded else torch.empty
        mix_in = alloc((T, self.out_proj.in_features), dtype=h.dtype,
                       device=h.device)
        for (tag, scale, _), mod, o_off in zip(self._mix_meta, self.mixers,
                                               self.out_offsets):
            mod(proj, off, tag, fb, kv, mix_in, o_off, scale)
        y = self.out_proj(mix_in)
        hops.gated_norm_residual(x, y, proj, off["rg"], self.norm1, self.eps,
                                 self.mult, h_out)
        if self.ff:
            proj = self.ff_in(h)
            off = self.ff_in.offsets
            act = hops.gelu_tanh_mul(proj, off["gate"], off["up"], self.ff)
            y = self.ff_out(act)
            hops.gated_norm_residual(x, y, proj, off["rg"], self.norm2,
                                     self.eps, self.mult, h_out)


class VodinexModel(nn.Module):
    """Same engine-facing surface as Qwen3Model: forward(fb, kv) -> hidden
    rows, compute_logits(hidden), cache_layout(), init_random_weights()."""

    def __init__(self, spec: HybridSpec, dtype: torch.dtype, max_len: int,
                 tp: Optional[TPContext] = None):
        super().__init__()
        self.spec = spec
        self.tp = tp or TPContext()
        if self.tp.size > 1:
            raise NotImplementedError(
                "layer-list decoders run on one GPU per replica (the "
                "recurrent state is not sharded); use data parallelism")
        self.embed_tokens = nn.Embedding(spec.vocab_size, spec.hidden_size,
                                         dtype=dtype)
        self.layers = nn.ModuleList(
            [HybridBlock(spec, layer, i, dtype)
             for i, layer in enumerate(spec.layers)])
        self.final_norm = nn.Parameter(torch.ones((), dtype=torch.float32))
        self.lm_head = nn.Linear(spec.hidden_size, spec.vocab_size, bias=False,
                                 dtype=dtype)
        self.act_dtype = dtype
        # debugging aid: when set to a list, the fp32 residual stream after
        # every layer is appended to it
        self.layer_taps: Optional[list] = None

    def cache_layout(self):
        """(per-layer KV shapes, per-layer recurrent state shapes)."""
        return ([blk.kv_shape() for blk in self.layers],
                [blk.state_shape() for blk in self.layers])

    def checkpoint_targets(self) -> Dict[str, tuple]:
        t = {"embed": ("embed_tokens.weight", 0, 0, self.spec.vocab_size, 1.0),
             "head": ("lm_head.weight", 0, 0, self.spec.vocab_size, 1.0),
             "final.norm": ("final_norm", None, 0, 0, 1.0)}
        for i, blk in enumerate(self.layers):
            t.update(blk.checkpoint_targets(f"layers.{i}."))
        return t

    @torch.no_grad()
    def forward(self, fb: ForwardBatch, kv: PagedKVCache) -> torch.Tensor:
        # per-step scratch (rotation tables) is rebuilt on every pass: a batch
        # object that is run again (graph warm-up, then capture) must not keep
        # tables of the earlier pass
        fb.aux.clear()
        h = self.embed_tokens(fb.input_ids)
        if h.dtype == torch.float32:
            x = h = h.clone()
        else:
            x = h.float()
        for blk in self.layers:
            blk(x, h, fb, kv)
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        return hops.scalar_rmsnorm(x, self.final_norm, self.spec.norm_eps,
                                   self.act_dtype)

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden)

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0) -> None:
        """Deterministic random init on the parameters' own device, scaled so
        activations and decays stay in a sane range at any width."""
        for name, p in sorted(self.named_parameters()):
            gen = torch.Generator(device=p.device)
            gen.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))

            def rnd(shape, std):
                return torch.randn(shape, generator=gen, dtype=torch.float32,
                                   device=p.device) * std

            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm"):
                p.fill_(1.0)
            elif leaf in ("q_norm", "k_norm", "norm_w"):
                p.copy_(1.0 + rnd(p.shape, 0.05))
            elif leaf == "a_log":
                p.copy_(rnd(p.shape, 0.3) - 0.5)
            elif leaf == "dt_bias":
                p.copy_(rnd(p.shape, 0.5) - 1.0)
            elif leaf == "conv_w":
                p.copy_(rnd(p.shape, 0.4))
            elif leaf == "bias":
                p.copy_(rnd(p.shape, 0.02).to(p.dtype))
            elif "embed" in name:
                p.copy_(rnd(p.shape, 1.0).to(p.dtype))
            else:
                p.copy_(rnd(p.shape, 1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        # padding rows/columns of merged projections stay zero
        for blk in self.layers:
            for lin in ([blk.in_proj] + ([blk.ff_in] if blk.ff else [])):
                keep = torch.zeros(lin.out_features, dtype=torch.bool,
                                   device=lin.weight.device)
                for sec, o in lin.offsets.items():
                    keep[o:o + lin.sizes[sec]] = True
                lin.weight[~keep] = 0
                if lin.bias is not None:
                    lin.bias[~keep] = 0
            keepc = torch.zeros(blk.out_proj.in_features, dtype=torch.bool,
                                device=blk.out_proj.weight.device)
            for mod, o in zip(blk.mixers, blk.out_offsets):
                keepc[o:o + mod.out_width] = True
            blk.out_proj.weight[:, ~keepc] = 0
