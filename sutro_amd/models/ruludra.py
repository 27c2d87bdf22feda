"""Ruludra: a layer-list decoder with sandwich norms and depth-weighted
layer inputs. Each layer has one token mixer (windowed attention whose values
are its keys, latent attention, or an mLSTM) and an optional PolyNorm
feed-forward.

Embedding: token row + hashed-bigram row + sinusoid of the position = X_0.
Layer i, with input x (X_0 for the first layer) and weighted RMS norms n_*:
    x <- x + n_1b(mixer(n_1(x)));  x <- x + n_2b(ff(n_2(x)))   (if it has one)
    X_{i+1} = x;   next input = sum_{j <= i+1} w_i[j] * X_j
Output: logits = head(n_final(last input)) * logit_scale.

The residual stream and every X_j are fp32; GEMM operands are the engine's
activation type. Per sublayer: one merged input GEMM, the mixer kernels, one
output GEMM, and ONE kernel that applies the post-norm, the residual add, (at
a layer's end) the depth-weighted sum and the next sublayer's pre-norm.
"""

from __future__ import annotations

import math
import zlib
from typing import Dict, Optional

import torch
import torch.nn as nn

from ..engine.batch import ForwardBatch
from ..engine.kv_cache import PagedKVCache
from ..ops import hybrid as hops
from ..parallel.tp import TPContext
from .hybrid_spec import (HybridLayerSpec, HybridSpec, LatentAttnMixerSpec,
                          MLSTMMixerSpec, TiedAttnMixerSpec)
from .layers import (MLSTM, LatentAttention, SectionedLinear,
                     TiedWindowAttention, _pad)


class SandwichBlock(nn.Module):
    """One layer: pre- and post-normed mixer sublayer, optional pre- and
    post-normed PolyNorm feed-forward, then the depth-weighted sum that makes
    the next layer's input."""

    def __init__(self, spec: HybridSpec, layer: HybridLayerSpec, idx: int,
                 dtype: torch.dtype):
        super().__init__()
        W = spec.hidden_size
        self.idx = idx
        self.eps = spec.norm_eps
        m = layer.mixer
        if isinstance(m, TiedAttnMixerSpec):
            self.mixer = TiedWindowAttention(m, spec.norm_eps, idx)
        elif isinstance(m, LatentAttnMixerSpec):
            self.mixer = LatentAttention(m, spec.norm_eps, idx, dtype)
        elif isinstance(m, MLSTMMixerSpec):
            self.mixer = MLSTM(m, spec.norm_eps, idx)
        else:
            raise ValueError(f"layer {idx}: unsupported mixer {type(m).__name__}")
        self.in_proj = SectionedLinear(W, self.mixer.in_sections(""), dtype)
        k = _pad(self.mixer.out_width)
        self.out_padded = k != self.mixer.out_width
        self.out_proj = nn.Linear(k, W, bias=False, dtype=dtype)
        f32 = torch.float32
        self.norm1 = nn.Parameter(torch.ones(W, dtype=f32))
        self.norm1b = nn.Parameter(torch.ones(W, dtype=f32))
        self.depth_w = nn.Parameter(torch.zeros(idx + 2, dtype=f32))
        self.ff = layer.ff
        if layer.ff:
            self.norm2 = nn.Parameter(torch.ones(W, dtype=f32))
            self.norm2b = nn.Parameter(torch.ones(W, dtype=f32))
            self.ff_up = nn.Linear(W, layer.ff, bias=False, dtype=dtype)
            self.ff_down = nn.Linear(layer.ff, W, bias=False, dtype=dtype)
            self.ff_coef = nn.Parameter(torch.zeros(4, dtype=f32))

    def checkpoint_targets(self, prefix: str) -> Dict[str, tuple]:
        lp = f"l{self.idx}"
        ck = lp + ".mix"
        W = self.norm1.numel()
        t: Dict[str, tuple] = {}
        t.update(self.mixer.param_targets(prefix + "mixer.", ck))
        t.update(self.in_proj.section_targets(
            prefix + "in_proj.", self.mixer.section_names("", ck)))
        t[ck + ".o"] = (prefix + "out_proj.weight", 1, 0,
                        self.mixer.out_width, 1.0)
        t[lp + ".norm1"] = (prefix + "norm1", 0, 0, W, 1.0)
        t[lp + ".norm1b"] = (prefix + "norm1b", 0, 0, W, 1.0)
        t[lp + ".dwa"] = (prefix + "depth_w", 0, 0, self.idx + 2, 1.0)
        if self.ff:
            t[lp + ".norm2"] = (prefix + "norm2", 0, 0, W, 1.0)
            t[lp + ".norm2b"] = (prefix + "norm2b", 0, 0, W, 1.0)
            t[lp + ".mlp.up"] = (prefix + "ff_up.weight", 0, 0, self.ff, 1.0)
            t[lp + ".mlp.down"] = (prefix + "ff_down.weight", 1, 0, self.ff, 1.0)
            t[lp + ".mlp.act"] = (prefix + "ff_coef", 0, 0, 4, 1.0)
        return t

    def forward(self, X: torch.Tensor, xw: torch.Tensor, h: torch.Tensor,
                fb: ForwardBatch, kv: PagedKVCache,
                next_w: torch.Tensor) -> None:
        """X [L+1, T, W] fp32: X[j] for j <= idx are filled, X[idx+1] is
        written. xw [T, W] fp32: this layer's input when idx > 0 (X[0] is the
        first layer's), overwritten with the next layer's input. h [T, W]
        activation type: this layer's normed input, overwritten with the next
        layer's (normed with `next_w`)."""
        i = self.idx
        x_in = X[0] if i == 0 else xw
        x_out = X[i + 1]
        T = h.shape[0]
        proj = self.in_proj(h)
        alloc = torch.zeros if self.out_padded else torch.empty
        mix_in = alloc((T, self.out_proj.in_features), dtype=h.dtype,
                       device=h.device)
        self.mixer(proj, self.in_proj.offsets, "", fb, kv, mix_in, 0, 1.0)
        y = self.out_proj(mix_in)
        if self.ff:
            hops.norm_residual(x_in, y, self.norm1b, self.eps, x_out,
                               next_w=self.norm2, h_out=h)
            act = hops.poly_act(self.ff_up(h), self.ff_coef, self.eps)
            y = self.ff_down(act)
            x_in = x_out
        hops.norm_residual(x_in, y, self.norm2b if self.ff else self.norm1b,
                           self.eps, x_out, stack=X, depth_w=self.depth_w,
                           mix_out=xw, next_w=next_w, h_out=h)


class RuludraModel(nn.Module):
    """Same engine-facing surface as the other models: forward(fb, kv) ->
    hidden rows, compute_logits(hidden), cache_layout(),
    checkpoint_targets(), init_random_weights()."""

    # the embedding looks at (previous token, token) pairs: the engine fills
    # ForwardBatch.prev_ids
    uses_prev_ids = True

    def __init__(self, spec: HybridSpec, dtype: torch.dtype, max_len: int,
                 tp: Optional[TPContext] = None):
        super().__init__()
        self.spec = spec
        self.tp = tp or TPContext()
        if self.tp.size > 1:
            raise NotImplementedError(
                "layer-list decoders run on one GPU per replica (the "
                "recurrent state is not sharded); use data parallelism")
        W = spec.hidden_size
        self.embed_tokens = nn.Embedding(spec.vocab_size, W, dtype=dtype)
        if spec.bigram:
            self.bigram = nn.Embedding(spec.bigram[0] + 1, W, dtype=dtype)
        if spec.pos_base:
            self.register_buffer(
                "pos_inv_freq", hops.sinusoid_inv_freq(W, spec.pos_base),
                persistent=False)
        self.layers = nn.ModuleList(
            [SandwichBlock(spec, layer, i, dtype)
             for i, layer in enumerate(spec.layers)])
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32))
        self.lm_head = nn.Linear(W, spec.vocab_size, bias=False, dtype=dtype)
        self.act_dtype = dtype
        # debugging aid: when set to a list, every layer's outgoing stream
        # (the next layer's input, fp32) is appended to it
        self.layer_taps: Optional[list] = None

    def cache_layout(self):
        """(per-layer KV shapes, per-layer recurrent state shapes)."""
        return ([blk.mixer.kv_shape() for blk in self.layers],
                [blk.mixer.state_shape() for blk in self.layers])

    def checkpoint_targets(self) -> Dict[str, tuple]:
        s = self.spec
        t = {"embed": ("embed_tokens.weight", 0, 0, s.vocab_size, 1.0),
             "head": ("lm_head.weight", 0, 0, s.vocab_size, 1.0),
             "final.norm": ("final_norm", 0, 0, s.hidden_size, 1.0)}
        if s.bigram:
            t["bigram"] = ("bigram.weight", 0, 0, s.bigram[0] + 1, 1.0)
        for i, blk in enumerate(self.layers):
            t.update(blk.checkpoint_targets(f"layers.{i}."))
        return t

    @torch.no_grad()
    def forward(self, fb: ForwardBatch, kv: PagedKVCache) -> torch.Tensor:
        fb.aux.clear()
        s = self.spec
        T = fb.input_ids.shape[0]
        L = len(self.layers)
        dev = fb.input_ids.device
        X = torch.empty((L + 1, T, s.hidden_size), dtype=torch.float32,
                        device=dev)
        big = s.bigram or (0, 0, 0)
        hops.token_embed(
            fb.input_ids, fb.prev_ids, fb.positions, self.embed_tokens.weight,
            self.bigram.weight if s.bigram else None, big[0], big[1], big[2],
            self.pos_inv_freq if s.pos_base else None, out=X[0])
        h = hops.weighted_rmsnorm(X[0], self.layers[0].norm1, s.norm_eps,
                                  self.act_dtype)
        xw = torch.empty((T, s.hidden_size), dtype=torch.float32, device=dev)
        for i, blk in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < L else self.final_norm
            blk(X, xw, h, fb, kv, nxt)
            if self.layer_taps is not None:
                self.layer_taps.append(xw.clone())
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden).float() * self.spec.logit_scale

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0) -> None:
        """Deterministic random init on the parameters' own device, scaled so
        activations, gates and the layer sums stay in a sane range."""
        for name, p in sorted(self.named_parameters()):
            gen = torch.Generator(device=p.device)
            gen.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))

            def rnd(shape, std):
                return torch.randn(shape, generator=gen, dtype=torch.float32,
                                   device=p.device) * std

            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "q_norm", "k_norm",
                        "dq_norm", "dkv_norm", "norm_w"):
                p.copy_(1.0 + rnd(p.shape, 0.05))
            elif leaf in ("norm1b", "norm2b"):
                p.copy_(0.5 + rnd(p.shape, 0.05))
            elif leaf == "depth_w":
                w = rnd(p.shape, 0.1).abs()
                w[-1] = 1.0
                p.copy_(w)
            elif leaf == "r1":
                p.copy_(rnd(p.shape, 0.3).abs())
            elif leaf == "r2":
                p.copy_(0.05 + rnd(p.shape, 0.2).abs())
            elif leaf == "ff_coef":
                p.copy_(torch.tensor([0.6, 0.3, 0.2, 0.0], device=p.device)
                        + rnd(p.shape, 0.05))
            elif leaf == "i_bias":
                p.copy_(rnd(p.shape, 0.5) - 1.0)
            elif leaf == "f_bias":
                p.copy_(rnd(p.shape, 0.5) + 3.0)
            elif name.startswith(("embed_tokens", "bigram")):
                p.copy_(rnd(p.shape, 1.0).to(p.dtype))
            else:
                p.copy_(rnd(p.shape, 1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        # padding rows/columns of merged projections stay zero
        for blk in self.layers:
            lin = blk.in_proj
            keep = torch.zeros(lin.out_features, dtype=torch.bool,
                               device=lin.weight.device)
            for sec, o in lin.offsets.items():
                keep[o:o + lin.sizes[sec]] = True
            lin.weight[~keep] = 0
            blk.out_proj.weight[:, blk.mixer.out_width:] = 0
