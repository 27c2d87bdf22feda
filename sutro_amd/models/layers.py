"""Reusable building blocks of layer-list decoders.

Every sublayer reads its input once: all projections that consume that input
(query/key/value of each mixer, low-rank gate inputs, the residual gate) are
rows of ONE merged weight, so a sublayer costs one input GEMM, a handful of
fused HIP kernels and one output GEMM. The kernels address their operands as
column sections of the merged GEMM output.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.batch import ForwardBatch
from ..engine.kv_cache import PagedKVCache
from ..ops import hybrid as hops
from .hybrid_spec import AttnMixerSpec, DeltaMixerSpec

_ALIGN = 8  # section starts are multiples of 8 columns (16 B in bf16)


def _pad(n: int) -> int:
    return (n + _ALIGN - 1) // _ALIGN * _ALIGN


class SectionedLinear(nn.Module):
    """One Linear whose output columns are named sections (each section a
    separate tensor in the checkpoint). Sections start on 8-column boundaries;
    padding rows are zero. A bias exists if any section has one (zero for the
    others)."""

    def __init__(self, in_features: int,
                 sections: Sequence[Tuple[str, int, bool]],
                 dtype: torch.dtype):
        super().__init__()
        self.offsets: Dict[str, int] = {}
        self.sizes: Dict[str, int] = {}
        self.biased: List[str] = []
        off = 0
        for name, rows, has_bias in sections:
            self.offsets[name] = off
            self.sizes[name] = rows
            if has_bias:
                self.biased.append(name)
            off += _pad(rows)
        self.out_features = off
        self.weight = nn.Parameter(torch.zeros(off, in_features, dtype=dtype))
        self.bias = (nn.Parameter(torch.zeros(off, dtype=dtype))
                     if self.biased else None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight, self.bias)

    def section_targets(self, prefix: str, names: Dict[str, str]):
        """Checkpoint tensor -> (parameter, dim, start, length, scale) for the
        loader. `names` maps section name -> checkpoint tensor name."""
        out = {}
        for sec, ck in names.items():
            o, n = self.offsets[sec], self.sizes[sec]
            out[ck] = (prefix + "weight", 0, o, n, 1.0)
            if sec in self.biased:
                out[ck + ".b"] = (prefix + "bias", 0, o, n, 1.0)
        return out


class LocalAttention(nn.Module):
    """Grouped-query softmax attention under a chunk and/or window mask, with
    per-head q/k RMS norm, rotation of a prefix of each head, split key and
    value sizes and a per-head sigmoid output gate. Owns no projection: it
    works on sections of the sublayer's merged projection and writes its
    gated heads into a slice of the merged output-projection input."""

    def __init__(self, spec: AttnMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        if spec.heads % spec.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim:
            raise ValueError("rot_dims must be even and at most dim")
        if spec.qk_norm:
            self.q_norm = nn.Parameter(torch.ones(spec.dim, dtype=torch.float32))
            self.k_norm = nn.Parameter(torch.ones(spec.dim, dtype=torch.float32))
        self.register_buffer("inv_freq",
                             hops.rope_inv_freq(spec.rot_dims, spec.rot_base),
                             persistent=False)

    def in_sections(self, tag: str):
        s = self.spec
        secs = [(tag + "q", s.heads * s.dim, s.bias),
                (tag + "k", s.kv_heads * s.dim, s.bias),
                (tag + "v", s.kv_heads * s.vdim, s.bias)]
        if s.out_gate:
            secs.append((tag + "g", s.heads, False))
        return secs

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def kv_shape(self):
        return (self.spec.kv_heads, self.spec.dim, self.spec.vdim)

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float) -> None:
        s = self.spec
        kc, vc = kv.k_cache[self.layer_idx], kv.v_cache[self.layer_idx]
        cos_sin = None
        if proj.is_cuda:
            # one cos/sin table per step and kind of rotation, shared by layers
            key = ("rope", s.rot_dims, s.rot_base)
            cos_sin = fb.aux.get(key)
            if cos_sin is None:
                cos_sin = fb.aux[key] = hops.rope_table(fb.positions,
                                                        self.inv_freq)
        q = hops.attn_prep(
            proj, off[tag + "q"], off[tag + "k"], off[tag + "v"], s.heads,
            s.kv_heads, s.dim, s.vdim,
            self.q_norm if s.qk_norm else None,
            self.k_norm if s.qk_norm else None,
            self.eps, self.inv_freq, fb.positions, fb.slot_mapping, kc, vc,
            cos_sin=cos_sin)
        hops.local_attention(
            q, kc, vc, fb.block_tables, fb.seq_lens, fb.query_start_locs,
            s.scale, s.chunk, s.window, proj,
            off[tag + "g"] if s.out_gate else -1, out, out_off, out_scale,
            token_seq=fb.token_seq, tile_seq=fb.tile_seq, tile_q0=fb.tile_q0,
            prefill_rows=fb.prefill_token_count)


class GatedDeltaRule(nn.Module):
    """Gated delta rule with per-channel decay: short causal filters + silu on
    q/k/v, unit-norm q and k, beta and decay gates in fp32, the token-by-token
    state update, then a per-head RMS norm with a low-rank sigmoid gate. The
    filter history and the memory matrix live in the engine's state cache."""

    def __init__(self, spec: DeltaMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        if spec.heads % spec.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        f32 = torch.float32
        ch = 2 * spec.kv_heads * spec.dim + spec.heads * spec.vdim
        self.channels = ch
        # small tensors the kernels read in fp32 (bf16 checkpoint values are
        # held exactly)
        self.conv_w = nn.Parameter(torch.zeros(ch, spec.conv, dtype=f32))
        self.a2 = nn.Parameter(torch.zeros(spec.heads * spec.dim,
                                           spec.decay_rank, dtype=f32))
        self.dt_bias = nn.Parameter(torch.zeros(spec.heads * spec.dim, dtype=f32))
        self.a_log = nn.Parameter(torch.zeros(spec.heads, dtype=f32))
        self.norm_w = nn.Parameter(torch.ones(spec.vdim, dtype=f32))
        self.g2 = nn.Parameter(torch.zeros(spec.heads * spec.vdim,
                                           spec.gate_rank, dtype=f32))
        self._t = None

    def in_sections(self, tag: str):
        s = self.spec
        return [(tag + "q", s.kv_heads * s.dim, False),
                (tag + "k", s.kv_heads * s.dim, False),
                (tag + "v", s.heads * s.vdim, False),
                (tag + "b", s.heads, False),
                (tag + "a1", s.decay_rank, False),
                (tag + "g1", s.gate_rank, False)]

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def state_shape(self):
        s = self.spec
        return (self.channels, s.conv, s.heads, s.dim, s.vdim)

    def param_targets(self, prefix: str, ck: str):
        """Checkpoint tensors of this mixer that are not projections of the
        sublayer input."""
        s = self.spec
        cq = s.kv_heads * s.dim
        return {
            ck + ".q.conv": (prefix + "conv_w", 0, 0, cq, 1.0),
            ck + ".k.conv": (prefix + "conv_w", 0, cq, cq, 1.0),
            ck + ".v.conv": (prefix + "conv_w", 0, 2 * cq, s.heads * s.vdim, 1.0),
            ck + ".a2": (prefix + "a2", 0, 0, s.heads * s.dim, 1.0),
            ck + ".dt_bias": (prefix + "dt_bias", 0, 0, s.heads * s.dim, 1.0),
            ck + ".A_log": (prefix + "a_log", 0, 0, s.heads, 1.0),
            ck + ".norm": (prefix + "norm_w", 0, 0, s.vdim, 1.0),
            ck + ".g2": (prefix + "g2", 0, 0, s.heads * s.vdim, 1.0),
        }

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float) -> None:
        s = self.spec
        st = kv.state
        if self._t is None or self._t[0].device != proj.device:
            # transposed copies of the low-rank up-projections, made once
            # (before any graph capture: capture is preceded by a warm-up run)
            self._t = (self.a2.detach().t().contiguous(),
                       self.g2.detach().t().contiguous(),
                       self.conv_w.detach().t().contiguous())
        qn, kn, v, decay, beta = hops.delta_prep(
            proj, off[tag + "q"], off[tag + "k"], off[tag + "v"],
            off[tag + "b"], off[tag + "a1"], s.heads, s.kv_heads, s.dim,
            s.vdim, self.conv_w, self.a2, self.dt_bias, self.a_log,
            st.conv[self.layer_idx], fb.state_slots, fb.query_start_locs,
            fb.seq_lens, token_seq=fb.token_seq, a2_t=self._t[0],
            conv_w_t=self._t[2])
        o = hops.delta_scan(qn, kn, v, decay, beta, st.ssm[self.layer_idx],
                            fb.state_slots, fb.query_start_locs, fb.seq_lens)
        hops.delta_out(o, self.norm_w, proj, off[tag + "g1"], self.g2,
                       self.eps, out, out_off, out_scale, g2_t=self._t[1])
