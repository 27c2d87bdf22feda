"""Ops of layer-list ("hybrid") decoders: scalar-gain norms with gated
residuals, tanh-GELU gating, local (chunked / windowed) paged attention with
split key/value sizes and partial rotation, and the gated delta rule.

GPU tensors run the HIP kernels of the `sutro_amd._C_mix` extension
(csrc/mix_*.hip), templated on the activation type: bf16 when the engine
serves in bf16, fp32 when it serves in fp32. CPU tensors run the torch
reference. A GPU tensor without the built extension raises.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import torch_ref

_M = None
_M_ERR: Optional[str] = None
try:
    from sutro_amd import _C_mix as _M  # type: ignore
except Exception as e:  # pragma: no cover - only without the built extension
    _M_ERR = f"{type(e).__name__}: {e}"


def mix_available() -> bool:
    return _M is not None


def _mix():
    global _M, _M_ERR
    if _M is None:  # the extension may have been built after this import
        try:
            import importlib

            _M = importlib.import_module("sutro_amd._C_mix")
        except Exception as e:
            _M_ERR = f"{type(e).__name__}: {e}"
    if _M is None:
        raise RuntimeError(
            "sutro_amd HIP extension (_C_mix) is not built but a GPU tensor "
            "was passed. Build it with `python setup.py build_ext --inplace` "
            f"(import error: {_M_ERR})")
    return _M


rope_inv_freq = torch_ref.rope_inv_freq


def gelu_tanh_mul(proj: torch.Tensor, gate_off: int, up_off: int,
                  ff: int) -> torch.Tensor:
    if proj.is_cuda:
        out = torch.empty((proj.shape[0], ff), dtype=proj.dtype,
                          device=proj.device)
        _mix().gelu_tanh_mul(out, proj, gate_off, up_off)
        return out
    return torch_ref.gelu_tanh_mul(proj, gate_off, up_off, ff)


def gated_norm_residual(x, y, proj, gate_off: int, gain, eps: float,
                        mult: float, h_out=None) -> None:
    if x.is_cuda:
        _mix().gated_norm_residual(x, y, proj, gate_off, gain, eps, mult,
                                   h_out)
        return
    torch_ref.gated_norm_residual(x, y, proj, gate_off, gain, eps, mult, h_out)


def scalar_rmsnorm(x, gain, eps: float, out_dtype: torch.dtype):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _mix().scalar_rmsnorm(out, x, gain, eps)
        return out
    return torch_ref.scalar_rmsnorm(x, gain, eps, out_dtype)


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """fp32 [T, 2*half]: cos | sin of the fp32 angle position * inv_freq.
    One table serves every layer of a step that rotates alike."""
    ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.unsqueeze(0)
    return torch.cat([ang.cos(), ang.sin()], dim=1).contiguous()


def attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv, q_norm_w, k_norm_w,
              eps, inv_freq, positions, slot_mapping, k_cache, v_cache,
              cos_sin=None):
    if proj.is_cuda:
        q = torch.empty((proj.shape[0], H, dk), dtype=proj.dtype,
                        device=proj.device)
        if cos_sin is None:
            cos_sin = rope_table(positions, inv_freq)
        _mix().attn_prep(q, proj, q_off, k_off, v_off, q_norm_w, k_norm_w,
                         eps, cos_sin, slot_mapping, k_cache, v_cache)
        return q
    return torch_ref.attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv,
                               q_norm_w, k_norm_w, eps, inv_freq, positions,
                               slot_mapping, k_cache, v_cache)


def local_attention(q, k_cache, v_cache, block_tables, seq_lens,
                    query_start_locs, scale: float, chunk: int, window: int,
                    proj, gate_off: int, out, out_off: int, out_scale: float,
                    token_seq=None, tile_seq=None, tile_q0=None,
                    prefill_rows: int = 0):
    """`tile_seq`/`tile_q0` (int32, 32 query rows a tile) cover the first
    `prefill_rows` rows: on the GPU in bf16 those rows run on the MFMA kernel
    when page size and head sizes allow it; the remaining (single-token) rows
    and all other cases run on the generic one-wave-per-row kernel."""
    if q.is_cuda:
        if tile_seq is None or tile_seq.numel() == 0:
            tile_seq = tile_q0 = None
            prefill_rows = 0
        _mix().local_attention(out, out_off, q, k_cache, v_cache,
                               block_tables, seq_lens, query_start_locs,
                               token_seq, scale, chunk, window, proj,
                               gate_off, out_scale, tile_seq, tile_q0,
                               prefill_rows)
        return
    torch_ref.local_attention(q, k_cache, v_cache, block_tables, seq_lens,
                              query_start_locs, scale, chunk, window, proj,
                              gate_off, out, out_off, out_scale)


def delta_prep(proj, q_off, k_off, v_off, b_off, a1_off, H, G, dk, dv,
               conv_w, a2, dt_bias, a_log, conv_state, state_slots,
               query_start_locs, seq_lens, token_seq=None, a2_t=None,
               conv_w_t=None):
    """`a2_t`, `conv_w_t`: a2 and conv_w transposed and contiguous ([rank,
    H*dk] and [taps, C], what the kernels read); made on the fly when the
    caller does not keep them."""
    if proj.is_cuda:
        if a2_t is None:
            a2_t = a2.t().contiguous()
        if conv_w_t is None:
            conv_w_t = conv_w.t().contiguous()
        T = proj.shape[0]
        f32 = dict(dtype=torch.float32, device=proj.device)
        qn = torch.empty((T, G, dk), **f32)
        kn = torch.empty((T, G, dk), **f32)
        v = torch.empty((T, H, dv), **f32)
        decay = torch.empty((T, H, dk), **f32)
        beta = torch.empty((T, H), **f32)
        _mix().delta_prep(qn, kn, v, decay, beta, proj, q_off, k_off, v_off,
                          b_off, a1_off, conv_w, a2_t, dt_bias, a_log,
                          conv_state, state_slots, query_start_locs, seq_lens,
                          token_seq, conv_w_t)
        return qn, kn, v, decay, beta
    return torch_ref.delta_prep(proj, q_off, k_off, v_off, b_off, a1_off, H,
                                G, dk, dv, conv_w, a2, dt_bias, a_log,
                                conv_state, state_slots, query_start_locs,
                                seq_lens)


def delta_scan(qn, kn, v, decay, beta, ssm_state, state_slots,
               query_start_locs, seq_lens):
    if v.is_cuda:
        o = torch.empty_like(v)
        _mix().delta_scan(o, qn, kn, v, decay, beta, ssm_state, state_slots,
                          query_start_locs, seq_lens)
        return o
    return torch_ref.delta_scan(qn, kn, v, decay, beta, ssm_state,
                                state_slots, query_start_locs, seq_lens)


def delta_out(o, norm_w, proj, g1_off: int, g2, eps: float, out,
              out_off: int, out_scale: float, g2_t=None) -> None:
    if o.is_cuda:
        if g2_t is None:
            g2_t = g2.t().contiguous()
        _mix().delta_out(out, out_off, o, norm_w, proj, g1_off, g2_t, eps,
                         out_scale)
        return
    torch_ref.delta_out(o, norm_w, proj, g1_off, g2, eps, out, out_off,
                        out_scale)
