"""HIP kernels of layer-list decoders vs the plain fp32 torch reference of the
same op, in fp32 and bf16 activations, on sizes that are not powers of two."""

import pytest
import torch

from sutro_amd.ops import hybrid as hops
from sutro_amd.ops import torch_ref as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _tol(dtype):
    return (2e-5, 2e-5) if dtype == torch.float32 else (2e-2, 2e-2)


def _close(a, b, dtype, scale=1.0):
    rtol, atol = _tol(dtype)
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=rtol,
                               atol=atol * scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu_tanh_mul(dtype):
    g = torch.Generator().manual_seed(1)
    proj = (torch.randn(37, 200, generator=g) * 2).to(dtype)
    out = hops.gelu_tanh_mul(proj.to(DEV), 8, 104, 88)
    _close(out, ref.gelu_tanh_mul(proj, 8, 104, 88), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [72, 1000])
def test_gated_norm_residual_and_scalar_norm(dtype, W):
    g = torch.Generator().manual_seed(2)
    T = 19
    x = torch.randn(T, W, generator=g)
    y = torch.randn(T, W, generator=g).to(dtype)
    proj = torch.randn(T, W + 16, generator=g).to(dtype)
    gain = torch.tensor(1.3)
    xr = x.clone()
    hr = torch.empty(T, W, dtype=dtype)
    ref.gated_norm_residual(xr, y, proj, 16, gain, 2e-5, 0.75, hr)
    xd = x.to(DEV)
    hd = torch.empty(T, W, dtype=dtype, device=DEV)
    hops.gated_norm_residual(xd, y.to(DEV), proj.to(DEV), 16, gain.to(DEV),
                             2e-5, 0.75, hd)
    _close(xd, xr, torch.float32)
    _close(hd, hr, dtype)
    out = hops.scalar_rmsnorm(xd, gain.to(DEV), 2e-5, dtype)
    _close(out, ref.scalar_rmsnorm(xr, gain, 2e-5, dtype), dtype)


def _batch(lens_new, lens_total, page, n_blocks, seed):
    """Flat-batch metadata for sequences with `lens_new` new tokens each and
    `lens_total` tokens after this step; pages are handed out shuffled."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens_new)
    perm = torch.randperm(n_blocks - 1, generator=g) + 1
    per = (n_blocks - 1) // S          # every sequence draws from its own run
    per = max(per, 1)
    tables = []
    for s, L in enumerate(lens_total):
        nb = (L + page - 1) // page
        assert nb <= per
        tables.append(perm[s * per:s * per + nb].tolist())
    width = max(len(t) for t in tables)
    bt = torch.zeros(S, width, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    qlocs = torch.zeros(S + 1, dtype=torch.int32)
    pos, slots, tok_seq = [], [], []
    for s, (n, L) in enumerate(zip(lens_new, lens_total)):
        qlocs[s + 1] = qlocs[s] + n
        for p in range(L - n, L):
            pos.append(p)
            slots.append(tables[s][p // page] * page + p % page)
            tok_seq.append(s)
    return dict(bt=bt, qlocs=qlocs,
                seq_lens=torch.tensor(lens_total, dtype=torch.int32),
                pos=torch.tensor(pos, dtype=torch.long),
                slots=torch.tensor(slots, dtype=torch.long),
                token_seq=torch.tensor(tok_seq, dtype=torch.int32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dk,dv,rot,chunk,window", [
    (4, 1, 64, 32, 32, 16, 0),
    (6, 3, 40, 72, 24, 0, 9),
    (2, 2, 96, 136, 0, 20, 7),
    (8, 1, 128, 128, 128, 0, 0),
])
def test_attn_prep_and_local_attention(dtype, H, G, dk, dv, rot, chunk, window):
    page, n_blocks = 8, 41
    g = torch.Generator().manual_seed(3)
    # two steps: first fills the cache with a prompt piece, the second mixes a
    # continuing piece, a fresh prompt and single-token rows
    steps = [([13, 30, 1, 5], [13, 30, 1, 5]),
             ([9, 1, 1, 70], [22, 31, 2, 75])]
    ncol = _round8(H * dk) + 2 * _round8(G * max(dk, dv)) + 8
    q_off, k_off = 0, _round8(H * dk)
    v_off = k_off + _round8(G * dk)
    g_off = v_off + _round8(G * dv)
    ncol = g_off + 8 + H
    kc = torch.zeros(n_blocks, G, page, dk, dtype=dtype)
    vc = torch.zeros(n_blocks, G, page, dv, dtype=dtype)
    kc_d, vc_d = kc.to(DEV), vc.to(DEV)
    qw = 1 + 0.1 * torch.randn(dk, generator=g)
    kw = 1 + 0.1 * torch.randn(dk, generator=g)
    inv = ref.rope_inv_freq(rot, 10000.0)
    b0 = None
    for lens_new, lens_total in steps:
        if b0 is None:
            b0 = _batch(lens_new, lens_total, page, n_blocks, 5)
            b = b0
        else:
            # same page tables, grown
            b = _batch(lens_new, lens_total, page, n_blocks, 5)
        T = sum(lens_new)
        proj = torch.randn(T, ncol, generator=g).to(dtype)
        qr = ref.attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv, qw, kw,
                           2e-5, inv, b["pos"], b["slots"], kc, vc)
        qd = hops.attn_prep(proj.to(DEV), q_off, k_off, v_off, H, G, dk, dv,
                            qw.to(DEV), kw.to(DEV), 2e-5, inv.to(DEV),
                            b["pos"].to(DEV), b["slots"].to(DEV), kc_d, vc_d)
        _close(qd, qr, dtype, scale=2.0)
        _close(kc_d, kc, dtype, scale=2.0)
        _close(vc_d, vc, dtype)
        out_r = torch.zeros(T, H * dv + 8, dtype=dtype)
        ref.local_attention(qr, kc, vc, b["bt"], b["seq_lens"], b["qlocs"],
                            0.2, chunk, window, proj, g_off + 8, out_r, 8, 0.55)
        out_d = torch.zeros(T, H * dv + 8, dtype=dtype, device=DEV)
        # the device kernel reads the reference's cache and q, so only the
        # attention itself is compared
        hops.local_attention(qr.to(DEV), kc.to(DEV), vc.to(DEV),
                             b["bt"].to(DEV), b["seq_lens"].to(DEV),
                             b["qlocs"].to(DEV), 0.2, chunk, window,
                             proj.to(DEV), g_off + 8, out_d, 8, 0.55,
                             token_seq=b["token_seq"].to(DEV))
        _close(out_d, out_r, dtype)


def _round8(n):
    return (n + 7) // 8 * 8


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,dk,dv,taps,rank", [
    (4, 2, 64, 96, 3, 12),
    (3, 3, 32, 48, 4, 20),
    (6, 2, 48, 40, 2, 5),
    (2, 1, 160, 24, 5, 16),
    (1, 1, 256, 200, 1, 8),
])
def test_delta_rule_ops(dtype, H, G, dk, dv, taps, rank):
    g = torch.Generator().manual_seed(7)
    Cq, Cv = G * dk, H * dv
    C = 2 * Cq + Cv
    q_off, k_off = 8, 8 + _round8(Cq)
    v_off = k_off + _round8(Cq)
    b_off = v_off + _round8(Cv)
    a1_off = b_off + _round8(H)
    g1_off = a1_off + _round8(rank)
    ncol = g1_off + _round8(rank)
    conv_w = torch.randn(C, taps, generator=g) * 0.5
    a2 = torch.randn(H * dk, rank, generator=g) * 0.3
    g2 = torch.randn(H * dv, rank, generator=g) * 0.3
    dt_bias = torch.randn(H * dk, generator=g)
    a_log = torch.randn(H, generator=g) * 0.5
    norm_w = 1 + 0.1 * torch.randn(dv, generator=g)
    n_slots = 6
    conv_r = torch.randn(n_slots, max(1, taps - 1), C, generator=g)  # stale
    ssm_r = torch.randn(n_slots, H, dk, dv, generator=g)             # stale
    conv_d, ssm_d = conv_r.to(DEV), ssm_r.to(DEV)
    slots = torch.tensor([4, 1, 5, 2], dtype=torch.int32)
    # step 1 starts every sequence (stale slot contents must be ignored);
    # later steps continue with pieces of 1, 2 and many tokens
    steps = [([3, 1, 17, 2], [3, 1, 17, 2]),
             ([1, 2, 1, 40], [4, 3, 18, 42]),
             ([2, 1, 1, 1], [6, 4, 19, 43])]
    for lens_new, lens_total in steps:
        T = sum(lens_new)
        qlocs = torch.tensor([0] + list(torch.tensor(lens_new).cumsum(0)),
                             dtype=torch.int32)
        seq_lens = torch.tensor(lens_total, dtype=torch.int32)
        token_seq = torch.repeat_interleave(
            torch.arange(4, dtype=torch.int32), torch.tensor(lens_new))
        proj = torch.randn(T, ncol, generator=g).to(dtype)
        r = ref.delta_prep(proj, q_off, k_off, v_off, b_off, a1_off, H, G, dk,
                           dv, conv_w, a2, dt_bias, a_log, conv_r, slots,
                           qlocs, seq_lens)
        d = hops.delta_prep(proj.to(DEV), q_off, k_off, v_off, b_off, a1_off,
                            H, G, dk, dv, conv_w.to(DEV), a2.to(DEV),
                            dt_bias.to(DEV), a_log.to(DEV), conv_d,
                            slots.to(DEV), qlocs.to(DEV), seq_lens.to(DEV),
                            token_seq=token_seq.to(DEV))
        for a, b in zip(d, r):
            _close(a, b, torch.float32, scale=2.0)
        used = slots.long()
        _close(conv_d[used], conv_r[used], torch.float32)
        o_r = ref.delta_scan(*r, ssm_r, slots, qlocs, seq_lens)
        o_d = hops.delta_scan(*[t.to(DEV) for t in r], ssm_d, slots.to(DEV),
                              qlocs.to(DEV), seq_lens.to(DEV))
        _close(o_d, o_r, torch.float32, scale=2.0)
        _close(ssm_d[used], ssm_r[used], torch.float32, scale=2.0)
        out_r = torch.zeros(T, Cv + 16, dtype=dtype)
        out_d = torch.zeros(T, Cv + 16, dtype=dtype, device=DEV)
        ref.delta_out(o_r, norm_w, proj, g1_off, g2, 2e-5, out_r, 16, 0.45)
        hops.delta_out(o_r.to(DEV), norm_w.to(DEV), proj.to(DEV), g1_off,
                       g2.to(DEV), 2e-5, out_d, 16, 0.45)
        _close(out_d, out_r, dtype)


@pytest.mark.parametrize("H,G,dk,dv,chunk,window", [
    (4, 2, 64, 56, 48, 0),
    (8, 2, 128, 128, 100, 0),
    (6, 3, 40, 72, 0, 45),
    (2, 1, 256, 136, 37, 50),
    (16, 1, 64, 64, 0, 0),
])
def test_local_attention_matrix_core_path(H, G, dk, dv, chunk, window):
    """bf16, page 32: prompt pieces run on the MFMA kernel (tile map given),
    trailing single-token rows on the generic kernel; both against the fp32
    reference. Pieces start inside pages and inside chunks."""
    dtype = torch.bfloat16
    page, n_blocks = 32, 41
    g = torch.Generator().manual_seed(13)
    kc = torch.zeros(n_blocks, G, page, dk, dtype=dtype)
    vc = torch.zeros(n_blocks, G, page, dv, dtype=dtype)
    inv = ref.rope_inv_freq(0, 1.0)
    q_off, k_off = 0, H * dk
    v_off = k_off + G * dk
    g_off = v_off + _round8(G * dv)
    ncol = g_off + _round8(H)
    steps = [([150, 33, 5, 70], [150, 33, 5, 70], 4),
             ([61, 40, 1, 1], [211, 73, 6, 71], 2),
             ([95, 1, 1, 1], [306, 74, 7, 72], 1)]
    for lens_new, lens_total, n_prefill in steps:
        b = _batch(lens_new, lens_total, page, n_blocks, 5)
        T = sum(lens_new)
        proj = torch.randn(T, ncol, generator=g).to(dtype)
        qr = ref.attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv, None, None,
                           2e-5, inv, b["pos"], b["slots"], kc, vc)
        out_r = torch.zeros(T, H * dv, dtype=torch.float32)
        ref.local_attention(qr.float(), kc.float(), vc.float(), b["bt"],
                            b["seq_lens"], b["qlocs"], dk ** -0.5, chunk,
                            window, proj, g_off, out_r, 0, 0.55)
        tiles_s, tiles_q0 = [], []
        for s in range(n_prefill):
            for j in range(0, lens_new[s], 32):
                tiles_s.append(s)
                tiles_q0.append(j)
        out_d = torch.zeros(T, H * dv, dtype=dtype, device=DEV)
        hops.local_attention(
            qr.to(DEV), kc.to(DEV), vc.to(DEV), b["bt"].to(DEV),
            b["seq_lens"].to(DEV), b["qlocs"].to(DEV), dk ** -0.5, chunk,
            window, proj.to(DEV), g_off, out_d, 0, 0.55,
            token_seq=b["token_seq"].to(DEV),
            tile_seq=torch.tensor(tiles_s, dtype=torch.int32, device=DEV),
            tile_q0=torch.tensor(tiles_q0, dtype=torch.int32, device=DEV),
            prefill_rows=sum(lens_new[:n_prefill]))
        torch.testing.assert_close(out_d.float().cpu(), out_r, rtol=2e-2,
                                   atol=2e-2)
