"""Vodinex on the engine against the plain float64 oracle (hybrid_oracle.py).

Every test builds its own small configuration and random checkpoint, loads it
through the framework's config reader and weight loader, runs it through the
engine (scheduler, paged cache, state slots, decode graphs on the GPU) and
compares logits with the oracle run on whole sequences. The CPU cases run the
torch reference ops; the `gpu` cases run the HIP kernels in fp32 and bf16.
"""

import math

import pytest
import torch

import hybrid_oracle as O
from sutro_amd.engine.config import EngineConfig
from sutro_amd.engine.engine import LLMEngine
from sutro_amd.engine.request import SamplingParams
from sutro_amd.models.registry import spec_from_dir
from sutro_amd.ops import hybrid as hops

BACKENDS = [
    pytest.param(("cpu", torch.float32), id="cpu"),
    pytest.param(("cuda", torch.float32), id="gpu-fp32", marks=pytest.mark.gpu),
    pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu),
]


@pytest.fixture(params=BACKENDS)
def backend(request):
    return request.param


def limit(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def row_errors(got, want):
    """Per position: root mean square of the difference (mean over the
    vocabulary taken off), relative to the spread of the expected logits."""
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()


def rel_err(got, want):
    return float(row_errors(got, want).max())


# ------------------------------------------------------------- configs ------

def config_a():
    """Parallel layers with grouped heads on both sides, a rotation that
    covers half of each head, chunks that are not a multiple of the page,
    different key and value sizes everywhere."""
    left = O.attn_cfg(heads=4, kv_heads=2, dim=16, vdim=24, chunk=12,
                      rot_dims=8, base=1000.0, scale=0.31)
    right = O.delta_cfg(heads=4, kv_heads=2, dim=8, vdim=16, conv=2)
    left2 = O.attn_cfg(heads=2, kv_heads=1, dim=24, vdim=8, chunk=7,
                       rot_dims=24, base=50.0, scale=0.2)
    right2 = O.delta_cfg(heads=2, kv_heads=2, dim=16, vdim=8, conv=3)
    return O.make_config(48, 272, [
        O.parallel_layer(left, right, 0.8, 1.3, ff=40),
        O.delta_layer(O.delta_cfg(heads=3, kv_heads=1, dim=16, vdim=8, conv=4),
                      ff=56),
        O.parallel_layer(left2, right2, 1.1, 0.4),
    ], eps=1e-4, mult=0.6)


def config_b():
    """Delta-only layers first and last, one head, a one-tap filter, chunk 1
    (every token sees itself only) and a chunk longer than the sequence."""
    return O.make_config(40, 264, [
        O.delta_layer(O.delta_cfg(heads=1, kv_heads=1, dim=40, vdim=24, conv=1)),
        O.parallel_layer(
            O.attn_cfg(heads=1, kv_heads=1, dim=8, vdim=8, chunk=1, rot_dims=0,
                       base=10.0, scale=1.0),
            O.delta_cfg(heads=2, kv_heads=1, dim=8, vdim=8, conv=5),
            1.0, 1.0, ff=24),
        O.parallel_layer(
            O.attn_cfg(heads=3, kv_heads=3, dim=8, vdim=16, chunk=1000,
                       rot_dims=4, base=7.0, scale=0.5),
            O.delta_cfg(heads=2, kv_heads=2, dim=8, vdim=8, conv=2),
            0.5, 2.0),
        O.delta_layer(O.delta_cfg(heads=2, kv_heads=2, dim=8, vdim=12, conv=3),
                      ff=32),
    ], eps=1e-6, mult=1.0)


def config_c():
    """A vocabulary smaller than the byte alphabet, widths that are not
    multiples of 8 anywhere (merged projections and the merged output
    projection need padding), head sizes of 6 and 10."""
    return O.make_config(36, 50, [
        O.parallel_layer(
            O.attn_cfg(heads=3, kv_heads=1, dim=10, vdim=6, chunk=5,
                       rot_dims=6, base=30.0, scale=0.4),
            O.delta_cfg(heads=3, kv_heads=3, dim=6, vdim=10, conv=3),
            0.9, 0.65, ff=20),
        O.delta_layer(O.delta_cfg(heads=2, kv_heads=1, dim=10, vdim=6, conv=2)),
    ], eps=2e-5, mult=0.8)


_CACHE = {}


def checkpoint(tmp_path_factory, name, cfg_fn, seed=0, tweak=None):
    key = (name, seed)
    if key not in _CACHE:
        cfg = cfg_fn()
        w = O.make_weights(cfg, seed=seed)
        if tweak:
            tweak(w)
        path = O.save_checkpoint(str(tmp_path_factory.mktemp(name)), cfg, w)
        _CACHE[key] = (path, cfg, w, {})
    return _CACHE[key]


def oracle_logits(ck, tokens):
    path, cfg, w, memo = ck
    key = tuple(tokens)
    if key not in memo:
        memo[key] = O.forward(cfg, w, list(tokens))
    return memo[key]


def engine(ck, backend, page=8, blocks=64, max_seqs=4, budget=4096, **kw):
    device, dtype = backend
    spec = spec_from_dir(ck[0])
    cfg = EngineConfig(spec=spec, device=device, dtype=dtype,
                       kv_block_size=page, max_model_len=page * (blocks - 1),
                       max_num_seqs=max_seqs, num_kv_blocks=blocks,
                       max_tokens_per_step=budget, **kw)
    return LLMEngine(cfg)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(3, cfg["vocab"], (n,), generator=g).tolist()


def replay(eng, seqs, schedule):
    """Run `schedule` (a list of steps, each a list of (name, count)) and
    return name -> logits of every position [len, vocab]."""
    live, at, out = {}, {k: 0 for k in seqs}, {k: [] for k in seqs}
    for step in schedule:
        entries = []
        for name, n in step:
            if name not in live:
                live[name] = eng.new_replay_request()
            lo = at[name]
            entries.append((live[name], seqs[name][lo:lo + n], list(range(n))))
            at[name] = lo + n
        logits = eng.replay_step(entries)
        k = 0
        for name, n in step:
            out[name].append(logits[k:k + n])
            k += n
        for name, _ in step:
            if at[name] == len(seqs[name]) and name in live:
                eng.finish_replay_request(live.pop(name))
    return {k: torch.cat(v) for k, v in out.items() if v}


def check(ck, got, seqs, dtype, names=None):
    """fp32: every position within the limit. bf16: rounding alone moves
    single positions of these tiny models by more than a real model's (the
    same figure comes out of the reference ops run in bf16 on the CPU), so
    the limit holds for the mean over positions and five times it for the
    worst one; faults of masks, pages or state show in the fp32 runs of the
    same kernels."""
    for name in names or got:
        want = oracle_logits(ck, seqs[name])
        assert got[name].shape == want.shape
        rows = row_errors(got[name], want)
        if dtype == torch.float32:
            assert float(rows.max()) < limit(dtype), \
                f"{name}: relative error {float(rows.max())}"
        else:
            assert float(rows.mean()) < limit(dtype), \
                f"{name}: mean relative error {float(rows.mean())}"
            assert float(rows.max()) < 5 * limit(dtype), \
                f"{name}: worst relative error {float(rows.max())}"


# ------------------------------------------------ whole prompts, decoding ---

@pytest.mark.parametrize("cfg_fn", [config_a, config_b, config_c])
def test_whole_prompt(tmp_path_factory, backend, cfg_fn):
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend)
    seqs = {"s": tokens_for(ck[1], 45, 1)}
    got = replay(eng, seqs, [[("s", 45)]])
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("cfg_fn", [config_a, config_b])
def test_first_tokens(tmp_path_factory, backend, cfg_fn):
    """Sequences of one, two and three tokens (filters longer than the
    sequence, first chunk, empty memory), alone and decoded one by one."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend)
    seqs = {f"n{n}": tokens_for(ck[1], n, 10 + n) for n in (1, 2, 3)}
    got = replay(eng, seqs, [[("n1", 1)], [("n2", 2)], [("n3", 3)]])
    check(ck, got, seqs, backend[1])
    got = replay(eng, seqs, [[("n3", 1), ("n2", 1)], [("n3", 1), ("n2", 1)],
                             [("n3", 1)]])
    check(ck, got, seqs, backend[1], names=["n2", "n3"])


@pytest.mark.parametrize("cfg_fn", [config_a, config_b, config_c])
def test_prefill_then_token_by_token(tmp_path_factory, backend, cfg_fn):
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend)
    seqs = {"s": tokens_for(ck[1], 45, 1)}
    got = replay(eng, seqs, [[("s", 9)]] + [[("s", 1)]] * 36)
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("page", [8, 32])
def test_portions_of_many_sizes(tmp_path_factory, backend, page):
    """Prompt pieces of 2, 3, 1, 11, 2, 5 ... tokens: cuts inside pages,
    inside chunks and inside the filters' reach. With pages of 32 the bf16
    prompt pieces take the matrix-core attention kernel."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"s": tokens_for(ck[1], 62, 2)}
    sizes = [2, 3, 1, 11, 2, 5, 1, 1, 13, 2, 8, 7, 2, 4]
    assert sum(sizes) == 62
    got = replay(eng, seqs, [[("s", n)] for n in sizes])
    check(ck, got, seqs, backend[1])


def test_long_decoding(tmp_path_factory, backend):
    """A short prompt and 100 decoded tokens: many chunk edges and page
    borders pass under single-token steps."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend)
    seqs = {"s": tokens_for(ck[1], 104, 3)}
    got = replay(eng, seqs, [[("s", 4)]] + [[("s", 1)]] * 100)
    check(ck, got, seqs, backend[1])


# ----------------------------------------------------- batches, reuse -------

@pytest.mark.parametrize("page", [8, 32])
def test_mixed_batch_equals_each_alone(tmp_path_factory, backend, page):
    """Unequal requests in one batch (prompt pieces beside single tokens,
    requests that sit out a step) give what each gives alone."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"a": tokens_for(ck[1], 40, 4), "b": tokens_for(ck[1], 17, 5),
            "c": tokens_for(ck[1], 9, 6), "d": tokens_for(ck[1], 26, 7)}
    schedule = [
        [("a", 13), ("b", 1)],
        [("a", 1), ("b", 1), ("c", 2)],
        [("b", 6), ("c", 1), ("d", 20), ("a", 1)],
        [("a", 20), ("c", 1), ("d", 1)],
        [("b", 9), ("d", 1), ("c", 5), ("a", 5)],
        [("d", 4)],
    ]
    got = replay(eng, seqs, schedule)
    check(ck, got, seqs, backend[1])
    alone = replay(engine(ck, backend), seqs, [[(k, len(v))] for k, v in seqs.items()])
    for k in seqs:
        e = rel_err(got[k], alone[k].double().cpu())
        assert e < (limit(backend[1]) if backend[1] == torch.float32 else 0.3)


def test_pages_and_state_slots_are_reused(tmp_path_factory, backend):
    """Two sequence slots and a pool of six pages serve eight requests one
    after another; a freed slot's memory and filter history and a freed
    page's keys must not leak into the next request."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend, page=8, blocks=7, max_seqs=2)
    seqs = {f"r{i}": tokens_for(ck[1], 9 + 3 * (i % 4), 20 + i) for i in range(8)}
    names = list(seqs)
    schedule = []
    for i in range(0, 8, 2):
        a, b = names[i], names[i + 1]
        la, lb = len(seqs[a]), len(seqs[b])
        schedule += [[(a, 5), (b, 2)], [(a, la - 5), (b, 1)], [(b, lb - 3)]]
    got = replay(eng, seqs, schedule)
    check(ck, got, seqs, backend[1])
    assert eng.kv.allocator.num_free == 6
    assert eng.kv.state.num_free == 2
    with pytest.raises(MemoryError):
        replay(eng, {"x": [3] * 8, "y": [4] * 8, "z": [5] * 8},
               [[("x", 2), ("y", 2), ("z", 2)]])


# ------------------------------------- far memory, edges made to stand out --

def _long_memory(w):
    """Decays close to one: the delta-rule memory keeps tokens from hundreds
    of steps back, so a lost or stale state changes late logits."""
    for k in list(w):
        if k.endswith(".A_log"):
            w[k] = torch.full_like(w[k], -9.0)


def test_far_memory_survives_portions_and_decoding(tmp_path_factory, backend):
    ck = checkpoint(tmp_path_factory, "config_b_long", config_b, seed=3,
                    tweak=_long_memory)
    toks = tokens_for(ck[1], 150, 8)
    # the oracle itself must depend on the first tokens at the end
    other = [5 if t != 5 else 6 for t in toks[:3]] + toks[3:]
    far = rel_err(oracle_logits(ck, other)[-5:].float(),
                  oracle_logits(ck, toks)[-5:])
    assert far > 0.5, far
    eng = engine(ck, backend)
    seqs = {"s": toks}
    sizes = [7, 2, 50, 1, 1, 31, 2, 2] + [1] * 54
    got = replay(eng, seqs, [[("s", n)] for n in sizes])
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("mode", ["prompt", "decoded"])
@pytest.mark.parametrize("page", [4, 8])
def test_chunk_edges_stand_out(backend, mode, page):
    """One key gets a score far above all others; it lies just inside or just
    outside the querying token's chunk, at and next to page borders. The
    output must be that key's value when it is visible and must not contain
    it when it is not."""
    device, dtype = backend
    H, G, dk, dv, chunk = 2, 1, 16, 8, 6
    T = 40
    g = torch.Generator().manual_seed(11)
    k = torch.randn(T, G, dk, generator=g) * 0.1
    v = torch.randn(T, G, dv, generator=g)
    q = torch.randn(T, H, dk, generator=g) * 0.1
    cases = []          # (query position, key position)
    for i in range(6, T):
        lo = (i // chunk) * chunk
        cases += [(i, lo), (i, lo - 1)]
    probes = []
    for n, (i, j) in enumerate(cases[::5]):
        probe = torch.zeros(dk)
        probe[n % dk] = 6.0
        k[j, 0] += probe
        q[i, n % H] += probe * 3
        probes.append((i, j, n % H))
    if dtype != torch.float32:      # the oracle sees what the kernels see
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
    want = torch.stack([
        torch.stack([O.masked_softmax_attention(q[:, h].double(), k[:, 0].double(),
                                                v[:, 0].double(), 1.0, chunk)
                     for h in range(H)], 1)])[0]          # [T, H, dv]
    # the framework's path: pages handed out in a scrambled order
    n_blocks = T // page + 3
    order = torch.randperm(n_blocks - 1, generator=g) + 1
    table = order[: (T + page - 1) // page].to(torch.int32)
    kc = torch.zeros(n_blocks, G, page, dk, dtype=dtype, device=device)
    vc = torch.zeros(n_blocks, G, page, dv, dtype=dtype, device=device)
    ncol = H * dk + G * dk + G * dv
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1)
    proj = proj.to(dtype).to(device)
    inv = torch.zeros(0, dtype=torch.float32, device=device)
    pieces = [T] if mode == "prompt" else [5] + [1] * (T - 5)
    got, done = [], 0
    for n in pieces:
        pos = torch.arange(done, done + n)
        slots = (table[pos // page].long() * page + pos % page)
        rows = proj[done:done + n]
        qq = hops.attn_prep(rows, 0, H * dk, H * dk + G * dk, H, G, dk, dv, None,
                            None, 1e-4, inv, pos.to(device), slots.to(device),
                            kc, vc)
        out = torch.zeros(n, H * dv, dtype=dtype, device=device)
        done += n
        hops.local_attention(
            qq, kc, vc, table[None].to(device),
            torch.tensor([done], dtype=torch.int32, device=device),
            torch.tensor([0, n], dtype=torch.int32, device=device), 1.0, chunk,
            0, rows, -1, out, 0, 1.0,
            token_seq=torch.zeros(n, dtype=torch.int32, device=device))
        got.append(out.float().cpu())
    got = torch.cat(got).view(T, H, dv)
    tol = 1e-4 if dtype == torch.float32 else 5e-2
    assert float((got.double() - want).abs().max()) < tol
    # the probes do what they are for: a visible probed key takes all the
    # weight, a hidden one none of it
    inside = [(i, j, h) for i, j, h in probes if j >= (i // chunk) * chunk]
    outside = [(i, j, h) for i, j, h in probes if j < (i // chunk) * chunk]
    assert inside and outside
    for i, j, h in inside:
        assert float((want[i, h] - v[j, 0].double()).abs().max()) < 1e-3
    for i, j, h in outside:
        assert float((want[i, h] - v[j, 0].double()).abs().max()) > 0.1


def test_delta_heads_share_keys_by_group(backend):
    """heads > kv_heads in the delta rule: value head h reads q/k head
    h // (heads / kv_heads). Distinct per-group keys make a wrong pairing
    show."""
    device, dtype = backend
    H, G, dk, dv, T = 6, 2, 8, 4, 9
    g = torch.Generator().manual_seed(5)
    qn = O.unit_vectors(torch.randn(T, G, dk, generator=g).double())
    kn = O.unit_vectors(torch.randn(T, G, dk, generator=g).double())
    v = torch.randn(T, H, dv, generator=g).double()
    decay = torch.rand(T, H, dk, generator=g).double() * 0.5 + 0.5
    beta = torch.rand(T, H, generator=g).double()
    want = torch.stack([O.delta_rule(qn[:, h // 3], kn[:, h // 3], v[:, h],
                                     beta[:, h], decay[:, h])[0]
                        for h in range(H)], 1)
    ssm = torch.randn(3, H, dk, dv).to(device)           # stale slot contents
    f = lambda t: t.float().contiguous().to(device)
    slots = torch.tensor([2], dtype=torch.int32, device=device)
    got, done = [], 0
    for n in (4, 1, 1, 3):
        sl = slice(done, done + n)
        done += n
        got.append(hops.delta_scan(
            f(qn[sl]), f(kn[sl]), f(v[sl]), f(decay[sl]), f(beta[sl]), ssm,
            slots, torch.tensor([0, n], dtype=torch.int32, device=device),
            torch.tensor([done], dtype=torch.int32, device=device)).cpu())
    assert float((torch.cat(got).double() - want).abs().max()) < 1e-4


def test_filter_history_across_short_pieces(backend):
    """A five-tap filter fed in pieces of 1, 2 and 3 tokens: the history that
    a piece needs may come from several earlier pieces."""
    device, dtype = backend
    H, G, dk, dv, taps, rank, T = 2, 1, 8, 8, 5, 3, 12
    g = torch.Generator().manual_seed(6)
    C = 2 * G * dk + H * dv
    ncol = C + 8 + 8 + 8
    proj = torch.randn(T, ncol, generator=g).to(dtype)
    conv_w = torch.randn(C, taps, generator=g).to(torch.bfloat16).float()
    a2 = torch.randn(H * dk, rank, generator=g)
    dtb = torch.randn(H * dk, generator=g)
    a_log = torch.randn(H, generator=g) * 0.3
    raw = proj[:, :C].double()
    y = O.short_filter_silu(raw, conv_w.double())
    want_q = O.unit_vectors(y[:, :dk].view(T, G, dk)) * dk ** -0.5
    want_k = O.unit_vectors(y[:, dk:2 * dk].view(T, G, dk))
    want_v = y[:, 2 * dk:].view(T, H, dv)
    pre = (proj[:, C + 8:C + 8 + rank].double() @ a2.double().T + dtb.double())
    want_decay = torch.stack([O.channel_decay(a_log[h], pre.view(T, H, dk)[:, h])
                              for h in range(H)], 1)
    want_beta = torch.sigmoid(proj[:, C:C + H].double())
    conv_state = torch.randn(2, taps - 1, C).to(device)   # stale
    slots = torch.tensor([1], dtype=torch.int32, device=device)
    outs, done = [], 0
    for n in (1, 2, 1, 3, 1, 1, 2, 1):
        rows = proj[done:done + n].to(device)
        done += n
        outs.append([t.cpu() for t in hops.delta_prep(
            rows, 0, G * dk, 2 * G * dk, C, C + 8, H, G, dk, dv,
            conv_w.to(device), a2.to(device), dtb.to(device), a_log.to(device),
            conv_state, slots,
            torch.tensor([0, n], dtype=torch.int32, device=device),
            torch.tensor([done], dtype=torch.int32, device=device),
            token_seq=torch.zeros(n, dtype=torch.int32, device=device))])
    got = [torch.cat([o[i] for o in outs]).double() for i in range(5)]
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    for a, b in zip(got, (want_q, want_k, want_v, want_decay, want_beta)):
        assert float((a - b).abs().max()) < tol


def test_rotation_of_a_prefix_and_head_norms(backend):
    """Only the first rot_dims dimensions rotate (pairing i with i +
    rot_dims/2); the rest pass through; q and k are normalised per head with a
    shared weight before the rotation."""
    device, dtype = backend
    H, G, dk, dv, rot, T = 3, 1, 12, 4, 6, 7
    g = torch.Generator().manual_seed(9)
    proj = torch.randn(T, H * dk + G * dk + G * dv, generator=g).to(dtype)
    qw = (1 + 0.2 * torch.randn(dk, generator=g)).to(torch.bfloat16).float()
    kw = (1 + 0.2 * torch.randn(dk, generator=g)).to(torch.bfloat16).float()
    pos = torch.tensor([0, 1, 2, 40, 41, 1000, 5])
    q = O.rms_unit(proj[:, :H * dk].double().view(T, H, dk), 1e-3) * qw.double()
    want = O.rotate_prefix(q, pos, rot, 100.0)
    kc = torch.zeros(2, G, 8, dk, dtype=dtype, device=device)
    vc = torch.zeros(2, G, 8, dv, dtype=dtype, device=device)
    got = hops.attn_prep(proj.to(device), 0, H * dk, H * dk + G * dk, H, G, dk,
                         dv, qw.to(device), kw.to(device), 1e-3,
                         hops.rope_inv_freq(rot, 100.0).to(device),
                         pos.to(device), torch.arange(8, 8 + T).to(device), kc,
                         vc)
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert float((got.double().cpu() - want).abs().max()) < tol
    k = O.rms_unit(proj[:, H * dk:H * dk + dk].double().view(T, G, dk), 1e-3) * kw.double()
    want_k = O.rotate_prefix(k, pos, rot, 100.0)
    assert float((kc[1, :, :T].double().cpu().transpose(0, 1) - want_k).abs().max()) < tol


def test_gated_residual_norm_and_feed_forward(backend):
    device, dtype = backend
    T, W, ff = 5, 24, 16
    g = torch.Generator().manual_seed(4)
    x = torch.randn(T, W, generator=g)
    proj = torch.randn(T, 2 * ff + W, generator=g).to(dtype)
    y = torch.randn(T, W, generator=g).to(dtype)
    gain = torch.tensor(0.8)
    z = y.double() * torch.sigmoid(proj[:, 2 * ff:].double())
    want = x.double() + 0.6 * O.rms_unit(z, 1e-4) * 0.8
    xd = x.clone().to(device)
    hops.gated_norm_residual(xd, y.to(device), proj.to(device), 2 * ff,
                             gain.to(device), 1e-4, 0.6, None)
    assert float((xd.double().cpu() - want).abs().max()) < 1e-4
    act = hops.gelu_tanh_mul(proj.to(device), 0, ff, ff)
    want_act = O.gelu_tanh(proj[:, :ff].double()) * proj[:, ff:2 * ff].double()
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert float((act.double().cpu() - want_act).abs().max()) < tol


# ------------------------------------------ generation through the engine ---

def test_greedy_generation_through_scheduler(tmp_path_factory, backend):
    """Requests go through add_request / step(): the scheduler cuts prompts by
    its own token budget, batches prefill with decode and samples greedily.
    Every generated token must be the oracle's argmax given the same prefix
    (ties within rounding excepted)."""
    device, dtype = backend
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend, budget=16, blocks=40)
    prompts = [tokens_for(ck[1], n, 30 + n) for n in (21, 5, 34, 2, 13)]
    reqs = [eng.add_request(p, SamplingParams(max_tokens=12, temperature=0.0))
            for p in prompts]
    steps = 0
    while eng.has_work():
        eng.step()
        steps += 1
        assert steps < 400
    checked = 0
    for p, r in zip(prompts, reqs):
        assert r.finished and len(r.output_token_ids) >= 1
        seq = p + r.output_token_ids
        logits = oracle_logits(ck, seq[:-1])
        for n, tok in enumerate(r.output_token_ids):
            row = logits[len(p) - 1 + n, :eng.tokenizer.vocab_size]
            best = int(row.argmax())
            margin = float(row[best] - row[tok])
            assert tok == best or margin < 20 * limit(dtype), (n, tok, best)
            checked += 1
    assert checked >= 20


def test_cli_generates_from_a_checkpoint_directory(tmp_path_factory):
    """`sutro generate --model DIR`: the registry resolves the directory by
    its config.json, the loader fills the model, the engine samples."""
    import json

    from click.testing import CliRunner

    from sutro_amd.cli import cli

    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    res = CliRunner().invoke(cli, ["generate", "--model", ck[0], "--prompt",
                                   "hello there", "--prompt", "two",
                                   "--max-tokens", "5", "--temperature", "0",
                                   "--device", "cpu", "--max-model-len", "256"])
    assert res.exit_code == 0, res.output
    lines = [json.loads(x) for x in res.output.strip().splitlines()]
    assert [x["prompt"] for x in lines] == ["hello there", "two"]


def test_registry_resolves_architectures_by_config(tmp_path, tmp_path_factory):
    import json

    from sutro_amd.models.hybrid_spec import HybridSpec
    from sutro_amd.models.registry import (ModelSpec, get_model_spec,
                                           register_model_dir)

    ck = checkpoint(tmp_path_factory, "config_b", config_b)
    spec = get_model_spec(ck[0])
    assert isinstance(spec, HybridSpec) and spec.arch == "vodinex"
    assert spec.num_layers == 4 and spec.layers[0].mixer.conv == 1
    assert spec.layers[1].mixer.right.decay_rank == 6      # from tensor shapes
    assert register_model_dir("my-vodinex", ck[0]).name == "my-vodinex"
    assert get_model_spec("my-vodinex").checkpoint_dir == ck[0]
    (tmp_path / "config.json").write_text(json.dumps({
        "architectures": ["Qwen3ForCausalLM"], "hidden_size": 64,
        "num_hidden_layers": 2, "num_attention_heads": 4,
        "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 128,
        "vocab_size": 512}))
    q = get_model_spec(str(tmp_path))
    assert isinstance(q, ModelSpec) and q.num_kv_heads == 2
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Nope"}))
    with pytest.raises(KeyError):
        get_model_spec(str(tmp_path))


def test_service_job_on_a_checkpoint_directory(tmp_path_factory, local_client):
    """A checkpoint directory is a model name for the job service too."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    job = local_client.infer(["alpha", "beta gamma"], model=ck[0],
                             sampling_params={"max_tokens": 4, "temperature": 0},
                             stay_attached=False)
    out = local_client.await_job_completion(job, timeout=120)
    assert out is not None and len(out) == 2
