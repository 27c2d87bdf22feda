"""Ruludra on the engine against the plain float64 oracle (ruludra_oracle.py).

Every test builds its own small configuration and random checkpoint, loads it
through the framework's config reader and weight loader, runs it through the
engine (scheduler, paged cache, state slots, decode graphs on the GPU) and
compares logits with the oracle run on whole sequences. The CPU cases run the
torch reference ops; the `gpu` cases run the HIP kernels in fp32 and bf16.
"""

import json

import pytest
import torch

import ruludra_oracle as O
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
    """All three mixers in an order of their own (recurrent layer first), two
    latent layers reading one cached latent, grouped key heads, value sizes
    unlike key sizes, a different window in every layer (one longer than any
    test sequence), layers with and without feed-forward for every mixer."""
    return O.make_config(48, 272, [
        O.layer("mlstm", O.mlstm_cfg(2, 8, 12, cap=6.0)),
        O.layer("latent_attention", O.latent_cfg(3, 8, 16, 24, 16, 9, 0.3), ff=40),
        O.layer("attention", O.attn_cfg(4, 2, 16, 11, 0.21, coef=0.4, every=5), ff=56),
        O.layer("latent_attention", O.latent_cfg(2, 16, 8, 16, 16, 5, 0.2, kv_from=1)),
        O.layer("attention", O.attn_cfg(2, 1, 24, 1000, 0.15, coef=0.1, every=3)),
        O.layer("mlstm", O.mlstm_cfg(3, 16, 8, cap=15.0), ff=32),
        O.layer("latent_attention", O.latent_cfg(1, 8, 8, 8, 16, 13, 0.4, kv_from=1), ff=24),
    ], eps=1e-5, logit_scale=0.5)


def config_b():
    """A vocabulary smaller than the byte alphabet and fewer bigram buckets
    than tokens, sizes that are multiples of 8 nowhere (merged projections
    need padding), one head, a window of one (a token sees only itself) and
    of two, a temperature that steps at every token."""
    return O.make_config(36, 50, [
        O.layer("attention", O.attn_cfg(3, 3, 10, 2, 0.4, coef=0.7, every=1), ff=20),
        O.layer("mlstm", O.mlstm_cfg(1, 10, 6, cap=3.0), ff=28),
        O.layer("latent_attention", O.latent_cfg(1, 6, 10, 12, 20, 1, 0.5)),
        O.layer("latent_attention", O.latent_cfg(3, 10, 6, 6, 12, 7, 0.3), ff=12),
        O.layer("attention", O.attn_cfg(1, 1, 12, 6, 0.3, coef=0.0, every=4)),
    ], eps=2e-4, logit_scale=1.7, buckets=11, mul_prev=5, mul_cur=3)


def config_c():
    """Sizes the matrix-core attention kernel takes (pages of 32, head and
    latent sizes that are multiples of 8), windows longer than a page and
    not a multiple of it."""
    return O.make_config(64, 300, [
        O.layer("attention", O.attn_cfg(4, 2, 32, 40, 0.18, coef=0.35, every=16), ff=96),
        O.layer("latent_attention", O.latent_cfg(4, 16, 24, 32, 32, 33, 0.25), ff=64),
        O.layer("mlstm", O.mlstm_cfg(2, 32, 40, cap=10.0)),
        O.layer("latent_attention", O.latent_cfg(2, 32, 16, 16, 32, 70, 0.2, kv_from=1)),
        O.layer("attention", O.attn_cfg(2, 2, 64, 35, 0.12, coef=0.2, every=7), ff=48),
    ], eps=1e-6, logit_scale=0.3, buckets=509, mul_prev=29, mul_cur=3)


_CACHE = {}


def checkpoint(tmp_path_factory, name, cfg_fn, seed=0, tweak=None):
    key = (name, seed)
    if key not in _CACHE:
        cfg = cfg_fn()
        w = O.make_weights(cfg, seed=seed)
        if tweak:
            tweak(w)
            w = {k: v.to(torch.bfloat16).to(O.F64) for k, v in w.items()}
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
    single positions of these tiny models by more than a real model's, so
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
    page = 32 if cfg_fn is config_c else 8
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"s": tokens_for(ck[1], 90 if cfg_fn is config_c else 45, 1)}
    got = replay(eng, seqs, [[("s", len(seqs["s"]))]])
    check(ck, got, seqs, backend[1])


def test_layer_streams_match(tmp_path_factory, backend):
    """The fp32 stream that leaves every layer (after the depth-weighted sum)
    against the oracle's: a fault shows in the layer that makes it."""
    device, dtype = backend
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend)
    toks = tokens_for(ck[1], 23, 9)
    want = []
    O.forward(ck[1], ck[2], toks, streams=want)
    eng.model.layer_taps = []
    replay(eng, {"s": toks}, [[("s", 23)]])
    taps = eng.model.layer_taps
    eng.model.layer_taps = None
    assert len(taps) == len(want)
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    for i, (g, e) in enumerate(zip(taps, want)):
        err = float((g.double().cpu() - e).abs().max() / e.abs().max())
        assert err < tol, f"layer {i}: {err}"


@pytest.mark.parametrize("cfg_fn", [config_a, config_b])
def test_first_tokens(tmp_path_factory, backend, cfg_fn):
    """Sequences of one, two and three tokens (the bigram's extra row, an
    empty memory with its stabiliser at 0, windows longer than the
    sequence), alone and decoded one by one."""
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
    eng = engine(ck, backend, page=32 if cfg_fn is config_c else 8, blocks=24)
    seqs = {"s": tokens_for(ck[1], 45, 1)}
    got = replay(eng, seqs, [[("s", 9)]] + [[("s", 1)]] * 36)
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("cfg_fn,page", [(config_a, 8), (config_a, 32),
                                         (config_c, 32)])
def test_portions_of_many_sizes(tmp_path_factory, backend, cfg_fn, page):
    """Prompt pieces of 2, 3, 1, 11, 2, 5 ... tokens: cuts inside pages and
    inside windows, the previous token of a piece's first token comes from
    the piece before. With pages of 32 the bf16 prompt pieces take the
    matrix-core attention kernel."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
    eng = engine(ck, backend, page=page, blocks=24)
    seqs = {"s": tokens_for(ck[1], 62, 2)}
    sizes = [2, 3, 1, 11, 2, 5, 1, 1, 13, 2, 8, 7, 2, 4]
    assert sum(sizes) == 62
    got = replay(eng, seqs, [[("s", n)] for n in sizes])
    check(ck, got, seqs, backend[1])


def test_long_decoding(tmp_path_factory, backend):
    """A short prompt and 120 decoded tokens: every window passes over
    decoded tokens, many page borders pass under single-token steps, the
    temperature steps several times."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    eng = engine(ck, backend)
    seqs = {"s": tokens_for(ck[1], 124, 3)}
    got = replay(eng, seqs, [[("s", 4)]] + [[("s", 1)]] * 120)
    check(ck, got, seqs, backend[1])


# ------------------------------------------------ random configurations -----

def random_config(seed):
    """Widths, head counts, head and latent sizes, windows, temperature
    steps, gate caps, hash constants, the order of layers and which of them
    have a feed-forward or borrow a latent: all drawn at random."""
    import random

    rnd = random.Random(seed)
    layers, owners = [], []
    for i in range(rnd.randint(3, 7)):
        kind = rnd.choice(["attention", "latent_attention", "mlstm"])
        ff = rnd.choice([None, 40, 72, 136])
        win = rnd.choice([3, 16, 33, 50, 64])
        if kind == "attention":
            G = rnd.choice([1, 2, 4])
            dim = rnd.choice([16, 24, 32, 40, 20])
            m = O.attn_cfg(G * rnd.choice([1, 2, 3]), G, dim, win,
                           dim ** -0.5 * rnd.choice([1.0, 0.7]),
                           coef=rnd.choice([0.0, 0.2, 0.5]),
                           every=rnd.choice([1, 7, 32]))
        elif kind == "latent_attention":
            dim = rnd.choice([16, 32, 24])
            kr = rnd.choice([16, 32, 40, 72])
            cands = [j for j in owners if layers[j]["mixer"]["kv_rank"] == kr]
            src = rnd.choice(cands) if cands and rnd.random() < 0.6 else None
            m = O.latent_cfg(rnd.choice([1, 2, 3, 6, 12]), dim,
                             rnd.choice([16, 48, 36]), rnd.choice([24, 40, 64]),
                             kr, win, dim ** -0.5, kv_from=src)
            if src is None:
                owners.append(i)
        else:
            m = O.mlstm_cfg(rnd.choice([1, 2, 5]), rnd.choice([16, 48, 24]),
                            rnd.choice([16, 64, 40]),
                            cap=rnd.choice([5.0, 12.0, 30.0]))
        layers.append(O.layer(kind, m, ff=ff))
    return O.make_config(rnd.choice([64, 96, 136]), rnd.choice([300, 512, 777]),
                         layers, eps=rnd.choice([1e-6, 1e-5]),
                         logit_scale=rnd.choice([0.2, 1.0, 2.0]),
                         buckets=rnd.choice([97, 613, 4093]),
                         mul_prev=rnd.choice([37, 7, 101]),
                         mul_cur=rnd.choice([19, 3, 29]))


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_configurations(tmp_path_factory, backend, seed):
    """A drawn configuration through a mixed schedule (portions beside single
    tokens, pages of 32, a pool smaller than the sum of the requests)."""
    ck = checkpoint(tmp_path_factory, f"random{seed}",
                    lambda: random_config(seed), seed=seed)
    eng = engine(ck, backend, page=32, blocks=8, max_seqs=3)
    seqs = {"a": tokens_for(ck[1], 90, seed), "b": tokens_for(ck[1], 31, seed + 1),
            "c": tokens_for(ck[1], 47, seed + 2)}
    schedule = [[("a", 40), ("b", 3)], [("a", 1), ("b", 20), ("c", 2)],
                [("a", 30), ("b", 1), ("c", 1)], [("a", 2), ("b", 1), ("c", 40)],
                [("a", 1), ("b", 1), ("c", 1)], [("a", 1), ("b", 1), ("c", 1)],
                [("a", 15), ("b", 4), ("c", 2)]]
    got = replay(eng, seqs, schedule)
    for k in seqs:
        rows = row_errors(got[k], oracle_logits(ck, seqs[k]))
        if backend[1] == torch.float32:
            assert float(rows.max()) < limit(backend[1]), (k, float(rows.max()))
        else:   # single positions of a drawn model can be ill-conditioned
            assert float(rows.mean()) < 3e-2, (k, float(rows.mean()))


# ----------------------------------------------------- batches, reuse -------

@pytest.mark.parametrize("cfg_fn,page", [(config_a, 8), (config_c, 32)])
def test_mixed_batch_equals_each_alone(tmp_path_factory, backend, cfg_fn, page):
    """Unequal requests in one batch (prompt pieces beside single tokens,
    requests that sit out a step) give what each gives alone."""
    ck = checkpoint(tmp_path_factory, cfg_fn.__name__, cfg_fn)
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
    alone = replay(engine(ck, backend, page=page, blocks=24), seqs,
                   [[(k, len(v))] for k, v in seqs.items()])
    for k in seqs:
        e = rel_err(got[k], alone[k].double().cpu())
        assert e < (limit(backend[1]) if backend[1] == torch.float32 else 0.3)


def test_pages_and_state_slots_are_reused(tmp_path_factory, backend):
    """Two sequence slots and a pool of six pages serve eight requests one
    after another; a freed slot's memory, normaliser and stabiliser and a
    freed page's keys and latents must not leak into the next request."""
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
    """Forget gates pinned near one and weak input gates: the matrix memory
    keeps the first tokens for hundreds of steps, so a lost or stale state
    changes late logits."""
    for k in list(w):
        if k.endswith(".f.b"):
            w[k] = torch.full_like(w[k], 9.0)
        if k.endswith(".mix.f") or k.endswith(".mix.i"):
            w[k] = w[k] * 0.05


def _mlstm_only():
    return O.make_config(40, 264, [
        O.layer("mlstm", O.mlstm_cfg(2, 16, 8, cap=12.0), ff=24),
        O.layer("mlstm", O.mlstm_cfg(1, 8, 24, cap=12.0)),
    ], eps=1e-6, logit_scale=1.0)


def test_far_memory_survives_portions_and_decoding(tmp_path_factory, backend):
    ck = checkpoint(tmp_path_factory, "mlstm_long", _mlstm_only, seed=3,
                    tweak=_long_memory)
    toks = tokens_for(ck[1], 150, 8)
    # the oracle itself must depend on the first tokens at the end
    other = [5 if t != 5 else 6 for t in toks[:3]] + toks[3:]
    far = rel_err(oracle_logits(ck, other)[-5:].float(),
                  oracle_logits(ck, toks)[-5:])
    assert far > 0.05, far
    eng = engine(ck, backend)
    seqs = {"s": toks}
    sizes = [7, 2, 50, 1, 1, 31, 2, 2] + [1] * 54
    got = replay(eng, seqs, [[("s", n)] for n in sizes])
    check(ck, got, seqs, backend[1])


@pytest.mark.parametrize("n,off", [(12, 3), (64, 8), (1032, 16)])
def test_section_norm_scatter_and_gate(backend, n, off):
    """Norm of a projection section into rows chosen by an index list (a
    latent into its pages) and the elementwise sigmoid gate, for sizes that
    take the plain and the 16-byte forms."""
    device, dtype = backend
    T = 9
    g = torch.Generator().manual_seed(n)
    proj = torch.randn(T, off + 2 * n + 8, generator=g).to(dtype)
    w = torch.rand(n, generator=g) + 0.5
    rows = torch.tensor([5, 0, 19, 7, 2, 11, 3, 18, 9])
    want = O.unit_rms(proj[:, off:off + n].double(), 1e-5) * w
    pages = torch.full((20, n), 3.0, dtype=dtype, device=device)
    hops.section_rmsnorm(proj.to(device), off, n, w.to(device), 1e-5, pages,
                         rows=rows.to(device))
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert float((pages[rows].double().cpu() - want).abs().max()) < tol
    untouched = [i for i in range(20) if i not in rows.tolist()]
    assert float((pages[untouched].float() - 3.0).abs().max()) == 0.0
    dense = torch.empty(T, n, dtype=dtype, device=device)
    hops.section_rmsnorm(proj.to(device), off, n, w.to(device), 1e-5, dense)
    assert float((dense.double().cpu() - want).abs().max()) < tol
    buf = torch.randn(T, n + 8, generator=g).to(dtype)
    v = buf.clone().to(device)
    hops.sigmoid_gate_mul(v[:, :n], proj.to(device), off + n)
    gate = torch.sigmoid(proj[:, off + n:off + 2 * n].double())
    assert float((v[:, :n].double().cpu() - buf[:, :n].double() * gate).abs().max()) < tol
    assert float((v[:, n:].float().cpu() - buf[:, n:].float()).abs().max()) == 0.0


@pytest.mark.parametrize("layout", ["tied", "latent", "latent_wide"])
@pytest.mark.parametrize("mode", ["prompt", "decoded"])
@pytest.mark.parametrize("page", [4, 8, 32])
def test_window_edges_stand_out(backend, layout, mode, page):
    """One key gets a score far above all others; it lies just inside
    (distance window-1) or just outside (distance window) the querying
    token's window, at and next to page borders, or far back. The output must
    be that key's value when it is visible and must not contain it when it is
    not. `tied`: whole-projection norms, values = raw keys, distance bias.
    `latent`: one shared latent read as key and value by every head
    (`latent_wide`: sixteen heads on a latent of 256)."""
    device, dtype = backend
    window = 11
    T = 75
    g = torch.Generator().manual_seed(11)
    if layout == "tied":
        H, G, dk = 4, 2, 8
    elif layout == "latent":
        H, G, dk = 3, 1, 16
    else:       # many heads on one wide latent
        H, G, dk = 16, 1, 256
    k = torch.randn(T, G, dk, generator=g) * 0.1
    q = torch.randn(T, H, dk, generator=g) * 0.1
    probes = []
    n = 0
    for i in range(window + 1, T, 3):
        for j in (i - window + 1, i - window, max(0, i - 40)):
            if n % 4 == 0:
                h = (n // 4) % H
                ch = (n // 4) % dk
                k[j, h // (H // G), ch] += 8.0
                q[i, h, ch] += 8.0
                probes.append((i, j, h))
            n += 1
    if dtype != torch.float32:
        q, k = (t.to(dtype).float() for t in (q, k))
    eps, scale = 1e-5, 9.0
    vis = O.window_visible(T, window)
    if layout == "tied":
        r1 = torch.tensor([0.3, 0.0, 0.6, 0.1])
        r2 = torch.tensor([0.5, 1.0, 0.05, 2.0])
        qw = torch.rand(H * dk, generator=g) + 0.5
        kw = torch.rand(G * dk, generator=g) + 0.5
        qn = (O.unit_rms(q.reshape(T, -1).double(), eps) * qw).view(T, H, dk)
        qn = qn * O.query_temperature(T, 0.25, 4)[:, None, None]
        kn = (O.unit_rms(k.reshape(T, -1).double(), eps) * kw).view(T, G, dk)
        if dtype != torch.float32:  # as the query rows and the K pages hold them
            qn, kn = (t.to(dtype).double() for t in (qn, kn))
        want = torch.stack([
            O.softmax_attention(qn[:, h], kn[:, h // (H // G)],
                                k[:, h // (H // G)].double(), scale, vis,
                                O.distance_bias(T, r1[h].double(), r2[h].double()))
            for h in range(H)], 1)
        vals = k
    else:
        want = torch.stack([
            O.softmax_attention(q[:, h].double(), k[:, 0].double(),
                                k[:, 0].double(), scale, vis)
            for h in range(H)], 1)
        vals = k
    # the framework's path: pages handed out in a scrambled order
    n_blocks = T // page + 3
    order = torch.randperm(n_blocks - 1, generator=g) + 1
    table = order[: (T + page - 1) // page].to(torch.int32)
    kc = torch.zeros(n_blocks, G, page, dk, dtype=dtype, device=device)
    vc = torch.zeros(n_blocks, G, page, dk, dtype=dtype, device=device)
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1)], 1).to(dtype).to(device)
    pieces = [T] if mode == "prompt" else [5] + [1] * (T - 5)
    got, done = [], 0
    for n in pieces:
        pos = torch.arange(done, done + n)
        slots = (table[pos // page].long() * page + pos % page).to(device)
        rows = proj[done:done + n]
        if layout == "tied":
            qq = hops.tied_attn_prep(
                rows, 0, H * dk, H, G, dk, qw.float().to(device),
                kw.float().to(device), eps, pos.to(device), 0.25, 4, slots,
                kc, vc)
            bias = dict(bias_r1=r1.to(device), bias_r2=r2.to(device))
            caches = (kc, vc)
        else:
            kc.view(-1, dk)[slots] = rows[:, H * dk:]
            qq = rows[:, :H * dk].reshape(n, H, dk).contiguous()
            bias = {}
            caches = (kc, kc)
        out = torch.zeros(n, H * dk, dtype=dtype, device=device)
        done += n
        tiles = {}
        if n > 1:      # prompt pieces carry the 32-row tile map
            tiles = dict(
                tile_seq=torch.zeros((n + 31) // 32, dtype=torch.int32, device=device),
                tile_q0=torch.arange(0, n, 32, dtype=torch.int32, device=device),
                prefill_rows=n)
        hops.local_attention(
            qq, caches[0], caches[1], table[None].to(device),
            torch.tensor([done], dtype=torch.int32, device=device),
            torch.tensor([0, n], dtype=torch.int32, device=device), scale, 0,
            window, rows, -1, out, 0, 1.0,
            token_seq=torch.zeros(n, dtype=torch.int32, device=device),
            **tiles, **bias)
        got.append(out.float().cpu())
    got = torch.cat(got).view(T, H, dk)
    tol = 1e-4 if dtype == torch.float32 else 5e-2
    assert float((got.double() - want).abs().max()) < tol
    inside = [(i, j, h) for i, j, h in probes if i - j < window]
    outside = [(i, j, h) for i, j, h in probes if i - j >= window]
    assert len(inside) >= 3 and len(outside) >= 6
    for i, j, h in inside:
        assert float((want[i, h] - vals[j, h // (H // G)].double()).abs().max()) < 2e-2
    for i, j, h in outside:
        assert float((want[i, h] - vals[j, h // (H // G)].double()).abs().max()) > 0.5


@pytest.mark.parametrize("W", [24, 15])
def test_bigram_rows_and_positions(backend, W):
    """The embedding alone: hashed rows with collisions, the extra row for a
    first token, previous tokens handed over between pieces, positions far
    from zero, an odd width (the last column has a sine and no cosine)."""
    device, dtype = backend
    V, buckets = 40, 7
    g = torch.Generator().manual_seed(4)
    emb = torch.randn(V, W, generator=g).to(dtype)
    big = torch.randn(buckets + 1, W, generator=g).to(dtype)
    toks = torch.randint(0, V, (30,), generator=g).tolist()
    want = (emb.double()[toks] + big.double()[O.bigram_rows(toks, buckets, 5, 9)]
            + O.sinusoid(3000 + 30, W)[3000:])
    ids = torch.tensor(toks, device=device)
    prev = torch.tensor([-1] + toks[:-1], device=device)
    pos = torch.arange(3000, 3030, device=device)
    got = hops.token_embed(ids, prev, pos, emb.to(device), big.to(device),
                           buckets, 5, 9,
                           hops.sinusoid_inv_freq(W, 10000.0).to(device))
    # position 3000 is not a sequence start here: only prev < 0 selects the
    # extra row; fp32 angles at 3000 rad carry ~1e-4 of absolute error
    assert float((got.double().cpu() - want).abs().max()) < 5e-4


def test_mlstm_stabiliser_and_denominator(backend):
    """Gate pre-activations that drive the running maximum both up and down
    (strong input gates after weak ones, long stretches of forgetting), a
    denominator that switches between |n.q| and exp(-m), heads of unequal
    key and value size; a prompt piece, then single tokens."""
    device, dtype = backend
    H, dk, dv, T, cap = 3, 12, 20, 50, 5.0
    g = torch.Generator().manual_seed(6)
    q = torch.randn(T, H, dk, generator=g)
    k = torch.randn(T, H, dk, generator=g)
    v = torch.randn(T, H, dv, generator=g)
    gate = torch.randn(T, H * dv, generator=g)
    ipre = torch.randn(T, H, generator=g) * 6.0
    fpre = torch.randn(T, H, generator=g) * 4.0 + 1.0
    ipre[20:30] -= 10.0
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1),
                      gate, ipre, fpre], 1).to(dtype)
    ib, fb = torch.tensor([0.5, -1.0, 0.0]), torch.tensor([1.0, 3.0, -2.0])
    nw = torch.rand(H * dv, generator=g) + 0.5
    p64 = proj.double()
    o_q, o_k = 0, H * dk
    o_v, o_g = 2 * H * dk, 2 * H * dk + H * dv
    o_i, o_f = o_g + H * dv, o_g + H * dv + H
    ig = cap * torch.tanh((p64[:, o_i:o_i + H] + ib) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((p64[:, o_f:o_f + H] + fb) / cap))
    heads = []
    for h in range(H):
        heads.append(O.unit_rms(O.mlstm_memory(
            p64[:, o_q + h * dk:o_q + (h + 1) * dk] * dk ** -0.5,
            p64[:, o_k + h * dk:o_k + (h + 1) * dk],
            p64[:, o_v + h * dv:o_v + (h + 1) * dv], ig[:, h], fg[:, h]), 1e-5))
    want = torch.cat(heads, -1) * nw * torch.sigmoid(p64[:, o_g:o_g + H * dv])
    mem = torch.full((3, H, dk, dv + 1), 7.0, device=device)   # stale slots
    ms = torch.full((3, H), -3.0, device=device)
    proj = proj.to(device)
    got, done = [], 0
    for n in [9] + [1] * 12 + [17, 2] + [1] * 10:
        rows = proj[done:done + n]
        done += n
        o, em = hops.mlstm_scan(
            rows, o_q, o_k, o_v, o_i, o_f, H, dk, dv, ib.to(device),
            fb.to(device), cap, mem, ms,
            torch.tensor([2], dtype=torch.int32, device=device),
            torch.tensor([0, n], dtype=torch.int32, device=device),
            torch.tensor([done], dtype=torch.int32, device=device))
        out = torch.zeros(n, H * dv, dtype=dtype, device=device)
        hops.mlstm_out(o, em, nw.to(device), rows, o_g, 1e-5, out, 0)
        got.append(out.float().cpu())
    assert done == T
    got = torch.cat(got)
    tol = 2e-4 if dtype == torch.float32 else 4e-2
    assert float((got.double() - want).abs().max()) < tol
    assert float(mem[1].min()) == 7.0          # other slots untouched


@pytest.mark.parametrize("W,F", [(40, 52), (38, 64), (2056, 4104)])
def test_sandwich_norms_depth_sum_and_polynorm(backend, W, F):
    """The fused post-norm + residual + depth-weighted sum + pre-norm, and
    PolyNorm, against their equations; row lengths that take the plain
    kernels and the register-resident vector forms with one and more chunks
    a thread."""
    device, dtype = backend
    T, n = 7, 4
    g = torch.Generator().manual_seed(8)
    X = torch.randn(n, T, W, generator=g) * 3
    x_in = torch.randn(T, W, generator=g) * 3
    y = torch.randn(T, W, generator=g).to(dtype)
    wb, wn = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    dw = torch.tensor([0.3, -0.2, 0.5, 1.1])
    eps = 1e-5
    r = x_in.double() + O.unit_rms(y.double(), eps) * wb
    z = dw[0] * X[0].double() + dw[1] * X[1].double() + dw[2] * X[2].double() + dw[3] * r
    h_want = O.unit_rms(z, eps) * wn
    Xd = X.to(device)
    xw = x_in.clone().to(device)    # input and sum share one buffer, as in the model
    h = torch.empty(T, W, dtype=dtype, device=device)
    hops.norm_residual(xw, y.to(device), wb.to(device), eps, Xd[n - 1],
                       stack=Xd, depth_w=dw.to(device), mix_out=xw,
                       next_w=wn.to(device), h_out=h)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert float((Xd[n - 1].double().cpu() - r).abs().max()) < 1e-5
    assert float((xw.double().cpu() - z).abs().max()) < 1e-5
    assert float((h.double().cpu() - h_want).abs().max()) < tol
    # without the sum, in place
    x2 = x_in.clone().to(device)
    hops.norm_residual(x2, y.to(device), wb.to(device), eps, x2,
                       next_w=wn.to(device), h_out=h)
    assert float((x2.double().cpu() - r).abs().max()) < 1e-5
    assert float((h.double().cpu() - O.unit_rms(r, eps) * wn).abs().max()) < tol
    zz = (torch.randn(T, F, generator=g) * 2).to(dtype)
    coef = torch.tensor([0.7, -0.4, 0.2, 0.05])
    got = hops.poly_act(zz.to(device), coef.to(device), eps)
    want = O.poly_norm(zz.double(), coef.double(), eps)
    assert float((got.double().cpu() - want).abs().max()) < tol


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


def test_lagged_decode_generates_the_same_tokens(tmp_path_factory, backend):
    """One-step-lagged decoding feeds the sampled-token tensor straight into
    the next step; the token before it (for the bigram row) is then the
    host's last known token. Greedy outputs must equal the synchronous ones."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    prompts = [tokens_for(ck[1], n, 50 + n) for n in (9, 4, 17)]
    outs = []
    for lagged in (False, True):
        eng = engine(ck, backend, blocks=40, async_decode=lagged)
        reqs = [eng.add_request(p, SamplingParams(max_tokens=10, temperature=0.0))
                for p in prompts]
        steps = 0
        while eng.has_work():
            eng.step()
            steps += 1
            assert steps < 200
        outs.append([r.output_token_ids for r in reqs])
    assert outs[0] == outs[1]


def test_service_job_on_a_checkpoint_directory(tmp_path_factory, local_client):
    """A checkpoint directory is a model name for the job service too."""
    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    job = local_client.infer(["alpha", "beta gamma"], model=ck[0],
                             sampling_params={"max_tokens": 4, "temperature": 0},
                             stay_attached=False)
    out = local_client.await_job_completion(job, timeout=120)
    assert out is not None and len(out) == 2


def test_cli_generates_from_a_checkpoint_directory(tmp_path_factory):
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


def test_registry_reads_every_size_from_the_config(tmp_path_factory):
    from sutro_amd.models.hybrid_spec import (HybridSpec, LatentAttnMixerSpec,
                                              MLSTMMixerSpec, TiedAttnMixerSpec)
    from sutro_amd.models.registry import get_model_spec

    ck = checkpoint(tmp_path_factory, "config_a", config_a)
    spec = get_model_spec(ck[0])
    assert isinstance(spec, HybridSpec) and spec.arch == "ruludra"
    kinds = [type(l.mixer) for l in spec.layers]
    assert kinds == [MLSTMMixerSpec, LatentAttnMixerSpec, TiedAttnMixerSpec,
                     LatentAttnMixerSpec, TiedAttnMixerSpec, MLSTMMixerSpec,
                     LatentAttnMixerSpec]
    assert spec.layers[3].mixer.kv_from == 1 and spec.layers[1].mixer.kv_from is None
    assert spec.layers[2].mixer.window == 11 and spec.layers[2].mixer.temp_every == 5
    assert spec.bigram == (97, 7, 13) and spec.logit_scale == 0.5
    assert [l.ff for l in spec.layers] == [0, 40, 56, 0, 0, 32, 24]
    # the cache holds keys + raw keys for attention, one latent for a latent
    # layer that owns it, nothing for one that borrows it, and state for mLSTM
    eng = engine(ck, ("cpu", torch.float32))
    kv, st = eng.model.cache_layout()
    assert kv[2] == (2, 16, 16) and kv[1] == (1, 16, 0) and kv[3] is None
    assert kv[0] is None and st[0] == {"mem": (2, 8, 13), "m": (2,)}
    bad = json.loads(json.dumps(ck[1]))
    bad["layers"][3]["mixer"]["kv_from"] = 5
    from sutro_amd.models.hybrid_spec import ruludra_spec
    with pytest.raises(ValueError):
        ruludra_spec(bad)
