"""A plain, slow float64 implementation of the Ruludra equations, one function
per mechanism, sharing no code with the package. It works on whole sequences
(no cache, no batching, no portions) and is the yardstick for the engine in
tests/test_ruludra.py. It also makes small configurations and random
checkpoints.

Notation: h [T, W] is a sublayer's input, weights are [out, in], `w` maps
checkpoint tensor names to float64 tensors (already rounded to bf16, which is
how they are stored).
"""

import json
import math
import os

import torch

F64 = torch.float64


# ---------------------------------------------------------------- pieces ----

def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token; the first token of a sequence
    has no predecessor and takes the extra last row."""
    rows = [buckets]
    for a, b in zip(tokens[:-1], tokens[1:]):
        rows.append((a * mul_prev + b * mul_cur) % buckets)
    return rows


def sinusoid(T, width):
    """[T, width]: column 2i = sin(p / 10000^(2i/width)), column 2i+1 = cos."""
    p = torch.arange(T, dtype=F64)[:, None]
    i = torch.arange((width + 1) // 2, dtype=F64)[None, :]
    ang = p * 10000.0 ** (-2.0 * i / width)
    out = torch.zeros(T, width, dtype=F64)
    out[:, 0::2] = torch.sin(ang)
    out[:, 1::2] = torch.cos(ang)[:, :width // 2]
    return out


def window_visible(T, size):
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (size 0: all
    earlier keys)."""
    d = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    vis = d >= 0
    if size > 0:
        vis = vis & (d < size)
    return vis


def softmax_attention(q, k, v, scale, vis, bias=None):
    """One head. q, k [T, dk]; v [T, dv]; vis [T, T] bool; bias [T, T] is
    taken off the scaled scores."""
    sc = (q @ k.T) * scale
    if bias is not None:
        sc = sc - bias
    sc = sc.masked_fill(~vis, -math.inf)
    return torch.softmax(sc, -1) @ v


def query_temperature(T, coef, every):
    p = torch.arange(T, dtype=F64)
    return 1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)


def distance_bias(T, r1, r2):
    d = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp(min=0)
    return r1 * torch.log(1.0 + r2 * d.to(F64))


def mlstm_memory(q, k, v, ig, fg):
    """One head of the mLSTM recurrence. q, k [T, dk] (q already scaled);
    v [T, dv]; ig, fg [T] log gates. Memory, normaliser start at zero, the
    running maximum at 0. Returns the normalised read-out [T, dv]."""
    T, dk = q.shape
    dv = v.shape[1]
    C = torch.zeros(dk, dv, dtype=F64)
    n = torch.zeros(dk, dtype=F64)
    m = torch.zeros((), dtype=F64)
    out = torch.zeros(T, dv, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(fg[t] + m, ig[t])
        keep = torch.exp(fg[t] + m - m_new)
        take = torch.exp(ig[t] - m_new)
        C = keep * C + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        den = torch.maximum((n @ q[t]).abs(), torch.exp(-m)) + 1e-6
        out[t] = (C.T @ q[t]) / den
    return out


def poly_norm(z, coef, eps):
    return (coef[0] * unit_rms(z, eps) + coef[1] * unit_rms(z * z, eps)
            + coef[2] * unit_rms(z ** 3, eps) + coef[3])


# ---------------------------------------------------------------- mixers ----

def attention_mixer(w, p, mc, h, eps):
    T = h.shape[0]
    H, G, dk = mc["heads"], mc["kv_heads"], mc["dim"]
    q = h @ w[p + "q"].T
    k = h @ w[p + "k"].T
    v = k.view(T, G, dk)                       # values: the keys as projected
    q = unit_rms(q, eps) * w[p + "q.norm"]     # one norm over all heads
    k = unit_rms(k, eps) * w[p + "k.norm"]
    qt = mc.get("q_temp")
    if qt:
        q = q * query_temperature(T, qt["coef"], qt["every"])[:, None]
    q, k = q.view(T, H, dk), k.view(T, G, dk)
    vis = window_visible(T, mc["mask"]["size"])
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        bias = distance_bias(T, w[p + "r1"][hh], w[p + "r2"][hh])
        heads.append(softmax_attention(q[:, hh], k[:, g], v[:, g],
                                       mc["scale"], vis, bias))
    return torch.cat(heads, -1) @ w[p + "o"].T


def latent_mixer(w, p, mc, h, eps, shared_latent=None):
    """Returns (output, latent); `shared_latent` replaces the layer's own."""
    T = h.shape[0]
    H, dk, dv = mc["heads"], mc["dim"], mc["vdim"]
    cq = unit_rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, dk)
    if shared_latent is None:
        c = unit_rms(h @ w[p + "dkv"].T, eps) * w[p + "dkv.norm"]
    else:
        c = shared_latent
    k = (c @ w[p + "uk"].T).view(T, H, dk)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    vis = window_visible(T, mc["mask"]["size"])
    heads = [softmax_attention(q[:, hh], k[:, hh], v[:, hh], mc["scale"], vis)
             for hh in range(H)]
    o = torch.cat(heads, -1) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, c


def mlstm_mixer(w, p, mc, h, eps):
    T = h.shape[0]
    H, dk, dv, cap = mc["heads"], mc["dim"], mc["vdim"], mc["gate_cap"]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(
        cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    heads = [unit_rms(mlstm_memory(q[:, hh], k[:, hh], v[:, hh], ig[:, hh],
                                   fg[:, hh]), eps) for hh in range(H)]
    o = torch.cat(heads, -1) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def feed_forward(w, p, h, eps):
    return poly_norm(h @ w[p + "up"].T, w[p + "act"], eps) @ w[p + "down"].T


# ----------------------------------------------------------------- model ----

def forward(config, w, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence. `streams`, a list, receives
    every layer's outgoing stream (the next layer's input)."""
    eps = config["norm"]["eps"]
    W = config["width"]
    T = len(tokens)
    big = config["embedding"]["bigram"]
    x = (w["embed"][tokens]
         + w["bigram"][bigram_rows(tokens, big["buckets"], big["mul_prev"],
                                   big["mul_cur"])]
         + sinusoid(T, W))
    kept = [x]
    latents = {}
    for i, layer in enumerate(config["layers"]):
        lp, mc = f"l{i}.", layer["mixer"]
        hin = unit_rms(x, eps) * w[lp + "norm1"]
        if layer["type"] == "attention":
            y = attention_mixer(w, lp + "mix.", mc, hin, eps)
        elif layer["type"] == "latent_attention":
            src = mc.get("kv_from")
            y, latents[i] = latent_mixer(
                w, lp + "mix.", mc, hin, eps,
                None if src is None else latents[src])
        else:
            y = mlstm_mixer(w, lp + "mix.", mc, hin, eps)
        x = x + unit_rms(y, eps) * w[lp + "norm1b"]
        if layer["mlp"] is not None:
            y = feed_forward(w, lp + "mlp.", unit_rms(x, eps) * w[lp + "norm2"],
                             eps)
            x = x + unit_rms(y, eps) * w[lp + "norm2b"]
        kept.append(x)
        x = sum(w[lp + "dwa"][j] * kept[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    return (unit_rms(x, eps) * w["final.norm"]) @ w["head"].T * config["logit_scale"]


# -------------------------------------------------- configs and weights -----

def attn_cfg(heads, kv_heads, dim, window, scale, coef=0.25, every=16):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
            "mask": {"size": window}, "scale": scale,
            "q_temp": {"coef": coef, "every": every}}


def latent_cfg(heads, dim, vdim, q_rank, kv_rank, window, scale, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank,
         "kv_rank": kv_rank, "mask": {"size": window}, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def mlstm_cfg(heads, dim, vdim, cap=15.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer,
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def make_config(width, vocab, layers, eps=1e-5, logit_scale=0.5,
                buckets=97, mul_prev=7, mul_cur=13):
    return {"architecture": "Ruludra", "width": width, "vocab": vocab,
            "norm": {"eps": eps}, "logit_scale": logit_scale,
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev,
                                     "mul_cur": mul_cur}},
            "layers": layers}


def make_weights(config, seed=0):
    """Random weights (already rounded to bf16) under checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    w = {}

    def rnd(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    def lin(out, inn):
        return rnd(out, inn, std=inn ** -0.5)

    def uni(n, lo, hi):
        return torch.rand(n, generator=g) * (hi - lo) + lo

    w["embed"] = rnd(config["vocab"], W)
    w["bigram"] = rnd(config["embedding"]["bigram"]["buckets"] + 1, W, std=0.7)
    w["head"] = lin(config["vocab"], W)
    w["final.norm"] = rnd(W, std=0.2, mean=1.0)
    for i, layer_ in enumerate(config["layers"]):
        lp, mc = f"l{i}.", layer_["mixer"]
        p = lp + "mix."
        for n in ("norm1", "norm1b"):
            w[lp + n] = rnd(W, std=0.2, mean=1.0)
        w[lp + "dwa"] = uni(i + 2, -0.4, 0.9)
        w[lp + "dwa"][-1] = 1.0
        if layer_["type"] == "attention":
            H, G, dk = mc["heads"], mc["kv_heads"], mc["dim"]
            w[p + "q"], w[p + "k"] = lin(H * dk, W), lin(G * dk, W)
            w[p + "q.norm"] = rnd(H * dk, std=0.2, mean=1.0)
            w[p + "k.norm"] = rnd(G * dk, std=0.2, mean=1.0)
            w[p + "r1"], w[p + "r2"] = uni(H, 0.1, 0.8), uni(H, 0.05, 1.5)
            w[p + "o"] = lin(W, H * dk)
        elif layer_["type"] == "latent_attention":
            H, dk, dv = mc["heads"], mc["dim"], mc["vdim"]
            qr, kr = mc["q_rank"], mc["kv_rank"]
            w[p + "dq"] = lin(qr, W)
            w[p + "dq.norm"] = rnd(qr, std=0.2, mean=1.0)
            w[p + "uq"] = lin(H * dk, qr)
            if mc.get("kv_from") is None:
                w[p + "dkv"] = lin(kr, W)
                w[p + "dkv.norm"] = rnd(kr, std=0.2, mean=1.0)
            w[p + "uk"], w[p + "uv"] = lin(H * dk, kr), lin(H * dv, kr)
            w[p + "g"], w[p + "o"] = lin(H * dv, W), lin(W, H * dv)
        else:
            H, dk, dv = mc["heads"], mc["dim"], mc["vdim"]
            w[p + "q"], w[p + "k"] = lin(H * dk, W), lin(H * dk, W)
            w[p + "v"], w[p + "g"] = lin(H * dv, W), lin(H * dv, W)
            w[p + "i"], w[p + "f"] = lin(H, W) * 2.0, lin(H, W) * 2.0
            w[p + "i.b"] = rnd(H, std=0.5, mean=-0.5)
            w[p + "f.b"] = rnd(H, std=0.7, mean=2.5)
            w[p + "norm"] = rnd(H * dv, std=0.2, mean=1.0)
            w[p + "o"] = lin(W, H * dv)
        if layer_["mlp"] is not None:
            ff = layer_["mlp"]["ff"]
            for n in ("norm2", "norm2b"):
                w[lp + n] = rnd(W, std=0.2, mean=1.0)
            w[lp + "mlp.up"], w[lp + "mlp.down"] = lin(ff, W), lin(W, ff)
            w[lp + "mlp.act"] = torch.tensor([0.7, 0.4, -0.3, 0.1]) + rnd(4, std=0.1)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in w.items()}


def save_checkpoint(path, config, w):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    return path
