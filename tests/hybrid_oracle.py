"""A plain, slow float64 implementation of the Vodinex equations, one function
per mechanism, written from the design's description and sharing no code with
the package. It works on whole sequences (no cache, no batching) and is the
yardstick for the engine in tests/test_vodinex*.py.

Notation: h [T, W] sublayer input; weights are [out, in]; `w` maps checkpoint
tensor names to tensors.
"""

import math

import torch

F64 = torch.float64


# ---------------------------------------------------------------- pieces ----

def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def short_filter_silu(x, taps_w):
    """Causal per-channel filter then silu. x [T, C]; taps_w [C, taps] with the
    last column acting on the current token; zeros before the start."""
    T, C = x.shape
    n = taps_w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(n):
            src = t - (n - 1 - j)
            if src >= 0:
                y[t] += taps_w[:, j] * x[src]
    return y * torch.sigmoid(y)


def unit_vectors(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def channel_decay(a_log_h, pre):
    """exp(-exp(A_log) * softplus(pre)) for one head; pre [T, dk]."""
    return torch.exp(-math.exp(float(a_log_h))
                     * torch.nn.functional.softplus(pre))


def delta_rule(q, k, v, beta, decay):
    """One head. q, k, decay [T, dk]; v [T, dv]; beta [T]. Returns o [T, dv]
    and the final memory S [dk, dv]."""
    T, dk = q.shape
    dv = v.shape[1]
    S = torch.zeros(dk, dv, dtype=F64)
    o = torch.zeros(T, dv, dtype=F64)
    for t in range(T):
        S = decay[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def rotate_prefix(x, positions, dims, base):
    """x [T, heads, d]: rotate dimension i with i + dims/2 (i < dims/2) by the
    angle position * base^(-2i/dims); dimensions >= dims pass through."""
    if dims == 0:
        return x
    half = dims // 2
    out = x.clone()
    for i in range(half):
        ang = positions.to(F64) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        a, b = x[..., i], x[..., i + half]
        out[..., i] = a * c - b * s
        out[..., i + half] = b * c + a * s
    return out


def visible(i, j, chunk):
    """May the query at position i see the key at position j?"""
    if j > i:
        return False
    return chunk <= 0 or (i // chunk) == (j // chunk)


def masked_softmax_attention(q, k, v, scale, chunk):
    """One head. q [T, dk], k [T, dk], v [T, dv] -> [T, dv]."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if visible(i, j, chunk)]
        sc = torch.stack([(q[i] @ k[j]) * scale for j in js])
        p = torch.softmax(sc, 0)
        out[i] = sum(p[n] * v[j] for n, j in enumerate(js))
    return out


# ---------------------------------------------------------------- mixers ----

def lin(w, name, h, bias=False):
    y = h @ w[name].to(F64).T
    if bias:
        y = y + w[name + ".b"].to(F64)
    return y


def delta_mixer(w, p, mc, h, eps):
    T = h.shape[0]
    H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    q = short_filter_silu(lin(w, p + ".q", h), w[p + ".q.conv"].to(F64)).view(T, G, dk)
    k = short_filter_silu(lin(w, p + ".k", h), w[p + ".k.conv"].to(F64)).view(T, G, dk)
    v = short_filter_silu(lin(w, p + ".v", h), w[p + ".v.conv"].to(F64)).view(T, H, dv)
    q = unit_vectors(q) * dk ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(lin(w, p + ".b", h))
    pre = (lin(w, p + ".a2", lin(w, p + ".a1", h))
           + w[p + ".dt_bias"].to(F64)).view(T, H, dk)
    gate = torch.sigmoid(lin(w, p + ".g2", lin(w, p + ".g1", h))).view(T, H, dv)
    heads = []
    for hh in range(H):
        kv = hh // (H // G)
        o, _ = delta_rule(q[:, kv], k[:, kv], v[:, hh], beta[:, hh],
                          channel_decay(w[p + ".A_log"][hh], pre[:, hh]))
        heads.append(rms_unit(o, eps) * w[p + ".norm"].to(F64) * gate[:, hh])
    return lin(w, p + ".o", torch.cat(heads, -1))


def attention_mixer(w, p, mc, h, eps):
    T = h.shape[0]
    H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    pos = torch.arange(T)
    q = lin(w, p + ".q", h, True).view(T, H, dk)
    k = lin(w, p + ".k", h, True).view(T, G, dk)
    v = lin(w, p + ".v", h, True).view(T, G, dv)
    q = rms_unit(q, eps) * w[p + ".q.norm"].to(F64)
    k = rms_unit(k, eps) * w[p + ".k.norm"].to(F64)
    q = rotate_prefix(q, pos, mc["rot"]["dims"], mc["rot"]["base"])
    k = rotate_prefix(k, pos, mc["rot"]["dims"], mc["rot"]["base"])
    gate = torch.sigmoid(lin(w, p + ".g", h))
    heads = []
    for hh in range(H):
        kv = hh // (H // G)
        o = masked_softmax_attention(q[:, hh], k[:, kv], v[:, kv], mc["scale"],
                                     mc["mask"]["size"])
        heads.append(o * gate[:, hh:hh + 1])
    return lin(w, p + ".o", torch.cat(heads, -1), True)


def mixer(w, i, layer, h, eps):
    p = f"l{i}.mix"
    if layer["type"] == "channel_delta":
        return delta_mixer(w, p, layer["mixer"], h, eps)
    mc = layer["mixer"]
    return (mc["left_scale"] * attention_mixer(w, p + ".left", mc["left"], h, eps)
            + mc["right_scale"] * delta_mixer(w, p + ".right", mc["right"], h, eps))


def feed_forward(w, i, h):
    p = f"l{i}.mlp"
    return lin(w, p + ".down", gelu_tanh(lin(w, p + ".gate", h)) * lin(w, p + ".up", h))


def gated_sublayer(w, gate_name, norm_name, x, y, eps, m):
    y = y * torch.sigmoid(lin(w, gate_name, x, True))
    return x + m * rms_unit(y, eps) * w[norm_name].to(F64)


def forward(config, w, tokens):
    """Logits [T, vocab] of one whole sequence."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    x = w["embed"].to(F64)[torch.tensor(tokens)]
    for i, layer in enumerate(config["layers"]):
        x = gated_sublayer(w, f"l{i}.rg1", f"l{i}.norm1", x,
                           mixer(w, i, layer, x, eps), eps, m)
        if layer["mlp"] is not None:
            x = gated_sublayer(w, f"l{i}.rg2", f"l{i}.norm2", x,
                               feed_forward(w, i, x), eps, m)
    x = rms_unit(x, eps) * w["final.norm"].to(F64)
    return x @ w["head"].to(F64).T


# ------------------------------------------------------ model construction --

def delta_cfg(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "conv": conv}


def attn_cfg(heads, kv_heads, dim, vdim, chunk, rot_dims, base, scale):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "mask": {"size": chunk}, "rot": {"dims": rot_dims, "base": base},
            "scale": scale}


def delta_layer(mix, ff=None):
    return {"type": "channel_delta", "mixer": mix,
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def parallel_layer(left, right, ls, rs, ff=None):
    return {"type": "parallel",
            "mixer": {"left": left, "right": right, "left_scale": ls,
                      "right_scale": rs},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(width, vocab, layers, eps=1e-4, mult=0.9):
    return {"architecture": "Vodinex", "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "vocab": vocab, "width": width}


def make_weights(config, seed=0, decay_rank=6, gate_rank=5):
    """Random bf16-representable weights in checkpoint naming."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    w = {}

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(tuple(shape), generator=g) * std + mean).to(torch.bfloat16)

    def delta(p, mc):
        H, G, dk, dv, n = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"], mc["conv"]
        for nm, rows in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
            w[f"{p}.{nm}"] = rnd(rows, W, std=W ** -0.5)
            w[f"{p}.{nm}.conv"] = rnd(rows, n, std=0.5)
        w[p + ".b"] = rnd(H, W, std=W ** -0.5)
        w[p + ".A_log"] = rnd(H, std=0.5, mean=-0.5)
        w[p + ".norm"] = rnd(dv, std=0.1, mean=1.0)
        w[p + ".a1"] = rnd(decay_rank, W, std=W ** -0.5)
        w[p + ".a2"] = rnd(H * dk, decay_rank, std=decay_rank ** -0.5)
        w[p + ".dt_bias"] = rnd(H * dk, std=0.7, mean=-1.0)
        w[p + ".g1"] = rnd(gate_rank, W, std=W ** -0.5)
        w[p + ".g2"] = rnd(H * dv, gate_rank, std=gate_rank ** -0.5)
        w[p + ".o"] = rnd(W, H * dv, std=(H * dv) ** -0.5)

    def attn(p, mc):
        H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
            w[f"{p}.{nm}"] = rnd(rows, W, std=W ** -0.5)
            w[f"{p}.{nm}.b"] = rnd(rows, std=0.1)
        w[p + ".q.norm"] = rnd(dk, std=0.1, mean=1.0)
        w[p + ".k.norm"] = rnd(dk, std=0.1, mean=1.0)
        w[p + ".g"] = rnd(H, W, std=W ** -0.5)
        w[p + ".o"] = rnd(W, H * dv, std=(H * dv) ** -0.5)
        w[p + ".o.b"] = rnd(W, std=0.1)

    w["embed"] = rnd(config["vocab"], W)
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}"
        w[p + ".norm1"] = rnd(1, std=0.1, mean=1.0).reshape(())
        w[p + ".rg1"] = rnd(W, W, std=W ** -0.5)
        w[p + ".rg1.b"] = rnd(W, std=0.3)
        if layer["type"] == "channel_delta":
            delta(p + ".mix", layer["mixer"])
        else:
            attn(p + ".mix.left", layer["mixer"]["left"])
            delta(p + ".mix.right", layer["mixer"]["right"])
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            w[p + ".norm2"] = rnd(1, std=0.1, mean=1.0).reshape(())
            w[p + ".mlp.gate"] = rnd(ff, W, std=W ** -0.5)
            w[p + ".mlp.up"] = rnd(ff, W, std=W ** -0.5)
            w[p + ".mlp.down"] = rnd(W, ff, std=ff ** -0.5)
            w[p + ".rg2"] = rnd(W, W, std=W ** -0.5)
            w[p + ".rg2.b"] = rnd(W, std=0.3)
    w["final.norm"] = rnd(1, std=0.1, mean=1.0).reshape(())
    w["head"] = rnd(config["vocab"], W, std=W ** -0.5)
    return w


def save_checkpoint(path, config, w):
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    return path
