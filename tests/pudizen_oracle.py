"""A plain float64 implementation of the Pudizen design, one function per
mechanism, for the tests to compare the serving path against. It shares no
code with the package: whole sequences only, no cache, no batching, dense
masks and python loops where they are clearest.

Weights are a dict name -> float64 tensor with the checkpoint's names
('embed', 'bigram', 'l<i>.norm1', 'l<i>.mix.q', ...); the config is the dict
that config.json holds.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """The width in `groups` equal consecutive parts, each divided by its own
    root mean square (eps under the root); the whole times w."""
    n, width = x.shape
    parts = x.reshape(n, groups, width // groups)
    return unit_rms(parts, eps).reshape(n, width) * w


def embedding(tokens, w, emb):
    """embed[t_n] * scale + bigram[r_n], r_n = (t_(n-1) * mul_prev + t_n *
    mul_cur) mod buckets, r_0 = buckets (the table's last row)."""
    b = emb["bigram"]
    rows = []
    for n, t in enumerate(tokens):
        if n == 0:
            r = int(b["buckets"])
        else:
            r = (tokens[n - 1] * int(b["mul_prev"]) + t * int(b["mul_cur"])) % int(b["buckets"])
        rows.append(w["embed"][t] * float(emb["scale"]) + w["bigram"][r])
    return torch.stack(rows)


def pair_frequencies(dims, base, scaling=None):
    """f_m = base^(-2m/dims), m < dims/2; with `scaling` {factor, low, high,
    original} by wavelength l = 2 pi / f: short waves (l < original/high)
    stay, long ones (l > original/low) are divided by factor, and between
    the two f is blended linearly in original/l."""
    out = []
    for m in range(dims // 2):
        f = float(base) ** (-2.0 * m / dims)
        if scaling:
            fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            lam = 2.0 * math.pi / f
            if lam > orig / lo:
                f = f / fac
            elif lam >= orig / hi:
                s = (orig / lam - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def turn(x, positions, freq, dims, interleaved, back=False):
    """x [n, heads, >= dims]: the first `dims` dimensions of every head turned
    by the token's position: pair m = (m, m + dims/2), or (2m, 2m + 1) when
    interleaved; (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = +-pos
    * freq[m]."""
    out = x.clone()
    for m in range(dims // 2):
        iu, iv = (2 * m, 2 * m + 1) if interleaved else (m, m + dims // 2)
        a = positions.to(F64) * freq[m] * (-1.0 if back else 1.0)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., iu], x[..., iv]
        out[..., iu] = u * c - v * s
        out[..., iv] = v * c + u * s
    return out


def _mask(n, window):
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    vis = j <= i
    if window:
        vis = vis & (i - j < window)
    return vis


def softmax_attention(h, w, pre, mx, eps):
    """Mixer 'attention': RMS norm over the whole q and the whole k
    projection, rotation in halves on q and k, values turned by their
    position over their whole width and the result turned back, causal (or
    windowed) softmax."""
    n = h.shape[0]
    H, G = int(mx["heads"]), int(mx.get("kv_heads", mx["heads"]))
    d, dv = int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    pos = torch.arange(n)
    q = unit_rms(h @ w[pre + "q"].T, eps) * w[pre + "q.norm"]
    k = unit_rms(h @ w[pre + "k"].T, eps) * w[pre + "k.norm"]
    q, k = q.view(n, H, d), k.view(n, G, d)
    v = (h @ w[pre + "v"].T).view(n, G, dv)
    rot = mx.get("rot") or {}
    if rot.get("dims"):
        f = pair_frequencies(int(rot["dims"]), rot["base"], rot.get("scaling"))
        q = turn(q, pos, f, int(rot["dims"]), False)
        k = turn(k, pos, f, int(rot["dims"]), False)
    fv = pair_frequencies(dv, rot.get("base", 10000.0))
    v = turn(v, pos, fv, dv, False)
    vis = _mask(n, int((mx.get("mask") or {}).get("size", 0)))
    out = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(mx["scale"])
        s = s.masked_fill(~vis, float("-inf"))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    out = turn(out, pos, fv, dv, False, back=True)
    return out.reshape(n, H * dv) @ w[pre + "o"].T


def sigmoid_attention(h, w, pre, mx, eps):
    """Mixer 'attention_2': rotation of neighbouring pairs on q and k, a
    sliding window, weights sigmoid(score + pb_h) that are not normalised."""
    n = h.shape[0]
    H, G = int(mx["heads"]), int(mx.get("kv_heads", mx["heads"]))
    d, dv = int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    pos = torch.arange(n)
    q = (h @ w[pre + "q"].T).view(n, H, d)
    k = (h @ w[pre + "k"].T).view(n, G, d)
    v = (h @ w[pre + "v"].T).view(n, G, dv)
    rot = mx.get("rot") or {}
    if rot.get("dims"):
        f = pair_frequencies(int(rot["dims"]), rot["base"], rot.get("scaling"))
        q = turn(q, pos, f, int(rot["dims"]), True)
        k = turn(k, pos, f, int(rot["dims"]), True)
    vis = _mask(n, int((mx.get("mask") or {}).get("size", 0)))
    out = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(mx["scale"]) + w[pre + "pb"][hd]
        out[:, hd] = (torch.sigmoid(s) * vis) @ v[:, g]
    return out.reshape(n, H * dv) @ w[pre + "o"].T


def latent_attention(h, w, pre, mx, eps):
    """Mixer 'latent_attention': keys and values expanded head by head from
    the normed latent, causal softmax, a sigmoid gate per head."""
    n = h.shape[0]
    H, d, dv = int(mx["heads"]), int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
    q = (h @ w[pre + "q"].T).view(n, H, d)
    c = unit_rms(h @ w[pre + "dkv"].T, eps) * w[pre + "dkv.norm"]
    k = (c @ w[pre + "uk"].T).view(n, H, d)
    v = (c @ w[pre + "uv"].T).view(n, H, dv)
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    vis = _mask(n, 0)
    out = torch.zeros(n, H, dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd].T) * float(mx["scale"])
        s = s.masked_fill(~vis, float("-inf"))
        out[:, hd] = (torch.softmax(s, dim=-1) @ v[:, hd]) * gate[:, hd:hd + 1]
    return out.reshape(n, H * dv) @ w[pre + "o"].T


def feed_forward(h, w, pre):
    a = torch.clamp(h @ w[pre + "up"].T, min=0.0)
    return (a * a) @ w[pre + "down"].T


MIXERS = {"attention": softmax_attention, "attention_2": sigmoid_attention,
          "latent_attention": latent_attention}


def forward(cfg, w, tokens, return_layers=False):
    eps = float(cfg["norm"]["eps"])
    groups = int(cfg["norm"].get("groups", 1))
    x = embedding(list(tokens), w, cfg["embedding"])
    layers = []
    for i, sp in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = group_norm(x, w[p + "norm1"], groups, eps)
        y = MIXERS[sp["type"]](h, w, p + "mix.", sp["mixer"], eps)
        if sp.get("mlp") is not None:
            y = y + feed_forward(h, w, p + "mlp.")
        x = x + y
        layers.append(x.clone())
    logits = group_norm(x, w["final.norm"], groups, eps) @ w["head"].T
    return (logits, layers) if return_layers else logits


def random_weights(cfg, seed=0):
    """Random weights for a config, rounded to bfloat16 (what a checkpoint
    holds) and returned in float64."""
    g = torch.Generator().manual_seed(seed)
    W, V = int(cfg["width"]), int(cfg["vocab"])
    w = {}

    def mat(name, rows, cols, scale=1.0):
        w[name] = torch.randn(rows, cols, generator=g) * (scale / math.sqrt(cols))

    def vec(name, n, mean=0.0, std=1.0):
        w[name] = mean + std * torch.randn(n, generator=g)

    mat("embed", V, W, math.sqrt(W))
    mat("bigram", int(cfg["embedding"]["bigram"]["buckets"]) + 1, W, math.sqrt(W))
    vec("final.norm", W, 1.0, 0.2)
    mat("head", V, W)
    for i, sp in enumerate(cfg["layers"]):
        p = f"l{i}."
        mx = sp["mixer"]
        vec(p + "norm1", W, 1.0, 0.2)
        H = int(mx["heads"])
        d, dv = int(mx["dim"]), int(mx.get("vdim", mx["dim"]))
        if sp["type"] == "latent_attention":
            r = int(mx["kv_rank"])
            mat(p + "mix.q", H * d, W, 2.0)
            mat(p + "mix.dkv", r, W)
            vec(p + "mix.dkv.norm", r, 1.0, 0.3)
            mat(p + "mix.uk", H * d, r, 2.0)
            mat(p + "mix.uv", H * dv, r)
            mat(p + "mix.g", H, W, 2.0)
        else:
            G = int(mx.get("kv_heads", H))
            mat(p + "mix.q", H * d, W, 2.0)
            mat(p + "mix.k", G * d, W, 2.0)
            mat(p + "mix.v", G * dv, W)
            if sp["type"] == "attention":
                vec(p + "mix.q.norm", H * d, 1.0, 0.3)
                vec(p + "mix.k.norm", G * d, 1.0, 0.3)
            else:
                vec(p + "mix.pb", H, -1.0, 1.0)
        mat(p + "mix.o", W, H * dv)
        mlp = sp.get("mlp")
        if mlp is not None:
            mat(p + "mlp.up", int(mlp["ff"]), W, 1.5)
            mat(p + "mlp.down", W, int(mlp["ff"]))
    return {k: v.to(torch.bfloat16).to(F64) for k, v in w.items()}
