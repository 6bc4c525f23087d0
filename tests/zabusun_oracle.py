"""A plain float64 implementation of the Zabusun design, one function per
mechanism, for the tests to compare the serving path against. It shares no
code with the package: whole sequences only, no cache, no batching, python
loops where they are clearest.

Weights are a dict name -> float64 tensor with the checkpoint's names
('embed', 'embed.norm', 'l<i>.norm1', 'l<i>.mix.left.q', ...); the config is
the dict that config.json holds.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last dimension."""
    r = torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return x / r * w


def rotary_frequencies(rot):
    """Per-pair frequencies and the cos/sin multiplier of a rotation spec
    {base, dims, scaling: {factor, original, fast, slow} | None}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def where(turns):   # the (fractional) pair index that makes `turns` turns
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(float(sc["fast"]))), 0)
    hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot):
    """x [n, heads, dim]: rotate the first rot.dims dimensions of every head,
    dimension i paired with i + dims/2; the rest passes unchanged."""
    dims = int(rot["dims"])
    half = dims // 2
    freq, mult = rotary_frequencies(rot)
    ang = positions.to(F64)[:, None] * freq[None, :]          # [n, half]
    c, s = (torch.cos(ang) * mult)[:, None, :], (torch.sin(ang) * mult)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def sigmoid_attention(h, w, pre, mx, eps, positions=None):
    """The left mixer: grouped heads, q/k norm, partial rotation, sigmoid
    weights with a per-head bias (not normalised over keys), causal, a
    per-head sigmoid output gate."""
    n = h.shape[0]
    H, G = int(mx["heads"]), int(mx.get("kv_heads", mx["heads"]))
    d, dv = int(mx["dim"]), int(mx["vdim"])
    pos = torch.arange(n) if positions is None else positions
    q = (h @ w[pre + "q"].T).view(n, H, d)
    k = (h @ w[pre + "k"].T).view(n, G, d)
    v = (h @ w[pre + "v"].T).view(n, G, dv)
    q = rms_norm(q, w[pre + "q.norm"], eps)
    k = rms_norm(k, w[pre + "k.norm"], eps)
    if mx.get("rot"):
        q, k = rotate(q, pos, mx["rot"]), rotate(k, pos, mx["rot"])
    gate = torch.sigmoid(h @ w[pre + "g"].T)                   # [n, H]
    out = torch.zeros(n, H, dv, dtype=F64)
    rep = H // G
    for hd in range(H):
        g = hd // rep
        s = q[:, hd] @ k[:, g].T * float(mx["scale"]) + w[pre + "pb"][hd]
        a = torch.sigmoid(s)
        a = torch.tril(a)                    # key j is seen by queries i >= j
        out[:, hd] = (a @ v[:, g]) * gate[:, hd:hd + 1]
    return out.reshape(n, H * dv) @ w[pre + "o"].T


def min_gru(h, w, pre, state=None):
    """The right mixer. Returns (output, final state)."""
    n = h.shape[0]
    z = torch.sigmoid(h @ w[pre + "z"].T + w[pre + "z.b"])
    u = h @ w[pre + "x"].T + w[pre + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = h @ w[pre + "g"].T
    gate = gate * torch.sigmoid(gate)
    s = torch.zeros(z.shape[1], dtype=F64) if state is None else state.clone()
    rows = []
    for t in range(n):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        rows.append(s * gate[t])
    return torch.stack(rows) @ w[pre + "o"].T, s


def parallel_mixer(h, w, pre, mx, eps):
    left = sigmoid_attention(h, w, pre + "left.", mx["left"], eps)
    right, _ = min_gru(h, w, pre + "right.")
    return float(mx["left_scale"]) * left + float(mx["right_scale"]) * right


def clamped_glu(h, w, pre, limit):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def routed_experts(h, w, pre, mlp):
    """Sigmoid scores, the `top` largest chosen, weights not renormalised and
    applied to the expert's INPUT. Returns (output, chosen ids)."""
    top = int(mlp["router"]["top"])
    limit = float(mlp["expert"]["limit"])
    s = torch.sigmoid(h @ w[pre + "router"].T)
    vals, ids = s.topk(top, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += clamped_glu((vals[t, j] * h[t])[None], w,
                                  f"{pre}e{e}.", limit)[0]
    return out, ids


def feed_forward(h, w, pre, mlp):
    if mlp.get("kind", "moe" if "router" in mlp else "dense") == "dense":
        return clamped_glu(h, w, pre, float(mlp["limit"]))
    return routed_experts(h, w, pre, mlp)[0]


def forward(cfg, w, tokens, return_layers=False):
    """Logits [n, vocab] of one whole sequence (and the residual stream after
    every layer)."""
    eps = float(cfg["norm"]["eps"])
    x = rms_norm(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    streams = []
    for i, sp in enumerate(cfg["layers"]):
        if sp["type"] != "parallel":
            raise ValueError(sp["type"])
        p = f"l{i}."
        x = x + rms_norm(parallel_mixer(x, w, p + "mix.", sp["mixer"], eps),
                         w[p + "norm1"], eps)
        if sp.get("mlp") is not None:
            x = x + rms_norm(feed_forward(x, w, p + "mlp.", sp["mlp"]),
                             w[p + "norm2"], eps)
        streams.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T * float(cfg["logit_scale"])
    if return_layers:
        return logits, torch.stack(streams)
    return logits


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
    vec("embed.norm", W, 1.0, 0.2)
    vec("final.norm", W, 1.0, 0.2)
    for i, sp in enumerate(cfg["layers"]):
        p = f"l{i}."
        vec(p + "norm1", W, 1.0, 0.2)
        lf, rt = sp["mixer"]["left"], sp["mixer"]["right"]
        H, G = int(lf["heads"]), int(lf.get("kv_heads", lf["heads"]))
        d, dv = int(lf["dim"]), int(lf["vdim"])
        mat(p + "mix.left.q", H * d, W, 2.0)
        mat(p + "mix.left.k", G * d, W, 2.0)
        mat(p + "mix.left.v", G * dv, W)
        vec(p + "mix.left.q.norm", d, 1.0, 0.3)
        vec(p + "mix.left.k.norm", d, 1.0, 0.3)
        vec(p + "mix.left.pb", H, -1.0, 1.0)
        mat(p + "mix.left.g", H, W, 2.0)
        mat(p + "mix.left.o", W, H * dv)
        R = int(rt["width"])
        mat(p + "mix.right.z", R, W, 2.0)
        vec(p + "mix.right.z.b", R, 0.0, 1.0)
        mat(p + "mix.right.x", R, W, 2.0)
        vec(p + "mix.right.x.b", R, 0.0, 0.5)
        mat(p + "mix.right.g", R, W, 2.0)
        mat(p + "mix.right.o", W, R)
        mlp = sp.get("mlp")
        if mlp is None:
            continue
        vec(p + "norm2", W, 1.0, 0.2)
        if mlp.get("kind", "moe" if "router" in mlp else "dense") == "dense":
            ff = int(mlp["ff"])
            mat(p + "mlp.gate", ff, W, 2.0)
            mat(p + "mlp.up", ff, W, 2.0)
            mat(p + "mlp.down", W, ff)
        else:
            ff = int(mlp["expert"]["ff"])
            mat(p + "mlp.router", int(mlp["router"]["experts"]), W, 2.0)
            for e in range(int(mlp["router"]["experts"])):
                mat(f"{p}mlp.e{e}.gate", ff, W, 3.0)
                mat(f"{p}mlp.e{e}.up", ff, W, 3.0)
                mat(f"{p}mlp.e{e}.down", W, ff)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in w.items()}
