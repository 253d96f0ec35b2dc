"""Tedalix, plainly: one slow function per mechanism, in 64-bit on the CPU, sharing no code with the product.

A model is (config, weights): ``config`` the content of a config.json, ``weights`` a dict name -> torch tensor.
Every function takes whole sequences [T, ...] and walks tokens in order where the mechanism has a memory; nothing
is cached, cut or batched here.  Notation: T tokens, W the stream's width, i a query's position, j a key's.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def lin(w, x, b=None):
    y = x.to(F64) @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def unit_rms(x, eps):
    """x over sqrt(mean(x^2) + eps) along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """The row in ``groups`` equal consecutive parts, each brought to unit RMS by itself; the whole times w."""
    t, n = x.shape
    parts = unit_rms(x.to(F64).reshape(t, groups, n // groups), eps)
    return parts.reshape(t, n) * w.to(F64)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def poly_norm(z, coeff, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e with N = unit RMS over the row."""
    a, b, c, e = (float(v) for v in coeff.to(F64))
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def dense_ff(h, w, p, eps):
    z = lin(w[p + "up"], h, w[p + "up.b"])
    return lin(w[p + "down"], poly_norm(z, w[p + "act"], eps), w[p + "down.b"])


def visible(i, j, size, keep_first):
    """Whether the query at i sees the key at j: never ahead; inside the window of ``size`` (0: no window), or among
    the first ``keep_first``."""
    if j > i:
        return False
    return size <= 0 or i - j < size or j < keep_first


def softmax_attention(q, k, v, scale, size=0, keep_first=0, softcap=0.0, slopes=None, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e].  score = q.k * scale, bent to cap * tanh(score / cap) when
    there is a cap, less slope_h * (i - j) when there are slopes; softmax over the visible keys, with exp(sink_h) as
    one more term of the denominator when there is a sink."""
    t, nh, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(t, nh, v.shape[2], dtype=F64)
    for h in range(nh):
        kv = h // (nh // g)
        for i in range(t):
            js = [j for j in range(i + 1) if visible(i, j, size, keep_first)]
            s = (k[js, kv] @ q[i, h]) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if slopes is not None:
                s = s - slopes[h] * torch.tensor([float(i - j) for j in js], dtype=F64)
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h].to(F64))
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h].to(F64) - m) if sink is not None else 0.0)
            out[i, h] = (e[:, None] * v[js, kv]).sum(0) / den
    return out


def distance_slopes(heads):
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=F64)


def window_attention(h, w, p, m, kv=None):
    """The ``attention`` mixer.  ``kv``: keys and values of another layer to read in place of projecting.  Returns
    (output, (keys, values))."""
    t = h.shape[0]
    q = lin(w[p + "q"], h).reshape(t, m["heads"], m["dim"])
    if kv is None:
        kv = (lin(w[p + "k"], h).reshape(t, m["kv_heads"], m["dim"]), lin(w[p + "v"], h).reshape(t, m["kv_heads"], m["vdim"]))
    mask = m.get("mask") or {}
    o = softmax_attention(q, kv[0], kv[1], m["scale"], mask.get("size", 0), mask.get("keep_first", 0))
    return lin(w[p + "o"], o.reshape(t, -1)), kv


def sink_attention(h, w, p, m, eps):
    """The left half of the ``parallel`` mixer."""
    t = h.shape[0]
    q = unit_rms(lin(w[p + "q"], h), eps) * w[p + "q.norm"].to(F64)
    k = unit_rms(lin(w[p + "k"], h), eps) * w[p + "k.norm"].to(F64)
    v = lin(w[p + "v"], h)
    mask = m.get("mask") or {}
    o = softmax_attention(q.reshape(t, m["heads"], m["dim"]), k.reshape(t, m["kv_heads"], m["dim"]),
                          v.reshape(t, m["kv_heads"], m["vdim"]), m["scale"], mask.get("size", 0), mask.get("keep_first", 0),
                          m.get("softcap", 0.0), distance_slopes(m["heads"]), w[p + "sink"])
    o = o * sigmoid(lin(w[p + "g"], h))[:, :, None]
    return lin(w[p + "o"], o.reshape(t, -1))


def short_conv(x, taps_w):
    """y_t[c] = sum_s taps_w[c, s] x_(t - (taps - 1 - s))[c], zeros before the start; then SiLU."""
    t, c = x.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, c, dtype=F64), x.to(F64)])
    y = torch.zeros(t, c, dtype=F64)
    for s in range(taps):
        y = y + padded[s:s + t] * taps_w[:, s].to(F64)
    return silu(y)


def gated_delta(h, w, p, m, eps):
    """The right half of the ``parallel`` mixer."""
    t = h.shape[0]
    nh, g, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv(lin(w[p + "q"], h), w[p + "q.conv"]).reshape(t, g, d)
    k = short_conv(lin(w[p + "k"], h), w[p + "k.conv"]).reshape(t, g, d)
    v = short_conv(lin(w[p + "v"], h), w[p + "v.conv"]).reshape(t, nh, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(lin(w[p + "b"], h))
    rate = torch.exp(w[p + "A_log"].to(F64))
    dt = softplus(lin(w[p + "a2"], lin(w[p + "a1"], h)) + w[p + "dt_bias"].to(F64)).reshape(t, nh, d)
    decay = torch.exp(-rate[None, :, None] * dt)
    o = torch.zeros(t, nh, e, dtype=F64)
    for hd in range(nh):
        kh = hd // (nh // g)
        s = torch.zeros(d, e, dtype=F64)
        for i in range(t):
            s = decay[i, hd][:, None] * s
            u = beta[i, hd] * (v[i, hd] - s.T @ k[i, kh])
            s = s + torch.outer(k[i, kh], u)
            o[i, hd] = s.T @ q[i, kh]
    o = unit_rms(o, eps) * w[p + "norm"].to(F64)
    gate = sigmoid(lin(w[p + "g2"], lin(w[p + "g1"], h))).reshape(t, nh, e)
    return lin(w[p + "o"], (o * gate).reshape(t, -1))


def parallel_mixer(h, w, p, m, eps):
    return m["left_scale"] * sink_attention(h, w, p + "left.", m["left"], eps) + \
        m["right_scale"] * gated_delta(h, w, p + "right.", m["right"], eps)


def rotate_half(x, dims, base, first_position=0):
    """x [T, heads, d]: the first ``dims`` of a head turned, dimension i with i + dims/2, by position * base^(-2i/dims)."""
    t = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = (torch.arange(t, dtype=F64) + first_position)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def retention(h, w, p, m, eps):
    t = h.shape[0]
    nh, d, e = m["heads"], m["dim"], m["vdim"]
    q = lin(w[p + "q"], h).reshape(t, nh, d)
    k = lin(w[p + "k"], h).reshape(t, nh, d)
    v = lin(w[p + "v"], h).reshape(t, nh, e)
    rot = m.get("rot")
    if rot:
        q, k = rotate_half(q, rot["dims"], rot["base"]), rotate_half(k, rot["dims"], rot["base"])
    k = k * d ** -0.5
    o = torch.zeros(t, nh, e, dtype=F64)
    for hd in range(nh):
        s = torch.zeros(d, e, dtype=F64)
        for i in range(t):
            s = m["decay"][hd] * s + torch.outer(k[i, hd], v[i, hd])
            o[i, hd] = s.T @ q[i, hd]
    o = unit_rms(o, eps).reshape(t, -1) * silu(lin(w[p + "g"], h))
    return lin(w[p + "o"], o)


def forward(config, w, tokens, layer_outputs=None):
    """Logits [T, vocab] in 64-bit for one whole sequence.  ``layer_outputs``: a list that receives the stream
    after every layer."""
    eps, groups = config["norm"]["eps"], config["norm"]["groups"]
    x = w["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norm = lambda name, y: group_norm(y, w[p + name], groups, eps)
        h = norm("norm1", x)
        if layer["type"] == "attention":
            y, kept[i] = window_attention(h, w, p + "mix.", m, kept[m["kv_from"]] if m.get("kv_from") is not None else None)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, w, p + "mix.", m, eps)
        elif layer["type"] == "retention":
            y = retention(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + norm("norm1b", y)
        if layer.get("mlp") is not None:
            x = x + norm("norm2b", dense_ff(norm("norm2", x), w, p + "mlp.", eps))
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return lin(w["head"], group_norm(x, w["final.norm"], groups, eps))


# ---- a model of one's own --------------------------------------------------------------------------------------------
def tensor_shapes(config):
    """Name -> shape of every tensor a model of this configuration has."""
    W = config["width"]
    out = {"embed": (config["vocab"], W), "final.norm": (W,), "head": (config["vocab"], W)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        if layer["type"] == "attention":
            out[p + "mix.q"] = (m["heads"] * m["dim"], W)
            if m.get("kv_from") is None:
                out[p + "mix.k"] = (m["kv_heads"] * m["dim"], W)
                out[p + "mix.v"] = (m["kv_heads"] * m["vdim"], W)
            out[p + "mix.o"] = (W, m["heads"] * m["vdim"])
        elif layer["type"] == "parallel":
            a, b = m["left"], m["right"]
            lp, rp = p + "mix.left.", p + "mix.right."
            out.update({lp + "q": (a["heads"] * a["dim"], W), lp + "k": (a["kv_heads"] * a["dim"], W),
                        lp + "v": (a["kv_heads"] * a["vdim"], W), lp + "q.norm": (a["heads"] * a["dim"],),
                        lp + "k.norm": (a["kv_heads"] * a["dim"],), lp + "sink": (a["heads"],), lp + "g": (a["heads"], W),
                        lp + "o": (W, a["heads"] * a["vdim"])})
            qk, vv, r = b["kv_heads"] * b["dim"], b["heads"] * b["vdim"], b.get("rank", max(8, W // 8))
            out.update({rp + "q": (qk, W), rp + "k": (qk, W), rp + "v": (vv, W), rp + "q.conv": (qk, b["conv"]),
                        rp + "k.conv": (qk, b["conv"]), rp + "v.conv": (vv, b["conv"]), rp + "b": (b["heads"], W),
                        rp + "A_log": (b["heads"],), rp + "norm": (b["vdim"],), rp + "a1": (r, W),
                        rp + "a2": (b["heads"] * b["dim"], r), rp + "dt_bias": (b["heads"] * b["dim"],), rp + "g1": (r, W),
                        rp + "g2": (vv, r), rp + "o": (W, vv)})
        else:
            out.update({p + "mix.q": (m["heads"] * m["dim"], W), p + "mix.k": (m["heads"] * m["dim"], W),
                        p + "mix.v": (m["heads"] * m["vdim"], W), p + "mix.g": (m["heads"] * m["vdim"], W),
                        p + "mix.o": (W, m["heads"] * m["vdim"])})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (W,), p + "norm2b": (W,), p + "mlp.up": (ff, W), p + "mlp.up.b": (ff,),
                        p + "mlp.down": (W, ff), p + "mlp.down.b": (W,), p + "mlp.act": (4,)})
    return out


def random_weights(config, seed, dtype=torch.bfloat16):
    """Weights of a size that keeps every layer's output of the order of its input; stored in ``dtype``."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm2", "norm1b", "norm2b", "norm") and len(shape) == 1:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith((".q.norm", ".k.norm")):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif last == "sink":
            t = torch.randn(shape, generator=g)
        elif last == "A_log":
            t = torch.log(0.5 + 4.0 * torch.rand(shape, generator=g))
        elif last == "dt_bias":
            t = torch.randn(shape, generator=g) - 2.0
        elif last == "act":
            t = torch.tensor([0.6, 0.3, 0.2, 0.05]) + 0.05 * torch.randn(4, generator=g)
        elif last == "b" and len(shape) == 1:
            t = 0.1 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        out[name] = t.to(dtype)
    return out


# ---- configurations of the tests' own --------------------------------------------------------------------------------
def _dense(ff):
    return {"kind": "dense", "ff": ff}


def tiny_config_p():
    """Three norm groups; a parallel layer whose delta rule shares key heads and has four taps; windowed attention with
    kept first tokens and values narrower than keys; a retention layer without feed-forward, half of a head turned, a
    decay of 1; a layer that reads the second layer's keys under a wider mask of its own; a mixer-only last layer."""
    return {"architecture": "Tedalix", "vocab": 96, "width": 48, "norm": {"eps": 1e-5, "groups": 3}, "layers": [
        {"type": "parallel", "mlp": _dense(80), "mixer": {
            "left": {"heads": 3, "kv_heads": 1, "dim": 16, "vdim": 24, "scale": 0.2, "softcap": 15.0, "mask": {"size": 20}},
            "right": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "conv": 4, "rank": 8},
            "left_scale": 0.7, "right_scale": 1.1}},
        {"type": "attention", "mlp": _dense(64), "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.25,
                                                          "mask": {"size": 24, "keep_first": 5}}},
        {"type": "retention", "mlp": None, "mixer": {"heads": 3, "dim": 16, "vdim": 8, "decay": [0.9, 0.99, 1.0],
                                                     "rot": {"base": 10000.0, "dims": 8}}},
        {"type": "attention", "mlp": _dense(64), "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.3,
                                                          "kv_from": 1, "mask": {"size": 40, "keep_first": 2}}},
        {"type": "retention", "mlp": None, "mixer": {"heads": 2, "dim": 8, "vdim": 24, "decay": [0.5, 0.97],
                                                     "rot": {"base": 500.0, "dims": 8}}},
    ]}


def tiny_config_q():
    """One norm group; attention under a plain window (no kept tokens) with keys and values of 64, attention that sees
    everything, a retention layer without rotation, a parallel layer of one head each without a score cap, two taps."""
    return {"architecture": "Tedalix", "vocab": 128, "width": 64, "norm": {"eps": 1e-6, "groups": 1}, "layers": [
        {"type": "attention", "mlp": _dense(96), "mixer": {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.125,
                                                          "mask": {"size": 33}}},
        {"type": "retention", "mlp": _dense(32), "mixer": {"heads": 1, "dim": 32, "vdim": 32, "decay": [0.98]}},
        {"type": "parallel", "mlp": None, "mixer": {
            "left": {"heads": 1, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.18, "mask": {"size": 7}},
            "right": {"heads": 1, "kv_heads": 1, "dim": 24, "vdim": 72, "conv": 2, "rank": 4},
            "left_scale": 1.0, "right_scale": 0.5}},
        {"type": "attention", "mlp": _dense(96), "mixer": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 32, "scale": 0.25}},
        {"type": "attention", "mlp": None, "mixer": {"heads": 8, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.11,
                                                     "kv_from": 0, "mask": {"size": 33}}},
    ]}


def tiny_config_r():
    """A width that is no whole 16-byte piece; more first tokens kept than the window is long; a convolution of one tap
    (no carried inputs); a delta rule wider than a wavefront's columns; five query heads."""
    return {"architecture": "Tedalix", "vocab": 70, "width": 36, "norm": {"eps": 1e-6, "groups": 2}, "layers": [
        {"type": "retention", "mlp": _dense(40), "mixer": {"heads": 2, "dim": 12, "vdim": 20, "decay": [0.0, 0.995],
                                                          "rot": {"base": 100.0, "dims": 12}}},
        {"type": "attention", "mlp": None, "mixer": {"heads": 5, "kv_heads": 5, "dim": 24, "vdim": 40, "scale": 0.2,
                                                     "mask": {"size": 8, "keep_first": 30}}},
        {"type": "parallel", "mlp": _dense(44), "mixer": {
            "left": {"heads": 5, "kv_heads": 5, "dim": 8, "vdim": 8, "scale": 0.35, "softcap": 5.0, "mask": {"size": 64}},
            "right": {"heads": 2, "kv_heads": 1, "dim": 48, "vdim": 72, "conv": 1, "rank": 6},
            "left_scale": 1.3, "right_scale": 1.0}},
    ]}
