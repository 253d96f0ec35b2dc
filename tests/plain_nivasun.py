"""Nivasun, plainly: one function per mechanism, in 64-bit, token by token where that is the clearest form.

Nothing here is shared with the product: no kernels, no parts, no cache.  A model is ``(cfg, w)``: the configuration as
the dictionary a config.json holds, and the tensors by name as float64 arrays.

The design.  x = embed[token] * scale + bigram[(prev * mul_prev + token * mul_cur) mod buckets] (row ``buckets`` for a
sequence's first token).  Layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row with the same weights,
``loop.step[t]`` added to x in front of pass t.  A layer: h = x / rms(x) * g (one number g); the mixer reads
h + conv(h) (a causal convolution over time per channel), the feed-forward h; x <- x + mixer + ff.  Mixers: attention
with the keys as values, rotation in halves, a temperature and a sink per head; attention through a latent with a gate
on the heads' outputs; differential attention (two maps over the same values, rotation in pairs).  All under a
sliding window.  Feed-forward: routed experts (softmax over the chosen logits) and a gated shared expert.  The head's
logits are capped by a tanh.
"""
import math

import numpy as np


def rms_unit(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def embed(tokens, table, scale, bigram, buckets, mul_prev, mul_cur):
    """Rows of ``table`` times ``scale`` plus the bigram row of (previous token, token)."""
    out = np.zeros((len(tokens), table.shape[1]))
    for t, tok in enumerate(tokens):
        row = buckets if t == 0 else (tokens[t - 1] * mul_prev + tok * mul_cur) % buckets
        out[t] = table[tok] * scale + bigram[row]
    return out


def time_conv(h, w):
    """conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the start.  h [T, C], w [C, taps]."""
    T, taps = h.shape[0], w.shape[1]
    out = np.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate(x, positions, dims, base, layout):
    """Turns the first ``dims`` dimensions of the last axis of x [T, heads, d].  ``layout`` 'halves': dimension i goes
    with i + dims/2; 'pairs': 2i with 2i + 1.  The pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2i/dims)."""
    out = x.copy()
    half = dims // 2
    for i in range(half):
        f = base ** (-2.0 * i / dims)
        a, b = (i, i + half) if layout == "halves" else (2 * i, 2 * i + 1)
        for t, p in enumerate(positions):
            c, s = math.cos(p * f), math.sin(p * f)
            u, v = x[t, :, a], x[t, :, b]
            out[t, :, a] = u * c - v * s
            out[t, :, b] = v * c + u * s
    return out


def windowed_softmax_sum(q, k, v, scale, window, sink=None):
    """One head.  q [T, d], k [T, d], v [T, dv]; the query at i sees the keys at j with 0 <= i - j < window; ``sink``:
    one more term exp(sink) of the denominator that brings no value."""
    T = q.shape[0]
    out = np.zeros((T, v.shape[1]))
    for i in range(T):
        lo = max(0, i - window + 1)
        s = (k[lo:i + 1] @ q[i]) * scale
        m = s.max() if sink is None else max(s.max(), sink)
        e = np.exp(s - m)
        den = e.sum() + (0.0 if sink is None else math.exp(sink - m))
        out[i] = (e / den) @ v[lo:i + 1]
    return out


def sink_attention(h, positions, w, m):
    """Grouped-query attention whose values are the keys as projected (unrotated), rotation in halves, score times
    scale times the head's temperature, a learned sink."""
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = k
    rot = m.get("rot")
    if rot and rot["dims"]:
        q = rotate(q, positions, rot["dims"], rot["base"], "halves")
        k = rotate(k, positions, rot["dims"], rot["base"], "halves")
    o = np.zeros((T, H, d))
    for a in range(H):
        g = a // (H // G)
        o[:, a] = windowed_softmax_sum(q[:, a], k[:, g], v[:, g], m["scale"] * w["temp"][a], m["mask"]["size"], w["sink"][a])
    return o.reshape(T, H * d) @ w["o"].T


def latent_attention(h, w, m, eps):
    """Queries through a normed latent, keys and values of every head from one normed latent a token, no positions,
    a sigmoid gate on the heads' outputs."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    cq = rms_unit(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(T, H, d)
    c = rms_unit(h @ w["dkv"].T, eps) * w["dkv.norm"]
    k = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for a in range(H):
        o[:, a] = windowed_softmax_sum(q[:, a], k[:, a], v[:, a], m["scale"], m["mask"]["size"])
    return (o.reshape(T, H * dv) * sigmoid(h @ w["g"].T)) @ w["o"].T


def differential_attention(h, positions, w, m, eps):
    """Two attention maps a head over the same values; o = a1 - lambda a2, each head over its own root mean square,
    times 1 - diff."""
    H, G, d, dv, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["diff"]
    T = h.shape[0]
    q = (h @ w["q"].T).reshape(T, H * 2, d)
    k = (h @ w["k"].T).reshape(T, G * 2, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q = rotate(q, positions, rot["dims"], rot["base"], "pairs")
        k = rotate(k, positions, rot["dims"], rot["base"], "pairs")
    lam = math.exp(float(w["lq1"] @ w["lk1"])) - math.exp(float(w["lq2"] @ w["lk2"])) + diff
    o = np.zeros((T, H, dv))
    for a in range(H):
        g = a // (H // G)
        a1 = windowed_softmax_sum(q[:, 2 * a], k[:, 2 * g], v[:, g], m["scale"], m["mask"]["size"])
        a2 = windowed_softmax_sum(q[:, 2 * a + 1], k[:, 2 * g + 1], v[:, g], m["scale"], m["mask"]["size"])
        o[:, a] = rms_unit(a1 - lam * a2, eps) * (1.0 - diff)
    return o.reshape(T, H * dv) @ w["o"].T


def gated_expert(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def routed_experts(h, w, f):
    """The ``top`` experts with the largest router logits, weighted by the softmax over those logits alone, plus the
    shared expert times sigmoid(w_sg . h)."""
    n, top = f["router"]["experts"], f["router"]["top"]
    z = h @ w["router"].T + w["router.b"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(n), key=lambda e: (-z[t, e], e))[:top]
        e = np.exp(z[t, order] - z[t, order].max())
        p = e / e.sum()
        for weight, ex in zip(p, order):
            out[t] += weight * gated_expert(h[t], w[f"e{ex}.gate"], w[f"e{ex}.up"], w[f"e{ex}.down"])
    if f.get("shared"):
        out += gated_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"]) * sigmoid(h @ w["shared.sg"].T)
    return out


def sub(w, prefix):
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def layer(x, positions, cfg, w, i):
    lc, eps = cfg["layers"][i], cfg["norm"]["eps"]
    p = f"l{i}."
    h = rms_unit(x, eps) * w[p + "norm1"]
    hm = h + time_conv(h, w[p + "canon1"])
    mw, m = sub(w, p + "mix."), lc["mixer"]
    if lc["type"] == "attention":
        y = sink_attention(hm, positions, mw, m)
    elif lc["type"] == "latent_attention":
        y = latent_attention(hm, mw, m, eps)
    elif lc["type"] == "attention_2":
        y = differential_attention(hm, positions, mw, m, eps)
    else:
        raise ValueError(lc["type"])
    if lc.get("mlp"):
        y = y + routed_experts(h, sub(w, p + "mlp."), lc["mlp"])
    return x + y


def run_order(cfg):
    """(layer, pass) in the order they run; pass is None outside the loop."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        out += [(i, t) for i in range(loop["start"], loop["stop"])]
    return out + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, w, tokens, streams=None):
    """Logits [T, vocab] of a whole sequence; ``streams`` (a list) receives x after every layer run."""
    e = cfg["embedding"]
    b = e["bigram"]
    x = embed(tokens, w["embed"], e["scale"], w["bigram"], b["buckets"], b["mul_prev"], b["mul_cur"])
    positions = list(range(len(tokens)))
    loop = cfg.get("loop")
    for i, t in run_order(cfg):
        if t is not None and i == loop["start"]:
            x = x + w["loop.step"][t]
        x = layer(x, positions, cfg, w, i)
        if streams is not None:
            streams.append(x.copy())
    z = (rms_unit(x, cfg["norm"]["eps"]) * w["final.norm"]) @ w["head"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z
