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


# ---- configurations and weights of the tests' own --------------------------------------------------------------------------
def _moe(ff, experts, top, shared):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def sink_layer(heads=4, kv_heads=2, dim=16, window=24, rot=8, base=10000.0, scale=0.25, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "mask": {"size": window}}
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent_layer(heads=3, dim=16, vdim=24, kv_rank=40, q_rank=24, window=20, scale=0.2, mlp=None):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                      "mask": {"size": window}}}


def diff_layer(heads=4, kv_heads=2, dim=8, vdim=24, window=18, rot=4, base=5000.0, scale=0.3, diff=0.25, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff, "mask": {"size": window}}
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def model(layers, width=48, vocab=90, loop=None, taps=3, buckets=37, mul_prev=5, mul_cur=11, scale=3.0, cap=8.0, eps=1e-5):
    cfg = {"architecture": "Nivasun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
           "embedding": {"scale": scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}},
           "layers": layers, "logit_softcap": cap}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tiny_config_p():
    """Every mixer once, the two in the middle run three times; heads over fewer KV heads; three taps."""
    return model([sink_layer(mlp=_moe(24, 6, 2, 40)), latent_layer(mlp=_moe(16, 4, 1, 0)), diff_layer(mlp=None),
                  sink_layer(heads=2, kv_heads=1, dim=32, window=40, rot=32, mlp=_moe(24, 5, 5, 24))],
                 loop=(1, 3, 3))


def tiny_config_q():
    """The whole model looped twice; heads of 64 (a size the matrix cores take); every expert chosen; two taps."""
    return model([diff_layer(heads=2, kv_heads=2, dim=32, vdim=64, window=33, rot=16, mlp=_moe(32, 3, 3, 16)),
                  sink_layer(heads=4, kv_heads=4, dim=64, window=70, rot=64, mlp=_moe(32, 8, 3, 16)),
                  latent_layer(heads=2, dim=64, vdim=64, kv_rank=64, q_rank=32, window=50, mlp=_moe(32, 8, 2, 16))],
                 width=64, vocab=120, loop=(0, 3, 2), taps=2, buckets=64, mul_prev=1, mul_cur=1, cap=30.0)


def tiny_config_r():
    """No loop, one tap (the convolution is a number a channel), no rotation anywhere, windows of one and two keys, a width that is
    no whole 16-byte pieces."""
    return model([latent_layer(heads=1, dim=8, vdim=8, kv_rank=12, q_rank=12, window=1, mlp=_moe(12, 2, 1, 12)),
                  sink_layer(heads=3, kv_heads=3, dim=12, window=2, rot=0, mlp=None),
                  diff_layer(heads=1, kv_heads=1, dim=12, vdim=12, window=64, rot=0, diff=0.6, mlp=_moe(12, 2, 2, 0))],
                 width=36, vocab=50, loop=None, taps=1, buckets=7, mul_prev=0, mul_cur=3, cap=0.0)


def tensor_shapes(cfg):
    """Tensor name -> shape, as the design's files hold them."""
    h, v = cfg["width"], cfg["vocab"]
    t = {"embed": (v, h), "bigram": (cfg["embedding"]["bigram"]["buckets"] + 1, h), "final.norm": (), "head": (v, h)}
    if cfg.get("loop"):
        t["loop.step"] = (cfg["loop"]["times"], h)
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        t[p + "norm1"] = ()
        t[p + "canon1"] = (h, cfg["canon"]["taps"])
        H, d = m["heads"], m["dim"]
        if lc["type"] == "attention":
            G = m["kv_heads"]
            t.update({p + "mix.q": (H * d, h), p + "mix.k": (G * d, h), p + "mix.temp": (H,), p + "mix.sink": (H,),
                      p + "mix.o": (h, H * d)})
        elif lc["type"] == "latent_attention":
            dv, r, rq = m["vdim"], m["kv_rank"], m["q_rank"]
            t.update({p + "mix.dq": (rq, h), p + "mix.dq.norm": (rq,), p + "mix.uq": (H * d, rq), p + "mix.dkv": (r, h),
                      p + "mix.dkv.norm": (r,), p + "mix.uk": (H * d, r), p + "mix.uv": (H * dv, r), p + "mix.g": (H * dv, h),
                      p + "mix.o": (h, H * dv)})
        else:
            G, dv = m["kv_heads"], m["vdim"]
            t.update({p + "mix.q": (H * 2 * d, h), p + "mix.k": (G * 2 * d, h), p + "mix.v": (G * dv, h), p + "mix.o": (h, H * dv)})
            t.update({p + "mix." + n: (d,) for n in ("lq1", "lk1", "lq2", "lk2")})
        f = lc.get("mlp")
        if f:
            ff, n = f["expert"]["ff"], f["router"]["experts"]
            t.update({p + "mlp.router": (n, h), p + "mlp.router.b": (n,)})
            for e in range(n):
                t.update({f"{p}mlp.e{e}.gate": (ff, h), f"{p}mlp.e{e}.up": (ff, h), f"{p}mlp.e{e}.down": (h, ff)})
            if f.get("shared"):
                s = f["shared"]["ff"]
                t.update({p + "mlp.shared.gate": (s, h), p + "mlp.shared.up": (s, h), p + "mlp.shared.down": (h, s),
                          p + "mlp.shared.sg": (1, h)})
    return t


def random_weights(cfg, seed):
    """Weights that bfloat16 holds exactly, as float64 arrays: matrices N(0, 1/sqrt(inputs)), norm weights and
    temperatures around 1, sinks, router biases and the loop's vectors of a size that shows."""
    import torch
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm1", "norm") or name.endswith(".temp"):
            x = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last in ("sink", "b"):
            x = 0.7 * torch.randn(shape, generator=g)
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            x = 0.3 * torch.randn(shape, generator=g)
        elif last == "canon1":
            x = 0.4 * torch.randn(shape, generator=g)
        elif name in ("loop.step", "bigram"):
            x = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            x = 0.4 * torch.randn(shape, generator=g)
        else:
            x = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        w[name] = x.to(torch.bfloat16).to(torch.float64).numpy()
    return w
