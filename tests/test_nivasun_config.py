"""Nivasun without a GPU: its configuration (every key's absence and every impossible value named), the specification
built from it (tensor names and shapes against the plain implementation's own list, the run order of a looped stretch,
caches and state per run), and the plain implementation against itself."""
import copy
import math

import numpy as np
import pytest

import plain_nivasun as pn
from prelude_amd import models  # noqa: F401
from prelude_amd.config import ConfigError, NivasunConfig
from prelude_amd.config.registry import resolve_architecture
from prelude_amd.models.causal_lm import CausalLM
from prelude_amd.models.nivasun import nivasun_spec, run_order

CONFIGS = [pn.tiny_config_p, pn.tiny_config_q, pn.tiny_config_r]


def build(cfg):
    arch = resolve_architecture(cfg)
    assert arch.name == "nivasun"
    return CausalLM(arch.build_spec(arch.parse_config(cfg)))


@pytest.mark.parametrize("make", CONFIGS)
def test_the_model_asks_for_the_tensors_a_file_holds(make):
    cfg = make()
    req = build(cfg).tensor_requests()
    want = pn.tensor_shapes(cfg)
    assert set(req) == set(want)
    for name, shape in want.items():
        assert tuple(req[name].shape) == tuple(shape), name


def test_the_run_order_of_a_looped_stretch():
    cfg = NivasunConfig.from_dict(pn.tiny_config_p())
    assert run_order(cfg) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert [(i, t) for i, t in run_order(cfg)] == [(i, t if i == 1 else None) for i, t in pn.run_order(pn.tiny_config_p())]
    spec = nivasun_spec(cfg)
    assert [r.layer for r in spec.order] == [0, 1, 2, 1, 2, 1, 2, 3] and spec.stream_rows == ("loop.step", 3)
    whole = NivasunConfig.from_dict(pn.tiny_config_q())
    assert [i for i, _ in run_order(whole)] == [0, 1, 2, 0, 1, 2]
    none = NivasunConfig.from_dict(pn.tiny_config_r())
    assert run_order(none) == [(0, None), (1, None), (2, None)] and nivasun_spec(none).stream_rows is None
    empty = pn.tiny_config_r()
    empty["loop"] = {"start": 2, "stop": 2, "times": 4}
    assert [i for i, _ in run_order(NivasunConfig.from_dict(empty))] == [0, 1, 2]
    assert build(empty).tensor_requests()["loop.step"].shape == (4, 36)     # the file holds them all the same
    tail = pn.tiny_config_r()
    tail["loop"] = {"start": 2, "stop": 3, "times": 2}
    assert run_order(NivasunConfig.from_dict(tail)) == [(0, None), (1, None), (2, 0), (2, 1)]


def test_every_run_has_caches_and_state_of_its_own():
    m = build(pn.tiny_config_p())
    # the embedding's previous token, then per run the convolution's inputs and the mixer's pages
    assert m.embedding_cache == 0 and m.cache_slots[0].run == -1
    assert m.run_cache == [(1, 2), (3, 4), (5, 6), (7, 8), (9, 10), (11, 12), (13, 14), (15, 16)]
    kinds = [type(c.spec).__name__ for c in m.cache_slots]
    assert kinds[1::2] == ["StateSpec"] * 8
    assert kinds[2::2] == ["KVCacheSpec", "LatentCacheSpec", "SharedValueKVCacheSpec", "LatentCacheSpec", "SharedValueKVCacheSpec",
                           "LatentCacheSpec", "SharedValueKVCacheSpec", "KVCacheSpec"]
    assert m.cache_slots[2].spec.window == 24 and m.cache_slots[16].spec.window == 40
    d = m.cache_slots[6].spec
    assert (d.num_kv_heads, d.num_value_heads, d.head_dim, d.v_dim) == (4, 2, 8, 24)
    assert m.needs_state and m.graph_safe and m.graph_safe_portions
    one_tap = build(pn.tiny_config_r())      # one tap: nothing to carry, the mixers' pages alone
    assert [type(c.spec).__name__ for c in one_tap.cache_slots] == ["StateSpec", "LatentCacheSpec", "KVCacheSpec", "SharedValueKVCacheSpec"]


def _without(cfg, path):
    cfg = copy.deepcopy(cfg)
    node = cfg
    for k in path[:-1]:
        node = node[k]
    del node[path[-1]]
    return cfg


def _with(cfg, path, value):
    cfg = copy.deepcopy(cfg)
    node = cfg
    for k in path[:-1]:
        node = node[k]
    node[path[-1]] = value
    return cfg


@pytest.mark.parametrize("path,named", [
    (("vocab",), "vocab"), (("width",), "width"), (("norm",), "norm"), (("norm", "eps"), "norm.eps"), (("canon",), "canon"),
    (("canon", "taps"), "canon.taps"), (("embedding",), "embedding"), (("embedding", "bigram"), "embedding.bigram"),
    (("embedding", "bigram", "buckets"), "embedding.bigram.buckets"), (("embedding", "bigram", "mul_prev"), "embedding.bigram.mul_prev"),
    (("layers",), "layers"), (("layers", 0, "type"), "type"), (("layers", 0, "mixer"), "layers[0].mixer"),
    (("layers", 0, "mixer", "heads"), "layers[0].mixer.heads"), (("layers", 0, "mixer", "kv_heads"), "layers[0].mixer.kv_heads"),
    (("layers", 0, "mixer", "scale"), "layers[0].mixer.scale"), (("layers", 0, "mixer", "mask"), "layers[0].mixer.mask"),
    (("layers", 0, "mixer", "mask", "size"), "layers[0].mixer.mask.size"), (("layers", 0, "mixer", "rot", "base"), "layers[0].mixer.rot.base"),
    (("layers", 1, "mixer", "kv_rank"), "layers[1].mixer.kv_rank"), (("layers", 1, "mixer", "q_rank"), "layers[1].mixer.q_rank"),
    (("layers", 1, "mixer", "vdim"), "layers[1].mixer.vdim"), (("layers", 2, "mixer", "diff"), "diff"),
    (("layers", 2, "mixer", "vdim"), "layers[2].mixer.vdim"), (("layers", 0, "mlp", "router"), "layers[0].mlp.router"),
    (("layers", 0, "mlp", "router", "top"), "layers[0].mlp.router.top"), (("layers", 0, "mlp", "expert"), "layers[0].mlp.expert"),
    (("loop", "times"), "loop.times"), (("loop", "start"), "start")])
def test_a_missing_key_is_named(path, named):
    with pytest.raises(ConfigError, match=named.replace("[", r"\[").replace("]", r"\]").replace(".", r"\.")):
        NivasunConfig.from_dict(_without(pn.tiny_config_p(), path))


@pytest.mark.parametrize("path,value,named", [
    (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"), (("layers", 0, "mixer", "rot", "dims"), 7, "rot.dims"),
    (("layers", 0, "mixer", "rot", "dims"), 18, "rot.dims"), (("layers", 0, "mixer", "vdim"), 8, "vdim"),
    (("layers", 0, "type"), "retention", "type"), (("layers", 0, "mlp", "router", "top"), 7, "router.top"),
    (("layers", 0, "mlp", "kind"), "dense", "kind"), (("loop", "stop"), 5, "loop"), (("loop", "start"), 4, "loop"),
    (("logit_softcap",), -1.0, "logit_softcap"), (("canon", "taps"), 0, "canon.taps"), (("layers",), [], "layers"),
    (("layers", 2, "mixer", "mask", "size"), 0, "mask.size")])
def test_an_impossible_value_is_named(path, value, named):
    with pytest.raises(ConfigError, match=named.replace(".", r"\.")):
        NivasunConfig.from_dict(_with(pn.tiny_config_p(), path, value))


def test_what_may_go_unsaid():
    cfg = pn.tiny_config_p()
    c = NivasunConfig.from_dict(_without(_without(cfg, ("loop",)), ("logit_softcap",)))
    assert (c.loop_start, c.loop_stop, c.loop_times, c.logit_cap) == (0, 0, 1, 0.0)
    c = NivasunConfig.from_dict(_without(cfg, ("layers", 0, "mixer", "rot")))
    assert c.layers[0].mixer.rot_dims == 0
    c = NivasunConfig.from_dict(_without(cfg, ("layers", 0, "mixer", "vdim")))      # the values are the keys
    assert c.layers[0].mixer.vdim == c.layers[0].mixer.dim
    assert c.layers[2].mlp is None and c.layers[1].mlp.shared_ff == 0 and c.layers[0].mlp.shared_ff == 40


# ---- the plain implementation against itself -------------------------------------------------------------------------------
def test_rotation_layouts_and_relative_positions():
    g = np.random.default_rng(0)
    x = g.standard_normal((5, 2, 12))
    for layout in ("halves", "pairs"):
        y = pn.rotate(x, [3, 4, 5, 6, 7], 8, 100.0, layout)
        assert np.allclose(y[..., 8:], x[..., 8:]) and np.allclose((y ** 2).sum(-1), (x ** 2).sum(-1))
        assert np.allclose(pn.rotate(x, [0] * 5, 8, 100.0, layout), x)
        # q.k depends on the distance alone
        a = pn.rotate(x[:1], [10], 8, 100.0, layout)[0, 0] @ pn.rotate(x[1:2], [7], 8, 100.0, layout)[0, 0]
        b = pn.rotate(x[:1], [110], 8, 100.0, layout)[0, 0] @ pn.rotate(x[1:2], [107], 8, 100.0, layout)[0, 0]
        assert abs(a - b) < 1e-9
    h = pn.rotate(x, [1] * 5, 4, 100.0, "halves")
    p = pn.rotate(x, [1] * 5, 4, 100.0, "pairs")
    assert np.allclose(h[..., 0], x[..., 0] * math.cos(1) - x[..., 2] * math.sin(1))
    assert np.allclose(p[..., 0], x[..., 0] * math.cos(1) - x[..., 1] * math.sin(1))
    assert np.allclose(p[..., 3], x[..., 3] * math.cos(0.1) + x[..., 2] * math.sin(0.1))


def test_time_convolution_is_a_sum_of_shifts():
    g = np.random.default_rng(1)
    h, w = g.standard_normal((9, 4)), g.standard_normal((4, 3))
    want = w[:, 2] * h
    want[1:] += w[:, 1] * h[:-1]
    want[2:] += w[:, 0] * h[:-2]
    assert np.allclose(pn.time_conv(h, w), want)
    assert np.allclose(pn.time_conv(h, w[:, :1]), w[:, 0] * h)


def test_window_and_sink():
    g = np.random.default_rng(2)
    q, k, v = g.standard_normal((30, 6)), g.standard_normal((30, 6)), g.standard_normal((30, 5))
    full = pn.windowed_softmax_sum(q, k, v, 0.4, 1000)
    s = (q @ k.T) * 0.4
    s[np.triu_indices(30, 1)] = -np.inf
    p = np.exp(s - s.max(1, keepdims=True))
    assert np.allclose(full, (p / p.sum(1, keepdims=True)) @ v)
    assert np.allclose(pn.windowed_softmax_sum(q, k, v, 0.4, 1), v)              # a window of one: the token's own value
    w7 = pn.windowed_softmax_sum(q, k, v, 0.4, 7)
    assert np.allclose(w7[:7], full[:7]) and not np.allclose(w7[7], full[7])
    k2 = k.copy()
    k2[10] += 5.0                                                                     # the key at 10 is seen by 10 .. 16 only
    moved = np.abs(pn.windowed_softmax_sum(q, k2, v, 0.4, 7) - w7).max(1)
    assert (moved[10:17] > 0).all() and (moved[:10] == 0).all() and (moved[17:] == 0).all()
    sunk = pn.windowed_softmax_sum(q, k, v, 0.4, 7, sink=-50.0)
    assert np.allclose(sunk, w7)
    half = pn.windowed_softmax_sum(q[:1], k[:1], v[:1], 0.4, 7, sink=float(q[0] @ k[0] * 0.4))
    assert np.allclose(half, 0.5 * v[:1])                                             # a sink as large as the only score


def test_experts_with_every_expert_chosen_are_a_softmax_mixture():
    cfg = pn.model([pn.sink_layer(mlp=pn._moe(8, 3, 3, 8))], width=16)
    w = pn.sub(pn.random_weights(cfg, 3), "l0.mlp.")
    h = np.random.default_rng(3).standard_normal((4, 16))
    z = h @ w["router"].T + w["router.b"]
    p = np.exp(z) / np.exp(z).sum(1, keepdims=True)
    want = sum(p[:, e:e + 1] * pn.gated_expert(h, w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"]) for e in range(3))
    want = want + pn.gated_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"]) * pn.sigmoid(h @ w["shared.sg"].T)
    assert np.allclose(pn.routed_experts(h, w, cfg["layers"][0]["mlp"]), want)
    one = dict(cfg["layers"][0]["mlp"], router={"experts": 3, "top": 1}, shared=None)
    best = z.argmax(1)
    got = pn.routed_experts(h, w, one)
    for t in range(4):
        e = best[t]
        assert np.allclose(got[t], pn.gated_expert(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"]))


def test_two_equal_maps_cancel_up_to_lambda():
    """With both maps' projections equal, a1 = a2 and the head's output is a1 (1 - lambda) normed: a unit-RMS vector
    times 1 - diff, its sign that of 1 - lambda."""
    m = pn.diff_layer(heads=2, kv_heads=1, dim=4, vdim=6, rot=0, diff=0.25)["mixer"]
    g = np.random.default_rng(4)
    q1, k1 = g.standard_normal((2, 4, 10)), g.standard_normal((1, 4, 10))
    w = {"q": np.concatenate([q1[:1], q1[:1], q1[1:], q1[1:]]).reshape(16, 10), "k": np.concatenate([k1, k1]).reshape(8, 10),
         "v": g.standard_normal((6, 10)), "o": np.eye(12), "lq1": np.zeros(4), "lk1": np.zeros(4), "lq2": np.ones(4) * 0.5, "lk2": np.ones(4)}
    h = g.standard_normal((7, 10))
    lam = 1.0 - math.exp(2.0) + 0.25
    out = pn.differential_attention(h, list(range(7)), w, m, 0.0).reshape(7, 2, 6)
    a1 = pn.windowed_softmax_sum(h @ q1[0].T, h @ k1[0].T, h @ w["v"].T, m["scale"], m["mask"]["size"])
    assert np.allclose(out[:, 0], pn.rms_unit(a1 * (1 - lam), 0.0) * 0.75)
    assert np.allclose((out ** 2).mean(-1), 0.75 ** 2)


def test_the_embedding_and_the_loop():
    cfg = pn.tiny_config_p()
    w = pn.random_weights(cfg, 5)
    toks = [3, 70, 70, 12]
    e = cfg["embedding"]
    x = pn.embed(toks, w["embed"], e["scale"], w["bigram"], 37, 5, 11)
    assert np.allclose(x[0], w["embed"][3] * 3.0 + w["bigram"][37])
    assert np.allclose(x[2], w["embed"][70] * 3.0 + w["bigram"][(70 * 5 + 70 * 11) % 37])
    streams = []
    pn.forward(cfg, w, toks, streams)
    assert len(streams) == 8
    w2 = dict(w)
    w2["loop.step"] = w["loop.step"].copy()
    w2["loop.step"][2] += 1.0                        # the third pass's vector: the runs before it are as they were
    other = []
    pn.forward(cfg, w2, toks, other)
    assert all(np.array_equal(a, b) for a, b in zip(streams[:5], other[:5])) and not np.allclose(streams[5], other[5])
    # a logit cap bounds the logits
    assert np.abs(pn.forward(cfg, w, toks)).max() < cfg["logit_softcap"]


def test_what_the_edge_tests_rest_on():
    """A changed token moves the plain logits at the window's oldest key through the convolution's oldest tap, and not at
    all one place further back; a token far back reaches the end through the runs' windows one after the other."""
    for make, over, taps in ((pn.sink_layer, dict(window=24), 1), (pn.latent_layer, dict(window=64), 2), (pn.diff_layer, dict(window=18), 1),
                             (pn.diff_layer, dict(window=65, dim=32, vdim=64, rot=8), 4)):
        cfg = pn.model([make(**over)], taps=taps, loop=None)
        w = pn.random_weights(cfg, 60)
        n = 2 * over["window"] + 21
        toks = list(np.random.default_rng(61).integers(0, cfg["vocab"], n))
        ref = pn.forward(cfg, w, toks)[-1]
        oldest = n - over["window"]
        for c, moves in ((oldest - taps, True), (oldest - taps - 1, False)):
            t = list(toks)
            t[c] = (t[c] + 1 + c) % cfg["vocab"]
            moved = np.abs(pn.forward(cfg, w, t)[-1] - ref).max()
            assert (moved > 1e-4 * ref.std()) == moves and (moves or moved == 0.0), (make.__name__, c, moved)
