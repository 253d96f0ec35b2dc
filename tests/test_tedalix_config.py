"""Tedalix without a GPU: its configuration (every error names its key), the specification built from it (a layer
that reads another's keys is one more reader of that layer's cache, a layer of two mixers keeps one cache per mixer),
the masks the caches are kept for, and the plain implementation against itself (each mechanism's own edge: a window,
kept first tokens, a sink, a state carried token by token)."""
import copy

import pytest
import torch

import plain_tedalix as pt
from prelude_amd import models  # noqa: F401  (registers the architectures)
from prelude_amd.cache.manager import peak_pages
from prelude_amd.config.model_config import ConfigError, TedalixConfig
from prelude_amd.config.registry import resolve_architecture
from prelude_amd.models.causal_lm import CausalLM
from prelude_amd.parts.attention import KeptFirstKVCacheSpec
from prelude_amd.parts.base import KVCacheSpec, StateSpec

F64 = torch.float64


def build(cfg):
    arch = resolve_architecture(cfg)
    assert arch.name == "tedalix"
    return CausalLM(arch.build_spec(arch.parse_config(cfg)))


def _set(cfg, path, value=None, delete=False):
    c = copy.deepcopy(cfg)
    d = c
    for k in path[:-1]:
        d = d[k]
    if delete:
        del d[path[-1]]
    else:
        d[path[-1]] = value
    return c


@pytest.mark.parametrize("make", [pt.tiny_config_p, pt.tiny_config_q, pt.tiny_config_r])
def test_the_model_asks_for_the_tensors_a_file_holds(make):
    cfg = make()
    m = build(cfg)
    want = pt.tensor_shapes(cfg)
    got = {k: tuple(v.shape) for k, v in m.tensor_requests().items()}
    assert got == want
    assert m.spec.eos_token_ids == () and m.spec.vocab_size == cfg["vocab"]


def test_the_inner_size_of_the_two_step_projections_is_left_to_the_tensors():
    cfg = pt.tiny_config_p()
    del cfg["layers"][0]["mixer"]["right"]["rank"]
    got = {k: tuple(v.shape) for k, v in build(cfg).tensor_requests().items()}
    assert got["l0.mix.right.a1"] == (-1, 48) and got["l0.mix.right.g2"] == (96, -1)


def test_caches_and_their_readers():
    m = build(pt.tiny_config_p())
    # parallel: keys and values of the left mixer, the state of the right; attention with kept tokens; retention's
    # state; the fourth layer reads the second's keys; retention again
    assert m.run_cache == [(0, 1), 2, 3, 2, 4]
    kinds = [type(c.spec) for c in m.cache_slots]
    assert kinds == [KVCacheSpec, StateSpec, KeptFirstKVCacheSpec, StateSpec, StateSpec]
    # the second layer's cache is kept for the wider of the two masks that read it
    assert m.cache_slots[2].spec == KeptFirstKVCacheSpec(2, 16, 40, 8, 5)
    assert m.cache_slots[0].spec == KVCacheSpec(1, 16, 20, 24)
    names = [t[0] for t in m.cache_slots[1].spec.tensors]
    assert names == ["conv", "s"] and m.cache_slots[1].spec.tensors[0][1] == (2 * 2 * 16 + 4 * 24, 3)
    assert m.needs_state and m.graph_safe_portions
    assert m.blocks[2].KIND == "sandwich_norm_mixer_only" and m.blocks[0].KIND == "sandwich_norm"
    q = build(pt.tiny_config_q())
    assert q.run_cache == [0, 1, (2, 3), 4, 0]
    assert q.cache_slots[4].spec == KVCacheSpec(4, 16, 0, 32), "no mask: every key is kept"
    assert q.cache_slots[0].spec == KVCacheSpec(1, 64, 33, 64)
    r = build(pt.tiny_config_r())
    # more first tokens kept than the window is long: the cache still holds the window beside them
    assert r.cache_slots[1].spec == KeptFirstKVCacheSpec(5, 24, 8, 40, 30)


def test_a_reader_that_sees_everything_keeps_every_key_of_the_layer_it_reads():
    cfg = pt.tiny_config_p()
    del cfg["layers"][3]["mixer"]["mask"]
    m = build(cfg)
    assert m.cache_slots[2].spec == KVCacheSpec(2, 16, 0, 8)
    own = m.spec.layers[1].parts["mixer"].params
    assert (own["window"], own["keep_first"], own["cache_window"]) == (24, 5, 0)


def test_sizes_and_constants_come_from_the_configuration():
    c = TedalixConfig.from_dict(pt.tiny_config_p())
    par, att, ret, rd = c.layers[0].mixer, c.layers[1].mixer, c.layers[2].mixer, c.layers[3].mixer
    assert (par.left_scale, par.right_scale, par.left.softcap, par.left.scale, par.left.mask.size) == (0.7, 1.1, 15.0, 0.2, 20)
    assert (par.right.heads, par.right.kv_heads, par.right.dim, par.right.vdim, par.right.conv, par.right.rank) == (4, 2, 16, 24, 4, 8)
    assert (att.heads, att.kv_heads, att.dim, att.vdim, att.mask.size, att.mask.keep_first, att.kv_from) == (4, 2, 16, 8, 24, 5, None)
    assert (ret.decay, ret.rot_base, ret.rot_dims) == ((0.9, 0.99, 1.0), 10000.0, 8) and c.layers[2].ff == 0
    assert rd.kv_from == 1 and (c.norm_eps, c.norm_groups) == (1e-5, 3)
    spec = build(pt.tiny_config_p()).spec
    left, right = spec.layers[0].parts["mixer"].params["members"]
    assert left["scale"] == 0.7 and right["scale"] == 1.1
    assert left["params"]["score_cap"] == 15.0 and left["params"]["sink"] == "learned" and left["params"]["head_gate"]
    assert left["params"]["slope_exponent"] == 8.0 and left["params"]["qk_norm"] == "whole"
    rp = spec.layers[2].parts["mixer"].params
    assert rp["key_scale"] == 16 ** -0.5 and rp["gate_activation"] == "silu" and rp["head_norm"] and not rp["norm_weight"]
    assert spec.layers[0].parts["pre_mixer_norm"].params == dict(size=48, eps=1e-5, groups=3)
    q = TedalixConfig.from_dict(pt.tiny_config_q())
    assert q.layers[1].mixer.rot_dims == 0 and q.layers[2].mixer.left.softcap == 0.0 and q.layers[3].mixer.mask.size == 0
    assert build(pt.tiny_config_q()).spec.layers[1].parts["mixer"].params["position"] is None


@pytest.mark.parametrize("path,key", [
    (("vocab",), "vocab"), (("width",), "width"), (("norm",), "norm"), (("norm", "eps"), "norm.eps"),
    (("layers", 0, "type"), "type"), (("layers", 0, "mixer"), "layers[0].mixer"),
    (("layers", 0, "mixer", "left"), "layers[0].mixer.left"), (("layers", 0, "mixer", "right", "conv"), "layers[0].mixer.right.conv"),
    (("layers", 0, "mixer", "left", "scale"), "layers[0].mixer.left.scale"), (("layers", 0, "mixer", "left_scale"), "layers[0].mixer.left_scale"),
    (("layers", 0, "mixer", "left", "mask", "size"), "layers[0].mixer.left.mask.size"),
    (("layers", 1, "mixer", "vdim"), "layers[1].mixer.vdim"), (("layers", 1, "mixer", "kv_heads"), "layers[1].mixer.kv_heads"),
    (("layers", 2, "mixer", "decay"), "layers[2].mixer.decay"), (("layers", 2, "mixer", "rot", "base"), "layers[2].mixer.rot.base"),
    (("layers", 0, "mlp", "ff"), "layers[0].mlp.ff"),
])
def test_a_missing_key_is_named(path, key):
    with pytest.raises(ConfigError) as e:
        TedalixConfig.from_dict(_set(pt.tiny_config_p(), path, delete=True))
    assert key in str(e.value), str(e.value)


@pytest.mark.parametrize("path,value,key", [
    (("layers", 0, "type"), "mamba", "type"),
    (("layers", 0, "mlp", "kind"), "moe", "mlp.kind"),
    (("layers", 1, "mixer", "heads"), 3, "heads"),
    (("layers", 0, "mixer", "right", "heads"), 3, "right.heads"),
    (("layers", 2, "mixer", "decay"), [0.5, 0.6], "decay"),
    (("layers", 2, "mixer", "decay"), [0.5, 0.6, 1.5], "decay"),
    (("layers", 2, "mixer", "rot", "dims"), 7, "rot.dims"),
    (("layers", 2, "mixer", "rot", "dims"), 18, "rot.dims"),
    (("layers", 3, "mixer", "kv_from"), 3, "kv_from"),
    (("layers", 3, "mixer", "kv_from"), 0, "kv_from"),
    (("layers", 3, "mixer", "kv_from"), 9, "kv_from"),
    (("layers", 3, "mixer", "dim"), 32, "layer 1"),
    (("layers", 1, "mixer", "kv_from"), 3, "kv_from"),
    (("norm", "groups"), 5, "norm.groups"),
    (("layers", 1, "mixer", "mask", "keep_first"), "six", "keep_first"),
    (("layers", 0, "mixer", "left", "softcap"), -1.0, "softcap"),
])
def test_an_impossible_value_is_named(path, value, key):
    with pytest.raises(ConfigError) as e:
        TedalixConfig.from_dict(_set(pt.tiny_config_p(), path, value))
    assert key in str(e.value), str(e.value)


def test_pages_a_window_with_kept_first_tokens_holds():
    # a request far longer than its window holds the window's pages, the chunk's, and those of the kept positions
    assert peak_pages(10_000, 1, 24, 8) == 4
    assert peak_pages(10_000, 1, 24, 8, keep_first=5) == 5
    assert peak_pages(10_000, 1, 24, 8, keep_first=17) == 7
    assert peak_pages(20, 1, 24, 8, keep_first=17) == 3, "never more than the request's own pages"


# ---- the plain implementation against itself ----------------------------------------------------------------------------
def test_the_mask():
    assert [j for j in range(12) if pt.visible(10, j, 4, 2)] == [0, 1, 7, 8, 9, 10]
    assert [j for j in range(12) if pt.visible(10, j, 4, 0)] == [7, 8, 9, 10]
    assert [j for j in range(5) if pt.visible(3, j, 0, 0)] == [0, 1, 2, 3]
    assert [j for j in range(12) if pt.visible(5, j, 3, 30)] == [0, 1, 2, 3, 4, 5]


def test_a_sink_takes_weight_and_brings_nothing():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(6, 1, 8, generator=g, dtype=F64) for _ in range(3))
    plain = pt.softmax_attention(q, k, v, 0.3)
    low = pt.softmax_attention(q, k, v, 0.3, sink=torch.tensor([-60.0], dtype=F64))
    assert torch.allclose(plain, low, atol=1e-12)
    high = pt.softmax_attention(q, k, v, 0.3, sink=torch.tensor([60.0], dtype=F64))
    assert float(high.abs().max()) < 1e-12
    # the first token alone beside a sink of 0 against a score of 0: half of its value
    z = pt.softmax_attention(torch.zeros(1, 1, 8, dtype=F64), k[:1], v[:1], 0.3, sink=torch.zeros(1, dtype=F64))
    assert torch.allclose(z[0, 0], 0.5 * v[0, 0])


def test_the_bias_by_distance_prefers_near_keys():
    v = torch.eye(5, dtype=F64).reshape(5, 1, 5)
    q = k = torch.zeros(5, 1, 3, dtype=F64)
    o = pt.softmax_attention(q, k, v, 1.0, slopes=torch.tensor([0.5], dtype=F64))[4, 0]
    want = torch.exp(-0.5 * torch.tensor([4.0, 3.0, 2.0, 1.0, 0.0], dtype=F64))
    assert torch.allclose(o, want / want.sum())


def test_the_delta_rule_stores_and_overwrites():
    """With no decay and a gate of one, writing (k, v) and reading with q = k gives v back; writing (k, v2) then
    replaces it: u = v2 - S^T k takes the old value off."""
    d, e = 4, 3
    k = torch.tensor([1.0, 0, 0, 0], dtype=F64)
    s = torch.zeros(d, e, dtype=F64)
    v1, v2 = torch.tensor([1.0, 2, 3], dtype=F64), torch.tensor([-1.0, 0, 5], dtype=F64)
    for v in (v1, v2):
        u = 1.0 * (v - s.T @ k)
        s = s + torch.outer(k, u)
        assert torch.allclose(s.T @ k, v)


def test_retention_in_its_sum_form():
    """o_i = sum_(j <= i) decay^(i - j) (q_i . k_j) v_j: the recurrence unrolled, through the plain mixer."""
    cfg = {"heads": 1, "dim": 4, "vdim": 4, "decay": [0.8]}
    g = torch.Generator().manual_seed(1)
    w = {n: torch.randn(4, 6, generator=g, dtype=F64) for n in ("q", "k", "v", "g")}
    w["o"] = torch.eye(4, dtype=F64)[:, :4]
    w = {"m." + n: t for n, t in w.items()}
    w["m.o"] = torch.randn(6, 4, generator=g, dtype=F64)
    h = torch.randn(7, 6, generator=g, dtype=F64)
    got = pt.retention(h, w, "m.", cfg, 1e-6)
    q, k, v = pt.lin(w["m.q"], h), pt.lin(w["m.k"], h) * 0.5, pt.lin(w["m.v"], h)
    o = torch.stack([sum(0.8 ** (i - j) * (q[i] @ k[j]) * v[j] for j in range(i + 1)) for i in range(7)])
    want = pt.lin(w["m.o"], pt.unit_rms(o, 1e-6) * pt.silu(pt.lin(w["m.g"], h)))
    assert torch.allclose(got, want, atol=1e-10)


def test_rotation_keeps_lengths_and_depends_on_the_difference_of_positions():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 1, 12, generator=g, dtype=F64).expand(9, 1, 12)
    r = pt.rotate_half(x, 8, 100.0)
    assert torch.allclose(r.norm(dim=-1), x.norm(dim=-1)) and torch.equal(r[..., 8:], x[..., 8:])
    assert torch.allclose(r[0], x[0])
    dots = [float(r[i, 0] @ r[i + 3, 0]) for i in range(5)]
    assert max(dots) - min(dots) < 1e-12
    shifted = pt.rotate_half(x[:4], 8, 100.0, first_position=5)
    assert torch.allclose(shifted, r[5:9])


def test_groups_are_normed_by_themselves():
    x = torch.cat([torch.full((1, 4), 3.0), torch.full((1, 4), -0.01)], dim=1).to(F64)
    y = pt.group_norm(x, torch.ones(8), 2, 1e-12)
    assert torch.allclose(y.abs(), torch.ones(1, 8, dtype=F64), atol=1e-6)
    one = pt.group_norm(x, torch.ones(8), 1, 1e-12)
    assert float(one[0, 4].abs()) < 0.01


def test_the_polynomial_activation():
    z = torch.tensor([[1.0, -2.0, 3.0, 0.5]], dtype=F64)
    got = pt.poly_norm(z, torch.tensor([0.5, 0.25, 2.0, -0.1]), 0.0)
    n = lambda u: u / u.pow(2).mean().sqrt()
    assert torch.allclose(got, 0.5 * n(z) + 0.25 * n(z ** 2) + 2.0 * n(z ** 3) - 0.1)
