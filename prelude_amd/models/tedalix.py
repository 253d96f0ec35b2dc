"""Tedalix: from its typed configuration to a model specification.

A decoder whose layers are listed one by one in the configuration.  Every branch has a norm in front of it and one
behind it, x <- x + norm1b(mixer(norm1(x))) and, where the layer has a feed-forward, x <- x + norm2b(ff(norm2(x))), over
a 32-bit stream (``sandwich_norm``); the norms are RMS norms in groups (``group_rms_norm``).  The mixer is

* ``attention``: grouped-query attention without rotation under a window that keeps the first tokens
  (``windowed_attention``); a layer with ``kv_from`` has no key and value projections and reads the cache of the layer it
  names, as one more reader of that run's cache;
* ``parallel``: two mixers on the same input whose outputs are added, each times a constant (``parallel_mixers``): on
  the left attention with queries and keys normed over the whole projection, capped scores, a bias by distance, a
  learned sink and a gate per head; on the right the gated delta rule (``gated_delta_rule``);
* ``retention``: linear attention with a fixed decay per head, rotary positions on queries and keys, the keys scaled,
  every head normed by itself without a weight, a SiLU gate (``lightning_attention`` with those parameters).

The feed-forward is dense with biases and the polynomial activation (``poly_norm_mlp``).
Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*`` (``.left.*`` and
``.right.*`` in a parallel layer), ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import TedalixConfig
from ..config.registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

# the design fixes these
SLOPE_EXPONENT = 8.0         # the bias by distance of head h of H has the slope 2^(-8 (h + 1) / H)
# no longest position is part of the design (angles are computed from the position, there is no table); the engine's
# bookkeeping wants a bound, and positions are 32-bit integers
MAX_POSITIONS = 1 << 24


def _cache_masks(cfg: TedalixConfig):
    """Per attention layer with keys of its own: the mask its cache is kept for, wide enough for every layer that
    reads it: (window, kept first positions), window 0 = every key."""
    out = {}
    for i, lc in enumerate(cfg.layers):
        if lc.type != "attention":
            continue
        owner = i if lc.mixer.kv_from is None else lc.mixer.kv_from
        m = lc.mixer.mask
        w, k = out.get(owner, (m.size, m.keep_first))
        w = 0 if (w == 0 or m.size == 0) else max(w, m.size)
        out[owner] = (w, max(k, m.keep_first) if w else 0)
    return out


def _attention_params(cfg: TedalixConfig, m, sink: bool) -> dict:
    p = dict(hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
             scale=m.scale, window=m.mask.size, keep_first=m.mask.keep_first, norm_eps=cfg.norm_eps)
    if sink:
        p.update(qk_norm="whole", score_cap=m.softcap, slope_exponent=SLOPE_EXPONENT, sink="learned", head_gate=True)
    return p


def _layer_spec(cfg: TedalixConfig, i: int, lc, positions, cache_masks) -> LayerSpec:
    h, p = cfg.width, f"l{i}."
    norm = lambda name: PartSpec("group_rms_norm", dict(size=h, eps=cfg.norm_eps, groups=cfg.norm_groups), {"weight": p + name})
    m = lc.mixer
    if lc.type == "attention":
        own = m.kv_from is None
        cw, ck = cache_masks[i if own else m.kv_from]
        params = _attention_params(cfg, m, sink=False)
        params.update(own_keys=own, cache_window=cw, cache_keep_first=ck)
        names = ("q", "k", "v", "o") if own else ("q", "o")
        mixer = PartSpec("windowed_attention", params, {n: f"{p}mix.{n}" for n in names})
    elif lc.type == "parallel":
        left, right = m.left, m.right
        members = [dict(kind="windowed_attention", params=_attention_params(cfg, left, sink=True), scale=m.left_scale),
                   dict(kind="gated_delta_rule", scale=m.right_scale, params=dict(
                       hidden_size=h, num_heads=right.heads, num_kv_heads=right.kv_heads, head_dim=right.dim,
                       value_dim=right.vdim, conv=right.conv, norm_eps=cfg.norm_eps, rank=right.rank))]
        w = {f"0.{n}": f"{p}mix.left.{n}" for n in ("q", "k", "v", "o", "q.norm", "k.norm", "sink", "g")}
        w.update({f"1.{n}": f"{p}mix.right.{n}" for n in ("q", "k", "v", "q.conv", "k.conv", "v.conv", "b", "A_log", "dt_bias",
                                                          "a1", "a2", "g1", "g2", "norm", "o")})
        mixer = PartSpec("parallel_mixers", dict(hidden_size=h, members=members), w)
    else:
        pos = None
        if m.rot_dims:
            pos = f"rot{m.rot_dims}@{m.rot_base!r}"
            positions.setdefault(pos, PartSpec("rotary_frequencies", dict(rotary_dim=m.rot_dims, theta=m.rot_base)))
        mixer = PartSpec("lightning_attention", dict(
            hidden_size=h, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, decay=m.decay, norm_eps=cfg.norm_eps,
            activation="none", position=pos, rotary_dim=m.rot_dims, key_scale=m.dim ** -0.5, head_norm=True,
            norm_weight=False, gate_activation="silu"), {n: f"{p}mix.{n}" for n in ("q", "k", "v", "g", "o")})
    if not lc.ff:
        return LayerSpec("sandwich_norm_mixer_only", {"pre_mixer_norm": norm("norm1"), "mixer": mixer,
                                                      "post_mixer_norm": norm("norm1b")})
    ffn = PartSpec("poly_norm_mlp", dict(hidden_size=h, intermediate_size=lc.ff, eps=cfg.norm_eps),
                   {n: f"{p}mlp.{n}" for n in ("up", "up.b", "down", "down.b", "act")})
    return LayerSpec("sandwich_norm", {"pre_mixer_norm": norm("norm1"), "mixer": mixer, "post_mixer_norm": norm("norm1b"),
                                       "pre_ffn_norm": norm("norm2"), "ffn": ffn, "post_ffn_norm": norm("norm2b")})


def tedalix_spec(cfg: TedalixConfig) -> ModelSpec:
    h = cfg.width
    positions = {}
    masks = _cache_masks(cfg)
    layers = [_layer_spec(cfg, i, lc, positions, masks) for i, lc in enumerate(cfg.layers)]
    # a layer is a run; one that reads another layer's keys and values reads that run's cache
    order = [RunSpec(i, lc.mixer.kv_from if lc.type == "attention" else None) for i, lc in enumerate(cfg.layers)]
    norm = PartSpec("group_rms_norm", dict(size=h, eps=cfg.norm_eps, groups=cfg.norm_groups), {"weight": "final.norm"})
    return ModelSpec(
        architecture="Tedalix", vocab_size=cfg.vocab, hidden_size=h, max_positions=MAX_POSITIONS, eos_token_ids=(),
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=h), {"weight": "embed"}),
        layers=layers, order=order, final_norm=norm,
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=h), {"weight": "head"}),
        positions=positions)


TEDALIX = register_architecture(Architecture(
    name="tedalix", architecture_aliases=("Tedalix",), model_type_aliases=("tedalix",),
    parse_config=TedalixConfig.from_dict, build_spec=tedalix_spec))
