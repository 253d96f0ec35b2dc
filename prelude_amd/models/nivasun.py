"""Nivasun: from its typed configuration to a model specification.

A decoder whose layers are listed one by one in the configuration.  The embedding is the token's row times a constant
plus a row chosen by the token and the one before it (``pair_hash_embedding``, 32-bit: it is the stream).  A layer has
one norm whose weight is a single number (``group_rms_norm`` with one group and ``scalar_weight``); the mixer reads its
output through a short convolution over time (``conv_input``), the feed-forward as it is, and both are added to the
32-bit stream together (``parallel_branches``).  The mixer is

* ``attention``: grouped-query attention whose values are its keys as projected, the first dimensions of a head rotated
  in halves, a learned temperature and a learned sink per head (``gqa_attention`` with those parameters);
* ``latent_attention``: queries, keys and values through normed latents, no positions, a sigmoid gate on the heads'
  outputs (``latent_attention`` without a rotated part);
* ``attention_2``: two attention maps a head over the same values, rotated in pairs, one taken off the other
  (``differential_attention``);

all under a sliding window.  The feed-forward is routed experts chosen by their logits, weighted by the softmax over the
chosen ones, with a gated shared expert (``routed_experts`` with those parameters), or absent.  The layers
``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row on the same tensors, each pass with caches and state
of its own (one run per pass in the order) and a learned vector added to the stream in front of it.  The head's logits
are capped by a tanh.
Tensor names: ``embed``, ``bigram``, ``loop.step``, ``l<i>.norm1``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import NivasunConfig
from ..config.registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

# no longest position is part of the design (angles are computed from the position, there is no table); the engine's
# bookkeeping wants a bound, and positions are 32-bit integers
MAX_POSITIONS = 1 << 24


def _position(positions, dims: int, base: float):
    if not dims:
        return None
    name = f"rot{dims}@{base!r}"
    positions.setdefault(name, PartSpec("rotary_frequencies", dict(rotary_dim=dims, theta=base)))
    return name


def _mixer(cfg: NivasunConfig, i: int, lc, positions):
    """(kind, parameters, local tensor name -> checkpoint name) of layer i's mixer."""
    h, m, p = cfg.width, lc.mixer, f"l{i}.mix."
    if lc.type == "attention":
        params = dict(hidden_size=h, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, norm_eps=cfg.norm_eps,
                      qk_norm=False, window=m.window, position=_position(positions, m.rot_dims, m.rot_base),
                      rotary_dim=m.rot_dims, scale=m.scale, values_from_keys=True, sink="learned", head_scale=True)
        names = {"q_proj.weight": p + "q", "k_proj.weight": p + "k", "o_proj.weight": p + "o", "sinks": p + "sink",
                 "head_scales": p + "temp"}
        return "gqa_attention", params, names
    if lc.type == "latent_attention":
        params = dict(hidden_size=h, num_heads=m.heads, head_dim=m.dim, rot_dim=0, value_dim=m.vdim, kv_rank=m.kv_rank,
                      q_rank=m.q_rank, norm_eps=cfg.norm_eps, scale=m.scale, window=m.window, output_gate=True)
        return "latent_attention", params, {n: p + n for n in ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o")}
    params = dict(hidden_size=h, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                  scale=m.scale, diff=m.diff, norm_eps=cfg.norm_eps, window=m.window,
                  position=_position(positions, m.rot_dims, m.rot_base), rotary_dim=m.rot_dims)
    return "differential_attention", params, {n: p + n for n in ("q", "k", "v", "o", "lq1", "lk1", "lq2", "lk2")}


def _layer_spec(cfg: NivasunConfig, i: int, lc, positions) -> LayerSpec:
    h, p = cfg.width, f"l{i}."
    norm = PartSpec("group_rms_norm", dict(size=h, eps=cfg.norm_eps, groups=1, scalar_weight=True), {"weight": p + "norm1"})
    kind, params, names = _mixer(cfg, i, lc, positions)
    weights = {"conv": p + "canon1"}
    weights.update({f"inner.{local}": name for local, name in names.items()})
    mixer = PartSpec("conv_input", dict(hidden_size=h, taps=cfg.taps, inner=dict(kind=kind, params=params)), weights)
    f = lc.mlp
    if f is None:
        return LayerSpec("parallel_branches_mixer_only", {"norm": norm, "mixer": mixer})
    w = {"router": p + "mlp.router", "router.b": p + "mlp.router.b"}
    for e in range(f.experts):
        for n in ("gate", "up", "down"):
            w[f"e{e}.{n}"] = f"{p}mlp.e{e}.{n}"
    if f.shared_ff:
        w.update({f"shared.{n}": f"{p}mlp.shared.{n}" for n in ("gate", "up", "down", "sg")})
    ffn = PartSpec("routed_experts", dict(hidden_size=h, num_experts=f.experts, top=f.top, expert_size=f.ff, activation="silu",
                                          router_bias=True, route="chosen_logits", correction=False,
                                          shared_size=f.shared_ff), w)
    return LayerSpec("parallel_branches", {"norm": norm, "mixer": mixer, "ffn": ffn})


def run_order(cfg: NivasunConfig):
    """The runs in order: (layer, the pass of the loop it opens or None)."""
    n = len(cfg.layers)
    if cfg.loop_stop <= cfg.loop_start:
        return [(i, None) for i in range(n)]
    out = [(i, None) for i in range(cfg.loop_start)]
    for t in range(cfg.loop_times):
        out += [(i, t if i == cfg.loop_start else None) for i in range(cfg.loop_start, cfg.loop_stop)]
    return out + [(i, None) for i in range(cfg.loop_stop, n)]


def nivasun_spec(cfg: NivasunConfig) -> ModelSpec:
    h = cfg.width
    positions = {}
    layers = [_layer_spec(cfg, i, lc, positions) for i, lc in enumerate(cfg.layers)]
    looped = cfg.has_loop   # a file of a configuration with a `loop` holds the passes' vectors, also where the stretch is empty
    return ModelSpec(
        architecture="Nivasun", vocab_size=cfg.vocab, hidden_size=h, max_positions=MAX_POSITIONS, eos_token_ids=(),
        embedding=PartSpec("pair_hash_embedding", dict(vocab_size=cfg.vocab, hidden_size=h, buckets=cfg.buckets,
                                                       mul_prev=cfg.mul_prev, mul_cur=cfg.mul_cur, scale=cfg.embed_scale),
                           {"weight": "embed", "pair": "bigram"}),
        layers=layers, order=[RunSpec(i, stream_row=t) for i, t in run_order(cfg)],
        stream_rows=("loop.step", cfg.loop_times) if looped else None,
        final_norm=PartSpec("group_rms_norm", dict(size=h, eps=cfg.norm_eps, groups=1, scalar_weight=True), {"weight": "final.norm"}),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=h, logit_cap=cfg.logit_cap), {"weight": "head"}),
        positions=positions)


NIVASUN = register_architecture(Architecture(
    name="nivasun", architecture_aliases=("Nivasun",), model_type_aliases=("nivasun",),
    parse_config=NivasunConfig.from_dict, build_spec=nivasun_spec))
