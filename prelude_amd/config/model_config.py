"""Typed model configuration read from an architecture's own config.json keys.

The keys, which of them are required, and the error for a missing one follow
crates/prelude-core/src/models/config.rs:4-22 (every field required except
``sliding_window``) and crates/prelude-core/src/engine/config.rs:122-170
(``eos_token_id``: an integer or a non-empty list, required for generation).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key."""


_MISSING = object()


def _get(raw: Mapping[str, Any], key: str, kind, arch: str, default=_MISSING):
    if key not in raw or raw[key] is None:
        if default is not _MISSING:
            return default
        raise ConfigError(f"failed to parse {arch} config: missing required key `{key}`")
    v = raw[key]
    if kind is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be true or false, got {v!r}")
        return v
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be an integer, got {v!r}")
        if v < 0:
            raise ConfigError(f"failed to parse {arch} config: `{key}` must not be negative, got {v!r}")
        return v
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be a number, got {v!r}")
        return float(v)
    if kind is str:
        if not isinstance(v, str):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be a string, got {v!r}")
        return v
    raise AssertionError(kind)


def parse_eos_token_ids(raw: Mapping[str, Any]) -> Tuple[int, ...]:
    """``eos_token_id`` as a tuple (crates/prelude-core/src/engine/config.rs:122-170)."""
    if "eos_token_id" not in raw or raw["eos_token_id"] is None:
        raise ConfigError("generation model config is missing required field `eos_token_id`")
    v = raw["eos_token_id"]
    if isinstance(v, bool):
        raise ConfigError("generation model config has invalid `eos_token_id` type")
    if isinstance(v, int):
        if v < 0:
            raise ConfigError("generation model config has invalid non-integer `eos_token_id`")
        return (v,)
    if isinstance(v, list):
        if not v:
            raise ConfigError("generation model config has empty `eos_token_id`")
        for e in v:
            if isinstance(e, bool) or not isinstance(e, int) or e < 0:
                raise ConfigError("generation model config has non-integer entry in `eos_token_id`")
        return tuple(v)
    raise ConfigError("generation model config has invalid `eos_token_id` type")


@dataclasses.dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense (crates/prelude-core/src/models/config.rs:4-22)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    attention_bias: bool
    max_position_embeddings: int
    sliding_window: Optional[int]
    max_window_layers: int
    tie_word_embeddings: bool
    rope_theta: float
    rms_norm_eps: float
    use_sliding_window: bool
    hidden_act: str
    eos_token_ids: Tuple[int, ...]

    ARCH = "Qwen3"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        a = cls.ARCH
        cfg = cls(
            vocab_size=_get(raw, "vocab_size", int, a),
            hidden_size=_get(raw, "hidden_size", int, a),
            intermediate_size=_get(raw, "intermediate_size", int, a),
            num_hidden_layers=_get(raw, "num_hidden_layers", int, a),
            num_attention_heads=_get(raw, "num_attention_heads", int, a),
            num_key_value_heads=_get(raw, "num_key_value_heads", int, a),
            head_dim=_get(raw, "head_dim", int, a),
            attention_bias=_get(raw, "attention_bias", bool, a),
            max_position_embeddings=_get(raw, "max_position_embeddings", int, a),
            sliding_window=_get(raw, "sliding_window", int, a, default=None),
            max_window_layers=_get(raw, "max_window_layers", int, a),
            tie_word_embeddings=_get(raw, "tie_word_embeddings", bool, a),
            rope_theta=_get(raw, "rope_theta", float, a),
            rms_norm_eps=_get(raw, "rms_norm_eps", float, a),
            use_sliding_window=_get(raw, "use_sliding_window", bool, a),
            hidden_act=_get(raw, "hidden_act", str, a),
            eos_token_ids=parse_eos_token_ids(raw),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        a = self.ARCH
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"failed to parse {a} config: `{key}` must be positive")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"failed to parse {a} config: `num_attention_heads` ({self.num_attention_heads}) is not a "
                f"multiple of `num_key_value_heads` ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"failed to parse {a} config: `head_dim` ({self.head_dim}) must be even for RoPE")
        if self.rms_norm_eps <= 0 or self.rope_theta <= 0:
            raise ConfigError(f"failed to parse {a} config: `rms_norm_eps` and `rope_theta` must be positive")
        if self.use_sliding_window and not self.sliding_window:
            raise ConfigError(f"failed to parse {a} config: `use_sliding_window` is true but `sliding_window` is unset")
        for e in self.eos_token_ids:
            if e >= self.vocab_size:
                raise ConfigError(f"failed to parse {a} config: `eos_token_id` {e} is outside the vocabulary")

    def layer_window(self, layer: int) -> Optional[int]:
        """Keys a layer attends to, or None for all of them.

        The reference parses the three window keys and refuses
        ``use_sliding_window`` (crates/prelude-core/src/models/qwen3.rs:50-52).
        Here they mean: layers with index >= ``max_window_layers`` see the
        last ``sliding_window`` keys, the query's own included.
        """
        if self.use_sliding_window and self.sliding_window and layer >= self.max_window_layers:
            return int(self.sliding_window)
        return None

    def to_dict(self) -> dict:
        d = dataclasses.asdict(self)
        eos = d.pop("eos_token_ids")
        d["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        d["architectures"] = ["Qwen3ForCausalLM"]
        d["model_type"] = "qwen3"
        return d


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json in model folder {model_dir!r}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"failed to parse {path}: {e}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"failed to parse {path}: top level is not an object")
    return raw


# ---------------------------------------------------------------------------
def _obj(raw: Mapping[str, Any], key: str, arch: str, where: str = "", optional: bool = False):
    if key not in raw or raw[key] is None:
        if optional:
            return None
        raise ConfigError(f"failed to parse {arch} config: missing required key `{where}{key}`")
    if not isinstance(raw[key], dict):
        raise ConfigError(f"failed to parse {arch} config: `{where}{key}` must be an object")
    return raw[key]


def _positive(raw: Mapping[str, Any], key: str, kind, arch: str, where: str):
    try:
        v = _get(raw, key, kind, arch)
    except ConfigError as e:
        raise ConfigError(str(e).replace(f"`{key}`", f"`{where}{key}`")) from None
    if not v > 0:
        raise ConfigError(f"failed to parse {arch} config: `{where}{key}` must be positive, got {v!r}")
    return v


@dataclasses.dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int          # unrotated query/key dimensions a head
    rot_dim: int      # rotated query/key dimensions a head (the key's are shared by all heads)
    vdim: int         # value dimensions a head
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    rot_dims: int     # how many of the rotated part's dimensions turn


@dataclasses.dataclass(frozen=True)
class LibodraMlpConfig:
    kind: str                 # "dense" | "moe"
    ff: int = 0               # dense: inner size; moe: an expert's inner size
    limit: float = 0.0        # dense: the clamp
    experts: int = 0
    top: int = 0
    shared_ff: int = 0        # moe: inner size of the shared expert, 0 = none


@dataclasses.dataclass(frozen=True)
class LibodraLayerConfig:
    type: str
    mixer: LatentMixerConfig
    mlp: Optional[LibodraMlpConfig]


@dataclasses.dataclass(frozen=True)
class LibodraConfig:
    """Libodra: a decoder of pre-norm layers listed one by one in ``layers``, each with a mixer that attends
    through a latent (a learned sink in its softmax) and a feed-forward that is dense (clamped gated pair), a
    mixture of experts chosen by token id from a table (with an optional shared expert), or absent.  Every size
    and constant is read from here; there is no longest position and no end-of-sequence id."""
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[LibodraLayerConfig, ...]

    ARCH = "Libodra"
    MIXERS = ("latent_attention",)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "LibodraConfig":
        a = cls.ARCH
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError(f"failed to parse {a} config: `layers` must be a non-empty list")
        layers = []
        for i, lr in enumerate(layers_raw):
            w = f"layers[{i}]."
            if not isinstance(lr, dict):
                raise ConfigError(f"failed to parse {a} config: `layers[{i}]` must be an object")
            kind = _get(lr, "type", str, a)
            if kind not in cls.MIXERS:
                raise ConfigError(f"failed to parse {a} config: `{w}type` {kind!r} is not one of {list(cls.MIXERS)}")
            m = _obj(lr, "mixer", a, w)
            mw = w + "mixer."
            rot = _obj(m, "rot", a, mw)
            rot_dim = _get(m, "rot_dim", int, a)
            mixer = LatentMixerConfig(
                heads=_positive(m, "heads", int, a, mw), dim=_positive(m, "dim", int, a, mw), rot_dim=rot_dim,
                vdim=_positive(m, "vdim", int, a, mw), kv_rank=_positive(m, "kv_rank", int, a, mw),
                q_rank=_positive(m, "q_rank", int, a, mw), scale=_positive(m, "scale", float, a, mw),
                rot_base=_positive(rot, "base", float, a, mw + "rot."), rot_dims=_get(rot, "dims", int, a))
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
                raise ConfigError(f"failed to parse {a} config: `{mw}rot.dims` ({mixer.rot_dims}) must be even and at "
                                  f"most `rot_dim` ({mixer.rot_dim})")
            f = _obj(lr, "mlp", a, w, optional=True)
            mlp = None
            if f is not None:
                fw = w + "mlp."
                fk = _get(f, "kind", str, a)
                if fk == "dense":
                    mlp = LibodraMlpConfig("dense", ff=_positive(f, "ff", int, a, fw), limit=_positive(f, "limit", float, a, fw))
                elif fk == "moe":
                    router = _obj(f, "router", a, fw)
                    shared = _obj(f, "shared", a, fw, optional=True)
                    mlp = LibodraMlpConfig(
                        "moe", ff=_positive(_obj(f, "expert", a, fw), "ff", int, a, fw + "expert."),
                        experts=_positive(router, "experts", int, a, fw + "router."),
                        top=_positive(router, "top", int, a, fw + "router."),
                        shared_ff=_positive(shared, "ff", int, a, fw + "shared.") if shared is not None else 0)
                    if mlp.top > mlp.experts:
                        raise ConfigError(f"failed to parse {a} config: `{fw}router.top` ({mlp.top}) exceeds "
                                          f"`router.experts` ({mlp.experts})")
                else:
                    raise ConfigError(f"failed to parse {a} config: `{fw}kind` {fk!r} is not one of ['dense', 'moe']")
            layers.append(LibodraLayerConfig(kind, mixer, mlp))
        norm = _obj(raw, "norm", a)
        return cls(vocab=_positive(raw, "vocab", int, a, ""), width=_positive(raw, "width", int, a, ""),
                   norm_eps=_positive(norm, "eps", float, a, "norm."), layers=tuple(layers))


# ---------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class LightningMixerConfig:
    heads: int
    dim: int                    # query/key dimensions a head
    vdim: int                   # value dimensions a head
    decay: Tuple[float, ...]    # one a head


@dataclasses.dataclass(frozen=True)
class LongWaveScaling:
    factor: float
    low: float
    high: float
    original: int


@dataclasses.dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                    # query/key dimensions a head; the values are the keys, so also the value's
    scale: float
    rot_base: float
    rot_dims: int               # how many of a head's first dimensions turn
    rot_scaling: Optional[LongWaveScaling]


@dataclasses.dataclass(frozen=True)
class FazopelMlpConfig:
    kind: str                   # "dense" | "moe"
    ff: int = 0                 # dense: inner size; moe: an expert's inner size
    limit: float = 0.0          # moe: an expert's clamp
    experts: int = 0
    top: int = 0
    route_scale: float = 1.0
    shared_ff: int = 0          # moe: inner size of the shared expert, 0 = none
    shared_limit: float = 0.0


@dataclasses.dataclass(frozen=True)
class FazopelLayerConfig:
    type: str                   # "lightning" | "attention"
    mixer: object               # LightningMixerConfig | SinkAttentionConfig
    mlp: Optional[FazopelMlpConfig]
    weights_of: Optional[int]   # the layer whose tensors this one uses (its own cache or state), itself a layer with tensors; None: its own


@dataclasses.dataclass(frozen=True)
class FazopelConfig:
    """Fazopel: a decoder whose layers are listed one by one in ``layers``; a layer norms each branch's output before
    adding it.  Its mixer is linear attention with a decaying state (``lightning``) or grouped-query attention whose
    values are its keys and whose softmax has an empty sink (``attention``); its feed-forward is dense (squared relu),
    a mixture of routed experts with an optional shared one, or absent.  A layer may use another layer's tensors
    (``weights_of``).  Every size and constant is read from here; there is no longest position and no
    end-of-sequence id."""
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[FazopelLayerConfig, ...]

    ARCH = "Fazopel"
    MIXERS = ("lightning", "attention")

    @classmethod
    def _mixer(cls, kind: str, m: Mapping[str, Any], mw: str):
        a = cls.ARCH
        heads = _positive(m, "heads", int, a, mw)
        dim = _positive(m, "dim", int, a, mw)
        # the values of the attention are its keys, so their size is the keys' and may go unsaid
        vdim = _positive(m, "vdim", int, a, mw) if (kind == "lightning" or m.get("vdim") is not None) else dim
        if kind == "lightning":
            decay = m.get("decay")
            if isinstance(decay, (int, float)) and not isinstance(decay, bool):
                decay = [decay] * heads          # one number for all heads
            if not isinstance(decay, list) or len(decay) != heads or \
                    not all(isinstance(x, (int, float)) and not isinstance(x, bool) and 0.0 <= x <= 1.0 for x in decay):
                raise ConfigError(f"failed to parse {a} config: `{mw}decay` must list one number in [0, 1] for each of "
                                  f"the {heads} heads, got {decay!r}")
            return LightningMixerConfig(heads, dim, vdim, tuple(float(x) for x in decay))
        kv_heads = _positive(m, "kv_heads", int, a, mw)
        if heads % kv_heads:
            raise ConfigError(f"failed to parse {a} config: `{mw}heads` ({heads}) is no multiple of `kv_heads` ({kv_heads})")
        if vdim != dim:
            raise ConfigError(f"failed to parse {a} config: `{mw}vdim` ({vdim}) must equal `dim` ({dim}): the values are the keys")
        rot = _obj(m, "rot", a, mw)
        rw = mw + "rot."
        dims = _get(rot, "dims", int, a)
        if dims % 2 or dims > dim:
            raise ConfigError(f"failed to parse {a} config: `{rw}dims` ({dims}) must be even and at most `dim` ({dim})")
        sc = _obj(rot, "scaling", a, rw, optional=True)
        scaling = None
        if sc is not None:
            sw = rw + "scaling."
            scaling = LongWaveScaling(_positive(sc, "factor", float, a, sw), _positive(sc, "low", float, a, sw),
                                      _positive(sc, "high", float, a, sw), _positive(sc, "original", int, a, sw))
            if not scaling.high > scaling.low:
                raise ConfigError(f"failed to parse {a} config: `{sw}high` ({scaling.high}) must exceed `low` ({scaling.low})")
        return SinkAttentionConfig(heads, kv_heads, dim, _positive(m, "scale", float, a, mw),
                                   _positive(rot, "base", float, a, rw), dims, scaling)

    @classmethod
    def _mlp(cls, f: Optional[Mapping[str, Any]], fw: str) -> Optional[FazopelMlpConfig]:
        a = cls.ARCH
        if f is None:
            return None
        fk = _get(f, "kind", str, a)
        if fk == "dense":
            return FazopelMlpConfig("dense", ff=_positive(f, "ff", int, a, fw))
        if fk != "moe":
            raise ConfigError(f"failed to parse {a} config: `{fw}kind` {fk!r} is not one of ['dense', 'moe']")
        router = _obj(f, "router", a, fw)
        expert = _obj(f, "expert", a, fw)
        shared = _obj(f, "shared", a, fw, optional=True)
        mlp = FazopelMlpConfig(
            "moe", ff=_positive(expert, "ff", int, a, fw + "expert."), limit=_positive(expert, "limit", float, a, fw + "expert."),
            experts=_positive(router, "experts", int, a, fw + "router."), top=_positive(router, "top", int, a, fw + "router."),
            route_scale=_positive(router, "scale", float, a, fw + "router."),
            shared_ff=_positive(shared, "ff", int, a, fw + "shared.") if shared is not None else 0,
            shared_limit=_positive(shared, "limit", float, a, fw + "shared.") if shared is not None else 0.0)
        if mlp.top > mlp.experts:
            raise ConfigError(f"failed to parse {a} config: `{fw}router.top` ({mlp.top}) exceeds `router.experts` ({mlp.experts})")
        return mlp

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FazopelConfig":
        a = cls.ARCH
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError(f"failed to parse {a} config: `layers` must be a non-empty list")
        layers = []
        for i, lr in enumerate(layers_raw):
            w = f"layers[{i}]."
            if not isinstance(lr, dict):
                raise ConfigError(f"failed to parse {a} config: `layers[{i}]` must be an object")
            kind = _get(lr, "type", str, a)
            if kind not in cls.MIXERS:
                raise ConfigError(f"failed to parse {a} config: `{w}type` {kind!r} is not one of {list(cls.MIXERS)}")
            src = _get(lr, "weights_of", int, a, default=None)
            layer = FazopelLayerConfig(kind, cls._mixer(kind, _obj(lr, "mixer", a, w), w + "mixer."),
                                       cls._mlp(_obj(lr, "mlp", a, w, optional=True), w + "mlp."), src)
            if src is not None:
                if not 0 <= src < len(layers_raw) or src == i:
                    raise ConfigError(f"failed to parse {a} config: `{w}weights_of` ({src}) names no other layer")
            layers.append(layer)
        for i, layer in enumerate(layers):
            # a layer may name one that itself names another: the tensors are those of the end of the chain
            j, seen = layer.weights_of, {i}
            while j is not None and layers[j].weights_of is not None:
                if j in seen:
                    raise ConfigError(f"failed to parse {a} config: `layers[{i}].weights_of` leads in a circle")
                seen.add(j)
                j = layers[j].weights_of
            if j is not None and j != layer.weights_of:
                layers[i] = dataclasses.replace(layer, weights_of=j)
        norm = _obj(raw, "norm", a)
        return cls(vocab=_positive(raw, "vocab", int, a, ""), width=_positive(raw, "width", int, a, ""),
                   norm_eps=_positive(norm, "eps", float, a, "norm."), layers=tuple(layers))


# ---------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class WindowMask:
    size: int          # the query at i sees the key at j <= i with i - j < size; 0: every earlier key
    keep_first: int    # ... or j < keep_first


@dataclasses.dataclass(frozen=True)
class TedalixAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask: WindowMask
    softcap: float = 0.0              # the sink mixer only; 0: none
    kv_from: Optional[int] = None     # the layer whose cached keys and values this one reads


@dataclasses.dataclass(frozen=True)
class TedalixDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    rank: Optional[int]     # inner size of the two-step projections; None: what the tensors have


@dataclasses.dataclass(frozen=True)
class TedalixParallelConfig:
    left: TedalixAttentionConfig
    right: TedalixDeltaConfig
    left_scale: float
    right_scale: float


@dataclasses.dataclass(frozen=True)
class TedalixRetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_base: float
    rot_dims: int           # 0: no rotation


@dataclasses.dataclass(frozen=True)
class TedalixLayerConfig:
    type: str               # "attention" | "parallel" | "retention"
    mixer: object
    ff: int                 # inner size of the dense feed-forward; 0: the layer has none


@dataclasses.dataclass(frozen=True)
class TedalixConfig:
    """Tedalix: a decoder whose layers are listed one by one in ``layers``, each with a norm in front of and behind
    every branch (RMS norms in ``norm.groups`` groups).  A layer's mixer is attention under a window that keeps the
    first tokens (``attention``; it may read another layer's cached keys and values, ``kv_from``), attention with a
    sink, capped scores, a bias by distance and a gate per head beside the gated delta rule (``parallel``), or linear
    attention with a fixed decay per head and rotary positions (``retention``).  The feed-forward is dense with the
    polynomial activation, or absent.  Every size and constant is read from here; there is no longest position and
    no end-of-sequence id."""
    vocab: int
    width: int
    norm_eps: float
    norm_groups: int
    layers: Tuple[TedalixLayerConfig, ...]

    ARCH = "Tedalix"
    MIXERS = ("attention", "parallel", "retention")

    @classmethod
    def _mask(cls, m: Mapping[str, Any], mw: str) -> WindowMask:
        a = cls.ARCH
        mask = _obj(m, "mask", a, mw, optional=True)
        if mask is None:
            return WindowMask(0, 0)
        size = _positive(mask, "size", int, a, mw + "mask.")
        try:
            keep = _get(mask, "keep_first", int, a, default=0)
        except ConfigError as e:
            raise ConfigError(str(e).replace("`keep_first`", f"`{mw}mask.keep_first`")) from None
        return WindowMask(size, keep)

    @classmethod
    def _attention(cls, m: Mapping[str, Any], mw: str, sink: bool) -> TedalixAttentionConfig:
        a = cls.ARCH
        heads, kv_heads = _positive(m, "heads", int, a, mw), _positive(m, "kv_heads", int, a, mw)
        if heads % kv_heads:
            raise ConfigError(f"failed to parse {a} config: `{mw}heads` ({heads}) is no multiple of `kv_heads` ({kv_heads})")
        softcap = 0.0
        if sink and m.get("softcap") is not None:
            softcap = _positive(m, "softcap", float, a, mw)
        src = None
        if not sink and m.get("kv_from") is not None:
            try:
                src = _get(m, "kv_from", int, a)
            except ConfigError as e:
                raise ConfigError(str(e).replace("`kv_from`", f"`{mw}kv_from`")) from None
        return TedalixAttentionConfig(heads, kv_heads, _positive(m, "dim", int, a, mw), _positive(m, "vdim", int, a, mw),
                                      _positive(m, "scale", float, a, mw), cls._mask(m, mw), softcap, src)

    @classmethod
    def _mixer(cls, kind: str, m: Mapping[str, Any], mw: str):
        a = cls.ARCH
        if kind == "attention":
            return cls._attention(m, mw, sink=False)
        if kind == "parallel":
            r = _obj(m, "right", a, mw)
            rw = mw + "right."
            heads, kv_heads = _positive(r, "heads", int, a, rw), _positive(r, "kv_heads", int, a, rw)
            if heads % kv_heads:
                raise ConfigError(f"failed to parse {a} config: `{rw}heads` ({heads}) is no multiple of `kv_heads` ({kv_heads})")
            rank = _positive(r, "rank", int, a, rw) if r.get("rank") is not None else None
            right = TedalixDeltaConfig(heads, kv_heads, _positive(r, "dim", int, a, rw), _positive(r, "vdim", int, a, rw),
                                       _positive(r, "conv", int, a, rw), rank)
            try:
                ls, rs = _get(m, "left_scale", float, a), _get(m, "right_scale", float, a)
            except ConfigError as e:
                raise ConfigError(str(e).replace("`left_scale`", f"`{mw}left_scale`").replace("`right_scale`", f"`{mw}right_scale`")) from None
            return TedalixParallelConfig(cls._attention(_obj(m, "left", a, mw), mw + "left.", sink=True), right, ls, rs)
        heads = _positive(m, "heads", int, a, mw)
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or \
                not all(isinstance(x, (int, float)) and not isinstance(x, bool) and 0.0 <= x <= 1.0 for x in decay):
            raise ConfigError(f"failed to parse {a} config: `{mw}decay` must list one number in [0, 1] for each of the "
                              f"{heads} heads, got {decay!r}")
        dim = _positive(m, "dim", int, a, mw)
        rot = _obj(m, "rot", a, mw, optional=True)
        base, dims = 1.0, 0
        if rot is not None:
            base, dims = _positive(rot, "base", float, a, mw + "rot."), _positive(rot, "dims", int, a, mw + "rot.")
            if dims % 2 or dims > dim:
                raise ConfigError(f"failed to parse {a} config: `{mw}rot.dims` ({dims}) must be even and at most `dim` ({dim})")
        return TedalixRetentionConfig(heads, dim, _positive(m, "vdim", int, a, mw), tuple(float(x) for x in decay), base, dims)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "TedalixConfig":
        a = cls.ARCH
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError(f"failed to parse {a} config: `layers` must be a non-empty list")
        layers = []
        for i, lr in enumerate(layers_raw):
            w = f"layers[{i}]."
            if not isinstance(lr, dict):
                raise ConfigError(f"failed to parse {a} config: `layers[{i}]` must be an object")
            kind = _get(lr, "type", str, a)
            if kind not in cls.MIXERS:
                raise ConfigError(f"failed to parse {a} config: `{w}type` {kind!r} is not one of {list(cls.MIXERS)}")
            f = _obj(lr, "mlp", a, w, optional=True)
            ff = 0
            if f is not None:
                fk = _get(f, "kind", str, a)
                if fk != "dense":
                    raise ConfigError(f"failed to parse {a} config: `{w}mlp.kind` {fk!r} is not one of ['dense']")
                ff = _positive(f, "ff", int, a, w + "mlp.")
            layers.append(TedalixLayerConfig(kind, cls._mixer(kind, _obj(lr, "mixer", a, w), w + "mixer."), ff))
        for i, layer in enumerate(layers):
            src = layer.mixer.kv_from if layer.type == "attention" else None
            if src is None:
                continue
            w = f"layers[{i}].mixer."
            if not 0 <= src < len(layers) or src == i or layers[src].type != "attention" or layers[src].mixer.kv_from is not None:
                raise ConfigError(f"failed to parse {a} config: `{w}kv_from` ({src}) must name another attention layer that "
                                  f"has keys and values of its own")
            if src > i:
                raise ConfigError(f"failed to parse {a} config: `{w}kv_from` ({src}) names a layer that runs later")
            m, o = layer.mixer, layers[src].mixer
            if (m.kv_heads, m.dim, m.vdim) != (o.kv_heads, o.dim, o.vdim):
                raise ConfigError(f"failed to parse {a} config: `{w}kv_heads`, `dim` and `vdim` must equal those of layer {src}, "
                                  f"whose keys and values it reads")
        norm = _obj(raw, "norm", a)
        width = _positive(raw, "width", int, a, "")
        groups = _positive(norm, "groups", int, a, "norm.") if norm.get("groups") is not None else 1
        if width % groups:
            raise ConfigError(f"failed to parse {a} config: `norm.groups` ({groups}) does not divide `width` ({width})")
        return cls(vocab=_positive(raw, "vocab", int, a, ""), width=width, norm_eps=_positive(norm, "eps", float, a, "norm."),
                   norm_groups=groups, layers=tuple(layers))


# ---------------------------------------------------------------------------
@dataclasses.dataclass(frozen=True)
class NivasunMixerConfig:
    heads: int
    kv_heads: int       # latent attention: as many as heads (every head has keys of its own, from the latent)
    dim: int
    vdim: int
    scale: float
    window: int         # the query at i sees the key at j with 0 <= i - j < window
    rot_dims: int = 0   # the first dimensions of a head (of a map) that turn; 0: none
    rot_base: float = 0.0
    kv_rank: int = 0    # latent attention
    q_rank: int = 0
    diff: float = 0.0   # differential attention


@dataclasses.dataclass(frozen=True)
class NivasunMlpConfig:
    ff: int
    experts: int
    top: int
    shared_ff: int      # 0: no shared expert


@dataclasses.dataclass(frozen=True)
class NivasunLayerConfig:
    type: str
    mixer: NivasunMixerConfig
    mlp: Optional[NivasunMlpConfig]


@dataclasses.dataclass(frozen=True)
class NivasunConfig:
    """Nivasun: a decoder whose layers are listed one by one in ``layers``; a stretch of them (``loop``) runs several
    times in a row on the same tensors.  A layer has one norm (a single number as its weight) whose output the mixer
    reads through a short convolution over time and the feed-forward as it is; both are added to the stream together.
    Mixers: ``attention`` (the keys are the values, rotation in halves, a temperature and a sink per head),
    ``latent_attention`` (queries, keys and values through latents, a gate on the output), ``attention_2`` (two maps a
    head, one taken off the other), all under a sliding window.  The feed-forward is routed experts with a gated shared
    one, or absent.  The embedding adds a row chosen by the token and the one before it; the logits are capped.  Every
    size and constant is read from here; there is no longest position and no end-of-sequence id."""
    vocab: int
    width: int
    norm_eps: float
    taps: int
    embed_scale: float
    buckets: int
    mul_prev: int
    mul_cur: int
    logit_cap: float            # 0: none
    loop_start: int
    loop_stop: int
    loop_times: int             # 1 with start == stop: no loop
    layers: Tuple[NivasunLayerConfig, ...]
    has_loop: bool = False      # the configuration has a `loop` (its file then holds a vector per pass, also for an empty stretch)

    ARCH = "Nivasun"
    MIXERS = ("attention", "latent_attention", "attention_2")

    @classmethod
    def _rot(cls, m: Mapping[str, Any], mw: str, dim: int):
        a = cls.ARCH
        rot = _obj(m, "rot", a, mw, optional=True)
        if rot is None:
            return 0, 0.0
        dims = _get(rot, "dims", int, a, default=0)
        if dims % 2 or dims > dim:
            raise ConfigError(f"failed to parse {a} config: `{mw}rot.dims` ({dims}) must be even and at most `dim` ({dim})")
        return dims, (_positive(rot, "base", float, a, mw + "rot.") if dims else 0.0)

    @classmethod
    def _mixer(cls, kind: str, m: Mapping[str, Any], mw: str) -> NivasunMixerConfig:
        a = cls.ARCH
        heads = _positive(m, "heads", int, a, mw)
        dim = _positive(m, "dim", int, a, mw)
        scale = _positive(m, "scale", float, a, mw)
        window = _positive(_obj(m, "mask", a, mw), "size", int, a, mw + "mask.")
        if kind == "latent_attention":
            return NivasunMixerConfig(heads, heads, dim, _positive(m, "vdim", int, a, mw), scale, window,
                                      kv_rank=_positive(m, "kv_rank", int, a, mw), q_rank=_positive(m, "q_rank", int, a, mw))
        kv_heads = _positive(m, "kv_heads", int, a, mw)
        if heads % kv_heads:
            raise ConfigError(f"failed to parse {a} config: `{mw}heads` ({heads}) is no multiple of `kv_heads` ({kv_heads})")
        dims, base = cls._rot(m, mw, dim)
        if kind == "attention":
            # the values are the keys, so their size is the keys' and may go unsaid
            vdim = _positive(m, "vdim", int, a, mw) if m.get("vdim") is not None else dim
            if vdim != dim:
                raise ConfigError(f"failed to parse {a} config: `{mw}vdim` ({vdim}) must equal `dim` ({dim}): the values are the keys")
            return NivasunMixerConfig(heads, kv_heads, dim, dim, scale, window, dims, base)
        diff = _get(m, "diff", float, a)
        return NivasunMixerConfig(heads, kv_heads, dim, _positive(m, "vdim", int, a, mw), scale, window, dims, base, diff=diff)

    @classmethod
    def _mlp(cls, f: Optional[Mapping[str, Any]], fw: str) -> Optional[NivasunMlpConfig]:
        a = cls.ARCH
        if f is None:
            return None
        fk = _get(f, "kind", str, a, default="moe")
        if fk != "moe":
            raise ConfigError(f"failed to parse {a} config: `{fw}kind` {fk!r} is not one of ['moe']")
        router = _obj(f, "router", a, fw)
        shared = _obj(f, "shared", a, fw, optional=True)
        mlp = NivasunMlpConfig(ff=_positive(_obj(f, "expert", a, fw), "ff", int, a, fw + "expert."),
                               experts=_positive(router, "experts", int, a, fw + "router."),
                               top=_positive(router, "top", int, a, fw + "router."),
                               shared_ff=_positive(shared, "ff", int, a, fw + "shared.") if shared is not None else 0)
        if mlp.top > mlp.experts:
            raise ConfigError(f"failed to parse {a} config: `{fw}router.top` ({mlp.top}) exceeds `router.experts` ({mlp.experts})")
        return mlp

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "NivasunConfig":
        a = cls.ARCH
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError(f"failed to parse {a} config: `layers` must be a non-empty list")
        layers = []
        for i, lr in enumerate(layers_raw):
            w = f"layers[{i}]."
            if not isinstance(lr, dict):
                raise ConfigError(f"failed to parse {a} config: `layers[{i}]` must be an object")
            kind = _get(lr, "type", str, a)
            if kind not in cls.MIXERS:
                raise ConfigError(f"failed to parse {a} config: `{w}type` {kind!r} is not one of {list(cls.MIXERS)}")
            layers.append(NivasunLayerConfig(kind, cls._mixer(kind, _obj(lr, "mixer", a, w), w + "mixer."),
                                             cls._mlp(_obj(lr, "mlp", a, w, optional=True), w + "mlp.")))
        n = len(layers)
        loop = _obj(raw, "loop", a, optional=True)
        start, stop, times = 0, 0, 1
        if loop is not None:
            start, stop = _get(loop, "start", int, a), _get(loop, "stop", int, a)
            times = _positive(loop, "times", int, a, "loop.")
            if not 0 <= start <= stop <= n:
                raise ConfigError(f"failed to parse {a} config: `loop.start` ({start}) and `loop.stop` ({stop}) must lie in "
                                  f"order within the {n} layers")
        emb = _obj(raw, "embedding", a)
        pair = _obj(emb, "bigram", a, "embedding.")
        pw = "embedding.bigram."
        mul = {}
        for key in ("mul_prev", "mul_cur"):   # any integers, also negative ones: the row is the sum modulo the buckets
            v = pair.get(key)
            if v is None:
                raise ConfigError(f"failed to parse {a} config: missing required key `{pw}{key}`")
            if isinstance(v, bool) or not isinstance(v, int):
                raise ConfigError(f"failed to parse {a} config: `{pw}{key}` must be an integer, got {v!r}")
            mul[key] = int(v)
        cap = _get(raw, "logit_softcap", float, a, default=0.0)
        if cap < 0:
            raise ConfigError(f"failed to parse {a} config: `logit_softcap` must not be negative, got {cap!r}")
        return cls(vocab=_positive(raw, "vocab", int, a, ""), width=_positive(raw, "width", int, a, ""),
                   norm_eps=_positive(_obj(raw, "norm", a), "eps", float, a, "norm."),
                   taps=_positive(_obj(raw, "canon", a), "taps", int, a, "canon."),
                   embed_scale=_get(emb, "scale", float, a, default=1.0), buckets=_positive(pair, "buckets", int, a, pw),
                   mul_prev=mul["mul_prev"], mul_cur=mul["mul_cur"], logit_cap=cap,
                   loop_start=start, loop_stop=stop, loop_times=times, layers=tuple(layers), has_loop=loop is not None)
