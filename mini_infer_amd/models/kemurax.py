"""Kemurax as a `ModelSpec`: a stack whose layers are listed in config.json one by one.  A layer
is a mixer and, where it has one, a dense gated feed-forward (tanh gelu), each behind an RMS
norm whose weight is stored around zero.  Two mixers: gated linear attention (a matrix state
per head that decays per key channel), and a pair side by side that read the same input, on
the left grouped-query attention inside chunks of positions (queries and keys normed head by
head, rotary positions with Llama-3.1 frequency scaling, an output gate), on the right a
state-space layer in its recurrent form behind a short convolution; the pair's outputs are
added with two weights.  The residual stream is kept in `streams` copies that every sublayer
reads through a vector and rewrites through a matrix and a vector of its own; without that key
there is one copy and a plain add.  In front a normed embedding, behind a norm over the sum of
the copies and a head that is the embedding table.

config.json gives every size and every constant that differs between models of the design
(`vocab`, `width`, `streams`, `norm.eps`, and per layer `type`, `mixer`, `mlp`); tensor names
are the checkpoint's own (`embed`, `embed.norm`, `l<i>.{norm1,norm2,mix.*,mlp.*,hc1.*,hc2.*}`,
`final.norm`).
"""

from __future__ import annotations

import dataclasses
from typing import Any

from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
from mini_infer_amd.registry import ARCHITECTURES

NAME = "Kemurax"
LAYER_TYPES = ("gla", "parallel")
FEED_FORWARD_KINDS = ("dense",)
NORM_WEIGHT_OFFSET = 1.0  # norm weights are stored around zero
MAX_STREAMS = 8


def _positive_int(where: str, value: Any) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"{where} must be a positive integer, got {value!r}")
    return value


def _number(where: str, value: Any) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"{where} must be a number, got {value!r}")
    return float(value)


def _section(raw: dict[str, Any], key: str, where: str = "config.json") -> dict[str, Any]:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{where} needs an object under {key!r}")
    return value


@dataclasses.dataclass(frozen=True)
class FrequencyScaling:
    factor: float
    low: float
    high: float
    original: int


@dataclasses.dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    scaling: FrequencyScaling | None


@dataclasses.dataclass(frozen=True)
class GatedLinearAttentionSizes:
    heads: int
    dim: int
    vdim: int
    tau: float
    # width of the narrow projection in front of the decay gates: config.json does not name it, a
    # checkpoint's shapes do (`with_checkpoint_shapes`); None: the default of `default_decay_rank`
    decay_rank: int | None = None


@dataclasses.dataclass(frozen=True)
class ChunkedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    chunk: int | None
    scale: float
    rot: Rotation


@dataclasses.dataclass(frozen=True)
class StateSpaceSizes:
    heads: int
    vdim: int
    state: int
    groups: int
    taps: int
    norm_groups: int


@dataclasses.dataclass(frozen=True)
class PairSizes:
    left: ChunkedAttentionSizes
    right: StateSpaceSizes
    left_scale: float
    right_scale: float


@dataclasses.dataclass(frozen=True)
class KemuraxLayer:
    type: str
    mixer: "GatedLinearAttentionSizes | PairSizes"
    ff: int | None  # None: the layer has no feed-forward


@dataclasses.dataclass(frozen=True)
class KemuraxConfig:
    architecture: str
    vocab: int
    width: int
    streams: int | None  # None: one copy of the stream and a plain add
    norm_eps: float
    layers: tuple[KemuraxLayer, ...]

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "KemuraxConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json needs a non-empty list under 'layers'")
        eps = _number("norm.eps", _section(raw, "norm").get("eps"))
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        streams = None
        if raw.get("streams") is not None:
            streams = _positive_int("streams", raw.get("streams"))
            if streams > MAX_STREAMS:
                raise ConfigError(f"streams={streams}: the stream kernels keep up to {MAX_STREAMS} copies")
        return cls(
            architecture=str(raw.get("architecture") or (raw.get("architectures") or [NAME])[0]),
            vocab=_positive_int("vocab", raw.get("vocab")),
            width=_positive_int("width", raw.get("width")),
            streams=streams,
            norm_eps=eps,
            layers=tuple(_parse_layer(f"layers[{i}]", entry) for i, entry in enumerate(layers)),
        )


def _parse_rotation(where: str, mixer: dict[str, Any], head_dim: int) -> Rotation:
    rot = _section(mixer, "rot", where)
    dims = _positive_int(f"{where}.rot.dims", rot.get("dims"))
    if dims % 2 or dims > head_dim:
        raise ConfigError(f"{where}.rot.dims={dims} must be even and at most dim={head_dim}")
    base = _number(f"{where}.rot.base", rot.get("base"))
    if base <= 0:
        raise ConfigError(f"{where}.rot.base must be positive, got {base}")
    scaling = None
    if rot.get("scaling") is not None:
        s = _section(rot, "scaling", f"{where}.rot")
        factor, low, high = (_number(f"{where}.rot.scaling.{k}", s.get(k)) for k in ("factor", "low", "high"))
        original = _positive_int(f"{where}.rot.scaling.original", s.get("original"))
        if factor <= 0 or low <= 0 or high <= low:
            raise ConfigError(f"{where}.rot.scaling needs factor > 0 and 0 < low < high, got {s!r}")
        scaling = FrequencyScaling(factor, low, high, original)
    return Rotation(base, dims, scaling)


def _parse_attention(where: str, m: dict[str, Any]) -> ChunkedAttentionSizes:
    heads, dim = _positive_int(f"{where}.heads", m.get("heads")), _positive_int(f"{where}.dim", m.get("dim"))
    kv_heads = _positive_int(f"{where}.kv_heads", m.get("kv_heads"))
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads={heads} is not a multiple of kv_heads={kv_heads}")
    # (no mask: every earlier position is seen)
    chunk = None if m.get("mask") is None else _positive_int(f"{where}.mask.size", _section(m, "mask", where).get("size"))
    return ChunkedAttentionSizes(
        heads=heads, kv_heads=kv_heads, dim=dim, vdim=_positive_int(f"{where}.vdim", m.get("vdim")), chunk=chunk,
        scale=_number(f"{where}.scale", m.get("scale")), rot=_parse_rotation(where, m, dim),
    )


def _parse_state_space(where: str, m: dict[str, Any]) -> StateSpaceSizes:
    sizes = StateSpaceSizes(
        heads=_positive_int(f"{where}.heads", m.get("heads")), vdim=_positive_int(f"{where}.vdim", m.get("vdim")),
        state=_positive_int(f"{where}.state", m.get("state")), groups=_positive_int(f"{where}.groups", m.get("groups")),
        taps=_positive_int(f"{where}.conv", m.get("conv")), norm_groups=_positive_int(f"{where}.norm_groups", m.get("norm_groups")),
    )
    if sizes.heads % sizes.groups or (sizes.heads * sizes.vdim) % sizes.norm_groups:
        raise ConfigError(f"{where}: heads must be a multiple of groups, heads*vdim of norm_groups, got {m!r}")
    return sizes


def _parse_layer(where: str, entry: Any) -> KemuraxLayer:
    if not isinstance(entry, dict):
        raise ConfigError(f"{where} must be an object")
    kind = entry.get("type")
    if kind not in LAYER_TYPES:
        raise ConfigError(f"{where}.type is {kind!r}; this design has {LAYER_TYPES}")
    m = _section(entry, "mixer", where)
    at = f"{where}.mixer"
    if kind == "gla":
        tau = _number(f"{at}.tau", m.get("tau"))
        if tau <= 0:
            raise ConfigError(f"{at}.tau must be positive, got {tau}")
        mixer: Any = GatedLinearAttentionSizes(
            heads=_positive_int(f"{at}.heads", m.get("heads")), dim=_positive_int(f"{at}.dim", m.get("dim")),
            vdim=_positive_int(f"{at}.vdim", m.get("vdim")), tau=tau,
            decay_rank=None if m.get("decay_rank") is None else _positive_int(f"{at}.decay_rank", m.get("decay_rank")),
        )
    else:
        mixer = PairSizes(
            left=_parse_attention(f"{at}.left", _section(m, "left", at)),
            right=_parse_state_space(f"{at}.right", _section(m, "right", at)),
            left_scale=_number(f"{at}.left_scale", m.get("left_scale")),
            right_scale=_number(f"{at}.right_scale", m.get("right_scale")),
        )
    ff = None
    mlp = entry.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind") not in FEED_FORWARD_KINDS:
            raise ConfigError(f"{where}.mlp must be null or an object of kind {FEED_FORWARD_KINDS}, got {mlp!r}")
        ff = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
    return KemuraxLayer(kind, mixer, ff)


def _attention_description(width: int, a: ChunkedAttentionSizes, eps: float) -> dict[str, Any]:
    position: dict[str, Any] = {
        "kind": "rotary", "head_dim": a.dim, "theta": a.rot.base, "rotary_dim": a.rot.dims, "interleaved": False,
        "exact_frequencies": True,
    }
    if a.rot.scaling is not None:
        s = a.rot.scaling
        position["llama3"] = {"factor": s.factor, "low_freq_factor": s.low, "high_freq_factor": s.high,
                              "original_max_position_embeddings": s.original}
    return {
        "kind": "gqa_attention", "hidden_size": width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
        "v_head_dim": a.vdim, "scale": a.scale, "chunk": a.chunk, "names": ("q", "k", "v", "o"), "suffix": "",
        "head_norm": {"eps": eps, "names": ("q.norm", "k.norm")}, "gate": {"name": "g", "activation": "logistic"},
        "position": position,
    }


def default_decay_rank(m: GatedLinearAttentionSizes) -> int:
    return max(16, m.heads * m.dim // 16)


def with_checkpoint_shapes(cfg: KemuraxConfig, shapes: dict[str, tuple[int, ...]]) -> KemuraxConfig:
    """The sizes that only a checkpoint's tensor shapes give: each gated-linear-attention layer's
    narrow decay projection is as wide as its `mix.a1` has rows."""
    layers = []
    for i, layer in enumerate(cfg.layers):
        shape = shapes.get(f"l{i}.mix.a1")
        if layer.type == "gla" and layer.mixer.decay_rank is None and shape is not None and len(shape) == 2:
            layer = dataclasses.replace(layer, mixer=dataclasses.replace(layer.mixer, decay_rank=int(shape[0])))
        layers.append(layer)
    return dataclasses.replace(cfg, layers=tuple(layers))


def kemurax_spec(cfg: KemuraxConfig) -> ModelSpec:
    copies = cfg.streams or 1
    norm = {"kind": "streams_rms_norm", "hidden_size": cfg.width, "eps": cfg.norm_eps, "copies": copies, "name": "",
            "weight_offset": NORM_WEIGHT_OFFSET}
    names = {"mixer_norm": "norm1", "mixer": "mix.", "ffn_norm": "norm2", "feed_forward": "mlp.",
             "mixer_connection": "hc1.", "ffn_connection": "hc2."}
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "gla":
            rank = m.decay_rank if m.decay_rank is not None else default_decay_rank(m)
            mixer: dict[str, Any] = {
                "kind": "gated_linear_attention", "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim,
                "v_head_dim": m.vdim, "decay_rank": rank, "tau": m.tau, "norm_eps": cfg.norm_eps,
            }
        else:
            r = m.right
            mixer = {
                "kind": "side_by_side", "left_scale": m.left_scale, "right_scale": m.right_scale,
                "left": _attention_description(cfg.width, m.left, cfg.norm_eps),
                "right": {
                    "kind": "state_space_duality", "hidden_size": cfg.width, "num_heads": r.heads, "v_head_dim": r.vdim,
                    "state_size": r.state, "groups": r.groups, "taps": r.taps, "norm_groups": r.norm_groups,
                    "norm_eps": cfg.norm_eps,
                },
            }
        block = {
            "kind": "hyper_connections", "norm": norm, "mixer": mixer, "copies": copies, "learned": cfg.streams is not None,
            "names": names,
            "feed_forward": None if layer.ff is None else {
                "kind": "swiglu", "hidden_size": cfg.width, "intermediate_size": layer.ff, "activation": "gelu_tanh",
                "names": ("gate", "up", "down"), "suffix": "",
            },
        }
        layers.append(LayerSpec(prefix=f"l{i}.", block=block))
    return ModelSpec(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        layers=layers,
        order=[LayerCall(i) for i in range(len(layers))],
        final_norm={**norm, "name": "norm"},
        final_norm_prefix="final.",
        embedding={"kind": "normed_streams_embedding", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed",
                   "norm_name": "embed.norm", "eps": cfg.norm_eps, "copies": copies, "weight_offset": NORM_WEIGHT_OFFSET},
        head={"kind": "linear_head", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "", "tied": True},
    )


KEMURAX = ARCHITECTURES.register(NAME, Architecture(
    name=NAME, parse_config=KemuraxConfig.from_dict, build_spec=kemurax_spec, with_checkpoint_shapes=with_checkpoint_shapes,
))
