"""Kunudra as a `ModelSpec`: a stack whose layers are listed in config.json one by one.  A layer is
normed BEHIND its sums, `x <- norm(alpha x + scale * sublayer(x))` for a mixer and then, where the
layer has one, a feed-forward; both read the stream as the last norm left it, and the norms'
weights are stored around zero.  Two mixers: grouped-query attention without rotation (queries and
keys normed over their whole projection, capped scores, a distance bias per head, a sliding
window, a learned sink per head, values that later layers mix with the first such layer's) and
attention over a low-rank latent whose queries go through a latent of their own (rotated key part
shared by the heads, window and sink as well).  Two feed-forwards: a dense gated one and a mixture
of experts (score correction for the choice, identity experts, a gated shared expert).  In front
the token's embedding plus a row of a second table chosen by a hash of the token and the one before
it; behind a norm and the embedding table as head.

config.json gives every size and every constant that differs between models of the design
(`vocab`, `width`, `postln_alpha`, `norm.eps`, `embedding.bigram`, and per layer `type`, `mixer`
and `mlp`); tensor names are the checkpoint's own (`embed`, `bigram`, `l<i>.{norm1,norm2,ls1,ls2,
mix.*,mlp.*}`, `final.norm`).  A key that config.json does not hold switches its mechanism off.
"""

from __future__ import annotations

import dataclasses
from typing import Any

from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
from mini_infer_amd.registry import ARCHITECTURES

NAME = "Kunudra"
MIXER_TYPES = ("attention", "latent_attention")
FEED_FORWARD_KINDS = ("dense", "moe")
SLOPE_TOTAL_EXPONENT = 8.0  # the distance bias of head h of H is 2^(-8 (h + 1) / H) a position
VALUE_MIX_KEY = "first"  # all layers that mix values mix in those of the first of them


def _positive_int(where: str, value: Any) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"{where} must be a positive integer, got {value!r}")
    return value


def _count(where: str, value: Any) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ConfigError(f"{where} must be a non-negative integer, got {value!r}")
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
class Rotation:
    base: float
    dims: int


@dataclasses.dataclass(frozen=True)
class PairTable:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclasses.dataclass(frozen=True)
class Experts:
    ff: int
    experts: int
    top: int
    identity: int = 0
    scale: float = 1.0
    shared_ff: int | None = None


@dataclasses.dataclass(frozen=True)
class KunudraLayer:
    type: str
    heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None = None
    kv_heads: int | None = None  # attention
    softcap: float | None = None  # attention
    v_mix: bool = False  # attention
    rot: Rotation | None = None  # latent_attention
    rot_dim: int | None = None  # latent_attention
    kv_rank: int | None = None  # latent_attention
    q_rank: int | None = None  # latent_attention
    dense_ff: int | None = None  # a dense feed-forward
    moe: Experts | None = None  # a mixture of experts (neither: the layer has no feed-forward)


@dataclasses.dataclass(frozen=True)
class KunudraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    alpha: float
    pair_table: PairTable | None
    layers: tuple[KunudraLayer, ...]

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "KunudraConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json needs a non-empty list under 'layers'")
        eps = _number("norm.eps", _section(raw, "norm").get("eps"))
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        pair_table = None
        embedding = raw.get("embedding")
        if isinstance(embedding, dict) and embedding.get("bigram") is not None:
            section = _section(embedding, "bigram", "embedding")
            pair_table = PairTable(
                _positive_int("embedding.bigram.buckets", section.get("buckets")),
                _count("embedding.bigram.mul_prev", section.get("mul_prev")),
                _count("embedding.bigram.mul_cur", section.get("mul_cur")),
            )
        parsed = tuple(_parse_layer(f"layers[{i}]", entry) for i, entry in enumerate(layers))
        shared_widths = {layer.kv_heads * layer.vdim for layer in parsed if layer.v_mix}
        if len(shared_widths) > 1:
            raise ConfigError(f"layers that mix values share rows of one width, got kv_heads * vdim of {sorted(shared_widths)}")
        return cls(
            architecture=str(raw.get("architecture") or (raw.get("architectures") or [NAME])[0]),
            vocab=_positive_int("vocab", raw.get("vocab")),
            width=_positive_int("width", raw.get("width")),
            norm_eps=eps,
            alpha=_number("postln_alpha", raw.get("postln_alpha", 1.0)),
            pair_table=pair_table,
            layers=parsed,
        )


def _parse_layer(where: str, entry: Any) -> KunudraLayer:
    if not isinstance(entry, dict):
        raise ConfigError(f"{where} must be an object")
    kind = entry.get("type")
    if kind not in MIXER_TYPES:
        raise ConfigError(f"{where}.type is {kind!r}; this design has {MIXER_TYPES}")
    mixer = _section(entry, "mixer", where)
    at = f"{where}.mixer"
    fields: dict[str, Any] = {"type": kind}
    for key in ("heads", "dim"):
        fields[key] = _positive_int(f"{at}.{key}", mixer.get(key))
    fields["vdim"] = _positive_int(f"{at}.vdim", mixer.get("vdim", fields["dim"]))
    fields["scale"] = _number(f"{at}.scale", mixer.get("scale"))
    if fields["scale"] <= 0:
        raise ConfigError(f"{at}.scale must be positive, got {fields['scale']}")
    if mixer.get("mask") is not None:
        fields["window"] = _positive_int(f"{at}.mask.size", _section(mixer, "mask", at).get("size"))
    if kind == "attention":
        fields["kv_heads"] = _positive_int(f"{at}.kv_heads", mixer.get("kv_heads", fields["heads"]))
        if fields["heads"] % fields["kv_heads"] != 0:
            raise ConfigError(f"{where}: heads={fields['heads']} is not a multiple of kv_heads={fields['kv_heads']}")
        if mixer.get("softcap") is not None:
            fields["softcap"] = _number(f"{at}.softcap", mixer.get("softcap"))
            if fields["softcap"] <= 0:
                raise ConfigError(f"{at}.softcap must be positive, got {fields['softcap']}")
        fields["v_mix"] = bool(mixer.get("v_mix", False))
    else:
        fields["kv_rank"] = _positive_int(f"{at}.kv_rank", mixer.get("kv_rank"))
        fields["q_rank"] = _positive_int(f"{at}.q_rank", mixer.get("q_rank"))
        fields["rot_dim"] = _positive_int(f"{at}.rot_dim", mixer.get("rot_dim"))
        rot = _section(mixer, "rot", at)
        dims = _positive_int(f"{at}.rot.dims", rot.get("dims"))
        base = _number(f"{at}.rot.base", rot.get("base"))
        if dims != fields["rot_dim"] or dims % 2 or base <= 0:
            raise ConfigError(f"{at}: the rotated part is rot_dim={fields['rot_dim']} wide (even) and all of it is rotated, got rot={rot!r}")
        fields["rot"] = Rotation(base, dims)
    mlp = entry.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind") not in FEED_FORWARD_KINDS:
            raise ConfigError(f"{where}.mlp must be null or an object of kind {FEED_FORWARD_KINDS}, got {mlp!r}")
        if mlp["kind"] == "dense":
            fields["dense_ff"] = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
        else:
            router = _section(mlp, "router", f"{where}.mlp")
            shared = mlp.get("shared")
            fields["moe"] = Experts(
                ff=_positive_int(f"{where}.mlp.expert.ff", _section(mlp, "expert", f"{where}.mlp").get("ff")),
                experts=_positive_int(f"{where}.mlp.router.experts", router.get("experts")),
                top=_positive_int(f"{where}.mlp.router.top", router.get("top")),
                identity=_count(f"{where}.mlp.router.identity", router.get("identity", 0)),
                scale=_number(f"{where}.mlp.router.scale", router.get("scale", 1.0)),
                shared_ff=None if shared is None else _positive_int(f"{where}.mlp.shared.ff", _section(mlp, "shared", f"{where}.mlp").get("ff")),
            )
            if fields["moe"].top > fields["moe"].experts + fields["moe"].identity:
                raise ConfigError(f"{where}.mlp.router: top={fields['moe'].top} is more than there are experts")
    return KunudraLayer(**fields)


def kunudra_spec(cfg: KunudraConfig) -> ModelSpec:
    norm = {"kind": "post_rms_norm", "hidden_size": cfg.width, "eps": cfg.norm_eps, "name": "", "weight_offset": 1.0}
    names = {"mixer_norm": "norm1", "ffn_norm": "norm2", "mixer": "mix.", "feed_forward": "mlp.", "mixer_scale": "ls1",
             "ffn_scale": "ls2"}
    layers = []
    mixing_seen = False
    for i, layer in enumerate(cfg.layers):
        if layer.type == "attention":
            mixer = {
                "kind": "whole_norm_attention", "hidden_size": cfg.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads,
                "head_dim": layer.dim, "v_head_dim": layer.vdim, "scale": layer.scale, "window": layer.window,
                "norm_eps": cfg.norm_eps, "learned_sink": True,
                "position": {"kind": "distance_slopes", "total_exponent": SLOPE_TOTAL_EXPONENT},
            }
            if layer.softcap is not None:
                mixer["softcap"] = layer.softcap
            if layer.v_mix:
                mixer["value_mix"] = {"key": VALUE_MIX_KEY, "source": not mixing_seen, "name": "vmix"}
                mixing_seen = True
        else:
            mixer = {
                "kind": "latent_attention", "hidden_size": cfg.width, "num_heads": layer.heads, "head_dim": layer.dim,
                "rot_dim": layer.rot_dim, "v_head_dim": layer.vdim, "kv_rank": layer.kv_rank, "q_rank": layer.q_rank,
                "scale": layer.scale, "norm_eps": cfg.norm_eps, "window": layer.window, "learned_sink": True,
                # exact_frequencies: base^(-2i/dims) evaluated in 64-bit before it becomes the float32 table
                "position": {"kind": "rotary", "head_dim": layer.rot_dim, "theta": layer.rot.base, "rotary_dim": layer.rot.dims,
                             "interleaved": True, "exact_frequencies": True},
            }
        feed_forward = None
        if layer.dense_ff is not None:
            feed_forward = {"kind": "swiglu", "hidden_size": cfg.width, "intermediate_size": layer.dense_ff,
                            "names": ("gate", "up", "down"), "suffix": ""}
        elif layer.moe is not None:
            feed_forward = {"kind": "routed_experts", "hidden_size": cfg.width, "intermediate_size": layer.moe.ff,
                            "experts": layer.moe.experts, "top": layer.moe.top, "identity": layer.moe.identity,
                            "route_scale": layer.moe.scale, "correction": True, "shared_size": layer.moe.shared_ff}
        block = {"kind": "post_norm", "norm": norm, "mixer": mixer, "feed_forward": feed_forward, "hidden_size": cfg.width,
                 "alpha": cfg.alpha, "layer_scale": True, "names": names}
        layers.append(LayerSpec(prefix=f"l{i}.", block=block))
    if cfg.pair_table is None:
        embedding = {"kind": "token_embedding", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed"}
    else:
        embedding = {"kind": "pair_hash_embedding", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed",
                     "pair_name": "bigram", "buckets": cfg.pair_table.buckets, "mul_prev": cfg.pair_table.mul_prev,
                     "mul_cur": cfg.pair_table.mul_cur}
    return ModelSpec(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        layers=layers,
        order=[LayerCall(i) for i in range(len(layers))],
        final_norm={**norm, "name": "norm"},
        final_norm_prefix="final.",
        embedding=embedding,
        head={"kind": "linear_head", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "head", "tied": True},
    )


KUNUDRA = ARCHITECTURES.register(NAME, Architecture(name=NAME, parse_config=KunudraConfig.from_dict, build_spec=kunudra_spec))
