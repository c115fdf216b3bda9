"""Zekonex as a `ModelSpec`: a stack whose layers are listed in config.json one by one, each
with one of three mixers (grouped-query attention with a sink in its softmax, a gated delta
rule recurrence behind short convolutions, attention over a low-rank latent), beside it a clamped
gated feed-forward that reads the same norm, both added to the stream together times one
number.  A stretch of the layers may run several times in a row with the same weights; each
pass has caches and state of its own and begins by adding a vector of its own to the stream.

config.json gives every size and every constant that differs between models of the design
(`vocab`, `width`, `embedding.scale`, `norm.eps`, `residual_mult`, `loop`, and per layer `type`,
`mixer` and `mlp`); tensor names are the checkpoint's own (`embed`, `loop.step`,
`l<i>.{norm1,mix.*,mlp.*}`, `final.norm`, `head`).
"""

from __future__ import annotations

import dataclasses
from typing import Any

from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
from mini_infer_amd.registry import ARCHITECTURES

NAME = "Zekonex"
MIXER_TYPES = ("attention", "delta", "latent_attention")
FEED_FORWARD_KINDS = ("dense",)
SINK_LOGIT = 0.0  # the attention's softmax has exp(0) = 1 more in its denominator
LOOP_VECTORS = "loop.step"


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
class Rotation:
    base: float
    dims: int


@dataclasses.dataclass(frozen=True)
class ZekonexLayer:
    type: str
    heads: int
    dim: int
    vdim: int
    kv_heads: int | None = None  # attention, delta
    scale: float | None = None  # attention, latent_attention
    rot: Rotation | None = None  # attention (may rotate nothing), latent_attention
    rot_dim: int | None = None  # latent_attention
    kv_rank: int | None = None  # latent_attention
    taps: int | None = None  # delta
    ff: int | None = None  # None: the layer has no feed-forward
    limit: float | None = None


@dataclasses.dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclasses.dataclass(frozen=True)
class ZekonexConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    residual_mult: float
    layers: tuple[ZekonexLayer, ...]
    loop: Loop | None

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ZekonexConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json needs a non-empty list under 'layers'")
        parsed = [_parse_layer(f"layers[{i}]", entry) for i, entry in enumerate(layers)]
        eps = _number("norm.eps", _section(raw, "norm").get("eps"))
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        loop = None
        if raw.get("loop") is not None:
            section = _section(raw, "loop")
            start, stop = section.get("start"), section.get("stop")
            if isinstance(start, bool) or isinstance(stop, bool) or not isinstance(start, int) or not isinstance(stop, int) \
                    or not 0 <= start < stop <= len(parsed):
                raise ConfigError(f"loop.start..loop.stop must name a non-empty stretch of the {len(parsed)} layers, got {start!r}..{stop!r}")
            loop = Loop(start, stop, _positive_int("loop.times", section.get("times")))
        return cls(
            architecture=str(raw.get("architecture") or (raw.get("architectures") or [NAME])[0]),
            vocab=_positive_int("vocab", raw.get("vocab")),
            width=_positive_int("width", raw.get("width")),
            embedding_scale=_number("embedding.scale", _section(raw, "embedding").get("scale")),
            norm_eps=eps,
            residual_mult=_number("residual_mult", raw.get("residual_mult")),
            layers=tuple(parsed),
            loop=loop,
        )


def _parse_rotation(where: str, mixer: dict[str, Any], limit: int) -> Rotation | None:
    if mixer.get("rot") is None:
        return None
    rot = _section(mixer, "rot", where)
    dims = _positive_int(f"{where}.rot.dims", rot.get("dims"))
    if dims % 2 or dims > limit:
        raise ConfigError(f"{where}.rot.dims={dims} must be even and at most {limit}")
    base = _number(f"{where}.rot.base", rot.get("base"))
    if base <= 0:
        raise ConfigError(f"{where}.rot.base must be positive, got {base}")
    return Rotation(base, dims)


def _parse_layer(where: str, entry: Any) -> ZekonexLayer:
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
    if kind in ("attention", "delta"):
        fields["kv_heads"] = _positive_int(f"{at}.kv_heads", mixer.get("kv_heads", fields["heads"]))
        if fields["heads"] % fields["kv_heads"] != 0:
            raise ConfigError(f"{where}: heads={fields['heads']} is not a multiple of kv_heads={fields['kv_heads']}")
    if kind in ("attention", "latent_attention"):
        fields["scale"] = _number(f"{at}.scale", mixer.get("scale"))
    if kind == "attention":
        fields["rot"] = _parse_rotation(at, mixer, fields["dim"])
    elif kind == "latent_attention":
        fields["kv_rank"] = _positive_int(f"{at}.kv_rank", mixer.get("kv_rank"))
        fields["rot_dim"] = _positive_int(f"{at}.rot_dim", mixer.get("rot_dim"))
        rot = _parse_rotation(at, mixer, fields["rot_dim"])
        if rot is None or rot.dims != fields["rot_dim"]:
            raise ConfigError(f"{at}: the rotated part is rot_dim={fields['rot_dim']} wide and all of it is rotated, got rot={mixer.get('rot')!r}")
        fields["rot"] = rot
    else:
        fields["taps"] = _positive_int(f"{at}.conv", mixer.get("conv"))
    mlp = entry.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind") not in FEED_FORWARD_KINDS:
            raise ConfigError(f"{where}.mlp must be null or an object of kind {FEED_FORWARD_KINDS}, got {mlp!r}")
        fields["ff"] = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
        fields["limit"] = _number(f"{where}.mlp.limit", mlp.get("limit"))
        if fields["limit"] <= 0:
            raise ConfigError(f"{where}.mlp.limit must be positive, got {fields['limit']}")
    return ZekonexLayer(**fields)


def _rotary(rot: Rotation, head_dim: int) -> dict[str, Any]:
    # exact_frequencies: base^(-2i/dims) evaluated in 64-bit before it becomes the float32 table
    return {"kind": "rotary", "head_dim": head_dim, "theta": rot.base, "rotary_dim": rot.dims, "interleaved": True,
            "exact_frequencies": True}


def zekonex_order(cfg: ZekonexConfig) -> list[LayerCall]:
    """The running order: the looped stretch `times` times in a row, each pass's first call
    adding that pass's row of `loop.step` to the stream."""
    count = len(cfg.layers)
    if cfg.loop is None:
        return [LayerCall(i) for i in range(count)]
    order = [LayerCall(i) for i in range(cfg.loop.start)]
    for turn in range(cfg.loop.times):
        for i in range(cfg.loop.start, cfg.loop.stop):
            order.append(LayerCall(i, stream_add=(LOOP_VECTORS, turn) if i == cfg.loop.start else None))
    return order + [LayerCall(i) for i in range(cfg.loop.stop, count)]


def zekonex_spec(cfg: ZekonexConfig) -> ModelSpec:
    norm = {"kind": "rms_norm", "hidden_size": cfg.width, "eps": cfg.norm_eps, "name": ""}
    names = {"norm": "norm1", "mixer": "mix.", "feed_forward": "mlp."}
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "attention":
            mixer = {
                "kind": "gqa_attention", "hidden_size": cfg.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads,
                "head_dim": layer.dim, "v_head_dim": layer.vdim, "scale": layer.scale, "sink_logit": SINK_LOGIT,
                "names": ("q", "k", "v", "o"), "suffix": "",
                "position": None if layer.rot is None else _rotary(layer.rot, layer.dim),
            }
        elif layer.type == "latent_attention":
            mixer = {
                "kind": "latent_attention", "hidden_size": cfg.width, "num_heads": layer.heads, "head_dim": layer.dim,
                "rot_dim": layer.rot_dim, "v_head_dim": layer.vdim, "kv_rank": layer.kv_rank, "scale": layer.scale,
                "norm_eps": cfg.norm_eps, "position": _rotary(layer.rot, layer.rot_dim),
            }
        else:
            mixer = {
                "kind": "gated_delta_rule", "hidden_size": cfg.width, "num_heads": layer.heads, "num_kv_heads": layer.kv_heads,
                "head_dim": layer.dim, "v_head_dim": layer.vdim, "taps": layer.taps, "norm_eps": cfg.norm_eps,
            }
        block = {
            "kind": "parallel", "norm": norm, "mixer": mixer, "scale": cfg.residual_mult, "names": names,
            "feed_forward": None if layer.ff is None else {
                "kind": "clamped_glu", "hidden_size": cfg.width, "intermediate_size": layer.ff, "limit": layer.limit,
            },
        }
        layers.append(LayerSpec(prefix=f"l{i}.", block=block))
    return ModelSpec(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        layers=layers,
        order=zekonex_order(cfg),
        final_norm={**norm, "name": "norm"},
        final_norm_prefix="final.",
        embedding={"kind": "scaled_embedding", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed",
                   "scale": cfg.embedding_scale},
        head={"kind": "linear_head", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "head", "tied": False},
        stream_vectors={} if cfg.loop is None else {LOOP_VECTORS: cfg.loop.times},
    )


ZEKONEX = ARCHITECTURES.register(NAME, Architecture(name=NAME, parse_config=ZekonexConfig.from_dict, build_spec=zekonex_spec))
