"""Nadosun as a `ModelSpec`: a stack that mixes minGRU layers with windowed attention layers
whose values are their keys, each sublayer normed on its output by a one-gain RMS norm and
scaled per column, a PolyNorm feed-forward where a layer has one, and a per-layer token side
input; scaled embedding plus a sinusoid of the position in front, a one-gain norm and an
untied head behind.

config.json gives every size and every constant that differs between models of the design
(`vocab`, `width`, `embedding.scale`, `norm.eps`, `token_side.dim`, and per layer `type`,
`mixer` sizes and `mlp`); tensor names are the checkpoint's own (`embed`, `side.embed`,
`l<i>.{norm1,norm2,ls1,ls2,mix.*,mlp.*,side.*}`, `final.norm`, `head`).
"""

from __future__ import annotations

import dataclasses
from typing import Any

from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models.spec import Architecture, LayerCall, LayerSpec, ModelSpec
from mini_infer_amd.registry import ARCHITECTURES

NAME = "Nadosun"
MIXER_TYPES = ("mingru", "attention")
FEED_FORWARD_KINDS = ("dense",)


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
class NadosunLayer:
    type: str
    width: int | None = None  # mingru: size of the recurrent state
    heads: int | None = None  # attention
    kv_heads: int | None = None
    dim: int | None = None
    window: int | None = None
    scale: float | None = None
    ff: int | None = None  # None: the layer has no feed-forward


@dataclasses.dataclass(frozen=True)
class NadosunConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    side_dim: int
    layers: tuple[NadosunLayer, ...]

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "NadosunConfig":
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json needs a non-empty list under 'layers'")
        parsed = []
        for i, entry in enumerate(layers):
            where = f"layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{where} must be an object")
            kind = entry.get("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}.type is {kind!r}; this design has {MIXER_TYPES}")
            mixer = _section(entry, "mixer", where)
            fields: dict[str, Any] = {"type": kind}
            if kind == "mingru":
                fields["width"] = _positive_int(f"{where}.mixer.width", mixer.get("width"))
            else:
                for key in ("heads", "kv_heads", "dim"):
                    fields[key] = _positive_int(f"{where}.mixer.{key}", mixer.get(key))
                if fields["heads"] % fields["kv_heads"] != 0:
                    raise ConfigError(f"{where}: heads={fields['heads']} is not a multiple of kv_heads={fields['kv_heads']}")
                vdim = mixer.get("vdim", fields["dim"])
                if vdim != fields["dim"]:
                    raise ConfigError(f"{where}: the values are the keys, so vdim={vdim} must equal dim={fields['dim']}")
                fields["window"] = _positive_int(f"{where}.mixer.mask.size", _section(mixer, "mask", f"{where}.mixer").get("size"))
                fields["scale"] = _number(f"{where}.mixer.scale", mixer.get("scale"))
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") not in FEED_FORWARD_KINDS:
                    raise ConfigError(f"{where}.mlp must be null or an object of kind {FEED_FORWARD_KINDS}, got {mlp!r}")
                fields["ff"] = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
            parsed.append(NadosunLayer(**fields))
        eps = _number("norm.eps", _section(raw, "norm").get("eps"))
        if eps <= 0:
            raise ConfigError(f"norm.eps must be positive, got {eps}")
        return cls(
            architecture=str(raw.get("architecture") or (raw.get("architectures") or [NAME])[0]),
            vocab=_positive_int("vocab", raw.get("vocab")),
            width=_positive_int("width", raw.get("width")),
            embedding_scale=_number("embedding.scale", _section(raw, "embedding").get("scale")),
            norm_eps=eps,
            side_dim=_positive_int("token_side.dim", _section(raw, "token_side").get("dim")),
            layers=tuple(parsed),
        )


def nadosun_spec(cfg: NadosunConfig) -> ModelSpec:
    norm = {"kind": "scalar_rms_norm", "hidden_size": cfg.width, "eps": cfg.norm_eps, "name": ""}
    names = {
        "mixer_norm": "norm1", "mixer": "mix.", "mixer_scale": "ls1",
        "ffn_norm": "norm2", "feed_forward": "mlp.", "ffn_scale": "ls2",
        "side": "side.", "side_norm": "side.",
    }
    layers = []
    for i, layer in enumerate(cfg.layers):
        if layer.type == "mingru":
            mixer = {"kind": "min_gru", "hidden_size": cfg.width, "width": layer.width}
        else:
            mixer = {
                "kind": "keys_as_values_attention", "hidden_size": cfg.width, "num_heads": layer.heads,
                "num_kv_heads": layer.kv_heads, "head_dim": layer.dim, "window": layer.window, "scale": layer.scale,
                "norm_eps": cfg.norm_eps,
            }
        block = {
            "kind": "output_norm",
            "hidden_size": cfg.width,
            "layer_scale": True,
            "norm": norm,
            "mixer": mixer,
            "feed_forward": None if layer.ff is None else {
                "kind": "dense_poly_norm", "hidden_size": cfg.width, "intermediate_size": layer.ff, "eps": cfg.norm_eps,
            },
            "side": {
                "kind": "token_side_input", "hidden_size": cfg.width, "dim": cfg.side_dim, "first_col": i * cfg.side_dim,
                "table_name": "side.embed", "vocab_size": cfg.vocab, "table_columns": len(cfg.layers) * cfg.side_dim,
            },
            # (a plain per-column weight, whatever the sublayers' norm is)
            "side_norm": {"kind": "rms_norm", "hidden_size": cfg.width, "eps": cfg.norm_eps, "name": "norm"},
            "names": names,
        }
        layers.append(LayerSpec(prefix=f"l{i}.", block=block))
    return ModelSpec(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        layers=layers,
        order=[LayerCall(i) for i in range(len(layers))],
        final_norm={**norm, "name": "norm"},
        final_norm_prefix="final.",
        embedding={"kind": "scaled_sinusoid_embedding", "vocab_size": cfg.vocab, "hidden_size": cfg.width,
                   "name": "embed", "scale": cfg.embedding_scale},
        head={"kind": "linear_head", "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "head", "tied": False},
    )


NADOSUN = ARCHITECTURES.register(NAME, Architecture(name=NAME, parse_config=NadosunConfig.from_dict, build_spec=nadosun_spec))
