"""Tiny Nadosun configurations and model folders for the tests.

The configurations differ in every size and constant and in the order of layers: attention
first or recurrence first, a feed-forward behind either kind of mixer or behind none, layers
of one kind with different sizes (two attention layers with different windows and head counts
get page groups of their own, recurrent layers get state rows of different widths), one
key/value head, as many as query heads, a window of a single key, sizes that no vector width
divides, and one model without any attention (no pages at all).  Weights are made with NumPy
and rounded to bfloat16, so both engines and the plain model read the same numbers.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import save_file


def attention(heads, kv_heads, dim, window, scale, ff=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                                           "mask": {"size": window}, "scale": scale},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def mingru(width, ff=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(vocab, width, layers, *, scale, eps, side):
    return {"architecture": "Nadosun", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "token_side": {"dim": side}, "layers": layers}


# attention first; peaked scores (scale well above 1/sqrt(dim)) so that one key more or less shows
TINY_P = config(160, 64, [attention(4, 2, 32, 24, 0.45, ff=96), mingru(80), mingru(48, ff=72),
                          attention(2, 1, 16, 7, 0.7)], scale=3.0, eps=1e-5, side=8)
TINY_P_BLOCK = 16
# sizes nothing divides, one key/value head per query head, a window of one key, page size 8
TINY_Q = config(131, 90, [mingru(50), attention(3, 3, 10, 5, 1.0, ff=70), attention(3, 1, 6, 1, 0.9),
                          mingru(34, ff=26)], scale=1.0, eps=3e-6, side=5)
TINY_Q_BLOCK = 8
# the smallest sizes at which the fast bfloat16 paths run (matrix-core attention, weight-streaming products)
TINY_R = config(300, 256, [mingru(320), attention(4, 1, 64, 33, 0.3, ff=512), mingru(256, ff=384),
                           attention(8, 4, 32, 18, 0.5)], scale=7.5, eps=2e-6, side=32)
TINY_R_BLOCK = 16
# no attention anywhere: state slots only
TINY_S = config(97, 48, [mingru(40, ff=64), mingru(56)], scale=2.0, eps=1e-6, side=4)
TINY_S_BLOCK = 4

CONFIGS = {"P": (TINY_P, TINY_P_BLOCK), "Q": (TINY_Q, TINY_Q_BLOCK), "R": (TINY_R, TINY_R_BLOCK),
           "S": (TINY_S, TINY_S_BLOCK)}


def bf16_round(values: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().float().numpy()


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    w, v, side = cfg["width"], cfg["vocab"], cfg["token_side"]["dim"]
    shapes: dict[str, tuple[int, ...]] = {"embed": (v, w), "side.embed": (v, side * len(cfg["layers"])),
                                          "final.norm": (), "head": (v, w)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = ()
        shapes[p + "ls1"] = (w,)
        if layer["type"] == "mingru":
            for n in ("z", "x", "g"):
                shapes[p + "mix." + n] = (m["width"], w)
            shapes[p + "mix.z.b"] = shapes[p + "mix.x.b"] = (m["width"],)
            shapes[p + "mix.o"] = (w, m["width"])
        else:
            q, k = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            shapes.update({p + "mix.q": (q, w), p + "mix.k": (k, w), p + "mix.q.norm": (q,), p + "mix.k.norm": (k,),
                           p + "mix.o": (w, q)})
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            shapes.update({p + "norm2": (), p + "ls2": (w,), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff),
                           p + "mlp.act": (4,)})
        shapes.update({p + "side.gate": (side, w), p + "side.proj": (w, side), p + "side.norm": (w,)})
    return shapes


def make_weights(cfg: dict, seed: int) -> dict[str, np.ndarray]:
    """Activations of order one everywhere; gains, layer scales and norm weights spread around
    one (so that a gain or a scale left out shows), biases and activation coefficients of order one."""
    rng = np.random.default_rng(seed)
    out: dict[str, np.ndarray] = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        leaf = name.split(".", 1)[-1] if name.startswith("l") else name
        if shape == ():
            values = rng.uniform(0.6, 1.6, size=())
        elif leaf in ("ls1", "ls2", "side.norm", "mix.q.norm", "mix.k.norm"):
            values = rng.uniform(0.5, 1.5, size=shape)
        elif leaf in ("mix.z.b", "mix.x.b"):
            values = rng.standard_normal(shape)
        elif leaf == "mlp.act":
            values = np.array([0.9, 0.5, -0.3, 0.2]) + 0.1 * rng.standard_normal(4)
        elif name in ("embed", "side.embed"):
            values = rng.standard_normal(shape)
        else:
            values = rng.standard_normal(shape) / np.sqrt(shape[1])
        out[name] = bf16_round(np.asarray(values, dtype=np.float32)).reshape(shape)
    return out


def write_model_dir(path: Path, cfg: dict, weights: dict[str, np.ndarray], dtype=torch.bfloat16) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    with (path / "config.json").open("w") as handle:
        json.dump(cfg, handle)
    tensors = {k: torch.from_numpy(np.ascontiguousarray(v, dtype=np.float32)).reshape(v.shape).to(dtype) for k, v in weights.items()}
    save_file(tensors, str(path / "model.safetensors"))
    return path


def random_tokens(cfg: dict, length: int, seed: int) -> list[int]:
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=length).tolist()
