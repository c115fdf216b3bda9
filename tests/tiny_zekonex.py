"""Tiny Zekonex configurations, weights and model folders for the tests.

The configurations differ in every size and constant, in the order of layers and in how
the stack loops: a loop that starts at the first layer and holds a recurrent layer (every pass
then has state of its own), a loop over one layer, none; value heads wider and narrower than
query heads; as many key/value heads as query heads and a single one; rotation of a whole head,
of a part, of nothing; a convolution of one tap (no tail to carry), two and five; sizes that no
vector width divides (odd head sizes where the kernels take them); layers without a
feed-forward; a model without any attention (no pages at all).  Weights are made with NumPy and
rounded to bfloat16, so both engines and the plain model read the same numbers.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import save_file


def mlp(ff, limit):
    return None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}


def attention(heads, kv_heads, dim, vdim, scale, rot=None, ff=None, limit=1.0):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "attention", "mixer": mixer, "mlp": mlp(ff, limit)}


def delta(heads, kv_heads, dim, vdim, conv, ff=None, limit=1.0):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp(ff, limit)}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base, ff=None, limit=1.0):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim}},
            "mlp": mlp(ff, limit)}


def config(vocab, width, layers, *, scale, eps, mult, loop=None):
    out = {"architecture": "Zekonex", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
           "residual_mult": mult, "layers": layers}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


# the loop starts at layer 0 and holds a recurrent layer; peaked scores (scales well above
# 1/sqrt(dim)) so that one key more or less shows; value heads wider than query heads
TINY_A = config(160, 64, [
    delta(4, 4, 12, 20, 3, ff=96, limit=0.8),
    attention(4, 2, 16, 24, 0.9, rot=(100.0, 8), ff=80, limit=2.0),
    latent(3, 10, 6, 14, 22, 0.8, 50.0),
    delta(2, 1, 16, 8, 5),
], scale=3.0, eps=1e-5, mult=0.5, loop=(0, 2, 3))
TINY_A_BLOCK = 16
# sizes nothing divides; a single tap; whole heads rotated; value heads narrower; page size 8
TINY_B = config(131, 90, [
    attention(3, 3, 10, 6, 1.1, rot=(1000.0, 10), ff=70, limit=1.2),
    delta(3, 1, 7, 9, 1, ff=26, limit=0.5),
    latent(5, 6, 2, 10, 18, 1.3, 7.0, ff=50, limit=3.0),
    attention(2, 1, 6, 6, 0.7),
    delta(6, 3, 5, 6, 2),
], scale=1.0, eps=3e-6, mult=1.0, loop=(2, 3, 2))
TINY_B_BLOCK = 8
# sizes at which the fast bfloat16 paths run (weight-streaming products, whole vector loads)
TINY_C = config(300, 256, [
    latent(4, 32, 32, 64, 96, 0.25, 10000.0, ff=512, limit=1.5),
    attention(8, 2, 64, 64, 0.3, rot=(500000.0, 32), ff=384, limit=1.5),
    delta(4, 2, 64, 128, 4, ff=256, limit=1.0),
    attention(4, 4, 32, 64, 0.45, rot=(10000.0, 32)),
], scale=7.5, eps=2e-6, mult=0.3)
TINY_C_BLOCK = 16
# no attention anywhere: state slots only, a loop over everything
TINY_D = config(97, 48, [delta(2, 2, 8, 8, 4, ff=64, limit=1.0), delta(3, 1, 20, 12, 2)], scale=2.0, eps=1e-6, mult=0.7,
                loop=(0, 2, 2))
TINY_D_BLOCK = 4

# the largest heads the kernels take and the corners of their fast paths: a latent layer whose value
# heads are wider than its expanded key heads (prompts then take the folded form in bfloat16 too) and one
# with the smallest head size the matrix cores take; attention heads of 128 with a sink on the matrix
# cores, and value heads half as wide as the query heads (plain kernel); a delta rule of 256 x 256 with two
# taps; the loop runs to the last layer
TINY_E = config(200, 128, [
    attention(2, 2, 128, 128, 0.12, rot=(10000.0, 128), ff=192, limit=2.5),
    latent(2, 48, 16, 96, 40, 0.3, 300.0, ff=64, limit=1.0),
    delta(2, 1, 256, 256, 2),
    latent(2, 24, 8, 16, 64, 0.4, 20000.0),
    attention(4, 1, 64, 32, 0.25, rot=(50.0, 2), ff=96, limit=0.9),
], scale=4.0, eps=1e-6, mult=0.4, loop=(1, 5, 3))
TINY_E_BLOCK = 16

CONFIGS = {"A": (TINY_A, TINY_A_BLOCK), "B": (TINY_B, TINY_B_BLOCK), "C": (TINY_C, TINY_C_BLOCK), "D": (TINY_D, TINY_D_BLOCK),
           "E": (TINY_E, TINY_E_BLOCK)}


def bf16_round(values: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().float().numpy()


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    w, v = cfg["width"], cfg["vocab"]
    shapes: dict[str, tuple[int, ...]] = {"embed": (v, w), "final.norm": (w,), "head": (v, w)}
    if cfg.get("loop"):
        shapes["loop.step"] = (cfg["loop"]["times"], w)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = (w,)
        if layer["type"] == "attention":
            shapes.update({p + "mix.q": (m["heads"] * m["dim"], w), p + "mix.k": (m["kv_heads"] * m["dim"], w),
                           p + "mix.v": (m["kv_heads"] * m["vdim"], w), p + "mix.o": (w, m["heads"] * m["vdim"])})
        elif layer["type"] == "latent_attention":
            shapes.update({p + "mix.q": (m["heads"] * (m["dim"] + m["rot_dim"]), w), p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], w),
                           p + "mix.dkv.norm": (m["kv_rank"],), p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]),
                           p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]), p + "mix.o": (w, m["heads"] * m["vdim"])})
        else:
            qk, vw = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (qk, w), p + "mix.k": (qk, w), p + "mix.v": (vw, w), p + "mix.q.conv": (qk, m["conv"]),
                           p + "mix.k.conv": (qk, m["conv"]), p + "mix.v.conv": (vw, m["conv"]), p + "mix.b": (m["heads"], w),
                           p + "mix.a": (m["heads"], w), p + "mix.A_log": (m["heads"],), p + "mix.dt_bias": (m["heads"],),
                           p + "mix.norm": (m["vdim"],), p + "mix.g": (vw, w), p + "mix.o": (w, vw)})
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            shapes.update({p + "mlp.gate": (ff, w), p + "mlp.gate.b": (ff,), p + "mlp.up": (ff, w), p + "mlp.up.b": (ff,),
                           p + "mlp.down": (w, ff), p + "mlp.down.b": (w,)})
    return shapes


def make_weights(cfg: dict, seed: int) -> dict[str, np.ndarray]:
    """Activations of order one everywhere; norm weights spread around one (a weight left out
    shows), biases of order one (a bias left out, or a clamp, shows), decay rates and step
    biases such that a head forgets over a few to a few dozen tokens, loop vectors of order one."""
    rng = np.random.default_rng(seed)
    out: dict[str, np.ndarray] = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        leaf = name.split(".", 1)[-1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "final.norm", "mix.dkv.norm", "mix.norm"):
            values = rng.uniform(0.5, 1.5, size=shape)
        elif leaf in ("mlp.gate.b", "mlp.up.b", "mlp.down.b", "loop.step", "mix.dt_bias"):
            values = rng.standard_normal(shape)
        elif leaf == "mix.A_log":
            values = rng.uniform(-2.5, 0.5, size=shape)
        elif leaf.endswith(".conv"):
            values = rng.standard_normal(shape) * 0.6
        elif name == "embed":
            values = rng.standard_normal(shape)
        else:
            values = rng.standard_normal(shape) / np.sqrt(shape[1]) * (2.0 if leaf in ("mix.q", "mix.k") else 1.0)
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
