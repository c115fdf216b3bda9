"""Zekonex, the plain way: NumPy float64, one function per mechanism, loops over tokens.

The yardstick the engine's Zekonex is measured against.  It shares no code with the
package: it reads the raw config.json keys itself, keeps no cache (every call sees a whole
sequence, or carries an explicit state dict for the recurrent mixer) and evaluates every
sum in 64-bit.

Notation: `x` is the stream [T, W]; `h` a normed copy of it; `p` positions counted from 0.

`store` (default: nothing) is applied to every tensor an engine would keep in its compute dtype
(projections, activations, sublayer outputs, cached rows; never the stream, the recurrent state
or anything inside a softmax or a norm).  With `bf16_round` the model shows how far bfloat16
storage alone, with exact arithmetic between, moves the logits: the yardstick of the bfloat16 tests.
"""

from __future__ import annotations

import math

import numpy as np

def keep(a):
    return a


def bf16_round(a: np.ndarray) -> np.ndarray:
    import torch

    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).bfloat16().double().numpy()


L2_EPS = 1e-6  # inside the root of the unit norms of the delta mixer
GATE_SLOPE = 1.702  # of the feed-forward's logistic gate


def rms_norm(x: np.ndarray, weight: np.ndarray | None, eps: float) -> np.ndarray:
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if weight is None else y * weight


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * logistic(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rotate_pairs(v: np.ndarray, position: int, base: float, dims: int) -> np.ndarray:
    """Rotate the first `dims` entries of the vector `v`, entry 2i with entry 2i+1, by the
    angle position * base^(-2i/dims); the rest pass."""
    out = np.array(v, dtype=np.float64)
    for i in range(dims // 2):
        angle = position * base ** (-2.0 * i / dims)
        a, b = v[2 * i], v[2 * i + 1]
        out[2 * i] = a * math.cos(angle) - b * math.sin(angle)
        out[2 * i + 1] = b * math.cos(angle) + a * math.sin(angle)
    return out


# ----------------------------------------------------------------------------------------
# mixers: each takes h [T, W] for positions first .. first + T - 1 of one sequence
# ----------------------------------------------------------------------------------------


def sink_attention(h: np.ndarray, w: dict, m: dict, first: int = 0, past: dict | None = None, store=keep) -> np.ndarray:
    """Grouped-query causal attention whose softmax has one more term in the denominator: a
    sink of score 0 that carries no value.  `past` (optional) holds the rotated keys and the
    values of the positions before `first` and is extended in place."""
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot")
    tokens = h.shape[0]
    q = store(h @ w["q"].T).reshape(tokens, heads, dim)
    k = store(h @ w["k"].T).reshape(tokens, groups, dim)
    v = store(h @ w["v"].T).reshape(tokens, groups, vdim)
    if rot is not None:
        for t in range(tokens):
            for a in range(heads):
                q[t, a] = rotate_pairs(q[t, a], first + t, rot["base"], rot["dims"])
            for g in range(groups):
                k[t, g] = rotate_pairs(k[t, g], first + t, rot["base"], rot["dims"])
        q, k = store(q), store(k)
    if past is not None:
        keys = np.concatenate([past["k"], k]) if "k" in past else k
        values = np.concatenate([past["v"], v]) if "v" in past else v
        past["k"], past["v"] = keys, values
    else:
        keys, values = k, v
    out = np.zeros((tokens, heads, vdim))
    per_group = heads // groups
    for t in range(tokens):
        visible = first + t + 1
        for a in range(heads):
            g = a // per_group
            s = keys[:visible, g] @ q[t, a] * m["scale"]
            top = max(s.max(), 0.0)
            e = np.exp(s - top)
            out[t, a] = (e @ values[:visible, g]) / (math.exp(-top) + e.sum())
    return store(store(out).reshape(tokens, heads * vdim) @ w["o"].T)


def latent_attention(h: np.ndarray, w: dict, m: dict, eps: float, first: int = 0, past: dict | None = None, store=keep) -> np.ndarray:
    """Attention whose keys and values are expanded per head from one small latent per token,
    beside one rotated key part that all heads share.  `past` holds latents and rotated parts."""
    heads, dim, rdim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base = m["rot"]["base"]
    tokens = h.shape[0]
    q = store(h @ w["q"].T).reshape(tokens, heads, dim + rdim)
    down = store(h @ w["dkv"].T)
    latent = store(rms_norm(down[:, :rank], w["dkv.norm"], eps))
    shared = store(np.stack([rotate_pairs(down[t, rank:], first + t, base, rdim) for t in range(tokens)]))
    if past is not None:
        latent = np.concatenate([past["c"], latent]) if "c" in past else latent
        shared = np.concatenate([past["r"], shared]) if "r" in past else shared
        past["c"], past["r"] = latent, shared
    k_plain = store(latent @ w["uk"].T).reshape(-1, heads, dim)
    values = store(latent @ w["uv"].T).reshape(-1, heads, vdim)
    out = np.zeros((tokens, heads, vdim))
    for t in range(tokens):
        visible = first + t + 1
        for a in range(heads):
            q_turn = rotate_pairs(q[t, a, dim:], first + t, base, rdim)
            s = (k_plain[:visible, a] @ q[t, a, :dim] + shared[:visible] @ q_turn) * m["scale"]
            e = np.exp(s - s.max())
            out[t, a] = (e @ values[:visible, a]) / e.sum()
    return store(store(out).reshape(tokens, heads * vdim) @ w["o"].T)


def new_delta_state(m: dict) -> dict:
    taps = m["conv"]
    return {
        "S": np.zeros((m["heads"], m["dim"], m["vdim"])),
        "q": np.zeros((taps - 1, m["kv_heads"] * m["dim"])),
        "k": np.zeros((taps - 1, m["kv_heads"] * m["dim"])),
        "v": np.zeros((taps - 1, m["heads"] * m["vdim"])),
    }


def short_convolution(z: np.ndarray, taps_weight: np.ndarray, tail: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per channel c: y[t, c] = sum_j taps_weight[c, j] * z[t - (taps - 1) + j, c], with `tail`
    (the taps - 1 inputs before z) standing in front; returns y and the new tail."""
    taps = taps_weight.shape[1]
    padded = np.concatenate([tail, z])
    y = np.zeros_like(z)
    for t in range(z.shape[0]):
        for j in range(taps):
            y[t] += taps_weight[:, j] * padded[t + j]
    return y, padded[padded.shape[0] - (taps - 1):]


def gated_delta(h: np.ndarray, w: dict, m: dict, eps: float, state: dict, store=keep) -> np.ndarray:
    """The gated delta rule, token by token; `state` (see `new_delta_state`) is updated in place."""
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    tokens = h.shape[0]
    q, state["q"] = short_convolution(store(h @ w["q"].T), w["q.conv"], state["q"])
    k, state["k"] = short_convolution(store(h @ w["k"].T), w["k.conv"], state["k"])
    v, state["v"] = short_convolution(store(h @ w["v"].T), w["v.conv"], state["v"])
    q = store(silu(q)).reshape(tokens, groups, dim)
    k = store(silu(k)).reshape(tokens, groups, dim)
    v = store(silu(v)).reshape(tokens, heads, vdim)
    q = q / np.sqrt(np.sum(q * q, axis=-1, keepdims=True) + L2_EPS) * dim ** -0.5
    k = k / np.sqrt(np.sum(k * k, axis=-1, keepdims=True) + L2_EPS)
    write = logistic(store(h @ w["b"].T))  # [T, heads]
    decay = np.exp(-np.exp(w["A_log"]) * softplus(store(h @ w["a"].T) + w["dt_bias"]))  # [T, heads]
    gate = silu(store(h @ w["g"].T)).reshape(tokens, heads, vdim)
    per_group = heads // groups
    out = np.zeros((tokens, heads, vdim))
    for t in range(tokens):
        for a in range(heads):
            g = a // per_group
            S = state["S"][a] * decay[t, a]
            u = write[t, a] * (v[t, a] - S.T @ k[t, g])
            S = S + np.outer(k[t, g], u)
            state["S"][a] = S
            out[t, a] = rms_norm(S.T @ q[t, g], w["norm"], eps) * gate[t, a]
    return store(store(out).reshape(tokens, heads * vdim) @ w["o"].T)


# ----------------------------------------------------------------------------------------
# feed-forward, layer, model
# ----------------------------------------------------------------------------------------


def clamped_gated_feed_forward(h: np.ndarray, w: dict, limit: float, store=keep) -> np.ndarray:
    g = np.minimum(store(h @ w["gate"].T) + w["gate.b"], limit)
    u = np.clip(store(h @ w["up"].T) + w["up.b"], -limit, limit)
    return store(store(g * logistic(GATE_SLOPE * g) * (u + 1.0)) @ w["down"].T) + w["down.b"]


def split_weights(weights: dict, prefix: str) -> dict:
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def layer_runs(config: dict) -> list[tuple[int, int | None]]:
    """(layer, number of the pass it opens or None) in running order."""
    loop, count = config.get("loop"), len(config["layers"])
    if not loop:
        return [(i, None) for i in range(count)]
    runs = [(i, None) for i in range(loop["start"])]
    for turn in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            runs.append((i, turn if i == loop["start"] else None))
    return runs + [(i, None) for i in range(loop["stop"], count)]


class PlainZekonex:
    """`weights`: tensor name -> float64 array.  A sequence is fed in portions through
    `forward(tokens, memory)`; `memory` (a dict, empty at first) carries what the mixers keep."""

    def __init__(self, config: dict, weights: dict, store=keep) -> None:
        self.config, self.weights, self.store = config, weights, store
        self.runs = layer_runs(config)

    def forward(self, tokens, memory: dict | None = None, streams: list | None = None) -> np.ndarray:
        cfg, w, store = self.config, self.weights, self.store
        memory = {} if memory is None else memory
        first = memory.get("length", 0)
        eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
        x = w["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
        for run, (i, opens) in enumerate(self.runs):
            layer, lw = cfg["layers"][i], split_weights(w, f"l{i}.")
            if opens is not None:
                x = x + w["loop.step"][opens]
            h = store(rms_norm(x, lw["norm1"], eps))
            mw, kind = split_weights(lw, "mix."), layer["type"]
            if kind == "attention":
                mixer = dict(layer["mixer"])
                mixer.setdefault("vdim", mixer["dim"])
                mixed = sink_attention(h, mw, mixer, first, memory.setdefault(run, {}), store)
            elif kind == "latent_attention":
                mixed = latent_attention(h, mw, layer["mixer"], eps, first, memory.setdefault(run, {}), store)
            elif kind == "delta":
                if run not in memory:
                    memory[run] = new_delta_state(layer["mixer"])
                mixed = gated_delta(h, mw, layer["mixer"], eps, memory[run], store)
            else:
                raise ValueError(f"unknown layer type {kind!r}")
            if layer.get("mlp") is not None:
                mixed = mixed + clamped_gated_feed_forward(h, split_weights(lw, "mlp."), layer["mlp"]["limit"], store)
            x = x + mult * mixed
            if streams is not None:
                streams.append(x.copy())
        memory["length"] = first + len(tokens)
        return store(store(rms_norm(x, w["final.norm"], eps)) @ w["head"].T)  # (the engine's head rounds its product too)


def logits(config: dict, weights: dict, tokens, store=keep) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence."""
    return PlainZekonex(config, weights, store).forward(tokens)


def greedy(row: np.ndarray) -> int:
    return int(np.argmax(row))
