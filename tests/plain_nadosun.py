"""A plain, slow Nadosun in NumPy float64: one function per mechanism, one token loop per recurrence.

It shares no code with the engine and reads the model the way a checkpoint stores it: a
raw configuration dictionary and tensors by name.  `store` rounds what an engine in
bfloat16 keeps in bfloat16 (the outputs of matrix products and the activations between
them), so that the same code gives the yardstick for the bfloat16 engine.

Notation: r is the residual stream [T, W]; a layer adds ls1 * N1(mix(r)), then, where it has
a feed-forward, ls2 * N2(ff(r)), then the token side input.  N is the one-gain norm
y / sqrt(mean(y^2) + eps) * gain.
"""

from __future__ import annotations

import numpy as np

SINUSOID_BASE = 10000.0
GELU_CUBIC = 0.044715


def _same(x):
    return x


def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """Rows of x divided by their root mean square, eps under the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + GELU_CUBIC * z**3)))


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-z))


def silu(z: np.ndarray) -> np.ndarray:
    return z * sigmoid(z)


def sinusoid(positions: np.ndarray, width: int) -> np.ndarray:
    """[T, width]: column 2i holds sin(p * base^(-2i/width)), column 2i+1 the cosine of the same angle."""
    out = np.zeros((len(positions), width))
    pairs = np.arange((width + 1) // 2)
    angle = positions[:, None].astype(np.float64) * SINUSOID_BASE ** (-2.0 * pairs / width)[None, :]
    out[:, 0::2] = np.sin(angle)[:, : out[:, 0::2].shape[1]]
    out[:, 1::2] = np.cos(angle)[:, : out[:, 1::2].shape[1]]
    return out


def embedding(table: np.ndarray, tokens: np.ndarray, scale: float, first_position: int = 0) -> np.ndarray:
    positions = first_position + np.arange(len(tokens))
    return table[tokens].astype(np.float64) * scale + sinusoid(positions, table.shape[1])


def gated_recurrence(z_in, u, gate, state=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t, token by token, from the gates' inputs (biases already
    added).  Returns (S_t * silu(gate_t) for every t, the last S)."""
    z = sigmoid(z_in)
    candidate = np.where(u >= 0, u + 0.5, sigmoid(u))
    s = np.zeros(z.shape[1]) if state is None else np.array(state, dtype=np.float64)
    rows = []
    for t in range(z.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * candidate[t]
        rows.append(s * silu(gate[t]))
    return np.array(rows).reshape(z.shape[0], -1), s


def min_gru(h, w, prefix, state=None, store=_same):
    """The gated recurrence over the rows of h.  Returns (output rows, last state)."""
    f = lambda name: w[prefix + name].astype(np.float64)  # noqa: E731
    z_in = store(h @ f("z").T) + f("z.b")
    u = store(h @ f("x").T) + f("x.b")
    gate = store(h @ f("g").T)
    rows, s = gated_recurrence(z_in, u, gate, state)
    return store(store(rows) @ f("o").T), s


def windowed_attention(h, w, prefix, mixer, eps, store=_same, past_k=None, past_v=None):
    """Keys double as values: the values are the key projection before its norm.  q and k are
    normed over their whole projection (all heads at once).  A query at position i sees the
    keys at i - window + 1 .. i.  Returns (output rows, normed keys so far, values so far)."""
    f = lambda name: w[prefix + name].astype(np.float64)  # noqa: E731
    heads, groups, dim = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"])
    window, scale = int(mixer["mask"]["size"]), float(mixer["scale"])
    q_raw, k_raw = store(h @ f("q").T), store(h @ f("k").T)
    q = store(rms(q_raw, eps) * f("q.norm"))
    k = store(rms(k_raw, eps) * f("k.norm"))
    v = k_raw
    if past_k is not None:
        k, v = np.concatenate([past_k, k]), np.concatenate([past_v, v])
    first = k.shape[0] - h.shape[0]
    out = np.zeros((h.shape[0], heads * dim))
    for t in range(h.shape[0]):
        i = first + t
        lo = max(0, i - window + 1)
        for head in range(heads):
            g = head // (heads // groups)
            keys = k[lo : i + 1, g * dim : (g + 1) * dim]
            scores = keys @ q[t, head * dim : (head + 1) * dim] * scale
            p = np.exp(scores - scores.max())
            p /= p.sum()
            out[t, head * dim : (head + 1) * dim] = p @ v[lo : i + 1, g * dim : (g + 1) * dim]
    return store(store(out) @ f("o").T), k, v


def poly_norm(z: np.ndarray, coefficients: np.ndarray, eps: float) -> np.ndarray:
    a, b, c, e = (float(x) for x in coefficients)
    return a * rms(z, eps) + b * rms(z**2, eps) + c * rms(z**3, eps) + e


def dense_feed_forward(h, w, prefix, eps, store=_same):
    f = lambda name: w[prefix + name].astype(np.float64)  # noqa: E731
    act = store(poly_norm(store(h @ f("up").T), f("act"), eps))
    return store(act @ f("down").T)


def token_side(r, tokens, w, layer: int, dim: int, eps: float, store=_same):
    """What the per-layer token input adds to the stream: a slice of the side table, gated by the
    stream, projected to the width and normed with a per-column weight."""
    p = f"l{layer}.side."
    e = w["side.embed"][tokens, layer * dim : (layer + 1) * dim].astype(np.float64)
    h = store(r)
    g = store(gelu_tanh(store(h @ w[p + "gate"].astype(np.float64).T)) * e)
    y = store(g @ w[p + "proj"].astype(np.float64).T)
    return rms(y, eps) * w[p + "norm"].astype(np.float64)


def layer_forward(r, tokens, cfg, w, layer: int, carry=None, store=_same):
    """One layer on the rows of r; `carry` is what the layer's mixer kept from earlier portions."""
    desc = cfg["layers"][layer]
    eps = float(cfg["norm"]["eps"])
    p = f"l{layer}."
    h = store(r)
    if desc["type"] == "mingru":
        mixed, carry = min_gru(h, w, p + "mix.", carry, store)
    elif desc["type"] == "attention":
        past_k, past_v = carry if carry is not None else (None, None)
        mixed, k, v = windowed_attention(h, w, p + "mix.", desc["mixer"], eps, store, past_k, past_v)
        carry = (k, v)
    else:
        raise ValueError(desc["type"])
    r = r + rms(mixed, eps) * float(w[p + "norm1"]) * w[p + "ls1"].astype(np.float64)
    if desc.get("mlp") is not None:
        fed = dense_feed_forward(store(r), w, p + "mlp.", eps, store)
        r = r + rms(fed, eps) * float(w[p + "norm2"]) * w[p + "ls2"].astype(np.float64)
    r = r + token_side(r, tokens, w, layer, int(cfg["token_side"]["dim"]), eps, store)
    return r, carry


def logits(cfg, w, tokens, store=_same, cuts=None, streams=None):
    """Logits [T, vocab] of one request.  `cuts`: feed the tokens in portions of these sizes
    (the carried state makes the result the same); `streams`, if a list, receives the stream after every layer."""
    tokens = np.asarray(tokens)
    cuts = [len(tokens)] if cuts is None else list(cuts)
    assert sum(cuts) == len(tokens)
    carries = [None] * len(cfg["layers"])
    eps = float(cfg["norm"]["eps"])
    out, at = [], 0
    per_layer = [[] for _ in cfg["layers"]]
    for n in cuts:
        ids = tokens[at : at + n]
        r = embedding(w["embed"], ids, float(cfg["embedding"]["scale"]), at)
        for layer in range(len(cfg["layers"])):
            r, carries[layer] = layer_forward(r, ids, cfg, w, layer, carries[layer], store)
            per_layer[layer].append(r)
        final = store(rms(r, eps) * float(w["final.norm"]))
        out.append(store(final @ w["head"].astype(np.float64).T))  # (the bfloat16 engine's head rounds its product too)
        at += n
    if streams is not None:
        streams.extend(np.concatenate(rows) for rows in per_layer)
    return np.concatenate(out)


def greedy(row: np.ndarray) -> int:
    return int(np.argmax(row))


def bf16_round(values: np.ndarray) -> np.ndarray:
    import torch

    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().double().numpy()
