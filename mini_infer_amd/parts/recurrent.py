"""Recurrent mixers: state of fixed size per request instead of pages of keys and values.

`MinGRU` is a gated recurrence whose gates read only the current token, so all gates of a
portion come from one stacked product and only the recurrence itself walks the tokens:

    z_t = sigmoid(W_z h_t + b_z)        u_t = W_x h_t + b_x
    c_t = u_t + 1/2  where u_t >= 0,  sigmoid(u_t)  where u_t < 0
    S_t = (1 - z_t) S_(t-1) + z_t c_t   (per column)
    y_t = W_o (S_t * silu(W_g h_t))

S starts at zero, is float32 whatever the compute dtype, and lives in the request's state
slot between steps (`cache.state`, one row per slot).
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import (
    CacheNeeds,
    LayerCache,
    Mixer,
    ParamSpec,
    StateNeeds,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.parts.linear import Linear
from mini_infer_amd.registry import register_mixer

DEFAULT_NAMES = {"z": "z", "x": "x", "g": "g", "o": "o", "z_bias": "z.b", "x_bias": "x.b"}


class MinGRU(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, width: int, dtype: torch.dtype, device, *, names: dict[str, str] | None = None,
                 suffix: str = "") -> None:
        super().__init__(dtype, device)
        if hidden_size <= 0 or width <= 0:
            raise ValueError(f"minGRU needs positive sizes, got hidden_size={hidden_size} width={width}")
        self.hidden_size = hidden_size
        self.width = width
        self.names = {**DEFAULT_NAMES, **(names or {})}
        n = self.names
        # one product yields [z | x | g] for every token of the step
        self.zxg = Linear(hidden_size, [width, width, width], [n["z"], n["x"], n["g"]], dtype, device, suffix=suffix)
        self.out = Linear(width, hidden_size, n["o"], dtype, device, suffix=suffix)
        self.bias_z: torch.Tensor | None = None
        self.bias_x: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {
            **self.zxg.param_specs(prefix),
            **self.out.param_specs(prefix),
            prefix + self.names["z_bias"]: ParamSpec((self.width,), dtype="float32"),
            prefix + self.names["x_bias"]: ParamSpec((self.width,), dtype="float32"),
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.zxg.load_params(prefix, get)
        self.out.load_params(prefix, get)
        self.bias_z = get(prefix + self.names["z_bias"]).float().contiguous()
        self.bias_x = get(prefix + self.names["x_bias"]).float().contiguous()

    def cache_needs(self, page_size: int) -> CacheNeeds:
        return CacheNeeds(state=StateNeeds((self.width,), torch.float32))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if not writes_cache:
            raise NotImplementedError("a recurrent mixer owns its state; it cannot read another call's")
        assert self.bias_z is not None and self.bias_x is not None, "minGRU used before its weights were loaded"
        assert isinstance(cache.state, torch.Tensor), "minGRU needs its state rows from the cache manager"
        assert self.zxg.weight is not None
        if (
            ctx.host_cu_seqlens_q is not None
            and ctx.max_q_len == 1
            and x.shape[0] == ctx.state_slots.numel()
            and ops.linear_gru_takes(x, self.zxg.weight)
        ):
            # a step of single tokens, few rows: the stacked product and the step of the recurrence are one kernel
            gated = ops.linear_gru(x, self.zxg.weight, self.bias_z, self.bias_x, cache.state, ctx.state_slots)
            return self.out.forward(gated)
        projected = self.zxg.forward(x)
        # (the most rows a request brings: known only where the host knows the step's boundaries)
        max_rows = ctx.max_q_len if ctx.host_cu_seqlens_q is not None else None
        gated = ops.gated_scan(projected, self.bias_z, self.bias_x, cache.state, ctx.cu_seqlens_q, ctx.state_slots, max_rows)
        return self.out.forward(gated)


@register_mixer("min_gru")
def build_min_gru(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> MinGRU:
    return MinGRU(int(desc["hidden_size"]), int(desc["width"]), dtype, device, names=desc.get("names"),
                  suffix=str(desc.get("suffix", "")))
