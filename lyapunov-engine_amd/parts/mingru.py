"""minGRU: a gated recurrence whose gates read the current token only.

    z_t = sigmoid(W_z x_t + b_z)        u_t = W_x x_t + b_x
    c_t = u_t + 1/2  where u_t >= 0,    sigmoid(u_t)  below
    S_t = (1 - z_t) S_(t-1) + z_t c_t   (element by element, S_0 = 0)
    y_t = W_o (S_t * silu(W_g x_t))

The three input projections are one matrix; gates, candidate and state are
32-bit, the state lives in a slot per live request.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS
from ..kernels import ops
from .base import LayerCache, Mixer, StateSpec, StepContext, WeightSource, WeightSpec


@MIXERS.register("mingru")
class MinGRU(Mixer):
    def __init__(self, hidden_size: int, width: int, names: Optional[dict] = None):
        self.hidden_size, self.width = int(hidden_size), int(width)
        n = dict(z="z", z_bias="z.b", x="x", x_bias="x.b", g="g", o="o")
        n.update(names or {})
        self.names = n
        self.in_proj: Optional[torch.Tensor] = None
        self.z_bias = self.x_bias = self.out_proj = None
        self.z_bias_f = self.x_bias_f = None

    CHUNKED_FROM = 32   # mean rows per request from which the scan runs in chunks

    def weight_specs(self):
        n, shape = self.names, (self.width, self.hidden_size)
        return [
            WeightSpec("in_proj", (WeightSource(n["z"], shape), WeightSource(n["x"], shape), WeightSource(n["g"], shape))),
            WeightSpec("z_bias", (WeightSource(n["z_bias"], (self.width,)),)),
            WeightSpec("x_bias", (WeightSource(n["x_bias"], (self.width,)),)),
            WeightSpec("out_proj", (WeightSource(n["o"], (self.hidden_size, self.width)),)),
        ]

    def materialize(self, device, dtype):
        self.z_bias_f = self.z_bias.float().contiguous()
        self.x_bias_f = self.x_bias.float().contiguous()

    def state_spec(self):
        return StateSpec((self.width,), torch.float32)

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        pre = ops.linear(x, self.in_proj, out_dtype=torch.float32)
        gated = torch.empty((ctx.T, self.width), dtype=ctx.dtype, device=pre.device)
        # long runs of rows go in chunks side by side; a step of few rows per request walks them in order
        ws = ctx.scratch("mingru_chunks", ops.mingru_scan_workspace(ctx.T, ctx.B, self.width)) \
            if ctx.T > self.CHUNKED_FROM * ctx.B else None
        ops.mingru_scan(pre, self.z_bias_f, self.x_bias_f, cache.state, ctx.q_start, ctx.positions, ctx.state_slots,
                        gated, ctx.B, ws)
        return ops.linear(gated, self.out_proj, out_dtype=ctx.dtype)
