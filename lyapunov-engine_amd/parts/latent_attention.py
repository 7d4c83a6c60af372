"""Attention through low-rank latents, over a paged cache of latents.

Per token x:
    c_q = rmsnorm(W_dq x)                       q   = W_uq c_q   (per head: dim plain, rot_dim to rotate)
    [c | r] = W_dkv x, c = rmsnorm(c)           r: one key part for all heads, rotated by position
    key_h = [W_uk,h c | r],  value_h = W_uv,h c
    weights = softmax over {scale * q_h . key_h (causal), sink_h}, the sink without a value
    y = W_o concat_h(sum weights * value_h)

Only (c, r) is kept per token: kv_rank + rot_dim numbers, whatever the number of
heads.  The scores and sums are taken on the latents themselves:
q_h . W_uk,h c = (W_uk,h^T q_h) . c, so every head's query is carried into the
latent space once ("absorbed"), all heads then read the same key row [c | r],
whose first kv_rank values are the value as well, and W_uv,h is applied to the
head's weighted sum of latents afterwards.  A whole prompt, a portion and a
decoded token take this one path.

Rotation: neighbouring pairs (2i, 2i+1) of the first ``rot_dims`` values of the
rotated part turn by position * base^(-2i / rot_dims).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from .base import (SLOT, LayerCache, Mixer, PagedSpec, PageTensor, StepBatch, StepContext, StepPlanner, WeightSource,
                   WeightSpec)


class ContextBound(StepPlanner):
    """The longest context of the step, as a host value (``meta["max_ctx"]``; in a recorded step
    the step's bound): what a kernel that cuts the keys into partitions sizes its launch by."""

    key = ("context_bound",)

    def plan(self, batch: StepBatch) -> tuple:
        bound = batch.fixed.max_context if batch.fixed is not None else int(batch.ctx_len.max())
        return {}, dict(max_ctx=max(1, bound))


_BOUND = ContextBound()


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int,
                 kv_rank: int, scale: float, eps: float, position: Optional[PartSpec] = None,
                 names: Optional[dict] = None):
        for what, v in (("heads", num_heads), ("vdim", vdim), ("q_rank", q_rank), ("kv_rank", kv_rank)):
            if v <= 0:
                raise ValueError(f"latent attention: {what} must be positive, got {v}")
        if dim < 0 or rot_dim < 0 or dim + rot_dim == 0:
            raise ValueError(f"latent attention: a head of {dim} plain and {rot_dim} rotated dimensions")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.dim, self.rot_dim, self.vdim = int(dim), int(rot_dim), int(vdim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.position = POSITION_ENCODINGS.build(position) if position is not None and rot_dim else None
        if self.position is not None and self.position.rotary_dim > rot_dim:
            raise ValueError("more rotated dimensions than the rotated part has")
        n = dict(dq="dq", q_norm="dq.norm", uq="uq", dkv="dkv", kv_norm="dkv.norm", uk="uk", uv="uv", sink="sink", o="o")
        n.update(names or {})
        self.names = n
        # sizes in multiples of 16 take the matrix-core kernel, any others the row-by-row one
        self.matrix_cores = ops.latent_attn_fits_matrix_cores(self.kv_rank, self.rot_dim)
        self.down_proj = self.q_norm = self.kv_norm = self.uq = self.uk = self.uv = self.sink = self.o_proj = None
        self.q_norm_f = self.kv_norm_f = self.sink_f = self.uk_t = self.uv_heads = None

    def weight_specs(self):
        n, H = self.names, self.num_heads
        return [
            WeightSpec("down_proj", (WeightSource(n["dq"], (self.q_rank, self.hidden_size)),
                                     WeightSource(n["dkv"], (self.kv_rank + self.rot_dim, self.hidden_size)))),
            WeightSpec("q_norm", (WeightSource(n["q_norm"], (self.q_rank,)),), init="ones"),
            WeightSpec("kv_norm", (WeightSource(n["kv_norm"], (self.kv_rank,)),), init="ones"),
            WeightSpec("uq", (WeightSource(n["uq"], (H * (self.dim + self.rot_dim), self.q_rank)),)),
            WeightSpec("uk", (WeightSource(n["uk"], (H * self.dim, self.kv_rank)),)),
            WeightSpec("uv", (WeightSource(n["uv"], (H * self.vdim, self.kv_rank)),)),
            WeightSpec("sink", (WeightSource(n["sink"], (H,)),)),
            WeightSpec("o_proj", (WeightSource(n["o"], (self.hidden_size, H * self.vdim)),)),
        ]

    def children(self):
        return {"rotary.": self.position} if self.position is not None else {}

    def materialize(self, device, dtype):
        super().materialize(device, dtype)
        H = self.num_heads
        self.q_norm_f = self.q_norm.float().contiguous()
        self.kv_norm_f = self.kv_norm.float().contiguous()
        self.sink_f = self.sink.float().contiguous()
        # every head's W_uk as [kv_rank, dim]: the matrix that carries the head's plain query part
        # into the latent space, stored as a projection weight [out, in]
        self.uk_t = self.uk.view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous() if self.dim else None
        self.uk = None
        self.uv_heads = self.uv.view(H, self.vdim, self.kv_rank)

    def step_planner(self):
        return _BOUND

    def cache_spec(self):
        return PagedSpec((PageTensor("latent", (SLOT, self.kv_rank + self.rot_dim)),), 0)

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        if not cache.writes:
            raise RuntimeError("latent attention keeps its own latents")
        g, T, H = cache.group, ctx.T, self.num_heads
        pages = cache.pages["latent"]
        table = self.position.table if self.position is not None else None
        dev = pages.device
        down = ops.linear(x, self.down_proj, out_dtype=ctx.dtype)
        cq = torch.empty((T, self.q_rank), dtype=ctx.dtype, device=dev)
        ops.latent_prep(down, self.q_norm_f, self.kv_norm_f, ctx.positions, table, g.slot_mapping, cq, pages,
                        q_rank=self.q_rank, kv_rank=self.kv_rank, rot_dim=self.rot_dim, eps=self.eps)
        q = ops.linear(cq, self.uq, out_dtype=ctx.dtype)
        qa = torch.empty((T, H, self.kv_rank + self.rot_dim), dtype=ctx.dtype, device=dev)
        if self.dim:
            ops.gemm_nt_heads(q.view(T, H, self.dim + self.rot_dim)[:, :, :self.dim], self.uk_t, qa[:, :, :self.kv_rank])
        else:
            qa[:, :, :self.kv_rank].zero_()
        ops.latent_query_rotate(q, ctx.positions, table, qa, num_heads=H, dim=self.dim, rot_dim=self.rot_dim,
                                kv_rank=self.kv_rank)
        # a recorded step may hold rows that belong to no request: nothing writes them
        padded_rows = ctx.fixed is not None and ctx.fixed.tokens > 0
        mixed = (torch.zeros if padded_rows else torch.empty)((T, H, self.kv_rank), dtype=ctx.dtype, device=dev)
        heads = torch.empty((T, H, self.vdim), dtype=ctx.dtype, device=dev)
        if self.matrix_cores:
            launch = ops.latent_attn_launch(T, ctx.B, H, ctx.plans[ContextBound.key].meta["max_ctx"], ctx.dtype,
                                            self.kv_rank, self.rot_dim)
            part_o = part_ml = None
            if launch["n_parts"] > 1:
                part_o = ctx.scratch("latent_part_o", launch["part_o"])
                part_ml = ctx.scratch("latent_part_ml", launch["part_ml"])
            few = T * H <= ops.HEADS_OUT_MAX_ROWS and not padded_rows
            ops.latent_attn(qa, pages, g.block_tables, ctx.q_start, ctx.positions, ctx.ctx_len, self.sink_f,
                            self.scale, mixed, launch, part_o, part_ml, kv_rank=self.kv_rank, rot_dim=self.rot_dim,
                            merge=not few)
            if few:   # few rows: the partitions' merge and the heads' value projection in one kernel
                if launch["n_parts"] > 1:
                    ops.latent_heads_out(self.uv_heads, heads, kv_rank=self.kv_rank, rot_dim=self.rot_dim, part_o=part_o,
                                         part_ml=part_ml, sink=self.sink_f, n_parts=launch["n_parts"])
                else:
                    ops.latent_heads_out(self.uv_heads, heads, kv_rank=self.kv_rank, rot_dim=self.rot_dim, mixed=mixed)
                return ops.linear(heads.view(T, H * self.vdim), self.o_proj, out_dtype=ctx.dtype)
        else:
            ops.latent_attn_rows(qa, pages, g.block_tables, ctx.q_start, ctx.positions, ctx.ctx_len, self.sink_f,
                                 self.scale, mixed, kv_rank=self.kv_rank, rot_dim=self.rot_dim)
        ops.gemm_nt_heads(mixed, self.uv_heads, heads)
        return ops.linear(heads.view(T, H * self.vdim), self.o_proj, out_dtype=ctx.dtype)
