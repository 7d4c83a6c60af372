"""Grouped-query attention with normed projections, a rotation of neighbouring
pairs, a window that keeps a sequence's first tokens, and a sink.

Per token x, with H query heads and G key/value heads (query head h reads
key/value head h // (H / G)), keys and queries of ``dim`` values a head, values
of ``vdim``:

    q = W_q x, k = W_k x, v = W_v x                      one fused product
    q <- rmsnorm(q) * w_qn, k <- rmsnorm(k) * w_kn       each over the whole projection, all heads at once (``qk_norm``)
    pairs (2i, 2i+1) of the first ``rot`` values of every head turn by position * f_i   (the position encoding's table)
    position p sees key j <= p when there is no window, p - j < window, or j < keep_first
    weights = softmax over {scale * q_h . k_j (visible j), sink_h}; the sink has no value  (``sink``)
    y = W_o concat_h(sum_j weights_j v_j)

Keys and values go to the request's pages first (keys [kv head][slot][dim],
values [kv head][vdim][slot]) and attention reads pages only, so a whole prompt,
a portion and a decoded token take one path; a windowed layer's pages are given
back once the window has passed them, except those of the kept first tokens.

Heads with dim == vdim in multiples of 16 (up to 256) run on the matrix-core
kernels of ``parts.attention`` (prompt tiles, one-token requests in
partitions); any other sizes on a row-by-row kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from .attention import AttentionWork, decode_launch, prefill_launch
from .base import LayerCache, Mixer, PagedSpec, StepContext, WeightSource, WeightSpec

_WORK = AttentionWork()


@MIXERS.register("sink_window_attention")
class SinkWindowAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int = 0, keep_first: int = 0, qk_norm: bool = True, sink: bool = True, eps: float = 1e-6,
                 position: Optional[PartSpec] = None, names: Optional[dict] = None):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not split over {num_kv_heads} key/value heads")
        if dim <= 0 or vdim <= 0 or window < 0 or keep_first < 0:
            raise ValueError(f"attention: heads of {dim}/{vdim}, window {window}, {keep_first} kept first tokens")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale = int(dim), int(vdim), float(scale)
        self.window = int(window)
        self.keep_first = int(keep_first) if window else 0     # without a window every token is seen anyway
        self.qk_norm, self.has_sink, self.eps = bool(qk_norm), bool(sink), float(eps)
        self.position = POSITION_ENCODINGS.build(position) if position is not None else None
        if self.position is not None and self.position.rotary_dim > dim:
            raise ValueError("more rotated dimensions than a head has")
        n = dict(q="q", k="k", v="v", q_norm="q.norm", k_norm="k.norm", sink="sink", o="o")
        n.update(names or {})
        self.names = n
        # equal key and value sizes in multiples of 16: the matrix-core kernels
        self.matrix_cores = self.dim == self.vdim and self.dim % 16 == 0 and self.dim <= 256
        self.qkv_proj = self.o_proj = self.q_norm = self.k_norm = self.sink = None
        self.q_norm_f = self.k_norm_f = self.sink_f = None

    def weight_specs(self):
        n, H, G = self.names, self.num_heads, self.num_kv_heads
        specs = [WeightSpec("qkv_proj", (WeightSource(n["q"], (H * self.dim, self.hidden_size)),
                                         WeightSource(n["k"], (G * self.dim, self.hidden_size)),
                                         WeightSource(n["v"], (G * self.vdim, self.hidden_size)))),
                 WeightSpec("o_proj", (WeightSource(n["o"], (self.hidden_size, H * self.vdim)),))]
        if self.qk_norm:
            specs += [WeightSpec("q_norm", (WeightSource(n["q_norm"], (H * self.dim,)),), init="ones"),
                      WeightSpec("k_norm", (WeightSource(n["k_norm"], (G * self.dim,)),), init="ones")]
        if self.has_sink:
            specs.append(WeightSpec("sink", (WeightSource(n["sink"], (H,)),)))
        return specs

    def children(self):
        return {"rotary.": self.position} if self.position is not None else {}

    def materialize(self, device, dtype):
        super().materialize(device, dtype)
        if self.qk_norm:
            self.q_norm_f = self.q_norm.float().contiguous()
            self.k_norm_f = self.k_norm.float().contiguous()
        if self.has_sink:
            self.sink_f = self.sink.float().contiguous()

    def cache_spec(self):
        return PagedSpec.keys_and_values(self.num_kv_heads, self.dim, self.window, value_dim=self.vdim,
                                         keep_first=self.keep_first)

    def step_planner(self):
        return _WORK if self.matrix_cores else None

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        if not cache.writes:
            raise RuntimeError("this attention keeps its own keys and values")
        g, H, G = cache.group, self.num_heads, self.num_kv_heads
        table = self.position.table if self.position is not None else None
        qkv = ops.linear(x, self.qkv_proj, out_dtype=ctx.dtype)
        ops.qk_norm_rope_kv(qkv, self.q_norm_f, self.k_norm_f, self.eps, ctx.positions, table, g.slot_mapping,
                            cache.k, cache.v, num_heads=H, num_kv_heads=G, dim=self.dim, vdim=self.vdim,
                            page_size=g.page_size)
        out = torch.empty((ctx.T, H * self.vdim), dtype=ctx.dtype, device=qkv.device)
        if not self.matrix_cores:
            ops.attn_rows(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.positions, ctx.ctx_len,
                          num_heads=H, num_kv_heads=G, dim=self.dim, vdim=self.vdim, scale=self.scale,
                          window=self.window, keep_first=self.keep_first, sink=self.sink_f)
            return ops.linear(out, self.o_proj, out_dtype=ctx.dtype)
        common = dict(num_heads=H, num_kv_heads=G, head_dim=self.dim, window=self.window, scale=self.scale,
                      keep_first=self.keep_first, sink=self.sink_f)
        work = ctx.plans[AttentionWork.key]
        sizes = dict(num_heads=H, num_kv_heads=G, head_dim=self.dim)
        pre = prefill_launch(work.meta, ctx.dtype, g.page_size, window=self.window, **sizes)
        if pre is not None:
            part_o = part_ml = None
            if pre["parts"] > 1:
                part_o = ctx.scratch("attn_part_o", pre["part_o"])
                part_ml = ctx.scratch("attn_part_ml", pre["part_ml"])
            ops.attn_prefill(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                             work.arrays["tile_seq"], work.arrays["tile_q0"], pre["n_tiles"], pair=pre["pair"],
                             parts=pre["parts"], part_o=part_o, part_ml=part_ml, **common)
        dec = decode_launch(work.meta, **sizes)
        if dec is not None:
            part_o = ctx.scratch("attn_part_o", dec["part_o"])
            part_ml = ctx.scratch("attn_part_ml", dec["part_ml"])
            ops.attn_decode(qkv, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                            work.arrays.get("dec"), dec["n_dec"], part_o, part_ml, dec["max_parts"], dec["part_keys"],
                            **common)
        return ops.linear(out, self.o_proj, out_dtype=ctx.dtype)
