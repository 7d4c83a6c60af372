"""Faledra on the GPU: each mechanism's kernel alone against the plain
implementation, then whole models through the engine's step function, cache and
state manager: whole prompts, token-by-token decoding, portions down to two
tokens, mixed batches with pages and slots used again, random schedules, long
decoding, and greedy generation through the entry point and the scheduler."""
import math
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import ROOT
from faledra_util import BLOCK_SIZE, CONFIGS, config, gru, latent, plain_greedy, plain_logits, write_model
from plain import faledra_plain as FP
from trace_util import Trace, compare, compare_with_alone, random_tokens, random_trace, replay

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"


def tdt(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


def close(got, want, dtype, what="", floor=1.0):
    """Largest difference against ``tol`` times the largest wanted value (at least ``floor``)."""
    got, want = got.double().cpu(), want.double().cpu()
    tol = 2e-5 if dtype == "float32" else 2e-2
    scale = max(floor, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol * scale, f"{what}: max error {err:.3e} at scale {scale:.3f}"


def step_tables(counts, starts, slots):
    """q_start, positions, state slots of a step on the device."""
    q_start = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    pos = np.concatenate([np.arange(s, s + c) for s, c in zip(starts, counts)]).astype(np.int32)
    to = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)
    return to(q_start), to(pos), to(slots)


# ---------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [72, 256, 1030])
def test_branch_join_and_following_norm(dtype, H):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H)
    T = 9
    h = torch.randn(T, H, generator=g) * 3
    y = (torch.randn(T, H, generator=g) * 5).to(tdt(dtype))
    wb, wn, shift = 1 + 0.3 * torch.randn(H, generator=g), 1 + 0.3 * torch.randn(H, generator=g), torch.randn(H, generator=g)
    want_h = h.double() + 0.7 * FP.rms_norm(y.double(), wb.double(), 1e-5) + shift.double()
    want_x = FP.rms_norm(want_h, wn.double(), 1e-6)
    hd = h.to(DEV)
    out = torch.empty(T, H, dtype=tdt(dtype), device=DEV)
    ops.branch_join(hd, y.to(DEV), wb.to(DEV), 0.7, 1e-5, shift=shift.to(DEV), next_weight=wn.to(DEV), eps_next=1e-6, out=out)
    close(hd, want_h, "float32", "joined stream")
    close(out, want_x, dtype, "following norm")
    # picked rows: the stream stays as it is
    hd = h.to(DEV)
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(3, H, dtype=tdt(dtype), device=DEV)
    ops.branch_join(hd, y.to(DEV), wb.to(DEV), 0.7, 1e-5, shift=shift.to(DEV), next_weight=wn.to(DEV), eps_next=1e-6,
                    out=out, rows=rows)
    assert torch.equal(hd.cpu(), h)
    close(out, want_x[[7, 0, 3]], dtype, "picked rows")
    # the join alone, and the shift alone
    hd = h.to(DEV)
    ops.branch_join(hd, y.to(DEV), wb.to(DEV), 1.0, 1e-5)
    close(hd, h.double() + FP.rms_norm(y.double(), wb.double(), 1e-5), "float32", "join alone")
    hd = h.to(DEV)
    ops.add_row(hd, shift.to(DEV))
    close(hd, h.double() + shift.double(), "float32", "shift alone")


@pytest.mark.parametrize("C", [70, 72])      # one channel a thread, and 16 bytes of channels a thread
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_short_conv_in_portions_with_slots_used_again(dtype, taps, C):
    """Three requests in portions of every size (shorter than the filter's memory too), beside each
    other and in slots another request used before, against the whole sequences."""
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(taps)
    w = torch.randn(C, taps, generator=g)
    seqs = {r: torch.randn(n, C, generator=g).to(tdt(dtype)) for r, n in (("a", 23), ("b", 9), ("c", 14))}
    want = {r: x.double() + FP.short_conv(x.double(), w.double()) for r, x in seqs.items()}
    state = torch.full((3, max(taps - 1, 1), C), 99.0, dtype=tdt(dtype), device=DEV)[:, :taps - 1]   # stale contents
    state = state.contiguous() if taps > 1 else None
    fed = {r: 0 for r in seqs}
    slot = {"a": 0, "b": 1}
    plan = [[("a", 1), ("b", 4)], [("a", 2), ("b", 1)], [("a", 1)], [("a", 7), ("b", 4)], [("a", 12), ("c", 1)],
            [("c", 3)], [("c", 10)]]
    for step in plan:
        if "c" in dict(step) and "c" not in slot:
            slot["c"] = slot.pop("b")                                      # b is done; c takes its slot
        x = torch.cat([seqs[r][fed[r]:fed[r] + n] for r, n in step]).to(DEV)
        q_start, pos, slots = step_tables([n for _, n in step], [fed[r] for r, _ in step], [slot[r] for r, _ in step])
        out = torch.empty_like(x)
        ops.short_conv(x, w.to(DEV), state, q_start, pos, slots, out, len(step))
        at = 0
        for r, n in step:
            close(out[at:at + n], want[r][fed[r]:fed[r] + n], dtype, f"taps {taps} request {r} from {fed[r]}")
            at += n
            fed[r] += n


@pytest.mark.parametrize("dtype", DTYPES)
def test_activations(dtype):
    from lyapunov_engine_amd.kernels import ops

    z = torch.linspace(-6, 6, 1001).to(tdt(dtype))
    params = torch.tensor([0.4, -1.1])
    got = ops.activation(z.to(DEV).clone(), "xielu", params.to(DEV))
    close(got, FP.xielu(z.double(), params[0].double(), params[1].double()), dtype, "xielu")
    got = ops.activation(z.to(DEV).clone(), "gelu_tanh")
    close(got, FP.gelu_tanh(z.double()), dtype, "gelu_tanh")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_norm_and_filter_in_one_kernel_for_steps_of_single_tokens(dtype, taps):
    """Three requests decode side by side for ten steps (one starts later, in a slot with stale
    contents): join, norm and filter in one kernel against the plain functions on whole sequences."""
    from lyapunov_engine_amd.kernels import ops

    H, n = 136, 10
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(H, taps, generator=g)
    wn, wb = 1 + 0.2 * torch.randn(H, generator=g), 1 + 0.2 * torch.randn(H, generator=g)
    hs = torch.randn(3, n, H, generator=g)
    ys = torch.randn(3, n, H, generator=g).to(tdt(dtype))
    state = torch.full((4, max(taps - 1, 1), H), 55.0, dtype=tdt(dtype), device=DEV)[:, :taps - 1].contiguous() if taps > 1 else None
    want = []
    for r in range(3):
        joined = hs[r].double() + 0.5 * FP.rms_norm(ys[r].double(), wb.double(), 1e-5)
        x = FP.rms_norm(joined, wn.double(), 1e-6)
        if dtype == "bfloat16":
            x = x.to(torch.bfloat16).double()          # the filter reads activations
        want.append(x + FP.short_conv(x, w.double()))
    for t in range(n):
        live = [0, 1] if t < 3 else [0, 1, 2]            # request 2 starts at step 3, at its own position 0
        pos = [t, t] if t < 3 else [t, t, t - 3]
        h = torch.stack([hs[r, p] for r, p in zip(live, pos)]).to(DEV)
        y = torch.stack([ys[r, p] for r, p in zip(live, pos)]).to(DEV)
        to = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
        out = torch.empty(len(live), H, dtype=tdt(dtype), device=DEV)
        ops.branch_join(h, y, wb.to(DEV), 0.5, 1e-5, next_weight=wn.to(DEV), eps_next=1e-6, out=out,
                        conv=(w.to(DEV), state, to([3, 0, 2][:len(live)]), to(pos)))
        for i, (r, p) in enumerate(zip(live, pos)):
            close(out[i], want[r][p], dtype, f"taps {taps} step {t} request {r}")


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_mingru_scan_in_portions(dtype, chunked):
    from lyapunov_engine_amd.kernels import ops

    W = 100
    g = torch.Generator().manual_seed(4)
    bz, bx = torch.randn(W, generator=g), torch.randn(W, generator=g)
    pre = {r: torch.randn(n, 3 * W, generator=g) * 2 for r, n in (("a", 300), ("b", 5))}

    def whole(p):
        z = torch.sigmoid(p[:, :W].double() + bz.double())
        u = p[:, W:2 * W].double() + bx.double()
        c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        gate = p[:, 2 * W:].double()
        s, rows = torch.zeros(W, dtype=torch.float64), []
        for t in range(p.shape[0]):
            s = (1 - z[t]) * s + z[t] * c[t]
            rows.append(s * gate[t] * torch.sigmoid(gate[t]))
        return torch.stack(rows)

    want = {r: whole(p) for r, p in pre.items()}
    state = torch.full((4, W), 7.0, device=DEV)                            # stale contents
    fed = {"a": 0, "b": 0}
    for step in ([("a", 1), ("b", 2)], [("a", 2)], [("b", 3), ("a", 200)], [("a", 1)], [("a", 96)]):
        x = torch.cat([pre[r][fed[r]:fed[r] + n] for r, n in step]).to(DEV)
        q_start, pos, slots = step_tables([n for _, n in step], [fed[r] for r, _ in step], [3 if r == "a" else 1 for r, _ in step])
        out = torch.empty(x.shape[0], W, dtype=tdt(dtype), device=DEV)
        ws = torch.full((ops.mingru_scan_workspace(x.shape[0], len(step), W),), float("nan"), device=DEV) if chunked else None
        ops.mingru_scan(x, bz.to(DEV), bx.to(DEV), state, q_start, pos, slots, out, len(step), ws)
        at = 0
        for r, n in step:
            close(out[at:at + n], want[r][fed[r]:fed[r] + n], dtype, f"request {r} from {fed[r]}")
            at += n
            fed[r] += n


def latent_case(dtype, T_ctx, H, kv_rank, rot_dim, page_size, seed, n_new, use_mfma=None):
    """One request of T_ctx tokens whose last n_new are the step's rows; returns what the kernels
    need and the plain result for those rows."""
    g = torch.Generator().manual_seed(seed)
    Dk = kv_rank + rot_dim
    keys = torch.randn(T_ctx, Dk, generator=g).to(tdt(dtype))
    qa = torch.randn(n_new, H, Dk, generator=g).to(tdt(dtype))
    sink = torch.randn(H, generator=g)
    return keys, qa, sink


KERNELS = ["rows", "cores", "cores in 3 partitions"]


def run_latent_attention(dtype, keys, qa, sink, scale, kv_rank, rot_dim, page_size, n_pages_extra=3, shuffle_seed=0,
                         kernel="rows"):
    """``kernel``: "rows" (any sizes, a workgroup per row and head) or "cores" (the matrix-core kernel;
    sizes in multiples of 16), the latter also with the keys forced into partitions."""
    from lyapunov_engine_amd.kernels import ops

    if kernel != "rows" and not ops.latent_attn_fits_matrix_cores(kv_rank, rot_dim):
        pytest.skip("sizes that only the row-by-row kernel takes")

    T_ctx, Dk = keys.shape
    n_new, H = qa.shape[0], qa.shape[1]
    n_blocks = -(-T_ctx // page_size)
    rng = random.Random(shuffle_seed)
    page_ids = list(range(n_blocks + n_pages_extra))
    rng.shuffle(page_ids)
    page_ids = page_ids[:n_blocks]
    pages = torch.full((n_blocks + n_pages_extra, page_size, Dk), float("nan"), dtype=tdt(dtype))
    for j in range(T_ctx):
        pages[page_ids[j // page_size], j % page_size] = keys[j]
    to = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)
    out = torch.empty(n_new, H, kv_rank, dtype=tdt(dtype), device=DEV)
    args = (qa.to(DEV), pages.to(DEV), to([page_ids]), to([0, n_new]), to(np.arange(T_ctx - n_new, T_ctx)), to([T_ctx]),
            sink.to(DEV), scale, out)
    if kernel == "rows":
        ops.latent_attn_rows(*args, kv_rank=kv_rank, rot_dim=rot_dim)
        return out
    launch = ops.latent_attn_launch(n_new, 1, H, T_ctx, tdt(dtype), kv_rank, rot_dim,
                                    n_parts=3 if "partitions" in kernel else None)
    part_o = torch.full((max(1, launch["part_o"]),), float("nan"), device=DEV)
    part_ml = torch.full((max(1, launch["part_ml"]),), float("nan"), device=DEV)
    ops.latent_attn(*args, launch, part_o, part_ml, kv_rank=kv_rank, rot_dim=rot_dim)
    return out


def plain_latent_attention(keys, qa, sink, scale, kv_rank):
    T_ctx, n_new, H = keys.shape[0], qa.shape[0], qa.shape[1]
    k, q = keys.double(), qa.double()
    out = torch.zeros(n_new, H, kv_rank, dtype=torch.float64)
    for i in range(n_new):
        n_keys = T_ctx - n_new + i + 1
        for h in range(H):
            s = (k[:n_keys] @ q[i, h]) * scale
            m = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - m)
            out[i, h] = (e[:, None] * k[:n_keys, :kv_rank]).sum(0) / (e.sum() + math.exp(float(sink[h]) - m))
    return out


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(37, 3, 40, 8, 4, 37), (300, 2, 24, 14, 16, 5), (130, 5, 64, 32, 16, 1),
                                   (1000, 4, 96, 16, 16, 1), (513, 1, 48, 16, 16, 70), (700, 3, 32, 0, 16, 300),
                                   (2100, 20, 16, 16, 64, 3)])
def test_latent_attention_over_pages(dtype, shape, kernel):
    T_ctx, H, kv_rank, rot_dim, page_size, n_new = shape
    keys, qa, sink = latent_case(dtype, T_ctx, H, kv_rank, rot_dim, page_size, seed=T_ctx, n_new=n_new)
    scale = (kv_rank + rot_dim) ** -0.5
    got = run_latent_attention(dtype, keys, qa, sink, scale, kv_rank, rot_dim, page_size, kernel=kernel)
    # sums over hundreds of keys are small: held to their own size, not to 1
    close(got, plain_latent_attention(keys, qa, sink, scale, kv_rank), dtype, f"latent attention {shape}", floor=1e-3)


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("where", [0, 1, 15, 16, 17, 63, 64, 255, 256, 319, 320, 600, 898, 899])
def test_latent_attention_finds_one_planted_key(dtype, where, kernel):
    """Among 900 keys one is made to carry the result (its score stands far above the rest): first
    tokens, page borders, far back, and the row's own position.  The sink is far below."""
    T_ctx, H, kv_rank, rot_dim, page_size = 900, 2, 32, 16, 16
    keys, qa, sink = latent_case(dtype, T_ctx, H, kv_rank, rot_dim, page_size, seed=5, n_new=1)
    keys = (keys.float() * 0.1).to(tdt(dtype))
    qa = (keys[where].float() * 400.0)[None, None, :].repeat(1, H, 1).to(tdt(dtype))
    sink = torch.full((H,), -50.0)
    got = run_latent_attention(dtype, keys, qa, sink, 1.0, kv_rank, rot_dim, page_size, shuffle_seed=where, kernel=kernel)
    want = plain_latent_attention(keys, qa, sink, 1.0, kv_rank)
    close(got, want, dtype, f"planted key at {where}")
    assert torch.allclose(want[0, 0], keys[where, :kv_rank].double(), atol=0.05), "the planted key must carry the result"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(16, 0), (16, 16), (32, 16), (48, 0), (16, 32), (64, 16), (32, 48), (96, 16), (64, 64),
                                   (128, 16), (128, 32)])
def test_matrix_core_kernel_finds_planted_keys_at_every_size(dtype, sizes):
    """The matrix-core kernel walks the key dimension in instructions of 32 and of 16 values, by
    sizes: every combination has to find a planted key at every place of a tile (with eight
    dimensions of a score missing, a planted key would still win most of the time, so all places of
    two tiles are tried)."""
    kv_rank, rot_dim = sizes
    T_ctx, H, page_size = 130, 3, 16
    keys, _, _ = latent_case(dtype, T_ctx, H, kv_rank, rot_dim, page_size, seed=kv_rank + rot_dim, n_new=1)
    keys = (keys.float() * 0.1).to(tdt(dtype))
    sink = torch.full((H,), -50.0)
    for where in range(0, T_ctx, 3):
        qa = (keys[where].float() * (19200.0 / (kv_rank + rot_dim)))[None, None, :].repeat(1, H, 1).to(tdt(dtype))
        got = run_latent_attention(dtype, keys, qa, sink, 1.0, kv_rank, rot_dim, page_size, kernel="cores")
        want = plain_latent_attention(keys, qa, sink, 1.0, kv_rank)
        close(got, want, dtype, f"sizes {sizes}, planted key at {where}", floor=1e-3)


@pytest.mark.parametrize("kernel", KERNELS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_attention_sink_takes_weight_and_the_future_is_not_seen(dtype, kernel):
    T_ctx, H, kv_rank, rot_dim, page_size = 64, 3, 16, 16, 16
    keys, qa, sink = latent_case(dtype, T_ctx, H, kv_rank, rot_dim, page_size, seed=9, n_new=20)
    sink = torch.tensor([30.0, 0.0, -30.0])                                # head 0: nearly everything goes to the sink
    got = run_latent_attention(dtype, keys, qa, sink, 0.2, kv_rank, rot_dim, page_size, kernel=kernel)
    want = plain_latent_attention(keys, qa, sink, 0.2, kv_rank)
    close(got, want, dtype, "sinks")
    assert float(got[:, 0].abs().max()) < 1e-6 < float(got[:, 2].abs().max())
    # a key just after a row's position, made overwhelming, must not be seen by that row
    keys2 = keys.clone()
    keys2[50] = (qa[5, 1].float() * 50).to(tdt(dtype))                     # row 5 stands at position 49
    got2 = run_latent_attention(dtype, keys2, qa, sink, 0.2, kv_rank, rot_dim, page_size, kernel=kernel)
    close(got2[:6], want[:6], dtype, "rows before the planted key")
    assert float((got2[6:].double().cpu() - want[6:]).abs().max()) > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(32, 16, 24), (128, 16, 40), (64, 32, 64)])
def test_merge_and_value_projection_in_one_kernel(dtype, sizes):
    """Steps of few rows: the partitions' results merged (with the sink) and multiplied by every
    head's value matrix in one kernel, and the same from rows that were already merged."""
    from lyapunov_engine_amd.kernels import ops

    kv_rank, rot_dim, vdim = sizes
    T_ctx, H, n_new, page_size = 700, 3, 2, 16
    keys, qa, sink = latent_case(dtype, T_ctx, H, kv_rank, rot_dim, page_size, seed=vdim, n_new=n_new)
    scale = (kv_rank + rot_dim) ** -0.5
    g = torch.Generator().manual_seed(3)
    w = torch.randn(H, vdim, kv_rank, generator=g).to(tdt(dtype))
    merged = plain_latent_attention(keys, qa, sink, scale, kv_rank)
    if dtype == "bfloat16":
        merged = merged.to(torch.bfloat16).double()
    want = torch.einsum("thr,hvr->thv", merged, w.double())
    to = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)
    n_blocks = -(-T_ctx // page_size)
    pages = torch.zeros(n_blocks, page_size, kv_rank + rot_dim, dtype=tdt(dtype))
    for j in range(T_ctx):
        pages[j // page_size, j % page_size] = keys[j]
    for n_parts in (4, 1):
        launch = ops.latent_attn_launch(n_new, 1, H, T_ctx, tdt(dtype), kv_rank, rot_dim, n_parts=n_parts)
        part_o = torch.full((max(1, launch["part_o"]),), float("nan"), device=DEV)
        part_ml = torch.full((max(1, launch["part_ml"]),), float("nan"), device=DEV)
        mixed = torch.full((n_new, H, kv_rank), float("nan"), dtype=tdt(dtype), device=DEV)
        ops.latent_attn(qa.to(DEV), pages.to(DEV), to([list(range(n_blocks))]), to([0, n_new]),
                        to(np.arange(T_ctx - n_new, T_ctx)), to([T_ctx]), sink.to(DEV), scale, mixed, launch, part_o, part_ml,
                        kv_rank=kv_rank, rot_dim=rot_dim, merge=False)
        out = torch.empty(n_new, H, vdim, dtype=tdt(dtype), device=DEV)
        if launch["n_parts"] > 1:
            assert torch.isnan(mixed.float()).all(), "without the merge pass nothing writes the merged rows"
            ops.latent_heads_out(w.to(DEV), out, kv_rank=kv_rank, rot_dim=rot_dim, part_o=part_o, part_ml=part_ml,
                                 sink=sink.to(DEV), n_parts=launch["n_parts"])
        else:
            ops.latent_heads_out(w.to(DEV), out, kv_rank=kv_rank, rot_dim=rot_dim, mixed=mixed)
        close(out, want, dtype, f"sizes {sizes}, {launch['n_parts']} partitions", floor=1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_prep_and_query_rotation(dtype):
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.rope import RotaryEncoding

    T, q_rank, kv_rank, rot_dim, dims, H, dim, page = 11, 28, 24, 14, 10, 3, 10, 4
    g = torch.Generator().manual_seed(2)
    d = (torch.randn(T, q_rank + kv_rank + rot_dim, generator=g) * 2).to(tdt(dtype))
    wq, wkv = 1 + 0.2 * torch.randn(q_rank, generator=g), 1 + 0.2 * torch.randn(kv_rank, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 42, 43, 44, 45, 500], dtype=torch.int32)
    slots = torch.tensor([8, 9, 10, 11, 0, 1, 2, 3, 4, 5, -1], dtype=torch.int32)   # the last row is padding
    enc = RotaryEncoding(dims, 500.0, 1024)
    enc.materialize(DEV, tdt(dtype))
    cq = torch.empty(T, q_rank, dtype=tdt(dtype), device=DEV)
    pages = torch.zeros(3, page, kv_rank + rot_dim, dtype=tdt(dtype), device=DEV)
    ops.latent_prep(d.to(DEV), wq.to(DEV), wkv.to(DEV), pos.to(DEV), enc.table, slots.to(DEV), cq, pages,
                    q_rank=q_rank, kv_rank=kv_rank, rot_dim=rot_dim, eps=1e-5)
    dd = d.double()
    close(cq, FP.rms_norm(dd[:, :q_rank], wq.double(), 1e-5), dtype, "query latent")
    want_c = FP.rms_norm(dd[:, q_rank:q_rank + kv_rank], wkv.double(), 1e-5)
    want_r = FP.rotate_pairs(dd[:, None, q_rank + kv_rank:], pos, 500.0, dims)[:, 0]
    flat = pages.view(-1, kv_rank + rot_dim)
    for t in range(T - 1):
        close(flat[int(slots[t]), :kv_rank], want_c[t], dtype, f"latent of row {t}")
        close(flat[int(slots[t]), kv_rank:], want_r[t], dtype, f"rotated key part of row {t}")
    q = torch.randn(T, H * (dim + rot_dim), generator=g).to(tdt(dtype))
    qa = torch.zeros(T, H, kv_rank + rot_dim, dtype=tdt(dtype), device=DEV)
    ops.latent_query_rotate(q.to(DEV), pos.to(DEV), enc.table, qa, num_heads=H, dim=dim, rot_dim=rot_dim, kv_rank=kv_rank)
    want = FP.rotate_pairs(q.double().view(T, H, dim + rot_dim)[..., dim:], pos, 500.0, dims)
    close(qa[..., kv_rank:], want, dtype, "rotated query part")
    assert float(qa[..., :kv_rank].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(5, 3, 20, 24), (70, 2, 12, 10), (200, 4, 32, 64)])
def test_products_of_all_heads_in_one_launch(dtype, shape):
    from lyapunov_engine_amd.kernels import ops

    M, G, N, K = shape
    g = torch.Generator().manual_seed(M)
    wide = torch.randn(M, G, K + 6, generator=g).to(tdt(dtype))           # a view into a wider tensor
    w = torch.randn(G, N, K, generator=g).to(tdt(dtype))
    out = torch.zeros(M, G, N + 4, dtype=tdt(dtype), device=DEV)
    a = wide.to(DEV)[:, :, :K]
    ops.gemm_nt_heads(a, w.to(DEV), out[:, :, :N])
    want = torch.einsum("mgk,gnk->mgn", wide[:, :, :K].double(), w.double())
    close(out[:, :, :N], want, dtype, f"heads {shape}")
    assert float(out[:, :, N:].abs().max()) == 0.0


# ------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in CONFIGS.items():
        out[name] = {dt: write_model(str(tmp_path_factory.mktemp(f"faledra{name}_{dt}")), cfg, seed=11 + ord(name), dtype=dt)
                     for dt in DTYPES}
    return out


LENGTHS = {"a": 1, "b": 7, "c": 33, "d": 70, "e": 100}


def requests_for(name, extra=None):
    lens = dict(LENGTHS, **(extra or {}))
    return {rid: random_tokens(n, CONFIGS[name]["vocab"], seed=300 + i) for i, (rid, n) in enumerate(sorted(lens.items()))}


def run(folders, name, dtype, t):
    return replay(folders[name][dtype], dtype, t, block_size=BLOCK_SIZE[name])


# bfloat16 against the 64-bit plain model on the same rounded weights: these models are made with
# wide weights so that attention is peaked and faults show, which also makes rounding show; the
# bounds are per row of the largest logit.
TOL16 = dict(rtol=0.0, atol=1.2e-1, median=3e-2)


def check(t, got, folders, name, dtype, label):
    want = plain_logits(folders[name][dtype], t.requests)
    compare(t, got, want, dtype, label, tol=None if dtype == "float32" else TOL16)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompts(folders, name, dtype):
    for rid, toks in requests_for(name).items():
        t = Trace({rid: toks})
        t.step([(rid, len(toks))], end=[rid])
        check(t, run(folders, name, dtype, t), folders, name, dtype, f"whole {name} {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_prefill_then_token_by_token(folders, name, dtype):
    for rid, toks in requests_for(name).items():
        if len(toks) < 33:
            continue
        t = Trace({rid: toks})
        t.step([(rid, len(toks) - 30)], want="last")
        for _ in range(30):
            t.step([(rid, 1)])
        got = run(folders, name, dtype, t)
        check(t, got, folders, name, dtype, f"decode {name} {rid}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"decode {name} {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_token_alone_from_the_first(folders, name, dtype):
    """The first tokens of a sequence one by one: an empty state, a filter that looks back before
    the start, a first page."""
    toks = requests_for(name)["c"]
    t = Trace({"c": toks})
    for _ in toks:
        t.step([("c", 1)])
    check(t, run(folders, name, dtype, t), folders, name, dtype, f"one by one {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_down_to_two_tokens(folders, name, dtype):
    sizes = [7, 2, 5, 3, 16, 2, 31, 4, 2, 9]
    for rid, toks in requests_for(name).items():
        if len(toks) < 9:
            continue
        t = Trace({rid: toks})
        left, i = len(toks), 0
        while left:
            n = min(sizes[i % len(sizes)], left)
            if left - n == 1:
                n += 1
            t.step([(rid, n)])
            left -= n
            i += 1
        got = run(folders, name, dtype, t)
        check(t, got, folders, name, dtype, f"portions {name} {rid}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"portions {name} {rid}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    reqs = requests_for(name, {"f": 90, "g": 12, "h": 50})
    t = Trace(reqs)
    t.step([("d", 40), ("a", 1)], end=["a"])
    t.step([("d", 2), ("b", 4), ("c", 20)])
    t.step([("d", 1), ("b", 1), ("c", 2), ("e", 30)])
    t.step([("b", 1), ("c", 1), ("e", 7)])                              # d sits this one out
    t.step([("d", 27), ("b", 1), ("c", 10)], end=["b", "c"])
    t.step([("e", 1), ("f", 64), ("g", 3)], end=["d"])                  # f and g take the slots and pages of b, c
    t.step([("e", 2), ("f", 1), ("g", 2), ("h", 33)])
    for _ in range(5):
        t.step([("e", 1), ("f", 1), ("g", 1), ("h", 1)])
    t.step([("e", 55), ("f", 20), ("g", 2), ("h", 12)], end=["e", "f", "g", "h"])
    total = sum(64 * -(-len(v) // 64) for v in reqs.values())
    assert t.max_tokens < total, "the pool is meant to be too small for all requests at once"
    got = run(folders, name, dtype, t)
    check(t, got, folders, name, dtype, f"mixed {name}")
    if dtype == "float32":
        compare_with_alone(t, got, folders[name][dtype], dtype, f"mixed {name}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_random_schedules(folders, name, dtype):
    for seed in range(6):
        rng = random.Random(77 * seed + ord(name))
        reqs, t = random_trace(rng, CONFIGS[name]["vocab"], 150)
        got = run(folders, name, dtype, t)
        check(t, got, folders, name, dtype, f"random schedule {name} {seed}")
        if dtype == "float32":
            compare_with_alone(t, got, folders[name][dtype], dtype, f"random schedule {name} {seed}")


def test_long_decoding_and_far_keys(folders):
    """400 tokens: most as portions that end inside pages, the last 150 one by one (the recurrent
    state carried for hundreds of steps, keys hundreds of tokens back, pages filling up)."""
    name, dtype = "C", "float32"
    toks = random_tokens(400, CONFIGS[name]["vocab"], seed=1)
    t = Trace({"x": toks})
    t.step([("x", 131)], want="last")
    t.step([("x", 119)], want="last")
    for _ in range(150):
        t.step([("x", 1)])
    check(t, run(folders, name, dtype, t), folders, name, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_given_shape_of_things_is_not_assumed(tmp_path, dtype):
    """Sizes that are equal, or 1, in one model and not in another: one layer, one head, one pass of
    a loop over everything, no filter, a multiplier of 1, rank larger than the width."""
    cfg = config(97, 48, [latent(1, 8, 24, 40, 56, 72, dims=24, ff=40)], loop=(0, 1, 1), mult=1.0, emb_scale=1.0)
    folder = write_model(str(tmp_path / "m"), cfg, seed=5, dtype=dtype)
    toks = random_tokens(45, 97, seed=3)
    t = Trace({"x": toks})
    t.step([("x", 20)])
    t.step([("x", 2)])
    for _ in range(23):
        t.step([("x", 1)])
    got = replay(folder, dtype, t, block_size=8)
    compare(t, got, plain_logits(folder, t.requests), dtype, "one of everything", tol=None if dtype == "float32" else TOL16)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layers", ["recurrent only", "no rotated part", "attention only, looped four times"])
def test_other_orders_of_layers(tmp_path, dtype, layers):
    """Models without any paged cache (recurrent layers alone), with heads that have no rotated
    part, and of attention layers alone in a loop: portions, then single tokens, two requests."""
    if layers == "recurrent only":
        cfg = config(111, 40, [gru(24, ff=56), gru(40)], taps=3, loop=(1, 2, 2), mult=0.9)
    elif layers == "no rotated part":
        cfg = config(111, 48, [latent(2, 16, 0, 16, 24, 32, ff=64), gru(32, ff=40)], taps=2)
    else:
        cfg = config(111, 64, [latent(4, 16, 16, 16, 32, 48, ff=96), latent(2, 32, 16, 24, 40, 64)], taps=5,
                     loop=(0, 2, 4), mult=0.5)
    folder = write_model(str(tmp_path / "m"), cfg, seed=9, dtype=dtype)
    reqs = {"x": random_tokens(50, 111, seed=1), "y": random_tokens(21, 111, seed=2)}
    t = Trace(reqs)
    t.step([("x", 30)])
    t.step([("x", 3), ("y", 19)])
    for _ in range(2):
        t.step([("x", 1), ("y", 1)])
    t.step([("x", 15)], end=["x", "y"])
    got = replay(folder, dtype, t, block_size=8)
    compare(t, got, plain_logits(folder, t.requests), dtype, layers, tol=None if dtype == "float32" else TOL16)


# ------------------------------------------------------------------- generation
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(folders, name, dtype):
    import lyapunov_engine_amd as L

    folder = folders[name][dtype]
    prompts = [random_tokens(n, CONFIGS[name]["vocab"], seed=60 + n) for n in (3, 19, 40)]
    llm = L.LLM(folder, dtype=dtype, num_blocks=96, block_size=BLOCK_SIZE[name], max_num_batched_tokens=32)
    outs = llm.generate(prompts, L.SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    for prompt, o in zip(prompts, outs):
        assert o.finished and o.prompt_tokens == prompt and len(o.output_tokens) == 12
        want, margins = plain_greedy(folder, prompt, 12)
        for i, (g, w) in enumerate(zip(o.output_tokens, want)):
            if g != w:
                assert dtype == "bfloat16" and margins[i] < 0.5, f"token {i}: engine {g}, plain {w}, margin {margins[i]}"
                break


def test_generation_with_and_without_recorded_steps_and_with_preemption(folders):
    import lyapunov_engine_amd as L

    folder = folders["C"]["float32"]
    prompts = [random_tokens(n, CONFIGS["C"]["vocab"], seed=80 + n) for n in (5, 30, 61, 12)]
    sp = L.SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    want = [plain_greedy(folder, p, 20)[0] for p in prompts]
    for kw in (dict(enable_graphs=True, num_blocks=64), dict(enable_graphs=False, num_blocks=64),
               dict(enable_graphs=True, num_blocks=12, max_num_batched_tokens=24)):   # few pages: preemption
        outs = L.LLM(folder, dtype="float32", block_size=16, **kw).generate(prompts, sp)
        assert [o.output_tokens for o in outs] == want, kw


def test_command_line_generate(folders):
    folder = folders["A"]["float32"]
    prompt = random_tokens(9, CONFIGS["A"]["vocab"], seed=8)
    want, _ = plain_greedy(folder, prompt, 8)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "lyapunov"), "generate", "--model", folder,
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0",
                           "--dtype", "float32", "--block-size", "4", "--num-blocks", "32"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.strip().splitlines()[-1].split() == [str(t) for t in want]
