"""The kernels behind Ronupel's mechanisms, each alone against the plain
implementation (tests/plain/ronupel_plain.py): the norm over a whole projection
with the rotation of neighbouring pairs and the page write; attention with a
window, kept first tokens and a sink on all three kernels (row by row, prompt
tiles, one-token requests in partitions) over shuffled pages, with single keys
made to carry the result just inside and just outside every edge; the router,
the sort by expert, the experts' products and the weighted sum."""
import math

import numpy as np
import pytest
import torch

from plain import ronupel_plain as RP

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"


def tdt(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


def close(got, want, dtype, what="", floor=1.0, tol=None):
    got, want = got.double().cpu(), want.double().cpu()
    tol = tol if tol is not None else (2e-5 if dtype == "float32" else 2e-2)
    scale = max(floor, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol * scale, f"{what}: max error {err:.3e} at scale {scale:.3f}"


def ints(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)


# ------------------------------------------------ norm, rotation, page write
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(3, 1, 10, 12, 6), (4, 2, 32, 32, 32), (2, 2, 7, 5, 4), (5, 5, 16, 24, 0), (8, 2, 64, 64, 16)])
@pytest.mark.parametrize("normed", [True, False])
def test_projection_norm_rotation_and_page_write(dtype, sizes, normed):
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.rope import RotaryEncoding

    H, G, D, V, rot = sizes
    T, page = 9, 4
    g = torch.Generator().manual_seed(H * 100 + D)
    qkv = (torch.randn(T, (H + G) * D + G * V, generator=g) * 2).to(tdt(dtype))
    wq, wk = 1 + 0.3 * torch.randn(H * D, generator=g), 1 + 0.3 * torch.randn(G * D, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 42, 777, 5], dtype=torch.int32)
    slots = torch.tensor([8, 9, 10, 11, 0, 1, 2, 5, -1], dtype=torch.int32)      # the last row is padding
    table = None
    if rot:
        enc = RotaryEncoding(rot, 300.0, 1024, scaling={"rope_type": "linear", "factor": 2.5}, precise=True)
        enc.materialize(DEV, tdt(dtype))
        table = enc.table
    kpool = torch.zeros(3, G, page, D, dtype=tdt(dtype), device=DEV)
    vpool = torch.zeros(3, G, V, page, dtype=tdt(dtype), device=DEV)
    dev = qkv.to(DEV)
    ops.qk_norm_rope_kv(dev, wq.to(DEV) if normed else None, wk.to(DEV) if normed else None, 1e-5, pos.to(DEV), table,
                        slots.to(DEV), kpool, vpool, num_heads=H, num_kv_heads=G, dim=D, vdim=V, page_size=page)
    x = qkv.double()
    q, k, v = x[:, :H * D], x[:, H * D:(H + G) * D], x[:, (H + G) * D:]
    if normed:
        q, k = RP.rms_norm(q, wq.double(), 1e-5), RP.rms_norm(k, wk.double(), 1e-5)
    q, k = q.view(T, H, D), k.view(T, G, D)
    if rot:
        q, k = RP.rotate_neighbours(q, pos, 300.0, rot, 2.5), RP.rotate_neighbours(k, pos, 300.0, rot, 2.5)
    close(dev[:, :H * D], q.reshape(T, H * D), dtype, "queries")
    for t in range(T - 1):
        p, o = int(slots[t]) // page, int(slots[t]) % page
        close(kpool[p, :, o, :], k[t], dtype, f"key of row {t}")
        close(vpool[p, :, :, o], v[t].view(G, V), dtype, f"value of row {t}")
    assert float(kpool[1, :, 2:, :].abs().max()) == 0.0 and float(kpool[1, :, 0, :].abs().max()) == 0.0, \
        "slots nobody named stay as they were"


def test_position_table_with_divided_frequencies():
    """The 64-bit table is the nearest float to cos and sin of position * base^(-2i/d) / factor, far out too."""
    from lyapunov_engine_amd.parts.rope import RotaryEncoding

    enc = RotaryEncoding(6, 30000.0, 5000, scaling={"rope_type": "linear", "factor": 6.0}, precise=True)
    enc.materialize(DEV, torch.float32)
    for p in (0, 1, 63, 4999):
        for i in range(3):
            a = p * 30000.0 ** (-2.0 * i / 6) / 6.0
            assert abs(float(enc.table[p, i]) - math.cos(a)) < 1e-7 and abs(float(enc.table[p, 3 + i]) - math.sin(a)) < 1e-7


# ------------------------------------------------------------------ attention
def paged(k, v, page, seed, spare=3):
    """Keys [n, G, D] and values [n, G, V] of one request into shuffled pages; pages nobody owns
    hold NaN, the slots past the request's end zeros."""
    n, G, D = k.shape
    V = v.shape[2]
    n_blocks = -(-n // page)
    order = torch.tensor(np.random.default_rng(seed).permutation(n_blocks + spare)[:n_blocks], dtype=torch.long)
    kpool = torch.full((n_blocks + spare, G, page, D), float("nan"), dtype=k.dtype)
    vpool = torch.full((n_blocks + spare, G, V, page), float("nan"), dtype=k.dtype)
    kp = torch.zeros(n_blocks * page, G, D, dtype=k.dtype)
    vp = torch.zeros(n_blocks * page, G, V, dtype=k.dtype)
    kp[:n], vp[:n] = k, v
    kpool[order] = kp.view(n_blocks, page, G, D).permute(0, 2, 1, 3)
    vpool[order] = vp.view(n_blocks, page, G, V).permute(0, 2, 3, 1)
    return kpool.to(DEV), vpool.to(DEV), ints([order.tolist()])


def plain_attention(q, k, v, q_pos, sink, scale, window, keep):
    """q [m, H, D] at positions q_pos over keys 0..n-1: [m, H, V] by the plain functions."""
    H, G = q.shape[1], k.shape[1]
    n = k.shape[0]
    size = window if window else n + 1
    mask = RP.visible(q_pos, torch.arange(n), size, keep if window else 0)
    out = torch.zeros(q.shape[0], H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        g = h // (H // G)
        s = q[:, h].double() @ k[:, g].double().T * scale
        if sink is None:
            p = torch.softmax(s.masked_fill(~mask, float("-inf")), -1)
        else:
            p = RP.sink_softmax(s, mask, sink[h].double())
        out[:, h] = p @ v[:, g].double()
    return out


def run_attention(kernel, dtype, q, k, v, n_new, sink, scale, window, keep, page, seed=0, lost=True):
    """The last ``n_new`` positions of a request of len(k) tokens as one step through ``kernel``:
    "rows", "tiles" (prompt tiles on the matrix cores) or "split" (one new token, keys in partitions)."""
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.attention import AttentionWork, PagedAttention
    from lyapunov_engine_amd.parts.base import StepBatch

    n, G, D = k.shape
    H, V = q.shape[1], v.shape[2]
    first = n - n_new
    lost_below = 0
    if lost and window:          # what the cache manager gives back before this step: behind the window, past the kept
        lost_below = max(0, first - window + 1)
    kept_pages = -(-keep // page) * page if window else 0
    kpool, vpool, table = paged(k, v, page, seed)
    if lost_below > kept_pages:
        tb = table.cpu().numpy().copy()
        for b in range(kept_pages // page, lost_below // page):
            kpool[tb[0, b]], vpool[tb[0, b]] = float("nan"), float("nan")
            tb[0, b] = -1
        table = ints(tb)
    qd = q.reshape(n_new, H * D).to(tdt(dtype)).to(DEV)
    out = torch.full((n_new, H * V), float("nan"), dtype=tdt(dtype), device=DEV)
    q_start, ctx_len, pos = ints([0, n_new]), ints([n]), ints(np.arange(first, n))
    sk = None if sink is None else sink.float().to(DEV)
    if kernel == "rows":
        ops.attn_rows(qd, out, kpool, vpool, table, q_start, pos, ctx_len, num_heads=H, num_kv_heads=G, dim=D, vdim=V,
                      scale=scale, window=window, keep_first=keep, sink=sk)
        return out.view(n_new, H, V)
    assert D == V
    batch = StepBatch(start=np.array([first], np.int32), count=np.array([n_new], np.int32),
                      q_start=np.array([0, n_new], np.int32), ctx_len=np.array([n], np.int32), T=n_new, B=1)
    arrays, meta = AttentionWork().plan(batch)
    common = dict(num_heads=H, num_kv_heads=G, head_dim=D, window=window, scale=scale, keep_first=keep, sink=sk)
    if kernel == "tiles":
        if n_new == 1:                                   # a lone token as a tile of its own
            arrays, meta = {"tile_seq": np.zeros(1, np.int32), "tile_q0": np.zeros(1, np.int32)}, dict(n_tiles=1)
        ops.attn_prefill(qd, out, kpool, vpool, table, q_start, ctx_len, ints(arrays["tile_seq"]), ints(arrays["tile_q0"]),
                         meta["n_tiles"], pair=False, **common)
    else:
        assert n_new == 1
        part = 256                                       # several partitions from 257 keys on
        max_parts = -(-n // part)
        part_o = torch.full((H * max_parts * D,), float("nan"), device=DEV)
        part_ml = torch.full((H * max_parts * 2,), float("nan"), device=DEV)
        ops.attn_decode(qd, out, kpool, vpool, table, q_start, ctx_len, None, 1, part_o, part_ml, max_parts, part,
                        **common)
    return out.view(n_new, H, V)


def attention_case(dtype, n, H, G, D, V, seed):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(n, G, D, generator=g).to(tdt(dtype))
    v = torch.randn(n, G, V, generator=g).to(tdt(dtype))
    sink = torch.randn(H, generator=g)
    return k, v, sink, g


CASES = [  # kernel, heads, kv heads, key size, value size, page
    ("rows", 3, 1, 10, 12, 4), ("rows", 2, 2, 32, 32, 16), ("rows", 4, 2, 24, 8, 8),
    ("tiles", 4, 2, 32, 32, 16), ("tiles", 2, 2, 16, 16, 4), ("tiles", 8, 1, 64, 64, 16), ("tiles", 3, 3, 48, 48, 8),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("mask", [(0, 0), (44, 5), (5, 0), (17, 70), (64, 16), (1, 1), (200, 3)])
def test_attention_over_pages(dtype, case, mask):
    """Random keys: whole prompts, a portion at the end of a long context, and the pages behind the
    window already given back."""
    kernel, H, G, D, V, page = case
    window, keep = mask
    for n, n_new in ((37, 37), (150, 150), (333, 70), (333, 2)):
        k, v, sink, g = attention_case(dtype, n, H, G, D, V, seed=n + window)
        q = torch.randn(n_new, H, D, generator=g).to(tdt(dtype))
        scale = 1.5 * D ** -0.5
        want = plain_attention(q, k, v, torch.arange(n - n_new, n), sink, scale, window, keep)
        got = run_attention(kernel, dtype, q, k, v, n_new, sink, scale, window, keep, page, seed=n)
        close(got, want, dtype, f"{case} mask {mask}: {n_new} new of {n}", floor=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 32, 16), (2, 1, 64, 16), (3, 3, 16, 4), (16, 1, 16, 16), (2, 2, 128, 16)])
@pytest.mark.parametrize("mask", [(0, 0), (44, 5), (300, 0), (17, 70), (64, 300), (1, 0)])
@pytest.mark.parametrize("n", [1, 5, 256, 257, 700, 1100])
def test_one_new_token_over_partitions(dtype, sizes, mask, n):
    H, G, D, page = sizes
    window, keep = mask
    k, v, sink, g = attention_case(dtype, n, H, G, D, D, seed=n + keep)
    q = torch.randn(1, H, D, generator=g).to(tdt(dtype))
    scale = 1.5 * D ** -0.5
    want = plain_attention(q, k, v, torch.tensor([n - 1]), sink, scale, window, keep)
    got = run_attention("split", dtype, q, k, v, 1, sink, scale, window, keep, page, seed=n)
    close(got, want, dtype, f"{sizes} mask {mask}: one new token at {n - 1}", floor=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kernel", ["rows", "tiles", "split"])
@pytest.mark.parametrize("mask", [(44, 5), (64, 1), (9, 17), (130, 66)])
def test_a_planted_key_is_found_exactly_where_the_mask_allows(dtype, kernel, mask):
    """One key that the last query matches far better than any other, planted in turn at every
    place of interest: the window's two edges, the kept tokens' edge, page and tile edges, the
    first token, far back.  Where the mask lets it be seen the output is its value; elsewhere
    nothing of it may show."""
    window, keep = mask
    H, G, D, page, n = 2, 1, 32, 16, 600
    pos = n - 1
    places = sorted({0, keep - 1, keep, keep + 1, 15, 16, 63, 64, 255, 256, 300, pos - window - 1, pos - window,
                     pos - window + 1, pos - window + 2, pos - 1, pos} & set(range(n)))
    for where in places:
        k, v, sink, g = attention_case(dtype, n, H, G, D, D, seed=where)
        k = (k.float() * 0.1).to(tdt(dtype))
        q = torch.randn(1, H, D, generator=g)
        k[where, 0] = (q[0, 0] * 4).to(tdt(dtype))            # head 0 finds it; head 1 has its own random query
        q = q.to(tdt(dtype))
        scale = 1.0
        seen = where <= pos and (pos - where < window or where < keep)
        want = plain_attention(q, k, v, torch.tensor([pos]), sink, scale, window, keep)
        if seen:
            assert float((want[0, 0] - v[where, 0].double()).abs().max()) < 1e-2, "the case is meant to be decided by one key"
        got = run_attention(kernel, dtype, q, k, v, 1, sink, scale, window, keep, page, seed=where)
        close(got, want, dtype, f"{kernel} mask {mask}: a key planted at {where} ({'seen' if seen else 'not seen'})", floor=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kernel", ["rows", "tiles", "split"])
def test_sink_takes_weight_and_has_no_value(dtype, kernel):
    """A sink far above every score leaves almost nothing of the values; one far below changes
    nothing; without keys in sight but the token itself the sink still counts once."""
    H, G, D, page = 2, 2, 16, 16
    for n, window, keep in ((300, 0, 0), (300, 20, 2), (1, 20, 2)):
        k, v, _, g = attention_case(dtype, n, H, G, D, D, seed=n)
        q = torch.randn(1, H, D, generator=g).to(tdt(dtype))
        for sink in (torch.tensor([30.0, -30.0]), torch.tensor([0.0, 1.0])):
            want = plain_attention(q, k, v, torch.tensor([n - 1]), sink, 0.3, window, keep)
            got = run_attention(kernel, dtype, q, k, v, 1, sink, 0.3, window, keep, page)
            close(got, want, dtype, f"{kernel}: sinks {sink.tolist()}, {n} keys, mask {(window, keep)}", floor=0.05)
            if float(sink[0]) == 30.0:
                assert float(got[0, 0].float().abs().max()) < 1e-6, "a sink that takes all the weight leaves no output"


@pytest.mark.parametrize("dtype", DTYPES)
def test_requests_side_by_side_on_the_matrix_cores(dtype):
    """Prompt portions and single tokens of three requests in one step, as the mixer launches them."""
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.attention import AttentionWork
    from lyapunov_engine_amd.parts.base import StepBatch

    H, G, D, page, window, keep = 4, 2, 32, 16, 30, 5
    lens, news = [90, 300, 41], [50, 1, 41]
    g = torch.Generator().manual_seed(7)
    ks = [torch.randn(n, G, D, generator=g).to(tdt(dtype)) for n in lens]
    vs = [torch.randn(n, G, D, generator=g).to(tdt(dtype)) for n in lens]
    qs = [torch.randn(m, H, D, generator=g).to(tdt(dtype)) for m in news]
    sink = torch.randn(H, generator=g)
    n_blocks = [-(-n // page) for n in lens]
    kpool = torch.zeros(sum(n_blocks), G, page, D, dtype=tdt(dtype))
    vpool = torch.zeros(sum(n_blocks), G, D, page, dtype=tdt(dtype))
    order = np.random.default_rng(1).permutation(sum(n_blocks))
    tables, at = np.full((3, max(n_blocks)), -1, np.int32), 0
    for b, n in enumerate(lens):
        for i in range(n_blocks[b]):
            pg = int(order[at]); at += 1
            tables[b, i] = pg
            for o in range(min(page, n - i * page)):
                kpool[pg, :, o, :], vpool[pg, :, :, o] = ks[b][i * page + o], vs[b][i * page + o]
    q_start = np.concatenate([[0], np.cumsum(news)]).astype(np.int32)
    batch = StepBatch(start=np.array([n - m for n, m in zip(lens, news)], np.int32), count=np.array(news, np.int32),
                      q_start=q_start, ctx_len=np.array(lens, np.int32), T=int(q_start[-1]), B=3)
    arrays, meta = AttentionWork().plan(batch)
    qd = torch.cat([q.reshape(-1, H * D) for q in qs]).to(DEV)
    out = torch.zeros(int(q_start[-1]), H * D, dtype=tdt(dtype), device=DEV)
    common = dict(num_heads=H, num_kv_heads=G, head_dim=D, window=window, scale=0.3, keep_first=keep, sink=sink.to(DEV))
    ops.attn_prefill(qd, out, kpool.to(DEV), vpool.to(DEV), ints(tables), ints(q_start), ints(lens), ints(arrays["tile_seq"]),
                     ints(arrays["tile_q0"]), meta["n_tiles"], pair=False, **common)
    part_o, part_ml = torch.empty(H * 2 * D, device=DEV), torch.empty(H * 2 * 2, device=DEV)
    ops.attn_decode(qd, out, kpool.to(DEV), vpool.to(DEV), ints(tables), ints(q_start), ints(lens), ints(arrays["dec"]),
                    meta["n_dec"], part_o, part_ml, 2, 256, **common)
    for b in range(3):
        want = plain_attention(qs[b], ks[b], vs[b], torch.arange(lens[b] - news[b], lens[b]), sink, 0.3, window, keep)
        close(out[q_start[b]:q_start[b + 1]].view(news[b], H, D), want, dtype, f"request {b}", floor=0.1)


# --------------------------------------------------------------- feed-forward
@pytest.mark.parametrize("dtype", DTYPES)
def test_gate_with_limits(dtype):
    from lyapunov_engine_amd.kernels import ops

    I = 37
    z = torch.linspace(-9, 9, 2 * I * 5).view(5, 2 * I).to(tdt(dtype))
    got = ops.glu_clamped(z.to(DEV), 2.0, 1.702)
    g = torch.clamp(z.double()[:, :I], max=2.0)
    u = torch.clamp(z.double()[:, I:], min=-2.0, max=2.0)
    close(got, g * torch.sigmoid(1.702 * g) * (u + 1), dtype, "gate")


@pytest.mark.parametrize("sizes", [(5, 2), (12, 3), (64, 8), (70, 5), (130, 1), (3, 3), (1, 1)])
def test_router_chooses_the_largest_and_weighs_them_alone(sizes):
    from lyapunov_engine_amd.kernels import ops

    E, top = sizes
    g = torch.Generator().manual_seed(E)
    z = torch.randn(50, E, generator=g) * 3
    bias = torch.randn(E, generator=g)
    idx, wgt = ops.moe_route(z.to(DEV), bias.to(DEV), top)
    val, want_idx = torch.topk(z.double() + bias.double(), top, dim=-1)
    assert torch.equal(idx.cpu().long(), want_idx), "the chosen experts, largest first"
    close(wgt, torch.softmax(val, -1), "float32", "weights over the chosen alone")
    assert float((wgt.sum(-1) - 1).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(5, 2, 72), (12, 3, 192), (64, 8, 100), (130, 4, 256), (300, 1, 64), (1, 1, 40)])
def test_router_product_and_choice_in_one_kernel(dtype, sizes):
    """Logits in 32-bit from the activations, then the choice, for 1, 16, 17 and many rows; one
    more expert that every token uses may be appended with weight 1."""
    from lyapunov_engine_amd.kernels import ops

    E, top, K = sizes
    g = torch.Generator().manual_seed(E + K)
    w = torch.randn(E, K, generator=g)
    bias = torch.randn(E, generator=g)
    for T in (1, 16, 17, 700):
        x = torch.randn(T, K, generator=g).to(tdt(dtype))
        z = x.double() @ w.double().T + bias.double()
        val, want_idx = torch.topk(z, top, dim=-1)
        srt = torch.sort(z, -1, descending=True).values
        clear = torch.ones(T, dtype=torch.bool) if top == E else (srt[:, top - 1] - srt[:, top]) > 1e-3
        gaps = (srt[:, :top - 1] - srt[:, 1:top]).min(-1).values if top > 1 else torch.ones(T)
        clear &= gaps > 1e-3                                   # the order among the chosen, too
        for always in (-1, E):
            idx, wgt = ops.moe_route_from(x.to(DEV), w.to(DEV), bias.to(DEV), top, always)
            assert torch.equal(idx.cpu().long()[clear][:, :top], want_idx[clear]), f"{T} rows"
            close(wgt[:, :top][clear.to(DEV)], torch.softmax(val, -1)[clear], "float32", "weights", tol=1e-4)
            if always >= 0:
                assert (idx[:, top] == E).all() and (wgt[:, top] == 1.0).all()


@pytest.mark.parametrize("shape", [(1, 1, 1), (7, 5, 2), (300, 12, 3), (2000, 8, 8), (1500, 70, 5), (1030, 3, 1)])
def test_pairs_sorted_by_expert_in_their_own_order(shape):
    from lyapunov_engine_amd.kernels import ops

    T, E, top = shape
    g = torch.Generator().manual_seed(T)
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).int()
    plan = ops.moe_sort(idx.to(DEV), E)
    torch.cuda.synchronize()
    flat = idx.view(-1).numpy()
    off, sp, place = plan.expert_off.cpu().numpy(), plan.sorted_pair.cpu().numpy(), plan.place_of.cpu().numpy()
    assert off[0] == 0 and off[-1] == T * top
    for e in range(E):
        run = sp[off[e]:off[e + 1]]
        assert (flat[run] == e).all() and (np.diff(run) > 0).all(), f"expert {e}: its pairs, in rising order"
        assert len(run) == int((flat == e).sum())
    assert (sp[place] == np.arange(T * top)).all()
    n_tiles = int(plan.n_tiles.cpu()[0])
    te, tr = plan.tile_expert.cpu().numpy()[:n_tiles], plan.tile_row0.cpu().numpy()[:n_tiles]
    covered = np.zeros(T * top, bool)
    for e, r0 in zip(te, tr):
        assert off[e] <= r0 < off[e + 1]
        covered[r0:min(r0 + plan.tile_rows, off[e + 1])] = True
    assert covered.all() and n_tiles <= plan.most_tiles


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 5, 2, 72, 40, 28), (7, 5, 2, 72, 40, 0), (300, 3, 3, 64, 20, 16), (40, 70, 5, 48, 8, 24),
                                   (700, 4, 1, 100, 52, 0), (33, 16, 4, 192, 96, 64), (9, 6, 2, 64, 48, 48),
                                   (900, 6, 2, 64, 48, 48), (70, 130, 3, 40, 16, 0), (600, 3, 2, 256, 512, 0), (600, 2, 1, 512, 512, 512),
                                   (5, 12, 3, 512, 64, 0), (40, 7, 2, 1024, 32, 32)])    # few rows of a wide model: choice and sort in one kernel
def test_routed_experts_against_the_plain_mixture(dtype, shape):
    """The whole feed-forward part, with another branch's output added in, for steps of one token,
    of few and of many (tiles of 16 and of 128 rows), sizes without 16-byte rows among them, and a
    shared expert of the routed experts' size and limit (it then rides in their products)."""
    from lyapunov_engine_amd.parts.base import StepContext
    from lyapunov_engine_amd.parts.routed_experts import RoutedExperts

    T, E, top, H, I, S = shape
    g = torch.Generator().manual_seed(T + E)
    shared_limit = 1.2 if S == I else 0.8
    part = RoutedExperts(H, E, top, I, limit=1.2, gate_slope=1.702, shared_size=S, shared_limit=shared_limit)
    assert part.shared_folded == (S == I)
    w = {}
    for ws in part.weight_specs():
        pieces = []
        for src in ws.sources:
            t = torch.randn(src.shape, generator=g) * (1.0 if src.name.startswith("router") else 2.5 / math.sqrt(src.shape[-1]))
            w[src.name] = t.to(tdt(dtype))
            pieces.append(w[src.name])
        setattr(part, ws.attr, torch.cat(pieces).to(DEV))
    part.materialize(DEV, tdt(dtype))
    x = torch.randn(T, H, generator=g).to(tdt(dtype))
    addend = torch.randn(T, H, generator=g).to(tdt(dtype))
    ctx = StepContext(device=torch.device(DEV), dtype=tdt(dtype), T=T, B=1, token_ids=None, positions=None, q_start=None,
                      ctx_len=None, state_slots=None, logit_rows=None, R=0, groups=[])
    got = part.forward(ctx, x.to(DEV), addend=addend.to(DEV))
    assert got.dtype == torch.float32 and tuple(got.shape) == (1, T, H)
    mlp = dict(router=dict(experts=E, top=top), expert=dict(ff=I, limit=1.2), shared=dict(ff=S, limit=shared_limit) if S else None)
    wd = {k: v.double() for k, v in w.items()}
    want = RP.moe(x.double(), wd, mlp) + addend.double()
    # a router decision that hangs on rounding is no fault: leave such tokens out
    z = x.double() @ wd["router"].T + wd["router.b"]
    srt = torch.sort(z, -1, descending=True).values
    clear = torch.ones(T, dtype=torch.bool) if top == E else (srt[:, top - 1] - srt[:, top]) > (1e-4 if dtype == "float32" else 0.15)
    assert int(clear.sum()) >= T // 2
    close(got[0][clear.to(DEV)], want[clear], dtype, f"mixture {shape}", tol=2e-5 if dtype == "float32" else 3e-2)


def test_stream_add():
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(0)
    h, b = torch.randn(5, 70, generator=g), torch.randn(5, 70, generator=g)
    parts = torch.randn(3, 5, 70, generator=g)
    a16 = torch.randn(5, 70, generator=g).to(torch.bfloat16)
    hd = h.to(DEV)
    ops.stream_add(hd, parts.to(DEV), b.to(DEV))
    close(hd, h.double() + parts.double().sum(0) + b.double(), "float32", "partial sums and a second stream")
    hd = h.to(DEV)
    ops.stream_add(hd, a16.to(DEV))
    close(hd, h.double() + a16.double(), "float32", "activations")
    hd = h.to(DEV)
    ops.stream_add(hd, None, b.to(DEV))
    close(hd, h.double() + b.double(), "float32", "a second stream alone")
