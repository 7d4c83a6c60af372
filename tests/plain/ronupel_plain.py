"""A plain, slow Ronupel in torch on the CPU: whole sequences, no cache, no
pages, one function per mechanism.  It is what the engine is compared with and
shares no code with it (it imports nothing from the package; a model folder is
read with the safetensors library).

Ronupel is a decoder whose layers read one norm of the stream with both
branches (x += mixer(n) + ff(n), n = norm(x)); the mixer is grouped-query
attention with one RMS norm over the whole query projection and one over the
whole key projection, a rotation of neighbouring pairs on part of each head
with slowed-down frequencies, a sliding window that also keeps a sequence's
first tokens, and a learned sink in the softmax; the feed-forward routes every
token to a few experts and adds a shared one; a stretch of layers may run
several times, the embedding's rows being added to the stream again before each
further pass.  Everything runs in the precision of the tensors it is given (the
tests use 64-bit).

Notation: x the residual stream [n, width]; W matrices stored [out, in]; a
sequence's positions count from 0.
"""
from __future__ import annotations

import json
import os

import torch


# ------------------------------------------------------------------ small parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last axis, the eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def rotate_neighbours(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int, factor: float) -> torch.Tensor:
    """v [n, heads, D]: entries (2i, 2i+1), i < dims/2, of every head turn by the angle
    position * base^(-2i/dims) / factor; entries from ``dims`` on pass."""
    out = v.clone()
    for i in range(dims // 2):
        ang = positions.to(v.dtype) * (base ** (-2.0 * i / dims) / factor)
        c, s = ang.cos()[:, None], ang.sin()[:, None]
        a, b = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def visible(pos_q: torch.Tensor, pos_k: torch.Tensor, size: int, keep_first: int) -> torch.Tensor:
    """[queries, keys] booleans: position i sees position j when j is not in the future and either
    within the last ``size`` positions (i's own included) or among the sequence's first ``keep_first``."""
    i, j = pos_q[:, None], pos_k[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def sink_softmax(scores: torch.Tensor, mask: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """Row-wise weights of the visible keys (``scores`` [queries, keys]) when each row's
    denominator also holds e^sink: the sink has no key and no value and counts once."""
    s = scores.masked_fill(~mask, float("-inf"))
    m = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - m))


# ---------------------------------------------------------------------- mixer
def attention(h: torch.Tensor, w: dict, m: dict, eps: float, positions: torch.Tensor | None = None) -> torch.Tensor:
    """h [n, width] -> [n, width].  ``w``: the mixer's tensors by their short names
    (q, k, v, q.norm, k.norm, sink, o); ``m``: the mixer's entry of the configuration."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n) if positions is None else positions
    q = rms_norm(h @ w["q"].T, w["q.norm"], eps).view(n, H, D)      # one norm over all heads' rows
    k = rms_norm(h @ w["k"].T, w["k.norm"], eps).view(n, G, D)
    v = (h @ w["v"].T).view(n, G, V)
    rot = m.get("rot")
    if rot and int(rot["dims"]):                                    # no entry, or no dimensions: nothing turns
        factor = float(rot["scaling"]["factor"]) if rot.get("scaling") else 1.0
        q = rotate_neighbours(q, pos, float(rot["base"]), int(rot["dims"]), factor)
        k = rotate_neighbours(k, pos, float(rot["base"]), int(rot["dims"]), factor)
    if m.get("mask"):
        size, keep = int(m["mask"]["size"]), int(m["mask"].get("keep_first", 0))
    else:
        size, keep = n + int(pos.max()) + 1, 0                      # no mask: every earlier token is seen
    mask = visible(pos, pos, size, keep)
    out = torch.zeros(n, H, V, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)                                        # the key/value head this query head reads
        p = sink_softmax(q[:, head] @ k[:, g].T * float(m["scale"]), mask, w["sink"][head])
        out[:, head] = p @ v[:, g]
    return out.reshape(n, H * V) @ w["o"].T


# --------------------------------------------------------------- feed-forward
def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float) -> torch.Tensor:
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h: torch.Tensor, router: torch.Tensor, bias: torch.Tensor, top: int, chosen: torch.Tensor | None = None):
    """-> (experts [n, top], weights [n, top], margin [n], size [n]): the ``top`` largest of
    W_router h + bias, and the softmax over those alone; the margin is what the last chosen logit has
    over the first one left out, the size the largest logit's magnitude.  With ``chosen`` the choice is given (another run's, where the two must route
    alike to be compared) and only the weights are worked out."""
    z = h @ router.T + bias
    srt = torch.sort(z, dim=-1, descending=True).values
    margin = srt[:, top - 1] - srt[:, top] if top < z.shape[1] else torch.full((z.shape[0],), float("inf"), dtype=z.dtype)
    if chosen is None:
        val, idx = torch.topk(z, top, dim=-1)
    else:
        idx = chosen.long()
        val = torch.gather(z, 1, idx)
    return idx, torch.softmax(val, dim=-1), margin, z.abs().max(-1).values


def moe(h: torch.Tensor, w: dict, mlp: dict, chosen: torch.Tensor | None = None, notes: dict | None = None) -> torch.Tensor:
    """``w``: the feed-forward's tensors by short name (router, router.b, e<j>.gate/up/down,
    shared.gate/up/down).  ``notes`` receives the choice and its margin."""
    idx, wt, margin, size = route(h, w["router"], w["router.b"], int(mlp["router"]["top"]), chosen)
    if notes is not None:
        notes.update(chosen=idx, margin=margin, size=size)
    out = torch.zeros_like(h)
    limit = float(mlp["expert"]["limit"])
    for t in range(h.shape[0]):
        for e, p in zip(idx[t].tolist(), wt[t]):
            out[t] += p * expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)[0]
    if mlp.get("shared"):
        out = out + expert(h, w["shared.gate"], w["shared.up"], w["shared.down"], float(mlp["shared"]["limit"]))
    return out


# ---------------------------------------------------------------------- model
def sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer(x: torch.Tensor, tensors: dict, i: int, lc: dict, eps: float, chosen=None, notes=None) -> torch.Tensor:
    """x + mixer(n) + ff(n) with n = norm1(x)."""
    n = rms_norm(x, tensors[f"l{i}.norm1"], eps)
    y = attention(n, sub(tensors, f"l{i}.mix."), lc["mixer"], eps)
    if lc.get("mlp"):
        y = y + moe(n, sub(tensors, f"l{i}.mlp."), lc["mlp"], chosen, notes)
    return x + y


def running_order(cfg: dict) -> list:
    """(layer, whether the embedding's rows are added before it) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or int(loop["stop"]) <= int(loop["start"]):
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(a)]
    for t in range(times):
        order += [(i, t > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg: dict, tensors: dict, tokens, collect: list | None = None, chosen: list | None = None,
            notes: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one sequence; ``collect`` receives the stream after every layer run.
    ``chosen``: for every layer run with a routed feed-forward, in running order, the experts to use
    [n, top]; ``notes`` receives a dict per such run (the choice made, its margin)."""
    routed = 0
    eps = float(cfg["norm"]["eps"])
    x0 = tensors["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    for i, again in running_order(cfg):
        if again:
            x = x + x0
        note = {} if notes is not None else None
        has_ff = bool(cfg["layers"][i].get("mlp"))
        x = layer(x, tensors, i, cfg["layers"][i], eps, chosen[routed] if chosen is not None and has_ff else None, note)
        if has_ff:
            routed += 1
            if notes is not None:
                notes.append(note)
        if collect is not None:
            collect.append(x.clone())
    return rms_norm(x, tensors["final.norm"], eps) @ tensors["embed"].T


def load(folder: str, dtype=torch.float64):
    """config.json and the tensors of model.safetensors as ``dtype``."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for k in f.keys():
            t = f.get_tensor(k)
            tensors[k] = t.to(dtype) if t.is_floating_point() else t
    return cfg, tensors
