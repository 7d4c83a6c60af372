"""A plain, slow Faledra in torch on the CPU: whole sequences, no cache, no
pages, one function per mechanism.  It is what the engine is compared with and
shares no code with it (it imports nothing from the package; a model folder is
read with the safetensors library).

Faledra is a decoder whose layers put a norm in front of and behind each branch,
filter the mixer's input with a short causal convolution over time, mix either
with attention through a low-rank latent (one shared rotated key part, a learned
sink in the softmax) or with a minGRU recurrence, feed forward through a dense
layer with the xIELU activation, and may run a stretch of layers several times.
Everything here runs in the precision of the tensors it is given (the tests use
64-bit).

Notation: x the residual stream [n, width]; W matrices stored [out, in]; a
sequence's positions count from 0.
"""
from __future__ import annotations

import json
import math
import os

import torch


# ------------------------------------------------------------------ small parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight, the eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def embed(tokens, table: torch.Tensor, scale: float) -> torch.Tensor:
    """Row lookup times a constant."""
    return table[torch.as_tensor(tokens, dtype=torch.long)] * scale


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(v: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(v))


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """z > 0:  softplus(p) z^2 + z/2;  z <= 0:  (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def short_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """Causal filter over time on each channel, h [n, C], w [C, taps]:
    out_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the start."""
    n, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate_pairs(v: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Rotation of neighbouring pairs (2i, 2i+1) of the first ``dims`` entries of
    the last axis by the angle position * base^(-2i/dims); the rest passes.
    v [n, ..., D], positions [n]."""
    out = v.clone()
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=v.dtype)
    ang = positions.to(v.dtype)[:, None] * freq[None, :]                 # [n, half]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [half]
    cos, sin = ang.cos().reshape(shape), ang.sin().reshape(shape)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def sink_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sink: torch.Tensor,
                           scale: float) -> torch.Tensor:
    """Causal attention of one sequence, q [n, H, Dk], k [n, H, Dk], v [n, H, Dv]:
    weights_ij = exp(s_ij) / (exp(sink_h) + sum_(j' <= i) exp(s_ij')), s = scale * q.k;
    the sink has no key, no value and no scale."""
    n, H = q.shape[0], q.shape[1]
    out = torch.zeros(n, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        s = (q[:, h] @ k[:, h].T) * scale                               # [n, n]
        mask = torch.ones(n, n).tril().bool()
        s = s.masked_fill(~mask, float("-inf"))
        m = torch.maximum(s.max(dim=-1).values, sink[h])
        e = torch.exp(s - m[:, None])
        denom = e.sum(-1) + torch.exp(sink[h] - m)
        out[:, h] = (e / denom[:, None]) @ v[:, h]
    return out


# ------------------------------------------------------------------------ mixers
def latent_attention(h: torch.Tensor, w: dict, cfg: dict, eps: float) -> torch.Tensor:
    """Attention whose queries, keys and values come out of low-rank latents.
    w: the layer's 'mix.*' tensors by their short names."""
    n = h.shape[0]
    H, dim, rot, vdim, rank = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    pos = torch.arange(n)
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(n, H, dim + rot)
    q_plain, q_rot = q[..., :dim], q[..., dim:]
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    k_rot = down[:, rank:]                                               # one rotated part for all heads
    k_plain = (c @ w["uk"].T).reshape(n, H, dim)
    v = (c @ w["uv"].T).reshape(n, H, vdim)
    base, dims = cfg["rot"]["base"], cfg["rot"]["dims"]
    q_rot = rotate_pairs(q_rot, pos, base, dims)
    k_rot = rotate_pairs(k_rot[:, None, :], pos, base, dims).expand(n, H, rot)
    qq = torch.cat((q_plain, q_rot), dim=-1)
    kk = torch.cat((k_plain, k_rot), dim=-1)
    o = sink_softmax_attention(qq, kk, v, w["sink"], cfg["scale"])
    return o.reshape(n, H * vdim) @ w["o"].T


def mingru(h: torch.Tensor, w: dict) -> torch.Tensor:
    """S_t = (1 - z_t) S_(t-1) + z_t c_t with gates that read the current token
    only; c = u + 1/2 for u >= 0, sigmoid(u) below; out = W_o (S_t * silu(W_g h))."""
    z = torch.sigmoid(h @ w["z"].T + w["z.b"])
    u = h @ w["x"].T + w["x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ w["g"].T
    state = torch.zeros(z.shape[1], dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        state = (1.0 - z[t]) * state + z[t] * cand[t]
        rows.append(state * (g[t] * torch.sigmoid(g[t])))
    return torch.stack(rows) @ w["o"].T


def dense_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    return xielu(h @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


# ------------------------------------------------------------------------- model
def layer_order(n_layers: int, loop) -> list:
    """[(layer, pass number or None, first of its pass)] in running order."""
    if not loop or int(loop.get("times", 1)) < 1:
        return [(i, None, False) for i in range(n_layers)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None, False) for i in range(start)]
    for t in range(times):
        order += [(i, t, i == start) for i in range(start, stop)]
    return order + [(i, None, False) for i in range(stop, n_layers)]


def sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(tokens, tensors: dict, config: dict, trace: list | None = None) -> torch.Tensor:
    """Logits [n, vocab] of one whole sequence.  ``trace`` collects the residual
    stream after every layer run."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    x = embed(tokens, tensors["embed"], config["embedding"]["scale"])
    for i, t, first in layer_order(len(config["layers"]), config.get("loop")):
        lc, p = config["layers"][i], f"l{i}."
        if first:
            x = x + tensors["loop.step"][t]
        h = rms_norm(x, tensors[p + "norm1"], eps)
        if p + "canon1" in tensors:
            h = h + short_conv(h, tensors[p + "canon1"])
        if lc["type"] == "latent_attention":
            y = latent_attention(h, sub(tensors, p + "mix."), lc["mixer"], eps)
        elif lc["type"] == "mingru":
            y = mingru(h, sub(tensors, p + "mix."))
        else:
            raise ValueError(lc["type"])
        x = x + m * rms_norm(y, tensors[p + "norm1b"], eps)
        if lc.get("mlp"):
            y = dense_ff(rms_norm(x, tensors[p + "norm2"], eps), sub(tensors, p + "mlp."))
            x = x + m * rms_norm(y, tensors[p + "norm2b"], eps)
        if trace is not None:
            trace.append(x.clone())
    return rms_norm(x, tensors["final.norm"], eps) @ tensors["head"].T


def load_folder(folder: str, dtype=torch.float64):
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for k in f.keys():
            t = f.get_tensor(k)
            tensors[k] = t.to(dtype) if t.is_floating_point() else t
    return config, tensors
