"""Small Faledra models with random weights for the tests, and their logits by
the plain implementation (tests/plain/faledra_plain.py, 64-bit)."""
import json
import os

import torch

from plain import faledra_plain as FP


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, *, dims=None, base=10000.0, scale=None, ff=None):
    mixer = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank,
                 scale=scale if scale is not None else (dim + rot_dim) ** -0.5,
                 rot=dict(base=base, dims=rot_dim if dims is None else dims))
    return dict(type="latent_attention", mixer=mixer, mlp=dict(kind="dense", ff=ff) if ff else None)


def gru(width, ff=None):
    return dict(type="mingru", mixer=dict(width=width), mlp=dict(kind="dense", ff=ff) if ff else None)


def config(vocab, width, layers, *, taps=None, loop=None, mult=1.0, emb_scale=1.0, eps=1e-5):
    c = dict(architecture="Faledra", vocab=vocab, width=width, residual_mult=mult, embedding=dict(scale=emb_scale),
             norm=dict(eps=eps), layers=layers)
    if taps:
        c["canon"] = dict(taps=taps)
    if loop:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return c


# Three configurations that differ in every size and option; none of their sizes coincide where a
# model's might by chance (plain and value sizes, heads x value size and width, feed-forward and
# width, rotated dimensions and rotated part).
#   A: odd sizes, four taps, a loop in the middle that runs three times, a layer without feed-forward,
#      fewer rotated dimensions than the rotated part has
#   B: no loop, one tap (a filter without memory), one head, a recurrence first
#   C: sizes in multiples of 16 (what the matrix-core attention kernel takes), two taps, a loop from
#      the first layer on that runs once
CONFIGS = {
    "A": config(203, 72, [gru(40, ff=100),
                          latent(3, 24, 8, 20, 36, 40, dims=6, ff=88),
                          latent(2, 10, 14, 12, 28, 24, base=500.0, scale=0.3),
                          gru(56)],
                taps=4, loop=(1, 3, 3), mult=0.6, emb_scale=3.0, eps=1e-5),
    "B": config(150, 64, [gru(64, ff=48),
                          latent(1, 32, 16, 48, 24, 48, ff=80),
                          latent(5, 16, 16, 8, 40, 32, ff=64)],
                taps=1, mult=1.0, emb_scale=1.0, eps=1e-6),
    "C": config(320, 128, [latent(4, 32, 32, 16, 64, 64, ff=192),
                           gru(96, ff=64),
                           latent(8, 16, 16, 32, 48, 96, base=20000.0)],
                taps=2, loop=(0, 2, 1), mult=0.8, emb_scale=8.0, eps=1e-6),
}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 16}


def write_model(folder: str, cfg: dict, seed: int, dtype: str, std: float = 0.2) -> str:
    """config.json and model.safetensors with weights drawn so that faults show: matrices wide
    enough for peaked attention, sinks and biases of order one, filter taps of order one half,
    norm weights around one."""
    from lyapunov_engine_amd.config.registry import architecture_of
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.weights.safetensors_io import write_safetensors

    arch = architecture_of(cfg)
    model = build_model(arch.to_spec(arch.config_class.from_dict(cfg)))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, init) in model.expected_tensors().items():
        t = torch.randn(shape, generator=g)
        if init == "ones":
            t = 1.0 + 0.2 * t
        elif name.endswith(".sink") or name.endswith(".b"):
            t = t * 1.0
        elif name.endswith("canon1") or name.endswith(".act") or name == "loop.step":
            t = t * 0.5
        elif name == "embed":
            t = t * 1.0
        else:
            t = t * std * (32.0 / shape[-1]) ** 0.5
        tensors[name] = t.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    os.makedirs(folder, exist_ok=True)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


_PLAIN: dict = {}


def plain_logits(folder: str, requests: dict) -> dict:
    """id -> [len, vocab] 64-bit logits of every whole request."""
    if folder not in _PLAIN:
        _PLAIN[folder] = FP.load_folder(folder)
    cfg, tensors = _PLAIN[folder]
    return {rid: FP.forward(toks, tensors, cfg) for rid, toks in requests.items()}


def plain_greedy(folder: str, prompt: list, n: int):
    """n greedy tokens after the prompt, and the margin between the best two logits at each."""
    toks, out, margins = list(prompt), [], []
    for _ in range(n):
        row = plain_logits(folder, {"g": toks})["g"][-1]
        top = torch.topk(row, 2)
        out.append(int(top.indices[0]))
        margins.append(float(top.values[0] - top.values[1]))
        toks.append(out[-1])
    return out, margins
