"""Small Ronupel models with random weights for the tests, and their logits by
the plain implementation (tests/plain/ronupel_plain.py, 64-bit)."""
import json
import os

import torch

from plain import ronupel_plain as RP


def attn(heads, kv_heads, dim, vdim, *, window=None, keep=0, dims=None, base=10000.0, factor=None, scale=None, mlp=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 2.0 * dim ** -0.5)
    if window is not None:
        mixer["mask"] = dict(size=window, keep_first=keep)
    dims = dim if dims is None else dims
    if dims:
        mixer["rot"] = dict(base=base, dims=dims)
        if factor is not None:
            mixer["rot"]["scaling"] = dict(factor=factor)
    return dict(type="attention", mixer=mixer, mlp=mlp)


def moe(experts, top, ff, limit, shared=None):
    d = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff, limit=limit))
    if shared is not None:
        d["shared"] = dict(ff=shared[0], limit=shared[1])
    return d


def config(vocab, width, layers, *, loop=None, eps=1e-5):
    c = dict(architecture="Ronupel", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)
    if loop:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    return c


# Three configurations that differ in every size and option; none of their sizes coincide where a
# model's might by chance (key and value sizes, heads x value size and width, experts' width and
# the shared expert's, rotated dimensions and the head's).
#   A: odd sizes (the row-by-row attention kernel, products without 16-byte rows), every query head
#      with a key/value head of its own and all sharing one, windows shorter than a page, a window
#      that keeps nothing, a layer without feed-forward, a loop from the first layer on run twice
#   B: sizes the matrix-core kernels take, every expert chosen and a single one chosen, no shared
#      expert and one, more kept first tokens than a tile of keys holds, no loop
#   C: heads of 64, a layer that sees everything (no mask) and does not rotate, frequencies scaled by
#      1, a loop in the middle run three times, limits that never bind and limits that bind all the time
CONFIGS = {
    "A": config(203, 72, [attn(3, 3, 24, 20, window=9, keep=2, dims=10, base=500.0, factor=3.0, scale=0.4,
                               mlp=moe(5, 2, 40, 1.5, shared=(28, 3.0))),
                          attn(4, 1, 10, 12, window=5, keep=0, scale=0.6),
                          attn(2, 2, 6, 30, window=3, keep=7, dims=2, base=50.0, factor=1.5, scale=0.8,
                               mlp=moe(3, 3, 20, 0.7))],
                loop=(0, 2, 2), eps=1e-5),
    "B": config(150, 128, [attn(4, 2, 32, 32, window=21, keep=3, dims=16, base=30000.0, factor=4.0, scale=0.35,
                                mlp=moe(8, 8, 48, 2.5)),
                           attn(2, 2, 16, 16, window=100, keep=70, dims=16, base=300.0, scale=0.5,
                                mlp=moe(6, 1, 80, 4.0, shared=(64, 1.0)))],
                eps=1e-6),
    "C": config(320, 96, [attn(2, 1, 64, 64, window=33, keep=1, dims=64, base=1e6, factor=1.0, scale=0.25,
                               mlp=moe(16, 4, 24, 50.0, shared=(40, 0.3))),
                          attn(6, 3, 16, 16, dims=0, scale=0.5, mlp=moe(4, 2, 56, 0.2)),
                          attn(3, 3, 32, 32, window=64, keep=16, dims=8, base=77.0, factor=16.0, scale=0.3,
                               mlp=moe(9, 3, 32, 1.0, shared=(32, 1.0)))],      # a shared expert like the routed ones
                loop=(1, 2, 3), eps=1e-6),
}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 16}


def write_model(folder: str, cfg: dict, seed: int, dtype: str, std: float = 0.25) -> str:
    """config.json and model.safetensors with weights drawn so that faults show: projections wide
    enough for peaked attention and for gates that reach their limits, sinks, router weights and
    biases of order one, norm weights around one."""
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
        elif name.endswith(".sink") or name.endswith(".b") or name == "embed":
            t = t * 1.0
        elif name.endswith(".router"):
            t = t * 0.5
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
        _PLAIN[folder] = RP.load(folder)
    cfg, tensors = _PLAIN[folder]
    return {rid: RP.forward(cfg, tensors, toks) for rid, toks in requests.items()}


class RouterLog:
    """Collects the engine's router choices while a trace is replayed (``with RouterLog() as log``)
    and sorts them by request: ``log.by_request(trace)`` -> id -> one tensor [len, top] per layer run
    with a routed feed-forward, in running order."""

    def __enter__(self):
        from lyapunov_engine_amd.parts.routed_experts import RoutedExperts

        self.cls = RoutedExperts
        self.cls.choices_log = self.calls = []
        return self

    def __exit__(self, *exc):
        self.cls.choices_log = None

    def by_request(self, trace) -> dict:
        steps = [s for s in trace.steps if s["entries"]]
        runs = len(self.calls) // len(steps)
        assert runs * len(steps) == len(self.calls)
        out = {rid: [[] for _ in range(runs)] for rid in trace.requests}
        for n, s in enumerate(steps):
            for r in range(runs):
                idx, at = self.calls[n * runs + r].cpu(), 0
                for e in s["entries"]:
                    out[e["id"]][r].append(idx[at:at + len(e["tokens"])])
                    at += len(e["tokens"])
        return {rid: [torch.cat(p) for p in per] if per and per[0] else [] for rid, per in out.items()}


def plain_logits_routed_alike(folder: str, requests: dict, chosen: dict, clear: float = 0.1) -> dict:
    """As ``plain_logits`` with the experts the engine chose.  A 16-bit run may decide a close call
    the other way, which says nothing about its kernels; what it must not do is choose otherwise
    where the plain model's margin is clear (more than ``clear`` of the token's largest router logit, and
    more than 0.5): that is asserted here."""
    if folder not in _PLAIN:
        _PLAIN[folder] = RP.load(folder)
    cfg, tensors = _PLAIN[folder]
    out = {}
    for rid, toks in requests.items():
        out[rid] = RP.forward(cfg, tensors, toks, chosen=chosen[rid])
        # the plain model's own choices, and where they differ from the engine's the margin must be small
        notes_free = []
        RP.forward(cfg, tensors, toks, notes=notes_free)
        for run, (nf, theirs) in enumerate(zip(notes_free, chosen[rid])):
            differs = (torch.sort(theirs.long(), -1).values != torch.sort(nf["chosen"], -1).values).any(-1)
            if differs.any():
                first = int(torch.nonzero(differs)[0])      # later tokens follow another history
                assert float(nf["margin"][first]) < max(0.5, clear * float(nf["size"][first])), (f"request {rid!r}, routed layer run {run}, position {first}: "
                                                            f"the engine chose {theirs[first].tolist()}, the plain model "
                                                            f"{nf['chosen'][first].tolist()} with a margin of {float(nf['margin'][first]):.3f}")
                break
    return out


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
