"""The Ronupel architecture as a ModelSpec.

A decoder whose layers read one norm of the stream with both branches
("parallel" arrangement: h += mixer(n) + ff(n), n = norm1(h)); the mixer is
grouped-query attention with one RMS norm over the whole query projection and
one over the whole key projection, a rotation of neighbouring pairs on part of
every head with frequencies divided by a constant, a window that also keeps a
sequence's first tokens, and a sink in the softmax; the feed-forward routes a
token to a few of many experts and adds a shared one.  A stretch of layers may
run several times in a row: every pass has a cache of its own, and before each
pass but the first the embedding's output is added to the stream again.  The
output head is the embedding's matrix.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.{q,k,v,q.norm,k.norm,sink,o}``,
``l<i>.mlp.{router,router.b,e<j>.{gate,up,down},shared.{gate,up,down}}``,
``final.norm``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.ronupel_config import RonupelConfig
from ..config.specs import LayerCall, LayerSpec, ModelSpec, PartSpec

# No longest sequence is part of the design; position tables get as many rows as the engine's
# pool and model length allow (DecoderModel.materialize).
POSITIONS = 1 << 20

LAYER_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp."}

# The constant in the experts' gate, g * sigmoid(GATE_SLOPE * g): fixed by the design.
GATE_SLOPE = 1.702


def running_order(cfg: RonupelConfig) -> tuple:
    """Layers before the loop, the looped stretch once per pass (a cache buffer of its own per
    pass; from the second pass on the embedding's output joins the stream before the pass's first
    layer), the layers after it."""
    n = len(cfg.layers)
    if not cfg.has_loop:
        return tuple(LayerCall(i, i) for i in range(n))
    calls, cache = [], 0
    for i in range(cfg.loop_start):
        calls.append(LayerCall(i, cache))
        cache += 1
    for t in range(cfg.loop_times):
        for i in range(cfg.loop_start, cfg.loop_stop):
            calls.append(LayerCall(i, cache, reinject=t > 0 and i == cfg.loop_start))
            cache += 1
    for i in range(cfg.loop_stop, n):
        calls.append(LayerCall(i, cache))
        cache += 1
    return tuple(calls)


def ronupel_spec(cfg: RonupelConfig) -> ModelSpec:
    def norm():
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "tensor": ""})

    layers = []
    for lc in cfg.layers:
        m = lc.mixer
        position = None
        rot = m.get("rot")
        if rot is not None and int(rot["dims"]) > 0:
            scaling = None
            if rot.get("scaling") is not None:
                scaling = {"rope_type": "linear", "factor": float(rot["scaling"]["factor"])}
            position = PartSpec("rope", {"dim": int(rot["dims"]), "theta": float(rot["base"]), "max_position": POSITIONS,
                                         "scaling": scaling, "precise": True})
        mask = m.get("mask") or {}
        mixer = PartSpec("sink_window_attention", {
            "hidden_size": cfg.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
            "dim": int(m["dim"]), "vdim": int(m["vdim"]), "scale": float(m["scale"]),
            "window": int(mask.get("size", 0)), "keep_first": int(mask.get("keep_first", 0)),
            "qk_norm": True, "sink": True, "eps": cfg.norm_eps, "position": position})
        ffn = None
        if lc.mlp is not None:
            shared = lc.mlp.get("shared")
            ffn = PartSpec("routed_experts", {
                "hidden_size": cfg.width, "num_experts": int(lc.mlp["router"]["experts"]),
                "top": int(lc.mlp["router"]["top"]), "intermediate_size": int(lc.mlp["expert"]["ff"]),
                "limit": float(lc.mlp["expert"]["limit"]), "gate_slope": GATE_SLOPE,
                "shared_size": int(shared["ff"]) if shared else 0,
                "shared_limit": float(shared["limit"]) if shared else 0.0})
        layers.append(LayerSpec(block="parallel", mixer=mixer, ffn=ffn, norm1=norm(), norm2=norm(), names=LAYER_NAMES))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), schedule=running_order(cfg),
        final_norm=norm(), tie_word_embeddings=True, max_position=POSITIONS,
        embed_prefix="embed", final_norm_prefix="final.norm", head_prefix="head", layer_prefix="l{i}.",
        embedding=PartSpec("lookup", {"tensor": ""}), head=PartSpec("linear", {"tensor": ""}),
        eos_token_ids=tuple(cfg.eos_token_id), init_std=0.05,
    )


register_architecture("Ronupel", RonupelConfig, ronupel_spec, replace=True)
