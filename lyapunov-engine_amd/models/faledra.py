"""The Faledra architecture as a ModelSpec.

A decoder whose layers wrap each branch in two norms ("sandwich" arrangement,
with a multiplier on what joins the stream), filter the mixer's input with a
short causal convolution, mix by latent attention (with a sink) or by a minGRU
recurrence, feed forward through a dense xIELU layer, and may run a stretch of
layers several times in a row: every pass has a cache and state of its own and
is entered with a learned vector added to the stream.

Tensor names: ``embed``, ``loop.step`` [passes, width], ``l<i>.norm1`` /
``norm1b`` / ``norm2`` / ``norm2b``, ``l<i>.canon1`` [width, taps],
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.faledra_config import FaledraConfig
from ..config.registry import register_architecture
from ..config.specs import LayerCall, LayerSpec, ModelSpec, PartSpec

# No longest sequence is part of the design; position tables get as many rows as the engine's
# pool and model length allow (DecoderModel.materialize).
POSITIONS = 1 << 20

LAYER_NAMES = {"norm1": "norm1", "norm1_out": "norm1b", "norm2": "norm2", "norm2_out": "norm2b", "mixer": "mix.",
               "ffn": "mlp.", "filter": "canon1"}


def running_order(cfg: FaledraConfig) -> tuple:
    """Layers before the loop, the looped stretch once per pass (a cache buffer of its own per
    pass, the pass's vector added before its first layer), the layers after it."""
    calls, cache = [], 0
    n = len(cfg.layers)
    if not cfg.has_loop:
        return tuple(LayerCall(i, i) for i in range(n))
    for i in range(cfg.loop_start):
        calls.append(LayerCall(i, cache))
        cache += 1
    for t in range(cfg.loop_times):
        for i in range(cfg.loop_start, cfg.loop_stop):
            calls.append(LayerCall(i, cache, shift=t if i == cfg.loop_start else None))
            cache += 1
    for i in range(cfg.loop_stop, n):
        calls.append(LayerCall(i, cache))
        cache += 1
    return tuple(calls)


def faledra_spec(cfg: FaledraConfig) -> ModelSpec:
    def norm():
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "tensor": ""})

    layers, ignorable = [], []
    for i, lc in enumerate(cfg.layers):
        m = lc.mixer
        if lc.type == "latent_attention":
            position = None
            if int(m["rot_dim"]) and int(m["rot"]["dims"]):
                position = PartSpec("rope", {"dim": int(m["rot"]["dims"]), "theta": float(m["rot"]["base"]),
                                             "max_position": POSITIONS})
            mixer = PartSpec("latent_attention", {
                "hidden_size": cfg.width, "num_heads": int(m["heads"]), "dim": int(m["dim"]),
                "rot_dim": int(m["rot_dim"]), "vdim": int(m["vdim"]), "q_rank": int(m["q_rank"]),
                "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "eps": cfg.norm_eps, "position": position})
        else:
            mixer = PartSpec("mingru", {"hidden_size": cfg.width, "width": int(m["width"])})
        ffn = None
        extra = {"norm1_out": norm()}
        if lc.mlp is not None:
            ffn = PartSpec("dense", {"hidden_size": cfg.width, "intermediate_size": int(lc.mlp["ff"]),
                                     "activation": "xielu"})
            extra["norm2_out"] = norm()
        else:
            ignorable += [f"l{i}.norm2", f"l{i}.norm2b"]
        if cfg.canon_taps:
            extra["filter"] = PartSpec("short_conv", {"channels": cfg.width, "taps": cfg.canon_taps, "tensor": ""})
        layers.append(LayerSpec(block="sandwich", mixer=mixer, ffn=ffn, norm1=norm(), norm2=norm(), names=LAYER_NAMES,
                                extra=extra, params={"mult": cfg.residual_mult}))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), schedule=running_order(cfg),
        final_norm=norm(), tie_word_embeddings=False, max_position=POSITIONS,
        embed_prefix="embed", final_norm_prefix="final.norm", head_prefix="head", layer_prefix="l{i}.",
        embedding=PartSpec("lookup", {"scale": cfg.embedding_scale, "tensor": ""}),
        head=PartSpec("linear", {"tensor": ""}),
        stream_shift=PartSpec("table", {"count": cfg.loop_times, "tensor": ""}) if cfg.has_loop else None,
        stream_shift_prefix="loop.step",
        eos_token_ids=tuple(cfg.eos_token_id), ignorable_tensors=tuple(ignorable),
        init_std=0.05,
    )


register_architecture("Faledra", FaledraConfig, faledra_spec, replace=True)
