"""Typed configuration of the Faledra decoder, read from config.json.

The file names its architecture in the singular (``"architecture": "Faledra"``)
and nests its constants: ``vocab``, ``width``, ``residual_mult``,
``embedding.scale``, ``norm.eps``, ``canon.taps`` (the input filter; absent or
null: none), ``loop`` (``start``, ``stop``, ``times``; absent or null: every
layer runs once) and ``layers``, a list whose entries give ``type`` (which
mixer), ``mixer`` (its sizes and constants) and ``mlp`` (``kind`` and ``ff``, or
null for a layer without a feed-forward).  Every size and constant comes from
the file; a missing one is an error.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

from .model_config import ConfigError

MIXER_TYPES = ("latent_attention", "mingru")
MLP_KINDS = ("dense",)


def _need(d: dict, keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ConfigError(f"{where} must be an object, got {type(d).__name__}")
    missing = [k for k in keys if k not in d]
    if missing:
        raise ConfigError(f"{where} lacks {missing}")


@dataclass(frozen=True)
class FaledraLayer:
    type: str
    mixer: dict                      # the mixer's sizes and constants as the file gives them
    mlp: Optional[dict]              # {"kind", "ff"} or None

    @staticmethod
    def from_dict(d: dict, i: int) -> "FaledraLayer":
        where = f"layers[{i}]"
        _need(d, ("type", "mixer"), where)
        kind, mixer, mlp = d["type"], d["mixer"], d.get("mlp")
        if kind == "latent_attention":
            _need(mixer, ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale"), where + ".mixer")
            if int(mixer["rot_dim"]) > 0:
                _need(mixer, ("rot",), where + ".mixer")
                _need(mixer["rot"], ("base", "dims"), where + ".mixer.rot")
                dims = int(mixer["rot"]["dims"])
                if dims % 2 or not 0 <= dims <= int(mixer["rot_dim"]) or not float(mixer["rot"]["base"]) > 0:
                    raise ConfigError(f"{where}.mixer.rot: {dims} rotated dimensions of {mixer['rot_dim']}, base "
                                      f"{mixer['rot']['base']}")
            for k in ("heads", "vdim", "q_rank", "kv_rank"):
                if int(mixer[k]) <= 0:
                    raise ConfigError(f"{where}.mixer.{k} must be positive, got {mixer[k]}")
            if int(mixer["dim"]) < 0 or int(mixer["rot_dim"]) < 0 or int(mixer["dim"]) + int(mixer["rot_dim"]) == 0:
                raise ConfigError(f"{where}.mixer: heads of {mixer['dim']} plain and {mixer['rot_dim']} rotated dimensions")
        elif kind == "mingru":
            _need(mixer, ("width",), where + ".mixer")
            if int(mixer["width"]) <= 0:
                raise ConfigError(f"{where}.mixer.width must be positive, got {mixer['width']}")
        else:
            raise ConfigError(f"{where}: mixer type {kind!r} is not implemented (known: {list(MIXER_TYPES)})")
        if mlp is not None:
            _need(mlp, ("kind", "ff"), where + ".mlp")
            if mlp["kind"] not in MLP_KINDS:
                raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r} is not implemented (known: {list(MLP_KINDS)})")
            if int(mlp["ff"]) <= 0:
                raise ConfigError(f"{where}.mlp.ff must be positive, got {mlp['ff']}")
        return FaledraLayer(kind, dict(mixer), dict(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": dict(self.mixer), "mlp": dict(self.mlp) if self.mlp is not None else None}


@dataclass(frozen=True)
class FaledraConfig:
    vocab: int
    width: int
    residual_mult: float
    embedding_scale: float
    norm_eps: float
    layers: tuple                    # of FaledraLayer
    canon_taps: int = 0              # 0: no input filter
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1              # layers loop_start .. loop_stop - 1 run this many times in a row
    architectures: tuple = ("Faledra",)
    eos_token_id: tuple = ()
    extra: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, d: dict) -> "FaledraConfig":
        _need(d, ("vocab", "width", "residual_mult", "embedding", "norm", "layers"), "config.json")
        _need(d["embedding"], ("scale",), "embedding")
        _need(d["norm"], ("eps",), "norm")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers must be a list with at least one entry")
        layers = tuple(FaledraLayer.from_dict(l, i) for i, l in enumerate(d["layers"]))
        taps = 0
        if d.get("canon") is not None:
            _need(d["canon"], ("taps",), "canon")
            taps = int(d["canon"]["taps"])
            if taps < 1:
                raise ConfigError(f"canon.taps must be at least 1, got {taps}")
        start = stop = 0
        times = 1
        if d.get("loop") is not None:
            _need(d["loop"], ("start", "stop", "times"), "loop")
            start, stop, times = int(d["loop"]["start"]), int(d["loop"]["stop"]), int(d["loop"]["times"])
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"loop: layers {start} .. {stop - 1} of {len(layers)}, {times} times")
        known = {"architecture", "architectures", "vocab", "width", "residual_mult", "embedding", "norm", "layers",
                 "canon", "loop", "eos_token_id"}
        eos = d.get("eos_token_id")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), residual_mult=float(d["residual_mult"]),
                  embedding_scale=float(d["embedding"]["scale"]), norm_eps=float(d["norm"]["eps"]), layers=layers,
                  canon_taps=taps, loop_start=start, loop_stop=stop, loop_times=times,
                  eos_token_id=() if eos is None else tuple(int(t) for t in (eos if isinstance(eos, list) else [eos])),
                  extra={k: v for k, v in d.items() if k not in known})
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.norm_eps > 0:
            raise ConfigError(f"vocab {cfg.vocab}, width {cfg.width}, norm.eps {cfg.norm_eps}")
        return cfg

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start

    def to_dict(self) -> dict:
        d = {"architecture": "Faledra", "vocab": self.vocab, "width": self.width, "residual_mult": self.residual_mult,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "layers": [l.to_dict() for l in self.layers]}
        if self.canon_taps:
            d["canon"] = {"taps": self.canon_taps}
        if self.has_loop:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d


__all__ = ["FaledraConfig", "FaledraLayer"]
