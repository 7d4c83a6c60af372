"""Typed configuration of the Ronupel decoder, read from config.json.

The file names its architecture in the singular (``"architecture": "Ronupel"``)
and nests its constants: ``vocab``, ``width``, ``norm.eps``, ``loop`` (``start``,
``stop``, ``times``; absent or null: every layer runs once) and ``layers``, a
list whose entries give ``type`` (which mixer), ``mixer`` (its sizes and
constants) and ``mlp`` (its feed-forward, or null for none):

    mixer   heads, kv_heads, dim, vdim, scale,
            mask {size, keep_first}          absent or null: every earlier token is seen
            rot {base, dims, scaling {factor}}   absent, null or dims 0: no rotation; no scaling: factor 1
    mlp     kind "moe", router {experts, top}, expert {ff, limit},
            shared {ff, limit}               absent or null: no shared expert

Every size and constant comes from the file; a missing one is an error.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

from .model_config import ConfigError

MIXER_TYPES = ("attention",)
MLP_KINDS = ("moe",)


def _need(d, keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ConfigError(f"{where} must be an object, got {type(d).__name__}")
    missing = [k for k in keys if k not in d]
    if missing:
        raise ConfigError(f"{where} lacks {missing}")


@dataclass(frozen=True)
class RonupelLayer:
    type: str
    mixer: dict                      # the mixer's sizes and constants as the file gives them
    mlp: Optional[dict]              # the feed-forward's, or None

    @staticmethod
    def from_dict(d: dict, i: int) -> "RonupelLayer":
        where = f"layers[{i}]"
        _need(d, ("type", "mixer"), where)
        kind, m, mlp = d["type"], d["mixer"], d.get("mlp")
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{where}: mixer type {kind!r} is not implemented (known: {list(MIXER_TYPES)})")
        _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where + ".mixer")
        for k in ("heads", "kv_heads", "dim", "vdim"):
            if int(m[k]) <= 0:
                raise ConfigError(f"{where}.mixer.{k} must be positive, got {m[k]}")
        if int(m["heads"]) % int(m["kv_heads"]):
            raise ConfigError(f"{where}.mixer: {m['heads']} query heads do not split over {m['kv_heads']} key/value heads")
        if m.get("mask") is not None:
            _need(m["mask"], ("size",), where + ".mixer.mask")
            if int(m["mask"]["size"]) < 1 or int(m["mask"].get("keep_first", 0)) < 0:
                raise ConfigError(f"{where}.mixer.mask: a window of {m['mask']['size']} that keeps "
                                  f"{m['mask'].get('keep_first', 0)} first tokens")
        if m.get("rot") is not None:
            _need(m["rot"], ("base", "dims"), where + ".mixer.rot")
            dims = int(m["rot"]["dims"])
            if dims % 2 or not 0 <= dims <= int(m["dim"]) or not float(m["rot"]["base"]) > 0:
                raise ConfigError(f"{where}.mixer.rot: {dims} rotated dimensions of {m['dim']}, base {m['rot']['base']}")
            if m["rot"].get("scaling") is not None:
                _need(m["rot"]["scaling"], ("factor",), where + ".mixer.rot.scaling")
                if not float(m["rot"]["scaling"]["factor"]) > 0:
                    raise ConfigError(f"{where}.mixer.rot.scaling.factor must be positive")
        if mlp is not None:
            _need(mlp, ("kind",), where + ".mlp")
            if mlp["kind"] not in MLP_KINDS:
                raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r} is not implemented (known: {list(MLP_KINDS)})")
            _need(mlp, ("router", "expert"), where + ".mlp")
            _need(mlp["router"], ("experts", "top"), where + ".mlp.router")
            _need(mlp["expert"], ("ff", "limit"), where + ".mlp.expert")
            experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
            if not 1 <= top <= experts or int(mlp["expert"]["ff"]) <= 0:
                raise ConfigError(f"{where}.mlp: {top} of {experts} experts of {mlp['expert']['ff']}")
            if mlp.get("shared") is not None:
                _need(mlp["shared"], ("ff", "limit"), where + ".mlp.shared")
                if int(mlp["shared"]["ff"]) <= 0:
                    raise ConfigError(f"{where}.mlp.shared.ff must be positive, got {mlp['shared']['ff']}")
        return RonupelLayer(kind, dict(m), dict(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": dict(self.mixer), "mlp": dict(self.mlp) if self.mlp is not None else None}


@dataclass(frozen=True)
class RonupelConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: tuple                    # of RonupelLayer
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1              # layers loop_start .. loop_stop - 1 run this many times in a row
    architectures: tuple = ("Ronupel",)
    eos_token_id: tuple = ()
    extra: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, d: dict) -> "RonupelConfig":
        _need(d, ("vocab", "width", "norm", "layers"), "config.json")
        _need(d["norm"], ("eps",), "norm")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers must be a list with at least one entry")
        layers = tuple(RonupelLayer.from_dict(l, i) for i, l in enumerate(d["layers"]))
        start = stop = 0
        times = 1
        if d.get("loop") is not None:
            _need(d["loop"], ("start", "stop", "times"), "loop")
            start, stop, times = int(d["loop"]["start"]), int(d["loop"]["stop"]), int(d["loop"]["times"])
            if not (0 <= start <= stop <= len(layers)) or times < 1:
                raise ConfigError(f"loop: layers {start} .. {stop - 1} of {len(layers)}, {times} times")
        known = {"architecture", "architectures", "vocab", "width", "norm", "layers", "loop", "eos_token_id"}
        eos = d.get("eos_token_id")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=float(d["norm"]["eps"]), layers=layers,
                  loop_start=start, loop_stop=stop, loop_times=times,
                  eos_token_id=() if eos is None else tuple(int(t) for t in (eos if isinstance(eos, list) else [eos])),
                  extra={k: v for k, v in d.items() if k not in known})
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.norm_eps > 0:
            raise ConfigError(f"vocab {cfg.vocab}, width {cfg.width}, norm.eps {cfg.norm_eps}")
        return cfg

    @property
    def has_loop(self) -> bool:
        return self.loop_stop > self.loop_start and self.loop_times > 1

    def to_dict(self) -> dict:
        d = {"architecture": "Ronupel", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": [l.to_dict() for l in self.layers]}
        if self.loop_stop > self.loop_start:
            d["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d


__all__ = ["RonupelConfig", "RonupelLayer"]
