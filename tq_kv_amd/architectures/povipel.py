"""Povipel: a decoder whose configuration lists its layers one by one.  The residual stream is kept in several copies that every
sublayer reads as a weighted sum and updates all at once; a sublayer is a layer norm and then the part, and what a mixer reads is
first mixed with the previous token's.  Mixers: "parallel" (attention over a window plus pooled blocks, with normed heads, values
turned by their position and a sink, beside a gated linear attention with a decay per key channel; the two outputs normed, added and
halved) and "retention" (linear attention with a fixed decay per head).  Feed-forwards: dense, or routed experts scored by a sigmoid
each with the weight on the expert's input.  A span of the layers may run several times with the same weights, every pass with a
cache and state of its own.

Which config.json keys the architecture reads and how they become a ModelSpec is csrc/engine/povipel.cpp's; this is the typed
configuration as Python sees it.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.registry import config_class, spec_from_dict


def _rot_out(m):
    m = dict(m)
    m["rot"] = {"base": m.pop("rot_base"), "dims": m.pop("rot_dims")}
    return m


def _freeze(v):
    if isinstance(v, dict):
        return tuple(sorted((k, _freeze(x)) for k, x in v.items()))
    if isinstance(v, list):
        return tuple(_freeze(x) for x in v)
    return v


@dataclass(frozen=True)
class PovipelLayer:
    type: str                   # "parallel" or "retention"
    mixer: dict                 # parallel: left {heads, kv_heads, dim, vdim, scale, window, pool, rot_base, rot_dims}, right {heads, dim, vdim, tau};
                                # retention: heads, dim, vdim, decay, rot_base, rot_dims
    mlp: Optional[dict]         # None, {"kind": "dense", "ff"} or {"kind": "moe", "ff", "experts", "top"}

    def mixer_dict(self):
        """The mixer as config.json writes it."""
        if self.type == "retention":
            return _rot_out(self.mixer)
        left = _rot_out(self.mixer["left"])
        left["mask"] = {"size": left.pop("window"), "pool": left.pop("pool")}
        return {"left": left, "right": dict(self.mixer["right"])}

    def mlp_dict(self):
        if self.mlp is None or self.mlp["kind"] == "dense":
            return self.mlp
        return {"kind": "moe", "expert": {"ff": self.mlp["ff"]}, "router": {"experts": self.mlp["experts"], "top": self.mlp["top"]}}

    def __hash__(self):
        return hash((self.type, _freeze(self.mixer), _freeze(self.mlp)))


@config_class("Povipel")
@dataclass(frozen=True)
class PovipelConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    streams: Optional[int]
    logit_softcap: Optional[float]
    max_positions: int
    layers: Tuple[PovipelLayer, ...]
    loop_start: int
    loop_stop: int
    loop_times: int

    @classmethod
    def from_typed(cls, typed):
        """From what the engine library made of a config.json (every key, defaults filled in)."""
        layers = tuple(PovipelLayer(l["type"], dict(l["mixer"]), l["mlp"]) for l in typed["layers"])
        return cls(typed["vocab"], typed["width"], typed["embedding_scale"], typed["norm_eps"], typed["streams"], typed["logit_softcap"],
                   typed["max_positions"], layers, typed["loop_start"], typed["loop_stop"], typed["loop_times"])

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        from ..config.registry import config_from_dict
        return config_from_dict(dict(raw, architecture="Povipel"), where)[1]

    def run_order(self):
        """The layers in the order they run: those before the span, the span `loop_times` times, the rest."""
        span = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + span * self.loop_times + list(range(self.loop_stop, len(self.layers)))

    def to_dict(self):
        """The config.json that reads back as this configuration."""
        d = {"architecture": "Povipel", "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
             "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions,
             "layers": [{"type": l.type, "mixer": l.mixer_dict(), "mlp": l.mlp_dict()} for l in self.layers],
             "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}}
        if self.streams is not None:
            d["streams"] = self.streams
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        return d


def build_spec(cfg: PovipelConfig):
    return spec_from_dict(cfg.to_dict())
