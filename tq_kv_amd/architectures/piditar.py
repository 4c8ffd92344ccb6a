"""Piditar: a decoder whose configuration lists its layers one by one, each a pre-norm block around one of three mixers
(grouped-query attention with biases, pair rotation and heads normed after it; the recurrent block with a real-gated linear
recurrent unit; the selective state-space mixer with a scalar decay per head) and an optional dense feed-forward.  A span of
the layers may run several times with the same weights, every pass with a cache and state of its own and the embedding's
output added in front of every pass after the first.

Which config.json keys the architecture reads and how they become a ModelSpec is
csrc/engine/piditar.cpp's; this is the typed configuration as Python sees it.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.registry import config_class, spec_from_dict


@dataclass(frozen=True)
class PiditarLayer:
    type: str                   # "attention", "rglru" or "mamba2"
    mixer: dict                 # attention: heads, kv_heads, dim, vdim, scale, softcap, rot_base, rot_dims; rglru: width, blocks, conv;
                                # mamba2: heads, vdim, state, groups, conv, norm_groups
    mlp: Optional[dict]         # None or {"kind": "dense", "ff"}

    def mixer_dict(self):
        m = dict(self.mixer)
        if self.type == "attention":
            m["rot"] = {"base": m.pop("rot_base"), "dims": m.pop("rot_dims")}
            if m.get("softcap") is None:
                m.pop("softcap", None)
        return m

    def __hash__(self):
        return hash((self.type, tuple(sorted(self.mixer.items())), None if self.mlp is None else tuple(sorted(self.mlp.items()))))


@config_class("Piditar")
@dataclass(frozen=True)
class PiditarConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    max_positions: int
    layers: Tuple[PiditarLayer, ...]
    loop_start: int
    loop_stop: int
    loop_times: int

    @classmethod
    def from_typed(cls, typed):
        """From what the engine library made of a config.json (every key, defaults filled in)."""
        layers = tuple(PiditarLayer(l["type"], dict(l["mixer"]), l["mlp"]) for l in typed["layers"])
        return cls(typed["vocab"], typed["width"], typed["embedding_scale"], typed["norm_eps"], typed["max_positions"], layers,
                   typed["loop_start"], typed["loop_stop"], typed["loop_times"])

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        from ..config.registry import config_from_dict
        return config_from_dict(dict(raw, architecture="Piditar"), where)[1]

    def to_typed(self):
        return {"vocab": self.vocab, "width": self.width, "embedding_scale": self.embedding_scale, "norm_eps": self.norm_eps,
                "max_positions": self.max_positions, "layers": [{"type": l.type, "mixer": dict(l.mixer), "mlp": l.mlp} for l in self.layers],
                "loop_start": self.loop_start, "loop_stop": self.loop_stop, "loop_times": self.loop_times}

    def run_order(self):
        """The layers in the order they run: those before the span, the span `loop_times` times, the rest."""
        span = list(range(self.loop_start, self.loop_stop))
        return list(range(self.loop_start)) + span * self.loop_times + list(range(self.loop_stop, len(self.layers)))

    def to_dict(self):
        """The config.json that reads back as this configuration."""
        return {"architecture": "Piditar", "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions,
                "layers": [{"type": l.type, "mixer": l.mixer_dict(), "mlp": l.mlp} for l in self.layers],
                "loop": {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}}


def build_spec(cfg: PiditarConfig):
    return spec_from_dict(cfg.to_dict())
