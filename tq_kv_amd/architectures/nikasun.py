"""Nikasun: a decoder whose configuration lists its layers one by one (attention through cached latents
with a window and an output gate, some layers reading an earlier layer's cache; dense or routed
feed-forwards, or none).

Which config.json keys the architecture reads and how they become a ModelSpec is
csrc/engine/nikasun.cpp's; this is the typed configuration as Python sees it.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.registry import config_class, spec_from_dict


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: Optional[int]
    kv_from: Optional[int]

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
             "kv_rank": self.kv_rank, "scale": self.scale}
        if self.rot_dim:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class NikasunLayer:
    type: str
    mixer: LatentMixer
    mlp: Optional[dict]         # None, {"kind": "dense", "ff"}, or {"kind": "moe", "experts", "top", "router_scale", "expert", "shared"}

    def mlp_dict(self):
        m = self.mlp
        if m is None:
            return None
        if m["kind"] == "dense":
            return {"kind": "dense", "ff": m["ff"]}
        d = {"kind": "moe", "router": {"experts": m["experts"], "top": m["top"], "scale": m["router_scale"]}, "expert": dict(m["expert"])}
        if m.get("shared"):
            d["shared"] = dict(m["shared"])
        return d


@config_class("Nikasun")
@dataclass(frozen=True)
class NikasunConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    max_positions: int
    layers: Tuple[NikasunLayer, ...]

    @classmethod
    def from_typed(cls, typed):
        """From what the engine library made of a config.json (every key, defaults filled in)."""
        layers = tuple(NikasunLayer(l["type"], LatentMixer(**l["mixer"]), l["mlp"]) for l in typed["layers"])
        return cls(typed["vocab"], typed["width"], typed["embedding_scale"], typed["norm_eps"], typed["max_positions"], layers)

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        from ..config.registry import config_from_dict
        return config_from_dict(dict(raw, architecture="Nikasun"), where)[1]

    def to_typed(self):
        return {"vocab": self.vocab, "width": self.width, "embedding_scale": self.embedding_scale, "norm_eps": self.norm_eps,
                "max_positions": self.max_positions,
                "layers": [{"type": l.type, "mixer": dict(l.mixer.__dict__), "mlp": l.mlp} for l in self.layers]}

    def to_dict(self):
        """The config.json that reads back as this configuration."""
        return {"architecture": "Nikasun", "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions,
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(), "mlp": l.mlp_dict()} for l in self.layers]}


def build_spec(cfg: NikasunConfig):
    return spec_from_dict(cfg.to_dict())
