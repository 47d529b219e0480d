"""Sizudra: a decoder whose configuration lists its layers one by one (an embedding of hashed token pairs beside the
token embedding; norms on the parts' outputs only; grouped-query attention with normed heads, values of their own
size and values mixed across layers, in one kind of layer with a score cap, a window that keeps the first positions
and a sink; dense feed-forwards, routed experts without a gate product, or none).

Which config.json keys the architecture reads and how they become a ModelSpec is
csrc/engine/sizudra.cpp's; this is the typed configuration as Python sees it.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.registry import config_class, spec_from_dict


@dataclass(frozen=True)
class SizudraMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int
    v_mix: bool
    softcap: Optional[float]
    window: Optional[int]
    keep_first: int

    def to_dict(self, second):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.v_mix:
            d["v_mix"] = True
        if second:
            d["softcap"] = self.softcap
            d["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return d


@dataclass(frozen=True)
class SizudraLayer:
    type: str                   # "attention" or "attention_2"
    mixer: SizudraMixer
    mlp: Optional[dict]         # None, {"kind": "dense", "ff"}, or {"kind": "moe", "experts", "top", "expert_ff", "shared_ff"}

    def mlp_dict(self):
        m = self.mlp
        if m is None:
            return None
        if m["kind"] == "dense":
            return {"kind": "dense", "ff": m["ff"]}
        d = {"kind": "moe", "router": {"experts": m["experts"], "top": m["top"]}, "expert": {"ff": m["expert_ff"]}}
        if m.get("shared_ff") is not None:
            d["shared"] = {"ff": m["shared_ff"]}
        return d


@config_class("Sizudra")
@dataclass(frozen=True)
class SizudraConfig:
    vocab: int
    width: int
    bigram_buckets: int
    bigram_mul_prev: int
    bigram_mul_cur: int
    norm_eps: float
    max_positions: int
    layers: Tuple[SizudraLayer, ...]

    @classmethod
    def from_typed(cls, typed):
        """From what the engine library made of a config.json (every key, defaults filled in)."""
        layers = tuple(SizudraLayer(l["type"], SizudraMixer(**l["mixer"]), l["mlp"]) for l in typed["layers"])
        return cls(typed["vocab"], typed["width"], typed["bigram_buckets"], typed["bigram_mul_prev"], typed["bigram_mul_cur"],
                   typed["norm_eps"], typed["max_positions"], layers)

    @classmethod
    def from_dict(cls, raw, where="config.json"):
        from ..config.registry import config_from_dict
        return config_from_dict(dict(raw, architecture="Sizudra"), where)[1]

    def to_typed(self):
        return {"vocab": self.vocab, "width": self.width, "bigram_buckets": self.bigram_buckets, "bigram_mul_prev": self.bigram_mul_prev,
                "bigram_mul_cur": self.bigram_mul_cur, "norm_eps": self.norm_eps, "max_positions": self.max_positions,
                "layers": [{"type": l.type, "mixer": dict(l.mixer.__dict__), "mlp": l.mlp} for l in self.layers]}

    def to_dict(self):
        """The config.json that reads back as this configuration."""
        return {"architecture": "Sizudra", "vocab": self.vocab, "width": self.width,
                "embedding": {"bigram": {"buckets": self.bigram_buckets, "mul_prev": self.bigram_mul_prev, "mul_cur": self.bigram_mul_cur}},
                "norm": {"eps": self.norm_eps}, "max_positions": self.max_positions,
                "layers": [{"type": l.type, "mixer": l.mixer.to_dict(l.type == "attention_2"), "mlp": l.mlp_dict()} for l in self.layers]}


def build_spec(cfg: SizudraConfig):
    return spec_from_dict(cfg.to_dict())
