"""The Zodolorn configuration: config.json as it is, one entry per layer.

Zodolorn is a decoder whose layers are listed one by one.  Every entry names its mixer (``type``), the mixer's
sizes (``mixer``) and its feed-forward (``mlp``: ``kind`` "dense" or "moe", or null for none); ``norm.eps``,
``embedding.scale``, ``vocab`` and ``width`` are the model's own.  Nothing is derived: every size is read.
``max_positions`` is this library's bound on a sequence's length (the rotation table is that long); config.json
may carry it, otherwise the default holds.
"""

from __future__ import annotations

import dataclasses
from typing import List

from .base import ModelConfig

MIXERS = ("latent_attention",)
MLP_KINDS = ("dense", "moe")


@dataclasses.dataclass
class ZodolornConfig(ModelConfig):
    architecture: str = "Zodolorn"
    vocab: int = 512
    width: int = 128
    layers: List[dict] = dataclasses.field(default_factory=list)
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    embedding: dict = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    max_positions: int = 131072

    def __post_init__(self):
        self.validate()

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0:
            raise ValueError("vocab, width and max_positions must be positive")
        if "eps" not in self.norm or "scale" not in self.embedding:
            raise ValueError("the configuration needs norm.eps and embedding.scale")
        for i, layer in enumerate(self.layers):
            if layer.get("type") not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {layer.get('type')!r} is not one of {MIXERS}")
            m = layer.get("mixer") or {}
            for key in ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "rot"):
                if key not in m:
                    raise ValueError(f"layer {i}: the mixer lacks {key!r}")
            if m["rot"].get("dims") != m["rot_dim"]:
                raise ValueError(f"layer {i}: the rotation covers {m['rot'].get('dims')} dimensions, the rotated part has {m['rot_dim']}")
            src = m.get("kv_from")
            if src is not None:
                if not 0 <= src < i or self.layers[src]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from {src} must name an earlier layer that has keys and values of its own")
                other = self.layers[src]["mixer"]
                if (other["kv_rank"], other["rot_dim"], other["rot"]) != (m["kv_rank"], m["rot_dim"], m["rot"]):
                    raise ValueError(f"layer {i}: latent size and rotation must equal those of layer {src}, whose cache it reads")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") not in MLP_KINDS:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not one of {MLP_KINDS}")

    @property
    def nlayers(self) -> int:
        return len(self.layers)
