"""The Defapel configuration: config.json as it is, one entry per layer.

Defapel is a decoder whose layers are listed one by one.  Every entry names its mixer (``type``: "parallel", softmax
attention with a window beside a gated delta rule, or "channel_delta", a gated delta rule with a decay per key channel),
the mixer's sizes (``mixer``) and its feed-forward (``mlp``: a mixture of experts, or null for none); ``norm.eps``,
``logit_scale``, ``vocab`` and ``width`` are the model's own.  Two sizes of a "channel_delta" mixer are not in
config.json but in the shapes of its tensors: the ranks of the low-rank pairs behind its decay and its gate.  A model
folder's tensor shapes fill them in (``decay_rank``, ``gate_rank`` in the mixer's entry); a configuration made without
a folder carries them itself.  ``max_positions`` is this library's bound on a sequence's length (the rotation table is
that long); config.json may carry it, otherwise the default holds.
"""

from __future__ import annotations

import copy
import dataclasses
from typing import Dict, List, Tuple

from .base import ModelConfig

LAYER_TYPES = ("parallel", "channel_delta")
_DELTA_KEYS = ("heads", "kv_heads", "dim", "vdim", "conv")
_ATTENTION_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "softcap", "mask", "rot")


@dataclasses.dataclass
class DefapelConfig(ModelConfig):
    architecture: str = "Defapel"
    vocab: int = 512
    width: int = 128
    layers: List[dict] = dataclasses.field(default_factory=list)
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    logit_scale: float = 1.0
    max_positions: int = 131072

    def __post_init__(self):
        self.validate()

    @staticmethod
    def _check_delta(i: int, m: dict, what: str) -> None:
        for key in _DELTA_KEYS:
            if key not in m:
                raise ValueError(f"layer {i}: the {what} lacks {key!r}")
        if m["heads"] <= 0 or m["kv_heads"] <= 0 or m["heads"] % m["kv_heads"]:
            raise ValueError(f"layer {i}: {m['heads']} heads are no multiple of {m['kv_heads']} query/key heads")

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0:
            raise ValueError("vocab, width and max_positions must be positive")
        if "eps" not in self.norm:
            raise ValueError("the configuration needs norm.eps")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type")
            if kind not in LAYER_TYPES:
                raise ValueError(f"layer {i}: mixer type {kind!r} is not one of {LAYER_TYPES}")
            m = layer.get("mixer") or {}
            if kind == "channel_delta":
                self._check_delta(i, m, "mixer")
            else:
                for side in ("left", "right", "left_scale", "right_scale"):
                    if side not in m:
                        raise ValueError(f"layer {i}: the mixer lacks {side!r}")
                for key in _ATTENTION_KEYS:
                    if key not in m["left"]:
                        raise ValueError(f"layer {i}: the left mixer lacks {key!r}")
                left = m["left"]
                if left["heads"] <= 0 or left["kv_heads"] <= 0 or left["heads"] % left["kv_heads"]:
                    raise ValueError(f"layer {i}: {left['heads']} query heads are no multiple of {left['kv_heads']} key/value heads")
                rot = left["rot"]
                if "dims" not in rot or "base" not in rot or rot["dims"] % 2 or not 0 < rot["dims"] <= left["dim"]:
                    raise ValueError(f"layer {i}: the rotation needs a base and an even number of dimensions within the head's {left['dim']}")
                if left["mask"].get("size", 0) <= 0:
                    raise ValueError(f"layer {i}: the window needs a positive mask.size")
                self._check_delta(i, m["right"], "right mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not 'moe'")
                router = mlp.get("router") or {}
                if "ff" not in (mlp.get("expert") or {}) or not 0 < router.get("top", 0) <= router.get("experts", 0):
                    raise ValueError(f"layer {i}: the experts need expert.ff, and router.top within router.experts")

    @property
    def nlayers(self) -> int:
        return len(self.layers)

    def with_sizes_from_tensors(self, shapes: Dict[str, Tuple[int, ...]]) -> "DefapelConfig":
        """The configuration with the sizes that only the checkpoint's tensor shapes give: the ranks of the low-rank
        pairs of every "channel_delta" mixer (`l<i>.mix.a1` is [decay_rank, width], `l<i>.mix.g1` [gate_rank, width])."""
        layers = copy.deepcopy(self.layers)
        for i, layer in enumerate(layers):
            if layer.get("type") != "channel_delta":
                continue
            for tensor, key in (("a1", "decay_rank"), ("g1", "gate_rank")):
                shape = shapes.get(f"l{i}.mix.{tensor}")
                if shape is not None:
                    layer["mixer"][key] = int(shape[0])
        return self.updated(layers=layers)
