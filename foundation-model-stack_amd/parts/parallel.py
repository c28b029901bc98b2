"""Two mixers side by side: both read the same input, and the layer's mixer output is
left_scale * left(h) + right_scale * right(h).

Each side ends in a projection back to the model's width.  The two projections run as one product over the two sides'
inputs laid next to each other, each already times its scale (the kernel that writes a side's last activation applies
it in float32, before the one rounding), so the weighted sum costs no kernel and no rounding of its own.  The sides keep
what they need of the cache: at most one of them keys and values in pages, and each its fixed-size state, whose tensors
carry the side's name.
"""

from __future__ import annotations

import torch

from ..cache import StateNeed
from .base import BranchOutput, Mixer, make_part, register_part
from .linear import Linear


class ParallelMixers(Mixer):
    def __init__(self, width: int, left: dict, right: dict, left_scale: float = 1.0, right_scale: float = 1.0, position_encoder=None):
        """left, right: {"kind": a registered mixer, "args": its arguments}.  The position encoding goes to the sides that
        say `"positional": True`."""
        super().__init__()
        self.width = width
        self.scales = (float(left_scale), float(right_scale))
        self.sides = []
        for name, spec in (("left", left), ("right", right)):
            pos = position_encoder if spec.get("positional") else None
            side = make_part("mixer", spec["kind"], width=width, position_encoder=pos, **spec.get("args", {}))
            if not hasattr(side, "forward_branch"):
                raise TypeError(f"mixer {spec['kind']!r} cannot run beside another: it has no forward_branch")
            side.state_prefix = name + "."
            self.sides.append(self.add_child(name, side))
        if sum(side.kv_need() is not None for side in self.sides) > 1:
            raise ValueError("at most one of two parallel mixers can keep keys and values in the cache")
        self._joint: Linear = None
        self._widths = None

    def kv_need(self):
        for side in self.sides:
            if side.kv_need() is not None:
                return side.kv_need()
        return None

    def state_need(self):
        tensors = []
        for side in self.sides:
            need = side.state_need()
            if need is not None:
                tensors += [(side.state_prefix + name, shape, dt) for name, shape, dt in need.tensors]
        return StateNeed(tuple(tensors)) if tensors else None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(side, "graph_safe", True) for side in self.sides)

    def check_step(self, max_position: int) -> None:
        for side in self.sides:
            side.check_step(max_position)

    def prefill_qblock(self, n_tokens: int, dtype) -> int:
        return max(side.prefill_qblock(n_tokens, dtype) for side in self.sides)

    def finalize(self, device, dtype) -> None:
        # the sides' output projections as one weight [width, K_left + K_right]; the sides' own tensors become views of it
        outs = [side.output_projection() for side in self.sides]
        if any(o.has_bias for o in outs):
            raise NotImplementedError("parallel mixers join output projections without biases")
        self._widths = [o.in_features for o in outs]
        joint = torch.cat([o.w["weight"] for o in outs], dim=1).contiguous()
        self._joint = Linear(sum(self._widths), self.width)
        self._joint.w["weight"] = joint
        at = 0
        for o in outs:
            o.w["weight"] = joint[:, at : at + o.in_features]
            at += o.in_features

    def forward(self, x: torch.Tensor, batch, cache) -> torch.Tensor:
        return self.forward_branch(x, batch, cache).value()

    def forward_branch(self, x: torch.Tensor, batch, cache) -> BranchOutput:
        both = torch.empty(x.shape[0], sum(self._widths), dtype=x.dtype, device=x.device)
        if batch.is_decode:
            both.zero_()  # a decode step may hold padding rows, which nobody writes and the joint product reads
        at = 0
        for side, scale, k in zip(self.sides, self.scales, self._widths):
            side.forward_branch(x, batch, cache, out=both[:, at : at + k], out_scale=scale)
            at += k
        return BranchOutput(both, self._joint)


register_part("mixer", "parallel", ParallelMixers)
