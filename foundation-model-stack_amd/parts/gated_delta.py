"""The gated delta rule: a recurrent mixer whose memory is one matrix per head instead of a cache of keys and values.

For every token, with q and k unit vectors of `dim` channels (q also times dim^-1/2) and v of `vdim` channels, each of
them the silu of a short causal convolution over time of a projection of the mixer's input h:

    S <- g * S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

beta = sigmoid(W_b h) per head; g = exp(-exp(A_log) softplus(a + dt_bias)) is a decay per head (a = W_a h) or, with
`decay_rank`, per head and key channel through a low-rank pair (a = W_a2 W_a1 h), scaling the rows of S.  Every head's
o is divided by its root mean square, times a weight shared by the heads, times a gate act(W_g h) (or act(W_g2 W_g1 h)
with `gate_rank`), and projected back to the model's width.  Query/key head h // (heads / kv_heads) serves head h.

What a sequence carries from token to token is S (float32) and the last `conv - 1` inputs of the convolution; both
are fixed-size state of the sequence's slot, so whole prompts, portions of prompts and single tokens run the same
kernels and differ by rounding only.  Everything behind the projections is float32.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import BranchOutput, Mixer, register_part
from .linear import Linear


class GatedDeltaRule(Mixer):
    def __init__(
        self,
        width: int,
        heads: int,
        kv_heads: int,
        dim: int,
        vdim: int,
        conv: int = 4,
        eps: float = 1e-6,
        decay_rank: int = 0,  # 0: one decay per head; r > 0: one per head and key channel, through r numbers
        gate_rank: int = 0,  # 0: the gate is a full projection; r > 0: through r numbers
        gate_activation: str = "silu",
        position_encoder=None,  # takes none: the recurrence knows the order of its tokens
    ):
        super().__init__()
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads:
            raise ValueError(f"{heads} heads are no multiple of {kv_heads} query/key heads")
        if not 1 <= conv <= ops.DELTA_MAX_TAPS:
            raise ValueError(f"a convolution of {conv} taps (1 to {ops.DELTA_MAX_TAPS})")
        if dim <= 0 or dim > ops.DELTA_MAX_DIM or vdim <= 0:
            raise ValueError(f"{dim} key channels (1 to {ops.DELTA_MAX_DIM}) and {vdim} value channels")
        if gate_activation not in ops.ACTIVATIONS:
            raise ValueError(f"gate activation {gate_activation!r} is not one of {sorted(ops.ACTIVATIONS)}")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.taps, self.eps = int(conv), float(eps)
        self.decay_rank, self.gate_rank, self.gate_activation = int(decay_rank), int(gate_rank), gate_activation
        self.per_channel = self.decay_rank > 0
        self.channels = 2 * kv_heads * dim + heads * vdim  # what passes the convolution: q | k | v
        # one product for everything that reads the mixer's input: [q | k | v | beta | decay (or its low rank) | gate (or its low rank)]
        self.col_b = self.channels
        self.col_a = self.col_b + heads
        self.col_g = self.col_a + (self.decay_rank or heads)
        self.in_proj = self.add_child("in_proj", Linear(width, self.col_g + (self.gate_rank or heads * vdim)))
        self.declare("conv.weight", (self.channels, self.taps))
        self.declare("A_log", (heads,), init="zeros", kind="scale")
        self.declare("dt_bias", (heads * dim if self.per_channel else heads,), init="zeros", kind="scale")
        self.declare("norm.weight", (vdim,), init="ones", kind="scale")
        if self.decay_rank:
            self.decay_up = self.add_child("decay_up", Linear(self.decay_rank, heads * dim))
        if self.gate_rank:
            self.gate_up = self.add_child("gate_up", Linear(self.gate_rank, heads * vdim))
        self.out = self.add_child("out", Linear(heads * vdim, width))
        self._a_log = self._dt_bias = None

    def unfused_parameters(self) -> dict:
        """The fused input projection as the tensors it is made of, in the order of its rows."""
        H, G, D, V = self.heads, self.kv_heads, self.dim, self.vdim
        pieces = [("q", G * D), ("k", G * D), ("v", H * V), ("b", H), ("a1" if self.decay_rank else "a", self.decay_rank or H),
                  ("g1" if self.gate_rank else "g", self.gate_rank or H * V)]
        return {"in_proj": tuple(pieces)}

    def state_need(self) -> StateNeed:
        return StateNeed((
            ("S", (self.heads, self.vdim, self.dim), "float32"),  # transposed: a value channel's key channels lie together
            ("conv", (max(self.taps - 1, 1), self.channels), "float32"),
        ))

    def output_projection(self) -> Linear:
        return self.out

    def finalize(self, device, dtype) -> None:
        self._a_log = self.w["A_log"].to(torch.float32).contiguous()
        self._dt_bias = self.w["dt_bias"].to(torch.float32).contiguous()

    def forward(self, x: torch.Tensor, batch, cache) -> torch.Tensor:
        return self.forward_branch(x, batch, cache).value()

    def forward_branch(self, x: torch.Tensor, batch, cache, out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> BranchOutput:
        """out (rows [T, heads*vdim] of any stride) and out_scale: where the input of the output projection is written, and
        a factor on it, for a caller that runs this mixer beside another and projects both at once."""
        H, G, D, V = self.heads, self.kv_heads, self.dim, self.vdim
        state = prefixed_state(cache.state, getattr(self, "state_prefix", ""))
        # decays, gates, unit vectors and the recurrence are formed from the float32 sums of this product
        proj = self.in_proj.forward(x, out_dtype=torch.float32)
        if self.decay_rank:
            low = ops.cast_cols(proj, self.col_a, self.decay_rank, x.dtype)
            a, col_a = self.decay_up.forward(low, out_dtype=torch.float32), 0
        else:
            a, col_a = proj, self.col_a
        if self.gate_rank:
            low = ops.cast_cols(proj, self.col_g, self.gate_rank, x.dtype)
            gate = self.gate_up.forward(low, out_dtype=torch.float32)
        else:
            gate = proj[:, self.col_g : self.col_g + H * V]
        qkv, beta, decay, kq = ops.delta_prepare(proj, self.col_b, a, col_a, self.w["conv.weight"], self._a_log, self._dt_bias,
                                             state["conv"], batch.seq_of_token, batch.slot_ids, H, G, D, V, self.per_channel, D ** -0.5)
        o = ops.delta_rule(qkv, beta, decay, kq, state["S"], batch.seq_starts, batch.seq_of_token, batch.slot_ids, batch.n_seqs, H, G, D, V,
                           self.per_channel, single_tokens=batch.is_decode)
        normed = ops.gated_head_norm(o, gate, self.w["norm.weight"], self.eps, self.gate_activation, H, V, x.dtype, batch.seq_of_token,
                                     scale=out_scale, out=out)
        return BranchOutput(normed, self.out)


def prefixed_state(state: dict, prefix: str) -> dict:
    """The tensors of a slot's state whose names start with `prefix`, under their names without it."""
    if not prefix:
        return state
    return {name[len(prefix):]: t for name, t in state.items() if name.startswith(prefix)}


register_part("mixer", "gated_delta", GatedDeltaRule)
