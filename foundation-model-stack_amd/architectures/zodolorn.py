"""Zodolorn: from its configuration to parts, and from its checkpoint's tensor names to the model's.

The model: a token embedding times a constant; layers in the order config.json lists them, each a block whose
branches are RMS-normed on both sides; the mixer is attention over a latent cache with a sink and an output gate,
and a layer may read the latent that an earlier layer cached; the feed-forward is a plain gelu one, a mixture of
clamped gated experts with a gated shared expert, or absent; a final RMS norm and a linear head.

A checkpoint names a layer's tensors ``l<i>.<part>`` without a ".weight"; the adapter gives them the model's names
and fuses what the model runs as one product (everything that reads a mixer's input; router and shared gate; the
experts stacked per layer).
"""

from __future__ import annotations

import re
from typing import List, Tuple

import torch

from ..config import ZodolornConfig
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..weights.adapters import register_adapter, register_adapter_step
from .registry import Architecture, register_architecture, register_model

NAME = "zodolorn"
# constants of the experts' activation that the design fixes: g * sigmoid(ALPHA * g) * (u + SHIFT)
EXPERT_ALPHA = 1.702
EXPERT_SHIFT = 1.0


def _rope_key(rot: dict) -> str:
    return f"rope_{rot['dims']}_{rot['base']!r}"


def _experts_args(mlp: dict) -> dict:
    shared = mlp.get("shared") or {}
    return {
        "experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "hidden_dim": mlp["expert"]["ff"],
        "limit": mlp["expert"]["limit"], "alpha": EXPERT_ALPHA, "shift": EXPERT_SHIFT,
        "shared_hidden_dim": shared.get("ff", 0), "shared_limit": shared.get("limit"), "shared_gate": bool(shared),
    }


def zodolorn_spec(config: ZodolornConfig) -> ModelSpec:
    eps = config.norm["eps"]
    norm = PartSpec("rmsnorm", {"eps": eps})
    layers, positions, schedule = [], {}, []
    for i, layer in enumerate(config.layers):
        m = layer["mixer"]
        key = _rope_key(m["rot"])
        positions.setdefault(key, PartSpec("rope", {"dim": m["rot"]["dims"], "theta": m["rot"]["base"], "max_seq_len": config.max_positions,
                                                    "exact_frequencies": True}))
        mixer = PartSpec("latent_attention", {
            "nheads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"], "q_rank": m["q_rank"],
            "kv_rank": m["kv_rank"], "scale": m["scale"], "eps": eps, "sink": True, "output_gate": True,
            "owns_kv": m.get("kv_from") is None,
        })
        mlp = layer.get("mlp")
        if mlp is None:
            ff = None
        elif mlp["kind"] == "dense":
            ff = PartSpec("mlp", {"hidden_dim": mlp["ff"], "activation": "gelu"})
        else:
            ff = PartSpec("experts", _experts_args(mlp))
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, block=PartSpec("sandwich_norm"), position=key))
        schedule.append(ScheduleEntry(i, cache_of=m.get("kv_from")))
    return ModelSpec(
        vocab=config.vocab, width=config.width, max_seq_len=config.max_positions, layers=layers, final_norm=norm,
        embedding=PartSpec("table", {"scale": config.embedding["scale"]}), positions=positions, schedule=schedule,
        embedding_name="embed", layer_name="l{i}", final_norm_name="final.norm", head_name="head",
    )


# ---- the checkpoint's names -> the model's ----------------------------------------------------------------------
_EXPERT = re.compile(r"^(l\d+\.mlp)\.e(\d+)\.(gate|up|down)$")


def _to_model_names(sd, **kw):
    out, experts = {}, {}
    for name, t in sd.items():
        m = _EXPERT.match(name)
        if m:
            experts.setdefault((m.group(1), m.group(3)), {})[int(m.group(2))] = t
            continue
        out[name] = t
    for (prefix, which), by_index in experts.items():
        out[f"{prefix}.experts.{which}"] = torch.stack([by_index[i] for i in sorted(by_index)], dim=0)
    prefixes = sorted({n[: -len(".mix.dq")] for n in out if n.endswith(".mix.dq")})
    for p in prefixes:
        pieces = [out.pop(f"{p}.mix.dq")]
        for part in ("g", "dkv"):
            if f"{p}.mix.{part}" in out:
                pieces.append(out.pop(f"{p}.mix.{part}"))
        out[f"{p}.mix.down.weight"] = torch.cat(pieces, dim=0)
        for src, dst in (("dq.norm", "q_norm.weight"), ("dkv.norm", "kv_norm.weight"), ("uq", "uq.weight"), ("uk", "uk.weight"),
                         ("uv", "uv.weight"), ("o", "o.weight")):
            if f"{p}.mix.{src}" in out:
                out[f"{p}.mix.{dst}"] = out.pop(f"{p}.mix.{src}")
    for p in sorted({n[: -len(".mlp.router")] for n in out if n.endswith(".mlp.router")}):
        rows = [out.pop(f"{p}.mlp.router")]
        if f"{p}.mlp.shared.sg" in out:
            rows.append(out.pop(f"{p}.mlp.shared.sg"))
        out[f"{p}.mlp.router.weight"] = torch.cat(rows, dim=0)
        if f"{p}.mlp.shared.gate" in out:
            out[f"{p}.mlp.shared.gate_up.weight"] = torch.cat([out.pop(f"{p}.mlp.shared.gate"), out.pop(f"{p}.mlp.shared.up")], dim=0)
            out[f"{p}.mlp.shared.down.weight"] = out.pop(f"{p}.mlp.shared.down")
    renamed = {}
    for name, t in out.items():
        if re.search(r"(^embed|^head|^final\.norm|\.norm[12]b?|\.mlp\.(up|down))$", name):
            name += ".weight"
        renamed[name] = t
    return renamed


register_adapter_step(NAME, "checkpoint_to_model_names", _to_model_names)
register_adapter(NAME, "hf", ["checkpoint_to_model_names"])


def detect_source(names: List[str]) -> str:
    return "fms" if any(n.endswith(".mix.down.weight") for n in names) else "hf"


def checkpoint_tensor_layout(config: ZodolornConfig) -> List[Tuple[str, Tuple[int, ...], str]]:
    """(name, shape, init) of every tensor of a Zodolorn checkpoint of this configuration."""
    W = config.width
    out = [("embed", (config.vocab, W), "normal")]
    for i, layer in enumerate(config.layers):
        p, m = f"l{i}.", layer["mixer"]
        H, D, P, V, Q, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
        out += [(p + n, (W,), "ones") for n in ("norm1", "norm1b")]
        out += [(p + "mix.dq", (Q, W), "normal"), (p + "mix.dq.norm", (Q,), "ones"), (p + "mix.uq", (H * (D + P), Q), "normal")]
        if m.get("kv_from") is None:
            out += [(p + "mix.dkv", (R + P, W), "normal"), (p + "mix.dkv.norm", (R,), "ones")]
        out += [(p + "mix.uk", (H * D, R), "normal"), (p + "mix.uv", (H * V, R), "normal"), (p + "mix.sink", (H,), "normal"),
                (p + "mix.g", (H, W), "normal"), (p + "mix.o", (W, H * V), "normal")]
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out += [(p + n, (W,), "ones") for n in ("norm2", "norm2b")]
        if mlp["kind"] == "dense":
            out += [(p + "mlp.up", (mlp["ff"], W), "normal"), (p + "mlp.down", (W, mlp["ff"]), "normal")]
            continue
        F = mlp["expert"]["ff"]
        for e in range(mlp["router"]["experts"]):
            out += [(p + f"mlp.e{e}.gate", (F, W), "normal"), (p + f"mlp.e{e}.up", (F, W), "normal"), (p + f"mlp.e{e}.down", (W, F), "normal")]
        out.append((p + "mlp.router", (mlp["router"]["experts"], W), "normal"))
        if mlp.get("shared"):
            S = mlp["shared"]["ff"]
            out += [(p + "mlp.shared.gate", (S, W), "normal"), (p + "mlp.shared.up", (S, W), "normal"), (p + "mlp.shared.down", (W, S), "normal"),
                    (p + "mlp.shared.sg", (1, W), "normal")]
    out += [("final.norm", (W,), "ones"), ("head", (config.vocab, W), "normal")]
    return out


register_architecture(
    Architecture(
        name=NAME,
        config_class=ZodolornConfig,
        build_spec=zodolorn_spec,
        hf_architectures=(),
        from_hf_dict=ZodolornConfig.from_dict,
        to_hf_dict=lambda config: config.as_dict(),
        hf_tensor_layout=checkpoint_tensor_layout,
        detect_source=detect_source,
    )
)


def make_config(width: int, vocab: int, nlayers: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int,
                dense_ff: int, experts: int = 0, top: int = 0, expert_ff: int = 0, shared_ff: int = 0, share_every: int = 2,
                rot_base: float = 10000.0, max_positions: int = 131072) -> ZodolornConfig:
    """A regular Zodolorn: layers alternate between one that caches its own latent with a plain feed-forward and one
    that reads its predecessor's latent with experts (every `share_every`-th layer; 0: no sharing, no experts)."""
    layers = []
    for i in range(nlayers):
        shares = share_every > 0 and i % share_every == share_every - 1
        mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                 "scale": (dim + rot_dim) ** -0.5, "rot": {"base": rot_base, "dims": rot_dim}}
        if shares:
            mixer["kv_from"] = i - 1
        if shares and experts:
            mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff, "limit": 7.0}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff, "limit": 7.0}
        else:
            mlp = {"kind": "dense", "ff": dense_ff}
        layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    return ZodolornConfig(vocab=vocab, width=width, layers=layers, norm={"eps": 1e-6}, embedding={"scale": width ** 0.5},
                          max_positions=max_positions)


def _variant(config: ZodolornConfig):
    def factory(**overrides) -> ZodolornConfig:
        return config.updated(**overrides)

    return factory


register_model(NAME, "micro", _variant(make_config(width=256, vocab=1024, nlayers=4, heads=4, dim=32, rot_dim=16, vdim=32, q_rank=96,
                                                   kv_rank=64, dense_ff=512, experts=8, top=2, expert_ff=128, shared_ff=128,
                                                   max_positions=4096)))
register_model(NAME, "4b-a1b", _variant(make_config(width=2048, vocab=65536, nlayers=24, heads=16, dim=128, rot_dim=64, vdim=128, q_rank=768,
                                                    kv_rank=512, dense_ff=8192, experts=32, top=4, expert_ff=1024, shared_ff=2048)))
