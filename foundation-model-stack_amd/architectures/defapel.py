"""Defapel: from its configuration to parts, and from its checkpoint's tensor names to the model's.

The model: a token embedding; layers in the order config.json lists them, each a pre-norm block whose RMS norms store
their scale around zero; the mixer is either softmax attention over a sliding window (biased projections, one RMS norm
over the whole query and key projections, rotation of a part of each head with stretched frequencies, capped scores, a
sigmoid gate on the output) beside a gated delta rule, the two summed with fixed scales, or a gated delta rule whose
decay has a factor per key channel; the feed-forward is a mixture of gated experts chosen and weighted by sigmoid scores,
the weight on the expert's input; a final norm and a head that is the embedding table times a constant.

A checkpoint names a layer's tensors ``l<i>.<part>`` without a ".weight"; the adapter gives them the model's names and
fuses what the model runs as one product (everything that reads a mixer's input; the experts stacked per layer).
"""

from __future__ import annotations

import re
from typing import List, Tuple

import torch

from ..config import DefapelConfig
from ..parts import LayerSpec, ModelSpec, PartSpec
from ..weights.adapters import register_adapter, register_adapter_step
from .registry import Architecture, register_architecture, register_model

NAME = "defapel"
# what the design fixes: the experts' activation is silu(gate) * up, g * sigmoid(ALPHA * g) * (u + SHIFT) without a clamp
EXPERT_ALPHA = 1.0
EXPERT_SHIFT = 0.0
NORM_WEIGHT_OFFSET = 1.0  # the block norms and the final norm store their scale minus one


def _rope_key(rot: dict) -> str:
    sc = rot.get("scaling") or {}
    return f"rope_{rot['dims']}_{rot['base']!r}_" + "_".join(f"{k}{sc[k]!r}" for k in sorted(sc))


def _rope_spec(rot: dict, head_dim: int, max_positions: int) -> PartSpec:
    args = {"dim": head_dim, "rot_dim": rot["dims"], "theta": rot["base"], "max_seq_len": max_positions, "exact_frequencies": True}
    sc = rot.get("scaling")
    if sc:
        args["scaling"] = {"rope_type": "llama3", "factor": sc["factor"], "low_freq_factor": sc["low"],
                           "high_freq_factor": sc["high"], "original_max_position_embeddings": sc["original"]}
    return PartSpec("rope", args)


def _delta_args(m: dict, eps: float, per_channel: bool) -> dict:
    args = {"heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"], "vdim": m["vdim"], "conv": m["conv"], "eps": eps}
    if per_channel:
        for key in ("decay_rank", "gate_rank"):
            if not m.get(key):
                raise ValueError(f"a channel_delta mixer needs {key!r}: a model folder's tensor shapes give it, a configuration "
                                 "made without one must carry it")
        args.update(decay_rank=m["decay_rank"], gate_rank=m["gate_rank"], gate_activation="sigmoid")
    else:
        args.update(gate_activation="silu")
    return args


def _attention_args(m: dict, eps: float) -> dict:
    return {"nheads": m["heads"], "kvheads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "qkv_bias": True,
            "out_bias": False, "qk_norm": "projection", "norm_eps": eps, "output_gate": True, "scale_factor": m["scale"],
            "window": m["mask"]["size"], "soft_cap": m["softcap"]}


def defapel_spec(config: DefapelConfig) -> ModelSpec:
    eps = config.norm["eps"]
    norm = PartSpec("rmsnorm", {"eps": eps, "weight_offset": NORM_WEIGHT_OFFSET})
    layers, positions = [], {}
    for layer in config.layers:
        m = layer["mixer"]
        key = None
        if layer["type"] == "parallel":
            left = m["left"]
            key = _rope_key(left["rot"]) + f"_{left['dim']}"
            positions.setdefault(key, _rope_spec(left["rot"], left["dim"], config.max_positions))
            mixer = PartSpec("parallel", {
                "left": {"kind": "attention", "positional": True, "args": _attention_args(left, eps)},
                "right": {"kind": "gated_delta", "args": _delta_args(m["right"], eps, per_channel=False)},
                "left_scale": m["left_scale"], "right_scale": m["right_scale"],
            })
        else:
            mixer = PartSpec("gated_delta", _delta_args(m, eps, per_channel=True))
        mlp = layer.get("mlp")
        ff = None
        if mlp is not None:
            ff = PartSpec("experts", {"experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "hidden_dim": mlp["expert"]["ff"],
                                      "limit": None, "alpha": EXPERT_ALPHA, "shift": EXPERT_SHIFT, "score": "sigmoid", "weight_on": "input"})
        block = PartSpec("pre_norm", {"names": ("norm1", "mix", "norm2", "mlp")})
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, block=block, position=key))
    return ModelSpec(
        vocab=config.vocab, width=config.width, max_seq_len=config.max_positions, layers=layers, final_norm=norm,
        head=PartSpec("linear", {"scale": config.logit_scale}), positions=positions, tie_heads=True,
        embedding_name="embed", layer_name="l{i}", final_norm_name="final.norm", head_name="head",
    )


# ---- the checkpoint's names -> the model's ----------------------------------------------------------------------
_EXPERT = re.compile(r"^(l\d+\.mlp)\.e(\d+)\.(gate|up|down)$")


def _fuse_delta(out: dict, p: str) -> None:
    """The tensors of a gated delta rule under prefix p (which ends in a dot), in place."""
    low_rank = p + "a1" in out
    rows = [out.pop(p + n) for n in ("q", "k", "v", "b")]
    rows.append(out.pop(p + ("a1" if low_rank else "a")))
    rows.append(out.pop(p + ("g1" if low_rank else "g")))
    out[p + "in_proj.weight"] = torch.cat(rows, dim=0)
    out[p + "conv.weight"] = torch.cat([out.pop(p + n + ".conv") for n in ("q", "k", "v")], dim=0)
    if low_rank:
        out[p + "decay_up.weight"] = out.pop(p + "a2")
        out[p + "gate_up.weight"] = out.pop(p + "g2")
    out[p + "norm.weight"] = out.pop(p + "norm")
    out[p + "out.weight"] = out.pop(p + "o")


def _fuse_attention(out: dict, p: str) -> None:
    """The tensors of the windowed attention under prefix p, in place: queries, keys, values and the gate's rows are
    one projection (the gate has no bias: zeros)."""
    parts = [out.pop(p + n) for n in ("q", "k", "v", "g")]
    biases = [out.pop(p + n + ".b") for n in ("q", "k", "v")]
    biases.append(torch.zeros(parts[3].shape[0], dtype=biases[0].dtype))
    out[p + "in_proj.qkv_fused.weight"] = torch.cat(parts, dim=0)
    out[p + "in_proj.qkv_fused.bias"] = torch.cat(biases, dim=0)
    out[p + "q_norm.weight"] = out.pop(p + "q.norm")
    out[p + "k_norm.weight"] = out.pop(p + "k.norm")
    out[p + "dense.weight"] = out.pop(p + "o")


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
    for name in [n for n in out if n.endswith(".A_log")]:
        _fuse_delta(out, name[: -len("A_log")])
    for name in [n for n in out if n.endswith(".mix.left.q")]:
        _fuse_attention(out, name[: -len("q")])
    renamed = {}
    for name, t in out.items():
        if re.search(r"(^embed|^final\.norm|\.norm[12]|\.mlp\.router)$", name):
            name += ".weight"
        renamed[name] = t
    return renamed


register_adapter_step(NAME, "checkpoint_to_model_names", _to_model_names)
register_adapter(NAME, "hf", ["checkpoint_to_model_names"])


def detect_source(names: List[str]) -> str:
    return "fms" if any(n.endswith(".in_proj.weight") for n in names) else "hf"


def _delta_layout(p: str, m: dict, W: int, per_channel: bool) -> list:
    H, G, D, V, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    out = [(p + "q", (G * D, W), "normal"), (p + "q.conv", (G * D, taps), "normal"), (p + "k", (G * D, W), "normal"),
           (p + "k.conv", (G * D, taps), "normal"), (p + "v", (H * V, W), "normal"), (p + "v.conv", (H * V, taps), "normal"),
           (p + "b", (H, W), "normal"), (p + "A_log", (H,), "zeros"), (p + "norm", (V,), "ones")]
    if per_channel:
        out += [(p + "a1", (m["decay_rank"], W), "normal"), (p + "a2", (H * D, m["decay_rank"]), "normal"), (p + "dt_bias", (H * D,), "zeros"),
                (p + "g1", (m["gate_rank"], W), "normal"), (p + "g2", (H * V, m["gate_rank"]), "normal")]
    else:
        out += [(p + "a", (H, W), "normal"), (p + "dt_bias", (H,), "zeros"), (p + "g", (H * V, W), "normal")]
    return out + [(p + "o", (W, H * V), "normal")]


def checkpoint_tensor_layout(config: DefapelConfig) -> List[Tuple[str, Tuple[int, ...], str]]:
    """(name, shape, init) of every tensor of a Defapel checkpoint of this configuration."""
    W = config.width
    out = [("embed", (config.vocab, W), "normal")]
    for i, layer in enumerate(config.layers):
        p, m = f"l{i}.", layer["mixer"]
        out.append((p + "norm1", (W,), "zeros"))
        if layer["type"] == "parallel":
            a = m["left"]
            H, G, D, V = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            out += [(q + "q", (H * D, W), "normal"), (q + "q.b", (H * D,), "zeros"), (q + "k", (G * D, W), "normal"), (q + "k.b", (G * D,), "zeros"),
                    (q + "v", (G * V, W), "normal"), (q + "v.b", (G * V,), "zeros"), (q + "q.norm", (H * D,), "ones"), (q + "k.norm", (G * D,), "ones"),
                    (q + "g", (H * V, W), "normal"), (q + "o", (W, H * V), "normal")]
            out += _delta_layout(p + "mix.right.", m["right"], W, per_channel=False)
        else:
            out += _delta_layout(p + "mix.", m, W, per_channel=True)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out.append((p + "norm2", (W,), "zeros"))
        F = mlp["expert"]["ff"]
        for e in range(mlp["router"]["experts"]):
            out += [(p + f"mlp.e{e}.gate", (F, W), "normal"), (p + f"mlp.e{e}.up", (F, W), "normal"), (p + f"mlp.e{e}.down", (W, F), "normal")]
        out.append((p + "mlp.router", (mlp["router"]["experts"], W), "normal"))
    out.append(("final.norm", (W,), "zeros"))
    return out


register_architecture(
    Architecture(
        name=NAME,
        config_class=DefapelConfig,
        build_spec=defapel_spec,
        hf_architectures=(),
        from_hf_dict=DefapelConfig.from_dict,
        to_hf_dict=lambda config: config.as_dict(),
        hf_tensor_layout=checkpoint_tensor_layout,
        detect_source=detect_source,
        sizes_from_tensors=lambda config, shapes: config.with_sizes_from_tensors(shapes),
    )
)


def make_config(width: int, vocab: int, pattern: str, heads: int, kv_heads: int, dim: int, vdim: int, window: int, delta_heads: int,
                delta_kv_heads: int, delta_dim: int, delta_vdim: int, experts: int, top: int, expert_ff: int, conv: int = 4,
                rot_dims: int = 0, rot_base: float = 500000.0, rot_scaling: dict = None, softcap: float = 30.0, rank: int = 0,
                left_scale: float = 1.0, right_scale: float = 1.0, logit_scale: float = 1.0, max_positions: int = 131072) -> DefapelConfig:
    """A regular Defapel: `pattern` has a letter per layer, "p" for a parallel mixer and "c" for a channel_delta one; all
    layers of a kind share their sizes."""
    layers = []
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff}} if experts else None
    for letter in pattern:
        if letter == "p":
            rot = {"base": rot_base, "dims": rot_dims or dim}
            if rot_scaling:
                rot["scaling"] = dict(rot_scaling)
            mixer = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "rot": rot,
                              "scale": dim ** -0.5, "softcap": softcap},
                     "right": {"heads": delta_heads, "kv_heads": delta_kv_heads, "dim": delta_dim, "vdim": delta_vdim, "conv": conv},
                     "left_scale": left_scale, "right_scale": right_scale}
            layers.append({"type": "parallel", "mixer": mixer, "mlp": mlp})
        elif letter == "c":
            r = rank or max(8, width // 16)
            mixer = {"heads": delta_heads, "kv_heads": delta_kv_heads, "dim": delta_dim, "vdim": delta_vdim, "conv": conv,
                     "decay_rank": r, "gate_rank": r}
            layers.append({"type": "channel_delta", "mixer": mixer, "mlp": mlp})
        else:
            raise ValueError(f"layer letter {letter!r} is not 'p' or 'c'")
    return DefapelConfig(vocab=vocab, width=width, layers=layers, norm={"eps": 1e-6}, logit_scale=logit_scale, max_positions=max_positions)


def _variant(config: DefapelConfig):
    def factory(**overrides) -> DefapelConfig:
        return config.updated(**overrides)

    return factory


register_model(NAME, "micro", _variant(make_config(width=256, vocab=1024, pattern="ppcp", heads=4, kv_heads=2, dim=64, vdim=64, window=128,
                                                   delta_heads=4, delta_kv_heads=2, delta_dim=32, delta_vdim=64, experts=8, top=2,
                                                   expert_ff=128, max_positions=4096)))
register_model(NAME, "3b-a1b", _variant(make_config(width=2048, vocab=65536, pattern="pppc" * 6, heads=16, kv_heads=4, dim=128, vdim=128,
                                                    window=1024, delta_heads=16, delta_kv_heads=8, delta_dim=128, delta_vdim=128,
                                                    experts=32, top=4, expert_ff=1024,
                                                    rot_scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192})))
