"""A plain, slow Zodolorn in PyTorch on the CPU: whole sequences, no cache, one function per mechanism.

It is the yardstick of the tests and shares nothing with the library.  Every function takes float32 (or float64)
tensors; `weights` maps the checkpoint's tensor names to tensors and `config` is the dictionary of config.json.

Notation: h is a mixer's or feed-forward's input [T, width]; p_t the position of token t, counted from 0.
"""

from __future__ import annotations

import json
import math
import os

import torch

# What a product's or an activation's result is stored as.  Identity for the exact run; a round trip through bfloat16
# for the run that shows what bfloat16 storage costs (scores, softmax, norms' statistics, the router and the residual
# sum stay as they are: the design computes them in 32-bit).
_store = lambda x: x  # noqa: E731
# When a list: every mixture-of-experts layer appends, per token, by how much the last chosen expert's logit
# exceeds the best logit not chosen (inf when all experts are chosen).  A small number marks a choice that rounding
# can turn: such a token's logits are no test of arithmetic.
router_margins = None


def _bf16(x):
    return x.to(torch.bfloat16).to(x.dtype)


def load_model_folder(folder):
    """(config dictionary, name -> float32 tensor) of a folder with config.json and model.safetensors."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    weights = {k: (v.float() if v.is_floating_point() else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, weights


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_pairs(x, positions, base, dims):
    """x [T, ..., D]: the first `dims` entries of the last axis are rotated in adjacent pairs (2i, 2i+1) by the
    angle p * base^(-2i/dims); the rest pass."""
    half = dims // 2
    freqs = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64).to(torch.float32)
    angle = positions.to(torch.float32)[:, None] * freqs[None, :]  # float32 angles, as a float32 model forms them
    cos, sin = torch.cos(angle.double()).to(x.dtype), torch.sin(angle.double()).to(x.dtype)
    while cos.dim() < x.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_kv(h, w, prefix, m, eps, positions):
    """The two things a latent-attention layer leaves for its keys and values: the normed latent [T, kv_rank] and
    the rotated key part that all heads share [T, rot_dim]."""
    r, rd = m["kv_rank"], m["rot_dim"]
    down = h @ w[prefix + "dkv"].T
    latent = _store(rms_norm(down[:, :r], w[prefix + "dkv.norm"], eps))
    shared = _store(rotate_pairs(down[:, r : r + rd], positions, m["rot"]["base"], m["rot"]["dims"]))
    return latent, shared


def latent_attention(h, w, prefix, m, eps, positions, latent, shared):
    """Causal attention whose keys and values are projections of `latent`, with a sink in the softmax's denominator
    and a gate per head on the output."""
    T = h.shape[0]
    H, d, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = _store(rms_norm(h @ w[prefix + "dq"].T, w[prefix + "dq.norm"], eps))
    q = _store(cq @ w[prefix + "uq"].T).view(T, H, d + rd)
    q_plain = q[:, :, :d]
    q_rot = _store(rotate_pairs(q[:, :, d:], positions, m["rot"]["base"], m["rot"]["dims"]))
    k_plain = _store(latent @ w[prefix + "uk"].T).view(T, H, d)
    value = _store(latent @ w[prefix + "uv"].T).view(T, H, dv)
    score = (torch.einsum("thd,shd->hts", q_plain, k_plain) + torch.einsum("thd,sd->hts", q_rot, shared)) * m["scale"]
    visible = positions[None, :] <= positions[:, None]  # [t, s]
    score = score.masked_fill(~visible[None], float("-inf"))
    sink = w[prefix + "sink"].to(score.dtype)
    top = torch.maximum(score.max(-1).values, sink[:, None])  # [H, T]
    e = torch.exp(score - top[..., None])
    denom = e.sum(-1) + torch.exp(sink[:, None] - top)
    prob = e / denom[..., None]
    mixed = torch.einsum("hts,shd->thd", prob, value)
    gate = torch.sigmoid(h @ w[prefix + "g"].T)  # [T, H]
    mixed = _store(mixed * gate[:, :, None])
    return _store(mixed.reshape(T, H * dv) @ w[prefix + "o"].T)


def dense_ff(h, w, prefix):
    z = _store(h @ w[prefix + "up"].T)
    z = _store(0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0))))
    return _store(z @ w[prefix + "down"].T)


def clamped_expert(h, w, prefix, limit):
    g = torch.clamp(h @ w[prefix + "gate"].T, max=limit)
    u = torch.clamp(h @ w[prefix + "up"].T, min=-limit, max=limit)
    return _store(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[prefix + "down"].T


def moe_ff(h, w, prefix, mlp):
    n, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = h.float() @ w[prefix + "router"].float().T
    chosen = torch.topk(logits, top, dim=-1)
    if router_margins is not None:
        ranked = torch.sort(logits, dim=-1, descending=True).values
        router_margins.append(ranked[:, top - 1] - ranked[:, top] if top < n else torch.full((h.shape[0],), float("inf")))
    share = torch.softmax(chosen.values, dim=-1).to(h.dtype)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen.indices[t, j])
            out[t] += share[t, j] * clamped_expert(h[t : t + 1], w, f"{prefix}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        s = _store(clamped_expert(h, w, prefix + "shared.", mlp["shared"]["limit"]))
        out = out + s * torch.sigmoid(h @ w[prefix + "shared.sg"].T)
    return _store(out)


def forward(config, weights, tokens, dtype=torch.float32, return_layers=False, storage=None, margins=None):
    """Logits [T, vocab] of one whole sequence; with return_layers also the stream after every layer.
    storage=torch.bfloat16: results of products and activations are rounded to bfloat16 where a bfloat16 model
    stores them."""
    global _store, router_margins
    _store = _bf16 if storage == torch.bfloat16 else (lambda x: x)
    router_margins = margins  # a list to be filled, or None
    try:
        return _forward(config, weights, tokens, dtype, return_layers)
    finally:
        _store = lambda x: x  # noqa: E731
        router_margins = None


def _forward(config, weights, tokens, dtype, return_layers):
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = w["embed"][ids] * config["embedding"]["scale"]
    kept = {}
    after = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = _store(rms_norm(x, w[p + "norm1"], eps))
        if layer["type"] != "latent_attention":
            raise ValueError(layer["type"])
        if m.get("kv_from") is None:
            kept[i] = latent_kv(h, w, p + "mix.", m, eps, positions)
            latent, shared = kept[i]
        else:
            latent, shared = kept[m["kv_from"]]
        y = latent_attention(h, w, p + "mix.", m, eps, positions, latent, shared)
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = _store(rms_norm(x, w[p + "norm2"], eps))
            y = dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, w, p + "mlp.", mlp)
            x = x + rms_norm(y, w[p + "norm2b"], eps)
        after.append(x)
    logits = _store(rms_norm(x, w["final.norm"], eps)) @ w["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy_generate(config, weights, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(config, weights, ids)[-1].argmax()))
    return ids[len(prompt):]
