"""A plain, slow Defapel in PyTorch on the CPU: whole sequences, no cache, one function per mechanism.

It is the yardstick of the tests and shares nothing with the library.  Every function takes float32 (or float64)
tensors; `weights` maps the checkpoint's tensor names to tensors and `config` is the dictionary of config.json.

Notation: h is a mixer's or feed-forward's input [T, width]; p_t the position of token t, counted from 0;
S is a head's recurrent state [key channels, value channels].
"""

from __future__ import annotations

import json
import math
import os

import torch

# What a product's or an activation's result is stored as.  Identity for the exact run; a round trip through bfloat16
# for the run that shows what bfloat16 storage costs (what the design computes in 32-bit stays as it is).
_store = lambda x: x  # noqa: E731
# When a list: every mixture-of-experts layer appends, per token, by how much the last chosen expert's router logit
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


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    """The norm in front of a branch: the weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


# ---- rotation ---------------------------------------------------------------------------------------------------
def rotation_frequencies(rot):
    """f_i = base^(-2i/dims), then stretched by wavelength as `scaling` says (if any): short waves stay, long waves
    are slowed by `factor`, and between the two the frequency moves on a straight line in original/wavelength."""
    dims, base = rot["dims"], rot["base"]
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if sc:
            wave = 2.0 * math.pi / f
            if wave < sc["original"] / sc["high"]:
                pass
            elif wave > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            else:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


def rotate_pairs(x, positions, rot):
    """x [T, heads, D]: the first rot.dims entries of every head are rotated in adjacent pairs (2i, 2i+1) by the angle
    p * f_i; the rest pass."""
    dims = rot["dims"]
    angle = positions.to(torch.float32)[:, None] * rotation_frequencies(rot)[None, :]  # float32 angles
    cos, sin = torch.cos(angle.double()).to(x.dtype)[:, None, :], torch.sin(angle.double()).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---- softmax attention with a window (the left half of a parallel mixer) -------------------------------------------
def window_attention(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = _store(h @ w[p + "q"].T + w[p + "q.b"])
    k = _store(h @ w[p + "k"].T + w[p + "k.b"])
    v = _store(h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, Dv)
    # one norm over the whole projection, before the heads are cut
    q = _store(rms(q, eps) * w[p + "q.norm"]).view(T, H, D)
    k = _store(rms(k, eps) * w[p + "k.norm"]).view(T, G, D)
    q = _store(rotate_pairs(q, positions, m["rot"]))
    k = _store(rotate_pairs(k, positions, m["rot"]))
    cap, size = m["softcap"], m["mask"]["size"]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    i = positions[:, None]
    j = positions[None, :]
    visible = (i - j >= 0) & (i - j < size)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~visible, float("-inf"))
        out[:, head] = _store(torch.softmax(s, dim=-1)) @ v[:, g]
    mixed = _store(out.reshape(T, H * Dv))
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return _store(_store(mixed * gate) @ w[p + "o"].T)


# ---- the gated delta rule -------------------------------------------------------------------------------------------
def short_convolution(x, taps_w):
    """x [T, C], taps_w [C, taps]: y_t = sum_j taps_w[:, j] * x_{t - (taps - 1) + j}, zeros before the start; then silu."""
    T, C = x.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + padded[j : j + T] * taps_w[:, j]
    return y * torch.sigmoid(y)


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """q, k [T, H, D], v [T, H, Dv], beta [T, H], decay [T, H, D] (one factor per key channel; a decay per head is
    the same number D times).  Per head: S = decay * S; u = beta (v - S^T k); S = S + k u^T; o = S^T q."""
    T, H, D = q.shape
    Dv = v.shape[-1]
    S = torch.zeros(H, D, Dv, dtype=torch.float64)
    out = torch.zeros(T, H, Dv, dtype=torch.float64)
    q, k, v, beta, decay = (t.double() for t in (q, k, v, beta, decay))
    for t in range(T):
        S = S * decay[t][:, :, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + torch.einsum("hd,hv->hdv", k[t], u)
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out.float()


def gated_delta(h, w, p, m, eps, per_channel):
    """per_channel False: a decay per head from W_a, output gate silu(W_g h).  True: a decay per head and key channel
    from W_a2 W_a1, output gate sigmoid(W_g2 W_g1 h)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = _store(short_convolution(_store(h @ w[p + "q"].T), w[p + "q.conv"])).view(T, G, D)
    k = _store(short_convolution(_store(h @ w[p + "k"].T), w[p + "k.conv"])).view(T, G, D)
    v = _store(short_convolution(_store(h @ w[p + "v"].T), w[p + "v.conv"])).view(T, H, Dv)
    q = unit(q) * D ** -0.5
    k = unit(k)
    rep = H // G
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    if per_channel:
        a = (_store(h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).view(T, H, D)
        decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * torch.nn.functional.softplus(a))
        gate = torch.sigmoid(_store(h @ w[p + "g1"].T) @ w[p + "g2"].T)
    else:
        a = h @ w[p + "a"].T + w[p + "dt_bias"]
        decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :] * torch.nn.functional.softplus(a))[:, :, None].expand(T, H, D)
        z = h @ w[p + "g"].T
        gate = z * torch.sigmoid(z)
    o = delta_rule(q, k, v, beta, decay)
    o = rms(o, eps) * w[p + "norm"]
    o = _store(o.reshape(T, H * Dv) * gate)
    return _store(o @ w[p + "o"].T)


# ---- feed-forward ----------------------------------------------------------------------------------------------------
def experts(h, w, p, mlp):
    """Every token's `top` experts by sigmoid score; the score scales the expert's input."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[p + "router"].T
    scores = torch.sigmoid(z)
    best, ids = torch.topk(scores, top, dim=-1)
    if router_margins is not None:
        rest = z.scatter(1, ids, float("-inf")).max(dim=-1).values if top < E else torch.full((h.shape[0],), float("-inf"))
        router_margins.append(z.gather(1, ids).min(dim=-1).values - rest)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for s, e in zip(best[t], ids[t]):
            x = _store(s * h[t])
            e = int(e)
            a = _store(x @ w[f"{p}e{e}.gate"].T)
            b = _store(x @ w[f"{p}e{e}.up"].T)
            out[t] += _store(a * torch.sigmoid(a) * b) @ w[f"{p}e{e}.down"].T
    return _store(out)


# ---- the model -------------------------------------------------------------------------------------------------------
def mixer(h, w, p, layer, eps, positions):
    m = layer["mixer"]
    if layer["type"] == "channel_delta":
        return gated_delta(h, w, p, m, eps, per_channel=True)
    if layer["type"] == "parallel":
        left = window_attention(h, w, p + "left.", m["left"], eps, positions)
        right = gated_delta(h, w, p + "right.", m["right"], eps, per_channel=False)
        return _store(m["left_scale"] * left + m["right_scale"] * right)
    raise ValueError(layer["type"])


def forward(config, w, tokens, rounding=None, return_layers=False):
    """Logits [T, vocab] of one whole sequence.  rounding "bfloat16": products and activations are stored in bfloat16."""
    global _store
    _store = _bf16 if rounding == "bfloat16" else (lambda x: x)
    try:
        eps = config["norm"]["eps"]
        ids = torch.as_tensor(tokens, dtype=torch.long)
        positions = torch.arange(len(ids))
        x = w["embed"][ids].clone()
        layers = []
        for i, layer in enumerate(config["layers"]):
            p = f"l{i}."
            x = x + mixer(_store(layer_norm(x, w[p + "norm1"], eps)), w, p + "mix.", layer, eps, positions)
            if layer.get("mlp") is not None:
                x = x + experts(_store(layer_norm(x, w[p + "norm2"], eps)), w, p + "mlp.", layer["mlp"])
            layers.append(x.clone())
        logits = _store(layer_norm(x, w["final.norm"], eps)) @ w["embed"].T * config["logit_scale"]
        return (logits, torch.stack(layers)) if return_layers else logits
    finally:
        _store = lambda x: x  # noqa: E731


def greedy_generate(config, w, prompt, n_new):
    """The n_new tokens that greedy decoding appends to `prompt` (the whole sequence is run again for every token)."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(config, w, ids)[-1])))
    return ids[len(prompt):]
