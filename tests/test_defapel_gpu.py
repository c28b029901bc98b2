"""Defapel on the GPU against the plain implementation (plain_defapel.py): every mechanism alone, then the engine
whole / token by token / in portions / in ragged batches with reused slots / through graphs and the generation loop,
in float32 and bfloat16, at sizes that differ from one another in everything.

bfloat16 is judged like the other models of this folder: the plain implementation run with bfloat16 storage shows what
that type costs at every position, and the engine may be a small multiple of that off."""

import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_defapel as P  # noqa: E402
from gpu_checks import Expected  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
BF16_MARGIN = 3.0
BF16_MEAN_MARGIN = 1.5
# A router's choice is "close" when the last chosen logit leads the first one not chosen by less than this: bfloat16
# rounding can turn it, the token then runs other experts, and its logits are no test of arithmetic.
CLOSE_CALL = 0.25


def attention(heads, kv, dim, vdim, window, rot_dims, base=10000.0, scaling=None, scale=0.2, softcap=15.0):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": {"size": window}, "rot": rot, "scale": scale, "softcap": softcap}


def delta(heads, kv, dim, vdim, conv, ranks=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}
    if ranks:
        m["decay_rank"], m["gate_rank"] = ranks
    return m


def moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def parallel(left, right, ls, rs, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def channel(m, mlp):
    return {"type": "channel_delta", "mixer": m, "mlp": mlp}


CONFIGS = {
    # values of another size than keys, grouped heads on both sides, a part of every head rotated, a layer without a
    # feed-forward, experts of which all are chosen, stretched frequencies, convolutions of 2, 3 and 4 taps
    "A": dict(vocab=300, width=128, norm={"eps": 1e-5}, logit_scale=1.5, max_positions=1024, layers=[
        parallel(attention(4, 2, 32, 24, 40, 16), delta(4, 2, 16, 24, 3), 0.7, 1.1, moe(6, 2, 48)),
        channel(delta(2, 1, 40, 20, 4, ranks=(12, 20)), None),
        parallel(attention(2, 1, 64, 48, 70, 64, base=1000.0, scaling=(4.0, 1.0, 2.0, 32)), delta(3, 1, 24, 40, 2), 1.3, 0.5, moe(4, 4, 40)),
        channel(delta(4, 4, 8, 16, 4, ranks=(8, 8)), moe(5, 3, 24)),
    ]),
    # sizes that are no multiples of 8 (rows that the matrix instructions cannot load), a window of five tokens, one
    # expert a token, a convolution of one tap (no state of its own) and one of five
    "B": dict(vocab=257, width=100, norm={"eps": 1e-6}, logit_scale=0.6, max_positions=1024, layers=[
        channel(delta(3, 3, 20, 12, 1, ranks=(6, 10)), moe(5, 1, 36)),
        parallel(attention(3, 3, 20, 20, 5, 4, base=500.0), delta(2, 2, 12, 36, 5), 1.0, 1.0, moe(3, 2, 20)),
    ]),
    # sizes at which bfloat16 runs the matrix-instruction products; 128 key channels a head; a window of two pages
    "C": dict(vocab=512, width=256, norm={"eps": 1e-6}, logit_scale=1.0, max_positions=2048, layers=[
        parallel(attention(8, 2, 64, 64, 128, 32, base=500000.0, scaling=(8.0, 1.0, 4.0, 64)), delta(4, 2, 128, 64, 4), 0.9, 0.8, moe(8, 2, 128)),
        channel(delta(4, 4, 64, 128, 4, ranks=(16, 16)), moe(8, 2, 128)),
    ]),
    # the other head sizes with matrix-instruction attention kernels of their own: 128 and 32; 256 key channels a head
    "D": dict(vocab=400, width=256, norm={"eps": 1e-6}, logit_scale=2.5, max_positions=2048, layers=[
        parallel(attention(4, 2, 128, 128, 100, 64, base=50000.0, softcap=25.0), delta(2, 1, 256, 32, 4), 1.0, 0.6, moe(4, 1, 64)),
        parallel(attention(8, 8, 32, 32, 64, 32, softcap=10.0), delta(8, 8, 32, 32, 4), 0.5, 1.0, None),
        # a head size between 64 and 128: capped scores of prompts run the generic kernel, single tokens the matrix-core one
        parallel(attention(2, 2, 96, 96, 50, 32, softcap=12.0), delta(1, 1, 16, 16, 3), 1.0, 1.0, moe(4, 2, 32)),
    ]),
    # no attention at all: the cache has no pages to keep, only state
    "E": dict(vocab=200, width=64, norm={"eps": 1e-6}, logit_scale=1.0, max_positions=512, layers=[
        channel(delta(2, 2, 32, 16, 4, ranks=(8, 4)), moe(4, 2, 32)),
        channel(delta(4, 1, 16, 8, 2, ranks=(4, 8)), None),
    ]),
}


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd
    from fms_amd.kernels import load

    load()
    return fms_amd


def write_folder(lib, folder, cfg_kw, seed, sharp=1.0):
    """A model folder with random weights: norm weights around zero, decays of every speed, biases.

    The experts' weights are not renormalized, so a router's choice that rounding turns moves a token's stream by much,
    and through the mixers every later token's: no comparison in bfloat16 would survive it.  The routers of these
    folders therefore decide by the token alone, and clearly: the stream's first channels (one per expert) hold, for
    every token, a permutation of numbers half a unit apart; no branch writes into those channels; expert e's router row
    reads channel e only.  (The router against arbitrary logits is tested by itself.)"""
    from fms_amd.weights import write_safetensors

    lib.write_model_folder(folder, lib.DefapelConfig(**cfg_kw), seed=seed, architecture="defapel", std=0.08)
    cfg, tensors = P.load_model_folder(folder)
    gen = torch.Generator().manual_seed(seed)

    def noise(t, std):
        return torch.randn(t.shape, generator=gen) * std

    for k in list(tensors):
        t = tensors[k]
        if k.endswith((".norm1", ".norm2")) or k == "final.norm":
            tensors[k] = noise(t, 0.2)
        elif k.endswith((".q.norm", ".k.norm", ".mix.norm", ".right.norm")):
            tensors[k] = 1 + noise(t, 0.2)
        elif k.endswith((".q.b", ".k.b", ".v.b")):
            tensors[k] = noise(t, 0.3)
        elif k.endswith(".A_log"):
            tensors[k] = noise(t, 1.0) - 1.0
        elif k.endswith(".dt_bias"):
            tensors[k] = noise(t, 1.0)
        elif k.endswith(".conv"):
            tensors[k] = noise(t, 0.5)
        elif k.endswith((".mix.b", ".right.b", ".left.g")):
            tensors[k] = t * 4  # gates and betas away from one half
    n_route = max([layer["mlp"]["router"]["experts"] for layer in cfg["layers"] if layer.get("mlp")] + [0])
    levels = (torch.arange(n_route) - (n_route - 1) / 2) * 0.5  # half a unit apart, whatever the number of experts
    tensors["embed"][:, :n_route] = torch.stack([levels[torch.randperm(n_route, generator=gen)] for _ in range(cfg["vocab"])])
    for k in list(tensors):
        if k.endswith((".mix.o", ".left.o", ".right.o", ".down")):
            tensors[k][:n_route] = 0
        elif k.endswith(".norm2"):
            tensors[k][:n_route] = 0
        elif k.endswith(".mlp.router"):
            tensors[k] = 1.5 * torch.eye(tensors[k].shape[0], tensors[k].shape[1])
    if sharp != 1.0:
        for k in tensors:
            if k.endswith(".left.q.norm"):  # the queries are normed, so their size is their norm weight's
                tensors[k] = tensors[k] * sharp
    tensors = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory, lib):
    return {name: write_folder(lib, str(tmp_path_factory.mktemp(f"defapel_{name}")), kw, 3 + i) for i, (name, kw) in enumerate(CONFIGS.items())}


_models, _plain, _expected = {}, {}, {}


def get(lib, folders, name, dtype):
    if (name, dtype) not in _models:
        _models[(name, dtype)] = lib.get_model("hf_pretrained", model_path=folders[name], data_type=dtype)
    return _models[(name, dtype)]


def plain(folders, name):
    if name not in _plain:
        _plain[name] = P.load_model_folder(folders[name])
    return _plain[name]


def tokens_for(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def expect(cfg, weights, ids, dtype) -> Expected:
    """Exact logits; for bfloat16 also the plain implementation's own error with bfloat16 storage, set to infinity at
    the positions where a router's choice is close (they are not compared), and its 90th percentile over the rest."""
    P.router_margins = []
    try:
        exact = P.forward(cfg, weights, ids)
        margins = P.router_margins
    finally:
        P.router_margins = None
    if dtype == "float32":
        return Expected(exact)
    rounded = P.forward(cfg, weights, ids, rounding="bfloat16")
    error = (rounded - exact).abs().amax(dim=-1)
    close = torch.zeros(len(ids), dtype=torch.bool)
    for gap in margins:
        close |= gap < CLOSE_CALL
    assert len(ids) < 32 or float(close.float().mean()) < 0.1, "many positions have close router calls: the test would compare little"
    typical = torch.quantile(error[~close], 0.9).expand_as(error)
    return Expected(exact, torch.where(close, torch.full_like(error, float("inf")), error), typical)


def expected_for(folders, name, n, seed, dtype):
    key = (name, n, seed, dtype)
    if key not in _expected:
        cfg, weights = plain(folders, name)
        ids = tokens_for(cfg["vocab"], n, seed)
        _expected[key] = (ids, expect(cfg, weights, ids, dtype))
    return _expected[key]


def judge(got, want, dtype):
    got = got.float().cpu()
    assert got.shape == want.shape, f"{tuple(got.shape)} logits, {tuple(want.shape)} expected"
    if dtype == "float32":
        torch.testing.assert_close(got, want.logits, atol=3e-4, rtol=1e-3)
        return
    error = (got - want.logits).abs().amax(dim=-1).flatten()
    ref, typical = want.ref_error.flatten(), want.typical.flatten()
    compared = torch.isfinite(ref)
    allowed = BF16_MARGIN * torch.maximum(ref, typical)
    worst = int(torch.argmax(torch.where(compared, error / allowed, torch.zeros_like(error))))
    assert bool((error[compared] <= allowed[compared]).all()), (
        f"bfloat16 logits are {float(error[worst]):.4g} off at row {worst}; the plain implementation with bfloat16 storage is "
        f"{float(ref[worst]):.4g} off there and typically {float(typical[worst]):.4g} (allowed: {BF16_MARGIN} times the larger)")
    if int(compared.sum()) >= 32:
        assert float(error[compared].mean()) <= BF16_MEAN_MARGIN * float(ref[compared].mean()), (
            f"bfloat16 logits are {float(error[compared].mean()):.4g} off on average, the plain implementation with bfloat16 "
            f"storage {float(ref[compared].mean()):.4g}")


# ---- mechanisms alone ------------------------------------------------------------------------------------------
def _delta_inputs(T, H, G, D, V, per_channel, seed):
    gen = torch.Generator().manual_seed(seed)
    C = 2 * G * D + H * V
    per = D if per_channel else 1
    proj = torch.randn(T, C + H + 3, generator=gen)  # three columns that nobody reads behind the betas
    a = torch.randn(T, H * per + 2, generator=gen)
    return proj, a, C


def _plain_delta(proj, a, conv_w, a_log, dt_bias, H, G, D, V, per_channel, C):
    """Everything between the projections and the head norm, from the plain implementation's functions."""
    T = proj.shape[0]
    y = P.short_convolution(proj[:, :C], conv_w)
    q = (P.unit(y[:, : G * D].view(T, G, D)) * D ** -0.5).repeat_interleave(H // G, dim=1)
    k = P.unit(y[:, G * D : 2 * G * D].view(T, G, D)).repeat_interleave(H // G, dim=1)
    v = y[:, 2 * G * D :].view(T, H, V)
    beta = torch.sigmoid(proj[:, C : C + H])
    per = D if per_channel else 1
    z = a[:, 1 : 1 + H * per] + dt_bias
    decay = torch.exp(-torch.exp(a_log).repeat_interleave(per) * torch.nn.functional.softplus(z)).view(T, H, per).expand(T, H, D)
    return P.delta_rule(q, k, v, beta, decay)


@pytest.mark.parametrize("sizes", [(4, 2, 16, 24, 3, False), (2, 1, 40, 20, 4, True), (3, 3, 20, 12, 1, True), (2, 2, 128, 64, 4, False),
                                   (1, 1, 160, 10, 2, True), (2, 1, 256, 33, 8, False), (5, 5, 32, 7, 4, True), (3, 1, 64, 130, 5, False),
                                   # so many heads and value channels that a column gets 16 lanes instead of 32
                                   (32, 32, 64, 272, 2, False), (36, 12, 40, 240, 3, True)])
def test_delta_rule_whole_in_portions_and_in_a_batch(lib, sizes):
    """The convolution, the unit vectors, the gates and the recurrence of one sequence: whole, cut into portions down to
    one and two tokens (the state carries over), and beside two other sequences in slots used before."""
    from fms_amd.kernels import ops

    H, G, D, V, taps, per_channel = sizes
    T = 150
    proj, a, C = _delta_inputs(T, H, G, D, V, per_channel, seed=D + V)
    gen = torch.Generator().manual_seed(7)
    conv_w = torch.randn(C, taps, generator=gen) * 0.5
    a_log = torch.randn(H, generator=gen) - 1
    dt_bias = torch.randn(H * (D if per_channel else 1), generator=gen)
    want = _plain_delta(proj, a, conv_w, a_log, dt_bias, H, G, D, V, per_channel, C).reshape(T, H * V)
    other = [_delta_inputs(n, H, G, D, V, per_channel, seed=n) for n in (9, 70)]
    want_other = [_plain_delta(p, x, conv_w, a_log, dt_bias, H, G, D, V, per_channel, C).reshape(-1, H * V) for p, x, _ in other]

    n_slots = 4
    S = torch.randn(n_slots, H, V, D, device=DEV)  # slots hold what earlier sequences left
    conv_state = torch.randn(n_slots, max(taps - 1, 1), C, device=DEV)

    def run(pieces, slots, single_tokens=False):
        """pieces: per sequence (proj rows, a rows); one step for all of them."""
        lens = [p.shape[0] for p, _ in pieces]
        seq = torch.repeat_interleave(torch.arange(len(pieces)), torch.tensor(lens)).to(torch.int32).to(DEV)
        starts = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32, device=DEV)
        slot_ids = torch.tensor(slots, dtype=torch.int32, device=DEV)
        pr = torch.cat([p for p, _ in pieces]).to(DEV)
        aa = torch.cat([x for _, x in pieces]).to(DEV)
        qkv, beta, decay, kq = ops.delta_prepare(pr, C, aa, 1, conv_w.to(DEV), a_log.to(DEV), dt_bias.to(DEV), conv_state, seq, slot_ids,
                                                 H, G, D, V, per_channel, D ** -0.5)
        out = ops.delta_rule(qkv, beta, decay, kq, S, starts, seq, slot_ids, len(pieces), H, G, D, V, per_channel, single_tokens=single_tokens)
        return torch.split(out.cpu(), lens)

    tol = dict(atol=5e-5, rtol=1e-4)
    for cuts in ([150], [1, 2, 1, 60, 3, 2, 17, 64], [2] * 5 + [140]):
        S[2].zero_()
        conv_state[2].zero_()
        got, at = [], 0
        for n in cuts:
            got.append(run([(proj[at : at + n], a[at : at + n])], [2])[0])
            at += n
        torch.testing.assert_close(torch.cat(got), want, **tol)
    # token by token as a decode step runs it (the kernel is told that no sequence brings more than one token)
    S[2].zero_()
    conv_state[2].zero_()
    got = [run([(proj[t : t + 1], a[t : t + 1])], [2], single_tokens=True)[0] for t in range(40)]
    torch.testing.assert_close(torch.cat(got), want[:40], **tol)
    # a batch of three unequal sequences in slots 3, 0, 1 (freshly zeroed, as the cache hands them out), then each goes on
    for s in (3, 0, 1):
        S[s].zero_()
        conv_state[s].zero_()
    first = run([(other[0][0][:5], other[0][1][:5]), (proj[:100], a[:100]), (other[1][0][:69], other[1][1][:69])], [3, 0, 1])
    second = run([(other[0][0][5:], other[0][1][5:]), (proj[100:], a[100:]), (other[1][0][69:], other[1][1][69:])], [3, 0, 1])
    torch.testing.assert_close(torch.cat([first[1], second[1]]), want, **tol)
    torch.testing.assert_close(torch.cat([first[0], second[0]]), want_other[0], **tol)
    torch.testing.assert_close(torch.cat([first[2], second[2]]), want_other[1], **tol)
    # a padding row (sequence -1) between live ones changes nothing and writes no state
    before = S.clone()
    seq = torch.tensor([-1], dtype=torch.int32, device=DEV)
    qkv, beta, decay, kq = ops.delta_prepare(proj[:1].to(DEV), C, a[:1].to(DEV), 1, conv_w.to(DEV), a_log.to(DEV), dt_bias.to(DEV), conv_state,
                                             seq, torch.tensor([2], dtype=torch.int32, device=DEV), H, G, D, V, per_channel, 1.0)
    ops.delta_rule(qkv, beta, decay, kq, S, torch.tensor([0, 1], dtype=torch.int32, device=DEV), seq,
                   torch.tensor([2], dtype=torch.int32, device=DEV), 1, H, G, D, V, per_channel)
    assert bool((S == before).all())


def test_a_lost_state_shows(lib):
    """The recurrence's memory matters: a value written long ago, read by a matching query much later, with decays near one."""
    from fms_amd.kernels import ops

    H, G, D, V, T = 1, 1, 32, 16, 400
    C = 2 * D + V
    qkv = torch.zeros(T, C)
    gen = torch.Generator().manual_seed(5)
    keys = torch.nn.functional.normalize(torch.randn(T, D, generator=gen), dim=-1)
    qkv[:, D : 2 * D] = keys
    qkv[:, 2 * D :] = torch.randn(T, V, generator=gen)
    qkv[:, :D] = keys[0]  # every query asks for what the first token wrote
    beta = torch.ones(T, H)
    decay = torch.full((T, H), 0.9995)
    want = P.delta_rule(qkv[:, :D].view(T, 1, D), keys.view(T, 1, D), qkv[:, 2 * D :].view(T, 1, V), beta, decay.view(T, 1, 1).expand(T, 1, D))
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    starts = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    slot = torch.zeros(1, dtype=torch.int32, device=DEV)
    S = torch.zeros(1, H, V, D, device=DEV)
    kq = (qkv[:, :D] * keys).sum(-1, keepdim=True)
    got = ops.delta_rule(qkv.to(DEV), beta.to(DEV), decay.to(DEV), kq.to(DEV), S, starts, seq, slot, 1, H, G, D, V, False).cpu()
    torch.testing.assert_close(got, want.view(T, V), atol=1e-4, rtol=1e-4)
    # the first token's value still holds a good part of the last read-out
    assert float((want[-1, 0] - 0).norm()) > 0.1
    S.zero_()
    first = ops.delta_rule(qkv[:300].to(DEV), beta[:300].to(DEV), decay[:300].to(DEV), kq[:300].to(DEV), S, torch.tensor([0, 300], dtype=torch.int32, device=DEV),
                           seq[:300], slot, 1, H, G, D, V, False)
    S.zero_()  # the state is lost between two steps
    rest = ops.delta_rule(qkv[300:].to(DEV), beta[300:].to(DEV), decay[300:].to(DEV), kq[300:].to(DEV), S, torch.tensor([0, 100], dtype=torch.int32, device=DEV),
                          seq[:100], slot, 1, H, G, D, V, False).cpu()
    assert float((rest - want.view(T, V)[300:]).abs().max()) > 0.05 and first.shape[0] == 300


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(3, 20, "sigmoid"), (4, 64, "silu"), (2, 130, "silu"), (1, 7, "sigmoid")])
def test_head_norm_with_a_gate(lib, dtype, sizes):
    from fms_amd.kernels import ops

    H, V, act = sizes
    T = 11
    gen = torch.Generator().manual_seed(V)
    o = torch.randn(T, H * V, generator=gen) * 3
    gate = torch.randn(T, H * V + 5, generator=gen)
    w = 1 + 0.3 * torch.randn(V, generator=gen)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    out = torch.zeros(T, H * V + 8, dtype=dtype, device=DEV)
    ops.gated_head_norm(o.to(DEV), gate.to(DEV)[:, 2 : 2 + H * V], w.to(DEV), 1e-5, act, H, V, dtype, seq, scale=0.7, out=out[:, 8:])
    g = gate[:, 2 : 2 + H * V]
    g = torch.sigmoid(g) if act == "sigmoid" else g * torch.sigmoid(g)
    want = (P.rms(o.view(T, H, V), 1e-5) * w).view(T, H * V) * g * 0.7
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(out[:, 8:].float().cpu(), want, **tol)
    assert float(out[:, :8].float().abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_over_whole_projections_gate_and_scales(lib, dtype):
    from fms_amd.kernels import ops

    gen = torch.Generator().manual_seed(1)
    T, nq, nk, nv = 9, 60, 36, 50
    proj = torch.randn(T, nq + nk + nv + 7, generator=gen) * 2
    wq, wk = (1 + 0.3 * torch.randn(nq, generator=gen)).to(dtype), (1 + 0.3 * torch.randn(nk, generator=gen)).to(dtype)
    got = ops.qk_projection_norm(proj.to(DEV), nq, nk, nv, wq.to(DEV), wk.to(DEV), 1e-5, dtype).float().cpu()
    want = torch.cat([P.rms(proj[:, :nq], 1e-5) * wq.float(), P.rms(proj[:, nq : nq + nk], 1e-5) * wk.float(), proj[:, nq + nk : nq + nk + nv]], dim=1)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=1e-2)
    torch.testing.assert_close(got, want, **tol)
    x = torch.randn(T, 44, generator=gen).to(dtype)
    gate = torch.randn(T, 50, generator=gen)
    out = torch.zeros(T, 60, dtype=dtype, device=DEV)
    ops.gate_mul(x.to(DEV), gate.to(DEV)[:, 3:47], "sigmoid", 0.8, out=out[:, 16:])
    torch.testing.assert_close(out[:, 16:].float().cpu(), x.float() * torch.sigmoid(gate[:, 3:47]) * 0.8, **tol)
    logits = torch.randn(5, 33, generator=gen)
    torch.testing.assert_close(ops.scale_(logits.to(DEV), 1.75).cpu(), logits * 1.75)
    torch.testing.assert_close(ops.cast_cols(proj.to(DEV), 3, 29, dtype).float().cpu(), proj[:, 3:32].to(dtype).float())
    # a norm whose weight is stored around zero
    from fms_amd.parts import make_part

    norm = make_part("norm", "rmsnorm", width=40, eps=1e-5, weight_offset=1.0)
    w = (0.2 * torch.randn(40, generator=gen)).to(dtype)
    norm.bind("weight", w.to(DEV))
    norm.finalize(torch.device(DEV), dtype)
    resid = torch.randn(6, 40, generator=gen)
    got = norm.add_norm(resid.to(DEV), None, dtype).float().cpu()
    torch.testing.assert_close(got, P.layer_norm(resid, w.float(), 1e-5), **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 32, 24, 40, 15.0), (3, 3, 20, 36, 5, 8.0), (2, 1, 64, 64, 0, 30.0), (2, 2, 16, 200, 64, 0.0)])
def test_attention_with_values_of_their_own_size_a_cap_and_a_window(lib, dtype, sizes):
    """Keys and values written by the cache-write kernel, read by the attention kernel; queries just inside and just
    outside the window's edge and a page's border; one query and one key scaled so that the key at the window's
    last place decides, and the one a place further must not be seen."""
    from fms_amd.kernels import ops

    H, K, D, V, window, cap = sizes
    gen = torch.Generator().manual_seed(D + V)
    n = 200
    rows = torch.randn(n, (H + K) * D + K * V, generator=gen).to(dtype)
    edge = window or 130
    far = n - edge  # the last key the last query sees (with a window); far - 1 is just outside
    k0 = H * D
    rows[far, k0 : k0 + D] *= 5
    rows[far - 1, k0 : k0 + D] *= 5
    rows[n - 1, :D] = rows[far, k0 : k0 + D] * 0.5
    pages = [5, 0, 3, 6]
    kc = torch.zeros(8, K, 64, D, dtype=dtype, device=DEV)
    vc = torch.zeros(8, K, V, 64, dtype=dtype, device=DEV)
    table = torch.tensor([pages], dtype=torch.int32, device=DEV)
    pos = torch.arange(n, dtype=torch.int32, device=DEV)
    seq = torch.zeros(n, dtype=torch.int32, device=DEV)
    qkv = rows.to(DEV).clone()
    ops.rope_kv_write(qkv, pos, seq, table, None, None, 0, kc, vc, H, K, D, V)
    got = ops.attention(qkv, pos, seq, table, kc, vc, H, K, D, 0.3, window, soft_cap=cap, value_dim=V, force_generic=True).float().cpu().view(n, H, V)
    q = rows[:, : H * D].float().view(n, H, D)
    k = rows[:, k0 : k0 + K * D].float().view(n, K, D)
    v = rows[:, k0 + K * D :].float().view(n, K, V)
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    visible = (j <= i) & ((i - j < window) if window else torch.ones(n, n, dtype=torch.bool))
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
    for h in range(H):
        g = h // (H // K)
        s = (q[:, h] @ k[:, g].T) * 0.3
        if cap:
            s = cap * torch.tanh(s / cap)
        p = torch.softmax(s.masked_fill(~visible, float("-inf")), dim=-1)
        torch.testing.assert_close(got[:, h], p @ v[:, g], **tol)
        if h == 0 and window:
            assert float(p[n - 1, far]) > 0.5 and float(p[n - 1, far - 1]) == 0.0


@pytest.mark.parametrize("sizes", [(12, 4, 1), (5, 1, 5), (64, 8, 300), (130, 6, 17)])
def test_router_with_sigmoid_scores(lib, sizes):
    from fms_amd.kernels import ops

    E, top, T = sizes
    logits = torch.randn(T, E + 1, generator=torch.Generator().manual_seed(E)) * 3
    want = torch.topk(logits[:, :E], top, dim=-1)
    ids, weights = ops.moe_route(logits.to(DEV), E, top, "sigmoid")
    assert ids.cpu().tolist() == want.indices.tolist()
    torch.testing.assert_close(weights.cpu(), torch.sigmoid(want.values), atol=1e-6, rtol=1e-5)
    ids, weights = ops.moe_route(logits.to(DEV), E, top, "sigmoid_normed")
    torch.testing.assert_close(weights.cpu(), torch.sigmoid(want.values) / torch.sigmoid(want.values).sum(-1, keepdim=True), atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(6, 2, 48, 128, 50), (5, 1, 36, 100, 7), (8, 8, 128, 256, 40), (4, 2, 64, 128, 300), (3, 1, 24, 70, 9)])
def test_experts_weighted_on_their_input(lib, dtype, sizes):
    """The part against the plain function: the score scales what the expert reads, not what it returns."""
    from fms_amd.parts import make_part

    E, top, ff, width, T = sizes
    gen = torch.Generator().manual_seed(ff)
    part = make_part("feed_forward", "experts", width=width, experts=E, top=top, hidden_dim=ff, limit=None, alpha=1.0, shift=0.0,
                     score="sigmoid", weight_on="input")
    w = {"router": torch.randn(E, width, generator=gen) * 0.5}
    for e in range(E):
        w[f"e{e}.gate"] = torch.randn(ff, width, generator=gen) / math.sqrt(width)
        w[f"e{e}.up"] = torch.randn(ff, width, generator=gen) / math.sqrt(width)
        w[f"e{e}.down"] = torch.randn(width, ff, generator=gen) / math.sqrt(ff)
    w = {k: v.to(dtype).float() for k, v in w.items()}
    torch_dtype = dtype
    part.router.bind("weight", w["router"].to(torch_dtype).to(DEV))
    for which in ("gate", "up", "down"):
        part.bind(f"experts.{which}", torch.stack([w[f"e{e}.{which}"] for e in range(E)]).to(torch_dtype).to(DEV))
    x = torch.randn(T, width, generator=gen).to(dtype)
    P.router_margins = []
    try:
        want = P.experts(x.float(), w, "", {"router": {"experts": E, "top": top}})
        clear = P.router_margins[0] > (0.0 if dtype == torch.float32 else 0.1)
    finally:
        P.router_margins = None
    got = part.forward(x.to(DEV)).float().cpu()
    tol = dict(atol=2e-4, rtol=1e-3) if dtype == torch.float32 else dict(atol=6e-2, rtol=3e-2)
    torch.testing.assert_close(got[clear], want[clear], **tol)
    # on the output instead, the result differs: the place of the weight is not a no-op in this test
    part.weight_on = "output"
    other = part.forward(x.to(DEV)).float().cpu()
    if dtype == torch.float32:
        assert float((other - got).abs().max()) > 0.01


# ---- the engine ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_sequence(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    ids, want = expected_for(folders, name, 150, 1, dtype)
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=256, max_slots=2)
    slot = engine.new_sequence()
    judge(engine.step([slot], [ids], "all"), want, dtype)
    engine.end_sequence(slot)
    engine.cache.check()


@pytest.mark.parametrize("name", ["A", "B"])
def test_the_stream_after_every_layer(lib, folders, name):
    """float32: the residual stream after each layer against the plain implementation's, so that a fault names its layer."""
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    ids = tokens_for(cfg["vocab"], 90, 2)
    _, layers = P.forward(cfg, weights, ids, return_layers=True)
    model = get(lib, folders, name, "float32")
    seen = []
    blocks = model.layers
    originals = [b.forward for b in blocks]

    def watch(i):
        def forward(stream, batch, cache, act_dtype, next_norm=None):
            originals[i](stream, batch, cache, act_dtype)
            resid = stream.resid.clone()  # what is still pending joins the stream in a copy: the stream after this layer
            seen.append((resid + stream.pending.float()).cpu() if stream.pending is not None else resid.cpu())
        return forward

    try:
        for i, b in enumerate(blocks):
            b.forward = watch(i)
        engine = Engine(model, max_tokens=128, max_slots=1)
        slot = engine.new_sequence()
        engine.step([slot], [ids], "last")
        engine.end_sequence(slot)
    finally:
        for b in blocks:
            del b.forward
    assert len(seen) == len(cfg["layers"])
    for i, got in enumerate(seen):
        torch.testing.assert_close(got, layers[i], atol=2e-4, rtol=1e-4, msg=lambda m, i=i: f"layer {i}: {m}")


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_prompt_then_token_by_token_and_the_first_tokens(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    ids, want = expected_for(folders, name, 150, 1, dtype)
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=256, max_slots=2)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:100]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[100:]]
    judge(torch.cat(got), want, dtype)
    engine.end_sequence(slot)
    # from the very first token one by one: the convolution's zeros before the start, the empty state, the window's start
    slot = engine.new_sequence()
    got = [engine.step([slot], [[t]], "last") for t in ids[:40]]
    judge(torch.cat(got), want[:40], dtype)
    engine.end_sequence(slot)
    engine.cache.check()


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_of_several_sizes(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    ids, want = expected_for(folders, name, 150, 1, dtype)
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=256, max_slots=1)
    for cuts in ([2, 2, 60, 1, 63, 2, 20], [64, 64, 22], [63, 2, 2, 83], [1, 127, 22]):
        slot = engine.new_sequence()
        got, at = [], 0
        for n in cuts:
            got.append(engine.step([slot], [ids[at : at + n]], "all"))
            at += n
        assert at == 150
        judge(torch.cat(got), want, dtype)
        engine.end_sequence(slot)
    engine.cache.check()


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_ragged_batches_with_pages_and_slots_used_again(lib, folders, name, dtype):
    """Unequal requests in one batch, decoded together; the short ones end early, their slots (with the state they
    left) and pages go to new requests that start while the long one goes on; every request equals itself alone."""
    from fms_amd.engine import Engine

    lens = {"a": (150, 1), "b": (70, 5), "c": (3, 6), "d": (129, 7), "e": (66, 8)}
    reqs = {k: expected_for(folders, name, n, seed, dtype) for k, (n, seed) in lens.items()}
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=64 * 6, max_slots=3)
    got = {k: [] for k in reqs}
    slots = {k: engine.new_sequence() for k in ("a", "b", "c")}
    prompt = {"a": 100, "b": 64, "c": 1}
    out = engine.step([slots[k] for k in ("a", "b", "c")], [reqs[k][0][: prompt[k]] for k in ("a", "b", "c")], "all")
    at = 0
    for k in ("a", "b", "c"):
        got[k].append(out[at : at + prompt[k]])
        at += prompt[k]
    done = dict(prompt)
    alive = ["a", "b", "c"]
    waiting = ["d", "e"]
    while alive:
        out = engine.step([slots[k] for k in alive], [[reqs[k][0][done[k]]] for k in alive], "last")
        for i, k in enumerate(alive):
            got[k].append(out[i : i + 1])
            done[k] += 1
        for k in [k for k in alive if done[k] == len(reqs[k][0])]:
            engine.end_sequence(slots.pop(k))
            alive.remove(k)
        if waiting and len(alive) < 2 and "a" in alive:
            k = waiting.pop(0)
            slots[k] = engine.new_sequence()
            n = len(reqs[k][0]) - 4
            got[k].append(engine.step([slots[k]], [reqs[k][0][:n]], "all"))
            done[k] = n
            alive.append(k)
    assert not waiting
    for k, (ids, want) in reqs.items():
        judge(torch.cat(got[k]), want, dtype)
    engine.cache.check()
    assert engine.cache.n_free_slots == 3 and all(g.pool.n_held == 0 for g in engine.cache.groups)


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_windows_edge_decides_in_prompts_and_in_decoding(lib, dtype, tmp_path):
    """Queries scaled up: single keys hold most of a query's weight, among them keys at the window's last place and
    at page borders.  The same weights run with a window one token longer or shorter must fail the same comparison."""
    from fms_amd.engine import Engine

    base = CONFIGS["C"]
    folder = write_folder(lib, str(tmp_path / "sharp"), base, seed=21, sharp=6.0)
    cfg, weights = P.load_model_folder(folder)
    ids = tokens_for(cfg["vocab"], 330, 3)
    want = expect(cfg, weights, ids, dtype)
    # sharp indeed, and at the edge: in layer 0 some late queries give the key at the window's last place a large weight
    m = cfg["layers"][0]["mixer"]["left"]
    h = P.layer_norm(weights["embed"][torch.tensor(ids)], weights["l0.norm1"], cfg["norm"]["eps"])
    pos = torch.arange(len(ids))
    q = P.rotate_pairs((P.rms(h @ weights["l0.mix.left.q"].T + weights["l0.mix.left.q.b"], cfg["norm"]["eps"]) * weights["l0.mix.left.q.norm"]).view(len(ids), m["heads"], -1), pos, m["rot"])
    k = P.rotate_pairs((P.rms(h @ weights["l0.mix.left.k"].T + weights["l0.mix.left.k.b"], cfg["norm"]["eps"]) * weights["l0.mix.left.k.norm"]).view(len(ids), m["kv_heads"], -1), pos, m["rot"])
    k = k.repeat_interleave(m["heads"] // m["kv_heads"], dim=1)
    s = m["softcap"] * torch.tanh(torch.einsum("thd,shd->hts", q, k) * m["scale"] / m["softcap"])
    size = m["mask"]["size"]
    visible = (pos[None, :] <= pos[:, None]) & (pos[:, None] - pos[None, :] < size)
    prob = torch.softmax(s.masked_fill(~visible, float("-inf")), -1)
    late = torch.arange(size, len(ids))
    assert float(prob[:, late, late - size + 1].max()) > 0.2

    def run(folder_, cut):
        model = lib.get_model("hf_pretrained", model_path=folder_, data_type=dtype)
        engine = Engine(model, max_tokens=384, max_slots=1)
        slot = engine.new_sequence()
        got = [engine.step([slot], [ids[:cut]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[cut:]]
        engine.end_sequence(slot)
        return torch.cat(got)

    judge(run(folder, 250), want, dtype)
    for other in (size + 1, size - 1):
        wrong = json.loads(json.dumps(cfg))
        wrong["layers"][0]["mixer"]["left"]["mask"]["size"] = other
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(wrong, f)
        with pytest.raises(AssertionError):
            judge(run(folder, 250), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_graphs_and_eager_steps(lib, folders, dtype):
    """300 tokens decoded one by one for three sequences of different lengths, across page borders and past the
    window, as captured graphs and as eager steps: the same logits as the plain implementation's."""
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    name = "C"
    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, dtype)
    seqs = [tokens_for(cfg["vocab"], n, 30 + n) for n in (360, 330, 301)]
    want = [expect(cfg, weights, s, dtype) for s in seqs]
    for use_graphs in (True, False):
        engine = Engine(model, max_tokens=64 * 18, max_slots=3, use_graphs=use_graphs)
        slots = [engine.new_sequence() for _ in seqs]
        engine.step(slots, [s[: len(s) - 300] for s in seqs], "last")
        got = [[] for _ in seqs]
        for i in range(300):
            feed = [s[len(s) - 300 + i] for s in seqs]
            if use_graphs:
                engine.decode_and_choose(slots, feed, SamplingParams(do_sample=False))
                logits = engine.last_graph.logits[: len(seqs)].clone()
            else:
                logits = engine.step(slots, [[t] for t in feed], "last")
            for b in range(len(seqs)):
                got[b].append(logits[b : b + 1])
        for b, s in enumerate(seqs):
            judge(torch.cat(got[b]), want[b][len(s) - 300 :], dtype)
        for s in slots:
            engine.end_sequence(s)
        engine.cache.check()
        assert bool(engine.graph_captures) == use_graphs


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_greedy_generation_through_the_entry_point_and_the_scheduler(lib, folders, name):
    from fms_amd.engine import Engine
    from fms_amd.generation import generate, generate_requests

    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, "float32")
    prompts = [tokens_for(cfg["vocab"], n, 40 + n) for n in (5, 70, 17, 1)]
    want = [P.greedy_generate(cfg, weights, p, 12) for p in prompts]
    for p, w in zip(prompts[:2], want):
        assert generate(model, torch.tensor(p), max_new_tokens=12, do_sample=False).tolist() == p + w
    # the scheduler: more requests than slots, so batches follow one another and slots are used again
    engine = Engine(model, max_tokens=64 * 4, max_slots=2)
    assert generate_requests(engine, prompts, max_new_tokens=12) == want
    stop = want[1][5]
    out = generate_requests(engine, prompts, max_new_tokens=12, stop_token_ids=[stop])
    for o, w in zip(out, want):
        assert o == (w[: w.index(stop) + 1] if stop in w else w)
    engine.cache.check()


def test_command_line_and_trace_replay(lib, folders, tmp_path):
    """The package's programs on a Defapel folder: the trace replay (float32 and bfloat16, a batch whose requests end
    at different steps) and the registry's view of the architecture."""
    name = "A"
    cfg, weights = plain(folders, name)
    assert "defapel" in lib.list_models() and "micro" in lib.list_variants("defapel")
    reqs = {"x": tokens_for(cfg["vocab"], 90, 51), "y": tokens_for(cfg["vocab"], 40, 52)}
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": reqs["x"][:80], "want": [0, 79]}, {"id": "y", "tokens": reqs["y"][:38], "want": [37]}], "end": []}]
    for i in range(10):
        entries = [{"id": "x", "tokens": [reqs["x"][80 + i]], "want": [0]}]
        if i < 2:
            entries.append({"id": "y", "tokens": [reqs["y"][38 + i]], "want": [0] if i == 1 else []})
        steps.append({"step": i + 1, "entries": entries, "end": (["y"] if i == 1 else []) + (["x"] if i == 9 else [])})
    for dtype in DTYPES:
        want = {k: expect(cfg, weights, v, dtype) for k, v in reqs.items()}
        out_dir = str(tmp_path / f"out_{dtype}")
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype,
                               "--out", out_dir, "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                              capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {i}" for i in range(11)]

        def read(step):
            return torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())

        judge(read(0), Expected.stack([want["x"][0], want["x"][79], want["y"][37]]), dtype)
        judge(read(2), Expected.stack([want["x"][81], want["y"][39]]), dtype)
        judge(read(10), want["x"][89:90], dtype)
    # many short requests at once, --max-tokens counting their tokens as they are (every request still takes a page and a slot)
    short = {f"s{i}": tokens_for(cfg["vocab"], 4 + i % 5, 60 + i) for i in range(14)}
    steps = [{"step": 0, "entries": [{"id": k, "tokens": v[:-2], "want": [len(v) - 3]} for k, v in short.items()], "end": []}]
    for j in (2, 1):
        steps.append({"step": len(steps), "entries": [{"id": k, "tokens": [v[-j]], "want": [0]} for k, v in short.items()],
                      "end": list(short) if j == 1 else []})
    out_dir = str(tmp_path / "out_short")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", "float32",
                           "--out", out_dir, "--max-tokens", str(sum(len(v) for v in short.values()))],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    want = {k: expect(cfg, weights, v, "float32") for k, v in short.items()}
    for step, back in ((0, 3), (1, 2), (2, 1)):
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]).copy())
        judge(got, Expected.stack([want[k][len(v) - back] for k, v in short.items()]), "float32")


def test_the_inference_program_and_a_model_from_the_registry(lib, folders):
    """bin/fms_inference with a Defapel folder (the model class comes from config.json; the text printed is the plain
    implementation's greedy continuation), and a registered variant with random weights through the engine."""
    from fms_amd.engine import Engine
    from fms_amd.tokenizers import CharTokenizer

    name = "A"  # its vocabulary holds the character tokenizer's
    cfg, weights = plain(folders, name)
    tok = CharTokenizer()
    prompt = [ord(c) for c in "delta rule"]
    new = P.greedy_generate(cfg, weights, prompt, 12)
    if tok.eos_token_id in new:
        new = new[: new.index(tok.eos_token_id)]
    env = dict(os.environ, PYTHONIOENCODING="utf-8")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "fms_inference"), "--architecture", "hf_pretrained", "--model_path", folders[name],
           "--tokenizer", "char_tokenizer", "--default_dtype", "fp32", "--max_new_tokens", "12", "--prompt_ids", ",".join(map(str, prompt))]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=110, env=env)
    assert proc.returncode == 0, proc.stderr.decode(errors="replace")
    assert tok.decode(prompt + new) in proc.stdout.decode("utf-8")

    model = lib.get_model("defapel", "micro", data_type="bfloat16")
    engine = Engine(model, max_tokens=256, max_slots=2)
    a, b = engine.new_sequence(), engine.new_sequence()
    logits = engine.step([a, b], [list(range(70)), [5, 6, 7]], "last")
    assert logits.shape == (2, model.spec.vocab) and bool(torch.isfinite(logits).all())
    alone = Engine(model, max_tokens=256, max_slots=1)
    s = alone.new_sequence()
    torch.testing.assert_close(alone.step([s], [[5, 6, 7]], "last"), logits[1:], atol=2e-2, rtol=2e-2)
