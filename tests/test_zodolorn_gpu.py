"""Zodolorn on the GPU against the plain implementation (plain_zodolorn.py): every mechanism alone, then the engine
whole / token by token / in portions / in ragged batches with reused slots / through graphs and the generation loop,
in float32 and bfloat16, at sizes that differ from one another in everything.

bfloat16 is judged like the other models of this folder (gpu_checks): the plain implementation run with bfloat16
storage shows what that type costs at every position, and the engine may be a small multiple of that off."""

import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_zodolorn as Z  # noqa: E402
from gpu_checks import Expected  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
# bfloat16: at every position the engine may be BF16_MARGIN times as far off as the plain implementation with bfloat16
# storage is there (or as it typically is), and on average BF16_MEAN_MARGIN times.  The engine rounds in other places
# than the plain implementation (queries and attention results in the latent space instead of keys and values).
BF16_MARGIN = 3.0
BF16_MEAN_MARGIN = 1.5
# A router's choice is "close" when the last chosen logit leads the first one not chosen by less than this: bfloat16
# rounding can turn it, the token then runs other experts, and its logits are no test of arithmetic.  Such positions
# are left out of bfloat16 comparisons (logits of the routers here spread over several units).
CLOSE_CALL = 0.25


def mixer(heads, dim, rot, vdim, q_rank, kv_rank, scale, base=10000.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts, top, ff, limit, shared=None):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def layer(m, mlp):
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


_mA = dict(heads=4, dim=16, rot=8, vdim=24, q_rank=48, kv_rank=40, scale=0.2)
_mB = dict(heads=3, dim=12, rot=4, vdim=20, q_rank=36, kv_rank=28, scale=0.31)
_mC = dict(heads=8, dim=64, rot=32, vdim=48, q_rank=128, kv_rank=128, scale=0.1)
CONFIGS = {
    # two layers read the first one's latent; a layer without a feed-forward; experts with and without a shared one,
    # one of them choosing all its experts
    "A": dict(vocab=300, width=128, norm={"eps": 1e-5}, embedding={"scale": 7.0}, max_positions=1024, layers=[
        layer(mixer(**_mA), {"kind": "dense", "ff": 160}),
        layer(mixer(**_mA, kv_from=0), moe(6, 2, 48, 1.5, shared=(64, 2.5))),
        layer(mixer(**_mA, kv_from=0), None),
        layer(mixer(**_mA), moe(4, 4, 40, 0.7)),
        layer(mixer(**_mA), {"kind": "dense", "ff": 96}),
    ]),
    # sizes that are no multiples of 8 (rows that the matrix instructions cannot load), one expert per token, layers
    # that differ in their rotation and sizes
    "B": dict(vocab=257, width=100, norm={"eps": 1e-6}, embedding={"scale": 1.0}, max_positions=1024, layers=[
        layer(mixer(**_mB, base=500.0), moe(5, 1, 36, 3.0, shared=(44, 1.0))),
        layer(mixer(heads=2, dim=20, rot=12, vdim=8, q_rank=24, kv_rank=36, scale=0.25, base=1e6), {"kind": "dense", "ff": 60}),
    ]),
    # sizes at which bfloat16 runs the matrix-instruction kernels throughout
    "C": dict(vocab=512, width=256, norm={"eps": 1e-6}, embedding={"scale": 16.0}, max_positions=2048, layers=[
        layer(mixer(**_mC), {"kind": "dense", "ff": 512}),
        layer(mixer(**_mC, kv_from=0), moe(8, 2, 128, 2.0, shared=(128, 4.0))),
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
    """A model folder with random weights: sinks of the size of the scores, noisy norm scales."""
    from fms_amd.weights import write_safetensors

    lib.write_model_folder(folder, lib.ZodolornConfig(**cfg_kw), seed=seed, architecture="zodolorn", std=0.08, norm_std=0.2)
    cfg, tensors = Z.load_model_folder(folder)
    gen = torch.Generator().manual_seed(seed)
    for k in list(tensors):
        if k.endswith(".mix.sink"):
            tensors[k] = torch.randn(tensors[k].shape, generator=gen) * 1.5
        if k.endswith(".mix.g") or k.endswith(".mlp.router") or k.endswith(".shared.sg"):
            tensors[k] = tensors[k] * 4  # gates away from one half, routers with clear choices
        if sharp != 1.0 and k.endswith(".mix.uq"):
            tensors[k] = tensors[k] * sharp
    tensors = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory, lib):
    return {name: write_folder(lib, str(tmp_path_factory.mktemp(f"zodolorn_{name}")), kw, 3 + i) for i, (name, kw) in enumerate(CONFIGS.items())}


_models, _plain, _expected = {}, {}, {}


def get(lib, folders, name, dtype):
    if (name, dtype) not in _models:
        _models[(name, dtype)] = lib.get_model("hf_pretrained", model_path=folders[name], data_type=dtype)
    return _models[(name, dtype)]


def plain(folders, name):
    if name not in _plain:
        _plain[name] = Z.load_model_folder(folders[name])
    return _plain[name]


def tokens_for(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def expect(cfg, weights, ids, dtype) -> Expected:
    """Exact logits; for bfloat16 also the plain implementation's own error with bfloat16 storage, set to infinity at
    the positions where a router's choice is close (they are not compared), and its 90th percentile over the rest."""
    margins = []
    exact = Z.forward(cfg, weights, ids, margins=margins)
    if dtype == "float32":
        return Expected(exact)
    rounded = Z.forward(cfg, weights, ids, storage=torch.bfloat16)
    error = (rounded - exact).abs().amax(dim=-1)
    close = torch.zeros(len(ids), dtype=torch.bool)
    for gap in margins:
        close |= gap < CLOSE_CALL
    assert float(close.float().mean()) < 0.5, "most positions have close router calls: the test would compare little"
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
        torch.testing.assert_close(got, want.logits, atol=2e-4, rtol=1e-3)
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
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 192, 1001, 3000, 4100])
def test_norm_behind_a_branch_sum_and_next_norm(lib, dtype, width):
    from fms_amd.kernels import ops

    gen = torch.Generator().manual_seed(width)
    resid = torch.randn(7, width, generator=gen) * 3
    branch = (torch.randn(7, width, generator=gen) * 5).to(dtype)
    wb, w = 1 + 0.3 * torch.randn(width, generator=gen), 1 + 0.3 * torch.randn(width, generator=gen)
    total = resid + Z.rms_norm(branch.float(), wb, 1e-3)
    want = Z.rms_norm(total, w, 1e-5)
    r = resid.to(DEV).clone()
    out = ops.norm_add_norm(r, branch.to(DEV), wb.to(DEV), 1e-3, w.to(DEV), 1e-5, dtype)
    torch.testing.assert_close(r.cpu(), total, atol=1e-5, rtol=1e-5)
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(out.float().cpu(), want, **tol)
    # chosen rows only (the final norm of a step): the stream stays as it was
    r2 = resid.to(DEV).clone()
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    out2 = ops.norm_add_norm(r2, branch.to(DEV), wb.to(DEV), 1e-3, w.to(DEV), 1e-5, dtype, rows=rows)
    torch.testing.assert_close(out2.float().cpu(), want[[5, 0, 5]], **tol)
    torch.testing.assert_close(r2.cpu(), resid)


def test_embedding_with_a_scale(lib):
    from fms_amd.kernels import ops

    table = torch.randn(50, 24).to(torch.bfloat16)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    got = ops.embed(ids.to(DEV), table.to(DEV), 13.25)
    torch.testing.assert_close(got.cpu(), table[ids.long()].float() * 13.25)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [33, 36])  # single elements, and four a load
def test_activations_beside_the_gated_ones(lib, dtype, hidden):
    from fms_amd.kernels import ops

    x = (torch.randn(9, 2 * hidden + 1 if hidden % 4 else 2 * hidden) * 3).to(dtype)
    tol = dict(atol=1e-6, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    xf = x.float()
    torch.testing.assert_close(ops.activation(x.to(DEV), "gelu").float().cpu(), 0.5 * xf * (1 + torch.erf(xf / math.sqrt(2))), **tol)
    gu = (torch.randn(9, 2 * hidden) * 3).to(dtype)
    g, u = gu.float()[:, :hidden].clamp(max=1.5), gu.float()[:, hidden:].clamp(-1.5, 1.5)
    want = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    torch.testing.assert_close(ops.clamped_gated_act(gu.to(DEV), 1.5, 1.702, 1.0).float().cpu(), want, **tol)
    assert float((gu.float().abs() > 1.5).float().mean()) > 0.3  # the limits were reached


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(5, 3, 12, 28), (37, 4, 16, 40), (20, 8, 64, 128), (3, 2, 128, 48), (150, 3, 64, 136), (129, 2, 40, 24)])
def test_a_product_per_head(lib, dtype, shape):
    from fms_amd.kernels import ops

    T, H, K, N = shape
    gen = torch.Generator().manual_seed(T)
    x = torch.randn(T, H * (K + 8), generator=gen).to(dtype)  # heads K + 8 apart: the product reads a part of each
    w = (torch.randn(H, N, K, generator=gen) / math.sqrt(K)).to(dtype)
    gate = torch.randn(T, H + 3, generator=gen)
    y = torch.zeros(T, H * N + 16, dtype=dtype, device=DEV)
    ops.headwise_linear(x.to(DEV), K + 8, w.to(DEV), y, N, gate=gate.to(DEV)[:, 2 : 2 + H])
    xs = x.float().view(T, H, K + 8)[:, :, :K]
    want = torch.einsum("thk,hnk->thn", xs, w.float()) * torch.sigmoid(gate[:, 2 : 2 + H])[:, :, None]
    tol = dict(atol=1e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    torch.testing.assert_close(y[:, : H * N].float().cpu().view(T, H, N), want, **tol)
    assert float(y[:, H * N :].float().abs().max()) == 0.0  # nothing written past the heads


def _latent_cache(lib, n_pages, width, dtype):
    return torch.zeros(n_pages, 1, 64, width, dtype=dtype, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(3, 24, 8, 0), (2, 40, 4, 70), (5, 128, 32, 0), (20, 96, 16, 0), (17, 32, 8, 100), (2, 512, 64, 0), (4, 192, 32, 0), (3, 384, 64, 50), (6, 256, 64, 0), (1, 16, 0, 0)])
def test_attention_over_a_latent_cache(lib, dtype, sizes):
    """Two sequences whose pages lie mixed in the pool; queries of the second at its last positions, the first one
    decoded alone; a sink that matters; one query and one far key scaled so that the far key decides."""
    from fms_amd.kernels import ops

    H, R, P, window = sizes
    W = R + P
    gen = torch.Generator().manual_seed(R)
    lens = [130, 200]
    rows = [torch.randn(n, W, generator=gen).to(dtype) for n in lens]
    far = 3  # a key far back, at the start of the second sequence
    rows[1][far] *= 4
    cache = _latent_cache(lib, 8, W, dtype)
    pages = [[6, 1, 4], [0, 7, 2, 5]]
    transposed = torch.zeros(8, 1, R, 64, dtype=dtype, device=DEV)  # the latent once more, for the matrix-core kernel
    for s, plist in enumerate(pages):
        for j in range(lens[s]):
            cache[plist[j // 64], 0, j % 64] = rows[s][j].to(DEV)
            transposed[plist[j // 64], 0, :, j % 64] = rows[s][j][:R].to(DEV)
    table = torch.tensor([pages[0] + [-1], pages[1]], dtype=torch.int32, device=DEV)
    q_pos = [(0, 129)] + [(1, p) for p in (0, 1, 63, 64, 65, 127, 128, 191, 199)]
    qa = torch.randn(len(q_pos), H, W, generator=gen).to(dtype)
    qa[-1, 0] = (rows[1][far].float() / rows[1][far].float().norm() * 6).to(dtype)  # head 0 of the last query looks at the far key
    sink = torch.randn(H, generator=gen) * 2
    scale = 0.3
    seq = torch.tensor([s for s, _ in q_pos], dtype=torch.int32, device=DEV)
    pos = torch.tensor([p for _, p in q_pos], dtype=torch.int32, device=DEV)
    got = ops.latent_attention(qa.view(len(q_pos), H * W).to(DEV), pos, seq, table, cache, sink.to(DEV), H, R, P, scale, window,
                               decode=False).float().cpu().view(len(q_pos), H, R)
    wants = []
    for i, (s, p) in enumerate(q_pos):
        lo = max(0, p - window + 1) if window else 0
        keys = rows[s][lo : p + 1].float()
        score = torch.einsum("hw,jw->hj", qa[i].float(), keys) * scale
        top = torch.maximum(score.max(-1).values, sink)
        e = torch.exp(score - top[:, None])
        prob = e / (e.sum(-1) + torch.exp(sink - top))[:, None]
        want = prob @ keys[:, :R]
        tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
        torch.testing.assert_close(got[i], want, **tol)
        wants.append(want)
        if i == len(q_pos) - 1 and not window:
            assert float(prob[0, far]) > 0.5  # the far key holds most of head 0's weight
    # without the sink the result differs: the sink is not a no-op in this test
    bare = ops.latent_attention(qa.view(len(q_pos), H * W).to(DEV), pos, seq, table, cache, None, H, R, P, scale, window).float().cpu()
    assert float((bare.view(len(q_pos), H, R) - got).abs().max()) > 0.05
    if dtype == torch.bfloat16 and ops.latent_attention_fits_mfma(R, P) and (H * W) % 8 == 0:
        # the matrix-core kernel: as for prompts (a wave a token), and as a decode step whose keys are dealt over
        # the waves of several blocks and merged (the queries here all have different tokens, as in such a step)
        tol = dict(atol=3e-2, rtol=3e-2)
        for how in (dict(decode=False), dict(decode=True, max_context=256), dict(decode=True, max_context=8192)):
            fast = ops.latent_attention(qa.view(len(q_pos), H * W).to(DEV), pos, seq, table, cache, sink.to(DEV), H, R, P, scale, window,
                                        vt_cache=transposed, **how).float().cpu().view(len(q_pos), H, R)
            torch.testing.assert_close(fast, torch.stack(wants), **tol)
        pad = torch.tensor([-1] * len(q_pos), dtype=torch.int32, device=DEV)  # padding rows of a captured step: skipped
        for how in (dict(decode=False), dict(decode=True, max_context=256)):
            none = ops.latent_attention(qa.view(len(q_pos), H * W).to(DEV), pos, pad, table, cache, sink.to(DEV), H, R, P, scale, window,
                                        vt_cache=transposed, **how)
            assert float(none.float().abs().max()) == 0.0


@pytest.mark.parametrize("sizes", [(12, 4, 1), (5, 1, 5), (64, 8, 300), (130, 6, 17)])
def test_router(lib, sizes):
    from fms_amd.kernels import ops

    E, top, T = sizes
    logits = torch.randn(T, E + 1, generator=torch.Generator().manual_seed(E)) * 3
    ids, weights = ops.moe_route(logits.to(DEV), E, top)
    want = torch.topk(logits[:, :E], top, dim=-1)
    assert ids.cpu().tolist() == want.indices.tolist()
    torch.testing.assert_close(weights.cpu(), torch.softmax(want.values, -1), atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(6, 2, 48, 128, 50), (5, 1, 36, 100, 7), (8, 8, 128, 256, 40), (3, 2, 20, 64, 1), (4, 2, 64, 128, 300), (3, 3, 200, 72, 150), (2, 2, 16, 4352, 3), (3, 1, 24, 70, 9)])
def test_experts_and_their_sum(lib, dtype, sizes):
    from fms_amd.kernels import ops

    E, top, ff, width, T = sizes
    gen = torch.Generator().manual_seed(ff)
    x = torch.randn(T, width, generator=gen).to(dtype)
    wg, wu = [(torch.randn(E, ff, width, generator=gen) * 2 / math.sqrt(width)).to(dtype) for _ in range(2)]
    wd = (torch.randn(E, width, ff, generator=gen) / math.sqrt(ff)).to(dtype)
    ids = torch.stack([torch.randperm(E, generator=gen)[:top] for _ in range(T)]).to(torch.int32)
    if T > 20:
        ids[:20, 0] = 1  # one expert with more rows than a tile holds
        ids[:20, 1:] = torch.stack([(torch.randperm(E - 1, generator=gen)[: top - 1] + 2) % E for _ in range(20)]).to(torch.int32) if top > 1 else ids[:20, 1:]
    weights = torch.softmax(torch.randn(T, top, generator=gen), -1)
    shared = torch.randn(T, width, generator=gen).to(dtype)
    sgate = torch.randn(T, 3, generator=gen)
    y = ops.moe_experts(x.to(DEV), ids.to(DEV), wg.to(DEV), wu.to(DEV), wd.to(DEV), 1.25, 1.702, 1.0)
    out = ops.moe_combine(y, weights.to(DEV), shared.to(DEV), sgate.to(DEV)[:, 1], dtype)
    want = torch.zeros(T, width)
    xf = x.float()
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            g = (xf[t] @ wg[e].float().T).clamp(max=1.25)
            u = (xf[t] @ wu[e].float().T).clamp(-1.25, 1.25)
            h = g * torch.sigmoid(1.702 * g) * (u + 1)
            if dtype == torch.bfloat16:
                h = h.to(dtype).float()
            want[t] += weights[t, j] * (h @ wd[e].float().T)
    want += torch.sigmoid(sgate[:, 1])[:, None] * shared.float()
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=4e-2, rtol=2e-2)
    torch.testing.assert_close(out.float().cpu(), want, **tol)


# ---- the engine ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_sequence_and_every_layer(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    ids, want = expected_for(folders, name, 150, 1, dtype)
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=256, max_slots=2)
    slot = engine.new_sequence()
    judge(engine.step([slot], [ids], "all"), want, dtype)
    engine.end_sequence(slot)
    engine.cache.check()


@pytest.mark.parametrize("name", ["A", "C"])
def test_the_stream_after_every_layer(lib, folders, name):
    """float32: the residual stream after each layer against the plain implementation's, so that a fault names its layer."""
    from fms_amd.engine import Engine
    from fms_amd.engine.model import DecoderModel

    cfg, weights = plain(folders, name)
    ids = tokens_for(cfg["vocab"], 70, 2)
    _, layers = Z.forward(cfg, weights, ids, return_layers=True)
    model = get(lib, folders, name, "float32")
    seen = []
    blocks = model.layers
    originals = [b.forward for b in blocks]

    def watch(i):
        def forward(stream, batch, cache, act_dtype, next_norm=None):
            originals[i](stream, batch, cache, act_dtype)
            # what is still pending joins the stream in a copy: the stream after this layer
            resid = stream.resid.clone()
            pending, norm = stream.pending, stream.pending_norm
            seen.append(resid.cpu() + Z.rms_norm(pending.float().cpu(), norm.w["weight"].float().cpu(), norm.eps))
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
    assert isinstance(model, DecoderModel) and len(seen) == len(cfg["layers"])
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
    # from the very first token one by one: the first positions of a sequence, where the sink weighs most
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
    """Unequal requests in one batch, decoded together; the short ones end early, their slots and pages go to new
    requests that start while the long one goes on; every request equals itself alone."""
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
            # a batch of its own for the newcomer (the freed slot and pages), then it goes on beside the others
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
def test_a_far_key_decides_in_prompts_and_in_decoding(lib, dtype, tmp_path):
    """Queries scaled up: single keys hold most of a query's weight, many of them hundreds of tokens back and on
    either side of page borders.  A key lost from the cache must fail the same comparison."""
    from fms_amd.engine import Engine

    folder = write_folder(lib, str(tmp_path / "sharp"), CONFIGS["A"], seed=21, sharp=8.0)
    cfg, weights = Z.load_model_folder(folder)
    ids = tokens_for(cfg["vocab"], 600, 3)
    want = expect(cfg, weights, ids, dtype)
    model = lib.get_model("hf_pretrained", model_path=folder, data_type=dtype)
    engine = Engine(model, max_tokens=640, max_slots=1)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:520]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[520:]]
    judge(torch.cat(got), want, dtype)
    engine.end_sequence(slot)
    # sharp indeed, and far: layer 0's heaviest key of the late queries
    m = cfg["layers"][0]["mixer"]
    x = weights["embed"][torch.tensor(ids)] * cfg["embedding"]["scale"]
    h = Z.rms_norm(x, weights["l0.norm1"], cfg["norm"]["eps"])
    pos = torch.arange(len(ids))
    latent, shared = Z.latent_kv(h, weights, "l0.mix.", m, cfg["norm"]["eps"], pos)
    cq = Z.rms_norm(h @ weights["l0.mix.dq"].T, weights["l0.mix.dq.norm"], cfg["norm"]["eps"])
    q = (cq @ weights["l0.mix.uq"].T).view(len(ids), m["heads"], -1)
    kp = (latent @ weights["l0.mix.uk"].T).view(len(ids), m["heads"], m["dim"])
    score = (torch.einsum("thd,shd->hts", q[..., : m["dim"]], kp)
             + torch.einsum("thd,sd->hts", Z.rotate_pairs(q[..., m["dim"]:], pos, m["rot"]["base"], m["rot"]["dims"]), shared)) * m["scale"]
    score = score.masked_fill(pos[None, :] > pos[:, None], float("-inf"))
    prob = torch.softmax(score[:, 520:], -1)
    heavy = prob.max(-1)
    decided = heavy.values > 0.5  # (head, late query) pairs whose weight sits on one key
    assert float(decided.float().mean()) > 0.05 and int((pos[520:][None] - heavy.indices)[decided].max()) > 300
    # negative control: the key that most late queries lean on is taken out of the cache
    lost_key = int(torch.mode(heavy.indices[decided]).values)
    assert lost_key < 520
    slot = engine.new_sequence()
    engine.step([slot], [ids[:520]], "last")
    group = engine.cache.groups[0]
    group.keys[:, group.pages[slot][lost_key // 64], :, lost_key % 64, :] = 0
    lost = torch.cat([engine.step([slot], [[t]], "last") for t in ids[520:]])
    engine.end_sequence(slot)
    with pytest.raises(AssertionError):
        judge(lost, want[520:], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_graphs_and_eager_steps(lib, folders, dtype):
    """300 tokens decoded one by one for three sequences of different lengths, across page borders, as captured graphs
    (fed the plain implementation's tokens through the loop's hook) and as eager steps: the same logits."""
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
    want = [Z.greedy_generate(cfg, weights, p, 12) for p in prompts]
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
    """The package's programs on a Zodolorn folder: the trace replay (float32 and bfloat16, a batch whose requests end
    at different steps) and the registry's view of the architecture."""
    name = "A"
    cfg, weights = plain(folders, name)
    assert "zodolorn" in lib.list_models() and "micro" in lib.list_variants("zodolorn")
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


def test_the_inference_program_on_a_zodolorn_folder(lib, folders):
    """bin/fms_inference with a Zodolorn folder and with a registered variant: the model class comes from config.json or
    from the registry, the text printed is the plain implementation's greedy continuation."""
    from fms_amd.tokenizers import CharTokenizer

    name = "A"  # its vocabulary holds the character tokenizer's
    cfg, weights = plain(folders, name)
    tok = CharTokenizer()
    prompt = [ord(c) for c in "latent keys"]
    new = Z.greedy_generate(cfg, weights, prompt, 12)
    if tok.eos_token_id in new:
        new = new[: new.index(tok.eos_token_id)]
    env = dict(os.environ, PYTHONIOENCODING="utf-8")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "fms_inference"), "--architecture", "hf_pretrained", "--model_path", folders[name],
           "--tokenizer", "char_tokenizer", "--default_dtype", "fp32", "--max_new_tokens", "12", "--prompt_ids", ",".join(map(str, prompt))]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=110, env=env)
    assert proc.returncode == 0, proc.stderr.decode(errors="replace")
    assert tok.decode(prompt + new) in proc.stdout.decode("utf-8")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "fms_inference"), "--architecture", "zodolorn", "--variant", "micro", "--tokenizer",
           "char_tokenizer", "--default_dtype", "bf16", "--max_new_tokens", "5", "--prompt_ids", "1,2,3", "--prompt_ids", "7,8"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=110, env=env)
    assert proc.returncode == 0, proc.stderr.decode(errors="replace")
    assert "loading complete" in proc.stdout.decode("utf-8")


def test_a_model_from_the_registry_alone(lib):
    """A registered variant with random weights runs: configuration -> parts -> engine, no folder."""
    from fms_amd.engine import Engine

    model = lib.get_model("zodolorn", "micro", data_type="bfloat16")
    engine = Engine(model, max_tokens=256, max_slots=2)
    a, b = engine.new_sequence(), engine.new_sequence()
    logits = engine.step([a, b], [list(range(70)), [5, 6, 7]], "last")
    assert logits.shape == (2, model.spec.vocab) and bool(torch.isfinite(logits).all())
    alone = Engine(model, max_tokens=256, max_slots=1)
    s = alone.new_sequence()
    torch.testing.assert_close(alone.step([s], [[5, 6, 7]], "last"), logits[1:], atol=2e-2, rtol=2e-2)
