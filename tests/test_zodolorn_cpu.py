"""Zodolorn without a GPU: configuration, the way from a configuration to parts and a schedule, the checkpoint
adapter, and what the mixer asks of the cache."""

import pytest
import torch

import fms_amd
from fms_amd.architectures import get_architecture
from fms_amd.cache import KVNeed, SequenceCache
from fms_amd.engine.model import DecoderModel
from fms_amd.weights.adapters import get_adapter


def _mixer(**over):
    m = {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 6, "q_rank": 12, "kv_rank": 10, "scale": 0.3, "rot": {"base": 100.0, "dims": 4}}
    m.update(over)
    return m


def _config(**over):
    layers = [
        {"type": "latent_attention", "mixer": _mixer(), "mlp": {"kind": "dense", "ff": 20}},
        {"type": "latent_attention", "mixer": _mixer(kv_from=0), "mlp": None},
        {"type": "latent_attention", "mixer": _mixer(kv_from=0),
         "mlp": {"kind": "moe", "router": {"experts": 3, "top": 2}, "expert": {"ff": 5, "limit": 2.0}, "shared": {"ff": 7, "limit": 1.0}}},
    ]
    kw = dict(vocab=40, width=16, layers=layers, norm={"eps": 1e-5}, embedding={"scale": 4.0})
    kw.update(over)
    return fms_amd.ZodolornConfig(**kw)


def test_the_configuration_round_trips_and_refuses_what_no_model_can_be_built_from(tmp_path):
    config = _config()
    config.save(tmp_path / "config.json")
    again = fms_amd.ZodolornConfig.load(tmp_path / "config.json")
    assert again == config and again.nlayers == 3
    bad = [dict(layers=[{"type": "convolution", "mixer": _mixer(), "mlp": None}]),
           dict(layers=[{"type": "latent_attention", "mixer": _mixer(kv_from=0), "mlp": None}]),
           dict(layers=config.layers[:1] + [{"type": "latent_attention", "mixer": _mixer(kv_from=0, kv_rank=12), "mlp": None}]),
           dict(layers=config.layers[:2] + [{"type": "latent_attention", "mixer": _mixer(kv_from=1), "mlp": None}]),
           dict(layers=[{"type": "latent_attention", "mixer": _mixer(), "mlp": {"kind": "conv"}}]),
           dict(vocab=0), dict(norm={})]
    for kw in bad:
        with pytest.raises(ValueError):
            _config(**kw)


def test_from_a_configuration_to_parts_and_a_schedule():
    arch = get_architecture("Zodolorn")  # config.json writes the name with a capital
    assert arch.name == "zodolorn"
    spec = arch.build_spec(_config())
    assert [e.cache_of for e in spec.resolved_schedule()] == [None, 0, 0]
    assert [layer.feed_forward.kind if layer.feed_forward else None for layer in spec.layers] == ["mlp", None, "experts"]
    model = DecoderModel(spec, torch.float32)
    kv, state = model.cache_needs()
    assert kv == [(0, KVNeed(1, 14, 0, values=False))] and state == []
    names = {n: s.shape for n, s, _, _ in model.named_specs()}
    assert names["l0.mix.down.weight"] == (12 + 2 + 14, 16) and names["l1.mix.down.weight"] == (12 + 2, 16)
    assert "l1.mix.kv_norm.weight" not in names and "l1.norm2.weight" not in names and "l1.mlp.up.weight" not in names
    assert names["l2.mlp.router.weight"] == (4, 16) and names["l2.mlp.experts.down"] == (3, 16, 5)
    # the cache keeps one row per token and layer that owns one, and no values
    cache = SequenceCache(kv, state, max_tokens=128, max_slots=2, max_seq_len=256)
    assert len(cache.groups) == 1 and cache.groups[0].bytes_per_token(2) == 28


def test_the_checkpoint_adapter_gives_every_parameter_its_tensor():
    config = _config()
    arch = get_architecture("zodolorn")
    layout = arch.hf_tensor_layout(config)
    tensors = {name: torch.full(shape, float(i)) for i, (name, shape, _) in enumerate(layout)}
    adapted = get_adapter("zodolorn", "hf")(tensors, model_config=config)
    model = DecoderModel(arch.build_spec(config), torch.float32)
    expected = {n: s.shape for n, s, _, _ in model.named_specs()}
    assert set(adapted) == set(expected)
    assert all(tuple(adapted[n].shape) == expected[n] for n in expected)
    down = adapted["l0.mix.down.weight"]
    assert torch.equal(down[:12], tensors["l0.mix.dq"]) and torch.equal(down[12:14], tensors["l0.mix.g"]) and torch.equal(down[14:], tensors["l0.mix.dkv"])
    assert torch.equal(adapted["l2.mlp.experts.up"][1], tensors["l2.mlp.e1.up"])
    assert torch.equal(adapted["l2.mlp.router.weight"][3:], tensors["l2.mlp.shared.sg"])
    assert arch.detect_source(list(tensors)) == "hf" and arch.detect_source(list(adapted)) == "fms"


def test_a_block_that_norms_its_branches_keeps_the_branch_norm_for_the_next_reader():
    from fms_amd.parts import ResidualStream

    calls = []

    class Norm:
        def add_norm(self, resid, branch, out_dtype, rows=None, branch_norm=None):
            calls.append((branch, branch_norm, rows))
            return "normed"

    stream = ResidualStream(torch.zeros(2, 4))
    post = object()
    stream.add_branch("mixer output", post_norm=post)
    with pytest.raises(RuntimeError):
        stream.add_branch("another", post_norm=post)
    assert stream.normed(Norm(), torch.float32) == "normed" and calls == [("mixer output", post, None)]
    assert stream.pending is None and stream.pending_norm is None
