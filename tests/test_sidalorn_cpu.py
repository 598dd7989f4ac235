"""Sidalorn without a GPU: configuration, the way from a configuration to parts, the checkpoint adapter, what the
layers ask of the cache and state manager, and the plain implementation's own mechanisms against hand-made cases."""

import math

import pytest
import torch

import fms_amd
import plain_sidalorn as S
from fms_amd.architectures import get_architecture
from fms_amd.architectures.registry import variant_config
from fms_amd.cache import KVNeed, SequenceCache
from fms_amd.engine.model import DecoderModel
from fms_amd.weights.adapters import get_adapter


def _attention(**over):
    m = {"heads": 2, "dim": 8, "vdim": 6, "kv_rank": 10, "scale": 0.3}
    m.update(over)
    return {"type": "latent_attention", "mixer": m}


def _recurrent(**over):
    m = {"width": 12, "blocks": 3, "conv": 3}
    m.update(over)
    return {"type": "rglru", "mixer": m}


def _moe(experts=3, identity=2, top=2, count=1, keep=1, scale=1.0, ff=5, shared=7):
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def _config(**over):
    layers = [
        dict(_recurrent(), mlp={"kind": "dense", "ff": 20}),
        dict(_attention(), mlp=None),
        dict(_attention(heads=3, dim=4, vdim=8, kv_rank=6), mlp=_moe(experts=4, identity=2, top=3, count=3, keep=2, scale=1.5)),
        dict(_recurrent(width=8, blocks=1, conv=2), mlp=_moe(experts=0, identity=4, top=1, shared=0)),
    ]
    kw = dict(vocab=40, width=16, layers=layers, norm={"eps": 1e-5, "groups": 2}, canon={"taps": 3})
    kw.update(over)
    return fms_amd.SidalornConfig(**kw)


def test_the_configuration_round_trips_and_refuses_what_no_model_can_be_built_from(tmp_path):
    config = _config()
    config.save(tmp_path / "config.json")
    again = fms_amd.SidalornConfig.load(tmp_path / "config.json")
    assert again == config and again.nlayers == 4
    bad = [dict(layers=[dict(_attention(), type="convolution", mlp=None)]),
           dict(layers=[dict(_recurrent(width=10, blocks=3), mlp=None)]),
           dict(layers=[{"type": "latent_attention", "mixer": {"heads": 2, "dim": 8}, "mlp": None}]),
           dict(layers=[dict(_attention(), mlp={"kind": "conv"})]),
           dict(layers=[dict(_attention(), mlp=_moe(experts=3, identity=2, top=6))]),
           dict(layers=[dict(_attention(), mlp=_moe(experts=4, identity=2, top=3, count=3, keep=1))]),  # one group of two cannot give three
           dict(layers=[dict(_attention(), mlp=_moe(experts=3, identity=2, top=2, count=2, keep=1))]),  # five outputs in two groups
           dict(norm={"eps": 1e-5, "groups": 3}), dict(norm={"eps": 1e-5}), dict(canon={}), dict(vocab=0)]
    for kw in bad:
        with pytest.raises(ValueError):
            _config(**kw)


def test_from_a_configuration_to_parts_and_what_they_ask_of_the_cache():
    arch = get_architecture("Sidalorn")  # config.json writes the name with a capital
    assert arch.name == "sidalorn"
    config = _config()
    spec = arch.build_spec(config)
    assert [layer.mixer.kind for layer in spec.layers] == ["rglru", "latent_attention", "latent_attention", "rglru"]
    assert [layer.feed_forward.kind if layer.feed_forward else None for layer in spec.layers] == ["mlp", None, "experts", "experts"]
    model = DecoderModel(spec, torch.float32)
    kv, state = model.cache_needs()
    # attention caches one normed latent row per token and no values; every layer keeps the stream's last taps - 1 rows,
    # a recurrent one also its state and its own convolution's last inputs
    assert kv == [(1, KVNeed(1, 10, 0, values=False)), (2, KVNeed(1, 6, 0, values=False))]
    by_entry = {n: {name: (shape, dtype) for name, shape, dtype in need.tensors} for n, need in state}
    assert sorted(by_entry) == [0, 1, 2, 3]
    assert by_entry[0] == {"block.conv": ((2, 16), "float32"), "S": ((12,), "float32"), "conv": ((2, 12), "float32")}
    assert by_entry[1] == {"block.conv": ((2, 16), "float32")}
    assert by_entry[3] == {"block.conv": ((2, 16), "float32"), "S": ((8,), "float32"), "conv": ((1, 8), "float32")}
    names = {n: s.shape for n, s, _, _ in model.named_specs()}
    assert names["l1.mix.down.weight"] == (2 * 8 + 10, 16) and names["l2.mix.down.weight"] == (3 * 4 + 6, 16)
    assert names["l0.mix.in_proj.weight"] == (24, 16) and names["l0.mix.ra.weight"] == (3, 4, 4) and names["l0.canon1"] == (16, 3)
    assert "l1.norm2.weight" not in names and "l1.mlp.up.weight" not in names and names["l0.mlp.act"] == (4,)
    assert names["l2.mlp.router.weight"] == (6, 16) and names["l2.mlp.correction"] == (6,) and names["l2.mlp.experts.down"] == (4, 16, 5)
    assert "l2.mlp.experts.gate" not in names and names["l2.mlp.shared.up.weight"] == (7, 16)
    # identity experts only: a router and a correction, no expert tensors at all
    assert names["l3.mlp.router.weight"] == (4, 16) and not any(n.startswith("l3.mlp.experts") or n.startswith("l3.mlp.shared") for n in names)
    cache = SequenceCache(kv, state, max_tokens=128, max_slots=2, max_seq_len=256, device="cpu")
    assert sorted(g.bytes_per_token(2) for g in cache.groups) == [12, 20]
    a, b = cache.alloc_slot(), cache.alloc_slot()
    assert a != b and cache.state_of_entry(0)["S"].shape == (2, 12) and cache.state_of_entry(1)["block.conv"].shape == (2, 2, 16)
    # a slot that is handed out again starts from zero state
    cache.state_of_entry(0)["S"][a] = 5.0
    cache.state_of_entry(3)["conv"][a] = 7.0
    cache.free_slot(a)
    again = cache.alloc_slot()
    assert again == a and float(cache.state_of_entry(0)["S"][a].abs().max()) == 0.0 and float(cache.state_of_entry(3)["conv"][a].abs().max()) == 0.0


def test_the_checkpoint_adapter_gives_every_parameter_its_tensor():
    config = _config()
    arch = get_architecture("sidalorn")
    layout = arch.hf_tensor_layout(config)
    tensors = {name: torch.full(shape, float(i)) for i, (name, shape, _) in enumerate(layout)}
    adapted = get_adapter("sidalorn", "hf")(tensors, model_config=config)
    model = DecoderModel(arch.build_spec(config), torch.float32)
    expected = {n: s.shape for n, s, _, _ in model.named_specs()}
    assert set(adapted) == set(expected)
    assert all(tuple(adapted[n].shape) == expected[n] for n in expected)
    down = adapted["l1.mix.down.weight"]
    assert torch.equal(down[:16], tensors["l1.mix.q"]) and torch.equal(down[16:], tensors["l1.mix.dkv"])
    both = adapted["l0.mix.in_proj.weight"]
    assert torch.equal(both[:12], tensors["l0.mix.y"]) and torch.equal(both[12:], tensors["l0.mix.x"])
    assert torch.equal(adapted["l0.mix.in_proj.bias"][12:], tensors["l0.mix.x.b"]) and torch.equal(adapted["l0.mix.out.weight"], tensors["l0.mix.o"])
    assert torch.equal(adapted["l2.mlp.experts.up"][1], tensors["l2.mlp.e1.up"]) and torch.equal(adapted["l0.mix.conv.bias"], tensors["l0.mix.conv.b"])
    assert arch.detect_source(list(tensors)) == "hf" and arch.detect_source(list(adapted)) == "fms"


def test_registered_variants_build():
    assert "sidalorn" in fms_amd.list_models() and {"micro", "3b-a1b"} <= set(fms_amd.list_variants("sidalorn"))
    arch = get_architecture("sidalorn")
    for variant in ("micro", "3b-a1b"):
        config = variant_config("sidalorn", variant)
        spec = arch.build_spec(config)
        assert len(spec.layers) == config.nlayers and spec.vocab == config.vocab


# ---- the plain implementation's mechanisms on cases worked by hand ---------------------------------------------------
def test_plain_norm_in_groups_and_convolution():
    v = torch.tensor([[3.0, 4.0, 0.0, 2.0]], dtype=torch.float64)
    w = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=torch.float64)
    got = S.norm_in_groups(v, w, 2, 0.0)
    r1, r2 = math.sqrt(12.5), math.sqrt(2.0)
    torch.testing.assert_close(got, torch.tensor([[3 / r1, 8 / r1, 0.0, 8 / r2]], dtype=torch.float64))
    x = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    k = torch.tensor([[2.0, 3.0, 5.0]], dtype=torch.float64)  # the last column is the token's own
    torch.testing.assert_close(S.convolution_over_time(x, k), torch.tensor([[5.0], [53.0], [532.0]], dtype=torch.float64))


def test_plain_softmax_with_a_sink_and_recurrence():
    scores = torch.zeros(2, 2, dtype=torch.float64)
    p = S.softmax_with_sink(scores, torch.tensor(0.0, dtype=torch.float64))
    torch.testing.assert_close(p, torch.tensor([[0.5, 0.0], [1 / 3, 1 / 3]], dtype=torch.float64))
    a = torch.tensor([[0.5], [0.5], [0.0]], dtype=torch.float64)
    b = torch.tensor([[1.0], [1.0], [7.0]], dtype=torch.float64)
    torch.testing.assert_close(S.linear_recurrence(a, b), torch.tensor([[1.0], [1.5], [7.0]], dtype=torch.float64))


def test_plain_router_keeps_groups_and_weighs_without_the_correction():
    # six outputs in three groups of two, two groups kept; the correction lifts output 4 (group 2) over everything,
    # group 0 holds the largest score; group 1's outputs, second and third by score, cannot be chosen
    logits = torch.log(torch.tensor([[0.30, 0.05, 0.25, 0.20, 0.10, 0.10]], dtype=torch.float64))
    correction = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.5, -0.2], dtype=torch.float64)
    r = {"experts": 4, "identity": 2, "top": 3, "scale": 2.0, "groups": {"count": 3, "keep": 2}}
    ids, weights = S.route(logits, correction, r)
    assert ids[0] == [4, 0, 1]  # 2 and 3 have larger scores than 1, but their group is shut out
    torch.testing.assert_close(weights[0], torch.tensor([0.10, 0.30, 0.05], dtype=torch.float64) / 0.45 * 2.0)
    r["groups"] = {"count": 3, "keep": 3}
    assert S.route(logits, correction, r)[0][0] == [4, 0, 2]
