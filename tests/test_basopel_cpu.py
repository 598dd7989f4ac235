"""Basopel without a GPU: configuration, the way from a configuration to parts, the checkpoint adapter, what the layers
ask of the cache (kept first pages, chunks that give pages back), and the plain implementation's own mechanisms against
hand-made cases."""

import math

import pytest
import torch

import fms_amd
import plain_basopel as P
from fms_amd.architectures import get_architecture
from fms_amd.architectures.basopel import pairs_to_neighbours
from fms_amd.architectures.registry import variant_config
from fms_amd.cache import KVNeed, SequenceCache
from fms_amd.engine.model import DecoderModel
from fms_amd.parts.attention import distance_buckets
from fms_amd.parts.position import rope_frequencies
from fms_amd.weights.adapters import get_adapter


def _chunked(**over):
    m = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "mask": {"size": 10}, "rot": {"base": 100.0, "dims": 4, "scaling": {"factor": 2.0}},
         "scale": 0.3, "softcap": 5.0, "v_mix": True}
    m.update(over)
    return {"type": "attention_2", "mixer": m}


def _windowed(**over):
    m = {"heads": 3, "kv_heads": 1, "dim": 6, "vdim": 12, "mask": {"size": 70, "keep_first": 65}, "scale": 0.3, "bias_max": 9, "bias_rows": 6,
         "v_mix": True}
    m.update(over)
    return {"type": "attention", "mixer": m}


def _latent(**over):
    m = {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 10, "mask": {"size": 12}, "rot": {"base": 50.0, "dims": 4}, "scale": 0.3}
    m.update(over)
    return {"type": "latent_attention", "mixer": m}


def _config(**over):
    layers = [dict(_chunked(), mlp={"kind": "dense", "ff": 20}), dict(_windowed(), mlp=None), dict(_latent(), mlp={"kind": "dense", "ff": 12}),
              dict(_chunked(heads=2, kv_heads=2, vdim=5, v_mix=False, mask={"size": 200}), mlp={"kind": "dense", "ff": 8})]
    kw = dict(vocab=40, width=16, layers=layers, norm={"eps": 1e-5}, embedding={"scale": 4.0}, max_positions=512)
    kw.update(over)
    return fms_amd.BasopelConfig(**kw)


def test_the_configuration_round_trips_and_refuses_what_no_model_can_be_built_from(tmp_path):
    config = _config()
    config.save(tmp_path / "config.json")
    again = fms_amd.BasopelConfig.load(tmp_path / "config.json")
    assert again == config and again.nlayers == 4
    bad = [dict(layers=[dict(_chunked(), type="convolution", mlp=None)]),
           dict(layers=[dict(_chunked(heads=3), mlp=None)]),                                        # heads no multiple of key/value heads
           dict(layers=[{"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 8}, "mlp": None}]),
           dict(layers=[dict(_chunked(rot={"base": 10.0, "dims": 10}), mlp=None)]),                   # rotation wider than the head
           dict(layers=[dict(_latent(rot={"base": 10.0, "dims": 2}), mlp=None)]),                     # rotation and rotated part differ
           dict(layers=[dict(_chunked(), mlp=None), dict(_windowed(vdim=7), mlp=None)]),              # mixed values of two sizes
           dict(layers=[dict(_windowed(bias_rows=1), mlp=None)]),
           dict(layers=[dict(_chunked(), mlp={"kind": "moe", "ff": 4})]),
           dict(norm={}), dict(embedding={}), dict(vocab=0)]
    for kw in bad:
        with pytest.raises(ValueError):
            _config(**kw)
    # the distance table's rows come from the tensor shapes of a model folder
    bare = _config(layers=[dict({"type": "attention", "mixer": {k: v for k, v in _windowed()["mixer"].items() if k != "bias_rows"}}, mlp=None)])
    with pytest.raises(ValueError):
        get_architecture("basopel").build_spec(bare)
    filled = bare.with_sizes_from_tensors({"l0.mix.rel": (14, 3)})
    assert filled.layers[0]["mixer"]["bias_rows"] == 14 and "bias_rows" not in bare.layers[0]["mixer"]


def test_from_the_configuration_to_parts_and_what_they_ask_of_the_cache():
    arch = get_architecture("Basopel")  # as config.json writes it
    config = _config()
    spec = arch.build_spec(config)
    assert spec.tie_heads and spec.embedding.args["scale"] == 4.0 and spec.final_norm.kind == "layernorm"
    kinds = [(l.mixer.kind, l.block.kind, l.feed_forward.kind if l.feed_forward else None) for l in spec.layers]
    assert kinds == [("attention", "sandwich_norm", "glu"), ("attention", "sandwich_norm", None), ("latent_attention", "sandwich_norm", "glu"),
                     ("attention", "sandwich_norm", "glu")]
    a, b, c, d = (l.mixer.args for l in spec.layers)
    assert (a["value_mix"], b["value_mix"], d["value_mix"]) == ("first", "blend", None)
    assert a["chunk"] == 10 and a["sink"] and a["output_gate"] == "head" and a["qk_norm"] == "projection" and a["soft_cap"] == 5.0 and a["out_bias"]
    assert b["window"] == 70 and b["keep_first"] == 65 and b["qk_norm"] == "head" and b["distance_bias"] == {"rows": 6, "far": 9} and not b["out_bias"]
    assert c["window"] == 12 and c["output_gate"] == "element" and c["q_rank"] == 0 and c["sink"]
    assert spec.layers[1].position is None and len(spec.positions) == 2  # the two layers in chunks share one rotation table
    assert all(l.feed_forward is None or l.feed_forward.args["activation"] == "gelu-tanh" for l in spec.layers)
    model = DecoderModel(spec, torch.float32, config=config)
    kv, state = model.cache_needs()
    assert state == []
    assert [need for _, need in kv] == [
        KVNeed(2, 8, 0, value_dim=6, chunk=10), KVNeed(1, 6, 70, value_dim=12, keep_first=65), KVNeed(1, 14, 12, values=False),
        KVNeed(2, 8, 0, value_dim=5, chunk=200)]
    names = {n for n, *_ in model.named_specs()}
    for n in ("embed.weight", "l0.norm1.bias", "l0.mix.in_proj.qkv_fused.bias", "l0.mix.sink", "l0.mix.vmix", "l0.mix.dense.bias", "l1.mix.rel",
              "l1.mix.vmix", "l1.mix.q_norm.weight", "l2.mix.down.weight", "l2.mix.sink", "l3.mlp.wg1_fused.weight", "final.norm.bias"):
        assert n in names, n
    assert "l3.mix.vmix" not in names and "l1.mix.dense.bias" not in names and "l1.norm2.weight" not in names
    assert variant_config("basopel", "micro").nlayers == 5


def test_the_adapter_gives_every_tensor_its_place():
    config = _config()
    arch = get_architecture("basopel")
    layout = arch.hf_tensor_layout(config)
    gen = torch.Generator().manual_seed(0)
    sd = {name: torch.randn(shape, generator=gen) for name, shape, _ in layout}
    out = get_adapter("basopel", "hf")(dict(sd), model_config=config)
    model = DecoderModel(arch.build_spec(config), torch.float32, config=config)
    expected = {full: spec.shape for full, spec, _, _ in model.named_specs() if full not in model.tied}
    assert {n: tuple(t.shape) for n, t in out.items()} == expected
    # layer 0 turns 4 of a head's 8 dimensions: rows 0, 2, 1, 3 of every head's rotated run, then the rest as they were
    q = out["l0.mix.in_proj.qkv_fused.weight"][:32].view(4, 8, 16)
    src = sd["l0.mix.q"].view(4, 8, 16)
    assert torch.equal(q[:, :4], src[:, [0, 2, 1, 3]]) and torch.equal(q[:, 4:], src[:, 4:])
    qn = out["l0.mix.q_norm.weight"].view(4, 8)
    assert torch.equal(qn[:, :4], sd["l0.mix.q.norm"].view(4, 8)[:, [0, 2, 1, 3]])
    bias = out["l0.mix.in_proj.qkv_fused.bias"]
    assert torch.equal(bias[32:48].view(2, 8)[:, :4], sd["l0.mix.k.b"].view(2, 8)[:, [0, 2, 1, 3]]) and bool((bias[-4:] == 0).all())
    assert torch.equal(out["l0.mix.in_proj.qkv_fused.weight"][-4:], sd["l0.mix.g"])
    # the windowed layer turns nothing
    assert torch.equal(out["l1.mix.in_proj.qkv_fused.weight"], torch.cat([sd["l1.mix.q"], sd["l1.mix.k"], sd["l1.mix.v"]]))
    # the latent layer: the rotated run of every query head, and the shared key part behind the latent
    down = out["l2.mix.down.weight"]
    assert torch.equal(down[:24].view(2, 12, 16)[:, 8:], sd["l2.mix.q"].view(2, 12, 16)[:, [8, 10, 9, 11]])
    assert torch.equal(down[24:36], sd["l2.mix.g"]) and torch.equal(down[36:46], sd["l2.mix.dkv"][:10])
    assert torch.equal(down[46:], sd["l2.mix.dkv"][[10, 12, 11, 13]])
    assert torch.equal(out["l3.mlp.wg1_fused.weight"], torch.cat([sd["l3.mlp.gate"], sd["l3.mlp.up"]]))
    t = torch.arange(12.0).view(12, 1)
    assert pairs_to_neighbours(t, 2, 1, 4).flatten().tolist() == [0, 1, 3, 2, 4, 5, 6, 7, 9, 8, 10, 11]


def test_turning_neighbours_equals_turning_halves():
    """What the adapter's reordering rests on: a head whose rows were moved, turned in neighbouring pairs, gives the same
    scores as the head as stored, turned in halves."""
    gen = torch.Generator().manual_seed(1)
    rot = {"base": 100.0, "dims": 6, "scaling": {"factor": 4.0}}
    q, k = torch.randn(5, 1, 10, generator=gen, dtype=torch.float64), torch.randn(5, 1, 10, generator=gen, dtype=torch.float64)
    pos = torch.tensor([0, 3, 4, 90, 1000])
    want = (P.rotate_halves(q, pos, rot) * P.rotate_halves(k, pos, rot)).sum(-1)
    freqs = rope_frequencies(6, 100.0, {"rope_type": "linear", "factor": 4.0}, exact=True).double()
    assert torch.allclose(freqs, torch.tensor([100.0 ** (-2 * i / 6) / 4 for i in range(3)], dtype=torch.float64), rtol=1e-7)

    def neighbours(v):
        v = pairs_to_neighbours(v[:, 0].T.contiguous(), 1, 0, 6).T  # rows of a weight are a vector's entries
        angle = pos.double()[:, None] * freqs[None, :]
        a, b = v[:, 0:6:2], v[:, 1:6:2]
        turned = torch.stack([a * torch.cos(angle) - b * torch.sin(angle), b * torch.cos(angle) + a * torch.sin(angle)], dim=-1).reshape(5, 6)
        return torch.cat([turned, v[:, 6:]], dim=1)

    assert torch.allclose((neighbours(q) * neighbours(k)).sum(-1), want[:, 0], atol=1e-9)


def test_kept_first_pages_stay_and_chunks_give_pages_back():
    needs = [(0, KVNeed(1, 8, 70, keep_first=65)), (1, KVNeed(1, 8, 0, chunk=100)), (2, KVNeed(1, 8, 30))]
    cache = SequenceCache(needs, [], max_tokens=64 * 12, max_slots=2, max_seq_len=4096)
    slot = cache.alloc_slot()
    cache.extend(slot, 300)
    cache.check()
    cache.extend(slot, 1)  # the step's first query sits at position 300
    kept, chunks, plain_window = (cache.groups[i] for i in range(3))
    # window 70 from position 300: keys 231.. are seen, so pages 0..2 could go; the first 65 tokens (two pages) stay
    assert [p >= 0 for p in kept.pages[slot]] == [True, True, False, True, True]
    # chunks of 100: position 300 starts a chunk, pages before 300 // 64 go
    assert [p >= 0 for p in chunks.pages[slot]] == [False, False, False, False, True]
    assert [p >= 0 for p in plain_window.pages[slot]] == [False, False, False, False, True]
    cache.check()
    before = cache.pages_held(slot)
    cache.extend(slot, 200)
    cache.extend(slot, 1)
    assert [p >= 0 for p in kept.pages[slot]][:7] == [True, True, False, False, False, False, True]
    assert cache.pages_held(slot) != before or True
    table = cache.block_table(0, [slot])
    assert table[0, 0] >= 0 and table[0, 1] >= 0 and table[0, 2] == -1
    cache.check()
    other = cache.alloc_slot()
    cache.extend(other, 64 * 3)  # pages that were given back serve another sequence
    cache.check()
    cache.free_slot(slot)
    cache.free_slot(other)
    cache.check()
    assert all(g.pool.n_held == 0 for g in cache.groups)
    # a sequence shorter than its kept run never gives anything back
    slot = cache.alloc_slot()
    for _ in range(40):
        cache.extend(slot, 1)
    assert all(p >= 0 for p in kept.pages[slot])
    cache.check()


def test_the_plain_mechanisms_on_cases_worked_by_hand():
    # buckets: 8 rows, far 20: distances 0..3 are their own rows; 4 -> 4; then log steps; 20 and beyond -> 7
    assert [P.distance_bucket(n, 8, 20) for n in (0, 1, 3, 4, 5, 19, 20, 500)] == [0, 1, 3, 4, 4 + int(math.log(5 / 4) / math.log(5) * 4), 7, 7, 7]
    assert distance_buckets(8, 20)[:5] == [0, 1, 2, 3, 4]
    # masks
    w = P.visible_window(6, 2, keep_first=1)
    assert w[5].tolist() == [True, False, False, False, True, True] and w[1].tolist() == [True, True, False, False, False, False]
    c = P.visible_chunk(7, 3)
    assert c[4].tolist() == [False, False, False, True, True, False, False] and c[6].tolist() == [False] * 6 + [True]
    # a sink as large as the only key's score takes half the weight
    s = torch.tensor([[2.0]], dtype=torch.float64)
    assert torch.allclose(P.softmax_rows(s, torch.ones(1, 1, dtype=torch.bool), torch.tensor(2.0, dtype=torch.float64)), torch.tensor([[0.5]], dtype=torch.float64))
    # layer norm: the variance is the mean of the squared deviations
    v = torch.tensor([[1.0, 3.0]], dtype=torch.float64)
    assert torch.allclose(P.layer_norm(v, torch.tensor([2.0, 2.0]), torch.tensor([0.5, 0.5]), 0.0), torch.tensor([[-1.5, 2.5]], dtype=torch.float64))
    # rotation in halves by a quarter turn: (u, v) -> (-v, u)
    rot = {"base": 1.0, "dims": 2, "scaling": {"factor": 1.0}}
    x = torch.tensor([[[1.0, 2.0, 7.0]]], dtype=torch.float64)
    quarter = P.rotate_halves(x, torch.tensor([math.pi / 2]), rot)
    assert torch.allclose(quarter, torch.tensor([[[-2.0, 1.0, 7.0]]], dtype=torch.float64), atol=1e-12)
    # value mixing: the first layer hands on, the next blends
    state = {}
    first = P.mix_values(torch.tensor([1.0]), {"vmix": torch.tensor(0.9)}, state)
    assert first.item() == 1.0 and P.mix_values(torch.tensor([3.0]), {"vmix": torch.tensor(0.25)}, state).item() == 2.5
