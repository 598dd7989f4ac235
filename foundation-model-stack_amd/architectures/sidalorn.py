"""Sidalorn: from its configuration to parts, and from its checkpoint's tensor names to the model's.

The model: a token embedding; layers in the order config.json lists them, each a block whose norms sit behind its
branches only (x += norm1(mixer(x + conv(x))); x += norm2(ff(x))), every norm an RMS norm in groups, the mixer's input
passed through a short causal convolution on the stream's channels; the mixer is attention without positions over a
cached latent, with a sink in the softmax, or a recurrent block with a real-gated linear recurrent unit; the
feed-forward is a plain one with a PolyNorm activation, a mixture of gelu experts routed in groups (with identity
experts, a choice correction and a shared expert), or absent; a final norm and a linear head.

A checkpoint names a layer's tensors ``l<i>.<part>`` without a ".weight"; the adapter gives them the model's names
and fuses what the model runs as one product (everything that reads a mixer's input; the experts stacked per layer).
"""

from __future__ import annotations

import re
from typing import List, Tuple

import torch

from ..config import SidalornConfig
from ..parts import LayerSpec, ModelSpec, PartSpec
from ..weights.adapters import register_adapter, register_adapter_step
from .registry import Architecture, register_architecture, register_model

NAME = "sidalorn"
# what the design fixes: the constant in the recurrence's decay, log a = -DECAY_CONSTANT * r * softplus(lam); the
# activation of the recurrent block's gate branch; the experts' activation
DECAY_CONSTANT = 8.0
RECURRENT_ACTIVATION = "gelu-tanh"
EXPERT_ACTIVATION = "gelu"


def _mixer_spec(layer: dict, eps: float) -> PartSpec:
    m = layer["mixer"]
    if layer["type"] == "latent_attention":
        return PartSpec("latent_attention", {
            "nheads": m["heads"], "dim": m["dim"], "rot_dim": 0, "vdim": m["vdim"], "q_rank": 0, "kv_rank": m["kv_rank"],
            "scale": m["scale"], "eps": eps, "sink": True, "output_gate": False,
        })
    return PartSpec("rglru", {"channels": m["width"], "blocks": m["blocks"], "conv": m["conv"], "decay_constant": DECAY_CONSTANT,
                              "activation": RECURRENT_ACTIVATION})


def _feed_forward_spec(mlp, eps: float):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartSpec("mlp", {"hidden_dim": mlp["ff"], "activation": "polynorm", "eps": eps})
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    shared = mlp.get("shared") or {}
    return PartSpec("experts", {
        "experts": r["experts"], "top": r["top"], "hidden_dim": (mlp.get("expert") or {}).get("ff", 0), "limit": None,
        "expert_gate": False, "activation": EXPERT_ACTIVATION, "score": "softmax_all", "identity": r.get("identity", 0),
        "correction": True, "groups": groups["count"], "keep": groups["keep"], "route_scale": r.get("scale", 1.0),
        "shared_hidden_dim": shared.get("ff", 0), "shared_gate": False,
    })


def sidalorn_spec(config: SidalornConfig) -> ModelSpec:
    eps = config.norm["eps"]
    norm = PartSpec("rmsnorm", {"eps": eps, "groups": config.norm["groups"]})
    block = PartSpec("post_norm", {"width": config.width, "input_taps": config.canon["taps"]})
    layers = [LayerSpec(mixer=_mixer_spec(layer, eps), feed_forward=_feed_forward_spec(layer.get("mlp"), eps), norm=norm, block=block)
              for layer in config.layers]
    return ModelSpec(
        vocab=config.vocab, width=config.width, max_seq_len=config.max_positions, layers=layers, final_norm=norm,
        embedding_name="embed", layer_name="l{i}", final_norm_name="final.norm", head_name="head",
    )


# ---- the checkpoint's names -> the model's ----------------------------------------------------------------------
_EXPERT = re.compile(r"^(l\d+\.mlp)\.e(\d+)\.(up|down)$")
_RENAMES = (  # checkpoint suffix -> model suffix, for tensors that keep their shape
    ("mix.dkv.norm", "mix.kv_norm.weight"), ("mix.uk", "mix.uk.weight"), ("mix.uv", "mix.uv.weight"), ("mix.o", "mix.o.weight"),
    ("mix.conv", "mix.conv.weight"), ("mix.conv.b", "mix.conv.bias"), ("mix.ra", "mix.ra.weight"), ("mix.ra.b", "mix.ra.bias"),
    ("mix.ri", "mix.ri.weight"), ("mix.ri.b", "mix.ri.bias"), ("mlp.router", "mlp.router.weight"),
    ("mlp.shared.up", "mlp.shared.up.weight"), ("mlp.shared.down", "mlp.shared.down.weight"), ("mlp.up", "mlp.up.weight"),
    ("mlp.down", "mlp.down.weight"), ("norm1", "norm1.weight"), ("norm2", "norm2.weight"),
)


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
    layers = sorted({n.split(".", 1)[0] for n in out if re.match(r"^l\d+\.", n)})
    for p in layers:
        if f"{p}.mix.q" in out:  # attention: queries and the latent's down-projection are one product
            out[f"{p}.mix.down.weight"] = torch.cat([out.pop(f"{p}.mix.q"), out.pop(f"{p}.mix.dkv")], dim=0)
        if f"{p}.mix.y" in out:  # the recurrent block: both branches are one product, the output projection is `out`
            out[f"{p}.mix.in_proj.weight"] = torch.cat([out.pop(f"{p}.mix.y"), out.pop(f"{p}.mix.x")], dim=0)
            out[f"{p}.mix.in_proj.bias"] = torch.cat([out.pop(f"{p}.mix.y.b"), out.pop(f"{p}.mix.x.b")], dim=0)
            out[f"{p}.mix.out.weight"] = out.pop(f"{p}.mix.o")
        for src, dst in _RENAMES:
            if f"{p}.{src}" in out:
                out[f"{p}.{dst}"] = out.pop(f"{p}.{src}")
    for name in ("embed", "head", "final.norm"):
        if name in out:
            out[name + ".weight"] = out.pop(name)
    return out


register_adapter_step(NAME, "checkpoint_to_model_names", _to_model_names)
register_adapter(NAME, "hf", ["checkpoint_to_model_names"])


def detect_source(names: List[str]) -> str:
    return "fms" if any(n.endswith(".weight") for n in names) else "hf"


def checkpoint_tensor_layout(config: SidalornConfig) -> List[Tuple[str, Tuple[int, ...], str]]:
    """(name, shape, init) of every tensor of a Sidalorn checkpoint of this configuration."""
    W = config.width
    out = [("embed", (config.vocab, W), "normal")]
    for i, layer in enumerate(config.layers):
        p, m = f"l{i}.", layer["mixer"]
        out.append((p + "norm1", (W,), "ones"))
        if layer["type"] == "latent_attention":
            H, D, V, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
            out += [(p + "mix.q", (H * D, W), "normal"), (p + "mix.dkv", (R, W), "normal"), (p + "mix.dkv.norm", (R,), "ones"),
                    (p + "mix.uk", (H * D, R), "normal"), (p + "mix.uv", (H * V, R), "normal"), (p + "mix.sink", (H,), "normal"),
                    (p + "mix.o", (W, H * V), "normal")]
        else:
            C, B = m["width"], m["blocks"]
            n = C // B
            out += [(p + "mix.y", (C, W), "normal"), (p + "mix.y.b", (C,), "zeros"), (p + "mix.x", (C, W), "normal"),
                    (p + "mix.x.b", (C,), "zeros"), (p + "mix.conv", (C, m["conv"]), "normal"), (p + "mix.conv.b", (C,), "zeros"),
                    (p + "mix.ra", (B, n, n), "normal"), (p + "mix.ra.b", (B, n), "zeros"), (p + "mix.ri", (B, n, n), "normal"),
                    (p + "mix.ri.b", (B, n), "zeros"), (p + "mix.lam", (C,), "normal"), (p + "mix.o", (W, C), "normal")]
        mlp = layer.get("mlp")
        if mlp is not None:
            out.append((p + "norm2", (W,), "ones"))
            if mlp["kind"] == "dense":
                out += [(p + "mlp.up", (mlp["ff"], W), "normal"), (p + "mlp.down", (W, mlp["ff"]), "normal"), (p + "mlp.act", (4,), "ones")]
            else:
                r = mlp["router"]
                F = (mlp.get("expert") or {}).get("ff", 0)
                for e in range(r["experts"]):
                    out += [(p + f"mlp.e{e}.up", (F, W), "normal"), (p + f"mlp.e{e}.down", (W, F), "normal")]
                outputs = r["experts"] + r.get("identity", 0)
                out += [(p + "mlp.router", (outputs, W), "normal"), (p + "mlp.correction", (outputs,), "zeros")]
                if mlp.get("shared"):
                    S = mlp["shared"]["ff"]
                    out += [(p + "mlp.shared.up", (S, W), "normal"), (p + "mlp.shared.down", (W, S), "normal")]
        out.append((p + "canon1", (W, config.canon["taps"]), "normal"))
    out += [("final.norm", (W,), "ones"), ("head", (config.vocab, W), "normal")]
    return out


register_architecture(
    Architecture(
        name=NAME,
        config_class=SidalornConfig,
        build_spec=sidalorn_spec,
        hf_architectures=(),
        from_hf_dict=SidalornConfig.from_dict,
        to_hf_dict=lambda config: config.as_dict(),
        hf_tensor_layout=checkpoint_tensor_layout,
        detect_source=detect_source,
    )
)


def make_config(width: int, vocab: int, pattern: str, heads: int, dim: int, vdim: int, kv_rank: int, recurrent_width: int, blocks: int,
                dense_ff: int, experts: int = 0, top: int = 0, expert_ff: int = 0, identity: int = 0, shared_ff: int = 0,
                group_count: int = 1, group_keep: int = 1, route_scale: float = 1.0, conv: int = 4, taps: int = 4, norm_groups: int = 1,
                eps: float = 1e-5, dense_layers: int = 1, max_positions: int = 131072) -> SidalornConfig:
    """A regular Sidalorn: `pattern` names every layer's mixer ("a": attention over the latent, "r": the recurrent block);
    the first `dense_layers` layers have the plain feed-forward, the others experts (if there are any)."""
    layers = []
    for i, kind in enumerate(pattern):
        if kind == "a":
            entry = {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": dim ** -0.5}}
        elif kind == "r":
            entry = {"type": "rglru", "mixer": {"width": recurrent_width, "blocks": blocks, "conv": conv}}
        else:
            raise ValueError(f"pattern letter {kind!r} is neither 'a' nor 'r'")
        if i < dense_layers or not (experts or identity):
            entry["mlp"] = {"kind": "dense", "ff": dense_ff}
        else:
            entry["mlp"] = {"kind": "moe", "expert": {"ff": expert_ff},
                            "router": {"experts": experts, "identity": identity, "top": top, "scale": route_scale,
                                       "groups": {"count": group_count, "keep": group_keep}}}
            if shared_ff:
                entry["mlp"]["shared"] = {"ff": shared_ff}
        layers.append(entry)
    return SidalornConfig(vocab=vocab, width=width, layers=layers, norm={"eps": eps, "groups": norm_groups}, canon={"taps": taps},
                          max_positions=max_positions)


def _variant(config: SidalornConfig):
    def factory(**overrides) -> SidalornConfig:
        return config.updated(**overrides)

    return factory


register_model(NAME, "micro", _variant(make_config(width=192, vocab=1024, pattern="araa", heads=6, dim=32, vdim=48, kv_rank=64,
                                                   recurrent_width=256, blocks=4, dense_ff=512, experts=6, top=3, expert_ff=128,
                                                   identity=3, shared_ff=192, group_count=3, group_keep=2, route_scale=1.5,
                                                   norm_groups=2, max_positions=4096)))
register_model(NAME, "3b-a1b", _variant(make_config(width=2048, vocab=65536, pattern="aar" * 8, heads=16, dim=128, vdim=128, kv_rank=512,
                                                    recurrent_width=2560, blocks=10, dense_ff=8192, experts=28, top=6, expert_ff=1024,
                                                    identity=4, shared_ff=2048, group_count=4, group_keep=2, route_scale=2.0,
                                                    norm_groups=4)))
