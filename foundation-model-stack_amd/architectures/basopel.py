"""Basopel: from its configuration to parts, and from its checkpoint's tensor names to the model's.

The model: a token embedding times a constant; layers in the order config.json lists them, each a block whose branches
pass a layer norm (weight and shift) on both sides; three kinds of attention as mixers (see config/basopel.py); a gated
feed-forward with the tanh form of gelu, or none; a final layer norm and a head that is the embedding table itself.

A checkpoint names a layer's tensors ``l<i>.<part>`` without a ".weight" and a shift or bias ``<tensor>.b``; the adapter
gives them the model's names and fuses what the model runs as one product (everything that reads a mixer's input; gate
and up rows of the feed-forward).  The checkpoint pairs rotated dimension i of a head with dimension i + dims/2; the
rotation kernels turn neighbouring pairs, so the adapter moves row i of a head's rotated run to row 2i and row
i + dims/2 to row 2i + 1, in queries and keys alike (a score is a sum over dimensions, and a norm over a whole projection
a sum of squares: neither cares about the order, as long as weights, biases and norm weights move together).
"""

from __future__ import annotations

import re
from typing import List, Tuple

import torch

from ..config import BasopelConfig
from ..parts import LayerSpec, ModelSpec, PartSpec
from ..weights.adapters import register_adapter, register_adapter_step
from .registry import Architecture, register_architecture, register_model

NAME = "basopel"
ACTIVATION = "gelu-tanh"  # the design fixes the feed-forward's activation


def _rope_key(rot: dict, size: int) -> str:
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    return f"rope_{size}_{rot['dims']}_{rot['base']!r}_{factor!r}"


def _rope_spec(rot: dict, size: int, max_positions: int) -> PartSpec:
    args = {"dim": size, "rot_dim": rot["dims"], "theta": rot["base"], "max_seq_len": max_positions, "exact_frequencies": True}
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    if factor != 1.0:
        args["scaling"] = {"rope_type": "linear", "factor": factor}
    return PartSpec("rope", args)


def _value_mix(config: BasopelConfig, i: int):
    """None, "first" (the first layer that mixes values: it hands its own on) or "blend"."""
    if not config.layers[i]["mixer"].get("v_mix"):
        return None
    earlier = any(l["mixer"].get("v_mix") and l["type"] != "latent_attention" for l in config.layers[:i])
    return "blend" if earlier else "first"


def basopel_spec(config: BasopelConfig) -> ModelSpec:
    eps = config.norm["eps"]
    norm = PartSpec("layernorm", {"eps": eps})
    layers, positions = [], {}
    for i, layer in enumerate(config.layers):
        m, kind, key = layer["mixer"], layer["type"], None
        mask = m.get("mask") or {}
        if kind == "latent_attention":
            key = _rope_key(m["rot"], m["rot_dim"])
            positions.setdefault(key, _rope_spec(m["rot"], m["rot_dim"], config.max_positions))
            mixer = PartSpec("latent_attention", {
                "nheads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"], "q_rank": 0, "kv_rank": m["kv_rank"],
                "scale": m["scale"], "eps": eps, "sink": True, "output_gate": "element", "window": mask.get("size", 0),
            })
        else:
            args = {"nheads": m["heads"], "kvheads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"], "qkv_bias": True,
                    "norm_eps": eps, "scale_factor": m["scale"], "value_mix": _value_mix(config, i)}
            if kind == "attention":
                if "bias_rows" not in m:
                    raise ValueError(f"layer {i}: the distance table's rows (bias_rows) come from a model folder's tensor shapes; "
                                     "a configuration made without one must carry them")
                args.update(out_bias=False, qk_norm="head", window=mask.get("size", 0), keep_first=mask.get("keep_first", 0),
                            distance_bias={"rows": m["bias_rows"], "far": m["bias_max"]})
            else:
                key = _rope_key(m["rot"], m["dim"])
                positions.setdefault(key, _rope_spec(m["rot"], m["dim"], config.max_positions))
                args.update(out_bias=True, qk_norm="projection", chunk=mask.get("size", 0), soft_cap=m.get("softcap", 0.0),
                            sink=True, output_gate="head")
            mixer = PartSpec("attention", args)
        mlp = layer.get("mlp")
        ff = PartSpec("glu", {"hidden_dim": mlp["ff"], "activation": ACTIVATION}) if mlp is not None else None
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, block=PartSpec("sandwich_norm"), position=key))
    return ModelSpec(
        vocab=config.vocab, width=config.width, max_seq_len=config.max_positions, layers=layers, final_norm=norm,
        embedding=PartSpec("table", {"scale": config.embedding["scale"]}), positions=positions, tie_heads=True,
        embedding_name="embed", layer_name="l{i}", final_norm_name="final.norm", head_name="head",
    )


# ---- the checkpoint's names -> the model's ----------------------------------------------------------------------
def pairs_to_neighbours(t: torch.Tensor, heads: int, offset: int, dims: int) -> torch.Tensor:
    """Rows of `heads` equal heads: in every head the run of `dims` rows from `offset` on is reordered so that row i and
    row i + dims/2 of the run become rows 2i and 2i + 1."""
    size = t.shape[0] // heads
    rest = t.shape[1:]
    v = t.reshape(heads, size, *rest)
    run = v[:, offset : offset + dims].reshape(heads, 2, dims // 2, *rest).transpose(1, 2).reshape(heads, dims, *rest)
    return torch.cat([v[:, :offset], run, v[:, offset + dims :]], dim=1).reshape(t.shape)


def _layer_of(name: str, model_config) -> dict:
    return model_config.layers[int(re.match(r"l(\d+)\.", name).group(1))]


def _to_model_names(sd, model_config=None, **kw):
    out = dict(sd)
    for name in [n for n in out if n.endswith(".mix.dkv")]:  # latent attention
        p = name[: -len("dkv")]
        m = _layer_of(name, model_config)["mixer"]
        H, D, P, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
        q = pairs_to_neighbours(out.pop(p + "q"), H, D, P)
        dkv = out.pop(p + "dkv")
        dkv = torch.cat([dkv[:R], pairs_to_neighbours(dkv[R:], 1, 0, P)], dim=0)
        out[p + "down.weight"] = torch.cat([q, out.pop(p + "g"), dkv], dim=0)
        for src, dst in (("dkv.norm", "kv_norm.weight"), ("uk", "uk.weight"), ("uv", "uv.weight"), ("o", "o.weight")):
            out[p + dst] = out.pop(p + src)
    for name in [n for n in out if n.endswith(".mix.k")]:  # the two kinds with key and value heads
        p = name[: -len("k")]
        layer = _layer_of(name, model_config)
        m = layer["mixer"]
        parts = {n: out.pop(p + n) for n in ("q", "k", "v")}
        biases = {n: out.pop(p + n + ".b") for n in ("q", "k", "v")}
        norms = {n: out.pop(p + n + ".norm") for n in ("q", "k")}
        if layer["type"] == "attention_2":
            dims = m["rot"]["dims"]
            for n, heads in (("q", m["heads"]), ("k", m["kv_heads"])):
                parts[n] = pairs_to_neighbours(parts[n], heads, 0, dims)
                biases[n] = pairs_to_neighbours(biases[n], heads, 0, dims)
                norms[n] = pairs_to_neighbours(norms[n], heads, 0, dims)
            gate = out.pop(p + "g")
            weights = [parts["q"], parts["k"], parts["v"], gate]
            bias = [biases["q"], biases["k"], biases["v"], torch.zeros(gate.shape[0], dtype=gate.dtype)]
            out[p + "dense.bias"] = out.pop(p + "o.b")
        else:
            weights, bias = [parts["q"], parts["k"], parts["v"]], [biases["q"], biases["k"], biases["v"]]
        out[p + "in_proj.qkv_fused.weight"] = torch.cat(weights, dim=0)
        out[p + "in_proj.qkv_fused.bias"] = torch.cat(bias, dim=0)
        out[p + "q_norm.weight"], out[p + "k_norm.weight"] = norms["q"], norms["k"]
        out[p + "dense.weight"] = out.pop(p + "o")
    for name in [n for n in out if n.endswith(".mlp.gate")]:
        p = name[: -len("gate")]
        out[p + "wg1_fused.weight"] = torch.cat([out.pop(p + "gate"), out.pop(p + "up")], dim=0)
        out[p + "w2.weight"] = out.pop(p + "down")
    renamed = {}
    for name, t in out.items():
        if re.search(r"(^final\.norm|\.norm[12]b?)\.b$", name):
            name = name[: -len(".b")] + ".bias"
        elif re.search(r"(^embed|^final\.norm|\.norm[12]b?)$", name):
            name += ".weight"
        renamed[name] = t
    return renamed


register_adapter_step(NAME, "checkpoint_to_model_names", _to_model_names)
register_adapter(NAME, "hf", ["checkpoint_to_model_names"])


def detect_source(names: List[str]) -> str:
    return "fms" if any(n.endswith(".weight") for n in names) else "hf"


def checkpoint_tensor_layout(config: BasopelConfig) -> List[Tuple[str, Tuple[int, ...], str]]:
    """(name, shape, init) of every tensor of a Basopel checkpoint of this configuration."""
    W = config.width
    out = [("embed", (config.vocab, W), "normal")]

    def norm(name):
        return [(name, (W,), "ones"), (name + ".b", (W,), "zeros")]

    for i, layer in enumerate(config.layers):
        p, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        out += norm(p + "norm1") + norm(p + "norm1b")
        q = p + "mix."
        if kind == "latent_attention":
            H, D, P, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out += [(q + "q", (H * (D + P), W), "normal"), (q + "dkv", (R + P, W), "normal"), (q + "dkv.norm", (R,), "ones"),
                    (q + "uk", (H * D, R), "normal"), (q + "uv", (H * V, R), "normal"), (q + "sink", (H,), "normal"),
                    (q + "g", (H * V, W), "normal"), (q + "o", (W, H * V), "normal")]
        else:
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            per_head = kind == "attention"
            out += [(q + "q", (H * D, W), "normal"), (q + "q.b", (H * D,), "zeros"), (q + "k", (G * D, W), "normal"), (q + "k.b", (G * D,), "zeros"),
                    (q + "v", (G * V, W), "normal"), (q + "v.b", (G * V,), "zeros"),
                    (q + "q.norm", (D if per_head else H * D,), "ones"), (q + "k.norm", (D if per_head else G * D,), "ones")]
            if per_head:
                out.append((q + "rel", (m["bias_rows"], H), "normal"))
            if m.get("v_mix"):
                out.append((q + "vmix", (), "normal"))
            if not per_head:
                out += [(q + "sink", (H,), "normal"), (q + "g", (H, W), "normal")]
            out.append((q + "o", (W, H * V), "normal"))
            if not per_head:
                out.append((q + "o.b", (W,), "zeros"))
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out += norm(p + "norm2") + norm(p + "norm2b")
        out += [(p + "mlp.gate", (mlp["ff"], W), "normal"), (p + "mlp.up", (mlp["ff"], W), "normal"), (p + "mlp.down", (W, mlp["ff"]), "normal")]
    out += norm("final.norm")
    return out


register_architecture(
    Architecture(
        name=NAME,
        config_class=BasopelConfig,
        build_spec=basopel_spec,
        hf_architectures=(),
        from_hf_dict=BasopelConfig.from_dict,
        to_hf_dict=lambda config: {k: v for k, v in config.as_dict().items()},
        hf_tensor_layout=checkpoint_tensor_layout,
        detect_source=detect_source,
        sizes_from_tensors=lambda config, shapes: config.with_sizes_from_tensors(shapes),
    )
)


def make_config(width: int, vocab: int, pattern: str, heads: int, kv_heads: int, dim: int, vdim: int, ff: int, chunk: int = 1024,
                window: int = 1024, keep_first: int = 4, bias_rows: int = 32, bias_max: int = 0, rot_dims: int = 0, rot_base: float = 10000.0,
                rot_factor: float = 1.0, softcap: float = 30.0, latent_dim: int = 0, latent_rot: int = 0, latent_vdim: int = 0,
                kv_rank: int = 0, latent_window: int = 1024, v_mix: bool = True, max_positions: int = 131072) -> BasopelConfig:
    """A regular Basopel: `pattern` has a letter per layer, "c" for attention in chunks, "w" for windowed attention with a
    distance bias, "l" for latent attention; all layers of a kind share their sizes."""
    layers = []
    mlp = {"kind": "dense", "ff": ff} if ff else None
    for letter in pattern:
        if letter == "c":
            rot = {"base": rot_base, "dims": rot_dims or dim}
            if rot_factor != 1.0:
                rot["scaling"] = {"factor": rot_factor}
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk}, "rot": rot,
                     "scale": dim ** -0.5, "softcap": softcap, "v_mix": v_mix}
            layers.append({"type": "attention_2", "mixer": mixer, "mlp": mlp})
        elif letter == "w":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window, "keep_first": keep_first},
                     "scale": dim ** -0.5, "bias_max": bias_max or window, "bias_rows": bias_rows, "v_mix": v_mix}
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        elif letter == "l":
            d, p = latent_dim or dim, latent_rot or max(2, dim // 2)
            mixer = {"heads": heads, "dim": d, "rot_dim": p, "vdim": latent_vdim or vdim, "kv_rank": kv_rank or 4 * dim,
                     "mask": {"size": latent_window}, "rot": {"base": rot_base, "dims": p}, "scale": (d + p) ** -0.5}
            layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
        else:
            raise ValueError(f"layer letter {letter!r} is not 'c', 'w' or 'l'")
    return BasopelConfig(vocab=vocab, width=width, layers=layers, norm={"eps": 1e-6}, embedding={"scale": width ** 0.5},
                         max_positions=max_positions)


def _variant(config: BasopelConfig):
    def factory(**overrides) -> BasopelConfig:
        return config.updated(**overrides)

    return factory


register_model(NAME, "micro", _variant(make_config(width=256, vocab=1024, pattern="ccwlc", heads=4, kv_heads=2, dim=64, vdim=64, ff=512,
                                                   chunk=128, window=160, latent_window=96, rot_dims=32, kv_rank=64, latent_dim=32,
                                                   latent_rot=16, max_positions=4096)))
register_model(NAME, "3b", _variant(make_config(width=2048, vocab=65536, pattern="ccwlc" * 5, heads=16, kv_heads=4, dim=128, vdim=128, ff=8192,
                                                chunk=2048, window=1024, kv_rank=512, latent_rot=64)))
