"""The Basopel configuration: config.json as it is, one entry per layer.

Basopel is a decoder whose layers are listed one by one.  Every entry names its mixer (``type``), the mixer's sizes and
constants (``mixer``) and its feed-forward (``mlp``: ``kind`` "dense", or null for none); ``norm.eps``,
``embedding.scale``, ``vocab`` and ``width`` are the model's own.  The mixers:

* ``attention``: grouped heads, no rotation, a learned bias by bucketed distance (``bias_max``: the distance at which
  the last bucket is reached), a sliding window (``mask.size``) that keeps the sequence's first ``mask.keep_first`` tokens;
* ``attention_2``: grouped heads, rotation of a part of each head (``rot``: ``base``, ``dims``, ``scaling.factor``), capped
  scores (``softcap``), positions cut into chunks of ``mask.size``, a sink in the softmax, a gate per head;
* ``latent_attention``: keys and values as projections of one cached latent (``kv_rank``) plus a rotated key part that all
  heads share (``rot_dim``), a sliding window, a sink, a gate per output element.

``v_mix`` marks the layers whose values are blended with those of the first such layer.  One size is in no key of
config.json but in a tensor's shape: the number of rows of an ``attention`` mixer's distance table.  A model folder's
tensor shapes fill it in (``bias_rows`` in the mixer's entry); a configuration made without a folder carries it itself.
``max_positions`` is this library's bound on a sequence's length (the rotation tables are that long); config.json may
carry it, otherwise the default holds.
"""

from __future__ import annotations

import copy
import dataclasses
from typing import Dict, List, Tuple

from .base import ModelConfig

MIXERS = ("attention", "attention_2", "latent_attention")
MLP_KINDS = ("dense",)
_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "scale", "bias_max"),
    "attention_2": ("heads", "kv_heads", "dim", "vdim", "scale", "rot"),
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"),
}


@dataclasses.dataclass
class BasopelConfig(ModelConfig):
    architecture: str = "Basopel"
    vocab: int = 512
    width: int = 128
    layers: List[dict] = dataclasses.field(default_factory=list)
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-6})
    embedding: dict = dataclasses.field(default_factory=lambda: {"scale": 1.0})
    max_positions: int = 131072

    def __post_init__(self):
        self.validate()

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0:
            raise ValueError("vocab, width and max_positions must be positive")
        if "eps" not in self.norm or "scale" not in self.embedding:
            raise ValueError("the configuration needs norm.eps and embedding.scale")
        mixed_values = None
        for i, layer in enumerate(self.layers):
            kind = layer.get("type")
            if kind not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {kind!r} is not one of {MIXERS}")
            m = layer.get("mixer") or {}
            for key in _KEYS[kind]:
                if key not in m:
                    raise ValueError(f"layer {i}: the mixer lacks {key!r}")
            mask = m.get("mask") or {}
            if mask.get("size", 0) < 0 or mask.get("keep_first", 0) < 0:
                raise ValueError(f"layer {i}: mask.size and mask.keep_first cannot be negative")
            if kind != "latent_attention":
                if m["heads"] <= 0 or m["kv_heads"] <= 0 or m["heads"] % m["kv_heads"]:
                    raise ValueError(f"layer {i}: {m['heads']} query heads are no multiple of {m['kv_heads']} key/value heads")
                if m.get("v_mix"):
                    size = m["kv_heads"] * m["vdim"]
                    if mixed_values is not None and size != mixed_values:
                        raise ValueError(f"layer {i}: layers that mix their values need value rows of one size ({size} here, {mixed_values} before)")
                    mixed_values = size
            if kind == "attention":
                if m["bias_max"] <= 0 or ("bias_rows" in m and (m["bias_rows"] < 2 or m["bias_max"] <= m["bias_rows"] // 2)):
                    raise ValueError(f"layer {i}: the distance table needs at least two rows and a bias_max beyond half of them")
            if "rot" in _KEYS[kind]:
                rot = m["rot"]
                size = m["rot_dim"] if kind == "latent_attention" else m["dim"]
                if "dims" not in rot or "base" not in rot or rot["dims"] % 2 or not 0 < rot["dims"] <= size:
                    raise ValueError(f"layer {i}: the rotation needs a base and an even number of dimensions within {size}")
                if kind == "latent_attention" and rot["dims"] != m["rot_dim"]:
                    raise ValueError(f"layer {i}: the rotation covers {rot['dims']} dimensions, the rotated part has {m['rot_dim']}")
                if (rot.get("scaling") or {}).get("factor", 1.0) <= 0:
                    raise ValueError(f"layer {i}: rot.scaling.factor must be positive")
            mlp = layer.get("mlp")
            if mlp is not None and (mlp.get("kind") not in MLP_KINDS or mlp.get("ff", 0) <= 0):
                raise ValueError(f"layer {i}: the feed-forward needs a kind of {MLP_KINDS} and a positive ff")

    @property
    def nlayers(self) -> int:
        return len(self.layers)

    def with_sizes_from_tensors(self, shapes: Dict[str, Tuple[int, ...]]) -> "BasopelConfig":
        """The configuration with the size that only the checkpoint's tensor shapes give: the rows of every
        ``attention`` mixer's distance table (`l<i>.mix.rel` is [rows, heads])."""
        layers = copy.deepcopy(self.layers)
        for i, layer in enumerate(layers):
            shape = shapes.get(f"l{i}.mix.rel")
            if layer.get("type") == "attention" and shape is not None:
                layer["mixer"]["bias_rows"] = int(shape[0])
        return self.updated(layers=layers)
