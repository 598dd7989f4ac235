"""The Sidalorn configuration: config.json as it is, one entry per layer.

Sidalorn is a decoder whose layers are listed one by one.  Every entry names its mixer (``type``: "latent_attention",
attention without positions over a cached latent, or "rglru", a recurrent block with a real-gated linear recurrent
unit), the mixer's sizes (``mixer``) and its feed-forward (``mlp``: ``kind`` "dense" or "moe", or null for none).
``norm.eps`` and ``norm.groups`` (every norm of the model splits its row into that many parts), ``canon.taps`` (the
short convolution on every mixer's input), ``vocab`` and ``width`` are the model's own.  Nothing is derived: every size
is read.  ``max_positions`` is this library's bound on a sequence's length; config.json may carry it, otherwise the
default holds.
"""

from __future__ import annotations

import dataclasses
from typing import List

from .base import ModelConfig

MIXERS = ("latent_attention", "rglru")
MLP_KINDS = ("dense", "moe")
_MIXER_KEYS = {"latent_attention": ("heads", "dim", "vdim", "kv_rank", "scale"), "rglru": ("width", "blocks", "conv")}


@dataclasses.dataclass
class SidalornConfig(ModelConfig):
    architecture: str = "Sidalorn"
    vocab: int = 512
    width: int = 128
    layers: List[dict] = dataclasses.field(default_factory=list)
    norm: dict = dataclasses.field(default_factory=lambda: {"eps": 1e-6, "groups": 1})
    canon: dict = dataclasses.field(default_factory=lambda: {"taps": 4})
    max_positions: int = 131072

    def __post_init__(self):
        self.validate()

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0:
            raise ValueError("vocab, width and max_positions must be positive")
        if "eps" not in self.norm or "groups" not in self.norm:
            raise ValueError("the configuration needs norm.eps and norm.groups")
        if self.norm["groups"] <= 0 or self.width % self.norm["groups"]:
            raise ValueError(f"{self.norm['groups']} norm groups do not divide the width {self.width}")
        if self.canon.get("taps", 0) <= 0:
            raise ValueError("the configuration needs a positive canon.taps")
        for i, layer in enumerate(self.layers):
            kind = layer.get("type")
            if kind not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {kind!r} is not one of {MIXERS}")
            m = layer.get("mixer") or {}
            for key in _MIXER_KEYS[kind]:
                if key not in m:
                    raise ValueError(f"layer {i}: the mixer lacks {key!r}")
            if kind == "rglru" and (m["blocks"] <= 0 or m["width"] % m["blocks"]):
                raise ValueError(f"layer {i}: {m['width']} channels do not split into {m['blocks']} equal blocks")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if mlp.get("kind") not in MLP_KINDS:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not one of {MLP_KINDS}")
            if mlp["kind"] == "dense":
                if mlp.get("ff", 0) <= 0:
                    raise ValueError(f"layer {i}: the dense feed-forward needs ff")
                continue
            r = mlp.get("router") or {}
            outputs = r.get("experts", 0) + r.get("identity", 0)
            groups = r.get("groups") or {"count": 1, "keep": 1}
            if r.get("experts", 0) and "ff" not in (mlp.get("expert") or {}):
                raise ValueError(f"layer {i}: the experts need expert.ff")
            if not 0 < r.get("top", 0) <= outputs:
                raise ValueError(f"layer {i}: router.top must lie within the {outputs} experts and identity experts")
            if groups["count"] <= 0 or outputs % groups["count"] or not 0 < groups["keep"] <= groups["count"] \
                    or groups["keep"] * (outputs // groups["count"]) < r["top"]:
                raise ValueError(f"layer {i}: {groups['count']} groups over {outputs} router outputs, {groups['keep']} kept, cannot give {r['top']} choices")

    @property
    def nlayers(self) -> int:
        return len(self.layers)
