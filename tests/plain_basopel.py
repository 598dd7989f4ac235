"""A plain, slow Basopel in PyTorch on the CPU: whole sequences, no cache, one function per mechanism.

It is the yardstick of the tests and shares nothing with the library.  `weights` maps the checkpoint's tensor names to
tensors, `config` is the dictionary of config.json.  Everything runs in float64 unless the caller asks for the
roundings of a bfloat16 model (`rounding="bfloat16"`: what a product or an activation leaves is stored in bfloat16;
scores, softmax, norms, angles and the residual sum stay as they are).

Notation: x is the residual stream [T, width]; h what a mixer or a feed-forward reads; i is a query's position, j a
key's, n = i - j their distance.
"""

from __future__ import annotations

import json
import math
import os

import torch

_store = lambda x: x  # noqa: E731


def _bf16(x):
    return x.to(torch.bfloat16).to(x.dtype)


def load_model_folder(folder):
    """(config dictionary, name -> float64 tensor) of a folder with config.json and model.safetensors."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    weights = {k: (v.double() if v.is_floating_point() else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, weights


# ---- norms ---------------------------------------------------------------------------------------------------------
def layer_norm(v, weight, bias, eps):
    mean = v.mean(-1, keepdim=True)
    var = ((v - mean) ** 2).mean(-1, keepdim=True)
    return (v - mean) / torch.sqrt(var + eps) * weight + bias


def rms_norm(v, weight, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


# ---- positions -------------------------------------------------------------------------------------------------------
def rotate_halves(v, positions, rot):
    """v [T, heads, size]: the first rot["dims"] entries of every head turned, entry i paired with entry i + dims/2, by the
    angle position * base^(-2i/dims) / factor."""
    dims = rot["dims"]
    half = dims // 2
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    freqs = torch.tensor([rot["base"] ** (-2.0 * i / dims) / factor for i in range(half)], dtype=torch.float64)
    angle = positions.double()[:, None] * freqs[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b, rest = v[..., :half], v[..., half:dims], v[..., dims:]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)


def distance_bucket(n, rows, far):
    """The row of a learned distance table for distance n >= 0: the distance itself below rows/2, then steps that grow
    with the logarithm and reach the last row at distance `far`."""
    near = rows // 2
    if n < near:
        return n
    return min(rows - 1, near + int(math.floor(math.log(n / near) / math.log(far / near) * (rows - near))))


def distance_bias(T, table, far):
    """[heads, T, T]: table[bucket(i - j), head] for j <= i, zero elsewhere."""
    rows, heads = table.shape
    out = torch.zeros(heads, T, T, dtype=table.dtype)
    by_distance = torch.stack([table[distance_bucket(n, rows, far)] for n in range(T)])  # [T, heads]
    for i in range(T):
        for h in range(heads):
            out[h, i, : i + 1] = by_distance[: i + 1, h].flip(0)
    return out


# ---- which keys a query sees -------------------------------------------------------------------------------------------
def visible_window(T, size, keep_first=0):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def visible_chunk(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def softmax_rows(scores, visible, sink=None):
    """scores [T, T] of one head; keys that are not visible get no weight; with a sink the denominator also holds
    exp(sink), which belongs to no key."""
    s = scores.masked_fill(~visible, float("-inf"))
    top = s.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink)
    e = torch.exp(s - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink - top)
    return e / total


# ---- mixers ------------------------------------------------------------------------------------------------------------
def mix_values(v, w, state):
    """The value mixing across layers: the first layer that mixes keeps its values for the later ones, which blend theirs
    with them by their own lambda."""
    if state.get("first_values") is None:
        state["first_values"] = v
        return v
    lam = w["vmix"]
    return (1 - lam) * v + lam * state["first_values"]


def attention_distance(h, w, m, eps, state):
    """Grouped-head attention without rotation: per-head RMS norm of queries and keys, a learned bias by bucketed
    distance, a sliding window that keeps the first tokens."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = _store(h @ w["q"].T + w["q.b"]).reshape(T, H, D)
    k = _store(h @ w["k"].T + w["k.b"]).reshape(T, G, D)
    v = _store(h @ w["v"].T + w["v.b"])
    q = _store(rms_norm(q, w["q.norm"], eps))
    k = _store(rms_norm(k, w["k.norm"], eps))
    if m.get("v_mix"):
        v = _store(mix_values(v, w, state))
    v = v.reshape(T, G, V)
    bias = distance_bias(T, w["rel"], m["bias_max"])
    visible = visible_window(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"] + bias[head]
        out[:, head] = _store(softmax_rows(s, visible)) @ v[:, g]
    return _store(out.reshape(T, H * V)) @ w["o"].T


def attention_chunked(h, w, m, eps, state, positions):
    """Grouped-head attention inside chunks of positions: RMS norm over the whole query and key projections, partial
    rotation, capped scores, a sink, a gate per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w["q"].T + w["q.b"], w["q.norm"], eps)
    k = rms_norm(h @ w["k"].T + w["k.b"], w["k.norm"], eps)
    v = _store(h @ w["v"].T + w["v.b"])
    q = _store(rotate_halves(_store(q).reshape(T, H, D), positions, m["rot"]))
    k = _store(rotate_halves(_store(k).reshape(T, G, D), positions, m["rot"]))
    if m.get("v_mix"):
        v = _store(mix_values(v, w, state))
    v = v.reshape(T, G, V)
    visible = visible_chunk(T, m["mask"]["size"])
    gate = torch.sigmoid(h @ w["g"].T)  # [T, H]
    cap = m.get("softcap")  # a configuration without one leaves the scores as they are
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        p = _store(softmax_rows(s, visible, w["sink"][head]))
        out[:, head] = (p @ v[:, g]) * gate[:, head : head + 1]
    return _store(out.reshape(T, H * V)) @ w["o"].T + w["o.b"]


def latent_attention(h, w, m, eps, positions):
    """Attention whose keys and values are projections of one normed latent per token, plus one rotated key part that all
    heads share; a sliding window, a sink, a gate per output element."""
    T = h.shape[0]
    H, D, P, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = _store(h @ w["q"].T).reshape(T, H, D + P)
    down = h @ w["dkv"].T
    c = _store(rms_norm(down[:, :R], w["dkv.norm"], eps))
    shared = _store(rotate_halves(down[:, None, R:], positions, m["rot"]))[:, 0]  # [T, P]
    q_rot = _store(rotate_halves(q[..., D:], positions, m["rot"]))
    keys = (c @ w["uk"].T).reshape(T, H, D)
    values = (c @ w["uv"].T).reshape(T, H, V)
    visible = visible_window(T, m["mask"]["size"])
    gate = torch.sigmoid(h @ w["g"].T)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for head in range(H):
        s = (q[:, head, :D] @ keys[:, head].T + q_rot[:, head] @ shared.T) * m["scale"]
        out[:, head] = _store(softmax_rows(s, visible, w["sink"][head])) @ values[:, head]
    return _store(out.reshape(T, H * V) * gate) @ w["o"].T


def gated_feed_forward(h, w):
    return _store(gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


# ---- the model -----------------------------------------------------------------------------------------------------------
def under(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config, weights, ids, rounding=None, layers_out=None):
    """Logits [T, vocab] of one sequence of token ids; `layers_out` (a list) receives the stream after every layer."""
    global _store
    _store = _bf16 if rounding == "bfloat16" else (lambda t: t)
    try:
        eps = config["norm"]["eps"]
        ids = torch.as_tensor(ids, dtype=torch.long)
        positions = torch.arange(len(ids))
        x = weights["embed"][ids] * config["embedding"]["scale"]
        state = {}
        for i, layer in enumerate(config["layers"]):
            p = f"l{i}."
            norm = lambda name, t: layer_norm(t, weights[p + name], weights[p + name + ".b"], eps)  # noqa: E731
            h = _store(norm("norm1", x))
            w, m = under(weights, p + "mix."), layer["mixer"]
            if layer["type"] == "attention":
                y = attention_distance(h, w, m, eps, state)
            elif layer["type"] == "attention_2":
                y = attention_chunked(h, w, m, eps, state, positions)
            elif layer["type"] == "latent_attention":
                y = latent_attention(h, w, m, eps, positions)
            else:
                raise ValueError(layer["type"])
            x = x + norm("norm1b", _store(y))
            if layer.get("mlp") is not None:
                h = _store(norm("norm2", x))
                x = x + norm("norm2b", _store(gated_feed_forward(h, under(weights, p + "mlp."))))
            if layers_out is not None:
                layers_out.append(x.clone())
        h = _store(layer_norm(x, weights["final.norm"], weights["final.norm.b"], eps))
        return h @ weights["embed"].T
    finally:
        _store = lambda t: t  # noqa: E731


def greedy_generate(config, weights, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(config, weights, ids)[-1].argmax()))
    return ids[len(prompt):]
