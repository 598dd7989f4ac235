"""A plain, slow Sidalorn in PyTorch on the CPU: whole sequences, no cache, no state, one function per mechanism.

It is the yardstick of the tests and shares nothing with the library.  `weights` maps the checkpoint's tensor names to
tensors, `config` is the dictionary of config.json.  Everything runs in float64 unless the caller says otherwise.

Notation: x is the residual stream [T, width]; h what a mixer or a feed-forward reads; taps are counted so that the
last column of a convolution's weight belongs to the token itself.
"""

from __future__ import annotations

import json
import math
import os

import torch

# What a product's or an activation's result is stored as.  Identity for the exact run; a round trip through bfloat16
# for the run that shows what bfloat16 storage costs (scores, softmax, norms, routers, the residual sum and everything
# behind the recurrent block's projection stay as they are: the design computes them in 32-bit).
_store = lambda x: x  # noqa: E731
# When a list: every mixture-of-experts layer appends, per token, by how much the last chosen output's choice score
# leads the best one not chosen (inf when all are chosen), and the last kept group the best one shut out, in units of
# the scores involved (about the change of a logit that turns the choice).  A small number marks a choice that rounding
# can turn: such a token's logits are no test of arithmetic.
router_margins = None

DECAY_CONSTANT = 8.0


def _bf16(x):
    return x.to(torch.bfloat16).to(x.dtype)


def load_model_folder(folder):
    """(config dictionary, name -> float64 tensor) of a folder with config.json and model.safetensors."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    weights = {k: (v.double() if v.is_floating_point() else v) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, weights


def root_mean_square_norm(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def norm_in_groups(v, weight, groups, eps):
    """Every row cut into `groups` equal consecutive parts, each divided by its own root mean square; then the weight."""
    T, W = v.shape
    parts = root_mean_square_norm(v.reshape(T, groups, W // groups), eps)
    return parts.reshape(T, W) * weight


def convolution_over_time(v, weight, bias=None):
    """out[t, c] = sum_j weight[c, j] v[t - taps + 1 + j, c], zeros before the sequence's start."""
    T, C = v.shape
    taps = weight.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=v.dtype), v])
    out = torch.zeros_like(v)
    for j in range(taps):
        out = out + padded[j : j + T] * weight[:, j]
    return out if bias is None else out + bias


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2)))


def softmax_with_sink(scores, sink):
    """scores [T, T] of one head (row i: query i), causal; the denominator also holds exp(sink)."""
    T = scores.shape[0]
    visible = torch.tril(torch.ones(T, T, dtype=torch.bool))
    s = scores.masked_fill(~visible, float("-inf"))
    top = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))


def latent_attention(h, w, m, eps):
    """Attention without positions: queries straight from h, keys and values expanded from one normed latent per token."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = _store(h @ w["q"].T).reshape(T, H, D)
    latent = _store(root_mean_square_norm(h @ w["dkv"].T, eps) * w["dkv.norm"])
    k = (latent @ w["uk"].T).reshape(T, H, D)
    v = (latent @ w["uv"].T).reshape(T, H, V)
    heads = []
    for a in range(H):
        p = softmax_with_sink((q[:, a] @ k[:, a].T) * m["scale"], w["sink"][a])
        heads.append(p @ v[:, a])
    return _store(_store(torch.cat(heads, dim=-1)) @ w["o"].T)


def recurrence_gates(u, w, m):
    """(a, b) of the recurrence S <- a S + b from the convolved branch u [T, C]."""
    T, C = u.shape
    B = m["blocks"]
    ub = u.reshape(T, B, C // B)
    r = torch.sigmoid(torch.einsum("bok,tbk->tbo", w["ra"], ub) + w["ra.b"]).reshape(T, C)
    i = torch.sigmoid(torch.einsum("bok,tbk->tbo", w["ri"], ub) + w["ri.b"]).reshape(T, C)
    a = torch.exp(-DECAY_CONSTANT * r * torch.nn.functional.softplus(w["lam"]))
    return a, torch.sqrt(1 - a * a) * i * u


def linear_recurrence(a, b):
    """S_t = a_t S_(t-1) + b_t from S = 0, token by token."""
    S = torch.zeros_like(a[0])
    out = []
    for t in range(a.shape[0]):
        S = a[t] * S + b[t]
        out.append(S)
    return torch.stack(out)


def recurrent_block(h, w, m):
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = convolution_over_time(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    a, b = recurrence_gates(u, w, m)
    return _store(_store(linear_recurrence(a, b) * y) @ w["o"].T)


def poly_norm(z, coefficients, eps):
    a, b, c, e = (float(v) for v in coefficients)
    return a * root_mean_square_norm(z, eps) + b * root_mean_square_norm(z ** 2, eps) + c * root_mean_square_norm(z ** 3, eps) + e


def dense_feed_forward(h, w, eps):
    return _store(_store(poly_norm(h @ w["up"].T, w["act"], eps)) @ w["down"].T)


def route(logits, correction, r):
    """(ids [T, top], weights [T, top]) from router logits over experts and identity experts together."""
    n = logits.shape[1]
    scores = torch.softmax(logits, dim=-1)
    choice = scores + correction
    groups = r.get("groups") or {"count": 1, "keep": 1}
    G, keep, per = groups["count"], groups["keep"], n // groups["count"]
    ids, weights = [], []
    for t in range(logits.shape[0]):
        group_score = choice[t].reshape(G, per).max(-1).values
        order = sorted(range(G), key=lambda g: (-float(group_score[g]), g))
        allowed = torch.full((n,), float("-inf"), dtype=logits.dtype)
        for g in order[:keep]:
            allowed[g * per : (g + 1) * per] = choice[t, g * per : (g + 1) * per]
        picked = sorted(range(n), key=lambda e: (-float(allowed[e]), e))[: r["top"]]
        if router_margins is not None:
            # how far the logits can move before the choice turns: a score moves by about itself times the change of
            # its logit, so a gap between two choice scores is measured in units of the two scores behind them
            def lead(x, y):
                return float((choice[t, x] - choice[t, y]) / (scores[t, x] + scores[t, y]))

            rest = [e for e in range(n) if e not in picked and allowed[e] > float("-inf")]
            gap = min((lead(picked[-1], e) for e in rest), default=float("inf"))
            if keep < G:
                best = [max(range(g * per, (g + 1) * per), key=lambda e: float(choice[t, e])) for g in order]
                gap = min(gap, min(lead(best[keep - 1], e) for e in best[keep:]))
            router_margins[-1].append(gap)
        s = scores[t, picked]
        ids.append(picked)
        weights.append(s / (s.sum() + 1e-20) * r.get("scale", 1.0))
    return ids, weights


def expert(h, up, down):
    return _store(_store(gelu_erf(h @ up.T)) @ down.T)


def experts_feed_forward(h, w, mlp):
    r = mlp["router"]
    E = r["experts"]
    logits = h @ w["router"].T
    if router_margins is not None:
        router_margins.append([])
    ids, weights = route(logits, w["correction"], r)
    rows = []
    for t in range(h.shape[0]):
        acc = torch.zeros_like(h[t])
        for e, weight in zip(ids[t], weights[t]):
            acc = acc + weight * (h[t] if e >= E else expert(h[t], w[f"e{e}.up"], w[f"e{e}.down"]))
        rows.append(acc)
    out = torch.stack(rows)
    if mlp.get("shared"):
        out = out + expert(h, w["shared.up"], w["shared.down"])
    return _store(out)


def under(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(config, weights, ids, rounding=None, layers_out=None, margins=None):
    """Logits [T, vocab] of one sequence.  rounding "bfloat16": products and activations are stored in bfloat16, as a
    bfloat16 model stores them.  layers_out: a list that receives the stream after every layer.  margins: a list that
    receives, for every mixture-of-experts layer, a tensor [T] of how clear each token's routing was."""
    global _store, router_margins
    _store = _bf16 if rounding == "bfloat16" else (lambda x: x)
    router_margins = [] if margins is not None else None
    try:
        eps, groups = config["norm"]["eps"], config["norm"]["groups"]
        x = weights["embed"][torch.tensor(ids)].double()
        for i, layer in enumerate(config["layers"]):
            w = under(weights, f"l{i}.")
            h = _store(x + convolution_over_time(x, w["canon1"]))
            if layer["type"] == "latent_attention":
                mixed = latent_attention(h, under(w, "mix."), layer["mixer"], eps)
            else:
                mixed = recurrent_block(h, under(w, "mix."), layer["mixer"])
            x = x + norm_in_groups(mixed, w["norm1"], groups, eps)
            mlp = layer.get("mlp")
            if mlp is not None:
                h = _store(x)
                f = dense_feed_forward(h, under(w, "mlp."), eps) if mlp["kind"] == "dense" else experts_feed_forward(h, under(w, "mlp."), mlp)
                x = x + norm_in_groups(f, w["norm2"], groups, eps)
            if layers_out is not None:
                layers_out.append(x.clone())
        return (_store(norm_in_groups(x, weights["final.norm"], groups, eps)) @ weights["head"].T).float()
    finally:
        _store = lambda x: x  # noqa: E731
        if margins is not None:
            margins.extend(torch.tensor(m, dtype=torch.float64) for m in router_margins)
        router_margins = None


def greedy_generate(config, weights, prompt, n_new):
    """The n_new tokens that follow `prompt` when the likeliest token is taken every time."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(config, weights, ids)[-1])))
    return ids[len(prompt):]
