"""Basopel on the GPU against the plain implementation (plain_basopel.py): every mechanism alone, then the engine
whole / token by token / in portions / in ragged batches with reused slots / through graphs and the generation loop,
in float32 and bfloat16, at sizes that differ from one another in everything.

bfloat16 is judged like the other models of this folder: the plain implementation run with bfloat16 storage shows what
that type costs at every position, and the engine may be a small multiple of that off."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_basopel as P  # noqa: E402
from gpu_checks import Expected  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
BF16_MARGIN = 3.0
BF16_MEAN_MARGIN = 1.5


def chunked(heads, kv, dim, vdim, size, rot_dims, base=10000.0, factor=None, scale=0.2, softcap=15.0, v_mix=False):
    rot = {"base": base, "dims": rot_dims}
    if factor:
        rot["scaling"] = {"factor": factor}
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": {"size": size}, "rot": rot, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention_2", "mixer": m}


def windowed(heads, kv, dim, vdim, size, keep, rows, far, scale=0.2, v_mix=False):
    mask = {"size": size}
    if keep is not None:
        mask["keep_first"] = keep
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "mask": mask, "scale": scale, "bias_max": far, "bias_rows": rows}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot, vdim, rank, size, base=10000.0, scale=0.25):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "mask": {"size": size},
                                                  "rot": {"base": base, "dims": rot}, "scale": scale}}


def layer(mixer, ff):
    return dict(mixer, mlp={"kind": "dense", "ff": ff} if ff else None)


CONFIGS = {
    # values of another size than keys; the values mixed across three layers of both kinds (key/value heads times value
    # size agree, the head counts do not); a part of every head rotated, stretched positions; a layer without a
    # feed-forward; a layer in chunks that does not mix its values; kept first tokens
    "A": dict(vocab=300, width=128, norm={"eps": 1e-5}, embedding={"scale": 7.0}, max_positions=1024, layers=[
        layer(chunked(4, 2, 32, 24, 40, 16, factor=2.0, v_mix=True), 160),
        layer(windowed(4, 1, 16, 48, 50, 3, 8, 20, v_mix=True), None),
        layer(latent(2, 16, 8, 20, 24, 30), 96),
        layer(chunked(6, 3, 24, 16, 25, 24, base=1000.0, softcap=9.0, v_mix=True), 64),
        layer(chunked(2, 2, 40, 8, 70, 8, softcap=30.0), 48),
    ]),
    # sizes that are no multiples of 8 (rows that the matrix instructions cannot load); the first mixing layer is a
    # windowed one; a window of five tokens that keeps one; chunks of seven; no stretching; as many key/value heads as heads
    "B": dict(vocab=257, width=100, norm={"eps": 1e-6}, embedding={"scale": 1.0}, max_positions=1024, layers=[
        layer(windowed(3, 3, 20, 12, 5, 1, 6, 9, v_mix=True), 60),
        layer(chunked(3, 1, 20, 36, 7, 4, base=500.0, softcap=8.0, v_mix=True), 36),
        layer(latent(3, 12, 4, 8, 20, 9, base=1e6), 44),
    ]),
    # sizes at which bfloat16 runs the matrix-instruction kernels; chunks of two pages; a window that keeps more than a
    # page of first tokens; a latent of the matrix-core kernel's sizes; a head size of 128 with chunks of one page, no cap
    "C": dict(vocab=512, width=256, norm={"eps": 1e-6}, embedding={"scale": 16.0}, max_positions=2048, layers=[
        layer(chunked(8, 2, 64, 64, 128, 32, base=500000.0, factor=8.0, softcap=30.0, v_mix=True), 512),
        layer(windowed(8, 2, 64, 64, 100, 70, 32, 128, v_mix=True), 256),
        layer(latent(4, 32, 16, 64, 64, 64), 256),
        layer(chunked(2, 2, 128, 128, 64, 64, softcap=None), 128),
    ]),
    # the other head sizes with matrix-instruction kernels of their own: 32 and 96; one key/value head; a window without
    # kept tokens and a bias that reaches its last row early; chunks longer than any test sequence
    "D": dict(vocab=400, width=192, norm={"eps": 1e-6}, embedding={"scale": 3.0}, max_positions=2048, layers=[
        layer(chunked(8, 1, 32, 32, 1000, 32, softcap=10.0, v_mix=True), 128),
        layer(windowed(2, 1, 96, 32, 130, None, 4, 3, v_mix=True), 96),
        layer(chunked(2, 2, 96, 96, 33, 48, factor=4.0, softcap=12.0), 64),
        layer(latent(2, 64, 32, 32, 128, 200, base=100.0), None),
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
    """A model folder with random weights in which every learned number matters: norm weights and shifts away from one
    and zero, biases, sinks, distance tables and blending factors of some size, gates away from one half.
    sharp: a factor on the queries, so that single keys hold most of a query's weight."""
    from fms_amd.weights import write_safetensors

    lib.write_model_folder(folder, lib.BasopelConfig(**cfg_kw), seed=seed, architecture="basopel", std=0.08)
    cfg, tensors = P.load_model_folder(folder)
    gen = torch.Generator().manual_seed(seed)

    def noise(t, std):
        return torch.randn(t.shape, generator=gen, dtype=torch.float64) * std

    for k in list(tensors):
        t = tensors[k]
        if k.endswith((".norm1", ".norm2", ".norm1b", ".norm2b", "final.norm", ".q.norm", ".k.norm", ".dkv.norm")):
            tensors[k] = 1 + noise(t, 0.2)
        elif k.endswith((".norm1.b", ".norm2.b", ".norm1b.b", ".norm2b.b", "final.norm.b")):
            tensors[k] = noise(t, 0.2)
        elif k.endswith((".q.b", ".k.b", ".v.b", ".o.b")):
            tensors[k] = noise(t, 0.3)
        elif k.endswith(".sink"):
            tensors[k] = noise(t, 1.5)
        elif k.endswith(".rel"):
            tensors[k] = noise(t, 1.0)
        elif k.endswith(".vmix"):
            tensors[k] = torch.rand((), generator=gen, dtype=torch.float64) * 0.6 + 0.2
        elif k.endswith(".mix.g"):
            tensors[k] = t * 4
    if sharp != 1.0:
        for i, entry in enumerate(cfg["layers"]):
            if entry["type"] == "latent_attention":
                tensors[f"l{i}.mix.q"] = tensors[f"l{i}.mix.q"] * sharp
            else:  # the queries are normed, so their size is their norm weight's
                tensors[f"l{i}.mix.q.norm"] = tensors[f"l{i}.mix.q.norm"] * sharp
    tensors = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory, lib):
    return {name: write_folder(lib, str(tmp_path_factory.mktemp(f"basopel_{name}")), kw, 3 + i) for i, (name, kw) in enumerate(CONFIGS.items())}


_models, _plain, _expected = {}, {}, {}


def get(lib, folders, name, dtype):
    if (name, dtype) not in _models:
        _models[(name, dtype)] = lib.get_model("hf_pretrained", model_path=folders[name], data_type=dtype)
    return _models[(name, dtype)]


def plain(folders, name):
    if name not in _plain:
        _plain[name] = P.load_model_folder(folders[name])
    return _plain[name]


def tokens_for(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def expect(cfg, weights, ids, dtype) -> Expected:
    """Exact logits; for bfloat16 also the plain implementation's own error with bfloat16 storage at every position, and
    its 90th percentile over the sequence."""
    exact = P.forward(cfg, weights, ids).float()
    if dtype == "float32":
        return Expected(exact)
    rounded = P.forward(cfg, weights, ids, rounding="bfloat16").float()
    error = (rounded - exact).abs().amax(dim=-1)
    return Expected(exact, error, torch.quantile(error, 0.9).expand_as(error))


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
        torch.testing.assert_close(got, want.logits, atol=3e-4, rtol=1e-3)
        return
    error = (got - want.logits).abs().amax(dim=-1).flatten()
    ref, typical = want.ref_error.flatten(), want.typical.flatten()
    allowed = BF16_MARGIN * torch.maximum(ref, typical)
    worst = int(torch.argmax(error / allowed))
    assert bool((error <= allowed).all()), (
        f"bfloat16 logits are {float(error[worst]):.4g} off at row {worst}; the plain implementation with bfloat16 storage is "
        f"{float(ref[worst]):.4g} off there and typically {float(typical[worst]):.4g} (allowed: {BF16_MARGIN} times the larger)")
    if error.numel() >= 32:
        assert float(error.mean()) <= BF16_MEAN_MARGIN * float(ref.mean()), (
            f"bfloat16 logits are {float(error.mean()):.4g} off on average, the plain implementation with bfloat16 storage {float(ref.mean()):.4g}")


# ---- mechanisms alone ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [100, 128, 257, 320, 4096, 5000])
def test_layer_norms_on_both_sides_of_a_branch(lib, dtype, width):
    """stream += LN_b(branch); out = LN(stream), also for chosen rows only (which must leave the stream alone), with a
    mean far from zero (the deviations, not the squares, must be summed) and with one side an RMS norm."""
    from fms_amd.kernels import ops

    gen = torch.Generator().manual_seed(width)
    T = 9
    resid = torch.randn(T, width, generator=gen) * 3 + 50.0
    branch = (torch.randn(T, width, generator=gen) * 2 + 7.0).to(dtype)
    wb, bb, w, b = (torch.randn(width, generator=gen) * s + o for s, o in ((0.3, 1), (0.3, 0), (0.3, 1), (0.3, 0)))
    tol = dict(atol=3e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=4e-2, rtol=2e-2)
    for mean_b, mean in ((True, True), (False, True), (True, False)):
        def one(v, weight, bias, use_mean):
            return P.layer_norm(v, weight, bias, 1e-5) if use_mean else P.rms_norm(v, weight, 1e-5) + bias
        summed = resid.double() + one(branch.double(), wb.double(), bb.double(), mean_b)
        want = one(summed, w.double(), b.double(), mean)
        r = resid.to(DEV).clone()
        got = ops.norm_add_norm_affine(r, branch.to(DEV), wb.to(DEV), bb.to(DEV), 1e-5, mean_b, w.to(DEV), b.to(DEV), 1e-5, mean, dtype)
        torch.testing.assert_close(r.cpu().double(), summed, atol=1e-4 if dtype == torch.float32 else 0.1, rtol=1e-5 if dtype == torch.float32 else 2e-2)
        torch.testing.assert_close(got.cpu().double(), want, **tol)
        rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
        r2 = resid.to(DEV).clone()
        got = ops.norm_add_norm_affine(r2, branch.to(DEV), wb.to(DEV), bb.to(DEV), 1e-5, mean_b, w.to(DEV), b.to(DEV), 1e-5, mean, dtype, rows=rows)
        assert bool((r2.cpu() == resid).all())
        torch.testing.assert_close(got.cpu().double(), want[[7, 0, 3]], **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 32, 24), (3, 3, 20, 12), (8, 1, 128, 64), (2, 2, 6, 50), (40, 8, 64, 16)])
def test_norms_head_by_head_blended_values_and_a_gate_per_head(lib, dtype, sizes):
    from fms_amd.kernels import ops

    H, G, D, V = sizes
    gen = torch.Generator().manual_seed(H * D + V)
    T = 70
    nq, nk, nv = H * D, G * D, G * V
    proj = torch.randn(T, nq + nk + nv + H + 3, generator=gen) * 2
    wq, wk = torch.randn(D, generator=gen) * 0.3 + 1, torch.randn(D, generator=gen) * 0.3 + 1
    first = torch.randn(T, nv + 5, generator=gen).to(dtype)[:, 2 : 2 + nv]  # rows of a stride of their own
    lam = torch.tensor([0.3])
    seq = torch.zeros(T, dtype=torch.int32)
    seq[5] = -1  # a padding row: not written
    out = ops.qk_projection_norm(proj.to(DEV), nq, nk, nv, wq.to(DEV), wk.to(DEV), 1e-5, dtype, seq.to(DEV), norm_dim=D,
                                 v_first=first.to(DEV), v_lambda=lam.to(DEV)).float().cpu()
    want_q = P.rms_norm(proj[:, :nq].double().view(T, H, D), wq.double(), 1e-5).reshape(T, nq)
    want_k = P.rms_norm(proj[:, nq : nq + nk].double().view(T, G, D), wk.double(), 1e-5).reshape(T, nk)
    want_v = 0.7 * proj[:, nq + nk : nq + nk + nv].double() + 0.3 * first.double()
    want = torch.cat([want_q, want_k, want_v], dim=1).float()
    live = seq >= 0
    tol = dict(atol=2e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(out[live], want[live], **tol)
    # one norm over all heads, values copied: what the other kind of layer runs
    wq2, wk2 = torch.randn(nq, generator=gen) * 0.3 + 1, torch.randn(nk, generator=gen) * 0.3 + 1
    out = ops.qk_projection_norm(proj.to(DEV), nq, nk, nv, wq2.to(DEV), wk2.to(DEV), 1e-5, dtype).float().cpu()
    want = torch.cat([P.rms_norm(proj[:, :nq].double(), wq2.double(), 1e-5), P.rms_norm(proj[:, nq : nq + nk].double(), wk2.double(), 1e-5),
                      proj[:, nq + nk : nq + nk + nv].double()], dim=1).float()
    torch.testing.assert_close(out, want, **tol)
    # a gate per head
    x = torch.randn(T, H * V, generator=gen).to(dtype)
    gate = proj[:, nq + nk + nv : nq + nk + nv + H]
    got = ops.gate_mul(x.to(DEV), gate.to(DEV), "sigmoid", group=V).float().cpu()
    want = (x.double().view(T, H, V) * torch.sigmoid(gate.double())[:, :, None]).reshape(T, H * V).float()
    torch.testing.assert_close(got, want, **tol)


def test_distance_rows_follow_the_bucket_rule(lib):
    from fms_amd.parts.attention import distance_buckets

    for rows, far in ((32, 128), (8, 20), (6, 9), (4, 3), (2, 2), (64, 4096), (33, 100)):
        got = distance_buckets(rows, far)
        assert got == [P.distance_bucket(n, rows, far) for n in range(len(got))]
        assert got[-1] == rows - 1 and rows - 1 not in got[:-1]
        assert all(P.distance_bucket(n, rows, far) == rows - 1 for n in (len(got), len(got) + 7, 100 * len(got)))


def _reference_attention(q, k, v, scale, visible, cap=0.0, sink=None, bias=None):
    """[n, H, V] from float64 q [n, H, D], k [n, G, D], v [n, G, V]; visible [n, n]; bias [H, n, n]."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=torch.float64)
    probs = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        if bias is not None:
            s = s + bias[h]
        p = P.softmax_rows(s, visible, None if sink is None else sink[h])
        probs.append(p)
        out[:, h] = p @ v[:, g]
    return out, probs


MASKS = [
    # (heads, kv heads, dim, vdim, window, keep_first, chunk, cap, sink, distance table rows / far)
    (4, 2, 32, 24, 40, 3, 0, 0.0, False, (8, 20)),       # values of their own size: the generic kernel in both types
    (3, 3, 20, 36, 5, 1, 0, 8.0, True, (6, 9)),
    (2, 1, 64, 64, 70, 66, 0, 0.0, False, (32, 64)),      # more than a page of kept keys
    (2, 2, 16, 40, 64, 0, 0, 0.0, True, None),
    (4, 2, 32, 24, 0, 0, 33, 15.0, True, None),           # chunks
    (8, 2, 64, 64, 0, 0, 64, 30.0, True, None),           # sizes of the matrix-core kernels: chunks of one page,
    (4, 4, 128, 128, 0, 0, 100, 0.0, True, None),         # ... of no multiple of a page, without a cap,
    (8, 1, 32, 32, 0, 0, 150, 10.0, False, None),         # ... without a sink,
    (2, 2, 96, 96, 0, 0, 7, 12.0, True, None),            # ... a head size between 64 and 128
    (2, 1, 128, 128, 50, 0, 0, 20.0, True, None),         # a window and a sink
    (4, 2, 128, 128, 70, 5, 0, 0.0, False, (32, 64)),     # kept keys and a distance table on the matrix-core prompt kernels:
    (4, 1, 64, 64, 40, 130, 0, 0.0, True, (16, 200)),     # ... three pages of kept keys, a table longer than the window,
    (2, 2, 32, 32, 100, 64, 0, 9.0, False, (8, 20)),      # ... a page of kept keys exactly, a cap,
    (3, 3, 80, 80, 30, 1, 0, 0.0, False, (6, 9)),         # ... a head size without a kernel of its own
    (2, 2, 48, 48, 64, 2, 0, 0.0, False, None),           # ... kept keys without a table
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", MASKS)
def test_attention_masks_sink_and_distance_bias(lib, dtype, sizes):
    """Keys and values written by the cache-write kernel into scattered pages, read by the attention kernels, as a prompt
    (all tokens in one step; for bfloat16 through the query blocks of the matrix-core kernel where the sizes fit) and
    token by token as decode steps.  The last query matches one key strongly: placed just inside its mask's edge that key
    must hold most of the weight, just outside none."""
    from fms_amd.kernels import ops

    H, K, D, V, window, keep, chunk, cap, has_sink, table = sizes
    gen = torch.Generator().manual_seed(D + V + chunk + window)
    n = 200
    base = torch.randn(n, (H + K) * D + K * V, generator=gen)
    sink = (torch.randn(H, generator=gen) * 1.5) if has_sink else None
    bias_t = None
    by_distance = None
    if table:
        rows, far = table
        rel = torch.randn(rows, H, generator=gen, dtype=torch.float64)
        bias_t = P.distance_bias(n, rel, far)
        from fms_amd.parts.attention import distance_buckets
        by_distance = rel.float()[torch.tensor(distance_buckets(rows, far))].t().contiguous().to(DEV)
    last = n - 1
    inside = last - last % chunk if chunk else last - window + 1
    edges = [(inside, True), (inside - 1, False)]
    if keep:
        edges += [(keep - 1, True), (keep, False)]
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    visible = P.visible_chunk(n, chunk) if chunk else P.visible_window(n, window, keep)
    k0 = H * D
    pages = [5, 0, 3, 6]
    table_t = torch.tensor([pages], dtype=torch.int32, device=DEV)
    pos = torch.arange(n, dtype=torch.int32, device=DEV)
    seq = torch.zeros(n, dtype=torch.int32, device=DEV)
    tol = dict(atol=3e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
    for key_at, seen in edges:
        rows_ = base.clone()
        rows_[key_at, k0 : k0 + D] *= 4
        rows_[last, :D] = rows_[key_at, k0 : k0 + D] * (4.0 / D ** 0.5)
        rows_ = rows_.to(dtype)
        kc = torch.zeros(8, K, 64, D, dtype=dtype, device=DEV)
        vc = torch.zeros(8, K, V, 64, dtype=dtype, device=DEV)
        qkv = rows_.to(DEV).clone()
        ops.rope_kv_write(qkv, pos, seq, table_t, None, None, 0, kc, vc, H, K, D, V)
        q = rows_[:, : H * D].double().view(n, H, D)
        k = rows_[:, k0 : k0 + K * D].double().view(n, K, D)
        v = rows_[:, k0 + K * D :].double().view(n, K, V)
        want, probs = _reference_attention(q, k, v, 0.3, visible, cap, sink.double() if has_sink else None, bias_t)
        if not cap:
            assert (float(probs[0][last, key_at]) > 0.5) == seen and (seen or float(probs[0][last, key_at]) == 0.0)
        common = dict(soft_cap=cap, value_dim=V, chunk=chunk, keep_first=keep, sink=sink.to(DEV) if has_sink else None, distance_bias=by_distance)
        # as a prompt
        qb = {}
        if dtype == torch.bfloat16 and D == V and D % 16 == 0 and (not ops.prefill_extras_are_generic(D) or (not keep and table is None)) and not ops.prefill_cap_is_generic(D, cap):
            size = ops.prefill_qblock(H, K, D, n)
            starts = list(range(0, n, size))
            qb = dict(qblock_start=torch.tensor(starts, dtype=torch.int32, device=DEV),
                      qblock_len=torch.tensor([min(size, n - s) for s in starts], dtype=torch.int32, device=DEV), qblock_tokens=size)
        got = ops.attention(qkv, pos, seq, table_t, kc, vc, H, K, D, 0.3, window, **qb, **common).float().cpu().view(n, H, V)
        torch.testing.assert_close(got.double(), want, **{k_: v_ for k_, v_ in tol.items()}, check_dtype=False)
        # token by token: decode steps over the same cache (a batch of the last 40 tokens, each its own row and context)
        rows_idx = list(range(n - 40, n))
        tq = qkv[rows_idx]
        tpos = pos[rows_idx].contiguous()
        # every row is a sequence of its own that shares the pages: same block table row for all
        tseq = torch.arange(len(rows_idx), dtype=torch.int32, device=DEV)
        ttable = table_t.expand(len(rows_idx), -1).contiguous()
        got = ops.attention(tq, tpos, tseq, ttable, kc, vc, H, K, D, 0.3, window, decode=True, max_context=n, **common).float().cpu().view(-1, H, V)
        torch.testing.assert_close(got.double(), want[rows_idx], **tol, check_dtype=False)


# ---- the engine --------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_sequence(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    ids, want = expected_for(folders, name, 150, 1, dtype)
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=256, max_slots=2)
    slot = engine.new_sequence()
    judge(engine.step([slot], [ids], "all"), want, dtype)
    engine.end_sequence(slot)
    engine.cache.check()


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_stream_after_every_layer(lib, folders, name):
    """float32: the residual stream after each layer against the plain implementation's, so that a fault names its layer."""
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    ids = tokens_for(cfg["vocab"], 70, 2)
    layers = []
    P.forward(cfg, weights, ids, layers_out=layers)
    model = get(lib, folders, name, "float32")
    seen = []
    blocks = model.layers
    originals = [b.forward for b in blocks]

    def watch(i):
        def forward(stream, batch, cache, act_dtype, next_norm=None):
            originals[i](stream, batch, cache, act_dtype)
            # what is still pending joins the stream in a copy: the stream after this layer
            pending, norm = stream.pending, stream.pending_norm
            seen.append(stream.resid.clone().cpu().double() + P.layer_norm(pending.double().cpu(), norm.w["weight"].double().cpu(),
                                                                           norm.w["bias"].double().cpu(), norm.eps))
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
    assert len(seen) == len(cfg["layers"])
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
    # from the very first token one by one: the kept first tokens, the first chunk, the sink against a single key
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
    """Unequal requests in one batch, decoded together; the short ones end early, their slots and pages go to new requests
    that start while the long one goes on (windows and chunks give pages back on the way, the kept first pages stay);
    every request equals itself alone."""
    from fms_amd.engine import Engine

    lens = {"a": (300, 1), "b": (70, 5), "c": (3, 6), "d": (129, 7), "e": (66, 8)}
    reqs = {k: expected_for(folders, name, n, seed, dtype) for k, (n, seed) in lens.items()}
    model = get(lib, folders, name, dtype)
    engine = Engine(model, max_tokens=64 * 9, max_slots=3)
    got = {k: [] for k in reqs}
    slots = {k: engine.new_sequence() for k in ("a", "b", "c")}
    prompt = {"a": 200, "b": 64, "c": 1}
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
        engine.cache.check()
        for k in [k for k in alive if done[k] == len(reqs[k][0])]:
            engine.end_sequence(slots.pop(k))
            alive.remove(k)
        if waiting and len(alive) < 2 and "a" in alive:
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


def _with_changed_mixer(cfg, i, path, value):
    wrong = json.loads(json.dumps(cfg))
    at = wrong["layers"][i]["mixer"]
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    return wrong


@pytest.mark.parametrize("name", ["A", "C"])
def test_the_edges_decide_in_prompts_and_in_decoding(lib, name, tmp_path):
    """Queries scaled up: single keys hold most of a query's weight, among them keys at a window's last place, a chunk's
    first, the last kept one, and at page borders.  The same weights run with a window or a chunk one token longer or
    shorter, with one kept token more or fewer, must fail the same comparison; so must a sink or a distance table that
    is left out (set to what leaves it out)."""
    from fms_amd.engine import Engine
    from fms_amd.weights import write_safetensors

    base = CONFIGS[name]
    folder = write_folder(lib, str(tmp_path / "sharp"), base, seed=21, sharp=5.0)
    cfg, weights = P.load_model_folder(folder)
    ids = tokens_for(cfg["vocab"], 330, 3)
    want = expect(cfg, weights, ids, "float32")

    def run(cut):
        model = lib.get_model("hf_pretrained", model_path=folder, data_type="float32")
        engine = Engine(model, max_tokens=384, max_slots=1)
        slot = engine.new_sequence()
        got = [engine.step([slot], [ids[:cut]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[cut:]]
        engine.end_sequence(slot)
        return torch.cat(got)

    def save(c):
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(c, f)

    judge(run(250), want, "float32")
    judge(run(40), want, "float32")
    changes = []
    for i, entry in enumerate(cfg["layers"]):
        size = entry["mixer"]["mask"]["size"]
        changes += [(i, ("mask", "size"), size + 1), (i, ("mask", "size"), size - 1)]
        keep = entry["mixer"]["mask"].get("keep_first")
        if keep:
            changes += [(i, ("mask", "keep_first"), keep + 1), (i, ("mask", "keep_first"), keep - 1)]
    for i, path, value in changes:
        save(_with_changed_mixer(cfg, i, path, value))
        with pytest.raises(AssertionError):
            judge(run(250), want, "float32")
    save(cfg)
    # a sink that is left out (a logit so low that it adds nothing), a distance table of zeros
    stored = {k: v.to(torch.bfloat16) for k, v in weights.items()}
    for suffix, value in ((".sink", -1e4), (".rel", 0.0)):
        for k in [k for k in stored if k.endswith(suffix)]:
            changed = dict(stored)
            changed[k] = torch.full_like(stored[k], value)
            write_safetensors(os.path.join(folder, "model.safetensors"), [(n, tuple(v.shape), v.dtype) for n, v in changed.items()],
                              lambda n: changed[n])
            with pytest.raises(AssertionError):
                judge(run(250), want, "float32")


def drawn_configuration(seed):
    """A configuration whose every size, count, constant and layer order is drawn at random (the layers that mix values
    agree in key/value heads times value size, as they must)."""
    import random

    rng = random.Random(seed)
    mixed = rng.choice([48, 96])  # key/value heads times value size of the layers that mix their values
    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.choice(["c", "c", "w", "l"])
        ff = rng.choice([None, 24, 50, 64, 128])
        if kind == "l":
            rot = rng.choice([2, 4, 8, 16, 32])
            layers.append(layer(latent(rng.randint(1, 4), rng.choice([8, 12, 16, 32, 64]), rot, rng.choice([8, 20, 32, 64]),
                                       rng.choice([8, 16, 24, 64]), rng.randint(1, 150), base=rng.choice([10.0, 1e4, 5e5]),
                                       scale=rng.uniform(0.1, 0.4)), ff))
            continue
        v_mix = rng.random() < 0.7
        if v_mix:
            kv = rng.choice([g for g in (1, 2, 3, 4, 6) if mixed % g == 0])
            vdim = mixed // kv
        else:
            kv, vdim = rng.choice([1, 2, 3]), rng.choice([8, 16, 40, 64])
        heads = kv * rng.choice([1, 2, 4])
        dim = rng.choice([8, 16, 20, 32, 48, 64, 96, 128]) if rng.random() < 0.7 else vdim + vdim % 2
        if kind == "c":
            dims = rng.choice([d for d in (2, 4, 8, 16, 32, 48, 64, 128) if d <= dim])
            layers.append(layer(chunked(heads, kv, dim, vdim, rng.randint(1, 180), dims, base=rng.choice([100.0, 1e4, 2.5e5]),
                                        factor=rng.choice([None, 2.0, 8.0]), scale=rng.uniform(0.1, 0.4), softcap=rng.choice([None, 5.0, 20.0, 50.0]),
                                        v_mix=v_mix), ff))
        else:
            rows = rng.choice([2, 4, 8, 16, 32])
            layers.append(layer(windowed(heads, kv, dim, vdim, rng.randint(1, 180), rng.choice([None, 0, 1, 4, 70]), rows,
                                         rng.randint(rows // 2 + 1, 200), scale=rng.uniform(0.1, 0.4), v_mix=v_mix), ff))
    return dict(vocab=rng.randint(50, 600), width=rng.choice([64, 96, 100, 128, 192]), norm={"eps": rng.choice([1e-6, 1e-5, 1e-3])},
                embedding={"scale": rng.uniform(0.5, 12.0)}, max_positions=1024, layers=layers)


@pytest.mark.parametrize("seed", range(24))
def test_configurations_drawn_at_random(lib, seed, tmp_path):
    """Every size, constant and layer order drawn: whole, in portions and token by token in float32; whole in bfloat16."""
    from fms_amd.engine import Engine

    folder = write_folder(lib, str(tmp_path / "drawn"), drawn_configuration(seed), seed=100 + seed)
    cfg, weights = P.load_model_folder(folder)
    ids = tokens_for(cfg["vocab"], 200, seed)
    for dtype in DTYPES:
        want = expect(cfg, weights, ids, dtype)
        model = lib.get_model("hf_pretrained", model_path=folder, data_type=dtype)
        engine = Engine(model, max_tokens=256, max_slots=1)
        slot = engine.new_sequence()
        judge(engine.step([slot], [ids], "all"), want, dtype)
        engine.end_sequence(slot)
        if dtype == "float32":
            for cuts in ([70, 1, 2, 127], [130] + [1] * 70):
                slot = engine.new_sequence()
                got, at = [], 0
                for n in cuts:
                    got.append(engine.step([slot], [ids[at : at + n]], "all"))
                    at += n
                judge(torch.cat(got), want, dtype)
                engine.end_sequence(slot)
        engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_graphs_and_eager_steps(lib, folders, dtype):
    """300 tokens decoded one by one for three sequences of different lengths, across page borders, past windows and
    over several chunks, as captured graphs and as eager steps: the same logits as the plain implementation's."""
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
    want = [P.greedy_generate(cfg, weights, p, 12) for p in prompts]
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
    """The package's programs on a Basopel folder: the trace replay (float32 and bfloat16, a batch whose requests end
    at different steps) and the registry's view of the architecture."""
    name = "A"
    cfg, weights = plain(folders, name)
    assert "basopel" in lib.list_models() and "micro" in lib.list_variants("basopel")
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


def test_the_inference_program_and_a_model_from_the_registry(lib, folders):
    """bin/fms_inference with a Basopel folder (the model class comes from config.json; the text printed is the plain
    implementation's greedy continuation), and a registered variant with random weights through the engine."""
    from fms_amd.engine import Engine
    from fms_amd.tokenizers import CharTokenizer

    name = "A"  # its vocabulary holds the character tokenizer's
    cfg, weights = plain(folders, name)
    tok = CharTokenizer()
    prompt = [ord(c) for c in "kept first"]
    new = P.greedy_generate(cfg, weights, prompt, 12)
    if tok.eos_token_id in new:
        new = new[: new.index(tok.eos_token_id)]
    env = dict(os.environ, PYTHONIOENCODING="utf-8")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "fms_inference"), "--architecture", "hf_pretrained", "--model_path", folders[name],
           "--tokenizer", "char_tokenizer", "--default_dtype", "fp32", "--max_new_tokens", "12", "--prompt_ids", ",".join(map(str, prompt))]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=110, env=env)
    assert proc.returncode == 0, proc.stderr.decode(errors="replace")
    assert tok.decode(prompt + new) in proc.stdout.decode("utf-8")
    model = lib.get_model("basopel", "micro", data_type="bfloat16", random_seed=5)
    engine = Engine(model, max_tokens=512, max_slots=2)
    slot = engine.new_sequence()
    ids = tokens_for(1024, 300, 9)
    whole = engine.step([slot], [ids], "all")
    engine.end_sequence(slot)
    slot = engine.new_sequence()
    cut = torch.cat([engine.step([slot], [ids[:170]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[170:]])
    engine.end_sequence(slot)
    assert bool(torch.isfinite(whole).all()) and float((whole - cut).abs().max()) < 0.15 * float(whole.abs().max())
