"""Serving benchmark: decode tokens per second of the Llama-3-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Random weights, synthetic token ids.  A "step" is one decode step of the whole batch through
the library's own generation path (step function, cache, kernels, sampler).  One JSON line is
printed: decode tokens/s at batch 8 (`value`), the prefill of 2,048 tokens, the decode step's
memory roofline (against the published peak and against what a pure read reaches on this GPU now),
the share of the step's time by kernel class, and further points: decode at batch 1, 64 and 192, at
batch 8 with every context near 8000 tokens, the Llama-2-7B shape at batch 8 (256 steps) and the
Llama-3-70B shape at batch 16 (128 steps).  Decode steps run as generation runs them: the host looks
at the chosen tokens every `steps_ahead` steps (`--steps-ahead 1`: after every step).

    python bench.py --zodolorn [--layers N]

is another workload (the default one and its record stay as they are): Zodolorn models of a few layer sizes beside
Llama models of the same width, depth, heads and feed-forward parameters: prefill and decode throughput of both, and
for every class of kernel its time in one eager prefill and one eager decode step over the time that its bytes and
flops would take at what this GPU delivers (`x_roofline`: 1 is the roofline).

    python bench.py --defapel [--layers N]

is the same comparison for Defapel (windowed attention beside a gated delta rule, a delta rule with a decay per channel,
experts weighted on their input) beside Llama of the same width, depth and heads.

    python bench.py --basopel [--layers N]

is the same comparison for Basopel (attention in chunks with a sink, in a window that keeps first tokens with a bias by
distance, and over a latent; layer norms on both sides of every branch) beside Llama of the same width, depth, heads and
gated feed-forward; every attention call is priced by the keys its own mask shows.

    python bench.py --sidalorn [--layers N]

is the same comparison for Sidalorn (attention without positions over a latent, a real-gated recurrent block, norms in
groups behind the branches, experts routed in groups) beside Zodolorn, the closest model of the library (attention over
a latent, experts), with the same width, depth, heads, latent and expert sizes.
"""

import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# published MI355X peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in the record)")
    ap.add_argument("--variant", default="3-8b")
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--prompt-min", type=int, default=128, help="shortest prompt of the decode batches")
    ap.add_argument("--prompt-max", type=int, default=2048, help="longest prompt of the decode batches")
    ap.add_argument("--skip-points", action="store_true", help="leave out the further points (batch 1 and 64, long contexts, the 7B shape)")
    ap.add_argument("--skip-70b", action="store_true", help="leave out the point at the Llama-3-70B shape (141 GB of weights)")
    ap.add_argument("--with-70b", action="store_true", help="accepted for older command lines: the 70B point is measured unless --skip-70b says no")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--steps-ahead", type=int, default=None,
                    help="decode steps that run before the host looks at their tokens (default: the generation loop's STEPS_AHEAD)")
    ap.add_argument("--only", choices=["decode", "prefill"], default=None,
                    help="run one phase only (for profiling); the record then lacks the other")
    # the workload options of the reference's scripts/benchmark_inference.py:70-87, by their names
    ap.add_argument("--seq_len", type=int, default=None, help="every prompt of the decode batches has this many tokens")
    ap.add_argument("--batch_size", type=int, default=None, help="the same as --batch")
    ap.add_argument("--max_new_tokens", type=int, default=None, help="the same as --steps: decode steps that are timed")
    ap.add_argument("--zodolorn", action="store_true",
                    help="another workload: Zodolorn beside Llama at equal layer sizes, with every kernel class's distance from its roofline")
    ap.add_argument("--basopel", action="store_true", help="another workload: Basopel beside Llama at equal layer sizes, likewise")
    ap.add_argument("--defapel", action="store_true", help="another workload: Defapel beside Llama at equal layer sizes, likewise")
    ap.add_argument("--sidalorn", action="store_true", help="another workload: Sidalorn beside Zodolorn at equal layer sizes, likewise")
    args = ap.parse_args()
    if args.seq_len is not None:
        args.prompt_min = args.prompt_max = args.seq_len
    if args.batch_size is not None:
        args.batch = args.batch_size
    if args.max_new_tokens is not None:
        args.steps = args.max_new_tokens
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py measures one GPU: this library runs on a single MI355X, --gpus {args.gpus} is not supported")
        return 2

    if args.zodolorn or args.defapel or args.sidalorn or args.basopel:
        return design_comparison(args, "zodolorn" if args.zodolorn else ("defapel" if args.defapel else ("sidalorn" if args.sidalorn else "basopel")))

    import torch

    import fms_amd
    from fms_amd.architectures import variant_config
    from fms_amd.engine import Engine
    from fms_amd.kernels import ops
    from fms_amd.sampling import SamplingParams, choose

    from fms_amd.generation.loop import STEPS_AHEAD

    if args.steps_ahead is None:
        args.steps_ahead = STEPS_AHEAD
    args.steps_ahead = max(1, args.steps_ahead)

    # what this GPU delivers now: a kernel that only reads, a kernel that only issues matrix instructions
    read_bps, mfma_flops = ops.measured_peaks()

    full = variant_config("llama", args.variant)
    overrides = {"max_expected_seq_len": args.context}
    if args.layers is not None:
        overrides["nlayers"] = args.layers
    model = fms_amd.get_model("llama", args.variant, data_type="bf16", device_type="cuda", random_seed=args.seed, **overrides)
    cfg = model.config
    E, H, K, D, F, V, L = (cfg.emb_dim, cfg.nheads, cfg.kv_heads, cfg.head_dim, cfg.ffn_hidden_dim, cfg.src_vocab_size,
                           cfg.nlayers)

    def step_bytes_of(c):
        """(bytes of weights a decode step reads: everything but the embedding table, once; cache bytes per token)"""
        e, h, k, d, f = c.emb_dim, c.nheads, c.kv_heads, c.head_dim, c.ffn_hidden_dim
        layer = (h + 2 * k) * d * e + e * h * d + 2 * f * e + e * f + 2 * e  # elements per layer, norms included
        return 2 * (c.nlayers * layer + e + c.src_vocab_size * e), 2 * c.nlayers * k * d * 2

    step_weight_bytes, kv_bytes_per_token = step_bytes_of(cfg)
    greedy = SamplingParams(do_sample=False)
    rng = random.Random(args.seed)

    def decode(batch: int, steps: int, warmup: int, model=model, prompt_min=args.prompt_min, prompt_max=args.prompt_max,
               shares=None):
        """(tokens/s, ms per step, bytes a step has to read) for `batch` sequences with prompts of prompt_min..prompt_max
        tokens.  shares: a dict that takes the share of an eager step's time by kernel class."""
        weight_bytes, kv_bytes = step_bytes_of(model.config)
        V = model.config.src_vocab_size
        lens = [rng.randint(prompt_min, prompt_max) for _ in range(batch)]
        room = sum(-(-(n + steps + warmup + 8) // 64) * 64 for n in lens)
        engine = Engine(model, max_tokens=room, max_slots=batch)
        slots = [engine.new_sequence() for _ in range(batch)]
        tokens = None
        per_group = max(1, 16384 // prompt_max)  # prompts in groups, so that activations stay small
        for i in range(0, batch, per_group):
            group = list(range(i, min(i + per_group, batch)))
            prompts = [[rng.randrange(V) for _ in range(lens[b])] for b in group]
            logits = engine.step([slots[b] for b in group], prompts, "last")
            first = choose(logits, greedy).tolist()
            tokens = first if tokens is None else tokens + first
        def run(n):  # n decode steps as the generation loop runs them: the host looks at the tokens every few steps
            nonlocal tokens
            done = 0
            while done < n:
                ahead = min(args.steps_ahead, n - done)
                tokens = engine.decode_and_choose_many(slots, tokens, greedy, steps=ahead)[-1]
                done += ahead

        run(warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        mean_ctx = sum(lens) + batch * (1 + warmup + steps / 2)
        if shares is not None:
            shares.update(kernel_shares(engine, slots, tokens))
        for s in slots:
            engine.end_sequence(s)
        del engine
        torch.cuda.empty_cache()
        return batch * steps / dt, 1000 * dt / steps, weight_bytes + kv_bytes * mean_ctx

    def kernel_shares(engine, slots, tokens):
        """The share of a decode step's GPU time by kernel class: three eager steps (the same kernels in the same
        shape as the replayed graph) with an event before and after every call into the kernel library."""
        classes = {"qkv_rope_write": "qkv_rope_cache", "attention": "attention", "gated_linear": "gate_up_act",
                   "sample": "sampling", "embed": "other", "add_norm": "other", "advance_positions_": "other"}
        spans, originals = [], {}

        def timed(name, fn):
            def call(*a, **kw):
                kind = classes.get(name)
                if name == "linear_into_stream":
                    kind = "o_proj_residual" if a[0].shape[1] == a[1].shape[0] else "down_residual"
                if name == "linear":
                    kind = "head" if a[1].shape[0] == engine.vocab else "other"
                first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                first.record()
                out = fn(*a, **kw)
                last.record()
                spans.append((kind, first, last))
                return out
            return call

        for name in list(classes) + ["linear_into_stream", "linear"]:
            originals[name] = getattr(ops, name)
            setattr(ops, name, timed(name, originals[name]))
        try:
            for _ in range(3):
                logits = engine.step(slots, [[t] for t in tokens], "last")
                tokens = choose(logits, greedy).tolist()
            torch.cuda.synchronize()
        finally:
            for name, fn in originals.items():
                setattr(ops, name, fn)
        total = {}
        for kind, first, last in spans:
            total[kind] = total.get(kind, 0.0) + first.elapsed_time(last)
        whole = sum(total.values()) or 1.0
        return {kind: round(ms / whole, 4) for kind, ms in sorted(total.items())}

    def prefill(n_tokens: int):
        engine = Engine(model, max_tokens=n_tokens + 64, max_slots=1)
        times = []
        for _ in range(4):
            slot = engine.new_sequence()
            ids = [rng.randrange(V) for _ in range(n_tokens)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.step([slot], [ids], "last")
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            engine.end_sequence(slot)
        del engine
        torch.cuda.empty_cache()
        t = sorted(times[1:])[len(times[1:]) // 2]
        flops = 2.0 * n_tokens * L * ((H + 2 * K) * D * E + E * H * D + 2 * F * E + E * F)
        flops += L * 4.0 * H * D * n_tokens * (n_tokens + 1) / 2  # causal scores and mixing
        flops += 2.0 * E * V  # the head for one row
        return n_tokens / t, 1000 * t, flops / t / PEAK_FLOPS["bf16"], flops / t / mfma_flops

    pre_tps = pre_ms = pre_frac = pre_frac_measured = 0.0
    tps = ms = step_bytes = 0.0
    shares = {}
    if args.only != "decode":
        pre_tps, pre_ms, pre_frac, pre_frac_measured = prefill(args.prefill_tokens)
    if args.only != "prefill":
        tps, ms, step_bytes = decode(args.batch, args.steps, args.warmup, shares=shares)
    achieved = step_bytes / (ms / 1000) / 1e9 if ms else 0.0
    points = {}

    def point(name, p_tps, p_ms, p_bytes):
        gbs = p_bytes / (p_ms / 1000) / 1e9
        points[name] = round(p_tps, 1)
        points[f"{name}_ms"] = round(p_ms, 3)
        points[f"{name}_gb"] = round(p_bytes / 1e9, 3)
        points[f"{name}_gbs"] = round(gbs, 1)
        points[f"{name}_frac"] = round(gbs / HBM_GBS, 4)

    if not args.skip_points and args.only is None:
        for b, steps, warmup in ((1, min(args.steps, 32), 4), (64, min(args.steps, 16), 2), (192, min(args.steps, 12), 2)):
            point(f"decode_b{b}", *decode(b, steps, warmup))
        # every context near the benchmark's context length
        near = min(8000, args.context - 64)
        point(f"decode_b8_ctx{near}", *decode(8, min(args.steps, 16), 2, prompt_min=near - 100, prompt_max=near))
        # the Llama-2-7B shape: batch 8, prompts of 64..1024 tokens, 256 decode steps, context 4096
        other = fms_amd.get_model("llama", "2-7b", data_type="bf16", device_type="cuda", random_seed=args.seed,
                                  max_expected_seq_len=4096)
        point("llama2_7b_b8", *decode(8, 256, 8, model=other, prompt_min=64, prompt_max=1024))
        del other
        torch.cuda.empty_cache()
        # the Llama-3-70B shape on the one GPU: batch 16, prompts of 256..4096 tokens, 128 decode steps; 141 GB of
        # weights and 25 GB of cache beside the models above, so only where that much memory is free
        if not args.skip_70b:
            if torch.cuda.mem_get_info()[0] > 200e9:
                big = fms_amd.get_model("llama", "3-70b", data_type="bf16", device_type="cuda", random_seed=args.seed,
                                        max_expected_seq_len=8192)
                point("llama3_70b_b16", *decode(16, 128, 4, model=big, prompt_min=256, prompt_max=4096))
                del big
                torch.cuda.empty_cache()
            else:
                points["llama3_70b_b16"] = None  # not measured: less than 200 GB free on this GPU

    record = {
        "metric": f"decode tok/s at batch {args.batch} (llama {args.variant} shape, {args.context} context); prefill tok/s at {args.prefill_tokens} tokens",
        "value": round(tps, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": f"synthetic: random weights N(0, 0.02), uniform random token ids, prompt lengths uniform in [{args.prompt_min}, {args.prompt_max}]",
        "config": {
            "model": f"llama {args.variant} shape",
            "global_batch": args.batch,
            "seq_len": args.context,
            "parallelism": "single GPU",
            "nlayers": L,
            "nlayers_full": full.nlayers,
            "emb_dim": E,
            "nheads": H,
            "kvheads": K,
            "head_dim": D,
            "ffn_hidden": F,
            "vocab": V,
            "rope_theta": cfg.rope_theta,
            "norm_eps": cfg.norm_eps,
            "prompt_len_min": args.prompt_min,
            "prompt_len_max": args.prompt_max,
            "prefill_tokens": args.prefill_tokens,
            "cache_page_tokens": 64,
            "steps_ahead": args.steps_ahead,
        },
        "prefill": {"value": round(pre_tps, 1), "tokens": args.prefill_tokens, "ms": round(pre_ms, 3), "frac": round(pre_frac, 4),
                    "frac_measured": round(pre_frac_measured, 4), "peak_measured_tflops": round(mfma_flops / 1e12, 1)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4), "peak_measured": round(read_bps / 1e9, 1),
                     "frac_measured": round(achieved / (read_bps / 1e9), 4)},
        "shares": shares,
        "points": points,
    }
    print(json.dumps(record))
    return 0


# ---- Zodolorn beside Llama ------------------------------------------------------------------------------------------
# (name, width, heads, [dim, rot, vdim, q_rank, kv_rank], dense ff, experts, top, expert ff, shared ff, vocabulary)
ZODOLORN_SIZES = [
    ("w2048", 2048, 16, (128, 64, 128, 768, 512), 8192, 32, 4, 1024, 2048, 32768),
    ("w4096", 4096, 32, (128, 64, 128, 1536, 512), 12288, 64, 6, 1536, 3072, 32768),
]


# (name, width, layer pattern, heads, kv heads, head size, window, delta heads, delta q/k heads, key channels, value channels,
#  experts, top, expert ff, vocabulary)
DEFAPEL_SIZES = [
    ("w2048", 2048, "pppc", 16, 4, 128, 1024, 16, 8, 128, 128, 32, 4, 1024, 32768),
    ("w4096", 4096, "pppc", 32, 8, 128, 1024, 32, 16, 128, 128, 64, 6, 1536, 32768),
]


# (name, width, layer pattern, heads, [dim, vdim, kv_rank], recurrent channels, blocks, dense ff, experts, identity experts, top,
#  expert ff, shared ff, groups, groups kept, norm groups, vocabulary)
SIDALORN_SIZES = [
    ("w2048", 2048, "aar", 16, (128, 128, 512), 2560, 10, 8192, 28, 4, 4, 1024, 2048, 4, 2, 4, 32768),
    ("w4096", 4096, "aar", 32, (128, 128, 512), 4096, 16, 12288, 60, 4, 6, 1536, 3072, 8, 4, 8, 32768),
]


# (name, width, layer pattern (c: attention in chunks, w: windowed with a distance bias, l: latent), heads, kv heads, head size,
#  feed-forward, chunk = window, latent size, vocabulary)
BASOPEL_SIZES = [
    ("w2048", 2048, "ccwl", 16, 4, 128, 8192, 1024, 512, 32768),
    ("w4096", 4096, "ccwl", 32, 8, 128, 12288, 1024, 512, 32768),
]


def design_comparison(args, design) -> int:
    import torch

    import fms_amd
    from fms_amd.architectures.zodolorn import make_config
    from fms_amd.engine import Engine
    from fms_amd.kernels import ops
    from fms_amd.sampling import SamplingParams, choose

    read_bps, mfma_flops = ops.measured_peaks()
    greedy = SamplingParams(do_sample=False)
    rng = random.Random(args.seed)
    layers = args.layers or 4
    context = 8192

    # bytes and flops of one call of an op, from its arguments (weights and caches are read once, activations once)
    # keys_read: the sum over the step's tokens of the keys each of them sees (flops); keys_loaded: the keys that have to
    # come from memory at least once (a prompt's keys serve all its queries; a decode step reads every context once)
    state = {"keys_read": 0, "keys_loaded": 0}

    def keys_of_call(a, kw):
        """(keys read, keys loaded) of one attention call, from the step's token runs (state["runs"]: first position and
        count per sequence, when the workload sets them) and the call's own mask: a window (a[10]), kept first keys, chunks."""
        runs = state.get("runs")
        if not runs:
            return state["keys_read"], state["keys_loaded"]
        window, chunk, keep = int(a[10]) if len(a) > 10 else 0, int(kw.get("chunk", 0) or 0), int(kw.get("keep_first", 0) or 0)

        def seen(p):
            if chunk:
                return p % chunk + 1
            return min(p + 1, window + min(keep, max(0, p + 1 - window))) if window else p + 1

        read = sum(seen(p) for first, count in runs for p in range(first, first + count))
        loaded = sum(max(seen(first + count - 1), min(first + count, count + seen(first) - 1)) for first, count in runs)
        return read, loaded

    def nbytes(*tensors):
        return sum(t.numel() * t.element_size() for t in tensors if t is not None)

    def cost(name, a, kw, out):
        if name in ("linear", "gated_linear", "linear_into_stream"):
            x, w = a[0], a[1]
            return nbytes(x, w) + (nbytes(out) if torch.is_tensor(out) else 0), 2.0 * x.shape[0] * w.shape[0] * w.shape[1]
        if name == "headwise_linear":
            x, w, y = a[0], a[2], a[3]
            return nbytes(w) + 2 * x.shape[0] * w.shape[0] * (w.shape[1] + w.shape[2]), 2.0 * x.shape[0] * w.numel()
        if name == "attention":  # grouped-query attention over keys and values of kvheads x head_dim
            H, K, D = a[6], a[7], a[8]
            read, loaded = keys_of_call(a, kw)
            return 2 * loaded * 2 * K * D + 2 * nbytes(a[0][:, : H * D]), 4.0 * read * H * D
        if name == "delta_rule":  # state read and written once a sequence; per token and head 4 passes over dim x vdim in float32
            qkv, st, n_seqs, H, D, V = a[0], a[4], a[8], a[9], a[11], a[12]
            vector_flops = 8.0 * qkv.shape[0] * H * D * V
            # priced at the float32 vector rate (the recurrence runs there), in units of the matrix rate the ideal is formed with
            return nbytes(qkv, a[1], a[2], out) + 2 * n_seqs * (st.numel() // st.shape[0]) * 4, vector_flops * mfma_flops / PEAK_FLOPS["fp32"]
        if name == "latent_attention":  # one row of rank + rot a key, and the latent once more as values
            H, R, P = a[6], a[7], a[8]
            read, loaded = keys_of_call(a, kw)
            return 2 * loaded * (2 * R + P) + nbytes(a[0]) + 2 * a[0].shape[0] * H * R, 2.0 * read * H * (2 * R + P)
        if name == "rglru_gates":  # two block-diagonal products on the float32 vector units, priced like the delta rule's passes
            u, ra = a[0], a[1]
            vector_flops = 4.0 * u.shape[0] * ra.numel()
            return nbytes(u, ra, a[3]) + 2 * u.numel() * 4, vector_flops * mfma_flops / PEAK_FLOPS["fp32"]
        if name == "rglru_scan":  # a, b and the other branch read once, the result written once
            return nbytes(a[0], a[1]) + a[0].numel() * 4 + nbytes(out), 0.0
        if name == "moe_experts" and a[2] is None:  # experts without a gate
            x, ids, _, u, d = a[:5]
            used = min(u.shape[0], ids.numel())
            return used * (nbytes(u, d) // u.shape[0]) + ids.numel() * (2 * x.shape[1] * x.element_size() + 4 * x.shape[1]), 4.0 * ids.numel() * u.shape[1] * u.shape[2]
        if name == "moe_experts":
            x, ids, g, u, d = a[:5]
            used = min(g.shape[0], ids.numel())  # experts whose weights are read at least once
            return used * (nbytes(g, u, d) // g.shape[0]) + ids.numel() * (2 * x.shape[1] * x.element_size() + 4 * x.shape[1]), 6.0 * ids.numel() * g.shape[1] * g.shape[2]
        tensors = [t for t in a if torch.is_tensor(t)] + ([out] if torch.is_tensor(out) else [])
        return nbytes(*[t for t in tensors if t.dim() == 2 and t.shape[0] == tensors[0].shape[0]]), 0.0

    watched = ["linear", "gated_linear", "linear_into_stream", "headwise_linear", "attention", "latent_attention", "moe_experts",
               "moe_route", "moe_combine", "add_norm", "norm_add_norm", "rms_norm_cols", "rope_kv_write", "qkv_rope_write",
               "latent_kv_write", "latent_q_rotate", "activation", "clamped_gated_act", "gated_act", "embed", "norm_add_norm_affine",
               "delta_rule", "delta_prepare", "gated_head_norm", "qk_projection_norm", "gate_mul", "scale_", "cast", "cast_cols",
               "rglru_gates", "rglru_scan", "short_conv", "group_norm_chain", "poly_norm", "moe_route_grouped"]
    small = {"moe_route", "moe_combine", "add_norm", "norm_add_norm", "norm_add_norm_affine", "rms_norm_cols", "rope_kv_write", "latent_kv_write",
             "latent_q_rotate", "activation", "clamped_gated_act", "gated_act", "embed", "delta_prepare", "gated_head_norm",
             "qk_projection_norm", "gate_mul", "scale_", "cast", "cast_cols", "short_conv", "group_norm_chain", "poly_norm",
             "moe_route_grouped"}

    def classes_of_a_step(run):
        """{class: (ms, ms at the roofline)} of the kernels of `run()`, by events around every call into the library."""
        spans, originals = [], {}

        def timed(name, fn):
            def call(*a, **kw):
                first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                first.record()
                out = fn(*a, **kw)
                last.record()
                b, f = cost(name, a, kw, out)
                spans.append(("elementwise" if name in small else name, first, last, b, f))
                return out
            return call

        for name in watched:
            originals[name] = getattr(ops, name)
            setattr(ops, name, timed(name, originals[name]))
        try:
            run()
            torch.cuda.synchronize()
        finally:
            for name, fn in originals.items():
                setattr(ops, name, fn)
        out = {}
        for kind, first, last, b, f in spans:
            ms, ideal = out.get(kind, (0.0, 0.0))
            out[kind] = (ms + first.elapsed_time(last), ideal + 1000 * max(b / read_bps, f / mfma_flops))
        return {k: {"ms": round(ms, 4), "x_roofline": round(ms / ideal, 2) if ideal else None} for k, (ms, ideal) in sorted(out.items())}

    def measure(model, vocab, window=0, per_call_masks=False):
        """window: the most keys a query of the model's attention sees (0: all before it), for the attention's flops.
        per_call_masks: the layers' masks differ, so every attention call is priced by its own (keys_of_call)."""
        def keys_seen(lengths):
            return sum(min(n, window) if window else n for n in lengths)

        out = {}
        for n in (512, 2048):
            engine = Engine(model, max_tokens=n + 64, max_slots=1, use_graphs=False)
            times = []
            for i in range(4):
                slot = engine.new_sequence()
                ids = [rng.randrange(vocab) for _ in range(n)]
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                engine.step([slot], [ids], "last")
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                engine.end_sequence(slot)
            t = sorted(times[1:])[1]
            out[f"prefill_{n}_tok_s"] = round(n / t, 1)
            out[f"prefill_{n}_ms"] = round(1000 * t, 3)
            if n == 2048:
                slot = engine.new_sequence()
                state.update(keys_read=keys_seen(range(1, n + 1)), keys_loaded=n, runs=[(0, n)] if per_call_masks else None)
                out["prefill_2048_kernels"] = classes_of_a_step(lambda: engine.step([slot], [ids], "last"))
                engine.end_sequence(slot)
            del engine
        for batch, prompt in ((1, 1024), (8, 1024), (64, 1024), (8, 7000)):
            steps, warmup = 32, 4
            lens = [rng.randint(prompt // 2, prompt) for _ in range(batch)]
            room = sum(-(-(n + steps + warmup + 16) // 64) * 64 for n in lens)
            engine = Engine(model, max_tokens=room, max_slots=batch)
            slots = [engine.new_sequence() for _ in range(batch)]
            tokens = []
            for b in range(batch):
                logits = engine.step([slots[b]], [[rng.randrange(vocab) for _ in range(lens[b])]], "last")
                tokens += choose(logits, greedy).tolist()

            def run(n):
                nonlocal tokens
                done = 0
                while done < n:
                    ahead = min(4, n - done)
                    tokens = engine.decode_and_choose_many(slots, tokens, greedy, steps=ahead)[-1]
                    done += ahead

            run(warmup)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            run(steps)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            name = f"decode_b{batch}_ctx{prompt}"
            out[f"{name}_tok_s"] = round(batch * steps / dt, 1)
            out[f"{name}_ms"] = round(1000 * dt / steps, 3)
            if (batch, prompt) in ((8, 1024), (8, 7000)):
                now = [n + warmup + steps + 1 for n in lens]
                state.update(keys_read=keys_seen(now), keys_loaded=keys_seen(now), runs=[(m - 1, 1) for m in now] if per_call_masks else None)
                out[f"{name}_kernels"] = classes_of_a_step(lambda: engine.step(slots, [[t] for t in tokens], "last"))
            for s in slots:
                engine.end_sequence(s)
            del engine
            torch.cuda.empty_cache()
        return out

    record = {"workload": f"{design} beside {'zodolorn' if design == 'sidalorn' else 'llama'} at equal layer sizes", "layers": layers, "dtype": "bf16",
              "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
              "peak_measured": {"read_gbs": round(read_bps / 1e9, 1), "mfma_tflops": round(mfma_flops / 1e12, 1)}, "sizes": {}}
    if design == "basopel":
        from fms_amd.architectures.basopel import make_config as make_basopel

        for name, width, pattern, heads, kv, dim, ff, span, kv_rank, vocab in BASOPEL_SIZES:
            pattern = (pattern * layers)[:layers]
            config = make_basopel(width=width, vocab=vocab, pattern=pattern, heads=heads, kv_heads=kv, dim=dim, vdim=dim, ff=ff, chunk=span,
                                  window=span, latent_window=span, kv_rank=kv_rank, latent_rot=64, rot_dims=dim // 2, rot_factor=4.0,
                                  max_positions=context)
            model = fms_amd.from_config(config, "basopel", data_type="bf16", random_seed=args.seed)
            mine = measure(model, vocab, per_call_masks=True)
            del model
            torch.cuda.empty_cache()
            # Llama of the same width, depth, heads and gated feed-forward (its attention sees every earlier key)
            llama = fms_amd.get_model("llama", "micro", data_type="bf16", random_seed=args.seed, emb_dim=width, nheads=heads, kvheads=kv,
                                      nlayers=layers, hidden_dim=ff, src_vocab_size=vocab, max_expected_seq_len=context)
            theirs = measure(llama, vocab, per_call_masks=True)
            del llama
            torch.cuda.empty_cache()
            record["sizes"][name] = {"basopel": dict(config=dict(width=width, pattern=pattern, heads=heads, kv_heads=kv, dim=dim, ff=ff,
                                                                   chunk=span, window=span, kv_rank=kv_rank, vocab=vocab), **mine),
                                     "llama": dict(config=dict(width=width, heads=heads, kvheads=kv, head_dim=width // heads, hidden=ff,
                                                               vocab=vocab), **theirs)}
        print(json.dumps(record))
        return 0
    if design == "defapel":
        from fms_amd.architectures.defapel import make_config as make_defapel

        for name, width, pattern, heads, kv, dim, window, dheads, dkv, ddim, dvdim, experts, top, expert_ff, vocab in DEFAPEL_SIZES:
            pattern = (pattern * layers)[:layers]
            config = make_defapel(width=width, vocab=vocab, pattern=pattern, heads=heads, kv_heads=kv, dim=dim, vdim=dim, window=window,
                                  delta_heads=dheads, delta_kv_heads=dkv, delta_dim=ddim, delta_vdim=dvdim, experts=experts, top=top,
                                  expert_ff=expert_ff, max_positions=context)
            model = fms_amd.from_config(config, "defapel", data_type="bf16", random_seed=args.seed)
            mine = measure(model, vocab, window=window)
            del model
            torch.cuda.empty_cache()
            # Llama of the same width, depth and heads; its gated feed-forward has the parameters of the experts a token uses
            hidden = top * expert_ff
            llama = fms_amd.get_model("llama", "micro", data_type="bf16", random_seed=args.seed, emb_dim=width, nheads=heads, kvheads=kv,
                                      nlayers=layers, hidden_dim=hidden, src_vocab_size=vocab, max_expected_seq_len=context)
            theirs = measure(llama, vocab)
            del llama
            torch.cuda.empty_cache()
            record["sizes"][name] = {"defapel": dict(config=dict(width=width, pattern=pattern, heads=heads, kv_heads=kv, dim=dim, window=window,
                                                                   delta_heads=dheads, delta_kv_heads=dkv, delta_dim=ddim, delta_vdim=dvdim,
                                                                   experts=experts, top=top, expert_ff=expert_ff, vocab=vocab), **mine),
                                     "llama": dict(config=dict(width=width, heads=heads, kvheads=kv, head_dim=width // heads, hidden=hidden,
                                                               vocab=vocab), **theirs)}
        print(json.dumps(record))
        return 0
    if design == "sidalorn":
        from fms_amd.architectures.sidalorn import make_config as make_sidalorn

        for (name, width, pattern, heads, (dim, vdim, kv_rank), channels, blocks, dense_ff, experts, identity, top, expert_ff, shared_ff,
             groups, keep, norm_groups, vocab) in SIDALORN_SIZES:
            pattern = (pattern * layers)[:layers]
            config = make_sidalorn(width=width, vocab=vocab, pattern=pattern, heads=heads, dim=dim, vdim=vdim, kv_rank=kv_rank,
                                   recurrent_width=channels, blocks=blocks, dense_ff=dense_ff, experts=experts, top=top, expert_ff=expert_ff,
                                   identity=identity, shared_ff=shared_ff, group_count=groups, group_keep=keep, route_scale=2.0,
                                   norm_groups=norm_groups, max_positions=context)
            model = fms_amd.from_config(config, "sidalorn", data_type="bf16", random_seed=args.seed)
            mine = measure(model, vocab)
            del model
            torch.cuda.empty_cache()
            # Zodolorn of the same width, depth, heads, latent and feed-forward sizes (its keys also carry a rotated part,
            # its queries pass a latent of their own, its experts have gates)
            other = make_config(width=width, vocab=vocab, nlayers=layers, heads=heads, dim=dim, rot_dim=64, vdim=vdim, q_rank=3 * kv_rank // 2,
                                kv_rank=kv_rank, dense_ff=dense_ff, experts=experts + identity, top=top, expert_ff=expert_ff,
                                shared_ff=shared_ff, max_positions=context)
            zodolorn = fms_amd.from_config(other, "zodolorn", data_type="bf16", random_seed=args.seed)
            theirs = measure(zodolorn, vocab)
            del zodolorn
            torch.cuda.empty_cache()
            record["sizes"][name] = {"sidalorn": dict(config=dict(width=width, pattern=pattern, heads=heads, dim=dim, vdim=vdim, kv_rank=kv_rank,
                                                                    recurrent_width=channels, blocks=blocks, dense_ff=dense_ff, experts=experts,
                                                                    identity=identity, top=top, expert_ff=expert_ff, shared_ff=shared_ff,
                                                                    groups=groups, keep=keep, norm_groups=norm_groups, vocab=vocab), **mine),
                                     "zodolorn": dict(config=dict(width=width, heads=heads, dim=dim, rot_dim=64, vdim=vdim, q_rank=3 * kv_rank // 2,
                                                                    kv_rank=kv_rank, dense_ff=dense_ff, experts=experts + identity, top=top,
                                                                    expert_ff=expert_ff, shared_ff=shared_ff, vocab=vocab), **theirs)}
        print(json.dumps(record))
        return 0
    for name, width, heads, (dim, rot, vdim, q_rank, kv_rank), dense_ff, experts, top, expert_ff, shared_ff, vocab in ZODOLORN_SIZES:
        config = make_config(width=width, vocab=vocab, nlayers=layers, heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=q_rank,
                             kv_rank=kv_rank, dense_ff=dense_ff, experts=experts, top=top, expert_ff=expert_ff, shared_ff=shared_ff,
                             max_positions=context)
        model = fms_amd.from_config(config, "zodolorn", data_type="bf16", random_seed=args.seed)
        mine = measure(model, vocab)
        del model
        torch.cuda.empty_cache()
        # Llama of the same width, depth and heads; its gated feed-forward has the parameters of the plain one (2/3 of its width)
        hidden = -(-dense_ff * 2 // 3 // 256) * 256
        llama = fms_amd.get_model("llama", "micro", data_type="bf16", random_seed=args.seed, emb_dim=width, nheads=heads, kvheads=8,
                                  nlayers=layers, hidden_dim=hidden, src_vocab_size=vocab, max_expected_seq_len=context)
        theirs = measure(llama, vocab)
        del llama
        torch.cuda.empty_cache()
        record["sizes"][name] = {"zodolorn": dict(config=dict(width=width, heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=q_rank,
                                                                kv_rank=kv_rank, dense_ff=dense_ff, experts=experts, top=top,
                                                                expert_ff=expert_ff, shared_ff=shared_ff, vocab=vocab), **mine),
                                 "llama": dict(config=dict(width=width, heads=heads, kvheads=8, head_dim=width // heads, hidden=hidden,
                                                           vocab=vocab), **theirs)}
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
