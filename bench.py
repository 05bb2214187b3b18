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


if __name__ == "__main__":
    sys.exit(main())
