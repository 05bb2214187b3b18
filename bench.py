"""Serving benchmark: decode tokens per second of the Llama-3-8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Random weights, synthetic token ids.  A "step" is one decode step of the whole batch through
the library's own generation path (step function, cache, kernels, sampler).  One JSON line is
printed: decode tokens/s at batch 8 (`value`), the prefill of 2,048 tokens, the decode step's
memory roofline, and decode at batch 1 and 64.
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
    ap.add_argument("--skip-points", action="store_true", help="leave out decode at batch 1 and 64")
    ap.add_argument("--seed", type=int, default=0)
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
    from fms_amd.sampling import SamplingParams, choose

    full = variant_config("llama", args.variant)
    overrides = {"max_expected_seq_len": args.context}
    if args.layers is not None:
        overrides["nlayers"] = args.layers
    model = fms_amd.get_model("llama", args.variant, data_type="bf16", device_type="cuda", random_seed=args.seed, **overrides)
    cfg = model.config
    E, H, K, D, F, V, L = (cfg.emb_dim, cfg.nheads, cfg.kv_heads, cfg.head_dim, cfg.ffn_hidden_dim, cfg.src_vocab_size,
                           cfg.nlayers)
    layer_weights = (H + 2 * K) * D * E + E * H * D + 2 * F * E + E * F + 2 * E  # elements per layer, norms included
    step_weight_bytes = 2 * (L * layer_weights + E + V * E)  # everything but the embedding table, read once
    kv_bytes_per_token = 2 * L * K * D * 2
    greedy = SamplingParams(do_sample=False)
    rng = random.Random(args.seed)

    def decode(batch: int, steps: int, warmup: int):
        """(tokens/s, ms per step, bytes a step has to read) for `batch` sequences with prompts of 128..2048 tokens."""
        lens = [rng.randint(args.prompt_min, args.prompt_max) for _ in range(batch)]
        room = sum(-(-(n + steps + warmup + 1) // 64) * 64 for n in lens)
        engine = Engine(model, max_tokens=room, max_slots=batch)
        slots = [engine.new_sequence() for _ in range(batch)]
        tokens = None
        per_group = max(1, 16384 // args.prompt_max)  # prompts in groups, so that activations stay small
        for i in range(0, batch, per_group):
            group = list(range(i, min(i + per_group, batch)))
            prompts = [[rng.randrange(V) for _ in range(lens[b])] for b in group]
            logits = engine.step([slots[b] for b in group], prompts, "last")
            first = choose(logits, greedy).tolist()
            tokens = first if tokens is None else tokens + first
        for _ in range(warmup):
            tokens = engine.decode_and_choose(slots, tokens, greedy)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            tokens = engine.decode_and_choose(slots, tokens, greedy)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        mean_ctx = sum(lens) + batch * (1 + warmup + steps / 2)
        for s in slots:
            engine.end_sequence(s)
        del engine
        torch.cuda.empty_cache()
        return batch * steps / dt, 1000 * dt / steps, step_weight_bytes + kv_bytes_per_token * mean_ctx

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
        return n_tokens / t, 1000 * t, flops / t / PEAK_FLOPS["bf16"]

    pre_tps = pre_ms = pre_frac = 0.0
    tps = ms = step_bytes = 0.0
    if args.only != "decode":
        pre_tps, pre_ms, pre_frac = prefill(args.prefill_tokens)
    if args.only != "prefill":
        tps, ms, step_bytes = decode(args.batch, args.steps, args.warmup)
    achieved = step_bytes / (ms / 1000) / 1e9 if ms else 0.0
    points = {}
    if not args.skip_points and args.only is None:
        for b, steps, warmup in ((1, min(args.steps, 32), 4), (64, min(args.steps, 16), 2)):
            p_tps, p_ms, p_bytes = decode(b, steps, warmup)
            gbs = p_bytes / (p_ms / 1000) / 1e9
            points[f"decode_b{b}"] = round(p_tps, 1)
            points[f"decode_b{b}_ms"] = round(p_ms, 3)
            points[f"decode_b{b}_gb"] = round(p_bytes / 1e9, 3)
            points[f"decode_b{b}_gbs"] = round(gbs, 1)
            points[f"decode_b{b}_frac"] = round(gbs / HBM_GBS, 4)

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
        },
        "prefill": {"value": round(pre_tps, 1), "tokens": args.prefill_tokens, "ms": round(pre_ms, 3), "frac": round(pre_frac, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": points,
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())
