"""Command line in the manner of the reference's scripts/inference.py (:23-113, :155-281).

    python -m fms_amd.cli.inference --architecture llama --variant micro --tokenizer char_tokenizer
    python -m fms_amd.cli.inference --architecture hf_pretrained --model_path DIR --tokenizer DIR

Option names and meanings are the reference's where it has them.  Options that steer things
this library does differently are accepted and answered with a note: the cache is always used,
weights stay fused, there is no tracing compiler, and one process drives one GPU.
"""

from __future__ import annotations

import argparse
import sys
import time

TEMPLATE = ("Below is an instruction that describes a task. Write a response that appropriately completes the request."
            "\n\n### Instruction:\n{}\n\n### Response:")


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(description="Script to run inference on a causal model")
    p.add_argument("--device_type", type=str, default="cuda")
    p.add_argument("--architecture", type=str, default="llama", help="The model architecture to run")
    p.add_argument("--variant", type=str, default=None, help="The model variant (configuration). E.g. 7b, 3-8b, micro.")
    p.add_argument("--model_path", type=str, help="Path to the folder or file with the weights (safetensors)")
    p.add_argument("--model_source", type=str, help="Source of the checkpoint. E.g. 'meta', 'hf', None")
    p.add_argument("--tokenizer", type=str, required=True, help="'char_tokenizer', a sentencepiece model, or a tokenizer.json")
    p.add_argument("--no_use_cache", action="store_false", help="Accepted for compatibility: this engine always uses its cache")
    p.add_argument("--unfuse_weights", action="store_true", help="Accepted for compatibility: weights stay fused on the device")
    p.add_argument("--default_dtype", type=str, default=None, choices=["bf16", "fp16", "fp32"],
                   help="Overrides the checkpoint's weight format (fp16 is not supported)")
    p.add_argument("--compile", action="store_true", help="Accepted for compatibility: there is no tracing compiler here")
    p.add_argument("--compile_mode", type=str, default="default", choices=["default", "reduce-overhead"])
    p.add_argument("--deterministic", action="store_true", help="Fix the seeds (42), as the reference does")
    p.add_argument("--distributed", action="store_true", help="Not supported: one process drives one GPU")
    p.add_argument("--batch_input", action="store_true", help="use a batch of prompts as input")
    p.add_argument("--min_pad_length", type=int, default=0, help="Pad inputs to a minimum length (padding never reaches the model)")
    p.add_argument("--attn_name", type=str, default="sdpa_causal", help="Only causal attention (sdpa_causal) exists here")
    p.add_argument("--context_file", type=str, default=None, help="File to summarize")
    # what the reference fixes in its script, as options
    p.add_argument("--max_new_tokens", type=int, default=100)
    p.add_argument("--do_sample", action="store_true", help="sample with --temperature and --top_k instead of greedy decoding")
    p.add_argument("--temperature", type=float, default=1.0)
    p.add_argument("--top_k", type=int, default=10)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--prompt", type=str, action="append", help="a prompt of your own (may be given several times)")
    p.add_argument("--prompt_ids", type=str, action="append", help="a prompt as comma separated token ids")
    p.add_argument("--random_seed", type=int, default=0, help="seed of the random weights when no --model_path is given")
    return p


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.distributed:
        print("--distributed: this library runs one process on one GPU", file=sys.stderr)
        return 2
    if args.attn_name != "sdpa_causal":
        print(f"--attn_name {args.attn_name}: only causal attention (sdpa_causal) exists here", file=sys.stderr)
        return 2
    if args.default_dtype == "fp16":
        print("--default_dtype fp16: models run in bf16 or fp32 here", file=sys.stderr)
        return 2
    for flag, note in ((not args.no_use_cache, "--no_use_cache: the engine always uses its cache"),
                       (args.unfuse_weights, "--unfuse_weights: weights stay fused on the device"),
                       (args.compile, "--compile: nothing to compile, the kernels are built ahead")):
        if flag:
            print("note:", note, file=sys.stderr)

    import torch

    from .. import get_model
    from ..generation import generate, pad_input_ids, trim_prefix, truncate_after_eos
    from ..tokenizers import get_tokenizer

    seed = 42 if args.deterministic else args.seed
    if args.architecture not in ("hf_pretrained", "hf_configured") and args.variant is None:
        print("--variant is needed with --architecture", args.architecture, file=sys.stderr)
        return 2
    print("loading model")
    try:
        if args.architecture in ("hf_pretrained", "hf_configured"):
            model = get_model(args.architecture, model_path=args.model_path or args.variant, device_type=args.device_type,
                              data_type=args.default_dtype, random_seed=args.random_seed)
        else:
            model = get_model(args.architecture, args.variant, model_path=args.model_path, device_type=args.device_type,
                              source=args.model_source, data_type=args.default_dtype, random_seed=args.random_seed)
    except (RuntimeError, KeyError, ValueError, FileNotFoundError) as err:  # no GPU, unknown names, a checkpoint that does not fit
        print(f"could not load the model: {err}", file=sys.stderr)
        return 1
    tokenizer = get_tokenizer(args.tokenizer)
    print("loading complete")

    def ids_for_prompt(text):
        return torch.tensor([tokenizer.bos_token_id] + list(tokenizer.encode(text)), dtype=torch.long)

    prompts = []
    for text in args.prompt or []:
        prompts.append(ids_for_prompt(text))
    for ids in args.prompt_ids or []:
        prompts.append(torch.tensor([int(t) for t in ids.split(",")], dtype=torch.long))
    if not prompts:
        if args.context_file is not None:
            with open(args.context_file) as f:
                long_prompt = f.read()
            texts = [long_prompt + "\nPlease give me a brief summary of this research paper in a few bullet points.",
                     long_prompt + "\nPlease write me the abstract for this paper."]
        else:
            texts = [TEMPLATE.format("Provide a list of instructions for preparing chicken soup."),
                     TEMPLATE.format("Explain some popular greetings in Spanish.")]
        prompts = [ids_for_prompt(t) for t in texts]
        if not args.batch_input:
            prompts = prompts[:1]

    padding_kwargs = None
    if len(prompts) > 1 or args.min_pad_length:
        ids, padding_kwargs = pad_input_ids(prompts, min_pad_length=args.min_pad_length)
    else:
        ids = prompts[0]

    print("generating output")
    print("use_cache True ;; do_sample", args.do_sample)
    print("==================")
    start = time.time()
    result = generate(model, ids, max_new_tokens=args.max_new_tokens, use_cache=True, do_sample=args.do_sample,
                      temperature=args.temperature, top_k=args.top_k, max_seq_len=model.spec.max_seq_len,
                      eos_token_id=tokenizer.eos_token_id, extra_kwargs=padding_kwargs, seed=seed)
    elapsed = time.time() - start
    if result.dim() == 1:
        result = result.unsqueeze(0)
    for row in result:
        if padding_kwargs is not None:
            row = trim_prefix(row)
        row = trim_prefix(row, tokenizer.bos_token_id)
        row = truncate_after_eos(row, tokenizer.eos_token_id)
        print(tokenizer.decode(row.tolist()))
        print()
    print(f"[{result.shape[0]} sequence(s), {elapsed:.2f} s]", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
