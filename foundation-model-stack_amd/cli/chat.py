"""A conversation at the terminal, in the manner of the reference's scripts/chat.py (:32-116 its options,
:162-281 its loop).

    python -m fms_amd.cli.chat --architecture hf_pretrained --model_path DIR --tokenizer DIR
    python -m fms_amd.cli.chat --architecture llama --variant micro --tokenizer char_tokenizer   # random weights

The conversation is kept as one list of token ids in the Llama-2 chat layout that the reference's script
describes (:162-173):

    <bos> <<SYS>>\\n system \\n<</SYS>>\\n\\n [INST] question [/INST] answer <eos> [INST] question [/INST] answer <eos> ...

The reference runs the whole list through `generate` at every question (:224-240); here the conversation
keeps its sequence in the cache, and a question runs only the tokens that are new.  Lines that
start with a slash are commands (/help, /set max_new_tokens=N, /buffer, /quit); anything else goes to the model.
(The reference's code closes the system message with a second "<<SYS>>", :184; the layout it cites closes it
with "<</SYS>>", which is what is written here.)
"""

from __future__ import annotations

import argparse
import re
import sys
from typing import Callable, List, Optional

B_SYS, E_SYS = "<<SYS>>\n", "\n<</SYS>>\n\n"
B_INST, E_INST = "[INST]", "[/INST]"

HELP = """Help on using the chat:
/help - show this message.
/set max_new_tokens=<value> - the longest answer, in tokens; longer answers are cut off.
/buffer - show the whole conversation as it is fed to the model.
/quit or /exit - leave (so do ctrl-c and ctrl-d).
Any other input is text for the model."""


class Conversation:
    """The token ids of a conversation and the turns that extend it.

    answer(ids, max_new_tokens) -> the new token ids for the conversation so far (a final end-of-text token may
    be among them or not; it is not kept twice).  The tokenizer needs encode, decode, bos_token_id, eos_token_id."""

    def __init__(self, tokenizer, answer: Callable[[List[int], int], List[int]], system_message: Optional[str] = None,
                 max_new_tokens: int = 500):
        self.tokenizer = tokenizer
        self.answer = answer
        self.max_new_tokens = max_new_tokens
        self.ids: List[int] = [tokenizer.bos_token_id]
        if system_message:
            self.ids += list(tokenizer.encode(B_SYS + system_message + E_SYS))

    def ask(self, text: str) -> str:
        eos = self.tokenizer.eos_token_id
        asked = list(self.tokenizer.encode(B_INST + text + E_INST))
        new = [int(t) for t in self.answer(self.ids + asked, self.max_new_tokens)]  # a question that is refused is not kept
        self.ids += asked
        if eos in new:  # nothing after the end of the answer is kept
            new = new[:new.index(eos)]
        self.ids += new + [eos]
        return self.tokenizer.decode(new)

    def text(self) -> str:
        return self.tokenizer.decode(self.ids)


def run_line(conversation: Conversation, line: str, out) -> bool:
    """One line of input; False when the conversation is over."""
    line = line.rstrip("\n")
    if not line.strip():
        return True
    if not line.startswith("/"):
        print(conversation.ask(line), file=out, flush=True)
        return True
    command, _, rest = line[1:].strip().partition(" ")
    if command in ("quit", "exit", "EOF"):
        print("Exiting...", file=out)
        return False
    if command == "help":
        print(HELP, file=out)
    elif command == "buffer":
        print(f"The conversation has {len(conversation.ids)} tokens:", file=out)
        print(conversation.text(), file=out)
    elif command == "set":
        parts = [p for p in re.split(r"[=\s]+", rest.strip()) if p]
        if len(parts) != 2 or parts[0] != "max_new_tokens" or not parts[1].isdigit() or int(parts[1]) < 1:
            print("usage: /set max_new_tokens=100", file=out)
        else:
            conversation.max_new_tokens = int(parts[1])
    else:
        print(f"Unknown command: {line}", file=out)
    return True


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(description="Interactive chat with a causal model")
    p.add_argument("--device_type", type=str, default="cuda")
    p.add_argument("--architecture", type=str, default="llama", help="The model architecture")
    p.add_argument("--variant", type=str, default=None, help="The model variant (configuration). E.g. 7b, 3-8b, micro.")
    p.add_argument("--model_path", type=str, help="Path to the folder or file with the weights (safetensors)")
    p.add_argument("--model_source", type=str, help="Source of the checkpoint. E.g. 'meta', 'hf', None")
    p.add_argument("--tokenizer", type=str, required=True, help="'char_tokenizer', a sentencepiece model, or a tokenizer.json")
    p.add_argument("--no_use_cache", action="store_false", help="Accepted for compatibility: this engine always uses its cache")
    p.add_argument("--compile", action="store_true", help="Accepted for compatibility: there is no tracing compiler here")
    p.add_argument("--compile_mode", type=str, default="default", choices=["default", "reduce-overhead"])
    p.add_argument("--deterministic", action="store_true", help="Greedy answers and fixed seeds (42), as the reference does")
    p.add_argument("--distributed", action="store_true", help="Not supported: one process drives one GPU")
    p.add_argument("--max_new_tokens", type=int, default=500, help="Maximum number of new tokens for each answer")
    p.add_argument("--system_message", type=str, default="",
                   help="Tells the chat how to behave; empty (the default here) for none.  The reference's default is "
                        "Llama-2's stock system message: pass it here to have it.")
    # beyond the reference's options
    p.add_argument("--default_dtype", type=str, default=None, choices=["bf16", "fp32"], help="Overrides the checkpoint's weight format")
    p.add_argument("--temperature", type=float, default=1.0)
    p.add_argument("--top_k", type=int, default=10)
    p.add_argument("--random_seed", type=int, default=0, help="seed of the random weights when no --model_path is given")
    return p


def main(argv=None, stdin=None, stdout=None) -> int:
    args = build_parser().parse_args(argv)
    stdin, stdout = stdin or sys.stdin, stdout or sys.stdout
    if args.distributed:
        print("--distributed: this library runs one process on one GPU", file=sys.stderr)
        return 2
    if args.architecture not in ("hf_pretrained", "hf_configured") and args.variant is None:
        print("--variant is needed with --architecture", args.architecture, file=sys.stderr)
        return 2

    from .. import get_model
    from ..engine import Engine
    from ..sampling import SamplingParams, choose
    from ..tokenizers import get_tokenizer

    print("loading model", file=stdout, flush=True)
    try:
        if args.architecture in ("hf_pretrained", "hf_configured"):
            model = get_model(args.architecture, model_path=args.model_path or args.variant, device_type=args.device_type,
                              data_type=args.default_dtype, random_seed=args.random_seed)
        else:
            model = get_model(args.architecture, args.variant, model_path=args.model_path, device_type=args.device_type,
                              source=args.model_source, data_type=args.default_dtype, random_seed=args.random_seed)
    except (RuntimeError, KeyError, ValueError, FileNotFoundError) as err:
        print(f"could not load the model: {err}", file=sys.stderr)
        return 1
    tokenizer = get_tokenizer(args.tokenizer)
    print("loading complete", file=stdout, flush=True)

    # The conversation keeps its place in the cache: a question runs only the tokens that are new since the last
    # answer (the reference's script runs the whole conversation again at every question, scripts/chat.py:224-240).
    engine = Engine(model, max_tokens=model.spec.max_seq_len, max_slots=1)
    slot = engine.new_sequence()
    sampling = SamplingParams(do_sample=not args.deterministic, temperature=args.temperature, top_k=args.top_k)
    turn = [0]

    def answer(ids: List[int], max_new_tokens: int) -> List[int]:
        held = engine.length(slot)  # the conversation up to the last token that was fed
        room = model.spec.max_seq_len - len(ids)
        if room < 1:
            raise ValueError(f"the conversation has {len(ids)} tokens, the model takes {model.spec.max_seq_len}")
        turn[0] += 1
        seed = 42 if args.deterministic else turn[0]
        logits = engine.step([slot], [ids[held:]], "last")
        new = choose(logits, sampling, [seed], [0]).tolist()
        while new[-1] != tokenizer.eos_token_id and len(new) < min(max_new_tokens, room):
            new += engine.decode_and_choose([slot], [new[-1]], sampling, [seed], [len(new)])
        return new

    conversation = Conversation(tokenizer, answer, args.system_message, args.max_new_tokens)
    print('Enter your prompts/questions or "/help" for usage instructions.\n', file=stdout, flush=True)
    interactive = stdin.isatty() if hasattr(stdin, "isatty") else False
    try:
        while True:
            if interactive:
                print("$ ", end="", file=stdout, flush=True)
            line = stdin.readline()
            if not line:  # ctrl-d, or the end of piped input
                print("Exiting...", file=stdout)
                return 0
            try:
                if not run_line(conversation, line, stdout):
                    return 0
            except ValueError as err:  # a conversation longer than the model takes
                print(f"error: {err}", file=stdout, flush=True)
    except KeyboardInterrupt:
        print("keyboard interrupt, exiting.", file=stdout)
        return 0


if __name__ == "__main__":
    sys.exit(main())
