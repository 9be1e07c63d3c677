"""The command line, in the manner of the reference's runner (src/bin/runner.rs:24-123): the same
option names and meanings where it has them.

    runner <MODEL_DIR> [-p PROMPT] [-n N] [--chat [--think]] [--temperature T] [--top-k K] [--top-p P]
           [--repetition-penalty R] [--seed S] [--ignore-eos] [--max-pages N] [--pages-per-seq N]
           [-t THREADS] [--device cuda|cpu] [--dtype bfloat16|float32] [--profile] [--random [--random-seed S]]

The prompt is text when the model folder has a tokenizer.json (read with the `tokenizers` package),
else a list of token ids (`-p "5 17 3"` or `--prompt-ids 5,17,3`); it is read from standard input when
omitted.  Several prompts (repeat `-p`, or one per input line with `--batch`) are served as a batch.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

from ..sampling import DEFAULT_SEED


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="runner", description="Text generation with a Qwen3 checkpoint on one MI355X")
    ap.add_argument("model_dir", help="HuggingFace checkpoint directory (config.json, *.safetensors, tokenizer.json)")
    ap.add_argument("-p", "--prompt", action="append", help="prompt text or token ids; read from stdin when omitted")
    ap.add_argument("--prompt-ids", action="append", help="a prompt as comma-separated token ids")
    ap.add_argument("--batch", action="store_true", help="read one prompt per line of standard input")
    ap.add_argument("-n", "--max-new-tokens", type=int, default=600, help="number of tokens to generate")
    ap.add_argument("--chat", action="store_true", help="wrap the prompt in the Qwen chat template")
    ap.add_argument("--think", action="store_true", help="with --chat, leave thinking mode enabled")
    ap.add_argument("--ignore-eos", action="store_true", help="keep generating past end-of-sequence tokens")
    ap.add_argument("--tokenizer", help="directory holding tokenizer.json, if not the model directory")
    ap.add_argument("--max-pages", type=int, default=256, help="KV cache pages per layer (a page holds 32 tokens, as the reference's: src/kvcache.rs:12)")
    ap.add_argument("--pages-per-seq", type=int, default=128, help="maximum KV pages per sequence")
    ap.add_argument("-t", "--threads", type=int, default=None, help="host worker threads (defaults to all cores)")
    ap.add_argument("--profile", action="store_true", help="print a per-step timing summary at the end")
    ap.add_argument("--temperature", type=float, default=0.0, help="sampling temperature; 0 = greedy")
    ap.add_argument("--top-k", type=int, default=0, help="keep only the k most likely tokens (0 = off)")
    ap.add_argument("--top-p", type=float, default=1.0, help="nucleus sampling threshold (1.0 = off)")
    ap.add_argument("--repetition-penalty", type=float, default=1.0, help="penalty for tokens already in the context")
    ap.add_argument("--seed", type=lambda s: int(s, 0), default=DEFAULT_SEED, help="sampling seed")
    ap.add_argument("--device", default="cuda", choices=["cuda", "cpu"],
                    help="cuda: the HIP kernels; cpu: the plain backend (float32, slow: for reading a checkpoint's "
                    "output without a GPU)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"], help="compute precision")
    ap.add_argument("--stop-token-ids", default=None, help="comma-separated ids that end a sequence "
                    "(default: eos_token_id of generation_config.json or config.json, if present)")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel")
    ap.add_argument("--batch-invariant", action="store_true", help="bfloat16 on the GPU: every step runs the same form "
                    "of every kernel, so that a request's tokens do not depend on its batch (slower, above all on prompts)")
    ap.add_argument("--random", action="store_true", help="MODEL_DIR needs only a config.json (or is one): the weights "
                    "are made in memory, N(0, 0.02) with gains 1 + N(0, 0.1), from --random-seed")
    ap.add_argument("--random-seed", type=int, default=0, help="seed of the weights made by --random")
    return ap


def chat_prompt(user: str, enable_thinking: bool) -> str:
    """The Qwen chat format for a single user turn; without thinking, an empty think block opens the
    answer (src/tokenizer/mod.rs:402-408)."""
    text = f"<|im_start|>user\n{user}<|im_end|>\n<|im_start|>assistant\n"
    if not enable_thinking:
        text += "<think>\n\n</think>\n\n"
    return text


class StreamPrinter:
    """Prints a sequence's text as its tokens arrive, holding back bytes that do not yet form whole
    characters (the reference's StreamDecoder: src/tokenizer/mod.rs:411-416)."""

    def __init__(self, tokenizer, out=sys.stdout):
        self.tokenizer, self.out, self.ids, self.printed = tokenizer, out, [], 0

    def push(self, token: int) -> None:
        if self.tokenizer is None:
            self.out.write(f"{token} ")
        else:
            self.ids.append(token)
            text = self.tokenizer.decode(self.ids)
            if not text.endswith("\ufffd"):                 # an unfinished character decodes to U+FFFD: wait for the rest
                self.out.write(text[self.printed:])
                self.printed = len(text)
        self.out.flush()


def load_tokenizer(folder: str):
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.exists(path):
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(path)


def default_stop_ids(model_dir: str) -> list[int]:
    for name in ("generation_config.json", "config.json"):
        path = os.path.join(model_dir, name)
        if os.path.exists(path):
            with open(path) as f:
                eos = json.load(f).get("eos_token_id")
            if eos is not None:
                return [int(e) for e in (eos if isinstance(eos, list) else [eos])]
    return []


def parse_ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = build_parser()
    args = ap.parse_args(argv)
    if args.think and not args.chat:
        ap.error("--think requires --chat")
    if args.threads:
        import torch
        torch.set_num_threads(args.threads)
    tokenizer = load_tokenizer(args.tokenizer or args.model_dir)
    if args.chat and tokenizer is None:
        print("error: --chat wraps text and needs a tokenizer.json", file=sys.stderr)
        return 1
    raw = list(args.prompt or [])
    try:
        id_prompts = [parse_ids(p) for p in (args.prompt_ids or [])]
    except ValueError:
        print("error: --prompt-ids takes token ids separated by commas or spaces", file=sys.stderr)
        return 1
    if not raw and not id_prompts:
        lines = [ln.rstrip("\n") for ln in sys.stdin]
        raw = [ln for ln in lines if ln.strip()] if args.batch else ["\n".join(lines).strip()]
    prompts = list(id_prompts)
    for p in raw:
        if args.chat:
            p = chat_prompt(p, args.think)                             # src/bin/runner.rs:233
        if tokenizer is not None:
            prompts.append(tokenizer.encode(p).ids)
            continue
        try:
            prompts.append(parse_ids(p))
        except ValueError:
            print(f"error: the prompt is text, and {args.tokenizer or args.model_dir} has no tokenizer.json to encode "
                  "it with: give token ids (-p \"5 17 3\" or --prompt-ids 5,17,3)", file=sys.stderr)
            return 1
    if not prompts or any(len(p) == 0 for p in prompts):
        print("error: empty prompt", file=sys.stderr)                  # src/bin/runner.rs:235-237
        return 1

    from .. import profiler
    from ..api import Model
    from ..cache import PAGE_SIZE
    from ..errors import InferenceError
    profiler.enable(args.profile)                                      # src/bin/runner.rs:207
    t0 = time.perf_counter()
    try:
        per_seq = args.pages_per_seq * PAGE_SIZE
        options = dict(max_batch=min(len(prompts), 64), max_seq_len=per_seq, max_tokens=args.max_pages * PAGE_SIZE,
                       use_graphs=not args.no_graphs)
        if args.device == "cpu":
            if args.random or args.profile:
                print("error: --device cpu reads a model folder and has no section timers", file=sys.stderr)
                return 1
            model = Model.load(args.model_dir, dtype="float32", device="cpu", **options)
        elif args.random:
            path = args.model_dir if os.path.isfile(args.model_dir) else os.path.join(args.model_dir, "config.json")
            with open(path) as f:
                model = Model.random(json.load(f), seed=args.random_seed, dtype=args.dtype,
                                     batch_invariant=args.batch_invariant, **options)
        else:
            model = Model.load(args.model_dir, dtype=args.dtype, batch_invariant=args.batch_invariant, **options)
    except (InferenceError, OSError, ValueError, json.JSONDecodeError) as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    print(f"loaded {args.model_dir} in {time.perf_counter() - t0:.2f} s", file=sys.stderr)
    stop = parse_ids(args.stop_token_ids) if args.stop_token_ids is not None else default_stop_ids(args.model_dir)

    single = len(prompts) == 1
    printer = StreamPrinter(tokenizer)

    def on_token(request, token):
        if single:                                                     # streamed, as the reference prints
            printer.push(token)

    try:
        res = model.generate(prompts, max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                             top_k=args.top_k, top_p=args.top_p, repetition_penalty=args.repetition_penalty,
                             seed=args.seed, stop_token_ids=stop, ignore_eos=args.ignore_eos, on_token=on_token)
    except InferenceError as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    if single:
        print()
    else:
        for toks in res.tokens:
            print(tokenizer.decode(toks) if tokenizer is not None else " ".join(str(t) for t in toks))
    st = res.stats
    print(f"prefill: {st.prompt_tokens} tokens in {st.prefill_seconds:.3f} s ({st.prefill_tokens_per_second:.1f} tok/s)",
          file=sys.stderr)                                             # src/bin/runner.rs:243-251
    print(f"decode: {st.decode_tokens} tokens in {st.decode_seconds:.3f} s ({st.decode_tokens_per_second:.1f} tok/s)",
          file=sys.stderr)
    if args.profile:
        per_step = 1e3 * st.decode_seconds / st.decode_steps if st.decode_steps else 0.0
        print(f"profile: {st.batches} batches, {st.decode_steps} decode steps, {per_step:.3f} ms per step",
              file=sys.stderr)
        print("\n" + profiler.report(), file=sys.stderr)                # src/bin/runner.rs:252-254
    return 0
