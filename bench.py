#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-8B-shaped model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C] [--model 8b|0.6b|1.7b|4b|14b|32b]

The default run has the layer sizes of Qwen3-8B with random weights
(N(0, 0.02), norm gains 1 + N(0, 0.1), seed 2), a batch of 8 and prompts of 2,048 tokens in a
context of 4,096.  A step is one decode step: every live sequence gets one more token, chosen
greedily on the device.  Prints one JSON line: decoded tokens a second at batch 8 (`value`), the
2,048-token prefill, the decode step's share of the HBM roofline, and under `points` decoding at batch 1
and 64 (tokens a second, and beside each its milliseconds a step, the GB/s of the bytes the step has to
read and their share of the HBM peak), then the two other workloads the baseline names: Qwen3-0.6B shapes
(16 prompts of 16 to 1,024 tokens, 256 steps, with the kernel launches a step costs) and Qwen3-32B shapes
(batch 1 after a prompt of 4,096 tokens).  A point that fails is left out; the headline never is.

Decoding is timed through the generation loop itself (`engine.generate`, greedy, stop tokens ignored): a
callback on the first request's tokens brackets exactly K decode steps, after W warm-up steps, with a
device synchronisation on both sides.
"""
import argparse
import gc
import json
import sys
import time

HBM_PEAK_GBS = 8000.0            # MI355X, published
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 151936, "hidden_size": 4096,
    "intermediate_size": 12288, "num_hidden_layers": 36, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
    "max_position_embeddings": 4096,
}

# The other two shapes that the baseline names: the small model whose decode step is bound by launches and
# latencies, and the large one (64 GB of weights).
QWEN3_0_6B = dict(QWEN3_8B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                  num_key_value_heads=8, tie_word_embeddings=True)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64,
                 num_key_value_heads=8)
# (and the three published sizes between them, for `--model`: not part of the default run)
QWEN3_1_7B = dict(QWEN3_8B, hidden_size=2048, intermediate_size=6144, num_hidden_layers=28, num_attention_heads=16,
                  num_key_value_heads=8, tie_word_embeddings=True)
QWEN3_4B = dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, num_hidden_layers=36, num_attention_heads=32,
                num_key_value_heads=8, tie_word_embeddings=True)
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=17408, num_hidden_layers=40, num_attention_heads=40,
                 num_key_value_heads=8)
MODELS = {"8b": ("Qwen3-8B shapes", QWEN3_8B, 2), "0.6b": ("Qwen3-0.6B shapes", QWEN3_0_6B, 3),
          "32b": ("Qwen3-32B shapes", QWEN3_32B, 4), "1.7b": ("Qwen3-1.7B shapes", QWEN3_1_7B, 5),
          "4b": ("Qwen3-4B shapes", QWEN3_4B, 6), "14b": ("Qwen3-14B shapes", QWEN3_14B, 7)}   # name, sizes, seed of the random weights


def layer_matrix_params(c):
    d, dh = c["hidden_size"], c["head_dim"]
    qkv = (c["num_attention_heads"] + 2 * c["num_key_value_heads"]) * dh * d
    return qkv + d * c["num_attention_heads"] * dh + 3 * d * c["intermediate_size"]


def decode_bytes(c, layers, batch, mean_context):
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    d = c["hidden_size"]
    weights = 2 * (layers * layer_matrix_params(c) + c["vocab_size"] * d + batch * d)        # bf16 (the head's matrix
    # is read once whether it is the embedding table or its own; of the table only the batch's rows are)
    gains = 4 * (layers * (2 * d + 2 * c["head_dim"]) + d)
    kv = batch * mean_context * layers * 2 * c["num_key_value_heads"] * c["head_dim"] * 2
    return weights + gains + kv


def prefill_flops(c, layers, tokens):
    linear = 2 * tokens * layers * layer_matrix_params(c) + 2 * c["vocab_size"] * c["hidden_size"]
    attention = layers * 4 * c["head_dim"] * c["num_attention_heads"] * tokens * (tokens + 1) // 2
    return linear + attention


class Bench:
    """One model's measurements."""

    def __init__(self, which, layers=None, context=4096, graphs=True):
        import torch
        from rust_inference_amd.parts import random_model
        self.torch = torch
        self.name, shapes, self.seed = MODELS[which]
        self.cfg = dict(shapes)
        self.full_layers = self.cfg["num_hidden_layers"]
        self.layers = layers or self.full_layers
        self.cfg["num_hidden_layers"] = self.layers
        self.cfg["max_position_embeddings"] = context
        self.context, self.graphs = context, graphs
        torch.manual_seed(self.seed)
        self.model = random_model(self.cfg, seed=self.seed, dtype=torch.bfloat16)
        self.gen = torch.Generator().manual_seed(self.seed)

    def prompts(self, batch, n, span=None):
        torch, vocab = self.torch, self.cfg["vocab_size"]
        if span and batch > 1:                                    # unequal lengths, prefilled together
            lens = torch.randint(span[0], span[1] + 1, (batch,), generator=self.gen).tolist()
            return [torch.randint(0, vocab, (m,), generator=self.gen).tolist() for m in lens]
        return torch.randint(0, vocab, (batch, n), generator=self.gen).tolist()

    def engine(self, batch):
        from rust_inference_amd.cache import PAGE_SIZE
        from rust_inference_amd.engine import Engine
        per_seq = -(-self.context // PAGE_SIZE) * PAGE_SIZE
        cache = self.model.new_cache(max_tokens=per_seq * batch, num_slots=batch, max_seq_len=self.context)
        return Engine(self.model, cache, use_graphs=self.graphs)

    def prefill(self, tokens):
        """Seconds of one prompt of `tokens` tokens with the logits at its last place (the best of two after a first)."""
        from rust_inference_amd.engine import StepEntry
        engine = self.engine(1)
        p = self.prompts(1, tokens)[0]
        times = []
        for _ in range(3):
            slot = engine.cache.acquire()
            self.torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.step([StepEntry(slot, p, "last")])
            self.torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            engine.cache.release(slot)
        return min(times[1:])

    def decode(self, batch, steps, warmup, prompt, span=None, count_launches=False):
        """`steps` decode steps of `batch` sequences through the generation loop after `warmup` untimed ones.
        Returns (seconds, mean number of keys a sequence attends in the timed steps, launches a step or None)."""
        from rust_inference_amd.engine import generate
        torch = self.torch
        warmup = max(1, warmup)                                   # the first decode step captures its graph
        engine = self.engine(batch)
        engine.keep_graphs = count_launches
        prompts = self.prompts(batch, prompt, span)
        marks = {}
        seen = [0]

        # Token i of a request (counted from 1) comes from the prompt (i = 1) or from decode step i - 1.  The loop
        # runs one step ahead of the ids it has read: when it hands over token i, step i has been launched.  A
        # synchronisation at token warmup + 1 therefore ends with step warmup + 1 done, one at token
        # warmup + 1 + steps with step warmup + 1 + steps done: exactly `steps` steps lie between them.
        def on_token(request, token):
            if request != 0:
                return
            seen[0] += 1
            if seen[0] == warmup + 1 or seen[0] == warmup + 1 + steps:
                torch.cuda.synchronize()
                marks[seen[0]] = time.perf_counter()

        res = generate(engine, prompts, max_new_tokens=warmup + steps + 2, ignore_eos=True, on_token=on_token)
        assert all(len(t) == warmup + steps + 2 for t in res.tokens)
        dt = marks[warmup + 1 + steps] - marks[warmup + 1]
        mean_prompt = sum(len(p) for p in prompts) / batch
        mean_context = mean_prompt + warmup + 1.5 + steps / 2.0   # step s attends prompt + s keys; s = warmup + 2 ...
        launches = None
        if count_launches:
            counts = engine.graph_launches()
            launches = max(counts.values()) if counts else None
        del engine
        return dt, mean_context, launches

    def point(self, batch, steps, warmup, prompt, span=None, count_launches=False):
        dt, ctx, launches = self.decode(batch, steps, warmup, prompt, span, count_launches)
        gbs = decode_bytes(self.cfg, self.layers, batch, ctx) / (dt / steps) / 1e9
        out = {"tok_s": round(batch * steps / dt, 1), "ms": round(1e3 * dt / steps, 3), "gbs": round(gbs, 1),
               "frac": round(gbs / HBM_PEAK_GBS, 4)}
        if launches is not None:
            out["launches"] = launches
        return out, ctx

    def close(self):
        self.model = None
        gc.collect()
        self.torch.cuda.empty_cache()


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--prompt-range", type=int, nargs=2, metavar=("LOW", "HIGH"), default=None,
                    help="decode after prompts of unequal lengths drawn uniformly from LOW..HIGH instead of --prompt")
    ap.add_argument("--model", choices=sorted(MODELS), default="8b", help="which shapes (default: Qwen3-8B)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points and the other models")
    ap.add_argument("--no-other-models", action="store_true", help="skip the Qwen3-0.6B and Qwen3-32B points")
    ap.add_argument("--no-graphs", action="store_true", help="launch every kernel of a decode step from the host")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this library is single-GPU, --gpus {args.gpus} is not run")
        return 2

    from rust_inference_amd.cache import PAGE_SIZE

    b = Bench(args.model, args.layers, args.context, not args.no_graphs)
    cfg, layers = b.cfg, b.layers
    prefill_s = b.prefill(args.prompt)
    head, mean_context = b.point(args.batch, args.steps, args.warmup, args.prompt, args.prompt_range,
                                 count_launches=not args.no_graphs)
    points = {}
    if not args.no_points:
        for n in (1, 64):                # the same number of steps as the headline run, each with its own roofline
            try:
                pt, _ = b.point(n, args.steps, args.warmup, args.prompt, args.prompt_range)
            except Exception as e:       # a point that fails is left out, the headline is not
                print(f"bench.py: batch {n} left out: {e}", file=sys.stderr)
                continue
            points[f"decode_b{n}"] = pt["tok_s"]
            points[f"decode_b{n}_ms"], points[f"decode_b{n}_gbs"], points[f"decode_b{n}_frac"] = pt["ms"], pt["gbs"], pt["frac"]
    b.close()

    # ---- the baseline's other two workloads, each model freed before the next
    if not args.no_points and not args.no_other_models and args.model == "8b" and args.layers is None:
        for key, which, kw in (
                ("qwen3_0_6b_b16", "0.6b", dict(batch=16, steps=256, warmup=8, prompt=1024, span=(16, 1024), context=2048,
                                                count_launches=True)),
                ("qwen3_32b_b1", "32b", dict(batch=1, steps=32, warmup=4, prompt=4096, span=None, context=8192))):
            other = None
            try:
                other = Bench(which, None, kw.pop("context"), not args.no_graphs)
                pt, _ = other.point(**kw)
                for name, v in pt.items():
                    points[key if name == "tok_s" else f"{key}_{name}"] = v
            except Exception as e:
                print(f"bench.py: {key} left out: {e}", file=sys.stderr)
            finally:
                if other is not None:
                    other.close()

    flops = prefill_flops(cfg, layers, args.prompt)
    out = {
        "metric": f"decode tok/s at batch {args.batch}, {b.name} bf16 (prefill {args.prompt} and batch 1/64 alongside)",
        "value": head["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": f"synthetic: random weights (seed {b.seed}), uniform random token ids",
        "config": {
            "model": b.name, "layers": layers, "layers_full": b.full_layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"], "rope_theta": cfg["rope_theta"],
            "rms_norm_eps": cfg["rms_norm_eps"], "tied": cfg["tie_word_embeddings"], "global_batch": args.batch, "seq_len": args.context,
            "prompt_len": "{}..{}".format(*args.prompt_range) if args.prompt_range else args.prompt,
            "mean_decode_context": round(mean_context, 1), "page_size": PAGE_SIZE, "launches_per_step": head.get("launches"),
            "parallelism": "single GPU",
        },
        "prefill": {"value": round(args.prompt / prefill_s, 1), "tokens": args.prompt, "ms": round(1e3 * prefill_s, 2),
                    "frac": round(flops / prefill_s / 1e12 / MFMA_PEAK_TFLOPS["bf16"], 4)},
        "roofline": {"bound": "hbm", "achieved": head["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac"]},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
