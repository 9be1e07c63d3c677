#!/usr/bin/env python3
"""Decode and prefill throughput of the Qwen3-8B-shaped model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C] [--model 8b|0.6b|32b]

The default run has the layer sizes of Qwen3-8B with random weights
(N(0, 0.02), norm gains 1 + N(0, 0.1), seed 2), a batch of 8 and prompts of 2,048 tokens in a
context of 4,096.  A step is one decode step: every live sequence gets one more token, chosen
greedily on the device.  Prints one JSON line: decoded tokens a second at batch 8 (`value`), the
2,048-token prefill, the decode step's share of the HBM roofline, and decoding at batch 1 and 64
(`points`: tokens a second, and beside each its milliseconds a step, the GB/s of the bytes the step has
to read and their share of the HBM peak).
"""
import argparse
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


# The other two shapes that the baseline names, for `--model`: the small model whose decode step is bound
# by launches and latencies, and the large one (64 GB of weights).
QWEN3_0_6B = dict(QWEN3_8B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                  num_key_value_heads=8, tie_word_embeddings=True)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64,
                 num_key_value_heads=8)
MODELS = {"8b": ("Qwen3-8B shapes", QWEN3_8B), "0.6b": ("Qwen3-0.6B shapes", QWEN3_0_6B),
          "32b": ("Qwen3-32B shapes", QWEN3_32B)}


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
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--no-graphs", action="store_true", help="launch every kernel of a decode step from the host")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this library is single-GPU, --gpus {args.gpus} is not run")
        return 2

    import torch
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.parts import random_model

    model_name, shapes = MODELS[args.model]
    cfg = dict(shapes)
    full_layers = cfg["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg["num_hidden_layers"] = layers
    cfg["max_position_embeddings"] = args.context
    torch.manual_seed(2)
    model = random_model(cfg, seed=2, dtype=torch.bfloat16)
    vocab = cfg["vocab_size"]
    gen = torch.Generator().manual_seed(2)

    def prompts(batch, n):
        if args.prompt_range and batch > 1:                       # unequal lengths, prefilled together
            low, high = args.prompt_range
            lens = torch.randint(low, high + 1, (batch,), generator=gen).tolist()
            return [torch.randint(0, vocab, (m,), generator=gen).tolist() for m in lens]
        return torch.randint(0, vocab, (batch, n), generator=gen).tolist()

    def fresh_engine(batch):
        per_seq = -(-args.context // 32) * 32
        return Engine(model, model.new_cache(max_tokens=per_seq * batch, num_slots=batch, max_seq_len=args.context),
                      use_graphs=not args.no_graphs)

    def sync():
        torch.cuda.synchronize()

    # ---- prefill of 2,048 tokens (one prompt, logits at its last place)
    engine = fresh_engine(1)
    p = prompts(1, args.prompt)[0]
    times = []
    for _ in range(3):
        slot = engine.cache.acquire()
        sync()
        t0 = time.perf_counter()
        engine.step([StepEntry(slot, p, "last")])
        sync()
        times.append(time.perf_counter() - t0)
        engine.cache.release(slot)
    prefill_s = min(times[1:])
    del engine

    # ---- decoding: the generation loop's steady state (engine/generate.py).  A step is launched with the ids
    # the step before picked, still on the device, and the host reads every step's ids while the next step runs;
    # where there is no captured graph for the step yet (or --no-graphs) the host reads them first.
    def decode_run(batch, steps, warmup):
        engine = fresh_engine(batch)
        slots = [engine.cache.acquire() for _ in range(batch)]
        logits = engine.step([StepEntry(s, q, "last") for s, q in zip(slots, prompts(batch, args.prompt))])
        ids = ops.argmax(logits)
        pinned = [torch.empty(batch, dtype=torch.int32, pin_memory=True) for _ in range(2)]

        def one_step(ids):
            out = engine.decode_on_device(slots, ids)
            if out is None:
                out = engine.step([StepEntry(s, [t], "last") for s, t in zip(slots, ids.tolist())])
            return ops.argmax(out)

        def run(n):
            nonlocal ids
            unread, read = None, 0
            for i in range(n):
                ids = one_step(ids)
                if unread is not None:
                    unread[0].synchronize()
                    read += len(unread[1].tolist())
                pinned[i & 1].copy_(ids, non_blocking=True)
                ev = torch.cuda.Event()
                ev.record()
                unread = (ev, pinned[i & 1])
            if unread is not None:
                unread[0].synchronize()
                read += len(unread[1].tolist())
            return read

        run(warmup)
        sync()
        first_context = sum(engine.cache.length(s) for s in slots) / batch + 1
        t0 = time.perf_counter()
        read = run(steps)
        sync()
        dt = time.perf_counter() - t0
        assert read == batch * steps
        mean_context = first_context + (steps - 1) / 2.0
        for s in slots:
            engine.cache.release(s)
        return dt, mean_context

    dt, mean_context = decode_run(args.batch, args.steps, args.warmup)
    value = args.batch * args.steps / dt
    step_bytes = decode_bytes(cfg, layers, args.batch, mean_context)
    achieved = step_bytes / (dt / args.steps) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):                # the same number of steps as the headline run, each with its own roofline
            pdt, pctx = decode_run(b, args.steps, args.warmup)
            points[f"decode_b{b}"] = round(b * args.steps / pdt, 1)
            points[f"decode_b{b}_ms"] = round(1e3 * pdt / args.steps, 3)
            points[f"decode_b{b}_gbs"] = round(decode_bytes(cfg, layers, b, pctx) / (pdt / args.steps) / 1e9, 1)
            points[f"decode_b{b}_frac"] = round(points[f"decode_b{b}_gbs"] / HBM_PEAK_GBS, 4)

    flops = prefill_flops(cfg, layers, args.prompt)
    out = {
        "metric": f"decode tok/s at batch {args.batch}, {model_name} bf16 (prefill {args.prompt} and batch 1/64 alongside)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(1e3 * dt / args.steps, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic: random weights (seed 2), uniform random token ids",
        "config": {
            "model": model_name, "layers": layers, "layers_full": full_layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": vocab, "rope_theta": cfg["rope_theta"],
            "rms_norm_eps": cfg["rms_norm_eps"], "tied": cfg["tie_word_embeddings"], "global_batch": args.batch, "seq_len": args.context,
            "prompt_len": "{}..{}".format(*args.prompt_range) if args.prompt_range else args.prompt, "mean_decode_context": round(mean_context, 1), "page_size": 32,
            "parallelism": "single GPU",
        },
        "prefill": {"value": round(args.prompt / prefill_s, 1), "tokens": args.prompt, "ms": round(1e3 * prefill_s, 2),
                    "frac": round(flops / prefill_s / 1e12 / MFMA_PEAK_TFLOPS["bf16"], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
