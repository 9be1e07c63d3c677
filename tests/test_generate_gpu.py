"""Generation through the Python entry point and the command line on the GPU, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from helpers import read_model_f64
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_greedy_with_margins(model_dir, prompts, steps, stop=()):
    cfg, w = read_model_f64(model_dir)
    out = []
    for p in prompts:
        toks, rows = P.greedy(cfg, w, p, steps, stop)
        margins = [float(np.sort(r)[-1] - np.sort(r)[-2]) for r in rows]
        out.append((toks, margins))
    return out


def assert_same_tokens(got, want, dtype_name, model_dir=None, prompts=None, stop=()):
    """Token for token; in bfloat16 a sequence may part from the plain one only at a place where the
    plain implementation's two best logits are closer than bfloat16 rounding of the logits.  With the model
    folder and the prompts at hand the tokens after such a place are not let go unchecked: the plain
    implementation is run again from the engine's own tokens up to there, and the engine's next tokens are
    held to that continuation in the same way."""
    for i, (g, (toks, margins)) in enumerate(zip(got, want)):
        base = 0                                  # tokens of g before this point were forced on the plain side
        while True:
            parted = None
            for j, (a, b) in enumerate(zip(g[base:], toks)):
                if a != b:
                    assert dtype_name == "bfloat16" and margins[j] < 0.08, \
                        f"request {i}, token {base + j}: {a} against {b} (margin {margins[j]:.3f}, {dtype_name})"
                    parted = base + j
                    break
            if parted is None:
                # one side may have ended on a stop token (which is not put out) where the other picked another
                # token: the same parting of ways, seen as a difference in length
                j = min(len(g) - base, len(toks))
                assert len(g) - base == len(toks) or (dtype_name == "bfloat16" and j < len(margins) and margins[j] < 0.08), \
                    f"request {i}: {len(g)} tokens against {base + len(toks)}"
                break
            if model_dir is None or parted + 1 >= len(g):
                break
            # go on from the engine's own choice: the plain implementation continues prompt + g[:parted + 1]
            cfg, w = read_model_f64(model_dir)
            left = len(g) - (parted + 1)          # the plain side's first token is g's token parted + 1
            toks, rows = P.greedy(cfg, w, list(prompts[i]) + list(g[:parted + 1]), left, stop)
            margins = [float(np.sort(r)[-1] - np.sort(r)[-2]) for r in rows]
            base = parted + 1


def prompts_for(cfg, lengths, seed):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for n in lengths]


@pytest.mark.parametrize("use_graphs", [False, True])
@pytest.mark.parametrize("name, lengths, steps, dtype_name", [
    ("A", [5, 11, 1, 17], 8, "float32"), ("A", [5, 11, 1, 17], 8, "bfloat16"),
    ("B", [33, 2, 40], 16, "float32"), ("B", [33, 2, 40], 16, "bfloat16"),
    ("D", [70, 2, 40], 16, "bfloat16"),
])
def test_greedy_generation_through_the_entry_point(model_dirs, name, lengths, steps, dtype_name, use_graphs):
    from rust_inference_amd import Model
    cfg, _ = read_model_f64(model_dirs[name])
    prompts = prompts_for(cfg, lengths, 3)
    model = Model.load(model_dirs[name], dtype=dtype_name, max_batch=4, max_seq_len=96, use_graphs=use_graphs, graph_after=0)
    res = model.generate(prompts, max_new_tokens=steps)
    assert_same_tokens(res.tokens, plain_greedy_with_margins(model_dirs[name], prompts, steps), dtype_name,
                       model_dirs[name], prompts)
    assert res.finish_reasons == ["length"] * len(prompts)
    assert res.stats.prompt_tokens == sum(lengths) and res.stats.decode_tokens == len(prompts) * (steps - 1)
    model.cache.check_consistent()
    assert model.cache.slots.free_count == 4


def test_batch_invariant_generation_gives_a_request_the_same_tokens_in_any_batch(model_dirs):
    """``batch_invariant=True``: sampled tokens (temperature, so that a last bit of a logit can show) of each
    request alone, in a batch of all and in batches of four and three are the same, with graphs and without."""
    from rust_inference_amd import Model, SamplingParams
    cfg, _ = read_model_f64(model_dirs["D"])
    prompts = prompts_for(cfg, [70, 2, 40, 1, 33, 17, 64], 5)
    # (sequence i of a call draws from the generator seeded seed + i)
    sampling = [SamplingParams(temperature=1.5, top_k=0, top_p=1.0, seed=100)] * len(prompts)
    outs = {}
    for graphs in (False, True):
        model = Model.load(model_dirs["D"], dtype="bfloat16", batch_invariant=True, max_batch=7, max_seq_len=128,
                           use_graphs=graphs, graph_after=0)
        outs[graphs, "together"] = model.generate(prompts, max_new_tokens=24, sampling=sampling).tokens
        outs[graphs, "in fours"] = model.generate(prompts, max_new_tokens=24, sampling=sampling, max_batch=4).tokens
        outs[graphs, "alone"] = [model.generate([p], max_new_tokens=24, temperature=1.5, seed=100 + i).tokens[0]
                                 for i, p in enumerate(prompts)]
    first = outs[False, "alone"]
    assert len({tuple(t) for t in first}) > 1
    for key, tokens in outs.items():
        assert tokens == first, f"{key}: a request's tokens depend on its batch"


@pytest.mark.parametrize("requests", [20, 40])
def test_batches_of_tens_of_sequences(model_dirs, requests):
    """Twenty and forty sequences a batch (the decode steps of 17 to 32 rows and of 33 to 64 take other kernels
    than the smaller ones), some stopping early so that the batch shrinks through those sizes: graphs and
    eager steps both give the plain implementation's tokens."""
    from rust_inference_amd import Model
    cfg, _ = read_model_f64(model_dirs["D"])
    rng = np.random.default_rng(requests)
    lengths = [int(n) for n in rng.integers(1, 50, size=requests)]
    prompts = prompts_for(cfg, lengths, 13)
    stop = [int(t) for t in rng.integers(0, cfg["vocab_size"], 12)]             # a few sequences end on them
    outs = []
    for graphs in (False, True):
        model = Model.load(model_dirs["D"], dtype="bfloat16", max_batch=requests, max_seq_len=96, use_graphs=graphs, graph_after=0)
        res = model.generate(prompts, max_new_tokens=12, stop_token_ids=stop)
        model.cache.check_consistent()
        assert model.cache.slots.free_count == requests
        outs.append(res)
    # (The loop over graphs runs one step ahead of the ids it has read, so a sequence that stops is carried one
    # step further than in the other loop: a step of 17 rows here is one of 16 there, on another kernel, and in
    # bfloat16 two logits closer than its rounding may then change places.  Both are held to the plain
    # implementation, which lets a sequence part from it at such a place only.)
    want = plain_greedy_with_margins(model_dirs["D"], prompts, 12, stop)
    for res in outs:
        assert "stop" in res.finish_reasons
        assert_same_tokens(res.tokens, want, "bfloat16", model_dirs["D"], prompts, stop)


def test_stop_tokens_and_batches_one_after_another(model_dirs):
    """Five requests on two slots: three batches, slots used again; a stop token ends sequences early."""
    from rust_inference_amd import Model
    cfg, _ = read_model_f64(model_dirs["A"])
    prompts = prompts_for(cfg, [4, 9, 2, 7, 12], 4)
    free = plain_greedy_with_margins(model_dirs["A"], prompts, 10)
    stop = [free[1][0][3], free[3][0][0]]                       # ends request 1 after 3 tokens, request 3 at once
    want = plain_greedy_with_margins(model_dirs["A"], prompts, 10, stop)
    model = Model.load(model_dirs["A"], dtype="float32", max_batch=2, max_seq_len=64)
    res = model.generate(prompts, max_new_tokens=10, stop_token_ids=stop)
    assert_same_tokens(res.tokens, want, "float32")
    assert res.stats.batches == 3 and res.finish_reasons[3] == "stop" and res.tokens[3] == []
    assert all(s not in toks for toks in res.tokens for s in stop)


# (the third case grows past 1,024 tokens while it decodes: the graphs are sized for a bound on the length,
# and the batch moves on to the next one)
@pytest.mark.parametrize("name, lengths, room", [("B", [33, 2, 40], 96), ("D", [270, 2, 40], 320),
                                                 ("D", [1015, 2, 40], 1100)])
def test_graph_and_eager_decoding_give_the_same_logits(model_dirs, name, lengths, room):
    import torch
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.parts import load_model
    model = load_model(model_dirs[name], torch.bfloat16)
    cfg, _ = read_model_f64(model_dirs[name])
    prompts = prompts_for(cfg, lengths, 5)
    outs = []
    for graphs in (False, True):
        eng = Engine(model, model.new_cache(max_tokens=3 * room, num_slots=3, max_seq_len=room), use_graphs=graphs)
        slots = [eng.cache.acquire() for _ in prompts]
        eng.step([StepEntry(s, p, "last") for s, p in zip(slots, prompts)])
        rows = []
        for step in range(20):
            live = slots if step < 12 else slots[:2]            # a sequence leaves: another batch size, another graph
            rows.append(eng.step([StepEntry(s, [(7 * step + s) % 300], "last") for s in live]).clone())
        outs.append(rows)
    for a, b in zip(*outs):
        assert torch.equal(a, b), "a captured step must compute what the launched one computes"


def test_an_engine_keeps_a_bounded_number_of_graphs(model_dirs):
    """With room for one graph, steps that alternate between two batch sizes drop and capture a graph every
    time; the logits stay those of the launched steps, and the engine never holds more than it may."""
    import torch
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.parts import load_model
    model = load_model(model_dirs["B"], torch.bfloat16)
    cfg, _ = read_model_f64(model_dirs["B"])
    prompts = prompts_for(cfg, [33, 2, 40], 5)
    outs = []
    for graphs in (False, True):
        eng = Engine(model, model.new_cache(max_tokens=3 * 96, num_slots=3, max_seq_len=96), use_graphs=graphs)
        eng.max_graphs = 1
        slots = [eng.cache.acquire() for _ in prompts]
        eng.step([StepEntry(s, p, "last") for s, p in zip(slots, prompts)])
        rows = []
        for step in range(8):
            live = slots if step % 2 == 0 else slots[:2]
            rows.append(eng.step([StepEntry(s, [(5 * step + s) % 300], "last") for s in live]).clone())
            assert len(eng._graphs) <= 1
        outs.append(rows)
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_a_graph_is_captured_after_a_batch_size_has_been_used_a_few_times(model_dirs):
    """``capture_after=3``: three steps of a batch size run with host launches, the fourth captures its graph; a size
    that is used twice never gets one.  The logits are those of an engine that captures at once, bit for bit."""
    import torch
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.parts import load_model
    model = load_model(model_dirs["B"], torch.float32)
    cfg, _ = read_model_f64(model_dirs["B"])
    prompts = prompts_for(cfg, [33, 2, 40], 5)
    outs = []
    for after in (0, 3):
        eng = Engine(model, model.new_cache(max_tokens=3 * 96, num_slots=3, max_seq_len=96), use_graphs=True,
                     capture_after=after)
        slots = [eng.cache.acquire() for _ in prompts]
        eng.step([StepEntry(s, p, "last") for s, p in zip(slots, prompts)])
        rows = []
        for step in range(8):
            live = slots if step < 6 else slots[:2]              # six steps of three sequences, two of two
            rows.append(eng.step([StepEntry(s, [(5 * step + s) % 300], "last") for s in live]).clone())
            if after:
                assert sorted(b for b, _ in eng._graphs) == ([3] if step >= 3 else [])
        outs.append(rows)
    for a, b in zip(*outs):
        assert torch.equal(a, b)


def test_temperature_sampling_is_seeded(model_dirs):
    from rust_inference_amd import Model
    cfg, _ = read_model_f64(model_dirs["A"])
    prompts = prompts_for(cfg, [6, 3], 6)
    model = Model.load(model_dirs["A"], dtype="float32", max_batch=2, max_seq_len=64)
    a = model.generate(prompts, max_new_tokens=12, temperature=0.8, seed=1).tokens
    b = model.generate(prompts, max_new_tokens=12, temperature=0.8, seed=1).tokens
    c = model.generate(prompts, max_new_tokens=12, temperature=0.8, seed=2).tokens
    alone = model.generate(prompts[:1], max_new_tokens=12, temperature=0.8, seed=1).tokens
    assert a == b and a != c and alone[0] == a[0]


def test_the_command_line_generates_what_the_plain_implementation_does(model_dirs):
    """bin/runner with prompts as token ids (the folder has no tokenizer.json): greedy, float32; one prompt
    is streamed to standard output, two are printed a line each; a stop token from the command line."""
    cfg, _ = read_model_f64(model_dirs["A"])
    prompts = prompts_for(cfg, [7, 12], 9)
    want = plain_greedy_with_margins(model_dirs["A"], prompts, 6)
    base = [sys.executable, os.path.join(ROOT, "bin", "runner"), model_dirs["A"], "--dtype", "float32", "-n", "6"]
    one = subprocess.run(base + ["-p", " ".join(map(str, prompts[0]))], capture_output=True, text=True, timeout=120)
    assert one.returncode == 0, one.stderr
    assert [int(t) for t in one.stdout.split()] == want[0][0]
    assert "prefill: 7 tokens" in one.stderr and "decode: 5 tokens" in one.stderr      # src/bin/runner.rs:243-251
    two = subprocess.run(base + ["--prompt-ids", ",".join(map(str, prompts[0])), "--prompt-ids",
                                 ",".join(map(str, prompts[1])), "--profile"], capture_output=True, text=True, timeout=120)
    assert two.returncode == 0, two.stderr
    assert [[int(t) for t in ln.split()] for ln in two.stdout.strip().splitlines()] == [w[0] for w in want]
    assert "profile: 1 batches, 5 decode steps" in two.stderr
    # the section table of src/profiler.rs:113-123 (src/bin/runner.rs:252-254): device time per kind of work
    table = two.stderr[two.stderr.index("section "):].splitlines()
    assert table[0].split() == ["section", "total(s)", "share", "calls"]
    rows = {ln[:30].strip(): ln[30:].split() for ln in table[1:] if ln.strip()}
    assert {"embedding", "attn q/k/v proj", "attention", "attn o proj", "rmsnorm", "dense mlp", "lm head",
            "sampling"} <= set(rows)
    assert rows["attention"][2] == "12" and rows["sampling"][2] == "6" and rows["lm head"][2] == "6"   # 2 layers x 6 steps
    assert abs(sum(float(r[1].rstrip("%")) for r in rows.values()) - 100.0) < 1.0
    assert "section " not in one.stderr                        # off unless asked for
    stop = want[1][0][2]
    cut = subprocess.run(base + ["-p", " ".join(map(str, prompts[1])), "--stop-token-ids", str(stop)],
                         capture_output=True, text=True, timeout=120)
    assert cut.returncode == 0 and [int(t) for t in cut.stdout.split()] == want[1][0][:want[1][0].index(stop)]


def test_the_command_line_with_random_weights(tmp_path):
    """--random: a config.json is enough; the same seed gives the same tokens, another seed others."""
    from conftest import TINY_C
    with open(tmp_path / "config.json", "w") as f:
        json.dump(TINY_C, f)
    base = [sys.executable, os.path.join(ROOT, "bin", "runner"), "-p", "5 17 3 250", "-n", "12", "--random"]
    runs = [subprocess.run(base + [where, "--random-seed", seed], capture_output=True, text=True, timeout=120)
            for where, seed in ((str(tmp_path), "4"), (str(tmp_path / "config.json"), "4"), (str(tmp_path), "5"))]
    assert all(r.returncode == 0 for r in runs), [r.stderr for r in runs]
    outs = [[int(t) for t in r.stdout.split()] for r in runs]
    assert len(outs[0]) == 12 and outs[0] == outs[1] and outs[0] != outs[2]
    missing = subprocess.run(base + [str(tmp_path / "nowhere")], capture_output=True, text=True, timeout=120)
    assert missing.returncode == 1 and "error:" in missing.stderr
