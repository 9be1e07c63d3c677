"""The engine against the plain implementation on the GPU, in float32 and in bfloat16: each request
alone and whole; with its last 32 tokens one by one; in batches of unequal lengths whose shorter
requests end earlier, one batch after another so that slots and pages are used again; long decoding;
the first tokens of a sequence; and the same through bin/trace_run."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import trace_plans as plans
from helpers import assert_logits_close, read_model_f64, rel_to_max
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
_plain_cache = {}
_last_read = {}


def plain_logits(model_dir, tokens):
    key = (model_dir, tuple(tokens))
    if key not in _plain_cache:
        if _last_read.get("dir") != model_dir:               # one folder's float64 weights are kept at a time
            _last_read.clear()
            _last_read.update(dir=model_dir, model=read_model_f64(model_dir))
        cfg, w = _last_read["model"]
        _plain_cache[key] = P.forward(cfg, w, list(tokens))
    return _plain_cache[key]


def requests_for(name, cfg, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"{name}{i}": [int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for i, n in enumerate(lengths)}


@pytest.fixture(scope="module")
def loaded(model_dirs):
    from rust_inference_amd.parts import load_model
    cache = {}

    def get(name, dtype_name):
        if (name, dtype_name) not in cache:
            cache[(name, dtype_name)] = load_model(model_dirs[name], DTYPES[dtype_name])
        return cache[(name, dtype_name)]
    return get


def replay_in_process(model, steps):
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    engine = engine_for_trace(model, plans.max_live_tokens(steps))
    player = Replayer(engine)
    outs = {}
    for s in steps:
        logits = player.feed(s)
        if logits is not None:
            outs[s["step"]] = logits.cpu().numpy()
    engine.cache.check_consistent()
    assert engine.cache.slots.free_count == engine.cache.num_slots, "a request's slot was not given back"
    assert all(f == g.pool.num_pages for f, g in zip(engine.cache.free_pages(), engine.cache.groups))
    return plans.collect(steps, lambda i: outs[i], model.spec.vocab_size)


def check_against_plain(model_dir, got, requests, dtype_name, what):
    for rid, toks in requests.items():
        assert_logits_close(got[rid], plain_logits(model_dir, toks), dtype_name, f"{what}, request {rid}")


CASES = [("A", [5, 11, 1, 17], 0), ("B", [33, 2, 40], 1), ("C", [70, 45, 3], 2), ("D", [300, 37, 130], 3)]


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, lengths, seed", CASES)
def test_each_request_alone_and_whole(model_dirs, loaded, name, lengths, seed, dtype_name):
    cfg, _ = read_model_f64(model_dirs[name])
    reqs = requests_for(name, cfg, [n + 20 for n in lengths], seed)
    got = replay_in_process(loaded(name, dtype_name), plans.whole(reqs))
    check_against_plain(model_dirs[name], got, reqs, dtype_name, "whole")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, lengths, seed", CASES)
def test_last_32_tokens_one_by_one(model_dirs, loaded, name, lengths, seed, dtype_name):
    cfg, _ = read_model_f64(model_dirs[name])
    reqs = requests_for(name, cfg, [n + 40 for n in lengths], seed + 10)      # prefixes 13.., crossing pages
    model = loaded(name, dtype_name)
    got = replay_in_process(model, plans.tail_one_by_one(reqs, 32))
    check_against_plain(model_dirs[name], got, reqs, dtype_name, "last 32 one by one")
    # decoding against whole prompts, engine against engine: a tighter bound than against the plain one
    whole = replay_in_process(model, plans.whole(reqs))
    bound = 2e-5 if dtype_name == "float32" else 2e-2
    for rid in reqs:
        err = rel_to_max(got[rid], whole[rid])
        assert err <= bound, f"{rid}: one by one differs from whole by {err:.2e} of the largest logit"


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name, lengths, seed", CASES)
def test_unequal_batches_one_after_another(model_dirs, loaded, name, lengths, seed, dtype_name):
    cfg, _ = read_model_f64(model_dirs[name])
    rng = np.random.default_rng(seed + 20)
    batches, reqs = [], {}
    for b in range(3):                                       # three batches on one cache: slots come back
        batch = {}
        order = list(rng.permutation(len(lengths)))
        for i in order:
            p = lengths[i]
            total = p + int(rng.integers(0, 14))             # unequal ends: some end at once, some late
            rid = f"{name}{b}_{i}"
            toks = [int(t) for t in rng.integers(0, cfg["vocab_size"], total)]
            batch[rid] = (toks, p)
            reqs[rid] = toks
        batches.append(batch)
    got = replay_in_process(loaded(name, dtype_name), plans.unequal_batches(batches))
    check_against_plain(model_dirs[name], got, reqs, dtype_name, "unequal batches")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_batch_composition_and_padding_change_nothing(model_dirs, loaded, dtype_name):
    """The same request alone, and as one of a batch of unequal others: equal beyond rounding."""
    cfg, _ = read_model_f64(model_dirs["B"])
    reqs = requests_for("B", cfg, [37, 5, 64, 1], 33)
    model = loaded("B", dtype_name)
    alone = replay_in_process(model, plans.whole(reqs))
    together = replay_in_process(model, plans.unequal_batches([{rid: (t, len(t)) for rid, t in reqs.items()}]))
    bound = 2e-5 if dtype_name == "float32" else 2e-2
    for rid in reqs:
        assert rel_to_max(together[rid], alone[rid]) <= bound


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_decoding(model_dirs, loaded, dtype_name):
    """A short prompt and 300 tokens one by one: ten pages, three tiles of keys."""
    cfg, _ = read_model_f64(model_dirs["C"])
    reqs = requests_for("C", cfg, [310], 44)
    got = replay_in_process(loaded("C", dtype_name), plans.tail_one_by_one(reqs, 300))
    check_against_plain(model_dirs["C"], got, reqs, dtype_name, "long decoding")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_decoding_over_thousands_of_keys(model_dirs, loaded, dtype_name):
    """4,200 tokens, the last 8 one by one, beside a request of 300: past 4,096 keys the decode attention
    joins its chunks in runs, and one batch holds a sequence on either side of that."""
    cfg, _ = read_model_f64(model_dirs["D"])
    reqs = requests_for("D", cfg, [4200, 300], 66)
    got = replay_in_process(loaded("D", dtype_name), plans.tail_one_by_one(reqs, 8))
    check_against_plain(model_dirs["D"], got, reqs, dtype_name, "thousands of keys")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(model_dirs, loaded, dtype_name):
    """Every token from the first one on its own step: position 0 sees one key only."""
    cfg, _ = read_model_f64(model_dirs["A"])
    reqs = requests_for("A", cfg, [6, 3], 55)
    got = replay_in_process(loaded("A", dtype_name), plans.tail_one_by_one(reqs, 32))
    check_against_plain(model_dirs["A"], got, reqs, dtype_name, "first tokens")


def test_a_prompt_in_pieces(model_dirs, loaded):
    """Several tokens in a later step (a prompt cut in three): the same code as any other cut."""
    cfg, _ = read_model_f64(model_dirs["B"])
    toks = requests_for("B", cfg, [75], 66)["B0"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:30], "want": list(range(30))}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[30:34], "want": [0, 1, 2, 3]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[34:], "want": list(range(41))}], "end": ["x"]}]
    got = replay_in_process(loaded("B", "float32"), steps)
    assert_logits_close(got["x"], plain_logits(model_dirs["B"], toks), "float32", "prompt in pieces")


def test_steps_that_want_nothing_still_fill_the_cache(model_dirs, loaded):
    cfg, _ = read_model_f64(model_dirs["A"])
    toks = requests_for("A", cfg, [20], 77)["A0"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:19], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[19:], "want": [0]}], "end": ["x"]}]
    got = replay_in_process(loaded("A", "float32"), steps)
    assert_logits_close(got["x"], plain_logits(model_dirs["A"], toks)[19:], "float32", "empty want")


def test_errors_leave_the_cache_whole(model_dirs, loaded):
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.errors import CacheError, ShapeError
    model = loaded("A", "float32")
    engine = Engine(model, model.new_cache(max_tokens=64, num_slots=2, max_seq_len=64))
    s = engine.cache.acquire()
    with pytest.raises(ShapeError, match="outside the vocabulary"):
        engine.step([StepEntry(s, [5, 256])])
    with pytest.raises(CacheError, match="per sequence"):
        engine.step([StepEntry(s, [1] * 65)])
    with pytest.raises(CacheError, match="not held"):
        engine.step([StepEntry(1, [1])])
    assert engine.cache.length(s) == 0
    assert engine.step([StepEntry(s, [1, 2, 3], "all")]).shape == (3, 256)


# ---------------------------------------------------------------- through the program
def run_trace_program(model_dir, dtype_name, steps, out_dir):
    """Drives bin/trace_run as a user would: one line in, wait for `done <step>`, next line."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype_name,
           "--out", out_dir, "--max-tokens", str(plans.max_live_tokens(steps))]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", f"after step {s['step']} the program said {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, tmp_path, dtype_name):
    cfg, _ = read_model_f64(model_dirs["B"])
    rng = np.random.default_rng(88)
    reqs = requests_for("B", cfg, [33, 2, 40, 70], 88)
    batches = [{rid: (t, max(1, len(t) - int(rng.integers(0, 9)))) for rid, t in list(reqs.items())[:3]},
               {rid: (t, len(t) - 32) for rid, t in list(reqs.items())[3:]}]
    steps = plans.unequal_batches(batches)
    out_dir = str(tmp_path / "out")
    run_trace_program(model_dirs["B"], dtype_name, steps, out_dir)
    vocab = cfg["vocab_size"]
    got = plans.collect(steps, lambda i: np.fromfile(os.path.join(out_dir, f"{i}.f32"), dtype="<f4"), vocab)
    check_against_plain(model_dirs["B"], got, reqs, dtype_name, "bin/trace_run")
    assert not os.path.exists(os.path.join(out_dir, f"{len(steps)}.f32"))


# ---------------------------------------------------------------- sizes drawn at random
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Every size a configuration may have, drawn from lists that mix what the fast kernels take (head
    sizes 32, 64, 128, widths that are multiples of 8) with what only the general ones do (head sizes 8, 24,
    40, 48, 72, 80, 160, 256, 320, odd widths, seven query heads a group): whole, last 32 one by one and an unequal
    batch, in both dtypes, against the plain implementation."""
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    rng = np.random.default_rng(1000 + seed)
    kv, group = int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 2, 3, 4, 7, 8, 16]))
    cfg = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": int(rng.integers(50, 700)),
           "hidden_size": int(rng.choice([33, 50, 72, 75, 104, 129, 136, 264])),
           "intermediate_size": int(rng.choice([9, 37, 88, 101, 232, 250])),
           "num_hidden_layers": int(rng.integers(1, 4)), "num_attention_heads": kv * group, "num_key_value_heads": kv,
           "head_dim": int(rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 80, 128, 160, 256, 320])),
           "rope_theta": float(rng.choice([1e4, 5e4, 1e6])), "rms_norm_eps": float(rng.choice([1e-6, 1e-5, 3e-6])),
           "tie_word_embeddings": bool(rng.integers(0, 2)), "max_position_embeddings": 512}
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=seed, dtype=torch.bfloat16, matrix_std=0.12, gain_std=0.1)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for i, n in enumerate(rng.integers(1, 200, 3))}
    for dtype_name in ("float32", "bfloat16"):
        model = load_model(folder, DTYPES[dtype_name])
        for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 32)),
                            ("batch", plans.unequal_batches([{k: (v, max(1, len(v) - 7)) for k, v in reqs.items()}]))):
            got = replay_in_process(model, steps)
            check_against_plain(folder, got, reqs, dtype_name, f"{cfg}, {what}")


@pytest.mark.parametrize("graphs", [False, True])
def test_a_batch_of_seventy_sequences_with_eight_kv_heads(tmp_path, graphs):
    """512 (sequence, kv head) pairs and more: the decode attention walks each sequence's pages in one run
    per workgroup, and the step's products go to the vendor library.  Seventy requests of unequal lengths
    start together and decode their last tokens one by one; the shorter ones end earlier, so the batch
    shrinks through the sizes at which the kernels change."""
    from rust_inference_amd.engine import Engine
    from rust_inference_amd.engine.replay import Replayer
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    cfg = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 300, "hidden_size": 72,
           "intermediate_size": 88, "num_hidden_layers": 2, "num_attention_heads": 16, "num_key_value_heads": 8,
           "head_dim": 32, "rope_theta": 1e4, "rms_norm_eps": 1e-6, "tie_word_embeddings": True}
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=11, dtype=torch.bfloat16, matrix_std=0.12, gain_std=0.1)
    rng = np.random.default_rng(70)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, 300, n)] for i, n in enumerate(rng.integers(4, 90, 70))}
    assert ops.decode_attention_streams(70, 8, 128)
    steps = plans.unequal_batches([{k: (v, max(1, len(v) - int(rng.integers(1, 9)))) for k, v in reqs.items()}])
    model = load_model(folder, torch.bfloat16)
    cache = model.new_cache(max_tokens=plans.max_live_tokens(steps), num_slots=70, max_seq_len=128)
    player, outs = Replayer(Engine(model, cache, use_graphs=graphs)), {}
    for s in steps:
        logits = player.feed(s)
        if logits is not None:
            outs[s["step"]] = logits.cpu().numpy().copy()
    got = plans.collect(steps, lambda i: outs[i], 300)
    check_against_plain(folder, got, reqs, "bfloat16", f"seventy sequences, graphs {graphs}")


def test_graphs_and_host_launches_choose_the_same_kernels(tmp_path):
    """Eight sequences of 8,200 to 8,300 tokens with eight kv heads: a graph of the decode step is sized for
    16,384 tokens, where the attention walks runs of pages, while the lengths themselves would still get a
    workgroup per chunk of 256 keys.  A step launched from the host takes the graph's bound, so both give the
    same logits bit for bit, and the logits of the plain implementation within rounding."""
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    cfg = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 300, "hidden_size": 72,
           "intermediate_size": 88, "num_hidden_layers": 1, "num_attention_heads": 8, "num_key_value_heads": 8,
           "head_dim": 32, "rope_theta": 1e4, "rms_norm_eps": 1e-6, "tie_word_embeddings": True}
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=12, dtype=torch.bfloat16, matrix_std=0.12, gain_std=0.1)
    assert ops.decode_attention_streams(8, 8, 16384) and not ops.decode_attention_streams(8, 8, 8310)
    rng = np.random.default_rng(8)
    prompts = [[int(t) for t in rng.integers(0, 300, n)] for n in rng.integers(8200, 8300, 8)]
    nxt = [[int(t) for t in rng.integers(0, 300, 3)] for _ in prompts]
    model = load_model(folder, torch.bfloat16)
    outs = []
    for graphs in (False, True):
        cache = model.new_cache(max_tokens=8 * 8320, num_slots=8, max_seq_len=20000)
        engine = Engine(model, cache, use_graphs=graphs)
        slots = [cache.acquire() for _ in prompts]
        engine.step([StepEntry(s, p, []) for s, p in zip(slots, prompts)])
        outs.append([engine.step([StepEntry(s, [t[i]], "last") for s, t in zip(slots, nxt)]).clone() for i in range(3)])
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # the last step against the plain implementation, for the longest request
    i = int(np.argmax([len(p) for p in prompts]))
    want = plain_logits(folder, prompts[i] + nxt[i])[-1:]
    assert_logits_close(outs[1][2][i:i + 1].cpu().numpy(), want, "bfloat16", f"request {i} of {len(prompts[i]) + 3} tokens")


def test_a_sequence_may_pass_max_position_embeddings(model_dirs, loaded):
    """The key is read and, as in the reference, bounds nothing (src/models/config.rs:30): configuration A
    says 128 positions, the request has 150 tokens, the last 20 decoded one by one."""
    cfg, _ = read_model_f64(model_dirs["A"])
    assert cfg["max_position_embeddings"] == 128
    reqs = requests_for("A", cfg, [150], 99)
    got = replay_in_process(loaded("A", "float32"), plans.tail_one_by_one(reqs, 20))
    check_against_plain(model_dirs["A"], got, reqs, "float32", "past max_position_embeddings")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_any_cut_of_the_work_gives_the_same_logits(model_dirs, loaded, name, dtype_name):
    """Steps of any shape: requests join at different times, and a step gives each live request between one
    token and a few dozen, some of them one token (a decode step for them) beside others' long pieces; a
    request that is finished leaves, and its slot serves the next one.  Every position's logits against the
    plain implementation."""
    from rust_inference_amd.engine import Engine, StepEntry
    cfg, _ = read_model_f64(model_dirs[name])
    rng = np.random.default_rng(7)
    reqs = requests_for(name, cfg, [int(n) for n in rng.integers(1, 160, 9)], 123)
    model = loaded(name, dtype_name)
    engine = Engine(model, model.new_cache(max_tokens=4 * 192, num_slots=4, max_seq_len=192))
    waiting, live, fed, got = list(reqs), {}, {}, {rid: [] for rid in reqs}
    while waiting or live:
        while waiting and len(live) < 4 and (not live or rng.random() < 0.5):
            rid = waiting.pop(0)
            live[rid], fed[rid] = engine.cache.acquire(), 0
        entries, order = [], []
        for rid, slot in live.items():
            left = len(reqs[rid]) - fed[rid]
            n = min(left, int(rng.choice([1, 1, 2, 7, 33, 64])))
            entries.append(StepEntry(slot, reqs[rid][fed[rid]:fed[rid] + n], "all"))
            order.append((rid, n))
        logits = engine.step(entries).cpu().numpy()
        at = 0
        for rid, n in order:
            got[rid].append(logits[at:at + n])
            at += n
            fed[rid] += n
            if fed[rid] == len(reqs[rid]):
                engine.cache.release(live.pop(rid))
    engine.cache.check_consistent()
    assert engine.cache.slots.free_count == 4
    check_against_plain(model_dirs[name], {rid: np.concatenate(rows) for rid, rows in got.items()}, reqs, dtype_name,
                        "any cut")


@pytest.mark.parametrize("name", ["B", "C", "D"])
def test_the_invariant_mode_gives_the_same_bits_however_the_work_is_cut(model_dirs, name):
    """bfloat16 with ``invariant``: whole prompts alone, the last 32 tokens one by one (as graphs), unequal
    batches in two orders and pieces of 70 tokens (two slices of the product kernel) give the same logits bit
    for bit, and they are the plain implementation's within the bfloat16 bound."""
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.parts import load_model
    cfg, _ = read_model_f64(model_dirs[name])
    reqs = requests_for(name, cfg, [150, 37, 70, 1, 97], 77)
    model = load_model(model_dirs[name], torch.bfloat16, invariant=True)
    assert model.rt.invariant
    whole = replay_in_process(model, plans.whole(reqs))
    check_against_plain(model_dirs[name], whole, reqs, "bfloat16", "invariant mode, whole")
    ids = list(reqs)
    cuts = {
        "one by one": replay_in_process(model, plans.tail_one_by_one(reqs, 32)),
        "a batch": replay_in_process(model, plans.unequal_batches([{r: (reqs[r], max(1, len(reqs[r]) - 9)) for r in ids}])),
        "the batch the other way round": replay_in_process(
            model, plans.unequal_batches([{r: (reqs[r], max(1, len(reqs[r]) - 20)) for r in reversed(ids)}])),
    }
    engine = Engine(model, model.new_cache(max_tokens=5 * 192, num_slots=5, max_seq_len=192))
    slots = {r: engine.cache.acquire() for r in ids}
    pieces = {r: [] for r in ids}
    for at in range(0, 150, 70):
        live = [r for r in ids if len(reqs[r]) > at]
        logits = engine.step([StepEntry(slots[r], reqs[r][at:at + 70], "all") for r in live]).cpu().numpy()
        row = 0
        for r in live:
            n = len(reqs[r][at:at + 70])
            pieces[r].append(logits[row:row + n])
            row += n
    cuts["pieces of 70"] = {r: np.concatenate(p) for r, p in pieces.items()}
    for what, got in cuts.items():
        for r in ids:
            assert got[r].shape == whole[r].shape
            differ = np.flatnonzero((got[r].view(np.uint32) != whole[r].view(np.uint32)).any(axis=1))
            assert differ.size == 0, (f"{what}, request {r}: position {differ[0]} is the first of {differ.size} whose "
                                      f"logits differ from the whole prompt's, by {rel_to_max(got[r], whole[r]):.1e}")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_one_layer_of_the_large_model(tmp_path_factory, dtype_name):
    """The layer sizes of Qwen3-8B (one layer, a small vocabulary): the sizes at which the decode kernels
    choose their forms (rows shared by four wavefronts, packed weights, norms left to the products, the
    attention kernel that also norms and rotates) run here end to end, eagerly and as graphs."""
    from rust_inference_amd.engine import Engine
    from rust_inference_amd.engine.replay import Replayer
    from rust_inference_amd.parts import load_model
    cfg = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 1000, "hidden_size": 4096,
           "intermediate_size": 12288, "num_hidden_layers": 1, "num_attention_heads": 32, "num_key_value_heads": 8,
           "head_dim": 128, "rope_theta": 1e6, "rms_norm_eps": 1e-6, "tie_word_embeddings": False}
    folder = _large_layer_folder(tmp_path_factory, cfg)
    rng = np.random.default_rng(5)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, 1000, n)] for i, n in enumerate([290, 41, 130])}
    model = load_model(folder, DTYPES[dtype_name])
    for graphs in (False, True):
        for what, steps in (("tail", plans.tail_one_by_one(reqs, 32)),
                            ("batch", plans.unequal_batches([{k: (v, max(1, len(v) - 9)) for k, v in reqs.items()}]))):
            cache = model.new_cache(max_tokens=plans.max_live_tokens(steps), num_slots=3, max_seq_len=320)
            player, outs = Replayer(Engine(model, cache, use_graphs=graphs)), {}
            for s in steps:
                logits = player.feed(s)
                if logits is not None:
                    outs[s["step"]] = logits.cpu().numpy().copy()
            got = plans.collect(steps, lambda i: outs[i], 1000)
            check_against_plain(folder, got, reqs, dtype_name, f"large layer, {what}, graphs {graphs}")


# The layer sizes of the published Qwen3 dense checkpoints (name: hidden, intermediate, heads, kv heads): what the
# kernels' rules choose at each (rows of 1,024 to 25,600 elements, 2 to 8 query heads a kv head, K of 2,560 and
# 9,728 that the ring of eight steps does not divide).
PUBLISHED = {"0.6B": (1024, 3072, 16, 8), "1.7B": (2048, 6144, 16, 8), "4B": (2560, 9728, 32, 8),
             "8B": (4096, 12288, 32, 8), "14B": (5120, 17408, 40, 8), "32B": (5120, 25600, 64, 8)}


@pytest.mark.parametrize("size", list(PUBLISHED))
def test_one_layer_of_every_published_size(tmp_path, size):
    """One layer and a small vocabulary at each size, bfloat16, through graphs: a request alone with its last
    tokens one by one (the one-row products), batches of five, twenty, forty-four and ninety of unequal lengths (the
    packed products of 2 to 16 rows, the wide ones of 17 to 32, of 33 to 64 and of 65 to 128, the library's for the
    prompts)."""
    from rust_inference_amd.engine import Engine
    from rust_inference_amd.engine.replay import Replayer
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    hidden, inter, heads, kv_heads = PUBLISHED[size]
    cfg = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 1000, "hidden_size": hidden,
           "intermediate_size": inter, "num_hidden_layers": 1, "num_attention_heads": heads,
           "num_key_value_heads": kv_heads, "head_dim": 128, "rope_theta": 1e6, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": size in ("0.6B", "1.7B", "4B")}
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=11, dtype=torch.bfloat16, matrix_std=0.02, gain_std=0.1)
    rng = np.random.default_rng(len(size) + hidden)
    model = load_model(folder, torch.bfloat16)
    try:
        # (150 at a time where the down product takes 129 to 256 rows in two passes of its own kernel)
        for count, tail in ((1, 12), (5, 6), (20, 5), (44, 4), (90, 4)) + (((150, 3),) if inter >= 16384 else ()):
            longest = 140 if count == 1 else 48 if count < 90 else 20 if count < 150 else 12
            reqs = {f"{size}_{count}_{i}": [int(t) for t in rng.integers(0, 1000, n)]
                    for i, n in enumerate(rng.integers(tail + 1, longest, count))}
            steps = (plans.tail_one_by_one(reqs, tail) if count == 1 else
                     plans.unequal_batches([{k: (v, len(v) - int(rng.integers(1, tail + 1))) for k, v in reqs.items()}]))
            cache = model.new_cache(max_tokens=plans.max_live_tokens(steps), num_slots=count, max_seq_len=192)
            player, outs = Replayer(Engine(model, cache, use_graphs=True)), {}
            for st in steps:
                logits = player.feed(st)
                if logits is not None:
                    outs[st["step"]] = logits.cpu().numpy().copy()
            got = plans.collect(steps, lambda i: outs[i], 1000)
            check_against_plain(folder, got, reqs, "bfloat16", f"one layer of {size}, {count} at a time")
    finally:
        _plain_cache.clear()
        _last_read.clear()                                    # (the float64 weights of the largest are 4 GB)


_large = {}


def _large_layer_folder(tmp_path_factory, cfg):
    """Written once for both dtypes (0.4 GB)."""
    if "folder" not in _large:
        from rust_inference_amd.weights import write_random_model
        _large["folder"] = write_random_model(str(tmp_path_factory.mktemp("large") / "m"), cfg, seed=3,
                                              dtype=torch.bfloat16, matrix_std=0.02, gain_std=0.1)
    return _large["folder"]
