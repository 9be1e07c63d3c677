"""The generation loop's decisions with a scripted step function (no GPU, no model)."""
import pytest
import torch

from rust_inference_amd.cache import Cache, KVNeed
from plain.step_layout_plain import plan_step
from rust_inference_amd.engine import generate, plan_batches, StepEntry, wanted_indices
from rust_inference_amd.errors import CacheError, ShapeError
from rust_inference_amd.sampling import SamplingParams

VOCAB = 50


class ScriptedEngine:
    """Stands in for the engine: the next token of a sequence is a function of its last token and length,
    so the expected output of every request is known whatever batch it is in."""

    def __init__(self, slots=4, max_tokens=1024, max_seq_len=256):
        self.cache = Cache([KVNeed(1, 16)], slots, max_tokens, max_seq_len, dtype=torch.float32, device="cpu",
                           allocate=False)
        self.steps = []                       # (slots, counts) of every step

    @staticmethod
    def rule(last_token, length):
        return (3 * last_token + length) % VOCAB

    def step(self, entries):
        slots = [e.slot for e in entries]
        counts = [len(e.tokens) for e in entries]
        self.cache.reserve(slots, counts)
        self.cache.commit(slots, counts)
        self.steps.append((slots, counts))
        logits = torch.zeros(len(entries), VOCAB)
        for i, e in enumerate(entries):
            assert e.want == "last"
            logits[i, self.rule(e.tokens[-1], self.cache.length(e.slot))] = 5.0
        return logits


def expected(prompt, n, stop=()):
    out, last, length = [], prompt[-1], len(prompt)
    for _ in range(n):
        nxt = ScriptedEngine.rule(last, length)
        if nxt in stop:
            return out, "stop"
        out.append(nxt)
        last, length = nxt, length + 1
    return out, "length"


def test_unequal_prompts_in_one_batch_match_each_alone():
    eng = ScriptedEngine()
    prompts = [[1, 2, 3, 4, 5], list(range(11)), [7], list(range(17))]
    res = generate(eng, prompts, max_new_tokens=8)
    for p, toks, why in zip(prompts, res.tokens, res.finish_reasons):
        assert (toks, why) == expected(p, 8)
    assert eng.steps[0] == ([0, 1, 2, 3], [5, 11, 1, 17])           # all prompts in one step
    assert all(c == [1, 1, 1, 1] for _, c in eng.steps[1:]) and len(eng.steps) == 8   # the 8th token is not fed
    assert res.stats.prompt_tokens == 34 and res.stats.decode_tokens == 4 * 7 and res.stats.decode_steps == 7
    eng.cache.check_consistent()
    assert eng.cache.slots.free_count == 4 and eng.cache.free_pages() == [32]


def test_first_token_counts_and_one_token_needs_no_decode_step():
    eng = ScriptedEngine()
    res = generate(eng, [[4, 5, 6]], max_new_tokens=1)
    assert res.tokens == [expected([4, 5, 6], 1)[0]] and res.finish_reasons == ["length"] and len(eng.steps) == 1
    with pytest.raises(ShapeError):
        generate(eng, [[1]], max_new_tokens=0)
    with pytest.raises(ShapeError, match="empty prompt"):
        generate(eng, [[1], []], max_new_tokens=2)


def test_stop_token_ends_a_sequence_early_and_is_not_output():
    prompts = [[1, 2, 3], [9, 9], [5]]
    full = [expected(p, 10)[0] for p in prompts]
    stop = {full[1][3]}                                            # the fourth token of request 1
    eng = ScriptedEngine()
    res = generate(eng, prompts, max_new_tokens=10, stop_token_ids=stop)
    for p, toks, why in zip(prompts, res.tokens, res.finish_reasons):
        assert (toks, why) == expected(p, 10, stop)
    assert res.finish_reasons[1] == "stop" and len(res.tokens[1]) <= 3 and next(iter(stop)) not in res.tokens[1]
    # after request 1 has ended, the steps carry the others only, and its slot went back at once
    sizes = [len(s) for s, _ in eng.steps]
    assert sizes[0] == 3 and sizes[-1] == 2 and sizes == sorted(sizes, reverse=True)
    assert all(1 not in s for s, _ in eng.steps[len(res.tokens[1]) + 1:])
    res2 = generate(ScriptedEngine(), prompts, max_new_tokens=10, stop_token_ids=stop, ignore_eos=True)
    assert res2.tokens == full and res2.finish_reasons == ["length"] * 3


def test_stop_token_as_the_very_first_token():
    p = [3, 4]
    first = expected(p, 1)[0][0]
    res = generate(ScriptedEngine(), [p, [8]], max_new_tokens=5, stop_token_ids=[first])
    assert res.tokens[0] == [] and res.finish_reasons[0] == "stop"
    assert (res.tokens[1], res.finish_reasons[1]) == expected([8], 5, {first})


def test_more_requests_than_slots_run_as_batches_one_after_another():
    eng = ScriptedEngine(slots=2)
    prompts = [[i + 1] * (i + 1) for i in range(5)]
    res = generate(eng, prompts, max_new_tokens=4)
    assert [t for t in res.tokens] == [expected(p, 4)[0] for p in prompts]
    assert res.stats.batches == 3
    assert [eng.steps[i][1] for i in (0, 4, 8)] == [[1, 2], [3, 4], [5]]     # a prompt step opens every batch
    # slots are used again by the later batches
    assert {s for sl, _ in eng.steps for s in sl} == {0, 1}
    eng.cache.check_consistent()
    assert eng.cache.slots.free_count == 2


class AheadEngine(ScriptedEngine):
    """The scripted engine with steps that take their tokens as ids "on the device" (here: a tensor the loop
    has not read), as the real engine's captured graphs do; like it, it has no such step for a batch size
    until a step with the tokens themselves has run at that size."""

    def __init__(self, *a, **k):
        super().__init__(*a, **k)
        self.known_sizes, self.on_device = set(), []

    def step(self, entries):
        if all(len(e.tokens) == 1 for e in entries):
            self.known_sizes.add(len(entries))
        return super().step(entries)

    def decode_on_device(self, slots, ids):
        if len(slots) not in self.known_sizes:
            return None
        assert ids.dtype == torch.int32 and ids.shape == (len(slots),)
        self.on_device.append(list(slots))
        return ScriptedEngine.step(self, [StepEntry(s, [int(t)], "last") for s, t in zip(slots, ids.tolist())])


def test_one_step_ahead_gives_the_same_tokens_and_carries_an_ended_sequence_one_step_at_most():
    prompts = [[1, 2, 3], [9, 9], [5], [4, 4, 4, 4]]
    full = [expected(p, 12)[0] for p in prompts]
    others = set(full[0]) | set(full[2])
    stop = {next(t for t in full[1][2:] if t not in others), next(t for t in full[3][5:] if t not in others)}
    plain = generate(ScriptedEngine(), prompts, max_new_tokens=12, stop_token_ids=stop)
    eng = AheadEngine()
    res = generate(eng, prompts, max_new_tokens=12, stop_token_ids=stop)
    assert res.tokens == plain.tokens and res.finish_reasons == plain.finish_reasons
    for p, toks, why in zip(prompts, res.tokens, res.finish_reasons):
        assert (toks, why) == expected(p, 12, stop)
    assert "stop" in res.finish_reasons and "length" in res.finish_reasons
    assert eng.on_device, "steps did run with ids the loop had not read"
    # what the statistics count is what the plain loop counts: steps and tokens that were asked for
    assert res.stats.decode_tokens == plain.stats.decode_tokens and res.stats.decode_steps == plain.stats.decode_steps
    # a sequence is fed at most one token more than the plain loop feeds it (the step that was launched before
    # its stop token was read), and never more than its pages were planned for
    fed = {r: 0 for r in range(len(prompts))}
    for slots, counts in eng.steps[1:]:
        for sl in slots:
            fed[sl] += 1
    for r, toks in enumerate(res.tokens):
        wanted = len(toks) if res.finish_reasons[r] == "stop" else len(toks) - 1
        assert wanted <= fed[r] <= wanted + 1 and fed[r] <= 11
    eng.cache.check_consistent()
    assert eng.cache.slots.free_count == 4 and eng.cache.free_pages() == [32]


def test_one_step_ahead_with_a_stop_token_first_and_batches_one_after_another():
    p = [3, 4]
    first = expected(p, 1)[0][0]
    res = generate(AheadEngine(), [p, [8]], max_new_tokens=5, stop_token_ids=[first])
    assert res.tokens[0] == [] and res.finish_reasons[0] == "stop"
    assert (res.tokens[1], res.finish_reasons[1]) == expected([8], 5, {first})
    eng = AheadEngine(slots=2)
    prompts = [[i + 1] * (i + 1) for i in range(5)]
    res = generate(eng, prompts, max_new_tokens=4)
    assert res.tokens == [expected(q, 4)[0] for q in prompts] and res.stats.batches == 3
    eng.cache.check_consistent()
    assert eng.cache.slots.free_count == 2
    one = generate(AheadEngine(), [[4, 5, 6]], max_new_tokens=1)
    assert one.tokens == [expected([4, 5, 6], 1)[0]] and one.finish_reasons == ["length"]
    # everything stops at once: the step launched ahead was for nobody, and is not counted
    q = [[7], [7]]
    second = expected([7], 2)[0][1]
    both = generate(AheadEngine(), q, max_new_tokens=9, stop_token_ids=[second])
    assert both.tokens == [expected([7], 9, {second})[0]] * 2 and both.finish_reasons == ["stop", "stop"]
    assert both.stats.decode_steps == 1 and both.stats.decode_tokens == 2


def test_one_step_ahead_draws_the_same_numbers_as_the_plain_loop():
    class Flat(AheadEngine):
        def step(self, entries):
            super().step(entries)
            return torch.zeros(len(entries), VOCAB)

        def decode_on_device(self, slots, ids):
            out = super().decode_on_device(slots, ids)
            return None if out is None else torch.zeros(len(slots), VOCAB)

    class FlatPlain(ScriptedEngine):
        def step(self, entries):
            super().step(entries)
            return torch.zeros(len(entries), VOCAB)
    prompts = [[1], [2], [3]]
    p = SamplingParams(temperature=1.0, seed=11)
    assert generate(Flat(), prompts, 9, p).tokens == generate(FlatPlain(), prompts, 9, p).tokens
    # with a repetition penalty the tokens are needed on the host before the next step: no step runs ahead
    eng = AheadEngine()
    generate(eng, prompts, 5, SamplingParams(repetition_penalty=1.2))
    assert not eng.on_device


def test_batches_are_cut_to_fit_the_pages():
    # pages of 32: each request of 40 + 30 - 1 = 69 tokens needs 3 pages; 7 pages hold two of them
    assert plan_batches([40, 40, 40], 30, 32, 7, 8, 256) == [range(0, 2), range(2, 3)]
    assert plan_batches([40, 40, 40], 30, 32, 9, 8, 256, max_batch=2) == [range(0, 2), range(2, 3)]
    assert plan_batches([1], 1, 32, 1, 1, 32) == [range(0, 1)]
    with pytest.raises(CacheError, match="needs 3 pages"):
        plan_batches([40], 30, 32, 2, 8, 256)
    with pytest.raises(CacheError, match="may hold"):
        plan_batches([250], 30, 32, 64, 8, 256)
    eng = ScriptedEngine(slots=8, max_tokens=7 * 32)
    res = generate(eng, [[1] * 40, [2] * 40, [3] * 40], max_new_tokens=30)
    assert res.stats.batches == 2 and all(len(t) == 30 for t in res.tokens)


def test_temperature_sampling_is_per_sequence_and_seeded():
    class Flat(ScriptedEngine):
        def step(self, entries):
            super().step(entries)
            return torch.zeros(len(entries), VOCAB)            # uniform: the draw decides alone
    prompts = [[1], [2], [3]]
    p = SamplingParams(temperature=1.0, seed=11)
    a = generate(Flat(), prompts, 6, p).tokens
    b = generate(Flat(), prompts, 6, p).tokens
    alone = generate(Flat(), prompts[:1], 6, p).tokens
    other = generate(Flat(), prompts, 6, SamplingParams(temperature=1.0, seed=12)).tokens
    assert a == b and a[0] == alone[0] and a != other and a[0] != a[1]


def test_plan_step_layout():
    entries = [StepEntry(3, [5, 6, 7], [0, 2]), StepEntry(0, [9], "last"), StepEntry(1, [1, 2], "none")]
    tokens, seq, pos, cu, want = (a.tolist() for a in plan_step(entries, [10, 0, 4], VOCAB))
    assert tokens == [5, 6, 7, 9, 1, 2] and seq == [0, 0, 0, 1, 2, 2] and pos == [10, 11, 12, 0, 4, 5]
    assert cu == [0, 3, 4, 6] and want == [0, 2, 3]
    assert wanted_indices(4, "all") == [0, 1, 2, 3]
    with pytest.raises(ShapeError, match="outside the vocabulary"):
        plan_step([StepEntry(0, [VOCAB])], [0], VOCAB)
    with pytest.raises(ShapeError, match="outside the entry"):
        plan_step([StepEntry(0, [1], [1])], [0], VOCAB)
    with pytest.raises(ShapeError, match="no token"):
        plan_step([StepEntry(0, [])], [0], VOCAB)
    one_each = plan_step([StepEntry(2, [5]), StepEntry(0, [6])], [7, 3], VOCAB)      # the decode step's short cut
    assert [a.tolist() for a in one_each] == [[5, 6], [0, 1], [7, 3], [0, 1, 2], [0, 1]]


def test_native_step_layout_is_the_plain_one():
    """The cache's native side lays a step out into one block of words; piece by piece it is what
    plan_step says, with the page tables of the step's slots behind."""
    import numpy as np
    from rust_inference_amd.cache import native
    cache = Cache([KVNeed(1, 16), KVNeed(2, 16, 40)], 4, 1024, 256, dtype=torch.float32, device="cpu", allocate=False)
    slots = [cache.acquire() for _ in range(3)]
    cache.reserve(slots[:2], [70, 5]); cache.commit(slots[:2], [70, 5])
    entries = [StepEntry(slots[2], [5, 6, 7], [0, 2]), StepEntry(slots[0], [9], "last"), StepEntry(slots[1], [1, 2], "none")]
    order, counts = [e.slot for e in entries], [len(e.tokens) for e in entries]
    want_plain = plan_step(entries, [cache.length(s) for s in order], VOCAB)
    cache.reserve(order, counts)
    width, words, offsets = 3, np.zeros(400, dtype=np.int32), np.zeros(7 + len(cache.groups), dtype=np.int64)
    arr = lambda a: np.asarray(a, dtype=np.int32)
    s_arr, c_arr, t_arr, w_arr = arr(order), arr(counts), want_plain[0], want_plain[4]
    used = native.lib().ri_cache_plan_step(cache.core.handle, s_arr.ctypes.data, c_arr.ctypes.data, 3, t_arr.ctypes.data,
                                           w_arr.ctypes.data, len(w_arr), VOCAB, width, words.ctypes.data, len(words),
                                           offsets.ctypes.data)
    assert used > 0 and all(o % 4 == 0 for o in offsets.tolist())
    sizes = [6, 6, 6, 4, 3, 3, len(w_arr)]
    got = [words[o:o + n].tolist() for o, n in zip(offsets.tolist(), sizes)]
    assert got[:4] == [a.tolist() for a in want_plain[:4]] and got[6] == w_arr.tolist()
    assert got[4] == order and got[5] == [3, 71, 7]
    for gi, g in enumerate(cache.groups):
        table = words[offsets[7 + gi]:offsets[7 + gi] + 3 * width].reshape(3, width)
        assert table.tolist() == g.pool.gather(order, width).tolist()
    assert native.lib().ri_cache_plan_step(cache.core.handle, s_arr.ctypes.data, c_arr.ctypes.data, 3, t_arr.ctypes.data,
                                           w_arr.ctypes.data, len(w_arr), 7, width, words.ctypes.data, len(words),
                                           offsets.ctypes.data) == -1            # token 9 in a vocabulary of 7
    assert "outside the vocabulary" in native.lib().ri_last_error().decode()


# ------------------------------------------------------------------------------------------------ the command line
def test_runner_options_are_the_references():
    """Names, short forms and defaults of src/bin/runner.rs:24-123 for the options this build has."""
    from rust_inference_amd.engine.runner import build_parser
    a = build_parser().parse_args(["some/dir"])
    assert (a.model_dir, a.prompt, a.max_new_tokens, a.chat, a.think, a.ignore_eos) == ("some/dir", None, 600, False, False, False)
    assert (a.max_pages, a.pages_per_seq, a.threads, a.profile) == (256, 128, None, False)
    assert (a.temperature, a.top_k, a.top_p, a.repetition_penalty, a.seed) == (0.0, 0, 1.0, 1.0, 0x5EED)
    b = build_parser().parse_args(["d", "-p", "hello", "-n", "7", "-t", "3", "--temperature", "0.5", "--top-k", "4", "--top-p",
                                   "0.9", "--repetition-penalty", "1.1", "--seed", "0x10", "--chat", "--think",
                                   "--ignore-eos", "--tokenizer", "tok", "--max-pages", "9", "--pages-per-seq", "2"])
    assert (b.prompt, b.max_new_tokens, b.threads, b.seed, b.tokenizer) == (["hello"], 7, 3, 16, "tok")
    assert b.chat and b.think and b.ignore_eos and (b.max_pages, b.pages_per_seq) == (9, 2)


def test_chat_prompt_and_streamed_text():
    from rust_inference_amd.engine.runner import StreamPrinter, chat_prompt
    # src/tokenizer/mod.rs:402-408
    assert chat_prompt("hi", True) == "<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n"
    assert chat_prompt("hi", False) == "<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n"

    class TwoByteTokenizer:                                  # ids are bytes: a character may span two tokens
        def decode(self, ids):
            return bytes(ids).decode("utf-8", errors="replace")

    import io
    out = io.StringIO()
    printer = StreamPrinter(TwoByteTokenizer(), out)
    pieces = []
    for b in "aé!".encode():
        printer.push(b)
        pieces.append(out.getvalue())
    assert pieces == ["a", "a", "aé", "aé!"]                 # nothing is printed for half a character
    out = io.StringIO()
    StreamPrinter(None, out).push(17)
    assert out.getvalue() == "17 "


def test_runner_refuses_what_it_cannot_do(tmp_path, capsys):
    from rust_inference_amd.engine.runner import main
    with pytest.raises(SystemExit):
        main([str(tmp_path), "-p", "1 2", "--think"])        # --think requires --chat
    assert main([str(tmp_path), "-p", "hello", "--chat"]) == 1          # no tokenizer.json in the folder
    assert "tokenizer.json" in capsys.readouterr().err
    assert main([str(tmp_path), "-p", ""]) == 1
    assert "empty prompt" in capsys.readouterr().err
    # a text prompt where there is no tokenizer.json, and ids that are none: `error: ...` and exit status 1,
    # as every other failure (src/bin/runner.rs:225-237), not a traceback
    assert main([str(tmp_path), "-p", "once upon a time"]) == 1
    err = capsys.readouterr().err
    assert err.startswith("error: the prompt is text") and "tokenizer.json" in err and "Traceback" not in err
    assert main([str(tmp_path), "--prompt-ids", "5,x,7"]) == 1
    assert capsys.readouterr().err.startswith("error: --prompt-ids")


def test_the_bound_that_sizes_a_decode_step():
    """A power of two of tokens, 1,024 at least, the cache's limit at most: the same for a step that is
    launched from the host and for its graph."""
    from types import SimpleNamespace
    from rust_inference_amd.engine.step import _decode_bound
    cache = SimpleNamespace(max_seq_len=20000)
    assert [_decode_bound(cache, n) for n in (1, 1024, 1025, 4096, 4097, 16384, 16385, 30000)] == \
        [1024, 1024, 2048, 4096, 8192, 16384, 20000, 20000]


def test_which_decode_steps_the_attention_walks_in_runs():
    """The rule is host code of the kernel library: one run a sequence from 512 (sequence, kv head) pairs on;
    below that, runs of eight chunks and more that make 512 workgroups, from 16,384 keys on; else chunks."""
    from rust_inference_amd.kernels import ops
    runs = ops.decode_attention_runs
    assert runs(64, 8, 2100) == 1 and runs(256, 2, 300) == 1 and runs(63, 8, 2100) == 0
    assert runs(8, 8, 32896) == 16 and runs(4, 8, 32896) == 16 and runs(1, 8, 131200) == 64
    assert runs(1, 8, 32896) == 0                      # 16 runs of eight chunks would be 128 workgroups
    assert runs(16, 8, 4200) == 0 and runs(48, 8, 2100) == 0 and runs(32, 8, 8192) == 0
    assert runs(8, 8, 16384) == 8 and runs(8, 8, 16000) == 0


def test_every_request_may_sample_in_its_own_way():
    """A list of sampling parameters, one per prompt: a request's tokens are those it gets when all requests
    share its parameters (its generator is seeded by its index either way), and a list of the wrong length is
    refused."""
    class Peaked(ScriptedEngine):
        def step(self, entries):
            logits = super().step(entries)
            return logits + 0.5 * torch.sin(torch.arange(VOCAB) * 0.7)[None, :]      # a few plausible tokens each

    prompts = [[1, 2, 3], [4, 5], [6], [7, 8, 9, 10]]
    kinds = [SamplingParams(), SamplingParams(temperature=5.0, seed=11), SamplingParams(temperature=5.0, top_k=3, seed=11),
             SamplingParams(temperature=2.0, top_p=0.5, repetition_penalty=1.3, seed=11)]
    mixed = generate(Peaked(), prompts, max_new_tokens=6, sampling=kinds).tokens
    for i, kind in enumerate(kinds):
        alone = generate(Peaked(), prompts, max_new_tokens=6, sampling=kind).tokens
        assert mixed[i] == alone[i], f"request {i}"
    assert len({tuple(t) for t in mixed}) > 1
    with pytest.raises(ShapeError, match="sampling parameters"):
        generate(Peaked(), prompts, max_new_tokens=2, sampling=kinds[:2])


def test_whether_a_graph_waits_for_a_batch_size_to_come_back_goes_by_the_models_size():
    """Capturing at a size's first step pays where launching a step costs what the step costs (a small model); a
    model whose weights take longer to read than its kernels to launch captures a size only when it has come back."""
    import types
    import bench
    from rust_inference_amd.api import capture_after_for
    from rust_inference_amd.config import config_from_dict
    from rust_inference_amd.parts.model import DecoderModel
    waits = {}
    for which, (_, shapes, _) in bench.MODELS.items():
        arch, cfg = config_from_dict(dict(shapes))
        model = DecoderModel(arch.build_spec(cfg))
        model.rt = types.SimpleNamespace(dtype=torch.bfloat16)
        waits[which] = capture_after_for(model)
    assert waits == {"0.6b": 0, "1.7b": 0, "4b": 0, "8b": 3, "14b": 3, "32b": 3}
    assert capture_after_for(object()) == 0                 # nothing known about it: as before
