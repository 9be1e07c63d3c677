"""The CPU backend (`Model.load(..., device="cpu")`, `runner --device cpu`): the whole model over the plain forms of
the parts (scalar C++ twins of the kernels, float32), through the same cache bookkeeping, step interface and
generation loop as the GPU engine.  Held here, without a GPU, to the float64 plain implementation on two tiny
configurations in every cut, and to the logits and tokens the reference's authors recorded for their fixture."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import trace_plans as plans
from helpers import read_model_f64, reference_fixture, rel_to_max
from plain import qwen3_plain as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name, lengths", [("A", [5, 11, 1, 17]), ("B", [33, 2, 40])])
def test_every_cut_matches_the_plain_implementation(model_dirs, name, lengths):
    from rust_inference_amd import Model
    from rust_inference_amd.engine.replay import Replayer
    cfg, w = read_model_f64(model_dirs[name])
    rng = np.random.default_rng(5)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab_size"], n + 9)] for i, n in enumerate(lengths)}
    want = {rid: P.forward(cfg, w, toks) for rid, toks in reqs.items()}
    for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 8)),
                        ("batches", plans.unequal_batches([{k: (v, len(v) - 9) for k, v in list(reqs.items())[:2]},
                                                           {k: (v, len(v) - 9) for k, v in list(reqs.items())[2:]}]))):
        model = Model.load(model_dirs[name], dtype="float32", device="cpu", max_batch=2, max_seq_len=64,
                           max_tokens=plans.max_live_tokens(steps))
        player, outs = Replayer(model.engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.numpy()
        model.cache.check_consistent()
        got = plans.collect(steps, lambda i: outs[i], cfg["vocab_size"])
        for rid in reqs:
            err = rel_to_max(got[rid], want[rid])
            assert err <= 1e-4, f"{name}, {what}, {rid}: {err:.2e} of the largest logit"


def test_generation_and_the_reference_fixture():
    """The fixture of the reference (tests/fixtures/tiny-qwen3): logits at every prompt position within its own bound
    (2e-4 of the largest + 1e-5, tests/model_parity.rs:23-28), then its seven greedy tokens through generate()."""
    folder = reference_fixture("tiny-qwen3")
    if folder is None:
        pytest.skip("the reference's fixture is not at hand")
    from rust_inference_amd import Model
    with open(os.path.join(folder, "expected.json")) as f:
        expected = json.load(f)
    prompt, vocab = expected["prompt"], 3072
    model = Model.load(folder, dtype="float32", device="cpu", max_batch=2, max_seq_len=64)
    slot = model.cache.acquire()
    logits = model.step([(slot, prompt, "all")]).numpy()
    model.cache.release(slot)
    want = np.fromfile(os.path.join(folder, "expected_prefill.f32"), dtype="<f4").reshape(len(prompt), vocab)
    assert np.abs(logits - want).max() <= 2e-4 * np.abs(want).max() + 1e-5
    res = model.generate([prompt, prompt[:4]], max_new_tokens=len(expected["generated"]))
    assert res.tokens[0] == expected["generated"] and res.finish_reasons == ["length", "length"]
    model.cache.check_consistent()
    assert model.cache.slots.free_count == 2


def test_the_runner_on_the_cpu(model_dirs):
    cfg, w = read_model_f64(model_dirs["A"])
    toks, _ = P.greedy(cfg, w, [5, 17, 3], 5)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "runner"), model_dirs["A"], "--device", "cpu", "-p", "5 17 3",
                          "-n", "5", "--ignore-eos"], capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert run.stdout.split() == [str(t) for t in toks]
    assert "decode: 4 tokens" in run.stderr
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "runner"), model_dirs["A"], "--device", "cpu", "--dtype",
                          "bfloat16", "--random", "-p", "1"], capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert bad.returncode == 1 and "error" in bad.stderr


def test_a_part_without_a_plain_form_is_named():
    from rust_inference_amd.errors import ConfigError
    from rust_inference_amd.parts import DecoderModel, Mixer, register_part
    from rust_inference_amd.parts.qwen3 import qwen3_spec
    from rust_inference_amd.config import config_from_dict
    from conftest import TINY_A
    import dataclasses

    @register_part("mixer", "toy_no_plain_form")
    class Opaque(Mixer):
        def __init__(self, **_):
            pass

    _, cfg = config_from_dict(TINY_A)
    spec = qwen3_spec(cfg)
    layer = spec.layers[0]
    from rust_inference_amd.parts import LayerSpec, PartSpec
    broken = LayerSpec("prenorm", {**dict(layer.parts), "mixer": PartSpec("toy_no_plain_form")})
    spec = dataclasses.replace(spec, layers=(broken,) + tuple(spec.layers[1:]))
    with pytest.raises(ConfigError, match="Opaque has no plain form"):
        DecoderModel(spec).bind_plain({})
