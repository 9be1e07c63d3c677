"""bench.py's contract where no GPU is needed: more than one GPU is refused with one line and exit status 2, and
the bytes and operations that the roofline figures are made of are the ones the configuration implies."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_one_line():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                         capture_output=True, text=True, cwd=ROOT, timeout=120)
    assert run.returncode == 2
    assert len(run.stdout.strip().splitlines()) == 1 and "one GPU" in run.stdout


def test_the_bytes_of_a_decode_step_and_the_operations_of_a_prompt():
    b = _bench()
    c = b.QWEN3_8B
    # a layer's matrices: q|k|v (32 + 2 x 8 heads of 128) x 4096, o 4096 x 4096, gate, up and down 3 x 4096 x 12288
    assert b.layer_matrix_params(c) == 6144 * 4096 + 4096 * 4096 + 3 * 4096 * 12288 == 192_937_984
    weights = 2 * (36 * 192_937_984 + 151936 * 4096 + 8 * 4096)
    gains = 4 * (36 * (2 * 4096 + 2 * 128) + 4096)
    cache = 8 * 2063.5 * 36 * 2 * 8 * 128 * 2                # keys and values of 8 kv heads of 128 in bfloat16, 36 layers
    assert b.decode_bytes(c, 36, 8, 2063.5) == weights + gains + cache
    assert abs(b.decode_bytes(c, 36, 8, 2063.5) / 1e9 - 17.57) < 0.01          # what a step at batch 8 has to read, GB
    t = 2048
    flops = 2 * t * 36 * 192_937_984 + 2 * 151936 * 4096 + 36 * 4 * 128 * 32 * t * (t + 1) // 2
    assert b.prefill_flops(c, 36, t) == flops
    assert abs(flops / 1e12 - 29.69) < 0.01                                    # TFLOP of a 2,048-token prompt
    # the peaks are the published ones
    assert b.HBM_PEAK_GBS == 8000.0 and b.MFMA_PEAK_TFLOPS == {"bf16": 2500.0, "fp32": 157.3}


def test_every_published_size_is_known():
    b = _bench()
    assert sorted(b.MODELS) == ["0.6b", "1.7b", "14b", "32b", "4b", "8b"]
    for name, shapes, seed in b.MODELS.values():
        assert shapes["architectures"] == ["Qwen3ForCausalLM"] and shapes["head_dim"] == 128
        assert shapes["num_attention_heads"] % shapes["num_key_value_heads"] == 0
