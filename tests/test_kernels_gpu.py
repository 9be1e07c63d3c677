"""Each HIP kernel alone against its plain reference, at other sizes than the tiny models use.
Where random inputs would hide a fault, the inputs are made so that it shows.

The same tests run without a GPU when the environment says RI_TEST_KERNELS=emulated: then the kernels are the
CPU build of the same sources (tests/emulated.py), every operand lies between guard pages, and a kernel that
touches memory outside a buffer ends the run with a report.  tests/test_kernels_emulated.py starts that run."""
import os

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

EMULATED = os.environ.get("RI_TEST_KERNELS") == "emulated"
pytestmark = [] if EMULATED else pytest.mark.gpu
DEV = "cpu" if EMULATED else "cuda:0"


@pytest.fixture(scope="module")
def ops():
    if EMULATED:
        import emulated
        return emulated.ops()
    from rust_inference_amd.kernels import ops
    return ops


@pytest.fixture(autouse=True)
def _guarded_buffers_go_back():
    """Emulated: what a test laid between guard pages is unmapped when it ends (a later touch of it would fault)."""
    yield
    if EMULATED:
        import gc
        import emulated
        gc.collect()
        emulated.free_all()


def guarded(x):
    """On the GPU the tensor itself; emulated, a copy between guard pages."""
    if EMULATED:
        import emulated
        return emulated.tensor(x.contiguous(), "a test's operand")
    return x


def t(a, dtype=torch.float32):
    return guarded(torch.tensor(np.asarray(a), dtype=dtype, device=DEV))


def f64(x):
    return x.detach().to("cpu", torch.float64).numpy()


# What a kernel that hands out bfloat16 is held to, from what the comparisons below measured on an MI355X (every
# comparison can write what it measures into the file RI_TEST_ERROR_REPORT names): a bfloat16 result is rounded once
# at the end, half a unit of its last place, which is up to 3.9e-3 of its own size; the attention kernels, the norms
# with rotation and the products with bfloat16 out measure 2.2e-3 to 3.8e-3 of the largest value, and are held to
# twice that.  Where the result went through two such roundings (the fused decode attention reads the key it has just
# rounded; a linked gate|up product rounds its normed input and its result) 4.2e-3 to 4.7e-3 was measured.  Where the
# wanted result is one value row picked out by a score that stands out, rounding hardly shows: 2.8e-4 measured.
BF16_OUT = 7.5e-3
BF16_TWICE = 9.5e-3
BF16_ONE_KEY = 6e-4


def close(got, want, rel, what=""):
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(f64(got) - want).max() / max(np.abs(want).max(), 1e-30)
    report = os.environ.get("RI_TEST_ERROR_REPORT")          # a file that collects what every comparison measured
    if report:
        with open(report, "a") as f:
            f.write(f"{os.environ.get('PYTEST_CURRENT_TEST', '?')}\t{what}\t{err:.3e}\t{rel:.0e}\n")
    assert err <= rel, f"{what}: error {err:.3e} of the largest value exceeds {rel:.0e}"


def test_the_extension_is_loaded_from_the_tree(ops):
    from rust_inference_amd.kernels import load_library
    lib = load_library()
    assert lib.ri_abi_version() >= 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding(ops, dtype):
    rng = np.random.default_rng(0)
    table = t(rng.normal(size=(1000, 200)), dtype)               # a vocabulary and a width that are no power of two
    ids = [999, 0, 2, 2, 517]
    got = ops.embed_gather(table, t(ids, torch.int32))
    assert got.dtype == torch.float32 and np.array_equal(f64(got), P.embedding(f64(table), ids))


@pytest.mark.parametrize("dim", [104, 4096, 5000])
@pytest.mark.parametrize("pending_dtype", [None, torch.float32, torch.bfloat16])
def test_add_rmsnorm(ops, dim, pending_dtype):
    rng = np.random.default_rng(dim)
    res = t(rng.normal(size=(7, dim)) * 3)
    pend = None if pending_dtype is None else t(rng.normal(size=(7, dim)), pending_dtype)
    gain = t(1 + 0.1 * rng.normal(size=dim))
    total = f64(res) + (0 if pend is None else f64(pend))
    want = P.rms_norm(total, f64(gain), 1e-5)
    before = guarded(res.clone())
    out = ops.add_rmsnorm(res, pend, gain, 1e-5, torch.float32)
    close(out, want, 2e-6, "norm")
    close(res, total, 1e-7, "residual written back")
    # rows: the same sums for a few rows, nothing written back
    res2 = guarded(before.clone())
    rows = t([5, 0, 5], torch.int32)
    out2 = ops.add_rmsnorm(res2, pend, gain, 1e-5, torch.bfloat16, rows)
    assert torch.equal(res2, before) and out2.dtype == torch.bfloat16
    close(out2, P.bf16_round(want[[5, 0, 5]].astype(np.float32)), 5e-3, "gathered rows")
    close(ops.add_rows(guarded(before.clone()), pend, rows), total[[5, 0, 5]], 1e-7, "add_rows")


def test_add_rmsnorm_adds_the_parts_of_a_split_product(ops):
    rng = np.random.default_rng(11)
    res, parts = t(rng.normal(size=(6, 4096))), t(rng.normal(size=(3, 6, 4096)))
    gain = t(1 + 0.1 * rng.normal(size=4096))
    total = f64(res) + f64(parts).sum(0)
    out = ops.add_rmsnorm(res, parts, gain, 1e-6, torch.float32)
    close(out, P.rms_norm(total, f64(gain), 1e-6), 2e-6, "norm over parts")
    close(res, total, 2e-7, "residual over parts")
    rows = t([4, 1], torch.int32)
    res2 = t(rng.normal(size=(6, 104)))
    p2 = t(rng.normal(size=(2, 6, 104)))
    g2 = t(np.ones(104))
    want = P.rms_norm((f64(res2) + f64(p2).sum(0))[[4, 1]], np.ones(104), 1e-6)
    close(ops.add_rmsnorm(res2, p2, g2, 1e-6, torch.float32, rows), want, 2e-6, "gathered rows over parts")


@pytest.mark.parametrize("n_parts", [2, 4, 5, 8, 9])
@pytest.mark.parametrize("dim", [72, 1000, 4096, 5120])
def test_the_norm_adds_any_number_of_parts_in_their_order(ops, n_parts, dim):
    """The parts are fetched four at a time; the sum is residual + part 0 + part 1 + ... in float32, bit for bit,
    whatever their number, and a row shorter than the threads' reach is not read beyond its end."""
    rng = np.random.default_rng(n_parts * dim)
    res = t(rng.normal(size=(5, dim)))
    parts = t(rng.normal(size=(n_parts, 5, dim)))
    gain = t(1 + 0.1 * rng.normal(size=dim))
    want_sum = guarded(res.clone())
    for q in range(n_parts):
        want_sum += parts[q]
    got = guarded(res.clone())
    out = ops.add_rmsnorm(got, parts, gain, 1e-6, torch.float32)
    assert torch.equal(got, want_sum)
    close(out, P.rms_norm(f64(want_sum), f64(gain), 1e-6), 2e-6, "norm over parts")


@pytest.mark.parametrize("pending_dtype", [torch.float32, torch.bfloat16])
def test_add_rows_in_place_and_bias(ops, pending_dtype):
    rng = np.random.default_rng(12)
    res, pend = t(rng.normal(size=(7, 104))), t(rng.normal(size=(7, 104)), pending_dtype)
    want = f64(res) + f64(pend)
    got = ops.add_rows(res, pend, in_place=True)
    assert got.data_ptr() == res.data_ptr()
    close(res, want, 1e-7, "the sum is written into the residual itself")
    bias = t(rng.normal(size=104))
    x = t(rng.normal(size=(5, 104)), pending_dtype)
    want = f64(x) + f64(bias)
    close(ops.add_bias(x, bias), want, 1e-7 if pending_dtype == torch.float32 else 5e-3, "bias")


@pytest.mark.parametrize("m, dim, partials, tiled", [(1, 104, 1, False), (5, 4096, 256, False), (16, 584, 37, True),
                                                      (40, 4096, 4096, True)])
def test_a_norm_left_to_a_product_can_be_finished_alone(ops, m, dim, partials, tiled):
    """xg = bfloat16(r * gain) and partial sums of r^2 per row: the normed rows are xg / sqrt(sum / dim + eps)."""
    rng = np.random.default_rng(m + dim)
    r, gain = rng.normal(size=(m, dim)), 1 + 0.1 * rng.normal(size=dim)
    xg = t(r * gain, torch.bfloat16)
    ssq = rng.dirichlet(np.ones(partials), size=m) * (r * r).sum(1, keepdims=True)      # any split of the sums
    if tiled:
        data = ops.TiledRows.empty(m, dim, DEV)
        data.data.zero_()
        padded = torch.zeros((data.data.shape[0] * 16, data.data.shape[1] * 32), dtype=torch.bfloat16, device=DEV)
        padded[:m, :dim] = xg
        data.data.copy_(padded.view(-1, 16, data.data.shape[1], 4, 8).permute(0, 2, 3, 1, 4).reshape(data.data.shape))
        assert torch.equal(data.rows(), xg)
        src = data
    else:
        src = xg
    got = ops.finish_norm(ops.NormedLater(src, t(ssq), 1e-6, dim))
    want = f64(xg) / np.sqrt((r * r).sum(1, keepdims=True) / dim + 1e-6)
    close(got, want, 5e-3, "finished norm")


def test_add_rmsnorm_fused_equals_unfused_bit_for_bit(ops):
    # src/ops/norm.rs:84-98
    a, r = t([[0.5, -1.0, 2.0, 0.25]]), t([[1.0, 1.0, -1.0, 0.0]])
    w = t([1.0, 0.5, 2.0, 1.0])
    res = guarded(r.clone())
    fused = ops.add_rmsnorm(res, a, w, 1e-6, torch.float32)
    plain_sum = (a + r).contiguous()
    assert torch.equal(res, plain_sum)
    assert torch.equal(fused, ops.add_rmsnorm(guarded(plain_sum.clone()), None, w, 1e-6, torch.float32))


def paged(rng, lens, hkv, dh, page_size=32, dtype=torch.float32, spare=3):
    """Keys and values of several sequences laid into pages in a shuffled physical order."""
    pages_per = [-(-n // page_size) for n in lens]
    num_pages = sum(pages_per) + spare
    order = list(rng.permutation(num_pages))
    width = max(pages_per) + 1
    table = np.full((len(lens), width), -1, dtype=np.int32)
    k = [rng.normal(size=(n, hkv, dh)) for n in lens]
    v = [rng.normal(size=(n, hkv, dh)) for n in lens]
    kp = np.zeros((num_pages, hkv, page_size, dh))
    vp = np.zeros((num_pages, hkv, dh, page_size))                 # values lie transposed inside a page
    for b, n in enumerate(lens):
        for lp in range(pages_per[b]):
            table[b, lp] = order.pop()
        for pos in range(n):
            kp[table[b, pos // page_size], :, pos % page_size] = k[b][pos]
            vp[table[b, pos // page_size], :, :, pos % page_size] = v[b][pos]
    return k, v, t(kp, dtype), t(vp, dtype), t(table, torch.int32)


@pytest.mark.parametrize("paged_values", [False, True])
@pytest.mark.parametrize("dtype, rel", [(torch.float32, 3e-6), (torch.bfloat16, BF16_OUT)])
@pytest.mark.parametrize("heads, kv_heads, dh", [(6, 2, 48), (4, 4, 128), (9, 1, 16), (2, 1, 256), (5, 5, 64), (8, 2, 32),
                                                 (4, 2, 8), (6, 3, 24), (3, 1, 40), (2, 2, 2), (2, 1, 328), (4, 2, 512)])
def test_qk_norm_rope_kv_write(ops, dtype, rel, heads, kv_heads, dh, paged_values):
    rng = np.random.default_rng(heads * dh)
    lens_before, new = [37, 0, 63, 30], [3, 2, 5, 70]            # writes cross page boundaries; one spans four pages
    lens = [a + b for a, b in zip(lens_before, new)]
    _, _, kp, vp, table = paged(rng, lens, kv_heads, dh, dtype=dtype)
    kp.zero_(); vp.zero_()
    tokens = sum(new)
    qkv = rng.normal(size=(tokens, (heads + 2 * kv_heads) * dh)) * 2
    qkv_t = t(qkv, dtype)
    qkv = f64(qkv_t)
    tok_seq = [b for b, n in enumerate(new) for _ in range(n)]
    tok_pos = [lens_before[b] + i for b, n in enumerate(new) for i in range(n)]
    qg, kg = 1 + 0.2 * rng.normal(size=dh), 1 + 0.2 * rng.normal(size=dh)
    theta, eps = 50000.0, 1e-5
    inv_freq = t(P.rope_inv_freq(dh, theta))
    # with the sequences' bounds the 16-byte kernels and the page-wise value writer run (where the head size fits)
    extra = dict(cu_seqlens=t(np.concatenate([[0], np.cumsum(new)]), torch.int32), max_new=max(new)) if paged_values else {}
    ops.qk_norm_rope_kv_write(qkv_t, t(qg), t(kg), eps, inv_freq, t(tok_pos, torch.int32), t(tok_seq, torch.int32),
                              table, kp, vp, heads, kv_heads, dh, **extra)
    ang = P.rope_angles(tok_pos, dh, theta)
    q = qkv[:, :heads * dh].reshape(tokens, heads, dh)
    k = qkv[:, heads * dh:(heads + kv_heads) * dh].reshape(tokens, kv_heads, dh)
    v = qkv[:, (heads + kv_heads) * dh:].reshape(tokens, kv_heads, dh)
    q_want = P.apply_rope(P.rms_norm(q, f64(t(qg)), eps), ang)
    k_want = P.apply_rope(P.rms_norm(k, f64(t(kg)), eps), ang)
    close(qkv_t[:, :heads * dh].reshape(tokens, heads, dh), q_want, rel, "q in place")
    tab = table.cpu().numpy()
    for i in range(tokens):
        page, off = tab[tok_seq[i], tok_pos[i] // 32], tok_pos[i] % 32
        close(kp[page, :, off], k_want[i], rel, f"k of token {i}")
        assert np.array_equal(f64(vp[page, :, :, off]), v[i]), "v is a copy"
    # nothing else was written: as many rows are non-zero as tokens
    assert int((kp.float().abs().sum(-1) > 0).sum()) == tokens * kv_heads
    assert int((vp.float().abs().sum(-2) > 0).sum()) == tokens * kv_heads
    # without gains and rotation the kernel only moves k and v
    qkv2 = t(qkv, dtype)
    ops.qk_norm_rope_kv_write(qkv2, None, None, eps, None, t(tok_pos, torch.int32), t(tok_seq, torch.int32),
                              table, kp, vp, heads, kv_heads, dh, **extra)
    assert np.array_equal(f64(qkv2), qkv)


@pytest.mark.parametrize("dtype, rel", [(torch.float32, 3e-6), (torch.bfloat16, BF16_OUT)])
@pytest.mark.parametrize("dh, rot", [(64, 16), (48, 24), (40, 8), (7, 4), (9, 0), (130, 128), (512, 64)])
def test_rotation_over_part_of_the_head(ops, dtype, rel, dh, rot):
    """The first `rot` elements of a head are rotated in pairs (i, i + rot/2) by frequencies of their own, the rest
    is normed only; `rot` 0: no rotation at all, which an odd head size allows."""
    rng = np.random.default_rng(dh + rot)
    heads, kv_heads, new = 3, 1, [5, 40]
    _, _, kp, vp, table = paged(rng, new, kv_heads, dh, dtype=dtype)
    kp.zero_(); vp.zero_()
    tokens = sum(new)
    qkv_t = t(rng.normal(size=(tokens, (heads + 2 * kv_heads) * dh)) * 2, dtype)
    qkv = f64(qkv_t)
    tok_seq = [b for b, n in enumerate(new) for _ in range(n)]
    tok_pos = [i for n in new for i in range(n)]
    qg, kg = 1 + 0.2 * rng.normal(size=dh), 1 + 0.2 * rng.normal(size=dh)
    inv = (1.0 / 10000.0 ** (np.arange(rot // 2) * 2.0 / max(rot, 1))).astype(np.float32) if rot else None
    ops.qk_norm_rope_kv_write(qkv_t, t(qg), t(kg), 1e-5, None if inv is None else t(inv), t(tok_pos, torch.int32),
                              t(tok_seq, torch.int32), table, kp, vp, heads, kv_heads, dh)

    def want(x, gain):
        y = P.rms_norm(x, f64(t(gain)), 1e-5)
        if rot:
            ang = (np.asarray(tok_pos, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)
            y = np.concatenate([P.apply_rope(y[..., :rot], ang), y[..., rot:]], -1)
        return y
    q = qkv[:, :heads * dh].reshape(tokens, heads, dh)
    k = qkv[:, heads * dh:(heads + kv_heads) * dh].reshape(tokens, kv_heads, dh)
    close(qkv_t[:, :heads * dh].reshape(tokens, heads, dh), want(q, qg), rel, "q")
    tab = table.cpu().numpy()
    k_want = want(k, kg)
    for i in range(tokens):
        close(kp[tab[tok_seq[i], tok_pos[i] // 32], :, tok_pos[i] % 32], k_want[i], rel, f"k of token {i}")
    with pytest.raises(Exception, match="frequencies"):
        ops.qk_norm_rope_kv_write(qkv_t, t(qg), t(kg), 1e-5, t(np.ones(dh // 2 + 1, dtype=np.float32)), t(tok_pos, torch.int32),
                                  t(tok_seq, torch.int32), table, kp, vp, heads, kv_heads, dh)


def attention_case(ops, rng, lens, new, heads, kv_heads, dh, dtype, window=None, boost=None, kernel="generic"):
    k, v, kp, vp, table = paged(rng, lens, kv_heads, dh, dtype=dtype, spare=12)
    tokens = sum(new)
    width = (heads + 2 * kv_heads) * dh
    qkv = np.zeros((tokens, width))
    qkv[:, :heads * dh] = rng.normal(size=(tokens, heads * dh))
    tok_seq = [b for b, n in enumerate(new) for _ in range(n)]
    tok_pos = [lens[b] - n + i for b, n in enumerate(new) for i in range(n)]
    if boost is not None:
        boost(qkv, k, kp, table)
    qkv_t = t(qkv, dtype)
    pos_t, seq_t = t(tok_pos, torch.int32), t(tok_seq, torch.int32)
    cu = t(np.concatenate([[0], np.cumsum(new)]), torch.int32)
    scale = 1.0 / np.sqrt(dh)
    if kernel == "generic":
        out = ops.attention(qkv_t, kp, vp, pos_t, seq_t, table, heads, kv_heads, dh, window, scale)
    elif kernel == "prefill":
        out = ops.attention_prefill_bf16(qkv_t, kp, vp, cu, pos_t, table, len(lens), max(new), heads, kv_heads, dh,
                                         window, scale)
    else:
        assert all(n == 1 for n in new)
        # a bound on the length well above the real one: it sizes grid and workspace, never the result
        out = ops.attention_decode_bf16(qkv_t, kp, vp, cu, pos_t, table, len(lens), max(lens) + 300, heads,
                                        kv_heads, dh, window, scale)
    q = f64(qkv_t)[:, :heads * dh].reshape(tokens, heads, dh)
    want = np.zeros((tokens, heads, dh))
    i = 0
    for b, n in enumerate(new):
        kb = np.stack([f64(kp[table[b, p // 32].item(), :, p % 32]) for p in range(lens[b])])
        vb = np.stack([f64(vp[table[b, p // 32].item(), :, :, p % 32]) for p in range(lens[b])])
        want[i:i + n] = P.attention(q[i:i + n], kb, vb, window=window)
        i += n
    return out.reshape(tokens, heads, dh), want


@pytest.mark.parametrize("dtype, rel", [(torch.float32, 3e-6), (torch.bfloat16, BF16_OUT)])
@pytest.mark.parametrize("heads, kv_heads, dh", [(4, 2, 16), (6, 2, 48), (8, 1, 128), (3, 3, 64), (9, 1, 32),
                                                 # any head size: the reference's own attention test runs 8
                                                 # (src/attention.rs:189-219); odd ones; beyond 256
                                                 (4, 2, 8), (6, 2, 24), (2, 1, 40), (3, 1, 7), (2, 2, 1), (2, 1, 328), (2, 1, 512)])
def test_attention_prompts_pieces_and_single_tokens(ops, dtype, rel, heads, kv_heads, dh):
    rng = np.random.default_rng(heads + dh)
    # a whole prompt, a piece of five tokens at the end of 300, one token at 257 (a tile's first key), one at 1
    out, want = attention_case(ops, rng, [70, 300, 257, 1], [70, 5, 1, 1], heads, kv_heads, dh, dtype)
    close(out, want, rel, "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key_among_hundreds(ops, dtype):
    """One key far back gets a score that stands out: the output must be its value, wherever it lies."""
    rng = np.random.default_rng(9)
    heads, kv_heads, dh = 4, 2, 64
    for far in (0, 31, 32, 255, 256, 511, 640):
        def boost(qkv, k, kp, table, far=far):
            # sequence 0's single query, head 1 (kv head 0): q = 8 * k_far / |k_far| * sqrt(dh)
            kf = f64(kp[table[0, far // 32].item(), 0, far % 32])
            qkv[0, dh:2 * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
        out, want = attention_case(ops, rng, [700], [1], heads, kv_heads, dh, dtype, boost=boost)
        close(out, want, 3e-6 if dtype == torch.float32 else BF16_ONE_KEY, f"far key {far}")
        # and the plain result really is that one value (the test is not vacuous)
        assert np.abs(want[0, 1]).max() > 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 32, 33, 100, 256, 300])
def test_attention_window_edges(ops, dtype, window):
    rng = np.random.default_rng(window)
    out, want = attention_case(ops, rng, [290, 40], [34, 40], 4, 2, 32, dtype, window=window)
    close(out, want, 3e-6 if dtype == torch.float32 else BF16_OUT, f"window {window}")


MFMA_SHAPES = [(4, 1, 32), (8, 2, 32), (6, 2, 64), (3, 3, 64), (32, 8, 128), (16, 1, 128), (5, 5, 128)]


@pytest.mark.parametrize("heads, kv_heads, dh", MFMA_SHAPES)
def test_mfma_prefill_attention(ops, heads, kv_heads, dh):
    rng = np.random.default_rng(heads * 7 + dh)
    # whole prompts of unequal lengths (one shorter than a tile, one of one token), and pieces that
    # continue sequences already in the cache, all in one call
    out, want = attention_case(ops, rng, [70, 300, 257, 1, 45, 131], [70, 5, 1, 1, 45, 99], heads, kv_heads, dh,
                               torch.bfloat16, kernel="prefill")
    close(out, want, BF16_OUT, "prefill attention on the matrix cores")


@pytest.mark.parametrize("heads, kv_heads, dh", MFMA_SHAPES)
def test_mfma_decode_attention(ops, heads, kv_heads, dh):
    rng = np.random.default_rng(heads * 11 + dh)
    # lengths at and around page and chunk edges: 1, 32, 33, 256, 257, 512, 700
    lens = [1, 32, 33, 256, 257, 512, 700, 5]
    out, want = attention_case(ops, rng, lens, [1] * len(lens), heads, kv_heads, dh, torch.bfloat16, kernel="decode")
    close(out, want, BF16_OUT, "decode attention on the matrix cores")


@pytest.mark.parametrize("window", [None, 4500])
def test_mfma_decode_attention_over_thousands_of_keys(ops, window):
    """Past 16 chunks of 256 keys the chunks are joined in runs: sequences on both sides of that edge in one
    call, and in the longest a key that stands out, placed in the first run, in a middle one and in the last."""
    heads, kv_heads, dh = 4, 2, 64
    lens = [4096, 4097, 6000, 700]
    for far in (0, 2500, 5999):
        rng = np.random.default_rng(31 + far)

        def boost(qkv, k, kp, table, far=far):
            kf = f64(kp[table[2, far // 32].item(), 0, far % 32])          # sequence 2, kv head 0: query head 1
            qkv[2, dh:2 * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
        out, want = attention_case(ops, rng, lens, [1] * len(lens), heads, kv_heads, dh, torch.bfloat16,
                                   window=window, boost=boost, kernel="decode")
        close(out, want, BF16_OUT, f"far key {far}, window {window}")


def test_mfma_decode_attention_joins_more_chunks_than_a_run_fetches_at_once(ops):
    """One kv head and 40,000 keys: 157 chunks, too few workgroups to stream, joined in eight runs of 20 chunks,
    which a run fetches sixteen at a time.  A key that stands out among the first sixteen chunks of a run, among
    its last four, and in the sequence's last chunk; beside it a sequence of 20 chunks (runs of three)."""
    heads, kv_heads, dh = 2, 1, 32
    lens = [40000, 5000]
    assert not ops.decode_attention_streams(len(lens), kv_heads, max(lens) + 300)
    for far in (100, 256 * 18 + 7, 39990):
        rng = np.random.default_rng(61 + far)

        def boost(qkv, k, kp, table, far=far):
            kf = f64(kp[table[0, far // 32].item(), 0, far % 32])          # sequence 0, query head 1
            qkv[0, dh:2 * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
        out, want = attention_case(ops, rng, lens, [1] * len(lens), heads, kv_heads, dh, torch.bfloat16, boost=boost,
                                   kernel="decode")
        close(out, want, BF16_OUT, f"far key {far}")
        assert np.abs(want[0, 1]).max() > 0


@pytest.mark.parametrize("heads, kv_heads, dh, window", [(16, 8, 32, None), (16, 8, 32, 100), (16, 8, 32, 300),
                                                         (32, 8, 128, None), (32, 8, 128, 300), (8, 8, 64, None)])
def test_mfma_decode_attention_streams_over_many_sequences(ops, heads, kv_heads, dh, window):
    """From 512 (sequence, kv head) pairs on a workgroup walks a sequence's pages in one run and writes the
    output itself: 64 sequences with lengths at and around page and chunk edges, one of them with a key that
    stands out early in a long sequence."""
    rng = np.random.default_rng(77)
    lens = [1, 32, 33, 256, 257, 512, 700, 5, 1025, 2048, 2049, 31] + [int(n) for n in rng.integers(1, 1500, 52)]
    assert ops.decode_attention_streams(len(lens), kv_heads, max(lens) + 300)

    def boost(qkv, k, kp, table):
        head = 3 * (heads // kv_heads)                                 # sequence 9, kv head 3: its first query head
        kf = f64(kp[table[9, 40 // 32].item(), 3, 40 % 32])
        qkv[9, head * dh:(head + 1) * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
    out, want = attention_case(ops, rng, lens, [1] * len(lens), heads, kv_heads, dh, torch.bfloat16, window=window,
                               boost=boost, kernel="decode")
    close(out, want, BF16_OUT, f"streaming decode attention, window {window}")


WIDE_LENS = [1, 32, 33, 256, 257, 512, 700, 5, 1025, 1200, 1199, 31, 64, 1024, 300, 97,
             2, 63, 65, 100, 129, 255, 258, 400, 511, 513, 640, 767, 769, 900, 1000, 1100]


@pytest.mark.parametrize("heads, kv_heads, dh, window", [(16, 8, 32, None), (16, 8, 32, 100), (32, 8, 128, None),
                                                         (16, 8, 128, 300), (8, 8, 64, None)])
def test_mfma_decode_attention_streams_short_sequences_with_eight_wavefronts(ops, heads, kv_heads, dh, window):
    """Thirty-two sequences of eight kv heads and up to 1,200 keys: a run for every compute unit and none a second, and
    no sequence longer than sixteen chunks, is walked in one run by workgroups of eight wavefronts; some of the
    sequences have fewer pages than wavefronts."""
    if ops.compute_units() != 256:
        pytest.skip("the rule is written for the machine's size")
    rng = np.random.default_rng(78)
    assert ops.decode_attention_runs(len(WIDE_LENS), kv_heads, max(WIDE_LENS) + 300) == 1
    assert ops.decode_attention_runs(len(WIDE_LENS) - 7, kv_heads, max(WIDE_LENS) + 300) == 0
    assert ops.decode_attention_runs(len(WIDE_LENS), kv_heads, 4097) == 0
    assert ops.decode_attention_runs(len(WIDE_LENS) + 1, kv_heads, max(WIDE_LENS) + 300) == 0

    def boost(qkv, k, kp, table):
        head = 3 * (heads // kv_heads)                                 # sequence 9, kv head 3: its first query head
        kf = f64(kp[table[9, 40 // 32].item(), 3, 40 % 32])
        qkv[9, head * dh:(head + 1) * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
    out, want = attention_case(ops, rng, WIDE_LENS, [1] * len(WIDE_LENS), heads, kv_heads, dh, torch.bfloat16,
                               window=window, boost=boost, kernel="decode")
    close(out, want, BF16_OUT, f"eight wavefronts a run, window {window}")


@pytest.mark.parametrize("heads, kv_heads, dh, window", [(16, 8, 32, None), (16, 8, 32, 40), (32, 8, 128, None),
                                                         (16, 8, 128, 40), (128, 8, 64, None)])
def test_fused_decode_attention_streams_short_sequences_with_eight_wavefronts(ops, heads, kv_heads, dh, window):
    """The same from the raw projection (two query heads a wavefront to norm where a kv head has sixteen)."""
    if ops.compute_units() != 256:
        pytest.skip("the rule is written for the machine's size")
    assert ops.decode_attention_runs(len(WIDE_LENS), kv_heads, max(WIDE_LENS) + 301) == 1
    fused_decode_case(ops, heads, kv_heads, dh, window, WIDE_LENS, steps=2 if dh == 32 else 1, repeats=2 if dh == 32 else 1)


@pytest.mark.parametrize("window", [None, 4500])
def test_mfma_decode_attention_streams_long_sequences_in_runs(ops, window):
    """Long sequences with 64 (sequence, kv head) pairs and more are cut into 16 runs of whole chunks each, by
    their own lengths, and the runs are joined in order: sequences of every size in one call (most of a short
    one's runs are empty), and in the longest a key that stands out in the first run and in a late one."""
    heads, kv_heads, dh = 8, 8, 32
    lens = [16400, 700, 1, 4097, 257, 33, 9000, 2048]
    assert ops.decode_attention_streams(len(lens), kv_heads, max(lens) + 300)
    for far in (3, 15000):
        rng = np.random.default_rng(41 + far)

        def boost(qkv, k, kp, table, far=far):
            kf = f64(kp[table[0, far // 32].item(), 5, far % 32])          # sequence 0, kv head 5 = query head 5
            qkv[0, 5 * dh:6 * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
        out, want = attention_case(ops, rng, lens, [1] * len(lens), heads, kv_heads, dh, torch.bfloat16,
                                   window=window, boost=boost, kernel="decode")
        close(out, want, BF16_OUT, f"far key {far}, window {window}")


def test_mfma_decode_attention_streams_one_very_long_sequence(ops):
    """Two sequences, one of 66,000 keys: 33 runs each, joined in eight groups side by side; the short
    sequence's runs are empty but the first.  A key that stands out in the first run, in a middle one, in the
    last."""
    heads, kv_heads, dh = 8, 8, 32
    lens = [66000, 300]
    assert ops.decode_attention_streams(len(lens), kv_heads, max(lens) + 300)
    for far in (100, 33000, 65990):
        rng = np.random.default_rng(51 + far)

        def boost(qkv, k, kp, table, far=far):
            kf = f64(kp[table[0, far // 32].item(), 2, far % 32])          # sequence 0, kv head 2 = query head 2
            qkv[0, 2 * dh:3 * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
        out, want = attention_case(ops, rng, lens, [1] * len(lens), heads, kv_heads, dh, torch.bfloat16, boost=boost,
                                   kernel="decode")
        close(out, want, BF16_OUT, f"far key {far}")
        assert np.abs(want[0, 2]).max() > 0


@pytest.mark.parametrize("kernel", ["prefill", "decode"])
def test_mfma_attention_finds_one_far_key(ops, kernel):
    rng = np.random.default_rng(19)
    heads, kv_heads, dh = 8, 2, 128
    for far in (0, 3, 4, 31, 32, 255, 256, 511, 640, 699):
        def boost(qkv, k, kp, table, far=far):
            kf = f64(kp[table[0, far // 32].item(), 1, far % 32])          # kv head 1: query heads 4..7
            qkv[0, 6 * dh:7 * dh] = 40.0 * kf / np.linalg.norm(kf) ** 2 * np.sqrt(dh)
        out, want = attention_case(ops, rng, [700], [1], heads, kv_heads, dh, torch.bfloat16, boost=boost,
                                   kernel=kernel)
        close(out, want, BF16_ONE_KEY, f"far key {far}")
        vfar = f64(out[0, 6])
        assert np.abs(vfar - want[0, 6]).max() < 0.05


@pytest.mark.parametrize("kernel", ["prefill", "decode"])
@pytest.mark.parametrize("window", [1, 32, 33, 100, 256, 300])
def test_mfma_attention_window_edges(ops, kernel, window):
    rng = np.random.default_rng(window + 5)
    new = [1, 1] if kernel == "decode" else [34, 40]
    out, want = attention_case(ops, rng, [290, 40], new, 4, 2, 64, torch.bfloat16, window=window, kernel=kernel)
    close(out, want, BF16_OUT, f"window {window}")


@pytest.mark.parametrize("heads, kv_heads, dh", MFMA_SHAPES)
@pytest.mark.parametrize("window", [None, 40])
def test_fused_decode_attention(ops, heads, kv_heads, dh, window):
    """Norm, rotation, cache write and attention from the raw projection, against the plain parts; twice in
    a row on the same buffers, then one token further."""
    fused_decode_case(ops, heads, kv_heads, dh, window, [1, 32, 33, 256, 257, 512, 700, 5])


@pytest.mark.parametrize("heads, kv_heads, dh, window", [(16, 8, 32, None), (16, 8, 32, 40), (32, 8, 128, None),
                                                         (32, 8, 128, 40), (16, 8, 64, None)])
def test_fused_decode_attention_streams_over_many_sequences(ops, heads, kv_heads, dh, window):
    """The same from 512 (sequence, kv head) pairs on, where a workgroup walks a sequence's pages in one run,
    and the one whose run ends at the new token stores its key and value before any page is read."""
    rng = np.random.default_rng(3)
    lens = [1, 32, 33, 256, 257, 512, 700, 5, 31, 64, 65, 1000] + [int(n) for n in rng.integers(1, 600, 52)]
    assert ops.decode_attention_streams(len(lens), kv_heads, max(lens) + 301)
    fused_decode_case(ops, heads, kv_heads, dh, window, lens, steps=2 if dh == 32 else 1, repeats=2 if dh == 32 else 1)


@pytest.mark.parametrize("heads, kv_heads, dh", [(8, 8, 32), (32, 8, 128)])
def test_fused_decode_attention_streams_long_sequences_in_runs(ops, heads, kv_heads, dh):
    """And with long sequences cut into 16 runs each: the last run that is not empty holds the new token."""
    lens = [16400, 700, 1, 4097, 257, 33, 8191, 8192]
    assert ops.decode_attention_streams(len(lens), kv_heads, max(lens) + 301)
    fused_decode_case(ops, heads, kv_heads, dh, None, lens, steps=1, repeats=1)


def fused_decode_case(ops, heads, kv_heads, dh, window, lens, steps=2, repeats=2):
    """`lens`: the sequences' lengths after the first step."""
    rng = np.random.default_rng(heads * 13 + dh)
    B = len(lens)
    k, v, kp, vp, table = paged(rng, [n + 1 for n in lens], kv_heads, dh, dtype=torch.bfloat16, spare=12)
    width = (heads + 2 * kv_heads) * dh
    qg, kg = t(1 + 0.2 * rng.normal(size=dh)), t(1 + 0.2 * rng.normal(size=dh))
    theta, eps = 50000.0, 1e-5
    inv_freq = t(P.rope_inv_freq(dh, theta))
    for step in range(steps):
        cur = [n + step for n in lens]
        pos = [n - 1 for n in cur]
        raw = t(rng.normal(size=(B, width)) * 2, torch.bfloat16)
        raw64 = f64(raw)
        for repeat in range(repeats):
            out = ops.attention_decode_fused_bf16(raw, qg, kg, eps, inv_freq, kp, vp, t(pos, torch.int32), table, B,
                                                  max(cur) + 300, heads, kv_heads, dh, window, 1.0 / np.sqrt(dh))
            assert torch.equal(raw, t(raw64, torch.bfloat16)), "the projection is read, not changed"
            q = raw64[:, :heads * dh].reshape(B, heads, dh)
            kn = raw64[:, heads * dh:(heads + kv_heads) * dh].reshape(B, kv_heads, dh)
            vn = raw64[:, (heads + kv_heads) * dh:].reshape(B, kv_heads, dh)
            ang = P.rope_angles(pos, dh, theta)
            q = P.bf16_round(P.apply_rope(P.rms_norm(q, f64(qg), eps), ang).astype(np.float32)).astype(np.float64)
            kn = P.apply_rope(P.rms_norm(kn, f64(kg), eps), ang)
            tab = table.cpu().numpy()
            for b in range(B):
                page, off = tab[b, pos[b] // 32], pos[b] % 32
                close(kp[page, :, off], kn[b], BF16_OUT, "the new key in its page")
                assert np.array_equal(f64(vp[page, :, :, off]), vn[b]), "the new value in its page"
                kb = np.stack([f64(kp[tab[b, p // 32], :, p % 32]) for p in range(cur[b])])
                vb = np.stack([f64(vp[tab[b, p // 32], :, :, p % 32]) for p in range(cur[b])])
                want = P.attention(q[b:b + 1], kb, vb, window=window)
                close(out[b].reshape(1, heads, dh), want, BF16_TWICE, f"sequence {b}, step {step}, repeat {repeat}")


def test_mfma_and_generic_attention_agree(ops):
    """The same call through all three kernels: decode against prefill against generic."""
    outs = []
    for kernel in ("generic", "prefill", "decode"):
        rng = np.random.default_rng(23)
        out, want = attention_case(ops, rng, [400, 77, 1], [1, 1, 1], 8, 2, 128, torch.bfloat16, kernel=kernel)
        outs.append(f64(out))
    assert np.abs(outs[0] - outs[1]).max() < 2e-2 and np.abs(outs[1] - outs[2]).max() < 2e-2


@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 9, 130])
def test_gemm_f32(ops, w_dtype, m):
    # sizes of the reference's own linear test (src/cpu/linear.rs:634-647): n = 37, k = 70
    rng = np.random.default_rng(m)
    x, w = t(rng.normal(size=(m, 70))), t(rng.normal(size=(37, 70)), w_dtype)
    close(ops.gemm_f32(x, w), f64(x) @ f64(w).T, 2e-6, "gemm_f32")


def test_gemm_f32_rows_do_not_depend_on_the_batch(ops):
    rng = np.random.default_rng(1)
    x, w = t(rng.normal(size=(100, 333))), t(rng.normal(size=(129, 333)))
    whole = ops.gemm_f32(x, w)
    assert torch.equal(whole[17:18], ops.gemm_f32(x[17:18].contiguous(), w))
    assert torch.equal(whole[60:], ops.gemm_f32(x[60:].contiguous(), w))


def test_gemm_f32_is_true_32_bit(ops):
    """Values that a reduced-precision matrix mode (tf32, bf16 inputs) would round away."""
    x = t([[1.0, 2.0 ** -12, 0.0, 0.0]]).repeat(1, 16)
    w = t([[1.0, 1.0, 0.0, 0.0]]).repeat(1, 16)
    assert ops.gemm_f32(x, w).item() == 16.0 * (1.0 + 2.0 ** -12)


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k", [584, 2560, 1544, 2048, 9728])      # steps of 512: one and a bit, five, three and a bit, four, nineteen
def test_gemv_bf16(ops, m, out_dtype, k):
    rng = np.random.default_rng(m)
    x, w = t(rng.normal(size=(m, k)), torch.bfloat16), t(rng.normal(size=(37, k)), torch.bfloat16)
    want = f64(x) @ f64(w).T
    close(ops.gemv_bf16(x, w, out_dtype), want, 2e-6 if out_dtype == torch.float32 else 5e-3, "gemv")
    wgu = t(rng.normal(size=(2 * 45, k)) * 0.1, torch.bfloat16)
    y = f64(x) @ f64(wgu).T
    close(ops.gemv_bf16(x, wgu, out_dtype, swiglu=True), P.silu(y[:, :45]) * y[:, 45:],
          3e-6 if out_dtype == torch.float32 else 5e-3, "gemv with swiglu")
    # a row's result does not depend on the other rows
    if m > 1:
        assert torch.equal(ops.gemv_bf16(x, w, out_dtype)[m - 1:], ops.gemv_bf16(x[m - 1:].contiguous(), w, out_dtype))


@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("n, k", [(37, 584), (100, 96), (4096, 4096), (50, 12288), (320, 104),
                                  (96, 2560), (48, 9728)])       # K whose share of a wavefront is no whole round of 8 steps
def test_gemm_skinny_packed_bf16(ops, m, n, k):
    rng = np.random.default_rng(m + n)
    x, w = t(rng.normal(size=(m, k)), torch.bfloat16), t(rng.normal(size=(n, k)), torch.bfloat16)
    want = f64(x) @ f64(w).T
    packed = ops.pack_for_mfma(w)
    close(ops.gemm_skinny_packed_bf16(x, packed, n, torch.float32), want, 3e-6, "packed skinny product")
    # a row's result does not depend on the other rows
    if m > 1:
        assert torch.equal(ops.gemm_skinny_packed_bf16(x, packed, n, torch.float32)[m - 1:],
                           ops.gemm_skinny_packed_bf16(x[m - 1:].contiguous(), packed, n, torch.float32))
    wgu = t(rng.normal(size=(2 * n, k)) * (4.0 / np.sqrt(k)), torch.bfloat16)
    y = f64(x) @ f64(wgu).T
    close(ops.gemm_skinny_packed_bf16(x, ops.pack_for_mfma(wgu, swiglu=True), n, torch.bfloat16, swiglu=True),
          P.silu(y[:, :n]) * y[:, n:], 5e-3, "packed, with swiglu")
    for parts in (2, 3):                                   # K cut in pieces: the pieces add up to the product
        got = ops.gemm_skinny_packed_bf16(x, packed, n, torch.float32, parts=parts)
        assert got.shape == (parts, m, n)
        close(got.sum(0), want, 3e-6, f"{parts} parts of K")


@pytest.mark.parametrize("m", [1, 16, 17, 33, 40, 49, 64])
@pytest.mark.parametrize("n, k", [(37, 72), (1000, 1024), (584, 12288), (4096, 4096), (70, 264)])
def test_wide_packed_product(ops, m, n, k):
    """The product for steps of 17 to 64 tokens: whole, in parts of K that add up, with the activation, from and
    into rows in the matrix cores' order; and a row's result does not depend on how many rows there are."""
    rng = np.random.default_rng(m + n + k)
    x, w = t(rng.normal(size=(m, k)), torch.bfloat16), t(rng.normal(size=(n, k)), torch.bfloat16)
    want = f64(x) @ f64(w).T
    packed = ops.pack_for_mfma(w)
    whole = ops.gemm_wide_packed_bf16(x, packed, n, torch.float32)
    close(whole, want, 3e-6, "wide product")
    close(ops.gemm_wide_packed_bf16(x, packed, n, torch.bfloat16), want, 5e-3, "wide product, bfloat16 out")
    for parts in (2, 3, ops.wide_product_plan(n, k, rows=m)[1]):
        got = ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, parts=parts)
        assert got.shape == ((parts, m, n) if parts > 1 else (m, n))
        if parts > 1:
            close(got.sum(0), want, 3e-6, f"{parts} parts of K")
            close(ops.sum_parts(got, torch.float32), want, 3e-6, "parts added by the kernel")
            assert torch.equal(ops.sum_parts(got, torch.bfloat16, tiled_out=True).rows(), ops.sum_parts(got, torch.bfloat16))
    wgu = t(rng.normal(size=(2 * n, k)) * (4.0 / np.sqrt(k)), torch.bfloat16)
    y = f64(x) @ f64(wgu).T
    pgu = ops.pack_for_mfma(wgu, swiglu=True)
    close(ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True), P.silu(y[:, :n]) * y[:, n:], 5e-3,
          "wide, with swiglu")
    raw = ops.gemm_wide_packed_bf16(x, pgu, n, torch.float32, swiglu=True, parts=2)        # the activation after the parts
    assert raw.shape == (2, m, 2 * n)
    close(ops.sum_parts(raw, torch.float32, swiglu=True), P.silu(y[:, :n]) * y[:, n:], 5e-6, "swiglu over parts")
    assert torch.equal(ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, depth=1), whole)    # the same sums either way
    # three row tiles a workgroup instead of four: the same sums again, whole, in parts and with the activation
    assert torch.equal(ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, waves=3), whole)
    assert torch.equal(ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, parts=3, waves=3, depth=1),
                       ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, parts=3))
    assert torch.equal(ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, waves=3, tiled_out=True).rows(),
                       ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True))
    # five to eight wavefronts a workgroup (matrices of more than a thousand pairs of row tiles): the same bits
    gated = ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, depth=1)
    for many in (5, 6, 7, 8):
        assert torch.equal(ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, depth=1, waves=many), gated)
    assert torch.equal(ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, depth=1, waves=7, tiled_out=True).rows(), gated)
    with pytest.raises(Exception, match="wavefronts"):
        ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, waves=5)
    waves, parts = ops.wide_product_plan(n, k, True)
    assert 3 <= waves <= 8 and parts == 1                   # the activation is never left to a second kernel
    assert ops.wide_product_plan(16 * 4 * ops.compute_units() + 16, k, True) == (5, 1)
    assert ops.wide_product_plan(16 * 7 * ops.compute_units(), k, True) == (7, 1)
    # rows in the matrix cores' order on either side: the same bits
    tiled = ops.sum_parts(x.float()[None].contiguous(), torch.bfloat16, tiled_out=True)
    assert torch.equal(tiled.rows(), x)
    assert torch.equal(ops.gemm_wide_packed_bf16(tiled, packed, n, torch.float32), whole)
    assert torch.equal(ops.gemm_wide_packed_bf16(x, packed, n, torch.bfloat16, tiled_out=True).rows(),
                       ops.gemm_wide_packed_bf16(x, packed, n, torch.bfloat16))
    if m > 1:
        assert torch.equal(whole[m - 1:], ops.gemm_wide_packed_bf16(x[m - 1:].contiguous(), packed, n, torch.float32))


@pytest.mark.parametrize("m", [65, 80, 81, 100, 113, 128, 129, 150, 200, 256])
@pytest.mark.parametrize("n, k", [(37, 72), (1000, 1024), (584, 12288), (4096, 4096), (70, 264), (16, 520)])
def test_wide_packed_product_of_65_to_256_rows(ops, m, n, k):
    """Five to eight tiles of x, two row tiles of the matrix a wavefront (an odd number of row tiles leaves the last
    wavefront one), past 128 rows in two passes (129 rows: five tiles and four): whole and in parts of K that add up,
    with three and four wavefronts a workgroup; a row's sums are those of the kernel for up to 64 rows, bit for bit."""
    rng = np.random.default_rng(m + n + k)
    x, w = t(rng.normal(size=(m, k)), torch.bfloat16), t(rng.normal(size=(n, k)), torch.bfloat16)
    want = f64(x) @ f64(w).T
    packed = ops.pack_for_mfma(w)
    whole = ops.gemm_wide_packed_bf16(x, packed, n, torch.float32)
    assert whole.shape == (m, n)
    close(whole, want, 3e-6, "wide product of more than 64 rows")
    waves, planned = ops.wide_product_plan(n, k, rows=m)
    assert waves in (3, 4) and planned >= 1
    for parts in (2, 3, planned):
        got = ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, parts=parts, waves=waves)
        assert got.shape == ((parts, m, n) if parts > 1 else (m, n))
        if parts > 1:
            close(got.sum(0), want, 3e-6, f"{parts} parts of K")
        assert torch.equal(got, ops.gemm_wide_packed_bf16(x, packed, n, torch.float32, parts=parts, waves=7 - waves))
        first = ops.gemm_wide_packed_bf16(x[:64].contiguous(), packed, n, torch.float32, parts=parts, depth=1)
        last = ops.gemm_wide_packed_bf16(x[m - 1:].contiguous(), packed, n, torch.float32, parts=parts, depth=1)
        assert torch.equal(got[..., :64, :], first) and torch.equal(got[..., m - 1:, :], last)
    if m <= 128:        # with the activation, five to eight wavefronts a workgroup: the bits of the kernel for 64 rows
        wgu = t(rng.normal(size=(2 * n, k)) * (4.0 / np.sqrt(k)), torch.bfloat16)
        y = f64(x) @ f64(wgu).T
        pgu = ops.pack_for_mfma(wgu, swiglu=True)
        gated = ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, waves=5)
        close(gated, P.silu(y[:, :n]) * y[:, n:], 5e-3, "more than 64 rows with the activation")
        for many in (6, 7, 8):
            assert torch.equal(ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, waves=many), gated)
        assert torch.equal(gated[:64], ops.gemm_wide_packed_bf16(x[:64].contiguous(), pgu, n, torch.bfloat16, swiglu=True, depth=1))
        with pytest.raises(Exception, match="wavefronts"):
            ops.gemm_wide_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True, waves=4)
    with pytest.raises(Exception, match="64"):
        ops.gemm_wide_packed_bf16(x, packed, n, torch.bfloat16)
    with pytest.raises(Exception, match="256"):
        ops.gemm_wide_packed_bf16(t(rng.normal(size=(257, k)), torch.bfloat16), packed, n, torch.float32)


@pytest.mark.parametrize("packed, m", [(False, 1), (False, 2), (False, 5), (True, 1), (True, 3), (True, 16)])
@pytest.mark.parametrize("hidden, k, inter", [(104, 72, 56), (4096, 4096, 1000), (584, 12288, 37)])
def test_products_linked_to_norms(ops, packed, m, hidden, k, inter):
    """A branch's last product adds into the residual stream and prepares the next RMSNorm; the
    product after it finishes that norm.  Checked against add, norm and products done one by one."""
    rng = np.random.default_rng(m + hidden)
    eps = 1e-5
    x = t(rng.normal(size=(m, k)), torch.bfloat16)
    w_out = t(rng.normal(size=(hidden, k)) / np.sqrt(k), torch.bfloat16)
    r0 = t(rng.normal(size=(m, hidden)) * 3)
    gain = t(1 + 0.3 * rng.normal(size=hidden))
    w_next = t(rng.normal(size=(inter, hidden)), torch.bfloat16)
    w_gu = t(rng.normal(size=(2 * inter, hidden)) * (4.0 / np.sqrt(hidden)), torch.bfloat16)
    prep = (lambda w, **kw: ops.pack_for_mfma(w, **kw)) if packed else (lambda w, **kw: w)

    r1 = f64(r0) + f64(x) @ f64(w_out).T
    residual = guarded(r0.clone())
    later = ops.linked_product(x, prep(w_out), hidden, packed, residual=residual, next_gain=gain, next_eps=eps)
    close(residual, r1, 3e-6, "residual after the linked product")
    close(later.xg, f64(residual) * f64(gain), 4e-3, "rows times gain")       # one rounding to bfloat16
    close(later.ssq.sum(1), (f64(residual) ** 2).sum(1), 1e-5, "sums of squares")
    assert later.dim == hidden and later.eps == eps
    # a second call leaves the same partial sums: they do not depend on scheduling
    again = ops.linked_product(x, prep(w_out), hidden, packed, residual=guarded(r0.clone()), next_gain=gain, next_eps=eps)
    assert torch.equal(again.ssq, later.ssq) and torch.equal(again.xg, later.xg)

    normed = P.rms_norm(f64(residual), f64(gain), eps)
    close(ops.linked_product(later, prep(w_next), inter, packed, torch.float32), normed @ f64(w_next).T, 6e-3,
          "product that finishes the norm")
    y = normed @ f64(w_gu).T
    close(ops.linked_product(later, prep(w_gu, swiglu=True) if packed else w_gu, inter, packed, torch.bfloat16,
                             swiglu=True), P.silu(y[:, :inter]) * y[:, inter:], BF16_TWICE, "the same with swiglu")
    # both sides at once: the next branch's product reads prepared rows and prepares the following norm
    w_back = t(rng.normal(size=(hidden, hidden)) / np.sqrt(hidden), torch.bfloat16)
    r2 = f64(residual) + normed @ f64(w_back).T
    chained = ops.linked_product(later, prep(w_back), hidden, packed, residual=residual, next_gain=gain, next_eps=eps)
    close(residual, r2, 6e-3, "residual after two linked products")
    close(chained.ssq.sum(1), (f64(residual) ** 2).sum(1), 1e-5, "sums of squares, second link")


@pytest.mark.parametrize("m", [1, 17, 32, 33, 41, 48, 50, 64])
@pytest.mark.parametrize("n, k", [(37, 72), (1000, 1024), (584, 12288)])
def test_packed_product_of_17_to_64_rows(ops, m, n, k):
    rng = np.random.default_rng(m + n)
    x = t(rng.normal(size=(m, k)), torch.bfloat16)
    w = t(rng.normal(size=(n, k)) / np.sqrt(k), torch.bfloat16)
    gu = t(rng.normal(size=(2 * n, k)) * (4.0 / np.sqrt(k)), torch.bfloat16)
    pw, pgu = ops.pack_for_mfma(w), ops.pack_for_mfma(gu, swiglu=True)
    out = ops.gemm_mid_packed_bf16(x, pw, n, torch.float32)
    close(out, f64(x) @ f64(w).T, 2e-5, "packed product, 17 to 64 rows")
    y = f64(x) @ f64(gu).T
    close(ops.gemm_mid_packed_bf16(x, pgu, n, torch.bfloat16, swiglu=True), P.silu(y[:, :n]) * y[:, n:], BF16_OUT,
          "the same with swiglu")
    # a row's result is the same whatever the number of rows, and the same as the kernel for up to 16 rows gives
    first = min(m, 16)
    assert torch.equal(out[:first], ops.gemm_skinny_packed_bf16(x[:first].contiguous(), pw, n, torch.float32))
    with pytest.raises(Exception, match="1 to 64"):
        ops.gemm_mid_packed_bf16(t(rng.normal(size=(65, k)), torch.bfloat16), pw, n)


@pytest.mark.parametrize("m", [1, 16, 17, 40, 64])
@pytest.mark.parametrize("dim, n", [(104, 56), (4096, 1000), (584, 40)])
def test_every_maker_of_rows_can_tile_them(ops, m, dim, n):
    """The norm, the decode attention and the product for 17 to 64 rows write their rows in the matrix cores'
    order on request, bit for bit the rows they write plainly; the products read them so."""
    rng = np.random.default_rng(5 * m + dim)
    residual = t(rng.normal(size=(m, dim)) * 2)
    pending = t(rng.normal(size=(m, dim)), torch.bfloat16)
    gain = t(1 + 0.2 * rng.normal(size=dim))
    plain = ops.add_rmsnorm(guarded(residual.clone()), pending, gain, 1e-5, torch.bfloat16)
    r2 = guarded(residual.clone())
    tiled = ops.add_rmsnorm(r2, pending, gain, 1e-5, torch.bfloat16, tiled=True)
    assert isinstance(tiled, ops.TiledRows) and tiled.shape == (m, dim) and torch.equal(tiled.rows(), plain)
    close(r2, f64(residual) + f64(pending), 1e-6, "the sum is written back either way")
    # into the products: the one for 17 to 64 rows takes fewer too
    pw = ops.pack_for_mfma(t(rng.normal(size=(n, dim)) / np.sqrt(dim), torch.bfloat16))
    pgu = ops.pack_for_mfma(t(rng.normal(size=(2 * n, dim)) * (4.0 / np.sqrt(dim)), torch.bfloat16), swiglu=True)
    want = ops.gemm_mid_packed_bf16(plain, pw, n)
    assert torch.equal(ops.gemm_mid_packed_bf16(tiled, pw, n), want)
    out_tiled = ops.gemm_mid_packed_bf16(tiled, pw, n, tiled_out=True)
    assert isinstance(out_tiled, ops.TiledRows) and torch.equal(out_tiled.rows(), want)
    assert torch.equal(ops.gemm_mid_packed_bf16(tiled, pgu, n, swiglu=True, tiled_out=True).rows(),
                       ops.gemm_mid_packed_bf16(plain, pgu, n, swiglu=True))
    if m <= 16:
        assert torch.equal(ops.gemm_skinny_packed_bf16(tiled, pw, n), want)
    with pytest.raises(Exception, match="64"):
        ops.add_rmsnorm(t(rng.normal(size=(65, dim))), None, gain, 1e-5, torch.bfloat16, tiled=True)


def test_streaming_attention_walks_a_run_of_more_pages_than_it_holds_table_entries_for(ops):
    """A wavefront of the streaming kernel fetches the page table's entries for 256 of its pages at a time; a run
    of more than 1,024 pages (32,768 keys) goes round that loop again.  64 sequences of one kv head each side of
    that length, eight kv heads (512 runs: one a sequence and kv head), against the generic kernel on the same
    pages; the sequences are of unequal length and one key far back in one of them gets a score that stands out."""
    heads, kv_heads, dh, B = 8, 8, 32, 64
    gen = torch.Generator(device=DEV).manual_seed(3)
    lens = [33_000 + 37 * b for b in range(B)]
    lens[5] = 40_000
    pages_per = [-(-n // 32) for n in lens]
    width = max(pages_per)
    num_pages = sum(pages_per)
    assert ops.decode_attention_runs(B, kv_heads, max(lens)) == 1
    kp = torch.randn((num_pages, kv_heads, 32, dh), device=DEV, generator=gen).to(torch.bfloat16)
    vp = torch.randn((num_pages, kv_heads, dh, 32), device=DEV, generator=gen).to(torch.bfloat16)
    order = torch.randperm(num_pages, device=DEV, generator=gen).to(torch.int32)
    table = torch.zeros((B, width), dtype=torch.int32, device=DEV)
    at = 0
    for b, n in enumerate(pages_per):
        table[b, :n] = order[at:at + n]
        at += n
    qkv = torch.randn((B, (heads + 2 * kv_heads) * dh), device=DEV, generator=gen).to(torch.bfloat16)
    # Queries that are a multiple of one far key, so that the output is that key's value: a key among a
    # wavefront's first 256 pages (position 9,000 of sequence 5) and keys among its later ones (pages from 1,024
    # on: position 39,990 of sequence 5, a key of sequence 9's last pages and one of sequence 20's page 1,024)
    for b, far, head in ((5, 9_000, 2), (5, 39_990, 3), (9, lens[9] - 100, 1), (20, 32_768 + 10, 4)):
        key = kp[table[b, far // 32].item(), head, far % 32].float()
        qkv[b, head * dh:(head + 1) * dh] = (8.0 * key / key.norm() * dh ** 0.25).to(torch.bfloat16)
    pos = t([n - 1 for n in lens], torch.int32)
    cu = t(np.arange(B + 1), torch.int32)
    seq = t(np.arange(B), torch.int32)
    got = ops.attention_decode_bf16(qkv, kp, vp, cu, pos, table, B, max(lens), heads, kv_heads, dh, None, dh ** -0.5)
    want = ops.attention(qkv, kp, vp, pos, seq, table, heads, kv_heads, dh, None, dh ** -0.5)
    close(got, f64(want), BF16_OUT, "a run of more than 1,024 pages")
    for b, head in ((5, 2), (5, 3), (9, 1), (20, 4)):       # and these rows are not drowned by the others' size
        row = slice(head * dh, (head + 1) * dh)
        assert want[b, row].float().abs().max() > 0.5
        close(got[b, row], f64(want[b, row]), BF16_OUT, f"sequence {b}, head {head}")


@pytest.mark.parametrize("fused", [False, True])
def test_decode_attention_writes_tiled_rows(ops, fused):
    rng = np.random.default_rng(77)
    heads, kv_heads, dh = 8, 2, 64
    lens = [int(x) for x in rng.integers(1, 600, size=20)]
    B = len(lens)
    k, v, kp, vp, table = paged(rng, [n + 1 for n in lens], kv_heads, dh, dtype=torch.bfloat16, spare=12)
    pos = t([n - 1 for n in lens], torch.int32)
    outs = []
    for tiles in (False, True):
        if fused:
            raw = t(np.random.default_rng(78).normal(size=(B, (heads + 2 * kv_heads) * dh)) * 2, torch.bfloat16)
            gains = t(np.ones(dh))
            out = ops.attention_decode_fused_bf16(raw, gains, gains, 1e-5, t(P.rope_inv_freq(dh, 1e4)), kp, vp, pos, table,
                                                  B, max(lens) + 50, heads, kv_heads, dh, None, dh ** -0.5, tiled_out=tiles)
        else:
            qkv = t(np.random.default_rng(79).normal(size=(B, (heads + 2 * kv_heads) * dh)), torch.bfloat16)
            cu = t(np.arange(B + 1), torch.int32)
            out = ops.attention_decode_bf16(qkv, kp, vp, cu, pos, table, B, max(lens) + 50, heads, kv_heads, dh, None,
                                            dh ** -0.5, tiled_out=tiles)
        assert isinstance(out, ops.TiledRows) == tiles
        outs.append(ops.as_rows(out))
    assert torch.equal(outs[0], outs[1]) and outs[0].shape == (B, heads * dh)


@pytest.mark.parametrize("m", [1, 3, 8, 13, 16])
@pytest.mark.parametrize("hidden, k, inter", [(104, 72, 56), (4096, 4096, 1000), (584, 12288, 40)])
def test_rows_in_the_matrix_cores_order(ops, m, hidden, k, inter):
    """A packed product can leave its result in the order the next packed product loads as an operand, and take
    its input in it: every such chain gives, bit for bit, what the same chain gives through plain rows."""
    rng = np.random.default_rng(3 * m + hidden)
    eps = 1e-5
    x = t(rng.normal(size=(m, k)), torch.bfloat16)
    pw_a = ops.pack_for_mfma(t(rng.normal(size=(hidden, k)) / np.sqrt(k), torch.bfloat16))
    pw_gu = ops.pack_for_mfma(t(rng.normal(size=(2 * inter, hidden)) * (4.0 / np.sqrt(hidden)), torch.bfloat16), swiglu=True)
    pw_b = ops.pack_for_mfma(t(rng.normal(size=(hidden, inter)) / np.sqrt(inter), torch.bfloat16))
    gain = t(1 + 0.3 * rng.normal(size=hidden))
    r0 = t(rng.normal(size=(m, hidden)) * 3)

    # the layout itself: rows() undoes it
    plain = ops.gemm_skinny_packed_bf16(x, pw_a, hidden)
    tiled = ops.gemm_skinny_packed_bf16(x, pw_a, hidden, tiled_out=True)
    assert isinstance(tiled, ops.TiledRows) and tiled.shape == (m, hidden)
    assert torch.equal(tiled.rows(), plain)
    # read back as an operand: with the activation, plain, and with K cut into parts
    pw_c = ops.pack_for_mfma(t(rng.normal(size=(inter, hidden)) / np.sqrt(hidden), torch.bfloat16))
    assert torch.equal(ops.gemm_skinny_packed_bf16(tiled, pw_gu, inter, torch.bfloat16, swiglu=True),
                       ops.gemm_skinny_packed_bf16(plain, pw_gu, inter, torch.bfloat16, swiglu=True))
    assert torch.equal(ops.gemm_skinny_packed_bf16(tiled, pw_c, inter), ops.gemm_skinny_packed_bf16(plain, pw_c, inter))
    assert torch.equal(ops.gemm_skinny_packed_bf16(tiled, pw_c, inter, torch.float32, parts=2),
                       ops.gemm_skinny_packed_bf16(plain, pw_c, inter, torch.float32, parts=2))
    # a layer's chain of links: norm left to the products, rows handed on in either layout
    outs = []
    for tiles in (False, True):
        residual = guarded(r0.clone())
        later = ops.linked_product(x, pw_a, hidden, True, residual=residual, next_gain=gain, next_eps=eps,
                                   tiled_out=tiles)
        assert isinstance(later.xg, ops.TiledRows) == tiles
        act = ops.linked_product(later, pw_gu, inter, True, torch.bfloat16, swiglu=True, tiled_out=tiles)
        later2 = ops.linked_product(act, pw_b, hidden, True, residual=residual, next_gain=gain, next_eps=eps,
                                    tiled_out=tiles)
        outs.append((residual, ops.as_rows(later.xg), ops.as_rows(act), ops.as_rows(later2.xg), later.ssq, later2.ssq))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    with pytest.raises(Exception, match="tiled"):
        ops.gemm_skinny_packed_bf16(x, pw_a, hidden, torch.float32, tiled_out=True)


@pytest.mark.parametrize("dtype, rel", [(torch.float32, 1e-6), (torch.bfloat16, 5e-3)])
def test_swiglu(ops, dtype, rel):
    assert f64(ops.swiglu(t([[0.0, 2.0, 3.0, 3.0]])))[0, 0] == 0.0                 # src/ops/elementwise.rs:59-70
    close(ops.swiglu(t([[0.0, 2.0, 3.0, 3.0]])), [[0.0, 6.0 / (1.0 + np.exp(-2.0))]], 1e-6)
    rng = np.random.default_rng(3)
    for inter in (333, 232, 1000):                 # odd, and multiples of 8 (the 16-byte form)
        y = t(rng.normal(size=(5, 2 * inter)) * 3, dtype)
        close(ops.swiglu(y), P.silu(f64(y)[:, :inter]) * f64(y)[:, inter:], rel, f"swiglu, {inter}")
        tiled = ops.swiglu(y, tiled_out=True)      # the matrix cores' order where the kernel can (16-byte form, bfloat16)
        if dtype == torch.bfloat16 and inter % 8 == 0:
            assert isinstance(tiled, ops.TiledRows) and torch.equal(tiled.rows(), ops.swiglu(y))
        else:
            assert torch.equal(tiled, ops.swiglu(y))


def test_argmax(ops):
    assert ops.argmax(t([[1.0, 3.0, 3.0], [-1.0, 0.0, -5.0]])).tolist() == [1, 1]   # src/ops/reduce.rs:75-78
    rng = np.random.default_rng(4)
    x = rng.normal(size=(5, 151937)).astype(np.float32)
    x[1, 70000] = x[1, 150000] = 9.0            # equal maxima far apart: the lower index wins
    x[2, 151936] = 10.0                         # the last element
    x[3, 0] = 10.0
    x[4, :] = -np.inf
    assert ops.argmax(t(x)).tolist() == [int(np.argmax(x[0])), 70000, 151936, 0, 0]


def test_kernels_refuse_what_they_cannot_do(ops):
    from rust_inference_amd.errors import KernelError, ShapeError
    if not EMULATED:
        with pytest.raises(KernelError, match="GPU only"):
            ops.swiglu(torch.zeros(2, 4))
    with pytest.raises(KernelError, match="1 to 8"):
        ops.gemv_bf16(torch.zeros(9, 16, dtype=torch.bfloat16, device=DEV), torch.zeros(4, 16, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="between 1 and 512"):
        ops.attention(torch.zeros(1, 3 * 520, device=DEV), torch.zeros(1, 1, 32, 520, device=DEV),
                      torch.zeros(1, 1, 520, 32, device=DEV), t([0], torch.int32), t([0], torch.int32),
                      t([[0]], torch.int32), 1, 1, 520, None, 1.0)
    with pytest.raises(ShapeError, match="contiguous"):
        ops.swiglu(torch.zeros(4, 8, device=DEV)[:, ::2])


def test_kernels_agree_with_their_plain_cpp_twins(ops):
    """Each kernel family beside its scalar C++ twin (csrc/plain), float32: norm with the add, q/k norm and rotation,
    attention over pages, the product, the activation, argmax."""
    from rust_inference_amd.kernels import plain as N
    rng = np.random.default_rng(21)
    res, pend, gain = rng.normal(size=(5, 104)), rng.normal(size=(5, 104)), 1 + 0.1 * rng.normal(size=104)
    r_t = t(res)
    out = ops.add_rmsnorm(r_t, t(pend), t(gain), 1e-5, torch.float32)
    total, want = N.add_rms_norm(res, pend, gain, 1e-5)
    assert np.array_equal(r_t.cpu().numpy(), total)
    close(out, want, 1e-6, "add + norm")
    x, w = rng.normal(size=(7, 200)), rng.normal(size=(33, 200))
    close(ops.gemm_f32(t(x), t(w)), N.linear(x, w), 2e-6, "product")
    y = rng.normal(size=(4, 2 * 40)) * 3
    close(ops.swiglu(t(y)), N.swiglu(y), 1e-6, "swiglu")
    logits = rng.normal(size=(3, 1000)).astype(np.float32)
    logits[1, 5] = logits[1, 700] = 9.0
    assert ops.argmax(t(logits)).tolist() == [N.argmax(r) for r in logits]
    heads, kv_heads, dh, lens = 6, 2, 24, [40, 70]
    _, _, kp, vp, table = paged(rng, lens, kv_heads, dh)
    kp.zero_(); vp.zero_()
    tokens = sum(lens)
    qkv = rng.normal(size=(tokens, (heads + 2 * kv_heads) * dh))
    tok_seq = [b for b, n in enumerate(lens) for _ in range(n)]
    tok_pos = [i for n in lens for i in range(n)]
    qg, kg = 1 + 0.2 * rng.normal(size=dh), 1 + 0.2 * rng.normal(size=dh)
    inv = N.rope_inv_freq(dh, 1e4)
    qkv_t = t(qkv)
    ops.qk_norm_rope_kv_write(qkv_t, t(qg), t(kg), 1e-6, t(inv), t(tok_pos, torch.int32), t(tok_seq, torch.int32),
                              table, kp, vp, heads, kv_heads, dh)
    q = qkv.astype(np.float32)[:, :heads * dh].reshape(tokens, heads, dh)
    q_want = N.rope(N.rms_norm(q, qg, 1e-6), tok_pos, inv)
    close(qkv_t[:, :heads * dh].reshape(tokens, heads, dh), q_want, 3e-6, "q norm and rotation")
    got = ops.attention(qkv_t, kp, vp, t(tok_pos, torch.int32), t(tok_seq, torch.int32), table, heads, kv_heads, dh, None,
                        1 / np.sqrt(dh))
    want = N.attention(qkv_t.cpu().numpy()[:, :heads * dh].reshape(tokens, heads, dh), kp.cpu().numpy(), vp.cpu().numpy(),
                       tok_pos, tok_seq, table.cpu().numpy(), None, 1 / np.sqrt(dh))
    close(got.reshape(tokens, heads, dh), want, 3e-6, "attention over the pages the kernel wrote")
