"""Each part alone against its plain counterpart, and the parts' generality: a toy architecture,
registered here and nowhere in the package, with a windowed attention layer that runs twice (its
weights shared, a cache entry per run), a toy mixer that keeps a state of its own per sequence, and
no position encoding in one layer, a position encoding of another kind (a learned table added to q and
k) and a feed-forward that routes every token to two of four experts in another; built and stepped
through the unchanged engine."""
import os
from dataclasses import dataclass
from typing import ClassVar

import numpy as np
import pytest
import torch

import trace_plans as plans
from helpers import assert_logits_close, rel_to_max
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def t(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def f64(x):
    return x.detach().to("cpu", torch.float64).numpy()


class _StubModel:
    """Just enough of a model for the engine to lay out a step for a part on its own."""
    def __init__(self, rt, vocab=1000):
        self.rt = rt
        self.spec = type("S", (), {"vocab_size": vocab})()


def context_for(rt, needs, counts, starts=None):
    from rust_inference_amd.cache import Cache
    from rust_inference_amd.engine import Engine, StepEntry
    cache = Cache(needs, num_slots=len(counts), max_tokens=4096, max_seq_len=1024, dtype=rt.dtype, device=rt.device)
    eng = Engine(_StubModel(rt), cache)
    slots = [cache.acquire() for _ in counts]
    if starts:                                   # pretend earlier steps: only the lengths matter to a test that
        for s, n in zip(slots, starts):          # writes the earlier keys itself
            if n:
                cache.reserve([s], [n]); cache.commit([s], [n])
    ctx = eng.build_context([StepEntry(s, [1] * n, "all") for s, n in zip(slots, counts)])
    return cache, ctx


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(dtype):
    from rust_inference_amd.parts import PartSpec, Runtime, build_part
    rng = np.random.default_rng(0)
    rt = Runtime(DEV, dtype)
    norm = build_part("norm", PartSpec("rmsnorm", {"dim": 104, "eps": 3e-6, "name": "n.weight"}))
    assert list(norm.tensors()) == ["n.weight"] and norm.tensors()["n.weight"].shape == (104,)
    gain = torch.tensor(1 + 0.1 * rng.normal(size=104)).to(torch.bfloat16)
    norm.bind({"n.weight": gain}, rt)
    res, pend = t(rng.normal(size=(5, 104))), t(rng.normal(size=(5, 104)), dtype)
    want = P.rms_norm(f64(res) + f64(pend), f64(gain), float(np.float32(3e-6)))
    out = norm.apply(res, pend, dtype)
    assert rel_to_max(f64(out), want) < (2e-6 if dtype == torch.float32 else 5e-3)


def test_rotate_half_part_table():
    from rust_inference_amd.parts import PartSpec, Runtime, build_part
    for dh, theta in ((16, 10000.0), (48, 50000.0), (128, 1e6)):
        pos = build_part("position", PartSpec("rotate_half", {"head_dim": dh, "theta": theta}))
        pos.bind({}, Runtime(DEV, torch.float32))
        got, want = pos.rotation_table().cpu().numpy(), P.rope_inv_freq(dh, theta)
        assert got.dtype == np.float32 and np.allclose(got, want, rtol=2e-7, atol=0)


@pytest.mark.parametrize("dtype, bound", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("heads, kv_heads, dh, window", [(6, 2, 48, None), (8, 2, 32, None), (4, 4, 64, 20), (4, 1, 128, None)])
def test_attention_part(dtype, bound, heads, kv_heads, dh, window):
    from rust_inference_amd.parts import PartSpec, Runtime, build_part
    rng = np.random.default_rng(heads + dh)
    rt, hidden, eps, theta = Runtime(DEV, dtype), 72, 1e-5, 30000.0
    mixer = build_part("mixer", PartSpec("attention", {
        "hidden": hidden, "heads": heads, "kv_heads": kv_heads, "head_dim": dh, "prefix": "a.", "qk_norm": True,
        "eps": eps, "window": window, "position": PartSpec("rotate_half", {"head_dim": dh, "theta": theta})}))
    w = {}
    for name, spec in mixer.tensors().items():
        std = 0.1 if spec.kind == "matrix" else 0.0
        base = 1.0 if spec.kind == "gain" else 0.0
        w[name] = torch.tensor(base + (std or 0.1) * rng.normal(size=spec.shape)).to(torch.bfloat16)
    mixer.bind(w, rt)
    counts = [37, 3, 70]                         # three sequences from their first token, unequal lengths
    cache, ctx = context_for(rt, [mixer.cache_need()], counts)
    x = t(rng.normal(size=(sum(counts), hidden)), dtype)
    out = mixer.forward(x, ctx, cache.kv(0), ctx.page_tables[0])
    w64 = {k: v.to(torch.float64).numpy() for k, v in w.items()}
    cfg = {"num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": dh, "rms_norm_eps": eps,
           "rope_theta": theta}
    i = 0
    for n in counts:
        want = P.attention_block(f64(x[i:i + n]), w64, "a.", cfg, np.arange(n), window=window)
        assert rel_to_max(f64(out[i:i + n]), want) < bound
        i += n


@pytest.mark.parametrize("dtype, bound", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("rows", [1, 7, 40])
def test_swiglu_part(dtype, bound, rows):
    from rust_inference_amd.parts import PartSpec, Runtime, build_part
    rng = np.random.default_rng(rows)
    ff = build_part("feed_forward", PartSpec("swiglu", {"hidden": 104, "inter": 232, "prefix": "m."}))
    w = {n: torch.tensor(0.1 * rng.normal(size=s.shape)).to(torch.bfloat16) for n, s in ff.tensors().items()}
    ff.bind(w, Runtime(DEV, dtype))
    x = t(rng.normal(size=(rows, 104)), dtype)
    w64 = {k: v.to(torch.float64).numpy() for k, v in w.items()}
    want = P.swiglu_mlp(f64(x), w64["m.gate_proj.weight"], w64["m.up_proj.weight"], w64["m.down_proj.weight"])
    assert rel_to_max(f64(ff.forward(x, None)), want) < bound


@pytest.mark.parametrize("rows", [1, 2, 5, 16, 17])
def test_prenorm_block_leaves_norms_to_the_products(rows):
    """Small bfloat16 steps: the branch's last product adds into the stream and prepares the next norm.
    The block must give the plain block's stream whether the link is taken (up to 16 rows), not offered
    (17 rows), or its preparation is for a norm that turns out not to read the stream next."""
    from rust_inference_amd.kernels.ops import NormedLater
    from rust_inference_amd.parts import PartSpec, Runtime, build_part
    from rust_inference_amd.parts.block import ResidualStream
    rng = np.random.default_rng(rows)
    rt, hidden, inter, eps = Runtime(DEV, torch.bfloat16), 104, 232, 1e-5
    ff = build_part("feed_forward", PartSpec("swiglu", {"hidden": hidden, "inter": inter, "prefix": "m."}))
    w = {n: torch.tensor(0.1 * rng.normal(size=s.shape)).to(torch.bfloat16) for n, s in ff.tensors().items()}
    norms = []
    for name in ("a", "b", "c"):
        norm = build_part("norm", PartSpec("rmsnorm", {"dim": hidden, "eps": eps, "name": name}))
        w[name] = torch.tensor(1 + 0.2 * rng.normal(size=hidden)).to(torch.bfloat16)
        norm.bind(w, rt)
        norms.append(norm)
    ff.bind(w, rt)
    w64 = {k: v.to(torch.float64).numpy() for k, v in w.items()}
    h0 = rng.normal(size=(rows, hidden))

    def plain_branch(h, gain):
        return h + P.swiglu_mlp(P.rms_norm(h, w64[gain], eps), w64["m.gate_proj.weight"], w64["m.up_proj.weight"],
                                w64["m.down_proj.weight"])

    # two feed-forward branches in a row, the first told that norm b reads the stream next
    stream = ResidualStream(t(h0))
    link = stream.link(norms[1], torch.bfloat16)
    assert (link is not None) == (rows <= 16)
    stream.push(ff.forward(stream.normed(norms[0], torch.bfloat16), None, link=link))
    h1 = plain_branch(h0, "a")
    if rows <= 16:                                # the down product of such steps takes the link (a small matrix:
        assert stream.later is not None and stream.pending is None      # it has a packed copy for 2 to 16 rows)
        assert rel_to_max(f64(stream.sum), h1) < 5e-3
    assert stream.link(norms[2], torch.bfloat16) is None          # something waits: no second offer
    x = stream.normed(norms[1], torch.bfloat16, later_ok=True)
    assert isinstance(x, NormedLater) == (rows <= 16)
    stream.push(ff.forward(x, None))
    stream.flush()
    assert rel_to_max(f64(stream.sum), plain_branch(h1, "b")) < 2e-2

    # prepared for b, read by c: the preparation is dropped and c norms the complete sum itself
    stream = ResidualStream(t(h0))
    stream.push(ff.forward(stream.normed(norms[0], torch.bfloat16), None, link=stream.link(norms[1], torch.bfloat16)))
    x = stream.normed(norms[2], torch.bfloat16, later_ok=True)
    assert not isinstance(x, NormedLater)
    assert rel_to_max(f64(x), P.rms_norm(h1, w64["c"], eps)) < 1e-2
    # and a reader of single rows (the output head's norm) gets plain rows too
    stream = ResidualStream(t(h0))
    stream.push(ff.forward(stream.normed(norms[0], torch.bfloat16), None, link=stream.link(norms[1], torch.bfloat16)))
    rows_wanted = torch.tensor([rows - 1], dtype=torch.int32, device=DEV)
    x = stream.normed(norms[1], torch.bfloat16, rows=rows_wanted, later_ok=True)
    assert rel_to_max(f64(x), P.rms_norm(h1[-1:], w64["b"], eps)) < 1e-2


def test_tiled_rows_reach_every_kind_of_product():
    """Rows in the matrix cores' order may meet a product that has no packed kernel for them (a matrix
    without a packed copy, the one-row kernel, the library): it gets plain rows and gives the same result."""
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.parts.runtime import PackedWeight, Runtime
    rt = Runtime(DEV, torch.bfloat16)
    rng = np.random.default_rng(41)
    n, k = 96, 160
    w = t(rng.normal(size=(n, k)) / np.sqrt(k), torch.bfloat16)
    plain_w, packed_w = PackedWeight(w, None, False), PackedWeight(w, ops.pack_for_mfma(w), False)
    maker = ops.pack_for_mfma(t(np.eye(k), torch.bfloat16))            # x itself comes out of a product, tiled
    for m in (1, 2, 5, 16):
        x = t(rng.normal(size=(m, k)), torch.bfloat16)
        xt = ops.gemm_skinny_packed_bf16(x, maker, k, tiled_out=True)
        assert torch.equal(xt.rows(), x)
        want = f64(x) @ f64(w).T
        for pw in (plain_w, packed_w):
            assert rel_to_max(f64(rt.linear_packed(xt, pw)), want) < 1e-2
            assert torch.equal(rt.linear_packed(xt, pw), rt.linear_packed(x, pw))
        # a prepared norm whose rows are tiled, read by a product that cannot take them so
        gain = t(1 + 0.2 * rng.normal(size=k))
        residual = t(rng.normal(size=(m, k)))
        later = ops.linked_product(x, maker, k, True, residual=residual, next_gain=gain, next_eps=1e-5, tiled_out=True)
        assert isinstance(later.xg, ops.TiledRows)
        normed = P.rms_norm(f64(residual), f64(gain), 1e-5)
        assert rel_to_max(f64(rt.linear_packed(later, plain_w, out_dtype=torch.float32)), normed @ f64(w).T) < 1e-2
        assert rel_to_max(f64(rt.linear_packed(later, packed_w, out_dtype=torch.float32)), normed @ f64(w).T) < 1e-2
        assert rel_to_max(f64(rt.normed_now(later)), normed) < 1e-2


# ------------------------------------------------------------------------------------------------ the toy architecture
TOY = {"architectures": ["ToyMixForCausalLM"], "vocab_size": 130, "hidden_size": 48, "inter": 80, "heads": 4,
       "kv_heads": 2, "head_dim": 16, "window": 24, "eps": 1e-5, "theta": 10000.0, "experts": 4, "period": 37}


def register_toy():
    from rust_inference_amd.cache import StateNeed
    from rust_inference_amd.config import ModelConfig, register_architecture
    from rust_inference_amd.parts import (FeedForward, LayerSpec, Mixer, ModelSpec, PartSpec, PositionEncoding, Run,
                                          register_part)
    from rust_inference_amd.weights import MATRIX, TensorSpec

    @register_part("position", "toy_additive")
    class AdditivePosition(PositionEncoding):
        """q and k of the token at position p get row ``p % period`` of a learned table added, in
        every head: an encoding that does not rotate and has a tensor of its own."""
        def __init__(self, head_dim, period, name):
            self.head_dim, self.period, self.name = head_dim, period, name

        def tensors(self):
            return {self.name: TensorSpec((self.period, self.head_dim), MATRIX)}

        def bind(self, weights, rt):
            self.rt = rt
            self.table = weights[self.name].to(rt.device, torch.float32)

        def apply(self, qkv, ctx, heads, kv_heads, head_dim):
            add = self.table[ctx.tok_pos.long() % self.period]                     # [T, head_dim]
            qk = qkv[:, :(heads + kv_heads) * head_dim].unflatten(1, (heads + kv_heads, head_dim))
            qk.copy_((qk.float() + add[:, None, :]).to(qkv.dtype))                 # a view: in place, one rounding

    @register_part("feed_forward", "toy_top2")
    class Top2Experts(FeedForward):
        """Four square experts; a token goes to the two with the largest router probability and
        weights them by their lead over the third, ``p_e - p_(3)``: zero for every other expert, and
        continuous in x, so that rounding cannot flip a result.  Router logits and softmax in
        float32.  (Every expert sees every token here, masked: the toy keeps to shapes that do not
        depend on the data.)"""
        def __init__(self, hidden, experts, prefix):
            self.hidden, self.experts, self.prefix = hidden, experts, prefix

        def tensors(self):
            t = {self.prefix + "router.weight": TensorSpec((self.experts, self.hidden), MATRIX)}
            for e in range(self.experts):
                t[f"{self.prefix}experts.{e}.weight"] = TensorSpec((self.hidden, self.hidden), MATRIX)
            return t

        def bind(self, weights, rt):
            self.rt = rt
            self.router = weights[self.prefix + "router.weight"].to(rt.device, torch.float32)
            self.w = torch.stack([weights[f"{self.prefix}experts.{e}.weight"] for e in range(self.experts)]).to(
                rt.device, torch.float32)

        def forward(self, x, ctx):
            p = torch.softmax(x.float() @ self.router.T, dim=-1)                   # [T, E]
            third = torch.topk(p, 3, dim=-1).values[:, 2:3]
            weight = torch.clamp(p - third, min=0.0)                               # two experts at most are non-zero
            return torch.einsum("te,ehd,td->th", weight, self.w, x.float())       # float32: the stream takes it as it is

    @register_part("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """y_t = W . mean(x_0 .. x_t): the state is the running sum and the count, per sequence."""
        def __init__(self, hidden, name):
            self.hidden, self.name = hidden, name

        def tensors(self):
            return {self.name: TensorSpec((self.hidden, self.hidden), MATRIX)}

        def bind(self, weights, rt):
            self.rt = rt
            self.w = weights[self.name].to(rt.device, torch.float32)

        def cache_need(self):
            return StateNeed((self.hidden + 1,), torch.float32)

        def forward(self, x, ctx, store, page_table):
            if ctx.is_decode:       # one token a sequence: all on the device, so that the step can be captured as a graph
                rows = ctx.slots.long()
                state = store.index_select(0, rows)
                total, count = state[:, :-1] + x.float(), state[:, -1] + 1
                store.index_copy_(0, rows, torch.cat([total, count[:, None]], 1))
                return ((total / count[:, None]) @ self.w.T).to(x.dtype)
            out = torch.empty_like(x)
            begin = 0
            for slot, n in zip(ctx.slot_list, ctx.new_counts):        # a sequence's tokens are contiguous, in order
                xs = x[begin:begin + n].float()
                total = store[slot, :-1] + torch.cumsum(xs, 0)
                count = store[slot, -1] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                out[begin:begin + n] = ((total / count[:, None]) @ self.w.T).to(x.dtype)
                store[slot, :-1], store[slot, -1] = total[-1], count[-1]
                begin += n
            return out

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        inter: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        window: int = 0
        eps: float = 1e-5
        theta: float = 1e4
        experts: int = 0
        period: int = 0
        ARCHITECTURE: ClassVar[str] = "ToyMixForCausalLM"
        MODEL_TYPE: ClassVar[str] = "toy_mix"

        @classmethod
        def from_dict(cls, raw):
            import dataclasses
            return cls(**{f.name: raw[f.name] for f in dataclasses.fields(cls)})

    def spec(c):
        d = c.hidden_size

        def norm(name):
            return PartSpec("rmsnorm", {"dim": d, "eps": c.eps, "name": name})

        def ff(p):
            return PartSpec("swiglu", {"hidden": d, "inter": c.inter, "prefix": p})
        windowed = LayerSpec(
            mixer_norm=norm("l0.n1"), feed_forward_norm=norm("l0.n2"), feed_forward=ff("l0.ff."),
            mixer=PartSpec("attention", {"hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                         "prefix": "l0.attn.", "qk_norm": False, "eps": c.eps, "window": c.window,
                                         "position": PartSpec("rotate_half", {"head_dim": c.head_dim, "theta": c.theta})}))
        stateful = LayerSpec(mixer_norm=norm("l1.n1"), feed_forward_norm=norm("l1.n2"), feed_forward=ff("l1.ff."),
                             mixer=PartSpec("toy_running_mean", {"hidden": d, "name": "l1.mean.weight"}))
        unrotated = LayerSpec(
            mixer_norm=norm("l2.n1"), feed_forward_norm=norm("l2.n2"), feed_forward=ff("l2.ff."),
            mixer=PartSpec("attention", {"hidden": d, "heads": 2, "kv_heads": 1, "head_dim": 32, "prefix": "l2.attn.",
                                         "qk_norm": True, "eps": c.eps, "window": None, "position": PartSpec("none")}))
        routed = LayerSpec(
            mixer_norm=norm("l3.n1"), feed_forward_norm=norm("l3.n2"),
            feed_forward=PartSpec("toy_top2", {"hidden": d, "experts": c.experts, "prefix": "l3.moe."}),
            mixer=PartSpec("attention", {"hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                         "prefix": "l3.attn.", "qk_norm": False, "eps": c.eps, "window": None,
                                         "position": PartSpec("toy_additive", {"head_dim": c.head_dim, "period": c.period,
                                                                               "name": "l3.attn.position.weight"})}))
        return ModelSpec(
            architecture="ToyMixForCausalLM", vocab_size=c.vocab_size, hidden_size=d,
            embedding=PartSpec("table", {"vocab": c.vocab_size, "dim": d, "name": "embed.weight"}),
            layers=(windowed, stateful, unrotated, routed),
            # layer 0 runs twice with the same weights; each run has a cache entry of its own
            schedule=(Run(0, 0), Run(1, 1), Run(0, 2), Run(2, 3), Run(3, 4)),
            final_norm=norm("final.weight"),
            head=PartSpec("linear", {"vocab": c.vocab_size, "dim": d, "name": "head.weight", "tied": False}),
            max_positions=512)

    register_architecture("ToyMixForCausalLM", ToyConfig, spec, model_types=("toy_mix",))


def toy_plain(w, ids):
    """The toy model, whole sequence, no cache, from the plain parts."""
    c = TOY
    d = c["hidden_size"]
    h = P.embedding(w["embed.weight"], ids)
    pos = np.arange(len(ids))

    def block(h, p, mixer):
        r = h + mixer(P.rms_norm(h, w[p + ".n1"], c["eps"]))
        return r + P.swiglu_mlp(P.rms_norm(r, w[p + ".n2"], c["eps"]), w[p + ".ff.gate_proj.weight"],
                                w[p + ".ff.up_proj.weight"], w[p + ".ff.down_proj.weight"])

    def windowed(x):
        s = x.shape[0]
        q = (x @ w["l0.attn.q_proj.weight"].T).reshape(s, c["heads"], c["head_dim"])
        k = (x @ w["l0.attn.k_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        v = (x @ w["l0.attn.v_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        ang = P.rope_angles(pos, c["head_dim"], c["theta"])
        o = P.attention(P.apply_rope(q, ang), P.apply_rope(k, ang), v, window=c["window"])
        return o.reshape(s, -1) @ w["l0.attn.o_proj.weight"].T

    def running_mean(x):
        return (np.cumsum(x, 0) / np.arange(1, x.shape[0] + 1)[:, None]) @ w["l1.mean.weight"].T

    def unrotated(x):
        s = x.shape[0]
        q = P.rms_norm((x @ w["l2.attn.q_proj.weight"].T).reshape(s, 2, 32), w["l2.attn.q_norm.weight"], c["eps"])
        k = P.rms_norm((x @ w["l2.attn.k_proj.weight"].T).reshape(s, 1, 32), w["l2.attn.k_norm.weight"], c["eps"])
        v = (x @ w["l2.attn.v_proj.weight"].T).reshape(s, 1, 32)
        return P.attention(q, k, v).reshape(s, -1) @ w["l2.attn.o_proj.weight"].T

    def additive(x):
        s = x.shape[0]
        add = w["l3.attn.position.weight"][pos % c["period"]][:, None, :]
        q = (x @ w["l3.attn.q_proj.weight"].T).reshape(s, c["heads"], c["head_dim"]) + add
        k = (x @ w["l3.attn.k_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"]) + add
        v = (x @ w["l3.attn.v_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        return P.attention(q, k, v).reshape(s, -1) @ w["l3.attn.o_proj.weight"].T

    def top2(x):
        logits = x @ w["l3.moe.router.weight"].T
        p = np.exp(logits - logits.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        out = np.zeros_like(x)
        for t in range(x.shape[0]):                          # token by token: the two chosen experts only
            order = np.argsort(-p[t])
            for e in order[:2]:
                out[t] += (p[t, e] - p[t, order[2]]) * (w[f"l3.moe.experts.{e}.weight"] @ x[t])
        return out

    h = block(h, "l0", windowed)
    h = block(h, "l1", running_mean)
    h = block(h, "l0", windowed)
    h = block(h, "l2", unrotated)
    r = h + additive(P.rms_norm(h, w["l3.n1"], c["eps"]))
    h = r + top2(P.rms_norm(r, w["l3.n2"], c["eps"]))
    return P.rms_norm(h, w["final.weight"], c["eps"]) @ w["head.weight"].T


@pytest.fixture(scope="module")
def toy_dir(tmp_path_factory):
    register_toy()
    from rust_inference_amd.weights import write_random_model
    return write_random_model(str(tmp_path_factory.mktemp("toy") / "m"), TOY, seed=7, dtype=torch.float32,
                              matrix_std=0.12)     # the scale of the other test models


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_toy_architecture_builds_and_steps_through_the_unchanged_engine(toy_dir, dtype_name):
    from rust_inference_amd.cache import KVNeed, StateNeed
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from safetensors import safe_open
    model = load_model(toy_dir, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name])
    needs = model.cache_needs()
    assert needs[0] == needs[2] == KVNeed(2, 16, 24) and isinstance(needs[1], StateNeed) and needs[3] == KVNeed(1, 32, None)
    assert needs[4] == KVNeed(2, 16, None)
    with safe_open(os.path.join(toy_dir, "model.safetensors"), framework="pt") as f:
        w = {k: f.get_tensor(k).to(torch.float64).numpy() for k in f.keys()}
    rng = np.random.default_rng(8)
    reqs = {f"r{i}": [int(x) for x in rng.integers(0, TOY["vocab_size"], n)] for i, n in enumerate([70, 9, 41, 100])}
    results = {}
    for plan_name, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 32)),
                             ("batches", plans.unequal_batches([
                                 {k: (v, max(1, len(v) - 20)) for k, v in list(reqs.items())[:2]},
                                 {k: (v, max(1, len(v) - 33)) for k, v in list(reqs.items())[2:]}]))):
        engine = engine_for_trace(model, plans.max_live_tokens(steps))
        assert len(engine.cache.groups) == 3                     # the windowed entries and the two full kinds: own storage
        player, outs = Replayer(engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.cpu().numpy()
        engine.cache.check_consistent()
        results[plan_name] = plans.collect(steps, lambda i: outs[i], TOY["vocab_size"])
        for rid, toks in reqs.items():
            assert_logits_close(results[plan_name][rid], toy_plain(w, toks), dtype_name, f"toy, {plan_name}, {rid}")
    # a window's pages go back while a sequence is still running: fewer pages held than a full group would
    engine = engine_for_trace(model, 128)
    slot = engine.cache.acquire()
    from rust_inference_amd.engine import StepEntry
    engine.step([StepEntry(slot, reqs["r3"], "last")])
    windowed = next(g for g in engine.cache.groups if g.need.window)
    full = next(g for g in engine.cache.groups if not g.need.window)
    assert len(windowed.pool.pages_of(slot)) == 2 and len(full.pool.pages_of(slot)) == 4


def test_toy_model_decodes_the_same_through_graphs(toy_dir):
    """Decode steps captured as graphs: the mixer with state is rehearsed once before the capture, and its
    state must count that step once; sequences leave, so another batch size gets a graph of its own."""
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.parts import load_model
    model = load_model(toy_dir, torch.bfloat16)
    rng = np.random.default_rng(9)
    prompts = [[int(x) for x in rng.integers(0, TOY["vocab_size"], n)] for n in (40, 3, 17)]
    outs = []
    for graphs in (False, True):
        eng = Engine(model, model.new_cache(max_tokens=3 * 128, num_slots=3, max_seq_len=128), use_graphs=graphs)
        slots = [eng.cache.acquire() for _ in prompts]
        eng.step([StepEntry(s, p, "last") for s, p in zip(slots, prompts)])
        rows = []
        for step in range(14):
            live = slots if step < 8 else slots[1:]
            rows.append(eng.step([StepEntry(s, [(5 * step + s) % TOY["vocab_size"]], "last") for s in live]).clone())
        outs.append(rows)
    for a, b in zip(*outs):
        assert torch.equal(a, b)


# ------------------------------------------------------------------------------------------------ another arrangement
SIDE = {"architectures": ["ToySideBySideForCausalLM"], "vocab_size": 90, "hidden_size": 64, "inter": 112, "heads": 4,
        "kv_heads": 1, "head_dim": 32, "eps": 1e-6, "theta": 5000.0}


def register_side_by_side():
    """An arrangement of its own, registered from here: one norm feeds the mixer and the feed-forward side by
    side, ``h' = h + mixer(n(h)) + ff(n(h))``, so two branch outputs wait for the stream at once."""
    from rust_inference_amd.config import ModelConfig, register_architecture
    from rust_inference_amd.parts import LayerSpec, ModelSpec, PartSpec, Run, register_part
    from rust_inference_amd.parts.registry import build_part

    @register_part("arrangement", "toy_side_by_side")
    class SideBySide:
        def __init__(self, layer_spec):
            self.norm = build_part("norm", layer_spec.mixer_norm)
            self.mixer = build_part("mixer", layer_spec.mixer)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward)

        def parts(self):
            return (self.norm, self.mixer, self.feed_forward)

        def forward(self, stream, ctx, store, page_table, act_dtype):
            h = stream.normed(self.norm, act_dtype)
            stream.push(self.mixer.forward(h, ctx, store, page_table))
            stream.push(self.feed_forward.forward(h, ctx))

    @dataclass(frozen=True)
    class SideConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        inter: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        eps: float = 1e-6
        theta: float = 1e4
        ARCHITECTURE: ClassVar[str] = "ToySideBySideForCausalLM"
        MODEL_TYPE: ClassVar[str] = "toy_side_by_side"

        @classmethod
        def from_dict(cls, raw):
            import dataclasses
            return cls(**{f.name: raw[f.name] for f in dataclasses.fields(cls)})

    def spec(c):
        d = c.hidden_size

        def norm(name):
            return PartSpec("rmsnorm", {"dim": d, "eps": c.eps, "name": name})

        def layer(p, arrangement):
            return LayerSpec(
                arrangement=arrangement, mixer_norm=norm(p + "n1"), feed_forward_norm=norm(p + "n2"),
                feed_forward=PartSpec("swiglu", {"hidden": d, "inter": c.inter, "prefix": p + "ff."}),
                mixer=PartSpec("attention", {"hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                             "prefix": p + "attn.", "qk_norm": True, "eps": c.eps, "window": None,
                                             "position": PartSpec("rotate_half", {"head_dim": c.head_dim, "theta": c.theta})}))
        return ModelSpec(
            architecture="ToySideBySideForCausalLM", vocab_size=c.vocab_size, hidden_size=d,
            embedding=PartSpec("table", {"vocab": c.vocab_size, "dim": d, "name": "embed.weight"}),
            layers=(layer("l0.", "toy_side_by_side"), layer("l1.", "prenorm"), layer("l2.", "toy_side_by_side")),
            schedule=(Run(0, 0), Run(1, 1), Run(2, 2)),
            final_norm=norm("final.weight"),
            head=PartSpec("linear", {"vocab": c.vocab_size, "dim": d, "name": "head.weight", "tied": True}),
            max_positions=256)

    register_architecture("ToySideBySideForCausalLM", SideConfig, spec, model_types=("toy_side_by_side",))


def side_plain(w, ids):
    c = SIDE
    h = P.embedding(w["embed.weight"], ids)
    ang = P.rope_angles(np.arange(len(ids)), c["head_dim"], c["theta"])

    def attn(x, p):
        s = x.shape[0]
        q = P.rms_norm((x @ w[p + "attn.q_proj.weight"].T).reshape(s, c["heads"], c["head_dim"]),
                       w[p + "attn.q_norm.weight"], c["eps"])
        k = P.rms_norm((x @ w[p + "attn.k_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"]),
                       w[p + "attn.k_norm.weight"], c["eps"])
        v = (x @ w[p + "attn.v_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        return P.attention(P.apply_rope(q, ang), P.apply_rope(k, ang), v).reshape(s, -1) @ w[p + "attn.o_proj.weight"].T

    def ff(x, p):
        return P.swiglu_mlp(x, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])

    def side_by_side(h, p):
        x = P.rms_norm(h, w[p + "n1"], c["eps"])
        return h + attn(x, p) + ff(x, p)

    h = side_by_side(h, "l0.")
    r = h + attn(P.rms_norm(h, w["l1.n1"], c["eps"]), "l1.")
    h = r + ff(P.rms_norm(r, w["l1.n2"], c["eps"]), "l1.")
    h = side_by_side(h, "l2.")
    return P.rms_norm(h, w["final.weight"], c["eps"]) @ w["embed.weight"].T


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_an_arrangement_of_its_own(tmp_path, dtype_name):
    """Layers whose two branches read one norm and are added together, around a pre-norm layer: registered
    here, built by the unchanged model class, stepped whole, token by token and through graphs."""
    register_side_by_side()
    from rust_inference_amd.engine import Engine, StepEntry
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    from safetensors import safe_open
    folder = write_random_model(str(tmp_path / "m"), SIDE, seed=11, dtype=torch.float32, matrix_std=0.12)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        w = {k: f.get_tensor(k).to(torch.float64).numpy() for k in f.keys()}
    assert "l0.n2" not in w and "l1.n2" in w          # the arrangement says which tensors a layer has
    model = load_model(folder, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name])
    rng = np.random.default_rng(12)
    reqs = {f"r{i}": [int(x) for x in rng.integers(0, SIDE["vocab_size"], n)] for i, n in enumerate([50, 7, 33])}
    for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 20))):
        engine = engine_for_trace(model, plans.max_live_tokens(steps))
        player, outs = Replayer(engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.cpu().numpy()
        got = plans.collect(steps, lambda i: outs[i], SIDE["vocab_size"])
        for rid, toks in reqs.items():
            assert_logits_close(got[rid], side_plain(w, toks), dtype_name, f"side by side, {what}, {rid}")
    if dtype_name == "bfloat16":                       # decode steps as graphs give what eager steps give
        rows = []
        for graphs in (False, True):
            eng = Engine(model, model.new_cache(max_tokens=2 * 64, num_slots=2, max_seq_len=64), use_graphs=graphs)
            slots = [eng.cache.acquire() for _ in range(2)]
            eng.step([StepEntry(s, p[:9], "last") for s, p in zip(slots, reqs.values())])
            rows.append([eng.step([StepEntry(s, [(3 * i + s) % SIDE["vocab_size"]], "last") for s in slots]).clone()
                         for i in range(6)])
        for a, b in zip(*rows):
            assert torch.equal(a, b)


# ------------------------------------------------------------------------------------------------ a layer that reads another's cache
SHARED = {"architectures": ["ToySharedCacheForCausalLM"], "vocab_size": 77, "hidden_size": 40, "inter": 72, "heads": 4,
          "kv_heads": 2, "head_dim": 16, "eps": 1e-5, "theta": 10000.0}


def register_shared_cache():
    """Two layers on one cache entry: an attention layer writes keys and values, and a mixer defined here
    reads that entry's values after it and writes nothing."""
    from rust_inference_amd.cache import KVNeed
    from rust_inference_amd.config import ModelConfig, register_architecture
    from rust_inference_amd.parts import LayerSpec, Mixer, ModelSpec, PartSpec, Run, register_part
    from rust_inference_amd.weights import MATRIX, TensorSpec

    @register_part("mixer", "toy_value_mean")
    class ValueMean(Mixer):
        """y_t = W . mean(v_0 .. v_t), v_j the values of all kv heads at position j as they lie in the cache."""
        def __init__(self, hidden, kv_heads, head_dim, name):
            self.hidden, self.kv_heads, self.head_dim, self.name = hidden, kv_heads, head_dim, name

        def tensors(self):
            return {self.name: TensorSpec((self.hidden, self.kv_heads * self.head_dim), MATRIX)}

        def bind(self, weights, rt):
            self.w = weights[self.name].to(rt.device, torch.float32)

        def cache_need(self):
            return KVNeed(self.kv_heads, self.head_dim, None)          # the writer's need: one entry serves both

        def forward(self, x, ctx, store, page_table):
            out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            begin = 0
            for b, (start, n) in enumerate(zip(ctx.starts, ctx.new_counts)):
                length = start + n
                pages = page_table[b, :-(-length // store.page_size)].long()
                v = store.v_pages[pages]                                # [pages, kv heads, head_dim, page]
                v = v.permute(0, 3, 1, 2).reshape(-1, self.kv_heads * self.head_dim)[:length].float()
                count = torch.arange(start + 1, length + 1, device=x.device, dtype=torch.float32)
                out[begin:begin + n] = (torch.cumsum(v, 0)[start:] / count[:, None]) @ self.w.T
                begin += n
            return out

    @dataclass(frozen=True)
    class SharedConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        inter: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        eps: float = 1e-5
        theta: float = 1e4
        ARCHITECTURE: ClassVar[str] = "ToySharedCacheForCausalLM"
        MODEL_TYPE: ClassVar[str] = "toy_shared_cache"

        @classmethod
        def from_dict(cls, raw):
            import dataclasses
            return cls(**{f.name: raw[f.name] for f in dataclasses.fields(cls)})

    def spec(c):
        d = c.hidden_size

        def norm(name):
            return PartSpec("rmsnorm", {"dim": d, "eps": c.eps, "name": name})

        def ff(p):
            return PartSpec("swiglu", {"hidden": d, "inter": c.inter, "prefix": p})
        writer = LayerSpec(
            mixer_norm=norm("l0.n1"), feed_forward_norm=norm("l0.n2"), feed_forward=ff("l0.ff."),
            mixer=PartSpec("attention", {"hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                         "prefix": "l0.attn.", "qk_norm": False, "eps": c.eps, "window": None,
                                         "position": PartSpec("rotate_half", {"head_dim": c.head_dim, "theta": c.theta})}))
        reader = LayerSpec(
            mixer_norm=norm("l1.n1"), feed_forward_norm=norm("l1.n2"), feed_forward=ff("l1.ff."),
            mixer=PartSpec("toy_value_mean", {"hidden": d, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                              "name": "l1.mean.weight"}))
        return ModelSpec(
            architecture="ToySharedCacheForCausalLM", vocab_size=c.vocab_size, hidden_size=d,
            embedding=PartSpec("table", {"vocab": c.vocab_size, "dim": d, "name": "embed.weight"}),
            layers=(writer, reader), schedule=(Run(0, 0), Run(1, 0)),       # both runs name cache entry 0
            final_norm=norm("final.weight"),
            head=PartSpec("linear", {"vocab": c.vocab_size, "dim": d, "name": "head.weight", "tied": False}),
            max_positions=256)

    register_architecture("ToySharedCacheForCausalLM", SharedConfig, spec, model_types=("toy_shared_cache",))


def shared_plain(w, ids):
    c = SHARED
    s = len(ids)
    h = P.embedding(w["embed.weight"], ids)
    ang = P.rope_angles(np.arange(s), c["head_dim"], c["theta"])
    x = P.rms_norm(h, w["l0.n1"], c["eps"])
    q = (x @ w["l0.attn.q_proj.weight"].T).reshape(s, c["heads"], c["head_dim"])
    k = (x @ w["l0.attn.k_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
    v = (x @ w["l0.attn.v_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
    r = h + P.attention(P.apply_rope(q, ang), P.apply_rope(k, ang), v).reshape(s, -1) @ w["l0.attn.o_proj.weight"].T
    h = r + P.swiglu_mlp(P.rms_norm(r, w["l0.n2"], c["eps"]), w["l0.ff.gate_proj.weight"], w["l0.ff.up_proj.weight"],
                         w["l0.ff.down_proj.weight"])
    mean = np.cumsum(v.reshape(s, -1), 0) / np.arange(1, s + 1)[:, None]
    r = h + mean @ w["l1.mean.weight"].T                     # the reader ignores its own input: only the cache counts
    h = r + P.swiglu_mlp(P.rms_norm(r, w["l1.n2"], c["eps"]), w["l1.ff.gate_proj.weight"], w["l1.ff.up_proj.weight"],
                         w["l1.ff.down_proj.weight"])
    return P.rms_norm(h, w["final.weight"], c["eps"]) @ w["head.weight"].T


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_layer_reads_the_cache_another_layer_wrote(tmp_path, dtype_name):
    register_shared_cache()
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    from safetensors import safe_open
    folder = write_random_model(str(tmp_path / "m"), SHARED, seed=21, dtype=torch.float32, matrix_std=0.12)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        w = {k: f.get_tensor(k).to(torch.float64).numpy() for k in f.keys()}
    model = load_model(folder, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name])
    assert len(model.cache_needs()) == 1                      # two runs, one entry
    rng = np.random.default_rng(22)
    reqs = {f"r{i}": [int(x) for x in rng.integers(0, SHARED["vocab_size"], n)] for i, n in enumerate([45, 6, 70, 33])}
    for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 32)),
                        ("batches", plans.unequal_batches([
                            {k: (v, max(1, len(v) - 20)) for k, v in list(reqs.items())[:2]},
                            {k: (v, max(1, len(v) - 33)) for k, v in list(reqs.items())[2:]}]))):
        engine = engine_for_trace(model, plans.max_live_tokens(steps))
        assert len(engine.cache.groups) == 1 and engine.cache.groups[0].entries == [0]
        player, outs = Replayer(engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.cpu().numpy()
        engine.cache.check_consistent()
        got = plans.collect(steps, lambda i: outs[i], SHARED["vocab_size"])
        for rid, toks in reqs.items():
            assert_logits_close(got[rid], shared_plain(w, toks), dtype_name, f"shared cache, {what}, {rid}")


# ------------------------------------------------------------------------------------------------ another norm
CENTRED = {"architectures": ["ToyCentredNormForCausalLM"], "vocab_size": 61, "hidden_size": 56, "inter": 88, "heads": 2,
           "kv_heads": 2, "head_dim": 32, "eps": 1e-4, "theta": 20000.0}


def register_centred_norm():
    """A norm with a mean, a gain and a bias, registered from here and used at every norm of a model."""
    from rust_inference_amd.config import ModelConfig, register_architecture
    from rust_inference_amd.parts import LayerSpec, ModelSpec, Norm, PartSpec, Run, register_part
    from rust_inference_amd.weights import GAIN, TensorSpec

    @register_part("norm", "toy_centred")
    class CentredNorm(Norm):
        def __init__(self, dim, eps, name):
            self.dim, self.eps, self.name = dim, eps, name

        def tensors(self):
            return {self.name + ".weight": TensorSpec((self.dim,), GAIN), self.name + ".bias": TensorSpec((self.dim,), GAIN)}

        def bind(self, weights, rt):
            self.w = rt.place_gain(weights[self.name + ".weight"])
            self.b = rt.place_gain(weights[self.name + ".bias"])

        def apply(self, residual, pending, out_dtype, rows=None):
            total = residual if pending is None else residual + pending.float()
            if rows is None:
                if pending is not None:
                    residual.copy_(total)                    # the stream takes the sum
                x = residual
            else:
                x = total[rows.long()]
            x = x - x.mean(-1, keepdim=True)
            y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.w + self.b
            return y.to(out_dtype)

    @dataclass(frozen=True)
    class CentredConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        inter: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        eps: float = 1e-5
        theta: float = 1e4
        ARCHITECTURE: ClassVar[str] = "ToyCentredNormForCausalLM"
        MODEL_TYPE: ClassVar[str] = "toy_centred_norm"

        @classmethod
        def from_dict(cls, raw):
            import dataclasses
            return cls(**{f.name: raw[f.name] for f in dataclasses.fields(cls)})

    def spec(c):
        d = c.hidden_size

        def norm(name):
            return PartSpec("toy_centred", {"dim": d, "eps": c.eps, "name": name})

        def layer(p):
            return LayerSpec(
                mixer_norm=norm(p + "n1"), feed_forward_norm=norm(p + "n2"),
                feed_forward=PartSpec("swiglu", {"hidden": d, "inter": c.inter, "prefix": p + "ff."}),
                mixer=PartSpec("attention", {"hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                             "prefix": p + "attn.", "qk_norm": True, "eps": c.eps, "window": None,
                                             "position": PartSpec("rotate_half", {"head_dim": c.head_dim, "theta": c.theta})}))
        return ModelSpec(
            architecture="ToyCentredNormForCausalLM", vocab_size=c.vocab_size, hidden_size=d,
            embedding=PartSpec("table", {"vocab": c.vocab_size, "dim": d, "name": "embed.weight"}),
            layers=(layer("l0."), layer("l1.")), schedule=(Run(0, 0), Run(1, 1)),
            final_norm=norm("final"),
            head=PartSpec("linear", {"vocab": c.vocab_size, "dim": d, "name": "head.weight", "tied": False}),
            max_positions=256)

    register_architecture("ToyCentredNormForCausalLM", CentredConfig, spec, model_types=("toy_centred_norm",))


def centred_plain(w, ids):
    c = CENTRED
    s = len(ids)
    ang = P.rope_angles(np.arange(s), c["head_dim"], c["theta"])

    def norm(x, name):
        x = x - x.mean(-1, keepdims=True)
        return x / np.sqrt((x * x).mean(-1, keepdims=True) + c["eps"]) * w[name + ".weight"] + w[name + ".bias"]

    h = P.embedding(w["embed.weight"], ids)
    for p in ("l0.", "l1."):
        x = norm(h, p + "n1")
        q = P.rms_norm((x @ w[p + "attn.q_proj.weight"].T).reshape(s, c["heads"], c["head_dim"]),
                       w[p + "attn.q_norm.weight"], c["eps"])
        k = P.rms_norm((x @ w[p + "attn.k_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"]),
                       w[p + "attn.k_norm.weight"], c["eps"])
        v = (x @ w[p + "attn.v_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        r = h + P.attention(P.apply_rope(q, ang), P.apply_rope(k, ang), v).reshape(s, -1) @ w[p + "attn.o_proj.weight"].T
        h = r + P.swiglu_mlp(norm(r, p + "n2"), w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"],
                             w[p + "ff.down_proj.weight"])
    return norm(h, "final") @ w["head.weight"].T


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_norm_of_its_own(tmp_path, dtype_name):
    """Every norm of the model is one registered here (mean, gain, bias): prompts whole, their tails token by
    token (steps small enough that the products would take over an RMSNorm: here they must not)."""
    register_centred_norm()
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    from safetensors import safe_open
    folder = write_random_model(str(tmp_path / "m"), CENTRED, seed=31, dtype=torch.float32, matrix_std=0.12)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        w = {k: f.get_tensor(k).to(torch.float64).numpy() for k in f.keys()}
    assert "l0.n1.bias" in w
    model = load_model(folder, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name])
    rng = np.random.default_rng(32)
    reqs = {f"r{i}": [int(x) for x in rng.integers(0, CENTRED["vocab_size"], n)] for i, n in enumerate([40, 5, 66])}
    for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 24))):
        engine = engine_for_trace(model, plans.max_live_tokens(steps))
        player, outs = Replayer(engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.cpu().numpy()
        got = plans.collect(steps, lambda i: outs[i], CENTRED["vocab_size"])
        for rid, toks in reqs.items():
            assert_logits_close(got[rid], centred_plain(w, toks), dtype_name, f"centred norm, {what}, {rid}")


# ------------------------------------------------------------------------------------------------ more parts than four
SANDWICH = {"architectures": ["ToySandwichForCausalLM"], "vocab_size": 101, "hidden_size": 56, "inter": 72, "heads": 4,
            "kv_heads": 2, "head_dim": 24, "rotated": 8, "period": 29, "eps": 1e-5, "theta": 10000.0}


def register_sandwich():
    """A layer with six named parts and two things kept per sequence: norms before AND after its attention
    branch, a second mixer with a state of its own beside the attention, an attention with biases whose
    position encoding rotates a third of each head and then, after the per-head norm, adds a learned row.

        x = n1(h);  r = h + n1b(attention(x)) + running_sum(x);  h' = r + ff(n2(r))
    """
    from rust_inference_amd.cache import StateNeed
    from rust_inference_amd.config import ModelConfig, register_architecture
    from rust_inference_amd.parts import LayerSpec, Mixer, ModelSpec, PartSpec, PositionEncoding, Run, register_part
    from rust_inference_amd.parts.registry import build_part
    from rust_inference_amd.weights import MATRIX, TensorSpec

    @register_part("position", "toy_part_rotary_then_add")
    class PartRotaryThenAdd(PositionEncoding):
        acts_after_norm = True

        def __init__(self, rotated, theta, period, head_dim, name):
            self.rotated, self.theta, self.period, self.head_dim, self.name = rotated, theta, period, head_dim, name

        def tensors(self):
            return {self.name: TensorSpec((self.period, self.head_dim), MATRIX)}

        def bind(self, weights, rt):
            self.rt = rt
            self.table = weights[self.name].to(rt.device, torch.float32)
            i = torch.arange(self.rotated // 2, dtype=torch.float32)
            self.inv_freq = (1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float32),
                                             2.0 * i / float(self.rotated))).to(rt.device).contiguous()

        def rotation_table(self):
            return self.inv_freq                              # shorter than head_dim / 2: part of the head rotates

        def apply_normed(self, qkv, ctx, heads, kv_heads, head_dim):
            add = self.table[ctx.tok_pos.long() % self.period]
            qk = qkv[:, :(heads + kv_heads) * head_dim].unflatten(1, (heads + kv_heads, head_dim))
            qk.copy_((qk.float() + add[:, None, :]).to(qkv.dtype))

    @register_part("mixer", "toy_running_sum")
    class RunningSum(Mixer):
        """y_t = W . (x_0 + .. + x_t) / 8: the state is the running sum, per sequence."""
        def __init__(self, hidden, name):
            self.hidden, self.name = hidden, name

        def tensors(self):
            return {self.name: TensorSpec((self.hidden, self.hidden), MATRIX)}

        def bind(self, weights, rt):
            self.rt = rt
            self.w = weights[self.name].to(rt.device, torch.float32)

        def cache_need(self):
            return StateNeed((self.hidden,), torch.float32)

        def forward(self, x, ctx, store, page_table):
            out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            begin = 0
            for slot, n in zip(ctx.slot_list, ctx.new_counts):
                total = store[slot] + torch.cumsum(x[begin:begin + n].float(), 0)
                out[begin:begin + n] = (total / 8.0) @ self.w.T
                store[slot] = total[-1]
                begin += n
            return out

    @register_part("arrangement", "toy_sandwich")
    class Sandwich:
        def __init__(self, layer_spec):
            p = layer_spec.parts                              # six parts by name: whatever this arrangement asks for
            assert set(p) == {"mixer_norm", "mixer", "after_mixer_norm", "side_mixer", "feed_forward_norm", "feed_forward"}
            self.mixer_norm = build_part("norm", p["mixer_norm"])
            self.mixer = build_part("mixer", p["mixer"])
            self.after_mixer_norm = build_part("norm", p["after_mixer_norm"])
            self.side_mixer = build_part("mixer", p["side_mixer"])
            self.feed_forward_norm = build_part("norm", p["feed_forward_norm"])
            self.feed_forward = build_part("feed_forward", p["feed_forward"])

        def parts(self):
            return (self.mixer_norm, self.mixer, self.after_mixer_norm, self.side_mixer, self.feed_forward_norm,
                    self.feed_forward)

        def cache_need(self):
            return (self.mixer.cache_need(), self.side_mixer.cache_need())    # keys and values, and a state

        def forward(self, stream, ctx, store, page_table, act_dtype):
            (kv, state), (table, _) = store, page_table
            x = stream.normed(self.mixer_norm, act_dtype)
            branch = self.mixer.forward(x, ctx, kv, table).float()
            stream.push(self.after_mixer_norm.apply(branch, None, torch.float32))     # the norm of the branch alone
            stream.push(self.side_mixer.forward(x, ctx, state, None))
            stream.push(self.feed_forward.forward(stream.normed(self.feed_forward_norm, act_dtype), ctx))

    @dataclass(frozen=True)
    class SandwichConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        inter: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        rotated: int = 0
        period: int = 0
        eps: float = 1e-5
        theta: float = 1e4
        ARCHITECTURE: ClassVar[str] = "ToySandwichForCausalLM"
        MODEL_TYPE: ClassVar[str] = "toy_sandwich"

        @classmethod
        def from_dict(cls, raw):
            import dataclasses
            return cls(**{f.name: raw[f.name] for f in dataclasses.fields(cls)})

    def spec(c):
        d = c.hidden_size

        def norm(name):
            return PartSpec("rmsnorm", {"dim": d, "eps": c.eps, "name": name})

        def layer(p):
            return LayerSpec("toy_sandwich", parts={
                "mixer_norm": norm(p + "n1"), "after_mixer_norm": norm(p + "n1b"), "feed_forward_norm": norm(p + "n2"),
                "side_mixer": PartSpec("toy_running_sum", {"hidden": d, "name": p + "sum.weight"}),
                "feed_forward": PartSpec("swiglu", {"hidden": d, "inter": c.inter, "prefix": p + "ff."}),
                "mixer": PartSpec("attention", {
                    "hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim, "prefix": p + "attn.",
                    "qk_norm": True, "eps": c.eps, "window": None, "qkv_bias": True, "o_bias": True,
                    "position": PartSpec("toy_part_rotary_then_add", {
                        "rotated": c.rotated, "theta": c.theta, "period": c.period, "head_dim": c.head_dim,
                        "name": p + "attn.position.weight"})})})
        return ModelSpec(
            architecture="ToySandwichForCausalLM", vocab_size=c.vocab_size, hidden_size=d,
            embedding=PartSpec("table", {"vocab": c.vocab_size, "dim": d, "name": "embed.weight"}),
            layers=(layer("l0."), layer("l1.")),
            schedule=(Run(0, (0, 1)), Run(1, (2, 3))),          # a run names both of its layer's cache entries
            final_norm=norm("final.weight"),
            head=PartSpec("linear", {"vocab": c.vocab_size, "dim": d, "name": "head.weight", "tied": False}),
            max_positions=256)

    register_architecture("ToySandwichForCausalLM", SandwichConfig, spec, model_types=("toy_sandwich",))


def sandwich_plain(w, ids):
    c = SANDWICH
    h = P.embedding(w["embed.weight"], ids)
    pos = np.arange(len(ids))
    rot, dh = c["rotated"], c["head_dim"]
    inv = (np.float32(1.0) / np.power(np.float32(c["theta"]), (np.float32(2.0) * np.arange(rot // 2, dtype=np.float32))
                                      / np.float32(rot), dtype=np.float32)).astype(np.float32)
    ang = (pos.astype(np.float32)[:, None] * inv[None, :]).astype(np.float32).astype(np.float64)

    def attn(x, p):
        s = x.shape[0]
        add = w[p + "attn.position.weight"][pos % c["period"]][:, None, :]

        def head(name, n, gain):
            y = (x @ w[f"{p}attn.{name}_proj.weight"].T + w[f"{p}attn.{name}_proj.bias"]).reshape(s, n, dh)
            if gain is None:
                return y
            y = P.rms_norm(y, w[p + gain], c["eps"])
            return np.concatenate([P.apply_rope(y[..., :rot], ang), y[..., rot:]], -1) + add
        o = P.attention(head("q", c["heads"], "attn.q_norm.weight"), head("k", c["kv_heads"], "attn.k_norm.weight"),
                        head("v", c["kv_heads"], None))
        return o.reshape(s, -1) @ w[p + "attn.o_proj.weight"].T + w[p + "attn.o_proj.bias"]

    for p in ("l0.", "l1."):
        x = P.rms_norm(h, w[p + "n1"], c["eps"])
        r = h + P.rms_norm(attn(x, p), w[p + "n1b"], c["eps"]) + (np.cumsum(x, 0) / 8.0) @ w[p + "sum.weight"].T
        h = r + P.swiglu_mlp(P.rms_norm(r, w[p + "n2"], c["eps"]), w[p + "ff.gate_proj.weight"],
                             w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
    return P.rms_norm(h, w["final.weight"], c["eps"]) @ w["head.weight"].T


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_a_layer_of_six_parts_that_keeps_two_things_per_sequence(tmp_path, dtype_name):
    """Registered here, built by the unchanged model class and stepped by the unchanged engine: a layer whose
    arrangement names six parts, whose run names two cache entries (keys and values, and a state), with a
    head size of 24, biased products, a rotation over a third of the head and an encoding that acts after
    the per-head norm.  Whole, token by token and in unequal batches on a cache whose slots come back."""
    register_sandwich()
    from rust_inference_amd.cache import KVNeed, StateNeed
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    from safetensors import safe_open
    folder = write_random_model(str(tmp_path / "m"), SANDWICH, seed=21, dtype=torch.float32, matrix_std=0.12)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        w = {k: f.get_tensor(k).to(torch.float64).numpy() for k in f.keys()}
    assert {"l0.n1b", "l1.sum.weight", "l0.attn.q_proj.bias", "l1.attn.o_proj.bias", "l0.attn.position.weight"} <= set(w)
    model = load_model(folder, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name])
    needs = model.cache_needs()
    assert needs[0] == needs[2] == KVNeed(2, 24, None) and isinstance(needs[1], StateNeed) and needs[1] == needs[3]
    rng = np.random.default_rng(22)
    reqs = {f"r{i}": [int(x) for x in rng.integers(0, SANDWICH["vocab_size"], n)] for i, n in enumerate([50, 7, 33, 70])}
    for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 20)),
                        ("batches", plans.unequal_batches([
                            {k: (v, max(1, len(v) - 12)) for k, v in list(reqs.items())[:2]},
                            {k: (v, max(1, len(v) - 30)) for k, v in list(reqs.items())[2:]}]))):
        engine = engine_for_trace(model, plans.max_live_tokens(steps))
        player, outs = Replayer(engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.cpu().numpy()
        engine.cache.check_consistent()
        got = plans.collect(steps, lambda i: outs[i], SANDWICH["vocab_size"])
        for rid, toks in reqs.items():
            assert_logits_close(got[rid], sandwich_plain(w, toks), dtype_name, f"sandwich, {what}, {rid}")


# ------------------------------------------------------------------------------------------------ positions at the embedding
LEARNED = {"architectures": ["ToyLearnedPositionsForCausalLM"], "vocab_size": 83, "hidden_size": 48, "inter": 80, "heads": 3,
           "kv_heads": 1, "head_dim": 16, "eps": 1e-5, "positions": 96}


def register_learned_positions():
    """An embedding of another kind, registered from here: the token's row plus a learned row for its position
    (absolute positions enter the model here and nowhere else: the attention has no rotation).  The output
    matrix is tied to this embedding's table, which the head finds among the model's parts by name."""
    from rust_inference_amd.config import ModelConfig, register_architecture
    from rust_inference_amd.kernels import ops
    from rust_inference_amd.parts import Embedding, LayerSpec, ModelSpec, PartSpec, Run, register_part
    from rust_inference_amd.weights import MATRIX, TensorSpec

    @register_part("embedding", "toy_table_and_positions")
    class TableAndPositions(Embedding):
        def __init__(self, vocab, dim, positions, name, positions_name):
            self.vocab, self.dim, self.positions, self.name, self.positions_name = vocab, dim, positions, name, positions_name

        def tensors(self):
            return {self.name: TensorSpec((self.vocab, self.dim), MATRIX),
                    self.positions_name: TensorSpec((self.positions, self.dim), MATRIX)}

        def bind(self, weights, rt):
            self.rt = rt
            self.table = rt.place_matrix(weights[self.name])
            self.where = rt.place_matrix(weights[self.positions_name])

        def forward(self, ctx):
            # both gathers by the library's kernel; the positions are the step's own (the cache lengths)
            return ops.embed_gather(self.table, ctx.tokens) + ops.embed_gather(self.where, ctx.tok_pos)

    @dataclass(frozen=True)
    class LearnedConfig(ModelConfig):
        vocab_size: int = 0
        hidden_size: int = 0
        inter: int = 0
        heads: int = 0
        kv_heads: int = 0
        head_dim: int = 0
        eps: float = 1e-5
        positions: int = 0
        ARCHITECTURE: ClassVar[str] = "ToyLearnedPositionsForCausalLM"
        MODEL_TYPE: ClassVar[str] = "toy_learned_positions"

        @classmethod
        def from_dict(cls, raw):
            import dataclasses
            return cls(**{f.name: raw[f.name] for f in dataclasses.fields(cls)})

    def spec(c):
        d = c.hidden_size

        def norm(name):
            return PartSpec("rmsnorm", {"dim": d, "eps": c.eps, "name": name})

        def layer(p):
            return LayerSpec(
                mixer_norm=norm(p + "n1.weight"), feed_forward_norm=norm(p + "n2.weight"),
                feed_forward=PartSpec("swiglu", {"hidden": d, "inter": c.inter, "prefix": p + "ff."}),
                mixer=PartSpec("attention", {"hidden": d, "heads": c.heads, "kv_heads": c.kv_heads, "head_dim": c.head_dim,
                                             "prefix": p + "attn.", "qk_norm": False, "eps": c.eps, "window": None,
                                             "position": PartSpec("none")}))
        return ModelSpec(
            architecture="ToyLearnedPositionsForCausalLM", vocab_size=c.vocab_size, hidden_size=d,
            embedding=PartSpec("toy_table_and_positions", {"vocab": c.vocab_size, "dim": d, "positions": c.positions,
                                                           "name": "embed.weight", "positions_name": "embed.positions"}),
            layers=(layer("l0."), layer("l1.")), schedule=(Run(0, 0), Run(1, 1)),
            final_norm=norm("final.weight"),
            head=PartSpec("linear", {"vocab": c.vocab_size, "dim": d, "name": "head.weight", "tied": True}),
            max_positions=c.positions)

    register_architecture("ToyLearnedPositionsForCausalLM", LearnedConfig, spec, model_types=("toy_learned_positions",))


def learned_plain(w, ids):
    c = LEARNED
    s = len(ids)
    h = P.embedding(w["embed.weight"], ids) + w["embed.positions"][:s]
    for p in ("l0.", "l1."):
        x = P.rms_norm(h, w[p + "n1.weight"], c["eps"])
        q = (x @ w[p + "attn.q_proj.weight"].T).reshape(s, c["heads"], c["head_dim"])
        k = (x @ w[p + "attn.k_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        v = (x @ w[p + "attn.v_proj.weight"].T).reshape(s, c["kv_heads"], c["head_dim"])
        r = h + P.attention(q, k, v).reshape(s, -1) @ w[p + "attn.o_proj.weight"].T
        h = r + P.swiglu_mlp(P.rms_norm(r, w[p + "n2.weight"], c["eps"]), w[p + "ff.gate_proj.weight"],
                             w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
    return P.rms_norm(h, w["final.weight"], c["eps"]) @ w["embed.weight"].T


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_an_embedding_that_adds_learned_positions(tmp_path, dtype_name):
    """The embedding part gets the step's context: one that adds a learned row per position (and ties the output
    matrix to its table) is registered here and runs through the unchanged model, whole prompts, their tails
    token by token and unequal batches on reused slots alike; without the positions the logits would not
    depend on the order of the earlier tokens' positions at all, so a cut that got them wrong would show."""
    register_learned_positions()
    from rust_inference_amd.engine.replay import Replayer, engine_for_trace
    from rust_inference_amd.parts import load_model
    from rust_inference_amd.weights import write_random_model
    from safetensors import safe_open
    folder = write_random_model(str(tmp_path / "m"), LEARNED, seed=41, dtype=torch.float32, matrix_std=0.15)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        w = {k: f.get_tensor(k).to(torch.float64).numpy() for k in f.keys()}
    assert "embed.positions" in w and "head.weight" not in w
    model = load_model(folder, {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name])
    assert model.head.weight is model.embedding.table
    rng = np.random.default_rng(42)
    reqs = {f"r{i}": [int(x) for x in rng.integers(0, LEARNED["vocab_size"], n)] for i, n in enumerate([40, 5, 66, 33])}
    # the positions matter: the same tokens one place later give other logits
    moved = learned_plain(w, [reqs["r0"][0]] + reqs["r0"])[1:]
    assert np.abs(moved - learned_plain(w, reqs["r0"])).max() > 1e-2
    for what, steps in (("whole", plans.whole(reqs)), ("tail", plans.tail_one_by_one(reqs, 24)),
                        ("batches", plans.unequal_batches([
                            {k: (v, max(1, len(v) - 20)) for k, v in list(reqs.items())[:2]},
                            {k: (v, max(1, len(v) - 30)) for k, v in list(reqs.items())[2:]}]))):
        engine = engine_for_trace(model, plans.max_live_tokens(steps))
        player, outs = Replayer(engine), {}
        for s in steps:
            logits = player.feed(s)
            if logits is not None:
                outs[s["step"]] = logits.cpu().numpy()
        engine.cache.check_consistent()
        got = plans.collect(steps, lambda i: outs[i], LEARNED["vocab_size"])
        for rid, toks in reqs.items():
            assert_logits_close(got[rid], learned_plain(w, toks), dtype_name, f"learned positions, {what}, {rid}")
