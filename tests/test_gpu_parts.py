"""Each part alone against the plain implementation's function for it, and a toy mixer with
state of its own that is registered, built and stepped without touching the framework."""
import numpy as np
import pytest

from conftest import TINY, read_weights
from gpu_util import bf16_round
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu


class Weights:
    """A weight source over host arrays, for parts built outside a model."""

    def __init__(self, rt, dtype, arrays):
        self.rt, self.dtype, self.arrays = rt, dtype, arrays

    def matrix(self, names, strip=False):
        from zse_amd.weights.safetensors import f32_to_bf16_bits
        a = np.concatenate([self.arrays[n] for n in names]).astype(np.float32)
        return self.rt.upload(f32_to_bf16_bits(a), "bfloat16") if self.dtype == "bfloat16" else self.rt.upload(a)

    def vector(self, name):
        return self.rt.upload(self.arrays[name].astype(np.float32))


class Ctx:
    """The least a part needs of a step."""

    def __init__(self, rt, dtype, tuned=True):
        from zse_amd.engine.runner import Arena
        self.rt, self.k, self.dtype, self.tuned, self.stream = rt, rt.kernels(dtype), dtype, tuned, rt.stream
        self.arena = Arena(rt, 1 << 20)
        self.workspace = rt.zeros((1 << 16,), "float32")
        self.gemm_workspace = None

    def alloc(self, shape, dtype=None):
        return self.arena.alloc(shape, dtype or self.dtype)


def up(rt, x, dtype):
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    x = np.ascontiguousarray(x, np.float32)
    return rt.upload(f32_to_bf16_bits(x), "bfloat16") if dtype == "bfloat16" else rt.upload(x)


def rounded(x, dtype):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    x = np.asarray(x, np.float32)
    return bf16_bits_to_f32(f32_to_bf16_bits(x)) if dtype == "bfloat16" else x


@pytest.fixture(scope="module")
def rt():
    from zse_amd.runtime.device import Runtime
    return Runtime.get()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_norm_ffn_embedding_head_alone(rt, tiny_folders, name, dtype):
    from zse_amd.models.gemma2 import Gemma2Config, gemma2_plan
    from zse_amd.parts import build_part
    cfg = TINY[name][0]
    plan = gemma2_plan(Gemma2Config.from_dict(cfg))
    w = {k: rounded(v, dtype) for k, v in read_weights(tiny_folders[(name, dtype)]).items()}
    src, ctx = Weights(rt, dtype, w), Ctx(rt, dtype)
    tol = 2e-5 if dtype == "float32" else 0.02
    rng = np.random.default_rng(0)
    T, H = 9, cfg["hidden_size"]
    # norm
    spec = plan.layers[1].norms["pre_ffn"]
    norm = build_part("norm", spec)
    norm.load(src, rt, dtype)
    x = rng.normal(size=(T, H)).astype(np.float32)
    got = rt.download_f32(norm.forward(ctx, rt.upload(x)))
    want = P.rmsnorm(x, w[spec.weight], cfg["rms_norm_eps"], np.float64)
    assert np.abs(got - want).max() < tol * np.abs(want).max()
    # feed-forward
    ffn = build_part("ffn", plan.layers[1].ffn)
    ffn.load(src, rt, dtype)
    xa = rounded(x, dtype)
    got = rt.download_f32(ffn.forward(ctx, up(rt, xa, dtype)))
    n = plan.layers[1].ffn.names
    want = P.geglu_ffn(xa, w[n["gate"]], w[n["up"]], w[n["down"]], np.float64)
    assert np.abs(got - want).max() < tol * max(1.0, np.abs(want).max())
    # embedding
    emb = build_part("embedding", plan.embedding)
    emb.load(src, rt, dtype)
    toks = rng.integers(0, cfg["vocab_size"], T).astype(np.int32)
    toks_dev = rt.upload(toks)
    ctx.T, ctx.tokens = T, toks_dev.ptr
    scale = np.float32(np.sqrt(H)) if dtype == "float32" else np.float32(bf16_round(np.sqrt(H)))
    assert np.array_equal(rt.download(emb.forward(ctx)), w[plan.embedding.weight][toks] * scale)
    # head: the embedding matrix itself, unscaled, then the soft cap
    head = build_part("head", plan.head)
    head.load(src, rt, dtype)
    out = rt.empty((T, cfg["vocab_size"]), "float32")
    head.forward(ctx, up(rt, xa, dtype), out)
    want = P.softcap(xa.astype(np.float64) @ w[plan.embedding.weight].astype(np.float64).T,
                     cfg["final_logit_softcapping"], np.float64)
    assert np.abs(rt.download(out) - want).max() < tol * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_attention_mixer_alone(rt, tiny_folders, name, dtype):
    """The mixer of a sliding layer and of a global one over a cache of their own: a portion of a
    prompt, then single tokens, against the plain rope + attention + projections."""
    from zse_amd.engine.model import CallCache
    from zse_amd.engine.runner import GroupView
    from zse_amd.models.gemma2 import Gemma2Config, gemma2_plan
    from zse_amd.parts import build_part
    cfg = TINY[name][0]
    c = P.read_config(cfg)
    plan = gemma2_plan(Gemma2Config.from_dict(cfg))
    w = {k: rounded(v, dtype) for k, v in read_weights(tiny_folders[(name, dtype)]).items()}
    src = Weights(rt, dtype, w)
    tol = 3e-5 if dtype == "float32" else 0.03
    rng = np.random.default_rng(1)
    T, H, bs, pages = 45, cfg["hidden_size"], 8, 12
    for layer in (0, 1):
        spec = plan.layers[layer].mixer
        mixer = build_part("mixer", spec)
        for p in [mixer] + mixer.children():
            p.load(src, rt, dtype)
        x = rounded(rng.normal(size=(T, H)), dtype)
        pos = np.arange(T)
        f64 = np.float64
        q = (x @ w[spec.names["q"]].T.astype(f64)).reshape(T, c["nh"], c["hd"])
        kk = (x @ w[spec.names["k"]].T.astype(f64)).reshape(T, c["nkv"], c["hd"])
        vv = (x @ w[spec.names["v"]].T.astype(f64)).reshape(T, c["nkv"], c["hd"])
        o = P.attention(P.rope(q, pos, c["theta"], f64), P.rope(kk, pos, c["theta"], f64), vv, pos,
                        c["qpas"] ** -0.5, c["attn_cap"], spec.window, f64)
        want = o.reshape(T, -1) @ w[spec.names["o"]].T.astype(f64)
        ctx = Ctx(rt, dtype)
        vt = mixer.wants_v_transposed(ctx.k, dtype, bs)
        cache = CallCache(group=0, k=rt.zeros((pages, c["nkv"], bs, c["hd"]), dtype),
                          v=rt.zeros((pages, c["nkv"], c["hd"], bs) if vt else (pages, c["nkv"], bs, c["hd"]), dtype),
                          v_transposed=vt)
        table = rng.permutation(pages)[:-(-T // bs)].astype(np.int32)
        got = []
        for start, n in [(0, 30)] + [(i, 1) for i in range(30, T)]:
            p_ = np.arange(start, start + n)
            slots = (table[p_ // bs] * bs + p_ % bs).astype(np.int32)
            tb = np.full((1, 8), -1, np.int32)
            tb[0, :len(table)] = table
            keep = [rt.upload(a) for a in (p_.astype(np.int32), np.zeros(n, np.int32), np.array([0, n], np.int32),
                                           np.array([start + n], np.int32), tb, slots)]
            ctx.T, ctx.R = n, 1
            ctx.positions, ctx.req_of_token, ctx.q_start, ctx.ctx_len = (t.ptr for t in keep[:4])
            ctx.group = lambda gid: GroupView(keep[4].ptr, 8, keep[5].ptr, bs)
            ctx.n_multi, ctx.max_q_len, ctx.max_ctx = (1 if n > 1 else 0), n, start + n
            ctx.arena.reset()
            got.append(rt.download_f32(mixer.forward(ctx, up(rt, x[start:start + n], dtype), cache)))
        got = np.concatenate(got)
        assert np.abs(got - want).max() < tol * max(1.0, np.abs(want).max()), f"layer {layer}"


def test_toy_mixer_with_state_is_registered_built_and_stepped(rt):
    """A mixer the framework has never heard of: out_t = s_t W^T with s_t = a * s_(t-1) + x_t kept per
    request in its state slot.  Its architecture is registered here, built through the registry and
    stepped in portions and in mixed batches; the cut must not change the result."""
    from dataclasses import dataclass
    from zse_amd.config import (Architecture, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerCall,
                                ModelPlan, NormSpec, register_architecture, unregister_architecture)
    from zse_amd.engine.loading import random_model
    from zse_amd.engine.runner import StepEntry, StepRunner
    from zse_amd.parts import Part, StateNeed, TensorReq, register_part, unregister_part
    from zse_amd.parts.ops import linear

    H, V, I, L, A = 64, 200, 96, 2, 0.75

    @dataclass(frozen=True)
    class DecaySpec:
        hidden_size: int
        decay: float
        weight: str
        kind: str = "toy_decay"

    class DecayMixer(Part):
        def __init__(self, spec):
            self.spec, self.w = spec, None

        def tensor_reqs(self):
            return [TensorReq(self.spec.weight, (self.spec.hidden_size, self.spec.hidden_size))]

        def load(self, weights, rt_, dtype):
            self.w = weights.matrix([self.spec.weight])

        def cache_need(self):
            return StateNeed(self.spec.hidden_size * 4)

        def forward(self, ctx, x, cache):
            # the recurrence runs on the host here (a toy): rows in, rows out, state in the slot
            xs = ctx.rt.download_f32(x)
            words = ctx.slot_bytes // 4
            state = ctx.rt.download(ctx.state)
            o0, n_w = cache.state_offset // 4, cache.state_bytes // 4
            out = np.empty_like(xs)
            t = 0
            for _, slot, _, n in ctx.entries:
                s = state[slot, o0:o0 + n_w].copy()
                for i in range(n):
                    s = np.float32(self.spec.decay) * s + xs[t + i]
                    out[t + i] = s
                state[slot, o0:o0 + n_w] = s
                t += n
            ctx.rt.copy_h2d(ctx.state.ptr, state)
            y = ctx.alloc(x.shape)
            ctx.rt.copy_h2d(y.ptr, out)
            return linear(ctx, y, self.w, ctx.alloc(x.shape))

    def plan_of(cfg):
        norm = lambda n: NormSpec(H, 1e-6, False, n)
        layers = tuple(BlockSpec("prenorm", DecaySpec(H, A, f"l{l}.mix.w"),
                                 GatedMLPSpec(H, I, "silu", {r: f"l{l}.ffn.{r}" for r in ("gate", "up", "down")}),
                                 {"pre_mixer": norm(f"l{l}.n1"), "pre_ffn": norm(f"l{l}.n2")}) for l in range(L))
        return ModelPlan("ToyDecayLM", H, V, 512, EmbeddingSpec(V, H, 1.0, "emb"), layers,
                         tuple(LayerCall(l) for l in range(L)), norm("final"), HeadSpec(V, H, None, "emb"))

    register_part("mixer", "toy_decay", DecayMixer)
    register_architecture(Architecture("ToyDecayLM", lambda d: d, plan_of))
    try:
        model = random_model({"architectures": ["ToyDecayLM"]}, "float32", seed=4, std=0.1, gain_std=0.1, rt=rt)
        runner = StepRunner(model, rt, "float32", page_size=4, cache_tokens=64, max_seqs=3, max_batch_tokens=64,
                            max_model_len=128, use_graphs=False)
        assert runner.slot_bytes == L * H * 4 and not runner.manager.groups       # state only, no pages
        rng = np.random.default_rng(0)
        a, b = rng.integers(0, V, 23).tolist(), rng.integers(0, V, 11).tolist()
        whole_a = runner.step([StepEntry("a", a, range(23))])
        whole_b = runner.step([StepEntry("b", b, range(11))])
        runner.finish("a"), runner.finish("b")
        rows_a, rows_b = [], []
        steps = [[("a", 5)], [("a", 2), ("b", 3)], [("a", 1), ("b", 1)], [("b", 7)], [("a", 15)]]
        fa = fb = 0
        for st in steps:
            es = []
            for r, n in st:
                src_, f = (a, fa) if r == "a" else (b, fb)
                es.append(StepEntry(r + "2", src_[f:f + n], range(n)))
            z = runner.step(es)
            at = 0
            for r, n in st:
                (rows_a if r == "a" else rows_b).append(z[at:at + n])
                at += n
                if r == "a":
                    fa += n
                else:
                    fb += n
        assert np.array_equal(np.concatenate(rows_a), whole_a)
        assert np.array_equal(np.concatenate(rows_b), whole_b)
        # the state slot is cleared when it is given to the next request
        runner.finish("a2"), runner.finish("b2")
        again = runner.step([StepEntry("c", a, range(23))])
        assert np.array_equal(again, whole_a)
        # and the state really carries: against the recurrence done by hand for layer 0's mixer input
        assert not np.allclose(whole_a[5], runner.step([StepEntry("d", a[5:6], [0])])[0])
    finally:
        unregister_part("mixer", "toy_decay")
        unregister_architecture("ToyDecayLM")
