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


def mixer_alone(rt, tiny_folders, name, dtype, build, before_rotation=None):
    """The mixer of a sliding layer and of a global one over a cache of their own: a portion of a
    prompt, then single tokens, against the plain rope + attention + projections.
    ``build(spec)`` makes the mixer; ``before_rotation(q, k)`` is what the plain side does to
    queries and keys [T, heads, hd] between the products and the rotation."""
    from zse_amd.engine.model import CallCache
    from zse_amd.engine.runner import GroupView
    from zse_amd.models.gemma2 import Gemma2Config, gemma2_plan
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
        mixer = build(spec)
        for p in [mixer] + mixer.children():
            p.load(src, rt, dtype)
        x = rounded(rng.normal(size=(T, H)), dtype)
        pos = np.arange(T)
        f64 = np.float64
        q = (x @ w[spec.names["q"]].T.astype(f64)).reshape(T, c["nh"], c["hd"])
        kk = (x @ w[spec.names["k"]].T.astype(f64)).reshape(T, c["nkv"], c["hd"])
        vv = (x @ w[spec.names["v"]].T.astype(f64)).reshape(T, c["nkv"], c["hd"])
        if before_rotation is not None:
            q, kk = before_rotation(q, kk)
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_attention_mixer_alone(rt, tiny_folders, name, dtype):
    from zse_amd.parts import build_part
    mixer_alone(rt, tiny_folders, name, dtype, lambda spec: build_part("mixer", spec))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_that_differs_between_product_and_rotation(rt, tiny_folders, dtype):
    """Attention whose queries and keys are scaled to unit length, head by head, before they are
    rotated: a subclass of the framework's attention that overrides one method and brings one
    kernel; product, rotation, cache, attention kernels and output product stay the framework's."""
    import toy_kernels  # noqa: F401  (registers zk_toy_head_norm)
    from zse_amd.parts.attention import PagedAttention

    class UnitLengthAttention(PagedAttention):
        def between_product_and_rotation(self, ctx, qkv):
            s = self.spec
            ctx.rt.kernels(ctx.dtype).zk_toy_head_norm(qkv.ptr, qkv.shape[0], qkv.shape[1],
                                                       s.num_heads + s.num_kv_heads, s.head_dim, ctx.stream)

    def unit(q, k):
        return (q / np.linalg.norm(q, axis=-1, keepdims=True), k / np.linalg.norm(k, axis=-1, keepdims=True))

    mixer_alone(rt, tiny_folders, "B", dtype, UnitLengthAttention, before_rotation=unit)


def test_toy_mixer_with_state_is_registered_built_and_stepped(rt):
    """A mixer the framework has never heard of: out_t = s_t W^T with s_t = a * s_(t-1) + x_t kept per
    request in its state slot.  Its architecture is registered here, built through the registry and
    stepped in portions and in mixed batches; the cut must not change the result."""
    from zse_amd.config import BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerCall, ModelPlan, NormSpec
    from zse_amd.engine.loading import random_model
    from zse_amd.engine.runner import StepEntry, StepRunner
    from toy_state import DecaySpec, toy_architecture

    H, V, I, L, A = 64, 200, 96, 2, 0.75

    def plan_of(cfg):
        norm = lambda n: NormSpec(H, 1e-6, False, n)
        layers = tuple(BlockSpec("prenorm", DecaySpec(H, A, f"l{l}.mix.w"),
                                 GatedMLPSpec(H, I, "silu", {r: f"l{l}.ffn.{r}" for r in ("gate", "up", "down")}),
                                 {"pre_mixer": norm(f"l{l}.n1"), "pre_ffn": norm(f"l{l}.n2")}) for l in range(L))
        return ModelPlan("ToyDecayLM", H, V, 512, EmbeddingSpec(V, H, 1.0, "emb"), layers,
                         tuple(LayerCall(l) for l in range(L)), norm("final"), HeadSpec(V, H, None, "emb"))

    with toy_architecture("ToyDecayLM", plan_of):
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
        assert not runner.graph_safe          # the toy reads the step's description on the host


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_part_brings_a_kernel_of_its_own(rt, dtype):
    """The toy mixer's recurrence as a kernel in a file beside the tests, registered with one
    call: the framework compiles it, calls it like its own, repeats it from launch lists and
    replays it inside captured graphs, and no file of the framework names it.  Same weights,
    same tokens: the bits of the toy mixer whose recurrence runs on the host."""
    import os
    import subprocess
    from conftest import ROOT
    from zse_amd.config import BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerCall, ModelPlan, NormSpec
    from zse_amd.config import Architecture, register_architecture, unregister_architecture
    from zse_amd.engine.loading import random_model
    from zse_amd.engine.runner import StepEntry, StepRunner
    from toy_state import DecaySpec, toy_architecture
    from toy_decay_device import DeviceDecaySpec

    H, V, I, L, A = 64, 200, 96, 2, 0.75

    def plan_with(spec, name):
        def plan_of(cfg):
            norm = lambda n: NormSpec(H, 1e-6, False, n)
            layers = tuple(BlockSpec("prenorm", spec(H, A, f"l{l}.mix.w"),
                                     GatedMLPSpec(H, I, "silu", {r: f"l{l}.ffn.{r}" for r in ("gate", "up", "down")}),
                                     {"pre_mixer": norm(f"l{l}.n1"), "pre_ffn": norm(f"l{l}.n2")}) for l in range(L))
            return ModelPlan(name, H, V, 512, EmbeddingSpec(V, H, 1.0, "emb"), layers,
                             tuple(LayerCall(l) for l in range(L)), norm("final"), HeadSpec(V, H, None, "emb"))
        return plan_of

    rng = np.random.default_rng(0)
    streams = {"a": rng.integers(0, V, 29).tolist(), "b": rng.integers(0, V, 17).tolist()}
    # portions of sizes that come back, then single tokens side by side: shapes repeat, so launch
    # lists run and the graph of bucket 2 is captured and replayed
    steps = [[("a", 5)], [("b", 5)], [("a", 5)], [("b", 5)], [("a", 5)], [("b", 2)]]
    steps += [[("a", 1), ("b", 1)] for _ in range(4)] + [[("b", 1)]] + [[("a", 1)] for _ in range(10)]

    def run(runner):
        fed = {r: 0 for r in streams}
        rows = {r: [] for r in streams}
        for st in steps:
            z = runner.step([StepEntry(r, streams[r][fed[r]:fed[r] + n], [n - 1]) for r, n in st])
            for (r, n), row in zip(st, z):
                rows[r].append(row.copy())
                fed[r] += n
        assert all(fed[r] == len(t) for r, t in streams.items())
        return {r: np.stack(v) for r, v in rows.items()}

    limits = dict(page_size=4, cache_tokens=64, max_seqs=3, max_batch_tokens=64, max_model_len=128)
    with toy_architecture("ToyDecayLM", plan_with(DecaySpec, "ToyDecayLM")):
        host_model = random_model({"architectures": ["ToyDecayLM"]}, dtype, seed=4, std=0.1, gain_std=0.1, rt=rt)
        want = run(StepRunner(host_model, rt, dtype, use_graphs=False, **limits))
    register_architecture(Architecture("ToyDecayDeviceLM", lambda d: d, plan_with(DeviceDecaySpec, "ToyDecayDeviceLM")))
    try:
        model = random_model({"architectures": ["ToyDecayDeviceLM"]}, dtype, seed=4, std=0.1, gain_std=0.1, rt=rt)
        plain = StepRunner(model, rt, dtype, use_graphs=False, use_steplists=False, **limits)
        assert plain.graph_safe and hasattr(plain.k, "zk_toy_decay")
        got_plain = run(plain)
        runner = StepRunner(model, rt, dtype, use_graphs=True, **limits)
        got = run(runner)
        assert runner.use_steplists and runner.steplist_runs >= 2, "the part's kernel kept steps from being written down"
        assert any(isinstance(g, int) for g in runner.graphs.values()), "no decode step was captured"
        names = {runner.k._dll.zk_steplist_name(h, i).decode() for h in runner.steplists.values()
                 for i in range(runner.k.steplist_size(h))}
        assert "zk_toy_decay" in names
        runner.close(), plain.close()
    finally:
        unregister_architecture("ToyDecayDeviceLM")
    for r in streams:
        assert np.array_equal(got[r], got_plain[r]), f"{r}: lists and graphs against launches from Python"
        assert np.array_equal(got[r], want[r]), f"{r}: the kernel against the recurrence on the host"
    # nothing under zse_amd/ knows the toy
    hits = subprocess.run(["grep", "-rl", "toy_decay", os.path.join(ROOT, "zse_amd"), "--include=*.py",
                           "--include=*.hip", "--include=*.h", "--include=*.cpp"], capture_output=True, text=True)
    assert hits.stdout.strip() == "", hits.stdout


def test_toy_mixer_with_state_through_the_engine(rt):
    """The same toy mixer behind the scheduler: layer 0 keeps its recurrence in the request's
    state slot, layer 1 is the framework's attention over pages.  Six requests share two slots
    and a pool so small that requests are preempted and computed again; every slot a request
    gets, first or again, must start from zero, so each request's tokens equal its run alone."""
    from zse_amd.config import (AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerCall,
                                ModelPlan, NormSpec, RotarySpec)
    from zse_amd.engine.engine import Engine
    from zse_amd.engine.loading import random_model
    from zse_amd.sampling import SamplingParams
    from toy_state import DecaySpec, toy_architecture

    H, V, I, nh, nkv, hd = 64, 200, 96, 4, 2, 16

    def plan_of(cfg):
        norm = lambda n: NormSpec(H, 1e-6, False, n)
        ffn = lambda l: GatedMLPSpec(H, I, "silu", {r: f"l{l}.ffn.{r}" for r in ("gate", "up", "down")})
        norms = lambda l: {"pre_mixer": norm(f"l{l}.n1"), "pre_ffn": norm(f"l{l}.n2")}
        attn = AttentionSpec(H, nh, nkv, hd, hd ** -0.5, None, None, RotarySpec(hd, hd, 10000.0),
                             {r: f"l1.attn.{r}" for r in "qkvo"})
        layers = (BlockSpec("prenorm", DecaySpec(H, 0.75, "l0.mix.w"), ffn(0), norms(0)),
                  BlockSpec("prenorm", attn, ffn(1), norms(1)))
        return ModelPlan("ToyStateAndPagesLM", H, V, 256, EmbeddingSpec(V, H, 1.0, "emb"), layers,
                         (LayerCall(0), LayerCall(1)), norm("final"), HeadSpec(V, H, None, "emb"))

    with toy_architecture("ToyStateAndPagesLM", plan_of):
        model = random_model({"architectures": ["ToyStateAndPagesLM"]}, "float32", seed=6, std=0.15,
                             gain_std=0.1, rt=rt)
        rng = np.random.default_rng(3)
        prompts = [rng.integers(0, V, n).tolist() for n in (9, 14, 5, 11, 7, 13)]
        sp = SamplingParams(max_tokens=12, temperature=0.0)
        alone = []
        for p in prompts:
            eng = Engine(model, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=64,
                         max_batch_seqs=2, prefill_chunk_size=5, max_seq_len=64)
            alone.append(eng.generate([p], sp)[0])
            eng.close()
        # 9 pages of 4 tokens: one request needs up to 7, two that decode side by side up to 12
        eng = Engine(model, dtype="float32", block_size=4, num_blocks=9, max_batch_tokens=64,
                     max_batch_seqs=2, prefill_chunk_size=5, max_seq_len=64)
        assert eng.runner.slot_bytes == H * 4 and len(eng.runner.manager.groups) == 1
        admitted = []
        clear = eng.runner.manager.on_admit
        eng.runner.manager.on_admit = lambda r, s: (admitted.append((r, s)), clear(r, s))
        together = eng.generate(prompts, sp)
        assert together == alone
        st = eng.stats()
        assert st.preemptions > 0                                   # slots were taken again after giving up
        assert len(admitted) >= len(prompts) + st.preemptions and {s for _, s in admitted} == {0, 1}
        eng.runner.manager.check()
        eng.close()
