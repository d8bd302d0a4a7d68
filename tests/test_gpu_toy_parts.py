"""Parts the framework has never heard of, defined here and registered from here: a feed-forward
with routing and another position encoding.  Each makes an architecture of its own out of the
framework's other parts, is written to a model folder with random weights, loaded, stepped whole
and in portions, and compared with the same model written out in NumPy.  Nothing under zse_amd/
changes for them.  (The toys do their own arithmetic on the host: they show the interfaces, not
speed.)"""
import os
from dataclasses import dataclass
from typing import Dict

import numpy as np
import pytest

from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu

F64 = np.float64


@pytest.fixture(scope="module")
def rt():
    from zse_amd.runtime.device import Runtime
    return Runtime.get()


def norm_plain(x, w, eps):
    return P.rmsnorm(x, w, eps, F64, unit_offset=False)


def host_rows(ctx):
    """(request slot, first position, count) of the step's rows, in row order."""
    return [(slot, start, n) for _, slot, start, n in ctx.entries]


def run_cuts(runner, streams, steps):
    """Feed ``streams`` (name -> token list) in the given steps [(name, n), ...]; logits of every
    token per stream, in order."""
    from zse_amd.engine.runner import StepEntry
    fed = {r: 0 for r in streams}
    rows = {r: [] for r in streams}
    for st in steps:
        es = [StepEntry(r, streams[r][fed[r]:fed[r] + n], range(n)) for r, n in st]
        z = runner.step(es)
        at = 0
        for r, n in st:
            rows[r].append(z[at:at + n])
            at += n
            fed[r] += n
    for r in streams:
        assert fed[r] == len(streams[r])
        runner.finish(r)
    return {r: np.concatenate(v) for r, v in rows.items()}


# ------------------------------------------------------------------ a feed-forward with routing
def test_toy_routed_feed_forward(rt, tmp_path):
    """Every token goes to the one expert its router scores highest (of three gated MLPs, the
    framework's own part as children), weighted by that expert's softmax probability."""
    from zse_amd.config import (Architecture, AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec,
                                LayerCall, ModelPlan, NormSpec, RotarySpec, register_architecture,
                                unregister_architecture)
    from zse_amd.engine.loading import load_model
    from zse_amd.engine.runner import StepRunner
    from zse_amd.parts import Part, TensorReq, build_part, register_part, unregister_part
    from zse_amd.weights import write_random_model
    from zse_amd.weights.safetensors import read_folder_f32

    H, V, I, L, E, nh, nkv, hd, theta, eps = 48, 150, 40, 2, 3, 4, 2, 16, 1000.0, 1e-5

    @dataclass(frozen=True)
    class RoutedSpec:
        hidden_size: int
        experts: tuple            # GatedMLPSpec of every expert
        router: str               # checkpoint name of the router matrix [experts, hidden]
        kind: str = "toy_routed"

    class RoutedFFN(Part):
        def __init__(self, spec):
            self.spec = spec
            self.experts = [build_part("ffn", e) for e in spec.experts]
            self.router = None

        def children(self):
            return list(self.experts)

        def tensor_reqs(self):
            return [TensorReq(self.spec.router, (len(self.spec.experts), self.spec.hidden_size))]

        def load(self, weights, rt_, dtype):
            self.router = rt_.download_f32(weights.matrix([self.spec.router])).astype(np.float32)

        def forward(self, ctx, x):
            xs = ctx.rt.download_f32(x)
            logits = xs.astype(F64) @ self.router.astype(F64).T
            pick = logits.argmax(-1)
            prob = np.exp(logits - logits.max(-1, keepdims=True))
            prob = prob / prob.sum(-1, keepdims=True)
            out = np.zeros_like(xs)
            for e, expert in enumerate(self.experts):
                rows = np.nonzero(pick == e)[0]
                if len(rows) == 0:
                    continue
                part = ctx.alloc((len(rows), xs.shape[1]))
                ctx.rt.copy_h2d(part.ptr, np.ascontiguousarray(xs[rows]))
                y = ctx.rt.download_f32(expert.forward(ctx, part))
                out[rows] = (y * prob[rows, e][:, None]).astype(np.float32)
            res = ctx.alloc(x.shape)
            ctx.rt.copy_h2d(res.ptr, out)
            return res

    def plan_of(cfg):
        norm = lambda n: NormSpec(H, eps, False, n)
        def block(l):
            experts = tuple(GatedMLPSpec(H, I, "gelu_tanh", {r: f"l{l}.e{e}.{r}" for r in ("gate", "up", "down")})
                            for e in range(E))
            mixer = AttentionSpec(H, nh, nkv, hd, hd ** -0.5, None, None, RotarySpec(hd, hd, theta),
                                  {r: f"l{l}.attn.{r}" for r in "qkvo"})
            return BlockSpec("prenorm", mixer, RoutedSpec(H, experts, f"l{l}.router"),
                             {"pre_mixer": norm(f"l{l}.n1"), "pre_ffn": norm(f"l{l}.n2")})
        return ModelPlan("ToyRoutedLM", H, V, 256, EmbeddingSpec(V, H, 1.0, "emb"), tuple(block(l) for l in range(L)),
                         tuple(LayerCall(l) for l in range(L)), norm("final"), HeadSpec(V, H, None, "emb"))

    def plain(w: Dict[str, np.ndarray], tokens):
        T = len(tokens)
        pos = np.arange(T)
        h = w["emb"][tokens].astype(F64)
        picks = []
        for l in range(L):
            x = norm_plain(h, w[f"l{l}.n1"], eps)
            q = (x @ w[f"l{l}.attn.q"].T.astype(F64)).reshape(T, nh, hd)
            k = (x @ w[f"l{l}.attn.k"].T.astype(F64)).reshape(T, nkv, hd)
            v = (x @ w[f"l{l}.attn.v"].T.astype(F64)).reshape(T, nkv, hd)
            o = P.attention(P.rope(q, pos, theta, F64), P.rope(k, pos, theta, F64), v, pos, hd ** -0.5, None, None, F64)
            h = h + o.reshape(T, -1) @ w[f"l{l}.attn.o"].T.astype(F64)
            x = norm_plain(h, w[f"l{l}.n2"], eps)
            logits = x @ w[f"l{l}.router"].T.astype(F64)
            pick = logits.argmax(-1)
            prob = np.exp(logits - logits.max(-1, keepdims=True))
            prob /= prob.sum(-1, keepdims=True)
            m = np.zeros_like(h)
            for e in range(E):
                rows = pick == e
                m[rows] = P.geglu_ffn(x[rows], w[f"l{l}.e{e}.gate"], w[f"l{l}.e{e}.up"], w[f"l{l}.e{e}.down"], F64) \
                    * prob[rows, e][:, None]
            h = h + m
            picks.append(pick)
        return norm_plain(h, w["final"], eps) @ w["emb"].T.astype(F64), picks

    register_part("ffn", "toy_routed", RoutedFFN)
    register_architecture(Architecture("ToyRoutedLM", lambda d: d, plan_of))
    try:
        folder = write_random_model(str(tmp_path / "routed"), {"architectures": ["ToyRoutedLM"]}, seed=11, std=0.15,
                                    gain_std=0.1, dtype="float32", std_of={"router": 1.0, "n1": 0.3, "n2": 0.3, "final": 0.3})
        w = read_folder_f32(folder)
        for n in list(w):                       # the norms' gains are plain gains here: keep them away from zero
            if n.endswith((".n1", ".n2")) or n == "final":
                w[n] = w[n] + 1.0
        from zse_amd.weights.safetensors import write_file
        write_file(os.path.join(folder, "model.safetensors"), {n: ("F32", a) for n, a in w.items()})
        model = load_model(folder, "float32", rt)
        assert {f"l1.e{e}.down" for e in range(E)} | {"l0.router"} <= {r.name for r in model.tensor_reqs()}
        runner = StepRunner(model, rt, "float32", page_size=4, cache_tokens=128, max_seqs=3, max_batch_tokens=64,
                            max_model_len=128, use_graphs=False)
        rng = np.random.default_rng(5)
        streams = {"a": rng.integers(0, V, 37).tolist(), "b": rng.integers(0, V, 20).tolist()}
        whole = run_cuts(runner, streams, [[("a", 37)], [("b", 20)]])
        for r, toks in streams.items():
            want, picks = plain(w, toks)
            assert all(len(set(p.tolist())) > 1 for p in picks), "the router should use more than one expert"
            assert np.abs(whole[r] - want).max() < 5e-5 * max(1.0, np.abs(want).max()), r
        cut = run_cuts(runner, streams, [[("a", 9)], [("a", 2), ("b", 13)], [("a", 1), ("b", 1)], [("a", 25), ("b", 6)]])
        for r in streams:
            assert np.abs(cut[r] - whole[r]).max() < 5e-5 * max(1.0, np.abs(whole[r]).max()), r
        assert all(p.free_pages == p.num_pages for p in runner.manager.pools)
    finally:
        unregister_part("ffn", "toy_routed")
        unregister_architecture("ToyRoutedLM")


# ------------------------------------------------------------------ another position encoding
def test_toy_learned_position_encoding(rt, tmp_path):
    """Queries and keys get a learned vector of their absolute position added (one table row per
    position, the same for every head); the mixer is the framework's attention, told by its spec
    to use this encoding instead of the rotary one."""
    from zse_amd.config import (Architecture, AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec,
                                LayerCall, ModelPlan, NormSpec, register_architecture, unregister_architecture)
    from zse_amd.engine.loading import load_model
    from zse_amd.engine.runner import StepRunner
    from zse_amd.parts import Part, TensorReq, register_part, unregister_part
    from zse_amd.weights import write_random_model
    from zse_amd.weights.safetensors import read_folder_f32, write_file

    H, V, I, L, nh, nkv, hd, eps, maxpos, window = 40, 90, 56, 2, 6, 3, 16, 1e-6, 64, 9

    @dataclass(frozen=True)
    class LearnedSpec:
        head_dim: int
        max_position: int
        table: str
        kind: str = "toy_learned"

    class LearnedPosition(Part):
        def __init__(self, spec):
            self.spec, self.table = spec, None

        def tensor_reqs(self):
            return [TensorReq(self.spec.table, (self.spec.max_position, self.spec.head_dim))]

        def load(self, weights, rt_, dtype):
            self.table = rt_.download_f32(weights.matrix([self.spec.table])).astype(np.float32)

        def rotary_tables(self):
            return None                          # not a rotation: the mixer calls apply()

        def apply(self, ctx, qkv, num_heads, num_kv_heads, head_dim):
            a = ctx.rt.download_f32(qkv)
            pos = np.concatenate([np.arange(start, start + n) for _, start, n in host_rows(ctx)])
            add = self.table[pos]                                     # [T, hd]
            heads = a.reshape(len(pos), -1, head_dim)
            heads[:, :num_heads + num_kv_heads] += add[:, None, :]    # q heads, then k heads; v is left alone
            ctx.rt.copy_h2d(qkv.ptr, np.ascontiguousarray(heads.reshape(a.shape)))

    def plan_of(cfg):
        norm = lambda n: NormSpec(H, eps, False, n)
        def block(l):
            mixer = AttentionSpec(H, nh, nkv, hd, 0.3, 25.0, window if l == 0 else None,
                                  LearnedSpec(hd, maxpos, f"l{l}.pos"), {r: f"l{l}.attn.{r}" for r in "qkvo"})
            ffn = GatedMLPSpec(H, I, "silu", {r: f"l{l}.ffn.{r}" for r in ("gate", "up", "down")})
            return BlockSpec("prenorm", mixer, ffn, {"pre_mixer": norm(f"l{l}.n1"), "pre_ffn": norm(f"l{l}.n2")})
        return ModelPlan("ToyLearnedPosLM", H, V, maxpos, EmbeddingSpec(V, H, 1.0, "emb"),
                         tuple(block(l) for l in range(L)), tuple(LayerCall(l) for l in range(L)), norm("final"),
                         HeadSpec(V, H, None, "emb"))

    def plain(w, tokens):
        T = len(tokens)
        pos = np.arange(T)
        h = w["emb"][tokens].astype(F64)
        for l in range(L):
            x = norm_plain(h, w[f"l{l}.n1"], eps)
            add = w[f"l{l}.pos"][pos].astype(F64)[:, None, :]
            q = (x @ w[f"l{l}.attn.q"].T.astype(F64)).reshape(T, nh, hd) + add
            k = (x @ w[f"l{l}.attn.k"].T.astype(F64)).reshape(T, nkv, hd) + add
            v = (x @ w[f"l{l}.attn.v"].T.astype(F64)).reshape(T, nkv, hd)
            o = P.attention(q, k, v, pos, 0.3, 25.0, window if l == 0 else None, F64)
            h = h + o.reshape(T, -1) @ w[f"l{l}.attn.o"].T.astype(F64)
            x = norm_plain(h, w[f"l{l}.n2"], eps)
            g = x @ w[f"l{l}.ffn.gate"].T.astype(F64)
            h = h + (g / (1 + np.exp(-g)) * (x @ w[f"l{l}.ffn.up"].T.astype(F64))) @ w[f"l{l}.ffn.down"].T.astype(F64)
        return norm_plain(h, w["final"], eps) @ w["emb"].T.astype(F64)

    register_part("position", "toy_learned", LearnedPosition)
    register_architecture(Architecture("ToyLearnedPosLM", lambda d: d, plan_of))
    try:
        folder = write_random_model(str(tmp_path / "learned"), {"architectures": ["ToyLearnedPosLM"]}, seed=3, std=0.2,
                                    gain_std=0.1, dtype="float32", std_of={".pos": 1.0})
        w = read_folder_f32(folder)
        for n in list(w):
            if n.endswith((".n1", ".n2")) or n == "final":
                w[n] = w[n] + 1.0
        write_file(os.path.join(folder, "model.safetensors"), {n: ("F32", a) for n, a in w.items()})
        model = load_model(folder, "float32", rt)
        runner = StepRunner(model, rt, "float32", page_size=4, cache_tokens=128, max_seqs=3, max_batch_tokens=64,
                            max_model_len=maxpos, use_graphs=False)
        assert [g.window for g in runner.manager.groups] == [window, None]      # one group of pages per need
        rng = np.random.default_rng(9)
        streams = {"a": rng.integers(0, V, 41).tolist(), "b": rng.integers(0, V, 17).tolist()}
        whole = run_cuts(runner, streams, [[("a", 41)], [("b", 17)]])
        for r, toks in streams.items():
            want = plain(w, toks)
            assert np.abs(whole[r] - want).max() < 5e-5 * max(1.0, np.abs(want).max()), r
        # the encoding matters: without it the logits are others
        w0 = dict(w)
        for l in range(L):
            w0[f"l{l}.pos"] = np.zeros_like(w[f"l{l}.pos"])
        assert np.abs(plain(w0, streams["a"]) - whole["a"]).max() > 1e-2
        cut = run_cuts(runner, streams, [[("a", 3)], [("b", 2), ("a", 10)], [("a", 1), ("b", 1)], [("b", 14), ("a", 27)]])
        for r in streams:
            assert np.abs(cut[r] - whole[r]).max() < 5e-5 * max(1.0, np.abs(whole[r]).max()), r
        assert all(p.free_pages == p.num_pages for p in runner.manager.pools)
    finally:
        unregister_part("position", "toy_learned")
        unregister_architecture("ToyLearnedPosLM")
