"""Generation through the entry points: ``Engine.generate`` and the ``zse generate`` command
against a greedy loop over the plain implementation; sampled requests against the plain
sampler on the engine's own logits."""
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT, TINY, random_tokens, read_weights
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu


def plain_greedy(cfg, w, prompt, n, margin_log=None):
    toks = list(prompt)
    for _ in range(n):
        z = P.forward(cfg, w, toks, np.float64)[-1]
        if margin_log is not None:
            s = np.sort(z)
            margin_log.append(s[-1] - s[-2])
        toks.append(int(np.argmax(z)))
    return toks[len(prompt):]


@pytest.mark.parametrize("name,lengths,n_new", [("A", (5, 11, 17), 8), ("B", (1, 9, 23, 40), 12)])
def test_greedy_generation_float32(tiny_folders, name, lengths, n_new):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY[name][0]
    folder = tiny_folders[(name, "float32")]
    w = read_weights(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 40 + n) for n in lengths]
    eng = Engine(folder, dtype="float32", block_size=4 if name == "A" else 8, num_blocks=64,
                 max_batch_tokens=32, max_batch_seqs=4, prefill_chunk_size=4 if name == "A" else 7,
                 max_seq_len=128)
    got = eng.generate(prompts, SamplingParams(max_tokens=n_new, temperature=0.0))
    for p, g in zip(prompts, got):
        assert g == plain_greedy(cfg, w, p, n_new)
    assert eng.stats().generated_tokens == n_new * len(prompts)
    # one prompt, the reference's call shape: prompt plus generated tokens come back
    both = eng.generate_tokens(prompts[0], max_tokens=3, temperature=0.0)
    assert both == prompts[0] + got[0][:3]
    assert list(eng.stream_generate_tokens(prompts[1], max_tokens=4, temperature=0.0)) == got[1][:4]
    eng.close()


def test_greedy_generation_bfloat16(tiny_folders):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY["A"][0]
    folder = tiny_folders[("A", "bfloat16")]
    w = read_weights(folder)
    prompts = [random_tokens(512, n, 60 + n) for n in (5, 11, 17)]
    eng = Engine(folder, dtype="bfloat16", block_size=4, num_blocks=64, max_batch_tokens=32,
                 max_batch_seqs=4, prefill_chunk_size=4, max_seq_len=128)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0))
    eng.close()
    for p, g in zip(prompts, got):
        toks = list(p)
        for i, t in enumerate(g):
            z = P.forward(cfg, w, toks, np.float64)[-1]
            s = np.sort(z)
            assert t == int(np.argmax(z)) or s[-1] - s[-2] < 0.05, f"token {i} of {p}"
            toks.append(t)


@pytest.mark.parametrize("temperature,top_k,top_p", [(0.0, 0, 1.0), (0.9, 0, 1.0), (0.9, 6, 0.8)])
def test_runs_of_steps_without_the_host_give_the_same_tokens(tiny_folders, temperature, top_k, top_p):
    """Decoding several steps in a row before the host reads an id (the ids go from step to step
    on the device) gives what step-by-step decoding gives: same tokens, same ends by length and
    by stop token (found late: the output is cut back to it), also when pages run short in the
    middle of a run and a request has to be recomputed."""
    from zse_amd.engine.engine import Engine
    from zse_amd.engine.request import FinishReason
    from zse_amd.sampling import SamplingParams
    cfg = TINY["B"][0]
    folder = tiny_folders[("B", "float32")]
    prompts = [random_tokens(cfg["vocab_size"], n, 70 + n) for n in (3, 9, 14, 6)]

    def run(decode_run, num_blocks, stops, seqs=4):
        eng = Engine(folder, dtype="float32", block_size=8, num_blocks=num_blocks, max_batch_tokens=32,
                     max_batch_seqs=seqs, prefill_chunk_size=7, max_seq_len=128, decode_run=decode_run)
        reqs = [eng.add_request(p, SamplingParams(max_tokens=m, temperature=temperature, seed=11 + i,
                                                  top_k=top_k, top_p=top_p, stop_tokens=stops))
                for i, (p, m) in enumerate(zip(prompts, (21, 5, 30, 13)))]
        eng.run()
        out = [(list(r.output_tokens), r.finish_reason) for r in reqs]
        st = eng.stats()
        assert st.generated_tokens == sum(len(o) for o, _ in out)
        assert len(st.ttft_ms) == len(reqs) and all(t >= 0 for t in st.ttft_ms + st.tpot_ms)      # every request reported once
        assert all(pool.free_pages == pool.num_pages for pool in eng.runner.manager.pools)
        eng.close()
        return out, st

    base, _ = run(1, 64, ())
    assert all(-1 not in o for o, _ in base)
    got, st = run(4, 64, ())
    assert got == base and st.steps >= 30
    # a stop token that some request produces in the middle of its output
    stop = base[2][0][len(base[2][0]) // 2]
    want, _ = run(1, 64, (stop,))
    assert any(r == FinishReason.STOP for _, r in want)
    assert run(4, 64, (stop,))[0] == want
    assert run(7, 64, (stop,))[0] == want
    # so few pages that a request is preempted and computed again while others are in a run
    tight, st1 = run(1, 8, ())
    assert st1.preemptions > 0 and [o for o, _ in tight] == [o for o, _ in base]
    assert run(4, 8, ())[0] == tight
    # more requests than places: runs go on while others wait, and the waiting ones get their turn
    few, st2 = run(4, 64, (stop,), seqs=2)
    assert few == want and st2.steps < run(1, 64, (stop,), seqs=2)[1].steps + 8


def test_sampled_requests_do_not_depend_on_the_batch(tiny_folders):
    """Temperature 0.8 with seed 7: the same tokens alone, in a batch, under another chunk size
    and after a forced recomputation; each token is what the plain sampler draws from the
    engine's own logits."""
    from zse_amd.engine.engine import Engine
    from zse_amd.engine.runner import StepEntry
    from zse_amd.sampling import SamplingParams, uniform
    cfg = TINY["B"][0]
    folder = tiny_folders[("B", "float32")]
    prompts = [random_tokens(1000, n, 80 + n) for n in (1, 9, 23, 40)]
    params = [SamplingParams(max_tokens=12, temperature=0.0), SamplingParams(max_tokens=12, temperature=0.8, seed=7),
              SamplingParams(max_tokens=12, temperature=0.0), SamplingParams(max_tokens=12, temperature=0.8, seed=7)]

    def run(chunk, seqs, blocks, which):
        eng = Engine(folder, dtype="float32", block_size=8, num_blocks=blocks, max_batch_tokens=64,
                     max_batch_seqs=seqs, prefill_chunk_size=chunk, max_seq_len=128)
        out = eng.generate([prompts[i] for i in which], [params[i] for i in which])
        st = eng.stats()
        eng.close()
        return out, st

    batch, _ = run(7, 4, 64, [0, 1, 2, 3])
    alone = [run(16, 1, 64, [i])[0][0] for i in range(4)]
    assert batch == alone
    tight, st = run(5, 4, 13, [0, 1, 2, 3])        # 13 pages of 8: pages run out while decoding
    assert st.preemptions > 0 and tight == batch
    # each sampled token is the plain sampler's draw on logits of the same position
    from gpu_util import make_runner
    runner = make_runner(folder, "float32", page_size=8, cache_tokens=128, max_seqs=2,
                         max_batch_tokens=128, max_model_len=128)
    seq = prompts[3] + batch[3]
    z = runner.step([StepEntry("s", seq, list(range(len(seq))))])
    for i, tok in enumerate(batch[3]):
        assert tok == P.sample(z[len(prompts[3]) - 1 + i], uniform(7, i), temperature=0.8)


def test_top_k_top_p_and_penalty_rows(tiny_folders):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    folder = tiny_folders[("A", "float32")]
    prompt = random_tokens(512, 9, 5)
    eng = Engine(folder, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=32,
                 max_batch_seqs=4, prefill_chunk_size=8, max_seq_len=64)
    greedy = eng.generate([prompt], SamplingParams(max_tokens=6, temperature=0.0))[0]
    k1 = eng.generate([prompt], SamplingParams(max_tokens=6, temperature=1.0, top_k=1, seed=3))[0]
    assert k1 == greedy                                     # top-1 sampling is greedy
    p_small = eng.generate([prompt], SamplingParams(max_tokens=6, temperature=1.0, top_p=1e-6, seed=3))[0]
    assert p_small == greedy
    pen = eng.generate([prompt], SamplingParams(max_tokens=6, temperature=0.0, repetition_penalty=50.0))[0]
    assert len(set(pen) | set(prompt)) == len(pen) + len(set(prompt))     # nothing is repeated
    stop = eng.generate([prompt], SamplingParams(max_tokens=6, temperature=0.0, stop_tokens=[greedy[-1]]))[0]
    assert stop == greedy[:greedy.index(greedy[-1]) + 1]
    # all of them together: the same tokens alone and beside other requests, and each token is what
    # the host implementation draws from logits of the same position
    from zse_amd.engine.runner import StepEntry
    from zse_amd.sampling import sample_host, uniform
    mixed = SamplingParams(max_tokens=10, temperature=0.8, top_k=7, top_p=0.85, repetition_penalty=1.3, seed=11)
    alone = eng.generate([prompt], mixed)[0]
    others = [random_tokens(512, n, 30 + n) for n in (3, 14)]
    batch = eng.generate([others[0], prompt, others[1]],
                         [SamplingParams(max_tokens=10, temperature=0.0), mixed,
                          SamplingParams(max_tokens=10, temperature=1.2, top_p=0.5, seed=2)])
    assert batch[1] == alone
    eng.close()
    from gpu_util import make_runner
    runner = make_runner(folder, "float32", page_size=4, cache_tokens=64, max_seqs=2, max_batch_tokens=64,
                         max_model_len=64)
    seq = prompt + alone
    z = runner.step([StepEntry("s", seq, list(range(len(seq))))])
    for i, tok in enumerate(alone):
        # the penalty grows with how often a token was produced; prompt tokens count once
        counts = {t: 1 for t in prompt}
        for t in alone[:i]:
            counts[t] = counts.get(t, 0) + 1
        assert tok == sample_host(z[len(prompt) - 1 + i], mixed, uniform(11, i), counts)


@pytest.mark.parametrize("seed", [0, 1])
def test_a_crowd_of_mixed_requests_each_gets_what_it_gets_alone(tiny_folders, seed):
    """Two dozen requests of random lengths and every manner of sampling, five places, so few
    pages that some are recomputed, runs of decode steps on: every request ends with the tokens
    and the reason it ends with when it has the engine to itself."""
    import random
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY["B"][0]
    folder = tiny_folders[("B", "float32")]
    rnd = random.Random(seed)
    V = cfg["vocab_size"]
    prompts, params = [], []
    for i in range(24):
        prompts.append(random_tokens(V, rnd.randint(1, 45), 500 + 31 * seed + i))
        kind = rnd.choice(["greedy", "temp", "topk", "topp", "both", "penalty"])
        kw = dict(max_tokens=rnd.randint(1, 20), seed=100 + i)
        if kind == "greedy":
            kw.update(temperature=0.0)
        elif kind == "temp":
            kw.update(temperature=0.9)
        elif kind == "topk":
            kw.update(temperature=1.1, top_k=rnd.choice([1, 3, 40]))
        elif kind == "topp":
            kw.update(temperature=0.7, top_p=rnd.choice([0.3, 0.9]))
        elif kind == "both":
            kw.update(temperature=1.0, top_k=20, top_p=0.8)
        else:
            kw.update(temperature=rnd.choice([0.0, 0.8]), repetition_penalty=1.4)
        if rnd.random() < 0.4:
            kw.update(stop_tokens=[rnd.randrange(V) for _ in range(40)])
        params.append(SamplingParams(**kw))

    def run(which, seqs, blocks):
        eng = Engine(folder, dtype="float32", block_size=8, num_blocks=blocks, max_batch_tokens=48,
                     max_batch_seqs=seqs, prefill_chunk_size=11, max_seq_len=128, decode_run=4)
        reqs = [eng.add_request(prompts[i], params[i]) for i in which]
        eng.run()
        out = [(list(r.output_tokens), r.finish_reason) for r in reqs]
        st = eng.stats()
        assert all(pool.free_pages == pool.num_pages for pool in eng.runner.manager.pools)
        eng.close()
        return out, st

    crowd, st = run(range(24), 5, 14)        # 14 pages of 8: the longest request alone needs 9
    assert st.preemptions > 0, "the pool was meant to be too small for five long requests"
    roomy = Engine(folder, dtype="float32", block_size=8, num_blocks=64, max_batch_tokens=48, max_batch_seqs=1,
                   prefill_chunk_size=16, max_seq_len=128, decode_run=1)
    for i in range(24):
        r = roomy.add_request(prompts[i], params[i])
        roomy.run()
        assert (list(r.output_tokens), r.finish_reason) == crowd[i], (i, params[i])
    roomy.close()


def test_zse_generate_command(tiny_folders, tmp_path):
    from zse_amd.engine.engine import Engine
    cfg = TINY["A"][0]
    folder = tiny_folders[("A", "float32")]
    w = read_weights(folder)
    prompts = [random_tokens(512, n, 90 + n) for n in (6, 13)]
    f = tmp_path / "prompts.txt"
    f.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    p = subprocess.run([sys.executable, "-m", "zse_amd", "generate", folder, "--prompt-ids-file", str(f),
                        "--max-tokens", "5", "--temperature", "0", "--dtype", "float32",
                        "--block-size", "4", "--num-blocks", "64", "--prefill-chunk-size", "4",
                        "--max-seq-len", "64", "--quiet"],
                       capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [list(map(int, l.split())) for l in p.stdout.strip().split("\n")]
    assert lines == [plain_greedy(cfg, w, q, 5) for q in prompts]


def test_bfloat16_generation_with_preemption_and_runs_of_steps(tiny_folders):
    """bfloat16 through the whole engine under pressure: so few pages that requests are
    preempted and computed again, and four steps in a row before the host reads an id.  A
    request's tokens equal those of its run alone wherever the plain implementation's two
    best logits lie further apart than bfloat16's error can bridge (0.05; the largest logit
    error seen is a third of that); at a nearer tie either may be chosen, and the comparison
    goes on from the token the engine took."""
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY["B"][0]
    folder = tiny_folders[("B", "bfloat16")]
    w = read_weights(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 90 + n) for n in (3, 9, 14, 6, 21)]
    sp = SamplingParams(max_tokens=24, temperature=0.0)

    def run(ps, num_blocks, decode_run, seqs):
        eng = Engine(folder, dtype="bfloat16", block_size=8, num_blocks=num_blocks, max_batch_tokens=32,
                     max_batch_seqs=seqs, prefill_chunk_size=7, max_seq_len=128, decode_run=decode_run)
        out = eng.generate(ps, sp)
        st = eng.stats()
        assert all(pool.free_pages == pool.num_pages for pool in eng.runner.manager.pools)
        eng.close()
        return out, st

    alone = [run([p], 64, 1, 1)[0][0] for p in prompts]
    crowd, st = run(prompts, 10, 4, 4)
    assert st.preemptions > 0
    checked = 0
    for p, a, c in zip(prompts, alone, crowd):
        assert len(a) == len(c) == 24
        for i in range(24):
            if a[i] == c[i]:
                checked += 1
                continue
            z = np.sort(P.forward(cfg, w, list(p) + c[:i], np.float64)[-1])
            assert z[-1] - z[-2] < 0.05, f"prompt {p}: token {i} differs at a margin of {z[-1] - z[-2]:.3f}"
            break                      # the two runs follow different tokens from here on
    assert checked > 24 * len(prompts) * 0.8


def test_zse_generate_with_random_weights_made_on_the_device(tmp_path):
    """``zse generate --random-weights`` needs a folder with a config.json only; the weights it
    draws on the device are those ``write_random_model`` writes for the same seed."""
    import json
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    from zse_amd.weights import write_random_model
    cfg = TINY["A"][0]
    bare = tmp_path / "bare"
    bare.mkdir()
    (bare / "config.json").write_text(json.dumps(cfg))
    prompt = random_tokens(512, 9, 77)
    p = subprocess.run([sys.executable, "-m", "zse_amd", "generate", str(bare), "--random-weights", "--weight-seed", "3",
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0",
                        "--dtype", "float32", "--block-size", "4", "--num-blocks", "32", "--max-seq-len", "64", "-q"],
                       capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    got = list(map(int, p.stdout.split()))
    folder = write_random_model(str(tmp_path / "written"), cfg, seed=3, dtype="float32")
    eng = Engine(folder, dtype="float32", block_size=4, num_blocks=32, max_seq_len=64)
    assert got == eng.generate([prompt], SamplingParams(max_tokens=6, temperature=0.0))[0]
    eng.close()


def test_the_windowed_group_gets_a_pool_of_its_own_size(tiny_folders):
    """Sliding layers never hold more than their window and one step's tokens per request, so
    the engine gives their group a small pool; requests far longer than the window run on it
    (pages are handed back as the window passes them) and give the plain implementation's tokens."""
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY["A"][0]                                   # window 8
    folder = tiny_folders[("A", "float32")]
    w = read_weights(folder)
    eng = Engine(folder, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=32, max_batch_seqs=2,
                 prefill_chunk_size=4, max_seq_len=128)
    m = eng.runner.manager
    assert [g.window for g in m.groups] == [8, None]
    assert [p.num_pages for p in m.pools] == [2 * (-(-(8 + 4) // 4) + 2), 64]       # 10 pages against 64
    prompts = [random_tokens(512, n, 300 + n) for n in (41, 33)]
    got = eng.generate(prompts, SamplingParams(max_tokens=20, temperature=0.0))
    st = eng.stats()
    assert st.preemptions == 0 and st.peak_pages[0] <= 10 and st.peak_pages[1] >= 2 * 13
    assert len(st.ttft_ms) == 2 and all(t > 0 for t in st.ttft_ms) and all(t > 0 for t in st.tpot_ms)
    assert set(st.by_kind) <= {"prefill", "mixed", "decode"} and sum(v[0] for v in st.by_kind.values()) == st.steps
    for p, g in zip(prompts, got):
        assert g == plain_greedy(cfg, w, p, 20)
    eng.close()


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_fed_on_the_device_to_any_entries_of_a_step(tiny_folders, dtype, graphs):
    """A step takes the tokens of some of its entries from the ids the step before left on the
    device, whatever the order of the entries, beside a portion of a prompt that brings its
    own tokens: the same logits, to the bit, as when the host brings those tokens."""
    from gpu_util import make_runner
    from zse_amd.engine.runner import StepEntry
    from zse_amd.sampling import DeviceSampler, SamplingParams
    cfg = TINY["A"][0]
    folder = tiny_folders[("A", dtype)]
    V = cfg["vocab_size"]
    prompts = {r: random_tokens(V, n, 30 + n) for r, n in (("a", 9), ("b", 4), ("c", 13), ("d", 21))}

    def run(on_device):
        runner = make_runner(folder, dtype, max_seqs=8, use_graphs=graphs)
        sampler = DeviceSampler(runner.rt, runner.k, 8)
        greedy = [{"params": SamplingParams(temperature=0.0), "u": 0.0} for _ in range(3)]
        logits = runner.step([StepEntry(r, prompts[r], [len(prompts[r]) - 1]) for r in "abc"], download=False)
        ids = sampler.sample_staged(logits, sampler.stage(greedy, V))
        host = ids.result()
        out = []
        # b and a decode in another order than they were sampled in, c sits the step out, d arrives with a portion
        entries = [StepEntry("d", prompts["d"][:12], []), StepEntry("b", [0 if on_device else host[1]], [0]),
                   StepEntry("a", [0 if on_device else host[0]], [0])]
        if on_device:
            out.append(runner.step(entries, tokens_from=ids.device_ptr, feed=[-1, 1, 0]))
        else:
            out.append(runner.step(entries))
        # and a step of single tokens through a graph or a launch list, fed in another order again
        logits = runner.step([StepEntry("a", [5], [0]), StepEntry("b", [6], [0]), StepEntry("c", [host[2]], [0])], download=False)
        ids = sampler.sample_staged(logits, sampler.stage(greedy, V))
        host = ids.result()
        entries = [StepEntry("c", [0 if on_device else host[2]], [0]), StepEntry("a", [0 if on_device else host[0]], [0]),
                   StepEntry("d", prompts["d"][12:14], [1])]
        out.append(runner.step(entries, tokens_from=ids.device_ptr, feed=[2, 0, -1]) if on_device else runner.step(entries))
        entries = [StepEntry(r, [7], [0]) for r in "cab"]
        logits = runner.step(entries, download=False)
        ids = sampler.sample_staged(logits, sampler.stage(greedy, V))
        host = ids.result()
        entries = [StepEntry("b", [0 if on_device else host[2]], [0]), StepEntry("c", [0 if on_device else host[0]], [0])]
        out.append(runner.step(entries, tokens_from=ids.device_ptr, feed=[2, 0]) if on_device else runner.step(entries))
        runner.close()
        return out

    for got, want in zip(run(True), run(False)):
        assert got.shape == want.shape and np.array_equal(got, want)
    with pytest.raises(ValueError):
        runner = make_runner(folder, dtype, max_seqs=8)
        try:
            runner.step([StepEntry("a", [1, 2], [1])], tokens_from=1, feed=[0])
        finally:
            runner.close()


def test_a_stream_of_tokens_never_shows_a_placeholder(tiny_folders):
    """``stream_generate_tokens`` and ``step`` hand out tokens the host has seen; ``run`` reads the
    ids some steps behind the steps it enqueues and ends with the same outputs."""
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY["B"][0]
    folder = tiny_folders[("B", "float32")]
    prompts = [random_tokens(cfg["vocab_size"], n, 170 + n) for n in (5, 12, 3)]
    eng = Engine(folder, dtype="float32", block_size=8, max_batch_tokens=32, max_batch_seqs=4, prefill_chunk_size=7,
                 max_seq_len=128, decode_run=4)
    kw = dict(max_tokens=19, temperature=0.8, top_k=20, seed=5)
    streamed = list(eng.stream_generate_tokens(prompts[0], **kw))
    assert len(streamed) == 19 and all(0 <= t < cfg["vocab_size"] for t in streamed)
    assert eng.generate([prompts[0]], SamplingParams(**kw))[0] == streamed
    params = [SamplingParams(max_tokens=m, temperature=t, seed=9 + i) for i, (m, t) in enumerate(((15, 0.0), (9, 1.1), (22, 0.7)))]
    by_run = eng.generate(prompts, params)
    reqs = [eng.add_request(p, sp) for p, sp in zip(prompts, params)]
    while eng.scheduler.has_work():
        eng.step()
        assert all(-1 not in r.output_tokens for r in reqs)
    assert [list(r.output_tokens) for r in reqs] == by_run
    eng.close()
