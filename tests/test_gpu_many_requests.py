"""Steps of 17 to 64 live requests, through the step function and through the engine, in
32-bit and in bfloat16: what the model-level tests with up to eight requests do not reach.
Decode steps of 9 to 16 requests replay the graph of bucket 16; larger ones are launched from
their written-down lists; the product kernel for 17 to 64 rows is fed by as many different
requests; keys and values of decoded tokens of different requests are stored side by side;
prompt portions of newcomers run beside dozens of decoded tokens; pools are small enough that
pages pass from request to request and, in the engine, that requests are preempted."""
import numpy as np
import pytest

from conftest import TINY, random_tokens, read_weights
from gpu_util import assert_close, make_runner, mixed_steps, reference_for, run_steps
from plain import gemma2_plain as P

pytestmark = pytest.mark.gpu

PAGE = {"A": 4, "B": 8}


def crowd_streams(name, n, lo, hi, seed):
    V = TINY[name][0]["vocab_size"]
    rng = np.random.default_rng(seed)
    return {f"q{i}": random_tokens(V, int(l), 1000 * seed + i) for i, l in enumerate(rng.integers(lo, hi, n))}


def lockstep_steps(streams, tails, per_step=16):
    """Prompts first, ``per_step`` requests a step, each without its last ``tails[r]`` tokens;
    then every live request brings one token a step until its tokens are used up."""
    names = list(streams)
    steps = []
    for i in range(0, len(names), per_step):
        steps.append(([(r, len(streams[r]) - tails[r]) for r in names[i:i + per_step]], []))
    left = dict(tails)
    while left:
        entries = [(r, 1) for r in left]
        ends = [r for r in left if left[r] == 1]
        steps.append((entries, ends))
        left = {r: n - 1 for r, n in left.items() if n > 1}
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_of_up_to_64_requests_against_the_plain_implementation(tiny_folders, name, dtype):
    folder = tiny_folders[(name, dtype)]
    page = PAGE[name]
    pages_of = lambda t: -(-len(t) // page)
    crowd = crowd_streams(name, 88, 16, 75, 7)
    together = {f"t{r}": t for r, t in crowd_streams(name, 64, 12, 60, 8).items()}
    rng = np.random.default_rng(3)
    crowd_tails = {r: int(min(len(t) - 2, rng.integers(6, 44))) for r, t in crowd.items()}
    together_tails = {r: int(min(len(t) - 2, rng.integers(3, 34))) for r, t in together.items()}
    # room for the 48 longest of the crowd: fewer pages than its 64 places could fill
    room = max(sum(sorted((pages_of(t) for t in crowd.values()), reverse=True)[:48]),
               sum(pages_of(t) for t in together.values()))
    runner = make_runner(folder, dtype, page_size=page, num_pages=room, max_seqs=64, max_batch_tokens=640,
                         max_model_len=256, use_graphs=True)
    assert runner.graph_max_batch == 16 and runner.use_steplists

    # 1. everybody decodes together: steps of 64 single tokens, then fewer and fewer
    steps = lockstep_steps(together, together_tails)
    sizes = [len(e) for e, _ in steps if all(n == 1 for _, n in e)]
    assert sizes[0] == 64 and sum(1 for s in sizes if 33 <= s <= 64) >= 3
    assert sum(1 for s in sizes if 17 <= s <= 32) >= 3 and sum(1 for s in sizes if 9 <= s <= 16) >= 3
    rows = run_steps(runner, together, steps)
    for r, t in together.items():
        assert_close(rows[r], reference_for(name, dtype, folder, t), dtype, f"together {r}")
    if runner.use_graphs:
        captured = {k[0] for k, g in runner.graphs.items() if isinstance(g, int)}
        assert 16 in captured and not any(b > 16 for b in captured), captured
    lists_before = runner.steplist_runs
    assert lists_before > 0, "no step of more than 16 requests ran from its written-down list"
    assert all(p.free_pages == p.num_pages for p in runner.manager.pools)

    # 2. a crowd: newcomers' prompt portions beside dozens of decoded tokens, pages handed on
    steps = mixed_steps(crowd, seed=3, max_live=64, decode_tail=crowd_tails, chunk_choices=(2, 3, 5, 9, 17),
                        room=room, page=page, skip=0.0)
    assert max(len(e) for e, _ in steps) >= 56
    assert any(sum(1 for _, n in e if n == 1) >= 40 and any(n > 1 for _, n in e) and sum(n for _, n in e) >= 64
               for e, _ in steps)
    rows = run_steps(runner, crowd, steps)
    for r, t in crowd.items():
        assert_close(rows[r], reference_for(name, dtype, folder, t), dtype, f"crowd {r}")
    assert all(p.free_pages == p.num_pages for p in runner.manager.pools)
    runner.close()


def plain_greedy(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(P.forward(cfg, w, toks, np.float64)[-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,seqs", [("A", 24), ("B", 64)])
def test_the_engine_with_24_and_64_places(tiny_folders, name, seqs, dtype):
    """More requests than places, every manner of sampling, stop tokens that are met in the
    middle of runs of four decode steps, so few pages that requests are computed again: every
    request gets the tokens it gets when it has an engine to itself (32-bit: equal; bfloat16:
    equal up to the first token at which the plain implementation's two best logits lie
    nearer than bfloat16's error can tell apart), and greedy requests those of the plain
    implementation."""
    import random
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling import SamplingParams
    cfg = TINY[name][0]
    folder = tiny_folders[(name, dtype)]
    w = read_weights(folder)
    V, page = cfg["vocab_size"], PAGE[name]
    rnd = random.Random(seqs)
    n_req = seqs + 24
    prompts, params = [], []
    for i in range(n_req):
        prompts.append(random_tokens(V, rnd.randint(1, 40), 7000 + i))
        # the last to arrive produce the most: they are still decoding, many at a time, when the
        # queue is empty and nothing but single tokens is left to run
        kw = dict(max_tokens=rnd.randint(2, 26) if i < 24 else rnd.randint(16, 30), seed=300 + i)
        if dtype == "bfloat16" or name == "A" or i % 3 == 0:
            # bfloat16: greedy only, so that a tie can be told; the 24 places: greedy only, so that
            # decode steps follow each other without the host (ids fed from step to step on the device)
            kw.update(temperature=0.0)
        elif i % 3 == 1:
            kw.update(temperature=0.9)
        else:
            kw.update(temperature=1.0, top_k=12, top_p=0.9)
        params.append(SamplingParams(**kw))

    def engine(places, blocks, decode_run):
        return Engine(folder, dtype=dtype, block_size=page, num_blocks=blocks, max_batch_tokens=256,
                      max_batch_seqs=places, prefill_chunk_size=11, max_seq_len=128, decode_run=decode_run)

    # alone: one place, one request after the other
    alone = []
    eng = engine(1, 64, 1)
    for p, sp in zip(prompts, params):
        r = eng.add_request(p, sp)
        eng.run()
        alone.append(list(r.output_tokens))
    eng.close()
    # stop tokens: for every fourth request the token in the middle of its own output
    for i in range(0, n_req, 4):
        if len(alone[i]) >= 4:
            params[i] = SamplingParams(**{**params[i].__dict__, "stop_tokens": [alone[i][len(alone[i]) // 2]]})
            alone[i] = alone[i][:alone[i].index(params[i].stop_tokens[0]) + 1]

    longest = max(len(p) + sp.max_tokens for p, sp in zip(prompts, params))
    full = sorted(-(-(len(p) + sp.max_tokens) // page) for p, sp in zip(prompts, params))
    # about half of what the requests in all places would hold at their ends
    blocks = max(-(-longest // page) + 1, int(0.5 * seqs * sum(full) / len(full)))
    eng = engine(seqs, blocks, 4)
    reqs = [eng.add_request(p, sp) for p, sp in zip(prompts, params)]
    most = 0
    while eng.scheduler.has_work():
        eng.step()
        most = max(most, len(eng.scheduler.running))
    st = eng.stats()
    assert most > 16 and most >= seqs * 5 // 8, most
    assert st.preemptions > 0, "the pool was meant to be too small"
    assert all(pool.free_pages == pool.num_pages for pool in eng.runner.manager.pools)
    # and a full house in lockstep: as many short prompts as there are places, all admitted in one
    # step, all greedy, all as long: every decode step brings one token of each, more than a
    # graph takes, so runs of four steps are launched from one written-down list, the ids fed
    # from step to step on the device
    lists0 = eng.runner.steplist_runs
    short = [random_tokens(V, 3, 9000 + i) for i in range(seqs)]
    together = eng.generate(short, SamplingParams(max_tokens=10, temperature=0.0))
    assert eng.runner.steplist_runs - lists0 >= 6, "decode steps of a full house did not run from their list"
    eng.close()
    eng = engine(1, 64, 1)
    for p, got in list(zip(short, together))[::5]:
        a = eng.generate([p], SamplingParams(max_tokens=10, temperature=0.0))[0]
        if dtype == "float32":
            assert got == a
        else:
            same_upto = next((j for j in range(10) if a[j] != got[j]), 10)
            if same_upto < 10:
                z = np.sort(P.forward(cfg, w, list(p) + got[:same_upto], np.float64)[-1])
                assert z[-1] - z[-2] < 0.05
    eng.close()

    same = 0
    for i, (r, a) in enumerate(zip(reqs, alone)):
        got = list(r.output_tokens)
        if dtype == "float32":
            assert got == a, (i, params[i])
            if params[i].temperature == 0.0 and not params[i].stop_tokens and i % 6 == 0:
                assert got == plain_greedy(cfg, w, prompts[i], len(got)), i
            continue
        for j in range(max(len(a), len(got))):
            if j < len(a) and j < len(got) and a[j] == got[j]:
                same += 1
                continue
            upto = min(j, len(got), len(a))
            z = np.sort(P.forward(cfg, w, list(prompts[i]) + got[:upto], np.float64)[-1])
            assert z[-1] - z[-2] < 0.05, f"request {i}: token {j} differs at a margin of {z[-1] - z[-2]:.3f}"
            break
    if dtype == "bfloat16":
        assert same > 0.8 * sum(len(a) for a in alone)
