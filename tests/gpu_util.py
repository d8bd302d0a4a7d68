"""Helpers shared by the GPU tests: loading tiny models, replaying traces, the plain logits."""
import numpy as np

from conftest import TINY, read_weights
from plain import gemma2_plain as P

# Tolerances.  float32: the engine and the plain float64 run differ by summation order
# only; a few 1e-6 is seen, 5e-5 leaves room for long sums.  bfloat16: inputs of every
# product are rounded to 8 bits of mantissa; the error is bounded relative to the
# largest logit.
F32_ATOL = 5e-5
BF16_REL = 0.02


def plain_logits(name, folder, tokens, embed_scale=None):
    cfg = TINY[name][0]
    return P.forward(cfg, read_weights(folder), tokens, np.float64, embed_scale=embed_scale)


def bf16_round(x):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    return float(bf16_bits_to_f32(f32_to_bf16_bits(np.array([x], np.float32)))[0])


def reference_for(name, dtype, folder, tokens):
    """Plain float64 logits with the embedding scale the engine uses for this dtype."""
    H = TINY[name][0]["hidden_size"]
    scale = np.float64(np.float32(np.sqrt(H)))
    if dtype == "bfloat16":
        scale = np.float64(bf16_round(np.sqrt(H)))
    return plain_logits(name, folder, tokens, embed_scale=scale)


def assert_close(got, want, dtype, what=""):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    err = np.abs(got - want)
    tol = F32_ATOL if dtype == "float32" else BF16_REL * np.abs(want).max()
    if not (err.max() <= tol):
        i = np.unravel_index(np.argmax(err), err.shape)
        first_bad = int(np.argmax((err > tol).any(axis=-1))) if err.ndim == 2 else -1
        raise AssertionError(f"{what}: max error {err.max():.3e} > {tol:.3e} at {i}; "
                             f"first wrong row {first_bad}")


def make_runner(folder, dtype, **kw):
    from zse_amd.engine.loading import load_model
    from zse_amd.engine.runner import StepRunner
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    model = load_model(folder, dtype, rt, tuned=kw.pop("tuned", True))
    kw.setdefault("use_graphs", False)
    return StepRunner(model, rt, dtype, **kw)


def run_steps(runner, streams, steps, observe=None):
    """``streams``: {req: tokens}; ``steps``: list of (entries, ends) with entries a list
    of (req, n).  Feeds each request's next n tokens, wants every logit.  Returns
    {req: [rows in position order]}.  ``observe(step index)`` is called after each step
    has run, before the requests it ends give their pages back."""
    from zse_amd.engine.runner import StepEntry
    fed = {r: 0 for r in streams}
    rows = {r: [] for r in streams}
    for step_index, (entries, ends) in enumerate(steps):
        es = []
        for r, n in entries:
            es.append(StepEntry(r, streams[r][fed[r]:fed[r] + n], list(range(n))))
        z = runner.step(es)
        at = 0
        for r, n in entries:
            rows[r].extend(z[at:at + n])
            at += n
            fed[r] += n
        if observe is not None:
            observe(step_index)
        for r in ends:
            runner.finish(r)
        runner.manager.check()
    return {r: np.stack(v) for r, v in rows.items() if v}


def whole_steps(streams):
    return [([(r, len(t))], [r]) for r, t in streams.items()]


def tail_decode_steps(streams, tail=32):
    steps = []
    for r, t in streams.items():
        head = max(len(t) - tail, 0)
        if head:
            steps.append(([(r, head)], []))
        for i in range(head, len(t)):
            steps.append(([(r, 1)], [r] if i == len(t) - 1 else []))
    return steps


def chunked_steps(streams, sizes=(7, 2, 5, 3, 2, 11, 2, 4)):
    steps = []
    for r, t in streams.items():
        i, k = 0, 0
        while i < len(t):
            n = min(sizes[k % len(sizes)], len(t) - i)
            i += n
            k += 1
            steps.append(([(r, n)], [r] if i == len(t) else []))
    return steps


def mixed_steps(streams, seed=0, max_live=4, decode_tail=12, chunk_choices=(2, 3, 5, 9), room=None, page=1,
                skip=0.15):
    """Up to ``max_live`` requests at a time: prompt portions of some beside single
    tokens of others (a request decodes one by one over its last ``decode_tail``
    tokens, or ``decode_tail[request]`` where a mapping is given); requests enter as others leave; some sit a step out (each with probability
    ``skip``).  ``room``: pages of
    ``page`` tokens the pool has; a request enters only while the live requests, each at
    its full length, and it fit together."""
    rng = np.random.default_rng(seed)
    waiting = list(streams)
    live, fed = [], {}
    steps = []
    pages_of = lambda r: -(-len(streams[r]) // page)
    while waiting or live:
        while waiting and len(live) < max_live:
            if room is not None and sum(pages_of(r) for r in live) + pages_of(waiting[0]) > room:
                break
            r = waiting.pop(0)
            live.append(r)
            fed[r] = 0
        entries, ends = [], []
        for r in list(live):
            if len(live) > 1 and rng.random() < skip:
                continue                                  # left out of this step
            left = len(streams[r]) - fed[r]
            tail = decode_tail[r] if isinstance(decode_tail, dict) else decode_tail
            n = 1 if left <= tail else min(int(rng.choice(chunk_choices)), left - tail)
            entries.append((r, n))
            fed[r] += n
            if fed[r] == len(streams[r]):
                ends.append(r)
                live.remove(r)
        if entries:
            steps.append((entries, ends))
    return steps
