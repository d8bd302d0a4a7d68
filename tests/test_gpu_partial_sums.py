"""A product that splits K may leave the adding up of its partial sums to the norm kernel that
reads them.  That is a matter between a block and the part it calls: the bits are the same as
with the product's own joining kernel, and a part called by another part never does it."""
import dataclasses

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# wide enough for the 17..64-row product to split K (N = 512 gives 8 column blocks)
CFG = dict(architectures=["Gemma2ForCausalLM"], model_type="gemma2", num_hidden_layers=2, hidden_size=512,
           num_attention_heads=4, num_key_value_heads=2, head_dim=64, query_pre_attn_scalar=64,
           intermediate_size=1024, vocab_size=320, rope_theta=10000.0, sliding_window=24,
           attn_logit_softcapping=50.0, final_logit_softcapping=30.0, rms_norm_eps=1e-6,
           max_position_embeddings=256)


@pytest.fixture(scope="module")
def rt():
    from zse_amd.runtime.device import Runtime
    return Runtime.get()


def logits_of(rt, model, tokens, seen_parts):
    """The last position's logits of one 40-token step; the numbers of partial-sum planes the
    joining kernel was handed go to ``seen_parts``."""
    from zse_amd.engine.runner import StepEntry, StepRunner
    runner = StepRunner(model, rt, "bfloat16", page_size=16, cache_tokens=256, max_seqs=2, max_batch_tokens=64,
                        use_graphs=False)
    k = runner.k
    real = k.zk_norm_add_norm

    def spy(sub, parts, *rest):
        seen_parts.append(parts)
        return real(sub, parts, *rest)

    k.zk_norm_add_norm = spy
    try:
        out = runner.step([StepEntry("a", tokens, [len(tokens) - 1])])
    finally:
        k.zk_norm_add_norm = real
    runner.finish("a")
    return np.array(out, np.float32)


def test_the_norm_kernel_adds_partial_sums_to_the_same_bits(rt, monkeypatch):
    from zse_amd.engine.loading import random_model
    from zse_amd.parts.block import Block
    model = random_model(CFG, "bfloat16", seed=3, std=0.05, rt=rt)
    tokens = np.random.default_rng(0).integers(0, CFG["vocab_size"], 40).tolist()
    handed = []
    got = logits_of(rt, model, tokens, handed)
    assert max(handed) > 1, "the 40-row products of these widths should have split K"
    monkeypatch.setattr(Block, "_joins_sums", staticmethod(lambda post: False))
    joined = []
    want = logits_of(rt, model, tokens, joined)
    assert max(joined) == 0
    assert np.array_equal(got, want)


def test_a_part_called_by_another_part_hands_over_whole_results(rt):
    from zse_amd.config import Architecture, register_architecture, unregister_architecture
    from zse_amd.engine.loading import random_model
    from zse_amd.models.gemma2 import Gemma2Config, gemma2_plan
    from zse_amd.parts import Part, build_part, register_part, unregister_part

    @dataclasses.dataclass(frozen=True)
    class WrapSpec:
        inner: object
        kind: str = "toy_wrap"

    class WrapFFN(Part):
        """Passes its input to the framework's feed-forward and its result on."""
        seen = []

        def __init__(self, spec):
            self.spec = spec
            self.inner = build_part("ffn", spec.inner)

        def children(self):
            return [self.inner]

        def forward(self, ctx, x):
            y = self.inner.forward(ctx, x)
            WrapFFN.seen.append(y.layout)
            return y

    def plan_of(cfg):
        plan = gemma2_plan(cfg)
        return dataclasses.replace(plan, layers=tuple(dataclasses.replace(b, ffn=WrapSpec(b.ffn)) for b in plan.layers))

    register_part("ffn", "toy_wrap", WrapFFN)
    register_architecture(Architecture("ToyWrapLM", Gemma2Config.from_dict, plan_of))
    try:
        tokens = np.random.default_rng(1).integers(0, CFG["vocab_size"], 40).tolist()
        wrapped = random_model(dict(CFG, architectures=["ToyWrapLM"], model_type="toy"), "bfloat16", seed=3, std=0.05, rt=rt)
        a_parts, b_parts = [], []
        got = logits_of(rt, wrapped, tokens, a_parts)
        assert WrapFFN.seen and set(WrapFFN.seen) == {"rows"}
        plain_model = random_model(CFG, "bfloat16", seed=3, std=0.05, rt=rt)
        want = logits_of(rt, plain_model, tokens, b_parts)
        assert max(a_parts) == 0 and max(b_parts) > 1      # only the part the block itself calls hands sums over
        assert np.array_equal(got, want)
    finally:
        unregister_part("ffn", "toy_wrap")
        unregister_architecture("ToyWrapLM")
