"""The kernels at the widths they are tuned for.  The tiny configurations of the other tests never reach the sizes
at which a kernel changes its shape (128-row attention tiles with 8-wave blocks, products with two column tiles per
block, weight copies of many chunks, key parts).  Here two layers of the benchmark's widths (for instance hidden 4096,
32 query and 8 key/value heads of 128, intermediate 12288) with a vocabulary that is no multiple of 16 run the same steps in
bfloat16 and in true float32 on the same weights (the bfloat16 values widened exactly); the float32 path is the one
that the other tests pin to the plain implementation."""
import pytest
import torch

from tests.gpu_util import require_gpu

pytestmark = pytest.mark.gpu

RAW = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=2, hidden_size=4096,
           num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=4099,
           rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=4096,
           bos_token_id=1, eos_token_id=2)


#: (hidden, query heads, key/value heads, head size, intermediate): the 8B and 14B widths of the benchmark, and one
#: with heads of 64 in groups of 8
WIDTHS = [(4096, 32, 8, 128, 12288), (5120, 40, 8, 128, 17408), (2048, 32, 4, 64, 6144)]


def _runners(dev, requests, pages, widths):
    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.runner import ModelRunner
    from spyinfer_amd.weights.random_init import random_tensors_on_device
    raw = dict(RAW, hidden_size=widths[0], num_attention_heads=widths[1], num_key_value_heads=widths[2], head_dim=widths[3],
               intermediate_size=widths[4])
    arch = architecture_of(raw)
    cfg = arch.config_cls.from_dict(raw)
    out = []
    w16 = None
    for dtype in ("bfloat16", "float32"):
        model = arch.build(cfg)
        if w16 is None:
            w16 = random_tensors_on_device(model.weight_specs(), 5, torch.bfloat16, dev, norm_std=0.05)
        weights = w16 if dtype == "bfloat16" else {k: (v.float() if v.dtype == torch.bfloat16 else v) for k, v in w16.items()}
        model.bind(weights, dev)
        out.append(ModelRunner(model, dtype, dev, 16, pages, requests, enforce_eager=True, max_model_len=1024))
    return out


def _close(a, b, what):
    """bfloat16 against float32 logits: the tolerance of the other bfloat16 tests, and the same first choice wherever
    the float32 logits do not nearly tie."""
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape
    err = (a - b).abs()
    assert torch.all(err <= 8e-2 + 2e-2 * b.abs()), "%s: bfloat16 and float32 differ by %g (logits up to %g)" % (what, err.max(), b.abs().max())
    top = torch.topk(b, 2, dim=-1).values
    clear = (top[:, 0] - top[:, 1]) > 0.2
    assert torch.equal(a.argmax(-1)[clear], b.argmax(-1)[clear]), what + ": another first choice"


@pytest.mark.parametrize("widths", WIDTHS)
def test_steps_at_real_widths(widths):
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    R = 44
    r16, r32 = _runners(dev, R, 220, widths)
    g = torch.Generator().manual_seed(9)
    lens = [300, 170] + [3 + (5 * i) % 38 for i in range(R - 2)]
    prompts = [torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist() for n in lens]
    folded = [0]
    real = ops.decode_linear_residual
    ops.decode_linear_residual = lambda *a, **k: (folded.__setitem__(0, folded[0] + 1), real(*a, **k))[1]
    try:
        caches = []
        for runner in (r16, r32):
            cs = [runner.manager.admit(i) for i in range(R)]
            for c, p in zip(cs, prompts):
                runner.manager.reserve(c, len(p))
            caches.append(cs)
        # the prompts in one step: two entries with 128-row tiles beside short ones; logits at the last place of each
        outs = [runner.step([StepEntry(c, p, [len(p) - 1]) for c, p in zip(cs, prompts)]) for runner, cs in zip((r16, r32), caches)]
        _close(outs[0], outs[1], "prompts")
        assert folded[0] == 0
        # three steps of all 44 requests (three row tiles), then of the first 9 (one row tile), then of one
        for live, steps in ((R, 3), (9, 3), (1, 2)):
            for s in range(steps):
                toks = torch.randint(0, RAW["vocab_size"], (live,), generator=g).tolist()
                outs = []
                for runner, cs in zip((r16, r32), caches):
                    for c in cs[:live]:
                        runner.manager.reserve(c, 1)
                    outs.append(runner.step([StepEntry(c, [t], [0]) for c, t in zip(cs[:live], toks)]))
                _close(outs[0], outs[1], "%d requests, step %d" % (live, s))
        assert folded[0] == 8 * 2 * 2, "the bfloat16 steps of single tokens ran %d folded products" % folded[0]
    finally:
        ops.decode_linear_residual = real
