"""The kernels at the widths they are tuned for.  The tiny configurations of the other tests never reach the sizes
at which a kernel changes its shape (128-row attention tiles with 8-wave blocks, products with two column tiles per
block, weight copies of many chunks, key parts).  Here two layers of the benchmark's widths (for instance hidden 4096,
32 query and 8 key/value heads of 128, intermediate 12288) with a vocabulary that is no multiple of 16 run the same steps in
bfloat16 and in true float32 on the same weights (the bfloat16 values widened exactly), and the float32 logits are
compared with the plain implementation on the CPU.  The steps: prompts whole (128-row attention tiles beside short
entries), a step with portions of 96 and 70 tokens behind cached prefixes beside single tokens of all the others, then
decode steps of 44, 9 and 1 requests.  A second set of weights has the q and k norm weights doubled, so that the
softmax is peaked and single far keys carry the weight."""
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


def _runners(dev, requests, pages, widths, sharp=False, dtypes=("bfloat16", "float32"), weight_copies=("both", "both")):
    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.runner import ModelRunner, bind_weights
    from spyinfer_amd.weights.random_init import random_tensors_on_device
    raw = dict(RAW, hidden_size=widths[0], num_attention_heads=widths[1], num_key_value_heads=widths[2], head_dim=widths[3],
               intermediate_size=widths[4])
    arch = architecture_of(raw)
    cfg = arch.config_cls.from_dict(raw)
    out = []
    w16 = None
    for dtype, copies in zip(dtypes, weight_copies):
        model = arch.build(cfg)
        if w16 is None:
            w16 = random_tensors_on_device(model.weight_specs(), 5, torch.bfloat16, dev, norm_std=0.05)
            if sharp:
                for k in w16:
                    if k.endswith("q_norm.weight") or k.endswith("k_norm.weight"):
                        w16[k] = (w16[k].float() * 2.0).to(torch.bfloat16)
        weights = w16 if dtype == "bfloat16" else {k: (v.float() if v.dtype == torch.bfloat16 else v) for k, v in w16.items()}
        bind_weights(model, dict(weights), dev, copies)       # a copy: parts take matrices out of the dictionary
        out.append(ModelRunner(model, dtype, dev, 16, pages, requests, enforce_eager=True, max_model_len=1024))
    return out, raw, w16


def _close(a, b, what, atol=8e-2):
    """bfloat16 against float32 logits: the tolerance of the other bfloat16 tests, and the same first choice wherever
    the float32 logits do not nearly tie."""
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape
    err = (a - b).abs()
    assert torch.all(err <= atol + 2e-2 * b.abs()), "%s: bfloat16 and float32 differ by %g (logits up to %g)" % (what, err.max(), b.abs().max())
    top = torch.topk(b, 2, dim=-1).values
    clear = (top[:, 0] - top[:, 1]) > 0.2
    assert torch.equal(a.argmax(-1)[clear], b.argmax(-1)[clear]), what + ": another first choice"


def _plain_close(got, ref, what):
    """float32 engine against the plain implementation: only the order of float32 sums differs (up to 17408 addends)."""
    got, ref = got.float().cpu(), ref.float()
    err = (got - ref).abs().max().item()
    assert err <= 1e-4 * max(1.0, ref.abs().max().item()), "%s: float32 logits differ from the plain implementation's by %g" % (what, err)


@pytest.mark.parametrize("widths,sharp", [(w, False) for w in WIDTHS] + [(WIDTHS[0], True)])
def test_steps_at_real_widths(widths, sharp):
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.kernels import ops
    from tests.plain.qwen3_plain import PlainQwen3
    dev = require_gpu()
    R = 44
    (r16, r32), raw, w16 = _runners(dev, R, 240, widths, sharp)
    plain = PlainQwen3(None, config=raw, weights=w16)
    # a peaked softmax amplifies the bfloat16 rounding of q and k (as in the replay tests with sharp attention)
    atol = 0.28 if sharp else 8e-2
    g = torch.Generator().manual_seed(9)
    lens = [300, 170] + [3 + (5 * i) % 38 for i in range(R - 2)]
    prompts = [torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist() for n in lens]
    seqs = [list(p) for p in prompts]
    checked = (0, 1, 43)                                   # requests whose float32 logits are compared with the plain pass
    folded = [0]
    real = ops.decode_linear_residual
    ops.decode_linear_residual = lambda *a, **k: (folded.__setitem__(0, folded[0] + 1), real(*a, **k))[1]

    def both(entries_of):
        outs = []
        for runner, cs in zip((r16, r32), caches):
            entries = entries_of(cs)
            for e in entries:
                runner.manager.reserve(e.cache, len(e.tokens))
            outs.append(runner.step(entries))
        return outs

    def against_plain(out32, rows, what):
        for i in checked:
            if i in rows:
                _plain_close(out32[rows.index(i)], plain.forward(seqs[i])[-1], "%s, request %d" % (what, i))

    try:
        caches = [[runner.manager.admit(i) for i in range(R)] for runner in (r16, r32)]
        # the prompts in one step: two entries with 128-row tiles beside short ones; logits at the last place of each
        outs = both(lambda cs: [StepEntry(c, p, [len(p) - 1]) for c, p in zip(cs, prompts)])
        _close(outs[0], outs[1], "prompts", atol)
        against_plain(outs[1], list(range(R)), "prompts")
        assert folded[0] == 0
        # portions of 96 and 70 tokens behind cached prefixes of 300 and 170 (128-row tiles with pos0 > 0) beside one
        # decoded token of each other request
        more = [torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist() for n in [96, 70] + [1] * (R - 2)]
        for q, m in zip(seqs, more):
            q.extend(m)
        outs = both(lambda cs: [StepEntry(c, m, [len(m) - 1]) for c, m in zip(cs, more)])
        _close(outs[0], outs[1], "portions beside single tokens", atol)
        against_plain(outs[1], list(range(R)), "portions beside single tokens")
        assert folded[0] == 0
        # three steps of all 44 requests (three row tiles), then of the first 9 (one row tile), then of one
        for live, steps in ((R, 3), (9, 3), (1, 2)):
            for s in range(steps):
                toks = torch.randint(0, RAW["vocab_size"], (live,), generator=g).tolist()
                for q, t in zip(seqs, toks):
                    q.append(t)
                outs = both(lambda cs: [StepEntry(c, [t], [0]) for c, t in zip(cs[:live], toks)])
                _close(outs[0], outs[1], "%d requests, step %d" % (live, s), atol)
            against_plain(outs[1], list(range(live)), "%d requests, last step" % live)
        assert folded[0] == 8 * 2 * 2, "the bfloat16 steps of single tokens ran %d folded products" % folded[0]
    finally:
        ops.decode_linear_residual = real


def test_decode_steps_of_65_to_128_requests_at_real_widths():
    """Decode steps of 100 and of 70 requests (eight and six row tiles of the folded products, which take their inputs in
    operand order only there) at the 8B widths: bfloat16 against float32 on the same weights, float32 against the plain
    implementation, and the folded products really ran."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.kernels import ops
    from tests.plain.qwen3_plain import PlainQwen3
    dev = require_gpu()
    R = 100
    (r16, r32), raw, w16 = _runners(dev, R, 400, WIDTHS[0])
    plain = PlainQwen3(None, config=raw, weights=w16)
    g = torch.Generator().manual_seed(11)
    prompts = [torch.randint(0, RAW["vocab_size"], (3 + (7 * i) % 40,), generator=g).tolist() for i in range(R)]
    seqs = [list(p) for p in prompts]
    folded = [0]
    real = ops.decode_linear_residual
    ops.decode_linear_residual = lambda *a, **k: (folded.__setitem__(0, folded[0] + 1), real(*a, **k))[1]

    def both(entries_of):
        outs = []
        for runner, cs in zip((r16, r32), caches):
            entries = entries_of(cs)
            for e in entries:
                runner.manager.reserve(e.cache, len(e.tokens))
            outs.append(runner.step(entries))
        return outs

    try:
        caches = [[runner.manager.admit(i) for i in range(R)] for runner in (r16, r32)]
        outs = both(lambda cs: [StepEntry(c, p, [len(p) - 1]) for c, p in zip(cs, prompts)])
        _close(outs[0], outs[1], "prompts")
        assert folded[0] == 0
        for live, steps in ((R, 2), (70, 2)):
            for s in range(steps):
                toks = torch.randint(0, RAW["vocab_size"], (live,), generator=g).tolist()
                for q, t in zip(seqs, toks):
                    q.append(t)
                outs = both(lambda cs: [StepEntry(c, [t], [0]) for c, t in zip(cs[:live], toks)])
                _close(outs[0], outs[1], "%d requests, step %d" % (live, s))
            for i in (0, live // 2, live - 1):
                _plain_close(outs[1][i], plain.forward(seqs[i])[-1], "%d requests, request %d" % (live, i))
        assert folded[0] == 4 * 2 * 2, "the bfloat16 steps of single tokens ran %d folded products" % folded[0]
    finally:
        ops.decode_linear_residual = real


def test_steps_with_matrices_kept_in_tiles_only():
    """EngineConfig.weight_copies = "tiled" at the 8B widths, in bfloat16 against the same model with both forms: no
    bfloat16 matrix keeps its rows; steps of many rows (the library's products on restored rows) and of single tokens
    (the folded products) give the same logits bit for bit; a step of 40 rows, where the decode kernel stands in for
    the library, the same within the bfloat16 tolerance."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    runners, raw, w16 = _runners(dev, 4, 64, WIDTHS[0], dtypes=("bfloat16", "bfloat16"), weight_copies=("both", "tiled"))
    layer = runners[1].model.layers[0]
    for m in (layer.mixer.w_qkv, layer.mixer.w_o, layer.ffn.w_gate_up, layer.ffn.w_down):
        assert isinstance(m, ops.TiledOnly)
    assert isinstance(runners[1].model.lm_head.weight, torch.Tensor)      # 4099 rows have no tiled form: they stay
    assert not isinstance(runners[0].model.layers[0].mixer.w_o, ops.TiledOnly)
    g = torch.Generator().manual_seed(13)
    prompts = [torch.randint(0, RAW["vocab_size"], (n,), generator=g).tolist() for n in (300, 170, 20, 5)]
    caches = [[runner.manager.admit(i) for i in range(4)] for runner in runners]

    def both(entries_of):
        outs = []
        for runner, cs in zip(runners, caches):
            entries = entries_of(cs)
            for e in entries:
                runner.manager.reserve(e.cache, len(e.tokens))
            outs.append(runner.step(entries))
        return outs

    outs = both(lambda cs: [StepEntry(c, p, [0, len(p) - 1]) for c, p in zip(cs, prompts)])
    assert torch.equal(outs[0], outs[1]), "prompts: other logits than with both forms"
    more = torch.randint(0, RAW["vocab_size"], (40,), generator=g).tolist()
    outs = both(lambda cs: [StepEntry(cs[0], more, [0, 39])])
    _close(outs[1], outs[0], "a portion of 40 tokens")
    for step in range(2):
        toks = torch.randint(0, RAW["vocab_size"], (4,), generator=g).tolist()
        outs = both(lambda cs: [StepEntry(c, [t], [0]) for c, t in zip(cs, toks)])
        if step == 0:
            _close(outs[1], outs[0], "single tokens after the portion")       # request 0's keys differ by rounding now
            assert torch.equal(outs[0][1:], outs[1][1:])
    assert torch.isfinite(outs[1]).all()
