"""Configurations drawn at random, each replayed in portions and mixed against the plain implementation: head sizes in
steps of 16 up to 256, any number of heads and groups, widths, intermediate sizes and vocabularies that are no power
of two (some of them multiples of 128, so that the tiled decode products and the folded norms take part), pages of 8 to
64 tokens, tied and untied heads.  A size that a kernel does not take must be refused by name, never computed wrongly:
every configuration here is one the engine says it takes, and every logit is compared.

Tolerances: float32 as everywhere (1e-4).  bfloat16: the rounding of activations to 8 bits moves a logit in proportion to
the logits' size; the 0.08 used elsewhere belongs to logits of standard deviation 0.7 (the tiny configurations), and the
wider models drawn here have logits of 1.4 to 1.6, so the absolute tolerance is 0.08 times rms / 0.7 where that is
more.  (250 further seeds of this test, run once: float32 within 1e-4 everywhere; in bfloat16 the largest error of a
configuration was 0.08 to 0.12 at logits of rms 1.4 to 1.6, the same whole and in portions, mean 0.012, 99th centile
0.04: a smooth tail, where a wrong page or a dropped key moves logits by their own size.)"""
import random

import pytest
import torch

from spyinfer_amd.kernels import key_pieces
from tests import replay_cases as rc
from tests.configs import INIT
from tests.gpu_util import require_gpu
from tests.plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(atol=1e-4, rtol=1e-4), "bfloat16": dict(atol=8e-2, rtol=2e-2)}


def draw_config(seed):
    rng = random.Random(1000 + seed)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 192, 256])
    n_kv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 5, 8])
    if seed % 3 == 0:                       # widths that the tiled decode products take
        hidden = rng.choice([128, 256, 384])
        inter = rng.choice([128, 256, 384, 640])
    else:
        hidden = 8 * rng.randint(5, 40)
        inter = 8 * rng.randint(6, 60)
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=rng.randint(1, 3),
                hidden_size=hidden, num_attention_heads=n_kv * group, num_key_value_heads=n_kv, head_dim=head_dim,
                intermediate_size=inter, vocab_size=rng.randint(90, 700), rope_theta=rng.choice([1e4, 5e4, 1e6]),
                rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]), tie_word_embeddings=rng.random() < 0.5,
                max_position_embeddings=512, bos_token_id=0, eos_token_id=1), rng.choice([8, 16, 32, 64])


@pytest.mark.parametrize("seed", range(10))
def test_random_configuration(seed, tmp_path):
    from spyinfer_amd.weights import write_random_model
    require_gpu()
    cfg, page = draw_config(seed)
    what = "seed %d: %s, page %d" % (seed, {k: cfg[k] for k in ("num_hidden_layers", "hidden_size", "num_attention_heads",
                                                               "num_key_value_heads", "head_dim", "intermediate_size", "vocab_size")}, page)
    print(what, flush=True)
    folder = write_random_model(str(tmp_path / "m"), cfg, 300 + seed, torch.bfloat16, **INIT)
    rng = random.Random(seed)
    reqs = rc.random_requests(cfg["vocab_size"], [rng.randint(1, 150) for _ in range(5)] + [70], seed=seed)
    plain = PlainQwen3(folder)
    ref = {rid: plain.forward(t) for rid, t in reqs.items()}
    rms = float(torch.cat(list(ref.values())).pow(2).mean().sqrt())
    for dtype in ("float32", "bfloat16"):
        for mode in ("portions", "mixed"):
            steps = rc.mixed(reqs, seed=seed) if mode == "mixed" else rc.portions(reqs)
            out = tmp_path / (dtype + mode)
            out.mkdir()
            rc.run_replay_inprocess(folder, dtype, str(out), steps, rc.max_live_tokens(steps, unit=max(64, page)),
                                    ["--kvcache-block-size", str(page)])
            tol = dict(TOL[dtype])
            if dtype == "bfloat16":
                tol["atol"] *= max(1.0, rms / 0.7)
            rc.compare(rc.collect(str(out), steps, cfg["vocab_size"]), ref, what="%s/%s/%s" % (what, mode, dtype), **tol)


@pytest.mark.parametrize("seed", range(8))
def test_random_decode_steps_of_uneven_lengths(seed, tmp_path):
    """Decode steps of 2 to 40 requests of 1 to 1900 tokens at head sizes 64 and 128, where the host cuts the keys into
    pieces: kv heads, groups, pages and lengths drawn at random, eagerly or from a recorded graph; every step's logits
    against the plain pass.  (60 further seeds, run once: no failure.)"""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    rng = random.Random(7000 + seed)
    d, n_kv, group, page = rng.choice([64, 128]), rng.choice([1, 2, 3, 4, 8]), rng.choice([1, 2, 4, 5, 8]), rng.choice([8, 16, 32, 64])
    cfg = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=rng.randint(1, 2),
               hidden_size=rng.choice([128, 256]), num_attention_heads=n_kv * group, num_key_value_heads=n_kv, head_dim=d,
               intermediate_size=rng.choice([128, 384]), vocab_size=rng.randint(90, 400), rope_theta=1e6, rms_norm_eps=1e-6,
               tie_word_embeddings=False, max_position_embeddings=2048, bos_token_id=0, eos_token_id=1)
    R = rng.randint(2, 40)
    lengths = [rng.randint(1, rng.choice([100, 600, 1500])) for _ in range(R)]
    if seed % 2:
        lengths[0] = 1900
    steps, eager = 5, seed % 3 == 0
    print("seed %d: head_dim %d, %d kv heads of %d, page %d, %d requests up to %d tokens, %s" % (
        seed, d, n_kv, group, page, R, max(lengths), "eager" if eager else "graphs"), flush=True)
    folder = write_random_model(str(tmp_path / "m"), cfg, 500 + seed, torch.bfloat16, **INIT)
    g = torch.Generator().manual_seed(seed)
    seqs = [torch.randint(0, cfg["vocab_size"], (n + steps,), generator=g).tolist() for n in lengths]
    plain = PlainQwen3(folder)
    ref = [plain.forward(q)[n:n + steps] for q, n in zip(seqs, lengths)]
    rms = float(torch.cat(ref).pow(2).mean().sqrt())
    atol = TOL["bfloat16"]["atol"] * max(1.0, rms / 0.7)
    runner = ModelRunner(load_model(folder, "bfloat16", dev), "bfloat16", dev, page, sum(-(-(n + steps) // page) for n in lengths) + 4, R,
                         enforce_eager=eager, max_model_len=2048)
    caches = [runner.manager.admit(i) for i in range(R)]
    for c, q, n in zip(caches, seqs, lengths):
        runner.manager.reserve(c, n)
        runner.step([StepEntry(c, q[:n], [])])
    cut = False
    for i in range(steps):
        for c in caches:
            runner.manager.reserve(c, 1)
        got = runner.step([StepEntry(c, [q[n + i]], [0]) for c, q, n in zip(caches, seqs, lengths)]).cpu()
        want = torch.stack([r[i] for r in ref])
        assert torch.allclose(got, want, atol=atol, rtol=TOL["bfloat16"]["rtol"]), "step %d: off by %s" % (i, (got - want).abs().max(1).values.tolist())
        rec = key_pieces.decode_pieces([n + i + 1 for n in lengths], n_kv, 0, head_dim=d)
        cut = cut or int(rec[:, 5].max()) > 1
    assert ops.workspace_counters_clean(dev)
    assert cut or max(lengths) < 300, "a long request among these is cut into parts"
