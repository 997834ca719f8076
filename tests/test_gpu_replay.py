"""Replay on the GPU, float32 and bfloat16: every request alone and whole; most of it in one step
and the last 32 tokens one by one; portions of changing size down to two tokens; up to four live
requests mixed, with so few pages that they are used again.  All compared with the plain
implementation, position by position."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import replay_cases as rc
from tests.configs import INIT, TINY_A, TINY_B, TINY_C, TINY_D, TINY_E
from tests.gpu_util import require_gpu
from tests.plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu

# the first requests of A and B are the workloads of those configurations; the further ones are there so that the mixed
# trace admits requests after others have ended (four are live at most)
CASES = {"A": (TINY_A, [5, 17, 33, 60, 44, 23, 9, 51], 16), "B": (TINY_B, [1, 40, 130, 75, 12, 100, 33], 8),
         "C": (TINY_C, [3, 70, 200, 45, 64, 97, 333], 16), "D": (TINY_D, [9, 50, 190, 77, 300, 21], 16),
         "E": (TINY_E, [2, 130, 425, 61, 90, 17], 16)}
# float32: only the order of sums differs.  bfloat16: activations are rounded to 8 bits between
# kernels; with these weights the CPU model of that rounding differs from float32 by up to 0.04
# on logits of standard deviation 0.7, hence twice that as the absolute tolerance.
TOL = {"float32": dict(atol=1e-4, rtol=1e-4), "bfloat16": dict(atol=8e-2, rtol=2e-2)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    out = {}
    for name, (cfg, lengths, page) in CASES.items():
        folder = write_random_model(str(tmp_path_factory.mktemp("model_" + name)), cfg, 21 + len(name), torch.bfloat16, **INIT)
        reqs = rc.random_requests(cfg["vocab_size"], lengths, seed=5)
        plain = PlainQwen3(folder)
        out[name] = (folder, reqs, {rid: plain.forward(t) for rid, t in reqs.items()})
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_replay_matches_plain(dtype, name, mode, models, tmp_path, monkeypatch):
    require_gpu()
    from spyinfer_amd.kernels import ops
    folded = []
    real = ops.decode_linear_residual
    monkeypatch.setattr(ops, "decode_linear_residual", lambda *a, **k: (folded.append(1), real(*a, **k))[1])
    cfg, lengths, page = CASES[name]
    folder, reqs, ref = models[name]
    steps = getattr(rc, mode)(reqs)
    handed_out = _count_pages_handed_out(monkeypatch)
    if mode == "mixed":
        rc.assert_mixed(steps, name)         # portions beside decoded tokens, requests admitted after others ended
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", str(page)])
    got = rc.collect(str(tmp_path), steps, cfg["vocab_size"])
    rc.compare(got, ref, what="%s/%s/%s" % (name, mode, dtype), **TOL[dtype])
    if mode != "whole" or len(lengths) > 1:
        assert max(handed_out.values()) >= 2, "no page of the pool was handed out a second time"
    # configurations D and E in bfloat16 are there for the decode products with folded norms: they must have run
    assert bool(folded) == (name in "DE" and dtype == "bfloat16")


@pytest.mark.parametrize("name", ["D", "E"])
@pytest.mark.parametrize("mode", ["whole", "portions", "mixed"])
def test_replay_with_tiles_of_256_rows(name, mode, models, tmp_path, monkeypatch):
    """Prompts long enough to fill the chip are cut into attention tiles of 256 rows instead of 128 (head sizes 64 and
    128: configurations D and E).  Here the threshold is lowered so that the tests' prompts take them."""
    require_gpu()
    from spyinfer_amd.kernels import ops
    monkeypatch.setattr(ops, "PREFILL_WIDE_TILES_MIN_BLOCKS", 1)
    seen = []
    real = ops.paged_attention
    monkeypatch.setattr(ops, "paged_attention", lambda *a, **k: (seen.append((a[4].big_rows, a[4].tiles["big"][2])), real(*a, **k))[1])
    cfg, lengths, page = CASES[name]
    folder, reqs, ref = models[name]
    steps = getattr(rc, mode)(reqs)
    rc.run_replay_inprocess(folder, "bfloat16", str(tmp_path), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", str(page)])
    rc.compare(rc.collect(str(tmp_path), steps, cfg["vocab_size"]), ref, what="256-row tiles/%s/%s" % (name, mode), **TOL["bfloat16"])
    assert any(rows == 256 and n > 0 for rows, n in seen) or mode != "whole"


def _count_pages_handed_out(monkeypatch):
    """{page: times it was handed out} over all pools made from now on."""
    from spyinfer_amd.cache.pages import PagePool
    count = {}
    real = PagePool.allocate

    def allocate(self):
        page = real(self)
        count[page] = count.get(page, 0) + 1
        return page
    monkeypatch.setattr(PagePool, "allocate", allocate)
    return count


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_page_numbering_does_not_matter(dtype, name, models, tmp_path, monkeypatch):
    """The mixed trace on a pool whose free list was shuffled: requests get pages in no order at all, pages handed out
    again come back in another order, and the logits are those of the plain implementation all the same."""
    import random
    require_gpu()
    from spyinfer_amd.cache.pages import PagePool
    real = PagePool.__init__

    def shuffled(self, num_pages):
        real(self, num_pages)
        random.Random(num_pages).shuffle(self._free)
    monkeypatch.setattr(PagePool, "__init__", shuffled)
    cfg, lengths, page = CASES[name]
    folder, reqs, ref = models[name]
    steps = rc.mixed(reqs, seed=3)
    rc.assert_mixed(steps, name)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", str(page)])
    rc.compare(rc.collect(str(tmp_path), steps, cfg["vocab_size"]), ref, what="shuffled/%s/%s" % (name, dtype), **TOL[dtype])


@pytest.fixture(scope="module")
def sharp_model(tmp_path_factory):
    """Config C with the q and k norm weights scaled up, so that scores are large and the softmax is
    peaked: single far keys carry most of the weight, and a key that is skipped, read from the wrong
    page or masked by mistake changes the logits by far more than the tolerance."""
    from safetensors.torch import load_file
    from spyinfer_amd.weights import write_file, write_random_model
    folder = write_random_model(str(tmp_path_factory.mktemp("model_sharp")), TINY_C, 77, torch.bfloat16, **INIT)
    path = os.path.join(folder, "model.safetensors")
    w = {k: v.clone() for k, v in load_file(path).items()}
    for k in w:
        if k.endswith("q_norm.weight") or k.endswith("k_norm.weight"):
            w[k] = (w[k].float() * 2.0).to(torch.bfloat16)
    write_file(path, w)
    reqs = rc.random_requests(TINY_C["vocab_size"], [600, 333, 150, 420, 64, 257], seed=6)
    plain = PlainQwen3(folder)
    return folder, reqs, {rid: plain.forward(t) for rid, t in reqs.items()}


def test_sharp_attention_is_really_sharp(sharp_model):
    """The construction does what it says: in the plain model, dropping one far key changes logits visibly."""
    folder, reqs, ref = sharp_model
    plain = PlainQwen3(folder)
    toks = reqs["r2"]
    full = plain.forward(toks)[-1]
    for drop in (1, 17, 75):                                # one key of 150 removed (later positions shift by one too)
        cut = plain.forward(toks[:drop] + toks[drop + 1:])[-1]
        assert (full - cut).abs().max() > 0.5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["bulk_tail", "portions", "mixed"])
def test_replay_with_sharp_attention_over_hundreds_of_keys(dtype, mode, sharp_model, tmp_path):
    require_gpu()
    folder, reqs, ref = sharp_model
    steps = getattr(rc, mode)(reqs)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps))
    got = rc.collect(str(tmp_path), steps, TINY_C["vocab_size"])
    # A peaked softmax amplifies the bfloat16 rounding of q and k: the CPU model of that rounding differs from
    # the plain implementation by up to 0.14 here, a dropped key by more than 0.5 (test above).
    tol = dict(TOL[dtype]) if dtype == "float32" else dict(atol=0.28, rtol=0.02)
    rc.compare(got, ref, what="sharp/%s/%s" % (mode, dtype), **tol)


def test_cuts_agree_with_each_other_under_sharp_attention(sharp_model, tmp_path):
    """bfloat16, the peaked model: the same requests whole, with the last 32 tokens one by one, in portions and mixed
    give each other's logits far closer than they give the plain implementation's (they round the same values, only
    the order of sums differs: up to 0.10 here, against 0.15 from the plain logits).  A key that one way of cutting
    drops, reads from a wrong page or masks by mistake moves a logit by more than 0.5 (test above) in that way only."""
    require_gpu()
    folder, reqs, _ref = sharp_model
    got = {}
    for mode in ("whole", "bulk_tail", "portions", "mixed"):
        steps = getattr(rc, mode)(reqs)
        out = tmp_path / mode
        out.mkdir()
        rc.run_replay_inprocess(folder, "bfloat16", str(out), steps, rc.max_live_tokens(steps))
        got[mode] = rc.collect(str(out), steps, TINY_C["vocab_size"])
    modes = list(got)
    for i, a in enumerate(modes):
        for b in modes[i + 1:]:
            common = sorted(set(got[a]) & set(got[b]), key=lambda k: (str(k[0]), k[1]))
            assert len(common) > 1000
            for k in common:
                err = float(np.abs(got[a][k].astype(np.float64) - got[b][k].astype(np.float64)).max())
                assert err <= 0.14, "%s and %s differ by %.3f at request %r position %d" % (a, b, err, k[0], k[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dtype, models, tmp_path):
    """bin/trace_run as a user starts it: a process of its own, steps on standard input."""
    require_gpu()
    cfg, lengths, page = CASES["B"]
    folder, reqs, ref = models["B"]
    steps = rc.mixed(reqs, seed=7)
    rc.assert_mixed(steps, "B")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out",
                        str(tmp_path), "--max-tokens", str(rc.max_live_tokens(steps)), "--poison-cache"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done %d" % s["step"] for s in steps]
    rc.compare(rc.collect(str(tmp_path), steps, cfg["vocab_size"]), ref, what="trace_run/" + dtype, **TOL[dtype])
