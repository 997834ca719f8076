"""Replay on the GPU, float32 and bfloat16: every request alone and whole; most of it in one step
and the last 32 tokens one by one; portions of changing size down to two tokens; up to four live
requests mixed, with so few pages that they are used again.  All compared with the plain
implementation, position by position."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import replay_cases as rc
from tests.configs import INIT, TINY_A, TINY_B, TINY_C
from tests.gpu_util import require_gpu
from tests.plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu

CASES = {"A": (TINY_A, [5, 17, 33, 60], 16), "B": (TINY_B, [1, 40, 130], 8), "C": (TINY_C, [3, 70, 200, 45, 64, 97, 333], 16)}
# float32: only the order of sums differs.  bfloat16: activations are rounded to 8 bits between
# kernels; with these weights the CPU model of that rounding differs from float32 by up to 0.04
# on logits of standard deviation 0.7 ("tolerances").
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
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_replay_matches_plain(dtype, name, mode, models, tmp_path):
    require_gpu()
    cfg, lengths, page = CASES[name]
    folder, reqs, ref = models[name]
    steps = getattr(rc, mode)(reqs)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", str(page)])
    got = rc.collect(str(tmp_path), steps, cfg["vocab_size"])
    rc.compare(got, ref, what="%s/%s/%s" % (name, mode, dtype), **TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dtype, models, tmp_path):
    """bin/trace_run as a user starts it: a process of its own, steps on standard input."""
    require_gpu()
    cfg, lengths, page = CASES["B"]
    folder, reqs, ref = models["B"]
    steps = rc.mixed(reqs, seed=7)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out",
                        str(tmp_path), "--max-tokens", str(rc.max_live_tokens(steps))],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done %d" % s["step"] for s in steps]
    rc.compare(rc.collect(str(tmp_path), steps, cfg["vocab_size"]), ref, what="trace_run/" + dtype, **TOL[dtype])
