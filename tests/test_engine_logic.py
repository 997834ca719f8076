"""The engine's logic (batch metadata, cache pages, block tables, every way of cutting) on the
CPU stand-in for the kernels, compared with the plain implementation."""
import numpy as np
import pytest
import torch

from tests import replay_cases as rc
from tests.configs import INIT, TINY_A, TINY_B, TINY_C
from tests.plain.qwen3_plain import PlainQwen3


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    out = {}
    for name, cfg, seed in (("A", TINY_A, 11), ("B", TINY_B, 12), ("C", TINY_C, 13)):
        out[name] = write_random_model(str(tmp_path_factory.mktemp("model_" + name)), cfg, seed, torch.bfloat16, **INIT)
    return out


CASES = {"A": (TINY_A, [5, 17, 33, 60]), "B": (TINY_B, [1, 40, 130]), "C": (TINY_C, [3, 70, 200, 45, 64, 97])}


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_cuts_match_plain(name, mode, folders, tmp_path, emu_ops):
    cfg, lengths = CASES[name]
    reqs = rc.random_requests(cfg["vocab_size"], lengths, seed=3)
    steps = getattr(rc, mode)(reqs)
    max_tokens = rc.max_live_tokens(steps)
    page = {"A": 16, "B": 8, "C": 16}[name]
    rc.run_replay_inprocess(folders[name], "float32", str(tmp_path), steps, max_tokens,
                            ["--device", "cpu", "--kvcache-block-size", str(page)])
    plain = PlainQwen3(folders[name])
    ref = {rid: plain.forward(t) for rid, t in reqs.items()}
    got = rc.collect(str(tmp_path), steps, cfg["vocab_size"])
    if mode != "mixed":
        assert len(got) == sum(lengths)
    rc.compare(got, ref, atol=2e-4, rtol=2e-4, what="%s/%s" % (name, mode))


def test_replay_lines_without_tokens_and_names_used_again(folders, tmp_path, emu_ops):
    """A line may bring no tokens at all (it only ends requests), a request may be left out of steps, and a name that
    has ended may be used again for a new request, which starts from an empty cache."""
    cfg = TINY_A
    reqs = rc.random_requests(cfg["vocab_size"], [21, 9], seed=5)
    a, b = reqs["r0"], reqs["r1"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:10], "want": [9]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": b, "want": [8]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": a[10:], "want": [10]}, {"id": "y", "tokens": [], "want": []}], "end": []},
             {"step": 3, "entries": [], "end": ["x", "y"]},
             {"step": 4, "entries": [{"id": "x", "tokens": b, "want": [0, 8]}], "end": ["x"]}]
    rc.run_replay_inprocess(folders["A"], "float32", str(tmp_path), steps, 128, ["--device", "cpu"])
    plain = PlainQwen3(folders["A"])
    ra, rb = plain.forward(a), plain.forward(b)
    V = cfg["vocab_size"]
    read = lambda i, n: torch.from_numpy(np.fromfile(str(tmp_path / ("%d.f32" % i)), dtype="<f4").reshape(n, V).copy())
    assert not (tmp_path / "3.f32").exists()
    for got, ref in ((read(0, 1), ra[[9]]), (read(1, 1), rb[[8]]), (read(2, 1), ra[[20]]), (read(4, 2), rb[[0, 8]])):
        assert torch.allclose(got, ref, atol=2e-4, rtol=2e-4)
