"""The sampling entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a caller
without torch's allocator would, against the entry point that takes a workspace."""
import ctypes

import pytest
import torch

from tests.gpu_util import require_gpu
from tests.plain.sampler_plain import choose

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _case(R, V, seed, dev):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(R, V, generator=g) * 3.0).to(dev)
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * (r % 5) for r in range(R)], dtype=torch.float32).to(dev)
    u = torch.rand(R, generator=g).to(dev)
    return logits, temperature, u


def test_sample_static_equals_sample():
    dev = require_gpu()
    from spyinfer_amd.kernels import build, ops
    lib = build.load()
    assert hasattr(lib, "spy_sample_static"), "the kernel library is older than its sources: build it again"
    lib.spy_sample_static.restype = ctypes.c_int
    lib.spy_last_error.restype = ctypes.c_char_p
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # two calls in a row on the one scratch array, the second smaller: what the first left behind must not show
    for R, V, seed in ((37, 1531, 1), (5, 331, 2)):
        logits, temperature, u = _case(R, V, seed, dev)
        want = ops.sample(logits, temperature, u)
        out = torch.full((R,), -7, dtype=torch.int32, device=dev)        # made before the call: the call allocates nothing
        torch.cuda.synchronize()
        rc = lib.spy_sample_static(_ptr(logits), _ptr(temperature), _ptr(u), _ptr(out), ctypes.c_int(R), ctypes.c_int(V), stream)
        assert rc == 0, lib.spy_last_error().decode()
        torch.cuda.synchronize()
        assert out.tolist() == want.tolist(), "R=%d V=%d" % (R, V)
        greedy = [r for r in range(R) if r % 3 == 0]
        assert out[greedy].tolist() == logits[greedy].argmax(dim=1).tolist()
        # the sampled rows against the plain sampler (float64 cumulative distribution over ascending ids): the two entry
        # points share their kernels, so agreeing with each other does not show that either is right
        lg, tp, uu, got = logits.cpu().double().numpy(), temperature.cpu().tolist(), u.cpu().tolist(), out.cpu().tolist()
        checked = 0
        for r in range(R):
            if tp[r] == 0.0:
                continue
            tok, margin = choose(lg[r], tp[r], uu[r])
            if margin > 1e-5:                                              # a draw at an interval's edge may fall either way in float32
                assert got[r] == tok, "row %d: %d, the plain sampler picks %d" % (r, got[r], tok)
                checked += 1
        assert checked >= (R - len(greedy)) * 3 // 4


def test_sample_static_refuses_more_rows_than_its_array_holds():
    dev = require_gpu()
    from spyinfer_amd.kernels import build
    lib = build.load()
    lib.spy_sample_static.restype = ctypes.c_int
    lib.spy_last_error.restype = ctypes.c_char_p
    R, V = 513, 8
    logits, temperature, u = _case(R, V, 3, dev)
    out = torch.zeros(R, dtype=torch.int32, device=dev)
    rc = lib.spy_sample_static(_ptr(logits), _ptr(temperature), _ptr(u), _ptr(out), ctypes.c_int(R), ctypes.c_int(V),
                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0 and b"512" in lib.spy_last_error()
    torch.cuda.synchronize()
