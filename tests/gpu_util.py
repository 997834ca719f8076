import pytest
import torch


def require_gpu():
    """The GPU tests fail (not skip) when the kernel library cannot be loaded on a GPU box."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from spyinfer_amd.kernels import ops
    ops.hip()
    return torch.device("cuda:0")


TOL = {torch.float32: dict(atol=2e-5, rtol=2e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


def close(got, ref, dtype, scale=1.0, what=""):
    """|got - ref| <= atol * scale * max(1, rms(ref)) + rtol * |ref|: rounding errors of sums grow
    with the typical size of the result, not with the size of the one element."""
    tol = TOL[dtype]
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    err = (got - ref).abs()
    rms = float(ref.pow(2).mean().sqrt()) if ref.numel() else 0.0
    lim = tol["atol"] * scale * max(1.0, rms) + tol["rtol"] * ref.abs()
    bad = ~(err <= lim)
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        raise AssertionError("%s: first wrong element at %s: got %r, expected %r (%d of %d wrong, max err %.3g)"
                             % (what, idx, got[tuple(idx)].item(), ref[tuple(idx)].item(), int(bad.sum()), bad.numel(), err.max().item()))
