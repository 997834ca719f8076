"""Each HIP kernel alone against a plain float64/float32 torch formula of the same operation, at
sizes other than the engine's: sizes that are no power of two, one row, many rows, odd head
counts and groups, pages of several sizes."""
import math

import pytest
import torch

from spyinfer_amd.kernels import key_pieces
from tests.gpu_util import close, require_gpu

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, dtype, dev, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(dev)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,V", [(1, 64, 10), (37, 200, 331), (300, 4096, 1000)])
def test_embedding(dtype, T, H, V):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    table = rnd((V, H), dtype, dev, 1)
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(2)).int().to(dev)
    out = ops.embedding(ids, table)
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), table.cpu()[ids.cpu().long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("T,H,eps", [(1, 64, 1e-6), (19, 200, 1e-5), (130, 4096, 1e-6), (3, 5120, 1e-2)])
def test_add_rms_norm(dtype, wdtype, T, H, eps):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    resid = rnd((T, H), torch.float32, dev, 3, 2.0)
    delta = rnd((T, H), dtype, dev, 4)
    w = (1 + 0.1 * rnd((H,), torch.float32, dev, 5)).to(wdtype)
    x = resid.double() + delta.double()
    ref = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.double()
    r2 = resid.clone()
    out = ops.add_rms_norm(r2, delta, w, eps, dtype)
    close(out, ref, dtype, what="add_rms_norm")
    close(r2, x, torch.float32, what="residual sum")
    # rows: only those rows, residual untouched; no delta
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32, device=dev)
    r3 = resid.clone()
    out = ops.add_rms_norm(r3, delta, w, eps, dtype, rows)
    close(out, ref[rows.long()], dtype, what="add_rms_norm rows")
    assert torch.equal(r3, resid)
    x0 = resid.double()
    out = ops.add_rms_norm(r3, None, w, eps, dtype)
    close(out, x0 / torch.sqrt((x0 * x0).mean(-1, keepdim=True) + eps) * w.double(), dtype, what="rms_norm without delta")
    assert torch.equal(r3, resid)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rms_norm_eps_matters(dtype):
    """A tiny row tells eps 1e-6 from 1e-5; an all-zero row gives zeros."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = torch.full((2, 96), 1e-3, dtype=dtype, device=dev)
    x[1] = 0
    w = torch.ones(96, dtype=dtype, device=dev)
    a = ops.rms_norm(x, w, 1e-6).float()
    b = ops.rms_norm(x, w, 1e-5).float()
    xv = float(x[0, 0])
    assert abs(a[0, 0].item() - xv / math.sqrt(xv * xv + 1e-6)) < 1e-2
    assert abs(b[0, 0].item() - xv / math.sqrt(xv * xv + 1e-5)) < 1e-2
    assert a[0, 0].item() > 2 * b[0, 0].item()
    assert torch.all(a[1] == 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 8, 10), (2, 4, 3), (4, 1024, 1024), (9, 1024, 1030), (120, 100, 1000), (1, 331, 88),
                                   (65, 200, 136), (7, 4096, 4096), (33, 160, 96)])
def test_linear(dtype, M, N, K):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = rnd((M, K), dtype, dev, 6)
    w = rnd((N, K), dtype, dev, 7, 0.05)
    ref = x.double() @ w.double().t()
    for od in (dtype, torch.float32):
        out = ops.linear(x, w, od)
        assert out.dtype == od and out.shape == (M, N)
        close(out, ref, dtype if od == dtype else (torch.float32 if dtype == torch.float32 else torch.bfloat16),
              scale=math.sqrt(K) * 0.05, what="linear %s->%s" % (dtype, od))


@pytest.mark.parametrize("M,N,K", [(1, 16, 128), (8, 4096, 4096), (16, 160, 256), (5, 1024, 12288), (3, 151936, 512)])
def test_linear_with_tiled_weights(M, N, K):
    """The decode kernel reading the copy of W in MFMA tile order gives what it gives on the row-major matrix."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = rnd((M, K), torch.bfloat16, dev, 17)
    w = rnd((N, K), torch.bfloat16, dev, 18, 0.05)
    wt = ops.tile_weight(w)
    assert wt is not None and wt.shape == w.shape
    for od in (torch.bfloat16, torch.float32):
        a, b = ops.linear(x, w, od, tiled=wt), ops.linear(x, w, od)
        close(a, x.double() @ w.double().t(), torch.bfloat16, scale=1.0, what="tiled linear")
        assert torch.allclose(a.float(), b.float(), atol=2e-2, rtol=2e-2)
    if N % 32 == 0:
        I = N // 2
        y = x.double() @ w.double().t()
        ref = y[:, :I] / (1 + torch.exp(-y[:, :I])) * y[:, I:]
        if I % 16 == 0:
            close(ops.linear_swiglu(x, w, wt), ref, torch.bfloat16, scale=2.0, what="tiled linear_swiglu")
    assert ops.tile_weight(rnd((24, 128), torch.bfloat16, dev, 1)) is None and ops.tile_weight(rnd((32, 96), torch.bfloat16, dev, 1)) is None


@pytest.mark.parametrize("N,K", [(16, 128), (48, 384), (4112, 1280), (24576, 4096)])
def test_untile_weight_restores_the_rows(N, K):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    w = rnd((N, K), torch.bfloat16, dev, 23, 0.05)
    assert torch.equal(ops.untile_weight(ops.tile_weight(w)), w)


def test_linear_with_a_matrix_kept_in_tiles_only(monkeypatch):
    """``weight_forms`` with the rows switched off keeps the tiled copy alone; ``linear`` then gives, for any number of
    rows, what it gives with both forms: the same kernel on the same values up to 16 rows and beyond 64 (there the
    library, on the restored rows), the decode kernel instead of the library between; also inside a captured graph,
    where the restored rows may not go to the scratch tensor that calls outside share."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    N, K = 1040, 640
    w = rnd((N, K), torch.bfloat16, dev, 31, 0.05)
    both = ops.weight_forms(w)
    assert both[0] is w and both[1] is not None
    monkeypatch.setattr(ops, "ROW_MAJOR_WEIGHTS", False)
    only, tiled = ops.weight_forms(w)
    assert isinstance(only, ops.TiledOnly) and only.shape == w.shape and torch.equal(tiled, both[1])
    kept, _ = ops.weight_forms(w, keep_rows=True)
    assert kept is w
    odd = rnd((24, 128), torch.bfloat16, dev, 1)                # no tiled form: the rows stay
    assert ops.weight_forms(odd)[0] is odd and ops.weight_forms(odd)[1] is None
    small = ops.weight_forms(rnd((32, 128), torch.bfloat16, dev, 2))[0]
    for M in (1, 16, 17, 40, 64, 65, 300):
        x = rnd((M, K), torch.bfloat16, dev, 32 + M)
        for od in (torch.bfloat16, torch.float32):
            a, b = ops.linear(x, only, od, tiled=tiled), ops.linear(x, w, od, tiled=both[1])
            close(a, x.double() @ w.double().t(), torch.bfloat16, scale=1.0, what="linear, tiles only, %d rows" % M)
            if M <= 16 or M > 64:
                assert torch.equal(a, b), "%d rows: another result than with both forms" % M
        ops.linear(x[:, :128].contiguous(), small)                # a smaller matrix takes its turn in the scratch tensor
    I = N // 2
    x = rnd((200, K), torch.bfloat16, dev, 50)
    assert torch.equal(ops.linear_swiglu(x, only, tiled), ops.linear_swiglu(x, w, both[1]))
    # captured: replays with other inputs, the scratch tensor used by calls in between
    xs = torch.zeros((200, K), dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ops.linear(xs, only)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = ops.linear(xs, only)
    for seed in (60, 61, 62):
        xs.copy_(rnd((200, K), torch.bfloat16, dev, seed))
        ops.linear(xs[:, :128].contiguous(), small)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, ops.linear(xs, w)), "replay with input %d" % seed


@pytest.mark.parametrize("M,H,I,NQKV,eps", [(1, 128, 256, 192, 1e-6), (7, 256, 384, 400, 1e-5), (16, 4096, 1024, 6144, 1e-6),
                                            (3, 5120, 128, 64, 1e-2), (17, 256, 128, 96, 1e-6), (32, 1024, 2048, 320, 1e-5),
                                            (41, 128, 384, 400, 1e-6), (64, 256, 128, 6144, 1e-6), (57, 128, 384, 6176, 1e-5),
                                            (33, 256, 128, 6240, 1e-6), (20, 128, 128, 6144, 1e-6), (48, 768, 384, 96, 1e-6), (25, 1280, 128, 64, 1e-5),
                                            (64, 2048, 384, 128, 1e-6),
                                            # many column tiles (two and more per compute unit): blocks that walk a run of
                                            # tiles, several at a time, the last group of a run with fewer
                                            (64, 128, 8320, 8208, 1e-6), (37, 256, 8448, 9008, 1e-5), (20, 128, 8192, 16400, 1e-6),
                                            (48, 128, 128, 151936, 1e-6), (16, 128, 8320, 8208, 1e-6),
                                            # stored products of very many columns at three and four row tiles: four-wave
                                            # blocks with twelve and eight column tiles at a time, a last group with fewer
                                            (64, 512, 128, 40000, 1e-6), (40, 1024, 128, 49168, 1e-5),
                                            # about a column tile per compute unit and a long K: K split over blocks, the
                                            # group's last block adding the parts (33 to 64 rows; a last group with fewer tiles; 2, 3, 4 parts)
                                            (64, 4096, 12288, 6144, 1e-6), (40, 4096, 8192, 6128, 1e-5), (52, 5120, 6400, 6160, 1e-6),
                                            # (three parts of 13, 13 and 14 chunks for eight waves each)
                                            (64, 5120, 5120, 6160, 1e-6),
                                            # two and a half column tiles per compute unit: blocks of five halves of tiles
                                            (8, 256, 128, 10240, 1e-6), (16, 128, 128, 10240, 1e-5),
                                            # 320 column tiles for 256 compute units: K split over blocks from the first row on
                                            (8, 5120, 5120, 96, 1e-6), (24, 5120, 6400, 96, 1e-5), (1, 5120, 3200, 64, 1e-6),
                                            # gated products with five pairs of column tiles per compute unit: four-wave blocks
                                            # that take a block's run as one group of six (four and three row tiles)
                                            (64, 1024, 17408, 96, 1e-6), (40, 256, 17408, 96, 1e-5),
                                            # more than 8 chunks of K for every wave in the loops that ask for the next step's operands ahead
                                            (40, 9216, 256, 8208, 1e-6), (50, 4096, 36864, 64, 1e-6)])
def test_decode_products_with_folded_norm(M, H, I, NQKV, eps):
    """The chain of a decode step's products with the norms folded in: the residual epilogue adds to the stream,
    prepares bf16(h * w) and the parts of sum(h^2); the next products scale their sums by rsqrt(mean(h^2) + eps).
    Compared with float64 formulas: RMS norm, product, SwiGLU, residual sum."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    resid0 = rnd((M, H), torch.float32, dev, 31, 1.5)
    wn1 = (1 + 0.1 * rnd((H,), torch.float32, dev, 32)).bfloat16()
    wn2 = (1 + 0.1 * rnd((H,), torch.float32, dev, 33)).bfloat16()
    w_in = rnd((H, I), torch.bfloat16, dev, 34, 0.05)
    w_qkv = rnd((NQKV, H), torch.bfloat16, dev, 35, 0.05)
    w_gu = rnd((2 * I, H), torch.bfloat16, dev, 36, 0.05)
    a = rnd((M, I), torch.bfloat16, dev, 37)

    def norm64(h, w):
        h = h.double()
        return h * torch.rsqrt((h * h).mean(1, keepdim=True) + eps) * w.double()

    # 1. the residual epilogue
    resid = resid0.clone()
    si = ops.decode_linear_residual(a, ops.tile_weight(w_in), resid, wn1, eps)
    h = resid0.double() + a.double() @ w_in.double().t()
    close(resid, h, torch.float32, scale=4.0, what="stream after the residual epilogue")
    assert isinstance(si.xw, ops.OperandRows), "outputs for the next product come in operand order"
    assert torch.equal(si.xw.to_rows(), (resid * wn1.float()).bfloat16()), "the prepared input is bf16(h * w) of the new stream"
    ss = si.ss_parts.sum(0)
    assert torch.allclose(ss[:M], (resid * resid).sum(1), rtol=1e-5) and (M % 16 == 0 or float(ss[M:].abs().max()) == 0.0)
    assert ss.shape[0] == -(-M // 16) * 16
    # 2. products of the normed rows: plain, float32 result (logits), gated
    for od in (torch.bfloat16, torch.float32):
        close(ops.decode_linear(si, ops.tile_weight(w_qkv), od), norm64(resid, wn1) @ w_qkv.double().t(), torch.bfloat16,
              scale=2.0, what="scaled decode_linear")
    y = norm64(resid, wn1) @ w_gu.double().t()
    close(ops.decode_linear_swiglu(si, ops.tile_weight(w_gu)), y[:, :I] / (1 + torch.exp(-y[:, :I])) * y[:, I:], torch.bfloat16,
          scale=2.0, what="scaled decode_linear_swiglu")
    # 3. a scaled input into a residual epilogue (the chain of two layers), with the second norm's weight
    w_sq = rnd((H, H), torch.bfloat16, dev, 38, 0.05)
    resid2 = resid.clone()
    si2 = ops.decode_linear_residual(si, ops.tile_weight(w_sq), resid2, wn2, eps)
    h2 = resid.double() + norm64(resid, wn1) @ w_sq.double().t()
    close(resid2, h2, torch.bfloat16, scale=2.0, what="stream after a scaled product")
    assert torch.equal(si2.xw.to_rows(), (resid2 * wn2.float()).bfloat16())
    # the same chain with row-major hand-over: the same numbers where both forms run through the same kernel (up to 16
    # rows); above that the kernels that walk or split differ by form and add in another order, and each form is held
    # against float64 by itself
    # (and where a tile per block fills the compute units evenly: with 320 column tiles for 256 units the products that hand
    # over in operand order split K over blocks from the first row on)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    same_kernel = M <= 16 and ((H // 16) % cus == 0 or H // 16 < cus // 4)
    ops.OPERAND_ORDER = False
    try:
        resid_r = resid0.clone()
        si_r = ops.decode_linear_residual(a, ops.tile_weight(w_in), resid_r, wn1, eps)
        assert not isinstance(si_r.xw, ops.OperandRows)
        qkv_r = ops.decode_linear(si_r, ops.tile_weight(w_qkv))
        g_rows = ops.decode_linear_swiglu(si_r, ops.tile_weight(w_gu), for_product=True)
        w_dn = rnd((H, I), torch.bfloat16, dev, 40, 0.05)
        rb = resid_r.clone()
        sb = ops.decode_linear_residual(g_rows, ops.tile_weight(w_dn), rb, wn2, eps)
    finally:
        ops.OPERAND_ORDER = True
    close(resid_r, h, torch.float32, scale=4.0, what="stream after the residual epilogue, row-major hand-over")
    assert torch.equal(si_r.xw, (resid_r * wn1.float()).bfloat16())
    y_r = norm64(resid_r, wn1) @ w_gu.double().t()
    close(qkv_r, norm64(resid_r, wn1) @ w_qkv.double().t(), torch.bfloat16, scale=2.0, what="scaled decode_linear, row-major hand-over")
    close(g_rows, y_r[:, :I] / (1 + torch.exp(-y_r[:, :I])) * y_r[:, I:], torch.bfloat16, scale=2.0, what="gated product, row-major hand-over")
    close(rb, resid_r.double() + g_rows.double() @ w_dn.double().t(), torch.float32, scale=4.0, what="down product, row-major hand-over")
    assert torch.equal(sb.xw, (rb * wn2.float()).bfloat16()) and torch.allclose(sb.ss_parts.sum(0)[:M], (rb * rb).sum(1), rtol=1e-5)
    g_tiled = ops.decode_linear_swiglu(si, ops.tile_weight(w_gu), for_product=True)
    assert isinstance(g_tiled, ops.OperandRows)
    if same_kernel:
        ra = resid.clone()
        sa = ops.decode_linear_residual(g_tiled, ops.tile_weight(w_dn), ra, wn2, eps)
        assert torch.equal(resid_r, resid) and torch.equal(si_r.xw, si.xw.to_rows())
        assert torch.equal(qkv_r, ops.decode_linear(si, ops.tile_weight(w_qkv))) and torch.equal(g_tiled.to_rows(), g_rows)
        assert torch.equal(ra, rb) and torch.equal(sa.xw.to_rows(), sb.xw) and torch.equal(sa.ss_parts, sb.ss_parts)
    # the down product (its input in operand order) against float64, K split where the shape allows
    rd = resid.clone()
    g_in = ops.decode_linear_swiglu(si, ops.tile_weight(w_gu), for_product=True)
    sd = ops.decode_linear_residual(g_in, ops.tile_weight(w_dn), rd, wn2, eps)
    close(rd, resid.double() + g_in.to_rows().double() @ w_dn.double().t(), torch.float32, scale=4.0, what="stream after the down product")
    assert torch.equal(sd.xw.to_rows(), (rd * wn2.float()).bfloat16())
    assert torch.allclose(sd.ss_parts.sum(0)[:M], (rd * rd).sum(1), rtol=1e-5)
    # 4. the scale matters: another eps or a missing part changes the result by far more than the tolerance
    far = ops.decode_linear(ops.ScaledInput(si.xw, si.ss_parts * 4.0, eps), ops.tile_weight(w_qkv), torch.float32)
    ref = (norm64(resid, wn1) @ w_qkv.double().t()).float()
    assert float((far - ref).abs().max()) > 0.3 * float(ref.abs().max())
    # 5. the embedding that starts such a chain
    table = rnd((50, H), torch.bfloat16, dev, 39)
    ids = torch.randint(0, 50, (M,), generator=torch.Generator().manual_seed(41)).int().to(dev)
    out, e = ops.embedding_scaled(ids, table, wn1, eps)
    assert torch.equal(out, ops.embedding(ids, table)) and torch.equal(e.xw.to_rows(), (out * wn1.float()).bfloat16())
    assert torch.allclose(e.ss_parts[0, :len(ids)], (out * out).sum(1), rtol=1e-5) and (len(ids) % 16 == 0 or float(e.ss_parts[0, len(ids):].abs().max()) == 0.0)


def _operand_rows(x):
    """[M, K] bfloat16 -> ops.OperandRows with the same values (rows beyond M: zeros)."""
    from spyinfer_amd.kernels import ops
    M, K = x.shape
    out = ops.OperandRows.empty(M, K, x.device)
    mt = out.tiles
    pad = torch.zeros((16 * mt, K), dtype=x.dtype, device=x.device)
    pad[:M] = x
    out.data.view(K // 32, mt, 4, 16, 8).copy_(pad.view(mt, 16, K // 32, 4, 8).permute(2, 0, 3, 1, 4))
    assert torch.equal(out.to_rows(), x)
    return out


@pytest.mark.parametrize("M,H,I,NQKV,eps", [(80, 4096, 12288, 6144, 1e-6), (128, 4096, 12288, 6144, 1e-6), (65, 5120, 6400, 6160, 1e-5),
                                            (100, 256, 384, 8208, 1e-6), (97, 128, 8320, 151936, 1e-6), (128, 4096, 36864, 64, 1e-6)])
def test_decode_products_beyond_64_rows(M, H, I, NQKV, eps):
    """65 to 128 rows (six or eight row tiles; inputs in operand order only): the chain residual product -> stored and
    gated products of the normed rows -> residual product of the gated result, each against float64; widths with a
    column tile per compute unit (K split over blocks), with many (blocks that walk), and small ones."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    resid0 = rnd((M, H), torch.float32, dev, 31, 1.5)
    wn1 = (1 + 0.1 * rnd((H,), torch.float32, dev, 32)).bfloat16()
    wn2 = (1 + 0.1 * rnd((H,), torch.float32, dev, 33)).bfloat16()
    w_in = rnd((H, I), torch.bfloat16, dev, 34, 0.05)
    w_qkv = rnd((NQKV, H), torch.bfloat16, dev, 35, 0.05)
    w_gu = rnd((2 * I, H), torch.bfloat16, dev, 36, 0.05)
    w_dn = rnd((H, I), torch.bfloat16, dev, 40, 0.05)
    a = rnd((M, I), torch.bfloat16, dev, 37)

    def norm64(h, w):
        h = h.double()
        return h * torch.rsqrt((h * h).mean(1, keepdim=True) + eps) * w.double()

    assert ops.row_tiles(M) == (6 if M <= 96 else 8)
    resid = resid0.clone()
    si = ops.decode_linear_residual(_operand_rows(a), ops.tile_weight(w_in), resid, wn1, eps)
    close(resid, resid0.double() + a.double() @ w_in.double().t(), torch.float32, scale=4.0, what="stream after the residual epilogue")
    assert isinstance(si.xw, ops.OperandRows) and torch.equal(si.xw.to_rows(), (resid * wn1.float()).bfloat16())
    ss = si.ss_parts.sum(0)
    assert ss.shape[0] == 16 * ops.row_tiles(M) and torch.allclose(ss[:M], (resid * resid).sum(1), rtol=1e-5) and (M == ss.shape[0] or float(ss[M:].abs().max()) == 0.0)
    for od in (torch.bfloat16, torch.float32):
        close(ops.decode_linear(si, ops.tile_weight(w_qkv), od), norm64(resid, wn1) @ w_qkv.double().t(), torch.bfloat16, scale=2.0,
              what="scaled decode_linear")
    y = norm64(resid, wn1) @ w_gu.double().t()
    gated = y[:, :I] / (1 + torch.exp(-y[:, :I])) * y[:, I:]
    close(ops.decode_linear_swiglu(si, ops.tile_weight(w_gu)), gated, torch.bfloat16, scale=2.0, what="gated product, row-major result")
    g = ops.decode_linear_swiglu(si, ops.tile_weight(w_gu), for_product=True)
    assert isinstance(g, ops.OperandRows)
    close(g.to_rows(), gated, torch.bfloat16, scale=2.0, what="gated product, result in operand order")
    rd = resid.clone()
    sd = ops.decode_linear_residual(g, ops.tile_weight(w_dn), rd, wn2, eps)
    close(rd, resid.double() + g.to_rows().double() @ w_dn.double().t(), torch.float32, scale=4.0, what="stream after the down product")
    assert torch.equal(sd.xw.to_rows(), (rd * wn2.float()).bfloat16()) and torch.allclose(sd.ss_parts.sum(0)[:M], (rd * rd).sum(1), rtol=1e-5)
    # what is not built beyond 64 rows is refused, not computed wrongly: a row-major input
    with pytest.raises(ops.KernelError, match="operand order"):
        ops.decode_linear_residual(a, ops.tile_weight(w_in), resid.clone(), wn1, eps)
    table = rnd((50, H), torch.bfloat16, dev, 39)
    ids = torch.randint(0, 50, (M,), generator=torch.Generator().manual_seed(41)).int().to(dev)
    out, e = ops.embedding_scaled(ids, table, wn1, eps)
    assert torch.equal(out, ops.embedding(ids, table)) and torch.equal(e.xw.to_rows(), (out * wn1.float()).bfloat16())
    assert torch.allclose(e.ss_parts[0, :M], (out * out).sum(1), rtol=1e-5) and (M == e.ss_parts.shape[1] or float(e.ss_parts[0, M:].abs().max()) == 0.0)


def test_products_with_k_split_over_blocks_repeat_exactly():
    """The product whose blocks hand their partial sums to the last block of a column group (long K, about a column
    tile per compute unit): 40 calls in a row without a wait between them, on changing inputs, give bit for bit what
    the same inputs gave before, and what float64 gives within the tolerance.  A part read before it was written, or
    a counter not left at zero, would show as a difference."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    M, N, K = 64, 4096, 12288
    w = rnd((N, K), torch.bfloat16, dev, 51, 0.02)
    wt = ops.tile_weight(w)
    wn = (1 + 0.1 * rnd((N,), torch.float32, dev, 52)).bfloat16()
    xs = []
    for i in range(4):
        x = ops.OperandRows.empty(M, K, dev)
        x.data.copy_(rnd(tuple(x.data.shape), torch.bfloat16, dev, 60 + i))
        xs.append(x)
    first = {}
    for call in range(40):
        i = call % 4
        resid = torch.zeros((M, N), dtype=torch.float32, device=dev)
        si = ops.decode_linear_residual(xs[i], wt, resid, wn, 1e-6)
        if i in first:
            assert torch.equal(resid, first[i][0]) and torch.equal(si.xw.data, first[i][1]) and torch.equal(si.ss_parts, first[i][2]), "call %d" % call
        else:
            first[i] = (resid, si.xw.data.clone(), si.ss_parts.clone())
    for i in range(4):
        close(first[i][0], xs[i].to_rows().double() @ w.double().t(), torch.float32, scale=4.0, what="input %d" % i)
    assert int(ops.decode_workspace(dev)[:16384].max()) == 0, "the counters are left at zero"


def test_decode_products_refuse_wrong_operands():
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    w = ops.tile_weight(rnd((64, 128), torch.bfloat16, dev, 1))
    with pytest.raises(ops.KernelError, match="rows"):
        ops.decode_linear(rnd((ops.FUSED_DECODE_MAX_ROWS + 1, 128), torch.bfloat16, dev, 2), w)
    with pytest.raises(ops.KernelError, match="bfloat16"):
        ops.decode_linear(rnd((4, 128), torch.float32, dev, 2), w)
    with pytest.raises(ops.KernelError, match="stream"):
        ops.decode_linear_residual(rnd((4, 128), torch.bfloat16, dev, 2), w, torch.zeros(4, 128, device=dev),
                                   torch.ones(64, dtype=torch.bfloat16, device=dev), 1e-6)
    with pytest.raises(ops.KernelError, match="parts"):
        ops.decode_linear(ops.ScaledInput(rnd((4, 128), torch.bfloat16, dev, 2), torch.zeros(3, 8, device=dev), 1e-6), w)


def test_linear_reference_vector():
    """test/test_linear.cpp:53-60 of the reference: x . W^T before the bias."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = torch.tensor([[1., 2, 3], [4, 5, 6]], device=dev)
    w = torch.tensor([[1., 2, 3], [4, 5, 6], [7, 8, 9], [10, 11, 12]], device=dev)
    assert ops.linear(x, w).cpu().tolist() == [[14, 32, 50, 68], [32, 77, 122, 167]]


def test_linear_float32_is_true_float32():
    """No reduced-precision matrix mode: products of numbers that need 24 bits come out exact."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = torch.tensor([[1.0 + 2 ** -20, 1.0]], device=dev)
    w = torch.tensor([[1.0, -1.0]], device=dev)
    assert ops.linear(x, w).item() == 2 ** -20


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_mixed_weight_dtype(dtype):
    """A weight stored in 32-bit stays so, beside bfloat16 activations."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = rnd((5, 72), dtype, dev, 8)
    w = rnd((40, 72), torch.float32, dev, 9)
    close(ops.linear(x, w), x.double() @ w.double().t(), dtype, scale=8.0, what="mixed linear")


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(dtype):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    # ramp of the reference's test (test/test_swiglu.cpp:43-46)
    n = 100100
    i = torch.arange(n)
    gate = ((i % 100).float() / 10.0 - 5.0)
    up = ((i % 70).float() / 15.0 - 2.0)
    T, I = 100, 1001
    gu = torch.cat([gate.view(T, I), up.view(T, I)], dim=1).to(dtype).to(dev)
    out = ops.swiglu(gu)
    g, u = gu[:, :I].double(), gu[:, I:].double()
    close(out, g / (1 + torch.exp(-g)) * u, dtype, what="swiglu")
    edge = torch.tensor([[0.0, 30.0, -30.0, 3.0, 3.0, 3.0]], dtype=dtype, device=dev)
    o = ops.swiglu(edge).float().cpu()[0]
    assert o[0] == 0 and abs(o[1] - 90) < 0.5 and abs(o[2]) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(1, 160, 96), (7, 200, 88), (16, 1000, 1024), (8, 12288, 4096), (40, 128, 64), (3, 24, 20)])
def test_linear_swiglu(dtype, M, I, K):
    """Gate and up products with the SwiGLU in one call (one kernel for few bfloat16 rows)."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    x = rnd((M, K), dtype, dev, 15)
    w = rnd((2 * I, K), dtype, dev, 16, 0.05)
    y = x.double() @ w.double().t()
    g, u = y[:, :I], y[:, I:]
    out = ops.linear_swiglu(x, w)
    assert out.shape == (M, I) and out.dtype == dtype
    close(out, g / (1 + torch.exp(-g)) * u, dtype, scale=2.0, what="linear_swiglu")


def plain_qk(qkv, n_q, n_kv, d, qw, kw, eps, theta, rot, pos):
    T = qkv.shape[0]
    x = qkv.double()
    q = x[:, :n_q * d].view(T, n_q, d)
    k = x[:, n_q * d:(n_q + n_kv) * d].view(T, n_kv, d)
    v = x[:, (n_q + n_kv) * d:].view(T, n_kv, d)
    if qw is not None:
        q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * qw.double()
        k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * kw.double()
    if rot:
        half = rot // 2
        freq = theta ** (-torch.arange(half, dtype=torch.float64) / half)
        ang = pos.double()[:, None] * freq[None]
        # complex form of the half-split rotation: (x[j] + i x[j + half]) * exp(i p freq_j)
        def r(t):
            z = torch.complex(t[..., :half], t[..., half:rot]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
            return torch.cat([z.real, z.imag, t[..., rot:]], -1)
        q, k = r(q), r(k)
    return q, k, v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_q,n_kv,d,rot,P,norm", [(4, 2, 16, 16, 16, True), (8, 2, 32, 32, 8, True), (6, 3, 48, 48, 16, True),
                                                   (3, 1, 80, 40, 4, False), (32, 8, 128, 128, 16, True), (5, 5, 256, 256, 32, True),
                                                   (2, 2, 64, 64, 16, False)])
@pytest.mark.parametrize("T", [23, 150])
def test_qk_norm_rope_store(dtype, n_q, n_kv, d, rot, P, norm, T):
    """T = 150 takes, in bfloat16 and for head sizes that allow it, the kernel with 16-byte accesses; its slots hold runs
    of tokens that follow each other in a page from an aligned slot (stored in pieces of 8), runs from an unaligned
    slot, scattered slots and a token without a slot."""
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts.rotary import RotaryEmbedding
    dev = require_gpu()
    pages, theta, eps = (9 if T == 23 else 2 * T // P + 4), 12345.0, 1e-5
    qkv = rnd((T, (n_q + 2 * n_kv) * d), dtype, dev, 10)
    qw = (1 + 0.2 * rnd((d,), torch.float32, dev, 11)).to(dtype) if norm else None
    kw = (1 + 0.2 * rnd((d,), torch.float32, dev, 12)).to(dtype) if norm else None
    pos = torch.randint(0, 500, (T,), generator=torch.Generator().manual_seed(13)).int()
    rope = RotaryEmbedding(d, theta, rot)
    rope.prepare(dev, 512)
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(14))[:T].int()
    if T > 100:
        free = [x for x in range(120, pages * P)]
        rest = torch.tensor(free)[torch.randperm(len(free), generator=torch.Generator().manual_seed(15))][:T - 75].int()
        slots = torch.cat([torch.arange(8, 8 + 45).int(), torch.arange(67, 67 + 30).int(), rest])
    slots[3] = -1
    kc = torch.full((pages, n_kv, P, d), 7.0, dtype=dtype, device=dev)
    vc = torch.full((pages, n_kv, d, P), 7.0, dtype=dtype, device=dev)
    q = ops.qk_norm_rope_store(qkv, n_q, n_kv, d, qw, kw, eps, rope.cos, rope.sin, rot, pos.to(dev), kc, vc, P, slots.to(dev))
    rq, rk, rv = plain_qk(qkv.cpu(), n_q, n_kv, d, None if qw is None else qw.cpu(), None if kw is None else kw.cpu(), eps, theta, rot, pos)
    # angles reach 500 rad in float32: allow for their rounding (|x| * 500 * 2^-24 * few)
    close(q.view(T, n_q, d), rq, dtype, scale=8.0, what="q")
    kc_ref = torch.full((pages, n_kv, P, d), 7.0, dtype=torch.float64)
    vc_ref = torch.full((pages, n_kv, d, P), 7.0, dtype=torch.float64)
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            kc_ref[s // P, :, s % P, :] = rk[t]
            vc_ref[s // P, :, :, s % P] = rv[t]
    close(kc, kc_ref, dtype, scale=8.0, what="k cache")
    assert torch.equal(vc.cpu().double(), vc_ref.to(dtype).double()), "values must be stored unchanged"


def plain_paged_attention(q, kc, vc, P, bt, token_entry, positions, n_q, n_kv, d, scale, window):
    T = q.shape[0]
    out = torch.zeros(T, n_q, d, dtype=torch.float64)
    qd = q.double().view(T, n_q, d)
    for t in range(T):
        s, p = int(token_entry[t]), int(positions[t])
        lo = 0 if not window else max(0, p - window + 1)
        keys = range(lo, p + 1)
        K = torch.stack([kc[bt[s][c // P], :, c % P, :] for c in keys]).double()
        V = torch.stack([vc[bt[s][c // P], :, :, c % P] for c in keys]).double()
        for h in range(n_q):
            g = h * n_kv // n_q
            pr = torch.softmax((K[:, g] @ qd[t, h]) * scale, 0)
            out[t, h] = pr @ V[:, g]
    return out.view(T, n_q * d)


def make_attention_case(dtype, dev, n_q, n_kv, d, P, entries, seed, window=None, spike=False, big_rows=128):
    """entries: list of (tokens already cached, tokens in this step).  Pages are dealt in a random
    order; unused pages and slots hold NaN."""
    from spyinfer_amd.kernels.ops import AttentionMeta
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(a + n) // P) for a, n in entries) + 3
    order = torch.randperm(total_pages, generator=g).tolist()
    kc = torch.full((total_pages, n_kv, P, d), float("nan"), dtype=dtype)
    vc = torch.full((total_pages, n_kv, d, P), float("nan"), dtype=dtype)
    bt, cu, pos0, kvl, te, ps = [], [0], [], [], [], []
    maxb = max(-(-(a + n) // P) for a, n in entries)
    for s, (a, n) in enumerate(entries):
        nb = -(-(a + n) // P)
        pages = [order.pop() for _ in range(nb)]
        bt.append(pages + [-1] * (maxb - nb))
        for c in range(a + n):
            kc[pages[c // P], :, c % P, :] = torch.randn(n_kv, d, generator=g).to(dtype)
            vc[pages[c // P], :, :, c % P] = torch.randn(n_kv, d, generator=g).to(dtype)
        cu.append(cu[-1] + n); pos0.append(a); kvl.append(a + n)
        te += [s] * n; ps += list(range(a, a + n))
    T = cu[-1]
    q = torch.randn(T, n_q * d, generator=g).to(dtype)
    if spike:
        # one far key per request gets a score that stands out: a kernel that skips or misplaces it fails
        for s, (a, n) in enumerate(entries):
            if a + n > 3:
                c = 1
                t = cu[s + 1] - 1
                for h in range(n_q):
                    gk = h * n_kv // n_q
                    kc[bt[s][c // P], gk, c % P, :] = (q[t].view(n_q, d)[h].float() * 1.5).to(dtype)
    G = n_q // n_kv
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    tiles = {}
    for kind, size in (("small", 16), ("big", big_rows)):
        tile_entry, tile_row0 = [], []
        for s, (a, n) in enumerate(entries):
            is_big = n * G >= 64 and d <= 128 and P & (P - 1) == 0
            if is_big == (kind == "big"):
                for r0 in range(0, n * G, size):
                    tile_entry.append(s); tile_row0.append(r0)
        tiles[kind] = (i32(tile_entry), i32(tile_row0), len(tile_entry))
    meta = AttentionMeta(i32(cu), i32(pos0), i32(kvl), i32(bt), i32(te), i32(ps), len(entries), T, maxb, max(kvl),
                         max(n for _, n in entries), tiles, G, big_rows=big_rows)
    return q, kc, vc, bt, te, ps, meta


ATT_CASES = [
    # n_q, n_kv, d, P, entries (cached, new), window
    (4, 2, 16, 16, [(0, 5)], None),
    (8, 2, 32, 8, [(0, 1), (0, 40), (7, 2)], None),
    (6, 3, 48, 16, [(0, 70), (33, 1), (100, 1), (15, 17)], None),
    (32, 8, 128, 16, [(300, 1), (17, 1), (0, 33)], None),
    (5, 5, 64, 32, [(0, 50), (90, 3)], None),
    (16, 1, 80, 16, [(130, 1), (0, 21)], None),
    (8, 4, 128, 16, [(0, 150), (140, 10), (149, 1)], 37),
    (4, 4, 256, 64, [(60, 9), (0, 3)], None),
    (3, 1, 112, 4, [(0, 19), (30, 1)], 8),
    (32, 8, 128, 16, [(1151, 1), (70, 1), (2000, 1), (0, 1)], None),      # single tokens only: keys split into parts
    (6, 2, 96, 8, [(700, 1), (333, 1)], 100),
    (16, 2, 64, 16, [(200, 100), (0, 3)], None),                            # a long portion that starts late: 800 rows
    (4, 4, 96, 32, [(50, 90), (0, 257)], None),
    (8, 2, 128, 8, [(0, 300), (64, 64), (500, 1)], 130),
    (4, 2, 64, 16, [(900, 70), (1300, 40)], None),                          # few big tiles, many keys: key parts + merge
    (8, 2, 128, 16, [(1500, 33)], 700),
    (8, 2, 64, 24, [(100, 1), (0, 30), (47, 2), (500, 1)], None),           # pages that are no power of two
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(ATT_CASES)))
@pytest.mark.parametrize("mfma", [False, True, 256])
def test_paged_attention(dtype, case, mfma):
    """mfma: False = the float32 kernel, True = the MFMA kernels with 128-row tiles for entries of many rows, 256 = the
    same with 256-row tiles (head sizes 64 and 128)."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    n_q, n_kv, d, P, entries, window = ATT_CASES[case]
    if mfma and not (dtype == torch.bfloat16 and d % 16 == 0 and P % 8 == 0):
        pytest.skip("the MFMA kernel takes bfloat16, head sizes in steps of 16 and pages of a multiple of 8")
    big_rows = 128
    if mfma == 256:
        if d not in (64, 128) or P & (P - 1) or not any(n * (n_q // n_kv) >= 64 for _, n in entries):
            pytest.skip("tiles of 256 rows are for head sizes 64 and 128 and entries of many rows")
        big_rows = 256
    q, kc, vc, bt, te, ps, meta = make_attention_case(dtype, dev, n_q, n_kv, d, P, entries, seed=case, window=window, spike=True,
                                                      big_rows=big_rows)
    scale = 1.0 / math.sqrt(d)
    ref = plain_paged_attention(q, kc, vc, P, bt, te, ps, n_q, n_kv, d, scale, window)
    old = ops.MFMA_ATTENTION
    ops.MFMA_ATTENTION = bool(mfma)
    try:
        out = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), P, meta, n_q, n_kv, d, scale, window)
    finally:
        ops.MFMA_ATTENTION = old
    close(out, ref, dtype, scale=2.0, what="attention case %d" % case)


@pytest.mark.parametrize("case", [(8, 2, 128, 16, [(700, 1), (333, 1), (90, 1)], 100), (4, 4, 64, 16, [(500, 3), (77, 1), (260, 2)], 70),
                                  (6, 2, 96, 8, [(300, 1), (40, 2)], 33),
                                  (8, 2, 128, 16, [(600, 40), (900, 1)], 200), (4, 1, 64, 32, [(1000, 100)], 300)])
def test_pages_that_a_window_has_passed_are_not_read(case):
    """Under a window a request gives back the pages that no later query reads, and its block table says -1 there.  A
    kernel's first block of keys may begin inside such a page (blocks are aligned, windows are not): those keys are
    masked, and what lies in page 0 in their place must not reach the result.  Here page 0 holds NaN and belongs to
    nobody, every page that the window has passed is taken out of the tables, and the result must be that of the keys
    inside the window: single tokens, short portions and portions that the prefill kernel takes, full head sizes and one
    that is not."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    n_q, n_kv, d, P, entries, window = case
    dtype = torch.bfloat16
    q, kc, vc, bt, te, ps, meta = make_attention_case(dtype, dev, n_q, n_kv, d, P, entries, seed=n_q, window=window, spike=True)
    scale = 1.0 / math.sqrt(d)
    ref = plain_paged_attention(q, kc, vc, P, bt, te, ps, n_q, n_kv, d, scale, window)
    nan_page = lambda t: torch.full_like(t[:1], float("nan"))
    kc2, vc2 = torch.cat([nan_page(kc), kc]), torch.cat([nan_page(vc), vc])              # every page one further on, page 0 poisoned
    table = torch.tensor(bt, dtype=torch.int32)
    table = torch.where(table >= 0, table + 1, table)
    gone = 0
    for s, (a, n) in enumerate(entries):
        passed = max(0, a - window + 1) // P                                              # the first query of the step sits at position a
        table[s, :passed] = -1
        gone += passed
    assert gone > 10
    meta.block_table = table.to(dev)
    out = ops.paged_attention(q.to(dev), kc2.to(dev), vc2.to(dev), P, meta, n_q, n_kv, d, scale, window)
    close(out, ref, dtype, scale=2.0, what="window %d over pages given back" % window)


def _long_case(dtype, dev, n_q, n_kv, d, P, entries, seed, big_rows=128):
    """As make_attention_case, for thousands of keys: filled and gathered with tensor operations.  Returns also the
    keys and values of each entry in order, for the reference."""
    from spyinfer_amd.kernels.ops import AttentionMeta
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(a + n) // P) for a, n in entries) + 5
    order = torch.randperm(total_pages, generator=g)
    kc = torch.full((total_pages, n_kv, P, d), float("nan"), dtype=dtype)
    vc = torch.full((total_pages, n_kv, d, P), float("nan"), dtype=dtype)
    maxb = max(-(-(a + n) // P) for a, n in entries)
    bt = torch.full((len(entries), maxb), -1, dtype=torch.int64)
    cu, used, kept = [0], 0, []
    for s, (a, n) in enumerate(entries):
        L, nb = a + n, -(-(a + n) // P)
        bt[s, :nb] = order[used:used + nb]
        used += nb
        K, V = torch.randn(L, n_kv, d, generator=g).to(dtype), torch.randn(L, n_kv, d, generator=g).to(dtype)
        kept.append((K, V))
        cu.append(cu[-1] + n)
    q = torch.randn(cu[-1], n_q * d, generator=g).to(dtype)
    for s, (a, n) in enumerate(entries):
        K, V = kept[s]
        # far keys that the last query of the entry scores high: one near the start, one at a page's first slot deep inside
        for c in (3, ((a + n) // 2) // P * P):
            for h in range(n_q):
                K[c, h * n_kv // n_q] = (q[cu[s + 1] - 1].view(n_q, d)[h].float() * 1.2).to(dtype)
        c = torch.arange(a + n)
        kc[bt[s][c // P], :, c % P, :] = K
        vc[bt[s][c // P], :, :, c % P] = V
    G = n_q // n_kv
    i32 = lambda x: torch.as_tensor(x, dtype=torch.int32).to(dev)
    tiles = {}
    for kind, size in (("small", 16), ("big", big_rows)):
        te, tr = [], []
        for s, (a, n) in enumerate(entries):
            if (n * G >= 64) == (kind == "big"):
                te += [s] * len(range(0, n * G, size)); tr += list(range(0, n * G, size))
        if kind == "big":                       # sorted by the keys read, most first, as the engine does
            keys = [entries[s][0] + min(entries[s][1], (r0 + size + G - 1) // G) for s, r0 in zip(te, tr)]
            idx = sorted(range(len(te)), key=lambda i: -keys[i])
            te, tr = [te[i] for i in idx], [tr[i] for i in idx]
        tiles[kind] = (i32(te), i32(tr), len(te))
    token_entry = [s for s, (a, n) in enumerate(entries) for _ in range(n)]
    positions = [a + i for a, n in entries for i in range(n)]
    meta = AttentionMeta(i32(cu), i32([a for a, n in entries]), i32([a + n for a, n in entries]), i32(bt), i32(token_entry),
                         i32(positions), len(entries), cu[-1], maxb, max(a + n for a, n in entries), max(n for _, n in entries), tiles, G,
                         big_rows=big_rows)
    return q, kc, vc, kept, cu, meta


@pytest.mark.parametrize("case", [(32, 8, 128, 16, [(9000, 1), (8191, 1), (4000, 1)]),        # 16 key parts and the merge
                                  (8, 2, 128, 16, [(8800, 200), (0, 300)]),                   # few 128-row tiles far into a request: key parts
                                  (16, 2, 64, 32, [(9100, 70), (5000, 1)])])                   # both kernels in one step
@pytest.mark.parametrize("big_rows", [128, 256])
def test_paged_attention_over_9000_keys(case, big_rows):
    """The lengths that the benchmarks run (15 000-key decode steps, portions late in 16 000-token prompts): block tables
    of hundreds of pages, the most key parts, tiles sorted by work.  Reference: float64 softmax over the entry's keys."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    n_q, n_kv, d, P, entries = case
    dtype = torch.bfloat16
    q, kc, vc, kept, cu, meta = _long_case(dtype, dev, n_q, n_kv, d, P, entries, seed=len(entries) + n_q, big_rows=big_rows)
    assert ops.key_parts_for(meta.max_kv_len) == 16
    scale = 1.0 / math.sqrt(d)
    out = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), P, meta, n_q, n_kv, d, scale, None).cpu().double()
    for s, (a, n) in enumerate(entries):
        K, V = (x.double() for x in kept[s])
        qs = q[cu[s]:cu[s + 1]].double().view(n, n_q, d)
        kv_of = torch.arange(n_q) * n_kv // n_q
        scores = torch.einsum("thd,chd->thc", qs, K[:, kv_of]) * scale
        masked = torch.arange(a + n)[None, :] > (a + torch.arange(n))[:, None]
        pr = torch.softmax(scores.masked_fill(masked[:, None, :], float("-inf")), dim=-1)
        ref = torch.einsum("thc,chd->thd", pr, V[:, kv_of]).reshape(n, n_q * d)
        # the far keys carry weight: for the last query head of a group (whose query the keys were made from) the
        # largest probability of the entry's last token lies on one of them
        assert int(pr[-1, n_q // n_kv - 1].argmax()) in (3, ((a + n) // 2) // P * P)
        close(out[cu[s]:cu[s + 1]], ref, dtype, scale=2.0, what="entry %d of %r" % (s, entries))


FUSED_CASES = [
    # n_q, n_kv, d, P, cached tokens of each single-token entry, window, norm, rotation
    (32, 8, 128, 16, [1151, 70, 2000, 0, 15, 16, 31, 32], None, True, True),
    (4, 1, 64, 16, [5, 0, 200], None, False, True),
    (8, 8, 256, 32, [300, 63, 64], 50, True, False),
    (16, 1, 64, 8, [99, 7], None, True, True),
    (6, 2, 128, 16, [33], 8, False, False),
    (8, 2, 128, 16, [(37 * i) % 700 for i in range(100)], None, True, True),      # 100 single tokens: seven row tiles of output
    (8, 2, 128, 24, [500, 47, 23, 24, 95], None, True, True),                     # pages that are no power of two
    (4, 2, 64, 40, [333, 79, 80, 600], 120, True, True),                          # the same under a window
]


def _with_pieces(meta, kv_len, n_kv, window, d, dev):
    """The step's keys cut on the host, as the attention part plans them."""
    from spyinfer_amd.kernels import ops
    rec = key_pieces.decode_pieces(kv_len, n_kv, int(window or 0), head_dim=d)
    meta.pieces = {(n_kv, int(window or 0), d): torch.from_numpy(rec).to(dev)}
    return rec


@pytest.mark.parametrize("case", range(len(FUSED_CASES)))
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("keys_per_part", [256, 32])
@pytest.mark.parametrize("cut", ["evenly", "by_the_host"])
def test_attention_taking_the_raw_product(case, wdtype, keys_per_part, cut, monkeypatch):
    """Single tokens: the attention kernel norms and rotates q and the new key itself, uses the new key and value and
    stores them.  The slots of the new tokens hold NaN before the call, so a kernel that read them before writing, or
    did not write, fails; the rest of the cache must stay as it was.  Positions at the edges of pages and of 32-key
    blocks; few and many parts of the keys, all entries in the same number of parts or cut by the host into pieces of
    even size."""
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts.rotary import RotaryEmbedding
    dev = require_gpu()
    n_q, n_kv, d, P, cached, window, norm, rotate = FUSED_CASES[case]
    dtype, theta, eps = torch.bfloat16, 23456.0, 1e-5
    entries = [(a, 1) for a in cached]
    _q, kc, vc, bt, te, ps, meta = make_attention_case(dtype, dev, n_q, n_kv, d, P, entries, seed=50 + case, window=window)
    monkeypatch.setattr(ops, "DECODE_KEYS_PER_SPLIT", keys_per_part)
    if cut == "by_the_host":
        if d > 128:
            pytest.skip("head sizes beyond 128 are not cut by the host")
        monkeypatch.setattr(key_pieces, "PIECE_MIN_BLOCKS", keys_per_part // 32)
        if keys_per_part < 256:                  # as many parts as there can be
            for name, value in (("PIECE_UNITS", 64 * len(cached)), ("PIECE_START_US", 0.0), ("PIECE_MERGE_US", 0.0), ("PIECE_MERGE_MORE_US", 0.0),
                                ("PIECE_ROUND_US", 0.0)):
                monkeypatch.setattr(key_pieces, name, value)
        rec = _with_pieces(meta, [a + 1 for a in cached], n_kv, window, d, dev)
        assert keys_per_part == 256 or max(cached) < 128 or rec[:, 5].max() > 1
        # (more than sixteen parts: the merging block's third and fourth round of eight)
        assert keys_per_part == 256 or max(cached) < 600 or window or rec[:, 5].max() > 16
    T = len(entries)
    qkv = rnd((T, (n_q + 2 * n_kv) * d), dtype, "cpu", 60 + case)
    qw = (1 + 0.2 * rnd((d,), torch.float32, "cpu", 61)).to(wdtype) if norm else None
    kw = (1 + 0.2 * rnd((d,), torch.float32, "cpu", 62)).to(wdtype) if norm else None
    pos = torch.tensor(cached, dtype=torch.int32)
    rope = RotaryEmbedding(d, theta, d)
    rope.prepare(dev, 2100)
    rq, rk, rv = plain_qk(qkv, n_q, n_kv, d, qw, kw, eps, theta, d if rotate else 0, pos)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    kc_dev, vc_dev = kc.clone(), vc.clone()
    for s, a in enumerate(cached):
        page = bt[s][a // P]
        kc_ref[page, :, a % P, :] = rk[s].to(dtype)
        vc_ref[page, :, :, a % P] = rv[s].to(dtype)
        kc_dev[page, :, a % P, :] = float("nan")
        vc_dev[page, :, :, a % P] = float("nan")
    scale = 1.0 / math.sqrt(d) if case % 2 == 0 else 0.21                # (a model may bring a scale of its own)
    ref = plain_paged_attention(rq.reshape(T, n_q * d).to(dtype), kc_ref, vc_ref, P, bt, te, ps, n_q, n_kv, d, scale, window)
    kc_dev, vc_dev = kc_dev.to(dev), vc_dev.to(dev)
    assert ops.fused_attention_ok(dtype, meta, n_q, n_kv, d, P, d if rotate else 0, qw, kw)
    raw = ops.RawQKV(qkv.to(dev), None if qw is None else qw.to(dev), None if kw is None else kw.to(dev), eps,
                     rope.cos if rotate else None, rope.sin if rotate else None, True)
    out = ops.paged_attention(None, kc_dev, vc_dev, P, meta, n_q, n_kv, d, scale, window, raw)
    close(out, ref, dtype, scale=3.0, what="fused attention case %d" % case)
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float().cpu(), nan=-77.0), torch.nan_to_num(b.float(), nan=-77.0))
    assert same(vc_dev, vc_ref), "values must be stored unchanged, and nothing else written"
    new = torch.zeros(kc.shape[:3], dtype=torch.bool)
    for s, a in enumerate(cached):
        new[bt[s][a // P], :, a % P] = True
    assert same(kc_dev[~new.to(dev)], kc_ref[~new]), "keys of other positions must stay as they were"
    close(kc_dev[new.to(dev)], kc_ref[new], dtype, scale=8.0, what="stored keys")
    # the same result in operand order, for the product that reads it next
    if T <= ops.FUSED_DECODE_MAX_ROWS:
        kc3, vc3 = kc_ref.to(dev), vc_ref.to(dev)
        o3 = ops.paged_attention(None, kc3, vc3, P, meta, n_q, n_kv, d, scale, window, raw, for_product=True)
        assert isinstance(o3, ops.OperandRows) and torch.equal(o3.to_rows(), out)
    # store = False: nothing is written and the new position is not read (the cache of another call)
    kc2, vc2 = kc_ref.to(dev), vc_ref.to(dev)
    raw.store = False
    out2 = ops.paged_attention(None, kc2, vc2, P, meta, n_q, n_kv, d, scale, window, raw)
    close(out2, ref, dtype, scale=3.0, what="fused attention without store, case %d" % case)
    assert same(kc2, kc_ref) and same(vc2, vc_ref)


@pytest.mark.parametrize("case", [(16, 4, 128, 16, 40, 2600, None), (8, 8, 64, 32, 70, 900, None), (32, 8, 128, 16, 9, 6000, 1500),
                                  (16, 2, 128, 16, 130, 400, None), (16, 8, 128, 16, 3, 16000, None), (8, 8, 64, 16, 2, 16000, None)])
def test_attention_of_requests_of_uneven_lengths_cut_by_the_host(case):
    """Dozens of single tokens whose requests have a few to thousands of keys: the host cuts the long ones into pieces,
    leaves the short ones whole, and the kernel's blocks take one piece each.  Every entry's far keys carry weight.
    Reference: float64 softmax over the entry's keys, the new key normed and rotated, in its place."""
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts.rotary import RotaryEmbedding
    dev = require_gpu()
    n_q, n_kv, d, P, S, top, window = case
    dtype, theta, eps = torch.bfloat16, 1e6, 1e-6
    gen = torch.Generator().manual_seed(S)
    cached = torch.randint(4, top, (S,), generator=gen).tolist()
    cached[0], cached[1] = 3 * top, 5
    entries = [(a, 1) for a in cached]
    _q, kc, vc, kept, cu, meta = _long_case(dtype, dev, n_q, n_kv, d, P, entries, seed=S)
    rec = _with_pieces(meta, [a + 1 for a in cached], n_kv, window, d, dev)
    assert rec[:, 5].max() > 1 and (rec[rec[:, 0] >= 0][:, 5] == 1).any(), "some entries cut, some whole"
    assert S > 3 or rec[:, 5].max() > 24, "a long request beside one or two others: more parts than sixteen"
    qkv = rnd((S, (n_q + 2 * n_kv) * d), dtype, "cpu", 7)
    qw, kw = ((1 + 0.2 * rnd((d,), torch.float32, "cpu", 8 + i)).to(dtype) for i in range(2))
    rope = RotaryEmbedding(d, theta, d)
    rope.prepare(dev, 3 * top + 1)
    rq, rk, rv = plain_qk(qkv, n_q, n_kv, d, qw, kw, eps, theta, d, torch.tensor(cached))
    # the far keys that _long_case planted follow its own queries; plant them again for the queries of this step
    kc = kc.clone()
    kv_of = torch.arange(n_q) * n_kv // n_q
    for s, a in enumerate(cached):
        K, V = kept[s]
        lo = max(0, a - window + 1) if window else 0
        for c in {min(a, lo + 3), (lo + a) // 2 // P * P}:
            if lo <= c < a:
                for h in range(n_q):
                    K[c, kv_of[h]] = (rq[s, h] * 1.2).to(dtype)
                kc[meta.block_table[s, c // P].item(), :, c % P, :] = K[c]
    raw = ops.RawQKV(qkv.to(dev), qw.to(dev), kw.to(dev), eps, rope.cos, rope.sin, True)
    scale = 1.0 / math.sqrt(d)
    kc_dev, vc_dev = kc.to(dev), vc.to(dev)
    out = ops.paged_attention(None, kc_dev, vc_dev, P, meta, n_q, n_kv, d, scale, window, raw).cpu().double()
    for s, a in enumerate(cached):
        K, V = (x.double().clone() for x in kept[s])
        K[a], V[a] = rk[s].to(dtype).double(), rv[s].to(dtype).double()
        lo = max(0, a - window + 1) if window else 0
        scores = torch.einsum("hd,chd->hc", rq[s].to(dtype).double(), K[lo:a + 1, kv_of]) * scale
        pr = torch.softmax(scores, dim=-1)
        ref = torch.einsum("hc,chd->hd", pr, V[lo:a + 1, kv_of]).reshape(1, n_q * d)
        close(out[s:s + 1], ref, dtype, scale=3.0, what="entry %d with %d keys" % (s, a + 1))
        # the new key and value are in the cache
        page = meta.block_table[s, a // P].item()
        close(kc_dev[page, :, a % P, :], rk[s], dtype, scale=8.0, what="stored key of entry %d" % s)
        assert torch.equal(vc_dev[page, :, :, a % P].cpu().double(), rv[s].to(dtype).double())
    assert ops.workspace_counters_clean(dev)


@pytest.mark.parametrize("case", range(len(ATT_CASES)))
@pytest.mark.parametrize("big_rows", [128, 256])
def test_attention_output_in_operand_order(case, big_rows):
    """Steps of at most 128 tokens can hand the attention's output over in MFMA operand order: the values are those of
    the ordinary output, element for element (portions through the 16-row tiles and through the 128- and 256-row tiles,
    single tokens, their mix, one and several key parts)."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    n_q, n_kv, d, P, entries, window = ATT_CASES[case]
    if not ops.mfma_attention_ok(torch.bfloat16, d, P):
        pytest.skip("the MFMA kernels take head sizes in steps of 16 and pages of a multiple of 8")
    big = d <= 128 and P & (P - 1) == 0 and any(n * (n_q // n_kv) >= 64 for _, n in entries)
    if big_rows == 256 and not (big and d in (64, 128)):
        pytest.skip("tiles of 256 rows are for head sizes 64 and 128 and entries of many rows")
    q, kc, vc, bt, te, ps, meta = make_attention_case(torch.bfloat16, dev, n_q, n_kv, d, P, entries, seed=case, window=window, big_rows=big_rows)
    scale = 1.0 / math.sqrt(d)
    rows = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), P, meta, n_q, n_kv, d, scale, window)
    got = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), P, meta, n_q, n_kv, d, scale, window, for_product=True)
    if meta.T <= ops.FUSED_DECODE_MAX_ROWS and (n_q * d) % 32 == 0:
        assert ops.attention_hands_over_operand_rows(torch.bfloat16, n_q, d, P)
        assert isinstance(got, ops.OperandRows) and got.rows == meta.T and torch.equal(got.to_rows(), rows)
    else:
        assert torch.equal(got, rows)


def test_attention_without_rotation_is_library_sdpa():
    """One request from an empty cache equals softmax(QK^T / sqrt(d) + causal) V of a library routine."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    n_q, n_kv, d, P, n = 4, 2, 32, 16, 45
    q, kc, vc, bt, te, ps, meta = make_attention_case(torch.float32, dev, n_q, n_kv, d, P, [(0, n)], seed=99)
    K = torch.stack([kc[bt[0][c // P], :, c % P, :] for c in range(n)])      # [n, n_kv, d]
    V = torch.stack([vc[bt[0][c // P], :, :, c % P] for c in range(n)])
    Kr = K.repeat_interleave(n_q // n_kv, dim=1).transpose(0, 1)             # [n_q, n, d]
    Vr = V.repeat_interleave(n_q // n_kv, dim=1).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q.view(n, n_q, d).transpose(0, 1), Kr, Vr, is_causal=True)
    out = ops.paged_attention(q.to(dev), kc.to(dev), vc.to(dev), P, meta, n_q, n_kv, d, 1 / math.sqrt(d), None)
    close(out.view(n, n_q, d), ref.transpose(0, 1), torch.float32, what="sdpa")


@pytest.mark.parametrize("V", [7, 384, 151936])
def test_sample(V):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(V)
    R = 9
    logits = torch.randn(R, V, generator=g) * 2
    logits[0, :] = 1.5                      # all equal: the first wins
    logits[1, V - 1] = 50; logits[1, V // 2] = 50
    temp = torch.tensor([0, 0, 0, 0.8, 0.8, 1.3, 0.05, 1.0, 1.0])
    u = torch.tensor([0, 0, 0, 0.0, 0.999, 0.5, 0.7, 0.25, 0.75])
    out = ops.sample(logits.to(dev), temp.to(dev), u.to(dev)).cpu()
    assert out[0] == 0 and out[1] == V // 2 and out[2] == int(torch.argmax(logits[2]))
    for r in range(3, R):
        p = torch.softmax(logits[r].double() / float(temp[r]), 0)
        c = torch.cumsum(p, 0)
        k = int(out[r])
        lo = float(c[k - 1]) if k > 0 else 0.0
        # the chosen id's cumulative interval holds u (up to float32 rounding of the sums)
        assert lo - 1e-4 <= float(u[r]) <= float(c[k]) + 1e-4, (r, k, lo, float(c[k]), float(u[r]))
        assert p[k] > 0


def test_sample_frequencies():
    """Empirical frequencies on a 4-token distribution follow softmax(logits / T)."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    R = 4000
    logits = torch.tensor([0.0, 1.0, 2.0, -1.0]).repeat(R, 1)
    u = torch.rand(R, generator=torch.Generator().manual_seed(0))
    out = ops.sample(logits.to(dev), torch.full((R,), 0.7).to(dev), u.to(dev)).cpu().long()
    freq = torch.bincount(out, minlength=4).double() / R
    p = torch.softmax(logits[0].double() / 0.7, 0)
    assert (freq - p).abs().max() < 0.03


def test_zz_the_workspace_counters_are_left_at_zero():
    """Runs after the kernel tests of this file: the counters that the products with K split over blocks and the attention
    with its parts merged by the last block share are at zero, as every call must leave them (a counter left away from
    zero would make no block of a later call count itself last)."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    torch.cuda.synchronize()
    assert ops.workspace_counters_clean(dev)
