"""Each part alone on the GPU against the plain implementation's function for it, at sizes of its own."""
import math

import pytest
import torch

from spyinfer_amd.kernels import key_pieces
from tests.gpu_util import close, require_gpu
from tests.plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, dtype, seed, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def bind(part, prefix, dtype, dev, seed, scale=0.1):
    w = {}
    for i, s in enumerate(part.weight_specs(prefix)):
        t = rnd(s.shape, dtype, seed + i, scale)
        if s.role == "norm":
            t = (1 + t.float()).to(dtype)
        w[s.name] = t
    part.bind(prefix, {k: v.to(dev) for k, v in w.items()})
    return {k: v.float() for k, v in w.items()}


def make_batch(manager, dtype, dev, spans):
    """spans: list of (request cache, number of new tokens)."""
    from spyinfer_amd.engine.batch import StepBatch, StepEntry
    entries = []
    for rc, n in spans:
        manager.reserve(rc, n)
        entries.append(StepEntry(rc, [0] * n, []))
    return StepBatch(entries, manager, dtype, dev), entries


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from spyinfer_amd.parts import RMSNorm
    dev = require_gpu()
    part = RMSNorm(200, 1e-5)
    w = bind(part, "n", dtype, dev, 1)
    resid, delta = rnd((7, 200), torch.float32, 2), rnd((7, 200), dtype, 3)
    r = resid.clone().to(dev)
    out = part.add_norm(r, delta.to(dev), dtype)
    close(out, P.rms_norm(resid + delta.float(), w["n.weight"], 1e-5), dtype, what="RMSNorm part")
    close(r, resid + delta.float(), torch.float32, what="residual")


def test_rotary_part_tables():
    from spyinfer_amd.parts import RotaryEmbedding
    dev = require_gpu()
    part = RotaryEmbedding(48, 50000.0)
    part.prepare(dev, 300)
    cos, sin = P.rope_tables(300, 48, 50000.0)
    assert torch.allclose(part.cos.cpu(), cos, atol=1e-6) and torch.allclose(part.sin.cpu(), sin, atol=1e-6)
    assert part.rotary()[2] == 48


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 9])
def test_attention_part_in_cuts(dtype, window):
    """The attention part on a whole sequence, and the same sequence cut in two steps with another
    request beside it, against the plain functions (projections, q/k norm, rotation, attention)."""
    from spyinfer_amd.cache import CacheManager
    from spyinfer_amd.cache.storage import CacheStorage
    from spyinfer_amd.parts import PagedAttention, RotaryEmbedding
    dev = require_gpu()
    H, nq, nkv, d, T = 72, 6, 2, 32, 29
    rope = RotaryEmbedding(d, 30000.0)
    rope.prepare(dev, 128)
    part = PagedAttention(H, nq, nkv, d, rope, qk_norm_eps=1e-5, window=window)
    w = bind(part, "a", dtype, dev, 10, 0.15)
    x = rnd((T, H), dtype, 20)
    xf = x.float()
    q = P.rms_norm(P.linear(xf, w["a.q_proj.weight"]).view(T, nq, d), w["a.q_norm.weight"], 1e-5)
    k = P.rms_norm(P.linear(xf, w["a.k_proj.weight"]).view(T, nkv, d), w["a.k_norm.weight"], 1e-5)
    v = P.linear(xf, w["a.v_proj.weight"]).view(T, nkv, d)
    cos, sin = P.rope_tables(T, d, 30000.0)
    pos = torch.arange(T)
    ref = P.linear(P.attention(P.rope_apply(q, pos, cos, sin), P.rope_apply(k, pos, cos, sin), v, window).reshape(T, nq * d),
                   w["a.o_proj.weight"])
    manager = CacheManager([part.cache_spec()], page_size=8, num_pages=12, max_num_seqs=3)
    storage = CacheStorage(manager, dtype, dev)

    def run(spans, xs):
        batch, entries = make_batch(manager, dtype, dev, spans)
        part.plan(batch)
        batch.upload()
        out = part.forward(torch.cat(xs).to(dev), batch, storage.layer(0))
        for e in entries:
            manager.commit(e.cache, len(e.tokens))
        return out

    a = manager.admit("a")
    close(run([(a, T)], [x]), ref, dtype, scale=2.0, what="whole")
    manager.release(a)
    a, b = manager.admit("a"), manager.admit("b")
    other = rnd((5, H), dtype, 21)
    first = run([(b, 5), (a, 11)], [other, x[:11]])
    second = run([(a, T - 11), (b, 1)], [x[11:], other[:1]])
    close(torch.cat([first[5:], second[:T - 11]]), ref, dtype, scale=2.0, what="cut")
    manager.check()


@pytest.mark.parametrize("window", [None, 900])
def test_attention_part_decoding_long_requests_with_the_keys_cut_by_the_host(window):
    """The attention part with heads of 64 in bfloat16: two requests of 1500 and 300 tokens, their prompts in portions,
    then 40 steps of single tokens.  The host cuts the long request's keys into more parts than the short one's;
    with a window of 900 the pages that it has passed are given back (the block table says -1 there) and the blocks
    are counted from the window's start.  Every decoded row against the plain functions over the whole sequences."""
    from spyinfer_amd.cache import CacheManager
    from spyinfer_amd.cache.storage import CacheStorage
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts import PagedAttention, RotaryEmbedding
    dev = require_gpu()
    dtype = torch.bfloat16
    H, nq, nkv, d, steps = 128, 4, 2, 64, 40
    lengths = (1500, 300)
    rope = RotaryEmbedding(d, 30000.0)
    rope.prepare(dev, 2048)
    part = PagedAttention(H, nq, nkv, d, rope, qk_norm_eps=1e-5, window=window)
    w = bind(part, "a", dtype, dev, 30, 0.1)
    xs = [rnd((n + steps, H), dtype, 40 + i) for i, n in enumerate(lengths)]
    refs = []
    for x in xs:
        T, xf = x.shape[0], x.float()
        q = P.rms_norm(P.linear(xf, w["a.q_proj.weight"]).view(T, nq, d), w["a.q_norm.weight"], 1e-5)
        k = P.rms_norm(P.linear(xf, w["a.k_proj.weight"]).view(T, nkv, d), w["a.k_norm.weight"], 1e-5)
        v = P.linear(xf, w["a.v_proj.weight"]).view(T, nkv, d)
        cos, sin = P.rope_tables(T, d, 30000.0)
        pos = torch.arange(T)
        refs.append(P.linear(P.attention(P.rope_apply(q, pos, cos, sin), P.rope_apply(k, pos, cos, sin), v, window).reshape(T, nq * d),
                             w["a.o_proj.weight"]))
    manager = CacheManager([part.cache_spec()], page_size=16, num_pages=130, max_num_seqs=2, max_step_tokens=512)
    storage = CacheStorage(manager, dtype, dev)
    caches = [manager.admit(i) for i in range(2)]

    def run(spans, rows):
        batch, entries = make_batch(manager, dtype, dev, spans)
        part.plan(batch)
        batch.upload()
        out = part.forward(torch.cat(rows).to(dev), batch, storage.layer(0))
        for e in entries:
            manager.commit(e.cache, len(e.tokens))
        return out, batch

    for c, x, n in zip(caches, xs, lengths):
        for lo in range(0, n, 512):
            run([(c, min(512, n - lo))], [x[lo:min(lo + 512, n)]])
    cut = set()
    for i in range(steps):
        out, batch = run([(c, 1) for c in caches], [x[n + i:n + i + 1] for x, n in zip(xs, lengths)])
        rec = batch.host_array("decode_pieces_%d_%d_%d" % (nkv, window or 0, d)).reshape(-1, key_pieces.PIECE_RECORD)
        cut.add((int(rec[rec[:, 0] == 0][0, 5]), int(rec[rec[:, 0] == 1][0, 5])))
        close(out, torch.stack([r[n + i] for r, n in zip(refs, lengths)]), dtype, scale=2.0, what="step %d" % i)
    assert all(long > short >= 1 for long, short in cut), cut
    if window:
        assert min(caches[0].tables[0][:30]) == -1, "the pages that the window has passed are given back"
    manager.check()
    assert ops.workspace_counters_clean(dev)


@pytest.mark.parametrize("dtype", DTYPES)
def test_mlp_part(dtype):
    from spyinfer_amd.parts import GatedMLP
    dev = require_gpu()
    part = GatedMLP(88, 200)
    w = bind(part, "m", dtype, dev, 30, 0.2)
    x = rnd((19, 88), dtype, 31)
    ref = P.linear(P.swiglu(P.linear(x.float(), w["m.gate_proj.weight"]), P.linear(x.float(), w["m.up_proj.weight"])), w["m.down_proj.weight"])
    close(part.forward(x.to(dev), None), ref, dtype, scale=2.0, what="GatedMLP part")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tied", [True, False])
def test_embedding_and_head_parts(dtype, tied):
    from spyinfer_amd.parts import LMHead, TokenEmbedding
    dev = require_gpu()
    emb = TokenEmbedding(331, 88)
    head = LMHead(331, 88, tied_to=emb if tied else None)
    we = bind(emb, "e", dtype, dev, 40)
    wh = bind(head, "h", dtype, dev, 41)
    ids = torch.tensor([0, 330, 17, 17], dtype=torch.int32)
    assert torch.equal(emb.forward(ids.to(dev)).cpu(), P.embedding(ids.long(), we["e.weight"]))
    x = rnd((3, 88), dtype, 42)
    out = head.forward(x.to(dev))
    assert out.dtype == torch.float32
    close(out, P.linear(x.float(), we["e.weight"] if tied else wh["h.weight"]), dtype, scale=2.0, what="LMHead part")


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part(dtype):
    """A pre-norm block with a feed-forward only (the mixer returns zero): residual sums and norm order."""
    from spyinfer_amd.parts import GatedMLP, PreNormBlock, RMSNorm
    from spyinfer_amd.parts.base import Mixer
    dev = require_gpu()

    class Zero(Mixer):
        def forward(self, x, batch, cache, store=True):
            return torch.zeros_like(x)

    class B:
        act_dtype = dtype

    blk = PreNormBlock(RMSNorm(64, 1e-6), Zero(), RMSNorm(64, 1e-6), GatedMLP(64, 96))
    w = bind(blk, "L", dtype, dev, 50, 0.2)
    resid, delta = rnd((6, 64), torch.float32, 51), rnd((6, 64), dtype, 52)
    r, f = blk.forward(resid.clone().to(dev), delta.to(dev), B, None)
    h = resid + delta.float()
    n2 = P.rms_norm(h, w["L.post_attention_layernorm.weight"], 1e-6)
    ref = P.linear(P.swiglu(P.linear(n2, w["L.mlp.gate_proj.weight"]), P.linear(n2, w["L.mlp.up_proj.weight"])), w["L.mlp.down_proj.weight"])
    close(r, h, torch.float32, what="residual stream")
    close(f, ref, dtype, scale=2.0, what="block addend")
