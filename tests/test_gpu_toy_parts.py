"""Parts that are not in the framework, defined here and put into a model without a change to the
framework's files: a position encoding that is added to the embeddings, a feed-forward that routes
every token to two of three experts, a norm that centres before it scales, and a run order in which
one call reads the keys and values that another call stored; a third kind of cache; other arrangements of the parts
in a block.  Each toy model is compared with a plain
forward pass of whole sequences written below, and with itself under other cuts of the same requests.
It is a toy: no model of anyone's."""
import dataclasses
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file

from tests import replay_cases as rc
from tests.configs import INIT
from tests.gpu_util import require_gpu
from tests.plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(atol=1e-4, rtol=1e-4), "bfloat16": dict(atol=8e-2, rtol=2e-2)}
EPS, WINDOW, TOP = 1e-5, 24, 2
HEAD = {"dim": 16}   # head size of the routed toy's attention layers (the test sets it)


def _toy():
    from spyinfer_amd.config import ModelConfig
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.models import DecoderModel, LayerCall
    from spyinfer_amd.parts import GatedMLP, LMHead, PagedAttention, PreNormBlock, TokenEmbedding
    from spyinfer_amd.parts.base import FeedForward, Norm, PositionEncoding
    from spyinfer_amd.weights import WeightSpec

    class LearnedPositions(PositionEncoding):
        """h[t] += table[position of t]; nothing is rotated."""

        def __init__(self, positions, hidden):
            self.positions, self.hidden = positions, hidden

        def weight_specs(self, prefix):
            return [WeightSpec(prefix + ".table", (self.positions, self.hidden))]

        def bind(self, prefix, weights):
            self.table = weights[prefix + ".table"]

        def on_embeddings(self, hidden, batch):
            return hidden + self.table[batch.positions.long()].float()

    class CentredNorm(Norm):
        """y = (x - mean(x)) / sqrt(var(x) + eps) * w, float32 inside."""

        def __init__(self, size, eps):
            self.size, self.eps = size, eps

        def weight_specs(self, prefix):
            return [WeightSpec(prefix + ".weight", (self.size,), "norm")]

        def bind(self, prefix, weights):
            self.weight = weights[prefix + ".weight"]

        def add_norm(self, resid, delta, out_dtype, rows=None):
            if rows is None:
                if delta is not None:
                    resid += delta.float()
                x = resid
            else:
                x = resid[rows.long()] if delta is None else resid[rows.long()] + delta[rows.long()].float()
            x = x - x.mean(-1, keepdim=True)
            return (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.weight.float()).to(out_dtype)

    class RoutedMLP(FeedForward):
        """Router logits in float32, the TOP largest experts per token, softmax over their logits as weights; every
        expert is the framework's gated feed-forward, run on the rows routed to it."""

        def __init__(self, hidden, inter, experts):
            self.hidden, self.n = hidden, experts
            self.experts = [GatedMLP(hidden, inter) for _ in range(experts)]

        def weight_specs(self, prefix):
            specs = [WeightSpec(prefix + ".router.weight", (self.n, self.hidden))]
            for i, e in enumerate(self.experts):
                specs += e.weight_specs("%s.experts.%d" % (prefix, i))
            return specs

        def bind(self, prefix, weights):
            self.router = weights[prefix + ".router.weight"]
            for i, e in enumerate(self.experts):
                e.bind("%s.experts.%d" % (prefix, i), weights)

        def forward(self, x, batch):
            logits = x.float() @ self.router.float().t()
            top, idx = torch.topk(logits, TOP, dim=-1)
            gate = torch.softmax(top, dim=-1)
            out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            for i, e in enumerate(self.experts):
                rows, slot = torch.nonzero(idx == i, as_tuple=True)
                if rows.numel():
                    y = e.forward(x[rows].contiguous(), batch)
                    out.index_add_(0, rows, y.float() * gate[rows, slot][:, None])
            return out.to(x.dtype)

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        hidden_size: int = 0
        vocab_size: int = 0
        intermediate_size: int = 0
        num_experts: int = 0
        max_positions: int = 0

    def build(cfg):
        H = cfg.hidden_size
        emb = TokenEmbedding(cfg.vocab_size, H)
        pos = LearnedPositions(cfg.max_positions, H)
        attn = lambda window: PagedAttention(H, 6, 2, HEAD["dim"], None, qk_norm_eps=None, window=window)
        norm = lambda: CentredNorm(H, EPS)
        layers = [PreNormBlock(norm(), attn(None), norm(), RoutedMLP(H, cfg.intermediate_size, cfg.num_experts)),
                  PreNormBlock(norm(), attn(WINDOW), norm(), GatedMLP(H, cfg.intermediate_size)),
                  PreNormBlock(norm(), attn(None), norm(), RoutedMLP(H, cfg.intermediate_size, cfg.num_experts))]
        # the third call has queries of its own and reads the keys and values that the first call stored
        order = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 0, store=False)]
        return DecoderModel(cfg, emb, pos, layers, norm(), LMHead(cfg.vocab_size, H), schedule=order,
                            max_positions=cfg.max_positions)

    return ToyConfig, build


def plain_forward(folder, tokens):
    """Whole sequence, no cache, float32, from the plain functions and the formulas in the docstrings above."""
    cfg = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    T, H = len(tokens), cfg["hidden_size"]

    def norm(x, name):
        x = x - x.mean(-1, keepdim=True)
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + EPS) * w[name + ".weight"]

    def mlp(x, p):
        return P.linear(P.swiglu(P.linear(x, w[p + ".gate_proj.weight"]), P.linear(x, w[p + ".up_proj.weight"])), w[p + ".down_proj.weight"])

    def routed(x, p):
        logits = P.linear(x, w[p + ".router.weight"])
        out = torch.zeros_like(x)
        for t in range(x.shape[0]):
            top = sorted(range(logits.shape[1]), key=lambda e: -float(logits[t, e]))[:TOP]
            g = torch.softmax(logits[t, top], dim=0)
            for gi, e in zip(g, top):
                out[t] += gi * mlp(x[t:t + 1], "%s.experts.%d" % (p, e))[0]
        return out

    def qkv(x, p):
        a = p + ".self_attn."
        return (P.linear(x, w[a + "q_proj.weight"]).view(T, 6, HEAD["dim"]), P.linear(x, w[a + "k_proj.weight"]).view(T, 2, HEAD["dim"]),
                P.linear(x, w[a + "v_proj.weight"]).view(T, 2, HEAD["dim"]))

    h = P.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"]) + w["model.position.table"][:T]
    kept = None
    for call, (layer, window, ffn) in enumerate(((0, None, routed), (1, WINDOW, mlp), (2, None, routed))):
        p = "model.layers.%d" % layer
        q, k, v = qkv(norm(h, p + ".input_layernorm"), p)
        if call == 0:
            kept = (k, v)
        if call == 2:
            k, v = kept
        h = h + P.linear(P.attention(q, k, v, window).reshape(T, -1), w[p + ".self_attn.o_proj.weight"])
        h = h + ffn(norm(h, p + ".post_attention_layernorm"), p + ".mlp")
    return P.linear(norm(h, "model.norm"), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("head_dim", [16, 128])
def test_toy_parts_and_shared_cache(dtype, head_dim, tmp_path, monkeypatch):
    """(Heads of 128: single tokens then take the attention that reads the raw product, here without head norms and
    without rotation, once over a cache that another call has stored, once under a window.)"""
    from spyinfer_amd.config import register_architecture, unregister_architecture
    from spyinfer_amd.weights import write_random_model
    require_gpu()
    monkeypatch.setitem(HEAD, "dim", head_dim)
    ToyConfig, build = _toy()
    register_architecture("ToyRoutedLM", ToyConfig, build)
    try:
        cfg = dict(architectures=["ToyRoutedLM"], hidden_size=72, vocab_size=113, intermediate_size=56, num_experts=3, max_positions=160)
        folder = write_random_model(str(tmp_path / "toy"), cfg, 81, torch.bfloat16, **INIT)
        reqs = rc.random_requests(113, [70, 9, 41, 120, 33], seed=10)
        ref = {rid: plain_forward(folder, t) for rid, t in reqs.items()}
        tol = TOL[dtype]
        outs = {}
        for mode in ("whole", "bulk_tail", "portions", "mixed"):
            steps = getattr(rc, mode)(reqs)
            out = str(tmp_path / mode)
            rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps))
            outs[mode] = rc.collect(out, steps, 113)
            if dtype == "float32":
                rc.compare(outs[mode], ref, what="toy/" + mode, **tol)
        # bfloat16: a token whose two best experts nearly tie may be routed otherwise after rounding, which changes its
        # logits by more than rounding does; so most rows, not all, must agree with the plain pass
        if dtype == "bfloat16":
            for mode, got in outs.items():
                good = sum(np.allclose(row, ref[rid][t].numpy(), atol=tol["atol"], rtol=tol["rtol"]) for (rid, t), row in got.items())
                assert good >= 0.9 * len(got), "%s: only %d of %d rows agree with the plain pass" % (mode, good, len(got))
        # the position table matters (no rotation here): the same tokens later in a request give other logits
        toks = reqs[next(iter(reqs))]
        shifted = plain_forward(folder, toks[:5] + toks[:5])
        assert not torch.allclose(shifted[5:], shifted[:5], atol=1e-2)
    finally:
        unregister_architecture("ToyRoutedLM")


# ---------------------------------------------------------------------------------------------
# A third kind of cache, defined here: one float32 tensor per group, a token's vector per page slot
# (another layout, another dtype, one tensor instead of two), and a mixer that reads it through the
# request's block table.

def _toy_latent():
    from spyinfer_amd.cache import CacheKind
    from spyinfer_amd.config import ModelConfig
    from spyinfer_amd.models import DecoderModel
    from spyinfer_amd.parts import GatedMLP, LMHead, PagedAttention, PreNormBlock, RMSNorm, RotaryEmbedding, TokenEmbedding
    from spyinfer_amd.parts.base import Mixer
    from spyinfer_amd.weights import WeightSpec

    class LatentLayer:
        def __init__(self, group, rows, page_size):
            self.group, self.rows, self.page_size = group, rows, page_size     # rows: [pages * page, width] float32

    @dataclasses.dataclass(frozen=True)
    class PagedLatent(CacheKind):
        """One float32 vector of ``width`` per token, in pages: ``[layers, pages, page, width]``."""
        width: int
        paged = True

        def page_bytes(self, page_size, act_dtype):
            return 4 * self.width * page_size

        def allocate(self, num_layers, count, page_size, act_dtype, device):
            return [torch.zeros((num_layers, count, page_size, self.width), dtype=torch.float32, device=device)]

        def layer_view(self, group, tensors, index, page_size):
            return LatentLayer(group, tensors[0][index].view(-1, self.width), page_size)

    class PagedMean(Mixer):
        """out[t] = gain * mean of the request's inputs at positions 0..t, every input kept in the paged cache."""

        def __init__(self, hidden):
            self.hidden = hidden

        def weight_specs(self, prefix):
            return [WeightSpec(prefix + ".gain", (self.hidden,), "norm")]

        def bind(self, prefix, weights):
            self.gain = weights[prefix + ".gain"]

        def cache_spec(self):
            return PagedLatent(self.hidden)

        def forward(self, x, batch, cache, store=True):
            if store:
                cache.rows[batch.slot_mapping(cache.group).long()] = x.float()
            table = batch.block_table(cache.group).long()                      # [S, max_blocks]
            P = cache.page_size
            out = torch.empty_like(x)
            lens, pos0 = batch.lens, batch.host_array("pos0")
            t0 = 0
            for s in range(batch.S):
                n, first = int(lens[s]), int(pos0[s])
                pos = torch.arange(first + n, device=x.device)
                rows = cache.rows[table[s][pos // P] * P + pos % P]            # every input of the request so far
                sums = torch.cumsum(rows, 0)[first:]
                out[t0:t0 + n] = (sums / (pos[first:] + 1).float()[:, None] * self.gain.float()).to(x.dtype)
                t0 += n
            return out

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        hidden_size: int = 0
        vocab_size: int = 0
        intermediate_size: int = 0

    def build(cfg):
        H = cfg.hidden_size
        emb, rope = TokenEmbedding(cfg.vocab_size, H), RotaryEmbedding(16, 10000.0)
        mixers = [PagedMean(H), PagedAttention(H, 4, 2, 16, rope), PagedMean(H)]
        layers = [PreNormBlock(RMSNorm(H, 1e-5), m, RMSNorm(H, 1e-5), GatedMLP(H, cfg.intermediate_size)) for m in mixers]
        return DecoderModel(cfg, emb, rope, layers, RMSNorm(H, 1e-5), LMHead(cfg.vocab_size, H, tied_to=emb), max_positions=256)

    return ToyConfig, build, PagedLatent


def plain_latent_forward(folder, tokens):
    cfg = json.load(open(os.path.join(folder, "config.json")))
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    T = len(tokens)
    cos, sin = P.rope_tables(T, 16, 10000.0)
    pos = torch.arange(T)
    h = P.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    for i in range(3):
        p = "model.layers.%d." % i
        n1 = P.rms_norm(h, w[p + "input_layernorm.weight"], 1e-5)
        if i == 1:
            q = P.rope_apply(P.linear(n1, w[p + "self_attn.q_proj.weight"]).view(T, 4, 16), pos, cos, sin)
            k = P.rope_apply(P.linear(n1, w[p + "self_attn.k_proj.weight"]).view(T, 2, 16), pos, cos, sin)
            v = P.linear(n1, w[p + "self_attn.v_proj.weight"]).view(T, 2, 16)
            a = P.linear(P.attention(q, k, v).reshape(T, -1), w[p + "self_attn.o_proj.weight"])
        else:
            a = torch.cumsum(n1, 0) / (pos + 1).float()[:, None] * w[p + "self_attn.gain"]
        h = h + a
        n2 = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], 1e-5)
        h = h + P.linear(P.swiglu(P.linear(n2, w[p + "mlp.gate_proj.weight"]), P.linear(n2, w[p + "mlp.up_proj.weight"])),
                         w[p + "mlp.down_proj.weight"])
    return P.linear(P.rms_norm(h, w["model.norm.weight"], 1e-5), w["model.embed_tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_third_kind_of_cache_defined_in_a_test(dtype, tmp_path):
    """The cache manager groups, the storage allocates and the step hands out a kind of cache that the framework does
    not know: pages of one float32 tensor, with a pool and block tables apart from the attention layer's keys and values."""
    from spyinfer_amd.config import register_architecture, unregister_architecture
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    ToyConfig, build, PagedLatent = _toy_latent()
    register_architecture("ToyLatentLM", ToyConfig, build)
    try:
        cfg = dict(architectures=["ToyLatentLM"], hidden_size=64, vocab_size=101, intermediate_size=96)
        folder = write_random_model(str(tmp_path / "toy"), cfg, 91, torch.bfloat16, **INIT)
        runner = ModelRunner(load_model(folder, dtype, dev), dtype, dev, 16, 8, 2)
        groups = runner.manager.page_groups
        assert [g.cache_ids for g in groups] == [[0, 2], [1]] and groups[0].spec == PagedLatent(64)
        elem = 2 if dtype == "bfloat16" else 4
        assert ModelRunner.bytes_per_page(runner.model, 16, dtype) == 2 * 4 * 64 * 16 + 2 * 2 * 16 * 16 * elem
        assert [tuple(t.shape) for t in runner.storage.tensors] == [(2, 8, 16, 64), (1, 8, 2, 16, 16), (1, 8, 2, 16, 16)]
        assert runner.storage.tensors[0].dtype == torch.float32
        reqs = rc.random_requests(101, [70, 9, 41, 120, 33], seed=12)
        ref = {rid: plain_latent_forward(folder, t) for rid, t in reqs.items()}
        for mode in ("whole", "bulk_tail", "portions", "mixed"):
            steps = getattr(rc, mode)(reqs)
            out = str(tmp_path / mode)
            rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps))
            rc.compare(rc.collect(out, steps, 101), ref, what="latent/%s/%s" % (mode, dtype), **TOL[dtype])
    finally:
        unregister_architecture("ToyLatentLM")


# ---------------------------------------------------------------------------------------------
# Other arrangements of norm, mixer and feed-forward in a block, defined here: one norm whose output both the mixer and
# the feed-forward read, their results added to the stream together; and norms before AND behind each of the two.  The
# toy model puts them between blocks of the framework's own arrangement, at widths whose decode steps fold the norms
# into the products: so a block that prepares the next norm's input stands before one that does not know of that, and
# behind one.

ARR = dict(hidden=128, heads=4, kv=2, head_dim=64, inter=256, vocab=131, eps=1e-5, theta=1e4, positions=256)


def _toy_arranged():
    from spyinfer_amd.config import ModelConfig
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.models import DecoderModel
    from spyinfer_amd.parts import GatedMLP, LMHead, PagedAttention, PreNormBlock, RMSNorm, RotaryEmbedding, TokenEmbedding
    from spyinfer_amd.parts.base import Block

    class Arranged(Block):
        """Parts by name under the layer's prefix; what a block must have beside ``forward``."""

        def _named(self, prefix):
            return [(part, prefix + "." + name) for name, part in self.parts.items()]

        def weight_specs(self, prefix):
            return [s for part, p in self._named(prefix) for s in part.weight_specs(p)]

        def bind(self, prefix, weights):
            for part, p in self._named(prefix):
                part.bind(p, weights)

        def capturable(self, batch):
            return all(part.capturable(batch) for part in self.parts.values())

    class ParallelBlock(Arranged):
        """n = norm(h);  h += mixer(n) + ffn(n)."""

        def __init__(self, norm, mixer, ffn):
            self.parts = dict(input_layernorm=norm, self_attn=mixer, mlp=ffn)
            self.norm, self.mixer, self.ffn = norm, mixer, ffn

        def forward(self, resid, pending, batch, cache, store=True, next_norm=None):
            # a prepared input of another block's norm means that the stream is complete: nothing is left to add
            delta = None if isinstance(pending, ops.ScaledInput) else pending
            n = self.norm.add_norm(resid, delta, batch.act_dtype)
            a = self.mixer.forward(n, batch, cache, store)
            f = self.ffn.forward(n, batch)
            return resid, (a.float() + f.float()).to(batch.act_dtype)

    class SandwichBlock(Arranged):
        """h += post1(mixer(pre1(h)));  h += post2(ffn(pre2(h))): the norms behind act on the branch, not on the stream."""

        def __init__(self, pre1, mixer, post1, pre2, ffn, post2):
            self.parts = dict(input_layernorm=pre1, self_attn=mixer, post_mixer_layernorm=post1, pre_mlp_layernorm=pre2, mlp=ffn,
                              post_mlp_layernorm=post2)
            self.pre1, self.mixer, self.post1, self.pre2, self.ffn, self.post2 = pre1, mixer, post1, pre2, ffn, post2

        def forward(self, resid, pending, batch, cache, store=True, next_norm=None):
            act = batch.act_dtype
            delta = None if isinstance(pending, ops.ScaledInput) else pending
            a = self.mixer.forward(self.pre1.add_norm(resid, delta, act), batch, cache, store)
            a = self.post1.add_norm(a.float(), None, act)
            f = self.ffn.forward(self.pre2.add_norm(resid, a, act), batch)
            return resid, self.post2.add_norm(f.float(), None, act)

    @dataclasses.dataclass
    class ArrangedConfig(ModelConfig):
        vocab_size: int = 0

    def build(cfg):
        H, eps = ARR["hidden"], ARR["eps"]
        rotary = RotaryEmbedding(ARR["head_dim"], ARR["theta"])
        attn = lambda: PagedAttention(H, ARR["heads"], ARR["kv"], ARR["head_dim"], rotary, qk_norm_eps=eps)
        norm, mlp = (lambda: RMSNorm(H, eps)), (lambda: GatedMLP(H, ARR["inter"]))
        layers = [PreNormBlock(norm(), attn(), norm(), mlp()),
                  ParallelBlock(norm(), attn(), mlp()),
                  PreNormBlock(norm(), attn(), norm(), mlp()),
                  SandwichBlock(norm(), attn(), norm(), norm(), mlp(), norm()),
                  PreNormBlock(norm(), attn(), norm(), mlp())]
        return DecoderModel(cfg, TokenEmbedding(cfg.vocab_size, H), rotary, layers, norm(), LMHead(cfg.vocab_size, H),
                            max_positions=ARR["positions"])

    return ArrangedConfig, build


def plain_arranged(folder, tokens):
    """Whole sequence, no cache, float32, from the plain functions and the formulas in the blocks' docstrings."""
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    T, d, eps = len(tokens), ARR["head_dim"], ARR["eps"]
    cos, sin = P.rope_tables(T, d, ARR["theta"])
    positions = torch.arange(T)

    def norm(x, name):
        return P.rms_norm(x, w[name + ".weight"], eps)

    def attn(n, p):
        a = p + ".self_attn."
        q = P.linear(n, w[a + "q_proj.weight"]).view(T, ARR["heads"], d)
        k = P.linear(n, w[a + "k_proj.weight"]).view(T, ARR["kv"], d)
        v = P.linear(n, w[a + "v_proj.weight"]).view(T, ARR["kv"], d)
        q = P.rope_apply(P.rms_norm(q, w[a + "q_norm.weight"], eps), positions, cos, sin)
        k = P.rope_apply(P.rms_norm(k, w[a + "k_norm.weight"], eps), positions, cos, sin)
        return P.linear(P.attention(q, k, v).reshape(T, -1), w[a + "o_proj.weight"])

    def mlp(n, p):
        return P.linear(P.swiglu(P.linear(n, w[p + ".mlp.gate_proj.weight"]), P.linear(n, w[p + ".mlp.up_proj.weight"])),
                        w[p + ".mlp.down_proj.weight"])

    h = P.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    for i, kind in enumerate(("pre", "parallel", "pre", "sandwich", "pre")):
        p = "model.layers.%d" % i
        if kind == "pre":
            h = h + attn(norm(h, p + ".input_layernorm"), p)
            h = h + mlp(norm(h, p + ".post_attention_layernorm"), p)
        elif kind == "parallel":
            n = norm(h, p + ".input_layernorm")
            h = h + attn(n, p) + mlp(n, p)
        else:
            h = h + norm(attn(norm(h, p + ".input_layernorm"), p), p + ".post_mixer_layernorm")
            h = h + norm(mlp(norm(h, p + ".pre_mlp_layernorm"), p), p + ".post_mlp_layernorm")
    return P.linear(norm(h, "model.norm"), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_arrangements_of_a_block(dtype, tmp_path):
    """Blocks arranged otherwise, defined above, between the framework's own: every way of cutting the requests against
    the plain pass; then through the entry point with recorded decode steps (the blocks say what their parts say about
    recording), greedy tokens against the plain pass in float32."""
    from spyinfer_amd.config import register_architecture, unregister_architecture
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights import write_random_model
    require_gpu()
    ArrangedConfig, build = _toy_arranged()
    register_architecture("ToyArrangedLM", ArrangedConfig, build)
    try:
        cfg = dict(architectures=["ToyArrangedLM"], vocab_size=ARR["vocab"])
        folder = write_random_model(str(tmp_path / "toy"), cfg, 91, torch.bfloat16, **INIT)
        reqs = rc.random_requests(ARR["vocab"], [70, 9, 41, 120, 33], seed=12)
        ref = {rid: plain_arranged(folder, t) for rid, t in reqs.items()}
        for mode in ("whole", "bulk_tail", "portions", "mixed"):
            steps = getattr(rc, mode)(reqs)
            out = str(tmp_path / mode)
            rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps))
            rc.compare(rc.collect(out, steps, ARR["vocab"]), ref, what="arranged/" + mode, **TOL[dtype])
        eng = LLMEngine(folder, dtype=dtype, max_model_len=200, num_kvcache_blocks=40, max_num_seqs=4)
        prompts = [t[:n] for t, n in zip(reqs.values(), (30, 9, 41, 5))]
        got = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
        assert eng.runner.graph_replays > 0, "decode steps of these blocks are recorded"
        if dtype == "float32":
            for p, g in zip(prompts, got):
                toks = list(p)
                for t in g:
                    assert t == int(torch.argmax(plain_arranged(folder, toks)[-1]))
                    toks.append(t)
    finally:
        unregister_architecture("ToyArrangedLM")
