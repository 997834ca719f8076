"""Parts that are not in the framework, defined here and put into a model without a change to the
framework's files: a position encoding that is added to the embeddings, a feed-forward that routes
every token to two of three experts, a norm that centres before it scales, and a run order in which
one call reads the keys and values that another call stored.  The toy model is compared with a plain
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
        attn = lambda window: PagedAttention(H, 6, 2, 16, None, qk_norm_eps=None, window=window)
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
        return (P.linear(x, w[a + "q_proj.weight"]).view(T, 6, 16), P.linear(x, w[a + "k_proj.weight"]).view(T, 2, 16),
                P.linear(x, w[a + "v_proj.weight"]).view(T, 2, 16))

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
def test_toy_parts_and_shared_cache(dtype, tmp_path):
    from spyinfer_amd.config import register_architecture, unregister_architecture
    from spyinfer_amd.weights import write_random_model
    require_gpu()
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
