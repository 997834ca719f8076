"""Pins the plain implementation by what fixes it beside the reference's text: vectors that the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

from tests.configs import INIT, TINY_A, TINY_B
from tests.plain import qwen3_plain as P


def test_linear_reference_vector():
    # test/test_linear.cpp:53-60: x [2,3], W [4,3] (a transposed W would not even have the shape)
    x = torch.tensor([[1., 2, 3], [4, 5, 6]])
    w = torch.tensor([[1., 2, 3], [4, 5, 6], [7, 8, 9], [10, 11, 12]])
    assert P.linear(x, w).tolist() == [[14, 32, 50, 68], [32, 77, 122, 167]]


def test_swiglu_reference_ramp():
    # test/test_swiglu.cpp:43-46, 68: gate in [-5, 4.9], up in [-2, 2.6]; silu on the gate, not on up
    i = torch.arange(100100)
    g = (i % 100).float() / 10.0 - 5.0
    u = (i % 70).float() / 15.0 - 2.0
    out = P.swiglu(g, u)
    assert torch.allclose(out, torch.nn.functional.silu(g) * u, atol=1e-5)
    assert not torch.allclose(out, g * torch.nn.functional.silu(u), atol=1e-2)
    assert P.swiglu(torch.tensor([0.0]), torch.tensor([3.0])).item() == 0.0
    assert abs(P.swiglu(torch.tensor([30.0]), torch.tensor([3.0])).item() - 90.0) < 1e-4


def test_rms_norm():
    # shape of test/test_rms_norm_cuda.cu:16-18
    g = torch.Generator().manual_seed(0)
    x = torch.rand(2, 512, generator=g) * 2 - 1
    w = torch.rand(512, generator=g) * 2 - 1
    y = P.rms_norm(x, w, 1e-6)
    assert torch.allclose(y, x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w, atol=1e-6)
    # the weight multiplies as it is: w = 0 gives 0 (a "1 + w" norm would not)
    assert P.rms_norm(x, torch.zeros(512), 1e-6).abs().max() == 0
    # eps sits inside the root and matters for a tiny row
    t = torch.full((1, 64), 1e-3)
    a, b = P.rms_norm(t, torch.ones(64), 1e-6)[0, 0].item(), P.rms_norm(t, torch.ones(64), 1e-5)[0, 0].item()
    assert abs(a - 1e-3 / math.sqrt(2e-6)) < 1e-5 and abs(b - 1e-3 / math.sqrt(1.1e-5)) < 1e-5
    # scale invariance for rows far above eps
    assert torch.allclose(P.rms_norm(7 * x, w, 1e-6), y, atol=1e-4)


def test_rope_is_half_split_and_a_rotation():
    d, theta = 16, 10000.0
    cos, sin = P.rope_tables(64, d, theta)
    # a vector with only x[0] and x[d/2] set rotates within that pair under half-split pairing;
    # under interleaved pairing x[1] and x[d/2 + 1] would appear
    x = torch.zeros(1, 1, d)
    x[0, 0, 0], x[0, 0, d // 2] = 1.0, 2.0
    y = P.rope_apply(x, torch.tensor([5]), cos, sin)[0, 0]
    assert abs(y[0].item() - (math.cos(5) - 2 * math.sin(5))) < 1e-5 and abs(y[d // 2].item() - (math.sin(5) + 2 * math.cos(5))) < 1e-5
    assert y[[i for i in range(d) if i not in (0, d // 2)]].abs().max() == 0
    # frequencies: theta^(-j / (d/2)); the last pair turns slowest
    assert abs(cos[1, d // 2 - 1].item() - math.cos(theta ** (-(d // 2 - 1) / (d // 2)))) < 1e-6
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, d, generator=g), torch.randn(1, 1, d, generator=g)
    assert torch.equal(P.rope_apply(q, torch.tensor([0]), cos, sin), q)                       # position 0 is the identity
    assert abs(P.rope_apply(q, torch.tensor([9]), cos, sin).norm() - q.norm()) < 1e-5          # norms are kept
    # the product of a rotated query and key depends on the distance only
    def dot(m, n):
        return (P.rope_apply(q, torch.tensor([m]), cos, sin) * P.rope_apply(k, torch.tensor([n]), cos, sin)).sum().item()
    assert abs(dot(12, 5) - dot(40, 33)) < 1e-4 and abs(dot(12, 5) - dot(5, 12)) > 1e-3


def test_attention_reduces_to_library_routines():
    g = torch.Generator().manual_seed(2)
    T, n_q, n_kv, d = 9, 4, 2, 8
    q, k, v = torch.randn(T, n_q, d, generator=g), torch.randn(T, n_kv, d, generator=g), torch.randn(T, n_kv, d, generator=g)
    out = P.attention(q, k, v)
    kr, vr = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)       # kv head = h * n_kv / n_q
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1), is_causal=True)
    assert torch.allclose(out, ref.transpose(0, 1), atol=1e-5)
    # one token: the output is its value; one head, no mask effect on the last row: plain softmax
    assert torch.allclose(P.attention(q[:1], k[:1], v[:1])[0, 3], v[0, 1])
    s = torch.softmax((k[:, 0] @ q[-1, 0]) / math.sqrt(d), 0)
    assert torch.allclose(out[-1, 0], s @ v[:, 0], atol=1e-5)
    # window w: the last row sees the last w keys only
    outw = P.attention(q, k, v, window=3)
    s = torch.softmax((k[-3:, 0] @ q[-1, 0]) / math.sqrt(d), 0)
    assert torch.allclose(outw[-1, 0], s @ v[-3:, 0], atol=1e-5)
    assert torch.allclose(outw[:3], out[:3], atol=1e-6)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    return P.PlainQwen3(write_random_model(str(tmp_path_factory.mktemp("plain_b")), TINY_B, 41, torch.bfloat16, **INIT))


def test_model_is_causal_and_shift_invariant(model_b):
    toks = torch.randint(0, 384, (20,), generator=torch.Generator().manual_seed(3)).tolist()
    full = model_b.forward(toks)
    assert torch.allclose(model_b.forward(toks[:11]), full[:11], atol=1e-5)       # later tokens do not reach back
    # only distances between positions count: a shift of all positions leaves the logits
    assert torch.allclose(model_b.forward(toks, first_position=37), full, atol=2e-4)
    # float64 agrees with float32: the formulas are well conditioned at these sizes
    m64 = P.PlainQwen3.__new__(P.PlainQwen3)
    m64.__dict__.update(model_b.__dict__)
    m64.compute = torch.float64
    m64.w = {k: v.double() for k, v in model_b.w.items()}
    m64._tables = None
    assert torch.allclose(m64.forward(toks).float(), full, atol=2e-4)


def test_a_zero_q_norm_weight_gives_uniform_attention(model_b):
    """The q norm's weight multiplies the queries: with a zero weight in layer 0 every score there is zero, the
    attention is the plain mean over the causal prefix (finite, different, and unchanged where there is one key).  Where
    the norms stand in the layer (before the rotation, before or after the residual sum, the final norm) is held by the
    mutations of the second transcription below, not here."""
    toks = [1, 2, 3, 4, 5]
    base = model_b.forward(toks)
    w = dict(model_b.w)
    try:
        model_b.w = dict(w)
        model_b.w["model.layers.0.self_attn.q_norm.weight"] = w["model.layers.0.self_attn.q_norm.weight"] * 0
        # zero queries: uniform attention over the causal prefix, still finite, and different
        z = model_b.forward(toks)
        assert torch.isfinite(z).all() and not torch.allclose(z, base, atol=1e-3)
        assert torch.allclose(z[0], base[0], atol=1e-5)            # one key: softmax is 1 either way
    finally:
        model_b.w = w


def test_tied_head(tmp_path):
    from spyinfer_amd.weights import write_random_model
    m = P.PlainQwen3(write_random_model(str(tmp_path / "a"), TINY_A, 42, torch.bfloat16, **INIT))
    assert m.w["lm_head.weight"] is m.w["model.embed_tokens.weight"]
    assert m.forward([3, 4]).shape == (2, 256)


# ---- the whole pass against a second, independent transcription ---------------------------------------------------
@pytest.fixture(scope="module")
def anchor_folders(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    from tests.configs import TINY_C
    return {name: write_random_model(str(tmp_path_factory.mktemp("anchor_" + name)), cfg, seed, torch.bfloat16, **INIT)
            for name, cfg, seed in (("A", TINY_A, 41), ("B", TINY_B, 42), ("C", TINY_C, 43))}


@pytest.mark.parametrize("name,length", [("A", 23), ("B", 37), ("C", 19)])
def test_whole_pass_equals_the_second_transcription(anchor_folders, name, length):
    """``qwen3_plain`` (CPU backend's formulas, whole sequences, torch) and ``qwen3_second`` (CUDA backend's formulas,
    the model's operation list token by token over growing key/value lists, numpy float64) give the same logits at every
    position.  The installed ``transformers`` package also holds a Qwen3 and would be a third anchor; model code of
    installed packages is not a source for this project, so it is neither imported nor read."""
    from tests.plain.qwen3_second import SecondQwen3
    vocab = {"A": 256, "B": 384, "C": 331}[name]
    toks = torch.randint(0, vocab, (length,), generator=torch.Generator().manual_seed(3)).tolist()
    first = P.PlainQwen3(anchor_folders[name], compute=torch.float64).forward(toks).numpy()
    second = SecondQwen3(anchor_folders[name]).forward(toks)
    assert first.shape == second.shape
    # float64 both; the second forms its rotation angles in float32 as the reference's table does, the first (asked for
    # float64) in float64: 2e-7 on the logits, none at position 0
    assert abs(first - second).max() < 1e-6, abs(first - second).max()
    assert abs(first[0] - second[0]).max() < 1e-12


def _small_queries(folder, dst, factor):
    """The model of ``folder`` with its q and k projections scaled down, so that the mean square of a head vector
    comes near the norms' eps and the eps of the q/k norm shows in the logits."""
    import json
    import os
    import shutil

    from safetensors.torch import load_file

    from spyinfer_amd.weights import write_file
    os.makedirs(dst, exist_ok=True)
    shutil.copy(os.path.join(folder, "config.json"), os.path.join(dst, "config.json"))
    w = {k: v.clone() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    for k in w:
        if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
            w[k] = (w[k].float() * factor).to(torch.bfloat16)
    write_file(os.path.join(dst, "model.safetensors"), w)
    return dst


@pytest.mark.parametrize("mutation", [dict(qk_norm_after_rope=True), dict(qk_eps=1e-4), dict(post_norm_before_add=True),
                                      dict(final_norm=False), dict(embed_scale=96 ** 0.5)])
def test_the_anchor_sees_a_misplaced_norm(anchor_folders, tmp_path, mutation):
    """Each plausible misreading of src/models/qwen3.hpp:113-301, made in the second transcription alone, moves the logits
    by far more than the 1e-4 at which the engine is compared with the plain implementation: the q/k norm after the
    rotation instead of before it, a q/k norm with an eps of its own instead of rms_norm_eps, the post-attention norm
    taken before the residual sum, no final norm, embeddings scaled by sqrt(hidden)."""
    from tests.plain.qwen3_second import SecondQwen3
    folder = anchor_folders["B"]
    if "qk_eps" in mutation:
        folder = _small_queries(folder, str(tmp_path / "small_q"), 2e-3)       # head vectors of mean square ~1e-6
    toks = torch.randint(0, 384, (29,), generator=torch.Generator().manual_seed(4)).tolist()
    first = P.PlainQwen3(folder, compute=torch.float64).forward(toks).numpy()
    assert abs(first - SecondQwen3(folder).forward(toks)).max() < 1e-6
    moved = abs(first - SecondQwen3(folder, **mutation).forward(toks)).max()
    assert moved > 5e-3, "the mutation %r moves the logits by only %g" % (mutation, moved)
