"""The engine on the GPU: greedy generation through the entry point, graphs against eager steps,
long decoding, the first tokens of a sequence, and a toy architecture with a stateful mixer that is
registered, built and stepped without a change to the framework's files."""
import dataclasses
import json
import os

import numpy as np
import pytest
import torch

from spyinfer_amd.kernels import key_pieces
from tests import replay_cases as rc
from tests.configs import INIT, TINY_A, TINY_B, TINY_C, TINY_D, TINY_E
from tests.gpu_util import require_gpu
from tests.plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(atol=1e-4, rtol=1e-4), "bfloat16": dict(atol=8e-2, rtol=2e-2)}


@pytest.fixture(scope="module")
def folder_c(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    return write_random_model(str(tmp_path_factory.mktemp("eng_c")), TINY_C, 61, torch.bfloat16, **INIT)


@pytest.fixture(scope="module")
def folder_a(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    return write_random_model(str(tmp_path_factory.mktemp("eng_a")), TINY_A, 62, torch.bfloat16, **INIT)


def prompts(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


@pytest.mark.parametrize("eager", [True, False])
def test_greedy_float32_equals_plain(folder_a, eager):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    ps = prompts(256, [5, 17, 33, 60], 1)
    plain = PlainQwen3(folder_a)
    want = [plain.greedy(p, 16) for p in ps]
    for opts in (dict(), dict(max_num_batched_tokens=24, num_kvcache_blocks=7)):
        kw = dict(dtype="float32", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=8, enforce_eager=eager)
        kw.update(opts)
        eng = LLMEngine(folder_a, **kw)
        assert eng.generate(ps, SamplingParams(max_new_tokens=16, ignore_eos=True)) == want
        if not eager:
            assert eng.runner.graph_replays > 0
        eng.runner.manager.check()


@pytest.mark.parametrize("eager", [True, False])
def test_requests_ending_while_a_step_is_in_flight(folder_a, eager):
    """Decode steps are launched ahead of the host.  Requests here end at an end-of-sequence token, which the host learns
    one step late: the step in flight still holds their row, their pages go back at once and are taken by requests
    that waited (the pool is small).  Every request's tokens are the plain implementation's, cut at its end token."""
    from collections import Counter
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    ps = prompts(256, [5, 17, 33, 9, 26, 40, 12, 21], 11)
    plain = PlainQwen3(folder_a)
    full = [plain.greedy(p, 14) for p in ps]
    eos = Counter(t for g in full for t in g[2:]).most_common(1)[0][0]
    want = [g[:g.index(eos) + 1] if eos in g else g for g in full]
    assert sum(len(w) < 14 for w in want) >= 2, "the chosen end token must end some requests early"
    eng = LLMEngine(folder_a, dtype="float32", max_model_len=128, num_kvcache_blocks=11, max_num_seqs=3, enforce_eager=eager)
    eng.eos_token_id = eos
    ahead = [0]
    real = eng._launch_ahead
    eng._launch_ahead = lambda flight: (lambda got: (ahead.__setitem__(0, ahead[0] + (got is not None)), got)[1])(real(flight))
    assert eng.generate(ps, SamplingParams(max_new_tokens=14)) == want
    assert ahead[0] >= 10
    eng.runner.manager.check()
    assert eng.runner.manager.num_free_pages() == [11]


@pytest.mark.parametrize("seed", [0, 1])
def test_random_arrivals_endings_and_removals(folder_a, seed):
    """A random serving day in float32 with graphs: requests arrive while others decode, end at an end token, by count
    or by removal, the pool is small enough for preemption.  Every request's tokens are the plain implementation's."""
    import random
    from collections import Counter
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    rng = random.Random(seed)
    lengths = [rng.randint(1, 50) for _ in range(18)]
    ps = prompts(256, lengths, 20 + seed)
    plain = PlainQwen3(folder_a)
    news = [rng.randint(1, 16) for _ in ps]
    full = [plain.greedy(p, n) for p, n in zip(ps, news)]
    eos = Counter(t for g in full for t in g[1:]).most_common(1)[0][0]
    use_eos = [rng.random() < 0.6 for _ in ps]
    want = [g[:g.index(eos) + 1] if (u and eos in g) else g for g, u in zip(full, use_eos)]
    eng = LLMEngine(folder_a, dtype="float32", max_model_len=128, num_kvcache_blocks=13, max_num_seqs=4,
                    max_num_batched_tokens=48)
    eng.eos_token_id = eos
    arrival = sorted((rng.randint(0, 60), i) for i in range(len(ps)))
    removed_at = {i: rng.randint(2, 8) for i in rng.sample(range(len(ps)), 3)}     # steps after arrival
    ids, born, gone, step = {}, {}, {}, 0
    while arrival or eng.has_unfinished_requests():
        while arrival and arrival[0][0] <= step:
            _, i = arrival.pop(0)
            ids[i] = eng.add_request(ps[i], SamplingParams(max_new_tokens=news[i], ignore_eos=not use_eos[i]))
            born[i] = step
        for i, after in removed_at.items():
            if i in ids and i not in gone and step == born[i] + after:
                gone[i] = eng.get_generated_tokens(ids[i])
                eng.remove_request(ids[i])
        eng.step()
        step += 1
        assert step < 2000
    for i in range(len(ps)):
        if i in gone:
            assert gone[i] == want[i][:len(gone[i])], "request %d, removed early, had other tokens" % i
        else:
            assert eng.get_generated_tokens(ids[i]) == want[i], "request %d" % i
    eng.runner.manager.check()
    assert eng.runner.manager.num_free_pages() == [13]
    assert eng.runner.graph_replays > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("eager", [True, False])
def test_config_b_workload(tmp_path_factory, dtype, eager):
    """The second tiny configuration's workload through the entry point on the GPU: prompts of 1 / 40 / 130 tokens in
    portions of 32 beside decoding requests, pages of 8, 24 tokens each; greedy tokens against the plain implementation,
    sampled tokens against the plain sampler on the plain logits."""
    from spyinfer_amd.weights import write_random_model
    from tests.workloads import run_config_b_workload
    require_gpu()
    folder = write_random_model(str(tmp_path_factory.mktemp("eng_b")), TINY_B, 32, torch.bfloat16, **INIT)
    run_config_b_workload(folder, PlainQwen3(folder), "cuda:0", dtype, enforce_eager=eager)


def test_captured_steps_share_their_memory():
    """Decode steps of two dozen shapes (batch sizes: the requests' lengths, from one to four key parts' worth, do not
    make a shape, the host cuts the keys) at a real width and vocabulary are
    captured as graphs into one memory pool with one logits tensor: the memory that torch holds grows by the metadata
    buffers and the activations of the largest step, not by a pool and a logits tensor per graph."""
    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner
    from spyinfer_amd.weights.random_init import random_tensors_on_device
    dev = require_gpu()
    V = 151936
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=2, hidden_size=4096,
               num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=V,
               rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=4096)
    arch = architecture_of(raw)
    model = arch.build(arch.config_cls.from_dict(raw))
    model.bind(random_tensors_on_device(model.weight_specs(), 3, torch.bfloat16, dev), dev)
    per, targets = 24, (100, 300, 550, 800)               # four groups of requests: 1, 2, 3 and 4 key parts
    R = per * len(targets)
    runner = ModelRunner(model, "bfloat16", dev, 16, 3000, R, enforce_eager=False, max_model_len=2048)
    eager = ModelRunner(model, "bfloat16", dev, 16, 3000, R, enforce_eager=True, max_model_len=2048)
    g = torch.Generator().manual_seed(1)
    caches = {r: [r.manager.admit(i) for i in range(R)] for r in (runner, eager)}

    def step(r, ids, tokens):
        for i, t in zip(ids, tokens):
            r.manager.reserve(caches[r][i], len(t))
        return r.step([StepEntry(caches[r][i], t, [len(t) - 1]) for i, t in zip(ids, tokens)])

    for k, target in enumerate(targets):                   # all prompts first, 12 requests a step
        for half in (0, 1):
            ids = list(range(k * per + half * 12, k * per + half * 12 + 12))
            fill = [torch.randint(0, V, (target,), generator=g).tolist() for _ in ids]
            for r in (runner, eager):
                step(r, ids, fill)
    base = None
    for k, target in enumerate(targets):
        for live in (range(1, 25) if k == 0 else (1, 2, 3, 5, 8, 9, 12, 16, 17, 20, 24)):
            ids = list(range(k * per, k * per + live))
            for rep in range(2):                           # a shape is captured at its second step
                toks = [[int(t)] for t in torch.randint(0, V, (live,), generator=g)]
                a, b = step(runner, ids, toks), step(eager, ids, toks)
                if not torch.allclose(a, b, atol=2e-2, rtol=2e-2):
                    d = (a - b).abs()
                    rows = (~(d <= 2e-2 + 2e-2 * b.abs())).any(1).nonzero().flatten().tolist()
                    raise AssertionError("graph and eager logits differ (%d requests near %d tokens, step %d of the shape): by up to %g in "
                                         "rows %s; NaN in %d / %d places" % (live, target, rep, d.nan_to_num(0.0).max().item(), rows,
                                                                             int(a.isnan().sum()), int(b.isnan().sum())))
            if base is None:
                torch.cuda.synchronize()
                base = torch.cuda.memory_reserved(dev)     # after the first capture: the pool and the logits tensor exist
    torch.cuda.synchronize()
    shapes = len(runner._graphs)
    grown = torch.cuda.memory_reserved(dev) - base
    assert shapes >= 24 and runner.graph_replays >= 40, (shapes, runner.graph_replays)
    assert runner._graph_logits.shape == (R, V)
    # 23 more graphs after the first.  With a pool of its own each would hold its logits (0.6 to 14.6 MB) in allocator
    # segments of 20 MB at least: more than 460 MB.  Shared, they add their metadata buffers and the activations of the
    # largest step (24 rows: a few MB), which the allocator rounds up to segments.
    bound = shapes * ModelRunner.graph_metadata_bytes(per, 1, runner.fixed_max_blocks, model.plan_ints(per)) + (128 << 20)
    assert grown <= bound, "captured steps grew torch's memory by %d bytes for %d shapes (bound %d)" % (grown, shapes, bound)
    assert runner.graph_memory_bound() >= 4 * R * V


def test_no_garbage_collection_inside_a_capture(folder_a):
    """While a step is captured as a graph Python's cycle collector rests: a
    dead engine freed inside a capture (its graphs, pools and pinned buffers) makes calls that HIP forbids while a
    stream captures, which ended the process.  Here a dead engine with captured graphs lies in a reference cycle when
    the next engine captures; the model's forward records what it sees."""
    import gc
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    ps = prompts(256, [9, 30], 5)
    sp = SamplingParams(max_new_tokens=6, ignore_eos=True)
    kw = dict(dtype="bfloat16", max_model_len=128, num_kvcache_blocks=40)
    dead = LLMEngine(folder_a, **kw)
    dead.generate(ps, sp)
    assert dead.runner._graphs
    dead.cycle = dead                                     # only the cycle collector can free it now
    del dead
    eng = LLMEngine(folder_a, **kw)
    seen = []
    real = eng.model.forward

    def forward(batch, storage, logits_out=None):
        if torch.cuda.is_current_stream_capturing():
            seen.append(gc.isenabled())
        return real(batch, storage, logits_out)
    eng.model.forward = forward
    try:
        assert gc.isenabled()
        eng.generate(ps, sp)
        assert seen and not any(seen), "the collector ran free inside %d of %d captures" % (sum(seen), len(seen))
        assert gc.isenabled()
    finally:
        eng.model.forward = real


def test_number_of_graphs_is_bounded(folder_a):
    """The runner captures a bounded number of step shapes (each captured step holds its activations); with room for
    two, a run whose batch shrinks from four requests to one runs its later shapes kernel by kernel and still gives
    the plain implementation's tokens."""
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    ps = prompts(256, [5, 17, 33, 9], 12)
    plain = PlainQwen3(folder_a)
    news = [30, 22, 14, 6]
    eng = LLMEngine(folder_a, dtype="float32", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=4)
    eng.runner.max_graphs = 2
    ids = [eng.add_request(p, SamplingParams(max_new_tokens=n, ignore_eos=True)) for p, n in zip(ps, news)]
    while eng.has_unfinished_requests():
        eng.step()
    assert len(eng.runner._graphs) == 2
    assert [eng.get_generated_tokens(i) for i in ids] == [plain.greedy(p, n) for p, n in zip(ps, news)]
    assert 5 < eng.runner.graph_replays < eng.runner.steps_run


def test_greedy_bfloat16_follows_plain(folder_a):
    """bfloat16 may leave the plain tokens only where the plain logits nearly tie."""
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    ps = prompts(256, [5, 17, 33, 60], 2)
    plain = PlainQwen3(folder_a)
    eng = LLMEngine(folder_a, dtype="bfloat16", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=8)
    got = eng.generate(ps, SamplingParams(max_new_tokens=16, ignore_eos=True))
    same = 0
    for p, g in zip(ps, got):
        toks = list(p)
        for t in g:
            logits = plain.forward(toks)[-1]
            best = int(torch.argmax(logits))
            if t != best:
                assert float(logits[best] - logits[t]) < 0.1, "a bfloat16 token differs where the plain logits are apart"
                break
            same += 1
            toks.append(t)
    assert same >= 40


def test_entry_point_with_matrices_in_tiles_only(tmp_path):
    """``weight_copies="tiled"`` through the entry point, with a small configuration whose matrices all have a tiled form
    (widths that are multiples of 128): no matrix of a layer keeps its rows, prompts of more than 64 tokens run through
    the restored rows, and the tokens are those of the engine that keeps both forms; they follow the plain
    implementation as far as its logits do not nearly tie."""
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights import write_random_model
    require_gpu()
    raw = dict(TINY_A, hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=32, intermediate_size=256,
               vocab_size=512, tie_word_embeddings=False, num_hidden_layers=2)
    folder = write_random_model(str(tmp_path / "m"), raw, 71, torch.bfloat16, **INIT)
    ps = prompts(512, [5, 90, 33, 70], 3)
    sp = SamplingParams(max_new_tokens=12, ignore_eos=True)
    kw = dict(dtype="bfloat16", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=8)
    both = LLMEngine(folder, **kw).generate(ps, sp)
    eng = LLMEngine(folder, weight_copies="tiled", **kw)
    layer = eng.model.layers[0]
    for m in (layer.mixer.w_qkv, layer.mixer.w_o, layer.ffn.w_gate_up, layer.ffn.w_down, eng.model.lm_head.weight):
        assert isinstance(m, ops.TiledOnly)
    assert isinstance(eng.model.embed.weight, torch.Tensor)
    got = eng.generate(ps, sp)
    assert got == both
    plain = PlainQwen3(folder)
    same = 0
    for p, g in zip(ps, got):
        toks = list(p)
        for t in g:
            logits = plain.forward(toks)[-1]
            best = int(torch.argmax(logits))
            if t != best:
                assert float(logits[best] - logits[t]) < 0.1, "a bfloat16 token differs where the plain logits are apart"
                break
            same += 1
            toks.append(t)
    assert same >= 24
    with pytest.raises(ValueError):
        LLMEngine(folder, weight_copies="rows", **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(folder_c, dtype):
    """Decode steps from a captured graph, replayed many times with the program's own work between
    them, give what eager steps give, step by step."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    dev = require_gpu()
    model = load_model(folder_c, dtype, dev)
    ps = prompts(331, [40, 3, 130], 3)
    runs = []
    for eager in (True, False):
        runner = ModelRunner(model, dtype, dev, 16, 64, 4, enforce_eager=eager, max_model_len=320)
        caches = [runner.manager.admit(i) for i in range(3)]
        for c, p in zip(caches, ps):
            runner.manager.reserve(c, len(p))
        runner.step([StepEntry(c, p, []) for c, p in zip(caches, ps)])
        g = torch.Generator().manual_seed(4)
        outs = []
        for i in range(40):
            toks = torch.randint(0, 331, (3,), generator=g).tolist()
            for c in caches:
                runner.manager.reserve(c, 1)
            outs.append(runner.step([StepEntry(c, [t], [0]) for c, t in zip(caches, toks)]).cpu().clone())
            _ = torch.randn(1000, device=dev).sum().item()          # other work and a synchronisation between replays
        runs.append(outs)
        if not eager:
            assert runner.graph_replays >= 38
    # graph steps split the keys into a fixed number of parts, eager steps by length: in bfloat16 the two
    # round differently, each within the distance that is allowed against the plain implementation
    tol = TOL[dtype]
    for i, (a, b) in enumerate(zip(*runs)):
        assert torch.allclose(a, b, atol=tol["atol"], rtol=tol["rtol"]), "step %d: graph and eager differ by %g" % (i, (a - b).abs().max())


def test_folded_decode_steps(tmp_path_factory):
    """Steps of few rows in bfloat16 with sizes that allow it run the products with the norms folded in.  With
    that switched off the same steps give the same logits up to bfloat16 rounding, eagerly and from graphs; a
    step of 3 decoded tokens beside a 5-token portion of which only some logits are wanted takes the folded
    layers and the plain output head."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    folder = write_random_model(str(tmp_path_factory.mktemp("eng_d")), TINY_D, 63, torch.bfloat16, **INIT)
    plain = PlainQwen3(folder)
    model = load_model(folder, "bfloat16", dev)
    ps = prompts(400, [40, 3, 130, 21], 3)
    runs, calls = [], []
    real = ops.decode_linear_residual
    for folded, eager in ((True, True), (True, False), (False, True)):
        ops.FUSED_DECODE = folded
        n = [0]
        ops.decode_linear_residual = lambda *a, **k: (n.__setitem__(0, n[0] + 1), real(*a, **k))[1]
        try:
            runner = ModelRunner(model, "bfloat16", dev, 16, 64, 4, enforce_eager=eager, max_model_len=320)
            caches = [runner.manager.admit(i) for i in range(4)]
            for c, p in zip(caches[:3], ps):
                runner.manager.reserve(c, len(p))
            runner.step([StepEntry(c, p, []) for c, p in zip(caches[:3], ps)])
            g = torch.Generator().manual_seed(4)
            outs, seqs = [], [list(p) for p in ps[:3]]
            for i in range(12):
                toks = torch.randint(0, 400, (3,), generator=g).tolist()
                for c in caches[:3]:
                    runner.manager.reserve(c, 1)
                entries = [StepEntry(c, [t], [0]) for c, t in zip(caches[:3], toks)]
                for q, t in zip(seqs, toks):
                    q.append(t)
                if i == 5:
                    runner.manager.reserve(caches[3], 5)
                    entries.insert(1, StepEntry(caches[3], ps[3][:5], [1, 4]))
                outs.append(runner.step(entries).cpu().clone())
            runs.append(outs)
            calls.append(n[0])
        finally:
            ops.FUSED_DECODE = True
            ops.decode_linear_residual = real
    assert calls[0] >= 12 * 2 * 3 and calls[2] == 0
    for i, (a, b, c) in enumerate(zip(*runs)):
        for x, what in ((b, "graphs"), (c, "plain norms")):
            assert a.shape == x.shape and torch.allclose(a, x, **TOL["bfloat16"]), "step %d: folded and %s differ by %g" % (
                i, what, (a - x).abs().max())
    # the last step against the plain implementation
    ref = torch.stack([plain.forward(q)[-1] for q in seqs])
    assert torch.allclose(runs[0][-1], ref, **TOL["bfloat16"]), (runs[0][-1] - ref).abs().max()
    mixed = runs[0][5]
    assert mixed.shape[0] == 5
    ref4 = plain.forward(ps[3][:5])
    assert torch.allclose(mixed[1:3], ref4[[1, 4]], **TOL["bfloat16"])


def test_portions_of_65_to_128_tokens_take_the_folded_products(tmp_path_factory):
    """Steps of 65 to 128 tokens that hold portions (a whole prompt of 100 tokens, 70 tokens of a prompt beside 20 decoded
    tokens, a portion of 128 late in a prompt) run the folded products too: both attention kernels hand their rows over
    in operand order.  Same logits, up to bfloat16 rounding, as with the library's products and norm kernels, and as
    the plain pass."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    folder = write_random_model(str(tmp_path_factory.mktemp("eng_e")), TINY_E, 65, torch.bfloat16, **INIT)
    plain = PlainQwen3(folder)
    model = load_model(folder, "bfloat16", dev)
    V = TINY_E["vocab_size"]
    g = torch.Generator().manual_seed(12)
    whole = torch.randint(0, V, (100,), generator=g).tolist()
    late = torch.randint(0, V, (50 + 70 + 128,), generator=g).tolist()
    others = [torch.randint(0, V, (n + 1,), generator=g).tolist() for n in range(3, 23)]      # 20 requests that decode one token
    runs, calls = [], []
    real = ops.decode_linear_residual
    for folded in (True, False):
        ops.FUSED_DECODE = folded
        n = [0]
        ops.decode_linear_residual = lambda *a, **k: (n.__setitem__(0, n[0] + 1), real(*a, **k))[1]
        try:
            runner = ModelRunner(model, "bfloat16", dev, 16, 80, 22, enforce_eager=True, max_model_len=320)
            caches = [runner.manager.admit(i) for i in range(22)]
            outs = []
            runner.manager.reserve(caches[0], 100)
            outs.append(runner.step([StepEntry(caches[0], whole, [0, 63, 64, 99])]).cpu().clone())
            for c, q in zip(caches[2:], others):
                runner.manager.reserve(c, len(q) - 1)
            runner.step([StepEntry(c, q[:-1], []) for c, q in zip(caches[2:], others)])
            runner.manager.reserve(caches[1], 50)
            runner.step([StepEntry(caches[1], late[:50], [])])
            before = n[0]
            for c in caches[1:]:
                runner.manager.reserve(c, 70 if c is caches[1] else 1)
            outs.append(runner.step([StepEntry(caches[1], late[50:120], [0, 69])] + [StepEntry(c, [q[-1]], [0]) for c, q in zip(caches[2:], others)]).cpu().clone())
            runner.manager.reserve(caches[1], 128)
            outs.append(runner.step([StepEntry(caches[1], late[120:], [0, 127])]).cpu().clone())
            calls.append((before, n[0]))
            runs.append(outs)
        finally:
            ops.FUSED_DECODE = True
            ops.decode_linear_residual = real
    layers = TINY_E["num_hidden_layers"]
    assert calls[0][1] - calls[0][0] == 2 * 2 * layers and calls[1] == (0, 0), calls      # two products a layer in each of the last two steps
    for a, b in zip(*runs):
        assert a.shape == b.shape and torch.allclose(a, b, **TOL["bfloat16"]), (a - b).abs().max()
    ref_whole, ref_late = plain.forward(whole), plain.forward(late)
    assert torch.allclose(runs[0][0], ref_whole[[0, 63, 64, 99]], **TOL["bfloat16"])
    assert torch.allclose(runs[0][1][:2], ref_late[[50, 119]], **TOL["bfloat16"])
    assert torch.allclose(runs[0][1][2:], torch.stack([plain.forward(q)[-1] for q in others]), **TOL["bfloat16"])
    assert torch.allclose(runs[0][2], ref_late[[120, 247]], **TOL["bfloat16"])


@pytest.mark.parametrize("requests", [19, 37, 57, 64, 70, 100, 130])
def test_folded_decode_steps_of_many_requests(tmp_path_factory, requests):
    """Decode steps of 17 to 128 requests take the folded products with two to eight row tiles (130 requests: the library's); their logits equal, up to
    bfloat16 rounding, those of the same steps with the norms as kernels of their own, from graphs as well, and the last
    step's equal the plain implementation's.  Parts may be built to fold up to fewer rows (48 here): the embedding then still prepares the first norm's input, which the unfolded block does not use."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    folder = write_random_model(str(tmp_path_factory.mktemp("eng_many")), TINY_D, 64, torch.bfloat16, **INIT)
    plain = PlainQwen3(folder)
    model = load_model(folder, "bfloat16", dev)
    ps = prompts(400, [3 + (7 * i) % 23 for i in range(requests)], 5)
    runs, calls = [], []
    real = ops.decode_linear_residual
    assert ops.default_fold_rows(1 << 20) == 128
    for folded, eager, fold_rows in ((True, True, None), (True, False, None), (False, True, None), (True, True, 48)):
        ops.FUSED_DECODE = folded
        for layer in model.layers:
            layer.mixer.fold_rows = layer.ffn.fold_rows = fold_rows
        n = [0]
        ops.decode_linear_residual = lambda *a, **k: (n.__setitem__(0, n[0] + 1), real(*a, **k))[1]
        try:
            runner = ModelRunner(model, "bfloat16", dev, 16, 4 * requests, requests, enforce_eager=eager, max_model_len=64)
            caches = [runner.manager.admit(i) for i in range(requests)]
            for c, p in zip(caches, ps):
                runner.manager.reserve(c, len(p))
            runner.step([StepEntry(c, p, []) for c, p in zip(caches, ps)])
            g = torch.Generator().manual_seed(6)
            outs, seqs = [], [list(p) for p in ps]
            for i in range(5):
                toks = torch.randint(0, 400, (requests,), generator=g).tolist()
                for c in caches:
                    runner.manager.reserve(c, 1)
                for q, t in zip(seqs, toks):
                    q.append(t)
                outs.append(runner.step([StepEntry(c, [t], [0]) for c, t in zip(caches, toks)]).cpu().clone())
            runs.append(outs)
            calls.append(n[0])
        finally:
            ops.FUSED_DECODE = True
            ops.decode_linear_residual = real
    if requests <= ops.FUSED_DECODE_MAX_ROWS:
        assert calls[0] >= 5 * 2 * 3 and calls[2] == 0 and (calls[3] == 0) == (requests > 48)
    else:
        assert calls == [0, 0, 0, 0]          # more rows than the folded products take: the library's, with norm kernels
    for i, (a, b, c, e) in enumerate(zip(*runs)):
        for x, what in ((b, "graphs"), (c, "plain norms"), (e, "parts that fold up to 48 rows")):
            assert a.shape == x.shape and torch.allclose(a, x, **TOL["bfloat16"]), "step %d: folded and %s differ by %g" % (
                i, what, (a - x).abs().max())
    ref = torch.stack([plain.forward(q)[-1] for q in seqs])
    assert torch.allclose(runs[0][-1], ref, **TOL["bfloat16"]), (runs[0][-1] - ref).abs().max()


def test_layers_that_fold_up_to_different_rows(tmp_path_factory):
    """A run order in which a block that folds follows one that does not (parts built to fold up to fewer rows): at
    100 single tokens the second block gets an ordinary addend, not the prepared input in operand order that the
    folded products need beyond 64 rows, and takes the plain path instead of asking a product for what it refuses."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    folder = write_random_model(str(tmp_path_factory.mktemp("eng_mixfold")), TINY_D, 65, torch.bfloat16, **INIT)
    plain = PlainQwen3(folder)
    model = load_model(folder, "bfloat16", dev)
    model.layers[0].mixer.fold_rows = model.layers[0].ffn.fold_rows = 48
    model.layers[2].ffn.fold_rows = 48                   # and a block whose mixer folds and whose feed-forward does not
    requests = 100
    ps = prompts(400, [3 + (5 * i) % 19 for i in range(requests)], 6)
    runner = ModelRunner(model, "bfloat16", dev, 16, 4 * requests, requests, enforce_eager=True, max_model_len=64)
    caches = [runner.manager.admit(i) for i in range(requests)]
    for c, p in zip(caches, ps):
        runner.manager.reserve(c, len(p))
    runner.step([StepEntry(c, p, []) for c, p in zip(caches, ps)])
    g = torch.Generator().manual_seed(7)
    seqs = [list(p) for p in ps]
    for i in range(3):
        toks = torch.randint(0, 400, (requests,), generator=g).tolist()
        for c in caches:
            runner.manager.reserve(c, 1)
        for q, t in zip(seqs, toks):
            q.append(t)
        got = runner.step([StepEntry(c, [t], [0]) for c, t in zip(caches, toks)]).cpu()
    ref = torch.stack([plain.forward(q)[-1] for q in seqs])
    assert torch.allclose(got, ref, **TOL["bfloat16"]), (got - ref).abs().max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(folder_c, dtype, tmp_path):
    require_gpu()
    reqs = rc.random_requests(331, [500, 1, 2], seed=8)
    plain = PlainQwen3(folder_c)
    ref = {rid: plain.forward(t) for rid, t in reqs.items()}
    steps = rc.bulk_tail(reqs, tail=480)                 # 20 tokens at once, then 480 one by one
    rc.run_replay_inprocess(folder_c, dtype, str(tmp_path), steps, rc.max_live_tokens(steps))
    got = rc.collect(str(tmp_path), steps, 331)
    assert len(got) == 503
    rc.compare(got, ref, what="long decoding " + dtype, **TOL[dtype])


def test_temperature_through_entry_point(folder_a):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    ps = prompts(256, [9, 30], 5)
    sp = SamplingParams(temperature=0.8, max_new_tokens=12, ignore_eos=True)
    kw = dict(dtype="float32", max_model_len=128, num_kvcache_blocks=40, seed=3)
    a = LLMEngine(folder_a, **kw).generate(ps, sp)
    b = LLMEngine(folder_a, max_num_batched_tokens=8, **kw).generate(ps, sp)
    assert a == b and a[0] != a[1]
    greedy = LLMEngine(folder_a, **kw).generate(ps, SamplingParams(max_new_tokens=12, ignore_eos=True))
    assert greedy != a


def test_command_line(folder_a, tmp_path):
    """python -m spyinfer_amd -m MODEL --prompt-ids ...: the generated ids of each prompt on a line; and the
    conversation loop with /new and /exit on standard input."""
    import subprocess
    import sys
    require_gpu()
    ps = prompts(256, [7, 21], 9)
    plain = PlainQwen3(folder_a)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    base = [sys.executable, "-m", "spyinfer_amd", "-m", folder_a, "--dtype", "float32", "--max-model-len", "128",
            "--num-kvcache-blocks", "32", "--max-new-tokens", "5", "--ignore-eos"]
    cmd = base + sum((["--prompt-ids", " ".join(map(str, p))] for p in ps), [])
    r = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.strip().splitlines() if l and l[0].isdigit()]
    assert [[int(x) for x in l.split()] for l in lines] == [plain.greedy(p, 5) for p in ps]
    # the same prompts from a file, one a line; and prompts drawn from --seed by their lengths
    path = tmp_path / "prompts.txt"
    path.write_text("".join(",".join(map(str, p)) + "\n" for p in ps) + "\n")
    r = subprocess.run(base + ["--prompt-file", str(path), "--random-prompts", "6,11", "--seed", "4"], cwd=root, capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [[int(x) for x in l.split()] for l in r.stdout.strip().splitlines() if l and l[0].isdigit()]
    g = torch.Generator().manual_seed(4)
    drawn = [torch.randint(0, 256, (n,), generator=g).tolist() for n in (6, 11)]
    assert lines == [plain.greedy(p, 5) for p in ps + drawn]
    talk = "%s\n/new\n%s\n/exit\n" % (",".join(map(str, ps[0])), " ".join(map(str, ps[1])))
    r = subprocess.run(base, cwd=root, input=talk, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    answers = [l.split("Assistant:")[1].split() for l in r.stdout.splitlines() if "Assistant:" in l]
    assert [[int(x) for x in a] for a in answers] == [plain.greedy(p, 5) for p in ps]
    assert "Starting new conversation." in r.stdout


# ---------------------------------------------------------------------------------------------
# A toy architecture defined here: blocks whose mixer keeps a running mean of its inputs per
# request (state of fixed size in a slot) beside ordinary attention blocks.

def _toy_parts(head_dim=16):
    from spyinfer_amd.cache import FixedState
    from spyinfer_amd.config import ModelConfig
    from spyinfer_amd.models import DecoderModel, LayerCall
    from spyinfer_amd.parts import GatedMLP, LMHead, PagedAttention, PreNormBlock, RMSNorm, RotaryEmbedding, TokenEmbedding
    from spyinfer_amd.parts.base import Mixer
    from spyinfer_amd.weights import WeightSpec

    class RunningMean(Mixer):
        """out[t] = gain * mean of the request's inputs up to t.  State: [H] sums and one count."""

        def __init__(self, hidden):
            self.hidden = hidden

        def weight_specs(self, prefix):
            return [WeightSpec(prefix + ".gain", (self.hidden,), "norm")]

        def bind(self, prefix, weights):
            self.gain = weights[prefix + ".gain"]

        def cache_spec(self):
            return FixedState((self.hidden + 1,), "float32")

        def forward(self, x, batch, cache, store=True):
            out = torch.empty_like(x)
            cu = batch.host_cu_q
            for s, e in enumerate(batch.entries):
                st = cache.state[e.cache.slot]
                xs = x[cu[s]:cu[s + 1]].float()
                sums = torch.cumsum(xs, 0) + st[:self.hidden]
                cnt = st[self.hidden] + torch.arange(1, xs.shape[0] + 1, device=x.device, dtype=torch.float32)
                out[cu[s]:cu[s + 1]] = (sums / cnt[:, None] * self.gain.float()).to(x.dtype)
                if store:
                    st[:self.hidden] = sums[-1]
                    st[self.hidden] = cnt[-1]
            return out

        def plan(self, batch):
            batch.host_cu_q = [0] + list(np.cumsum(batch.lens))

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        hidden_size: int = 0
        num_hidden_layers: int = 0
        vocab_size: int = 0
        intermediate_size: int = 0

    def build(cfg):
        emb = TokenEmbedding(cfg.vocab_size, cfg.hidden_size)
        rope = RotaryEmbedding(head_dim, 10000.0)
        layers = []
        for i in range(cfg.num_hidden_layers):
            mixer = RunningMean(cfg.hidden_size) if i % 2 == 0 else PagedAttention(cfg.hidden_size, 4, 2, head_dim, rope, window=24)
            layers.append(PreNormBlock(RMSNorm(cfg.hidden_size, 1e-5), mixer, RMSNorm(cfg.hidden_size, 1e-5),
                                       GatedMLP(cfg.hidden_size, cfg.intermediate_size)))
        # the run order names layer 1 twice (its weights run again with a cache of their own)
        order = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2), LayerCall(1, 3)]
        return DecoderModel(cfg, emb, rope, layers, RMSNorm(cfg.hidden_size, 1e-5), LMHead(cfg.vocab_size, cfg.hidden_size, tied_to=emb),
                            schedule=order, max_positions=512)

    return ToyConfig, build


def _plain_running_mean_lm(folder, tokens, head_dim=16):
    """The toy model of ``_toy_parts`` on a whole sequence, no cache, from the plain functions: layers 0 and 2 mix by a
    running mean, layer 1 by attention over a window of 24, and the run order is layers 0, 1, 2, 1."""
    from safetensors.torch import load_file
    from tests.plain import qwen3_plain as P
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    T = len(tokens)
    cos, sin = P.rope_tables(T, head_dim, 10000.0)
    pos = torch.arange(T)
    h = P.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    for layer in (0, 1, 2, 1):
        p = "model.layers.%d." % layer
        n1 = P.rms_norm(h, w[p + "input_layernorm.weight"], 1e-5)
        if layer == 1:
            q = P.rope_apply(P.linear(n1, w[p + "self_attn.q_proj.weight"]).view(T, 4, head_dim), pos, cos, sin)
            k = P.rope_apply(P.linear(n1, w[p + "self_attn.k_proj.weight"]).view(T, 2, head_dim), pos, cos, sin)
            v = P.linear(n1, w[p + "self_attn.v_proj.weight"]).view(T, 2, head_dim)
            a = P.linear(P.attention(q, k, v, 24).reshape(T, -1), w[p + "self_attn.o_proj.weight"])
        else:
            a = torch.cumsum(n1, 0) / (pos + 1).float()[:, None] * w[p + "self_attn.gain"]
        h = h + a
        n2 = P.rms_norm(h, w[p + "post_attention_layernorm.weight"], 1e-5)
        h = h + P.linear(P.swiglu(P.linear(n2, w[p + "mlp.gate_proj.weight"]), P.linear(n2, w[p + "mlp.up_proj.weight"])),
                         w[p + "mlp.down_proj.weight"])
    return P.linear(P.rms_norm(h, w["model.norm.weight"], 1e-5), w["model.embed_tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("head_dim", [16, 64])
def test_toy_architecture_with_state(dtype, head_dim, tmp_path):
    """(Heads of 64 take the attention kernels' paths for full head sizes, whose loads have no conditions: the window of
    24 then runs over pages that the requests have given back.)"""
    from spyinfer_amd.config import register_architecture, unregister_architecture
    from spyinfer_amd.weights import write_random_model
    require_gpu()
    ToyConfig, build = _toy_parts(head_dim)
    register_architecture("ToyRunningMeanLM", ToyConfig, build)
    try:
        cfg = dict(architectures=["ToyRunningMeanLM"], hidden_size=64, num_hidden_layers=3, vocab_size=97, intermediate_size=80)
        folder = write_random_model(str(tmp_path / "toy"), cfg, 71, torch.bfloat16, **INIT)
        reqs = rc.random_requests(97, [70, 9, 41, 120, 33], seed=9)
        outs = {}
        for mode in ("whole", "portions", "mixed"):
            steps = getattr(rc, mode)(reqs)
            out = str(tmp_path / mode)
            rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps))
            outs[mode] = rc.collect(out, steps, 97)
        tol = TOL[dtype]
        ref = {rid: _plain_running_mean_lm(folder, t, head_dim) for rid, t in reqs.items()}
        for mode in ("whole", "portions", "mixed"):
            rc.compare(outs[mode], ref, what="toy with state/%s/%s" % (mode, dtype), **tol)
        # the state matters: a request's logits differ from those of its second half alone
        first = next(iter(reqs))
        assert not np.allclose(outs["whole"][(first, 40)], outs["whole"][(first, 5)], atol=1e-3)
    finally:
        unregister_architecture("ToyRunningMeanLM")


def _running_mean_on_device(base):
    """The toy mixer again, written on the batch's device arrays alone (``slot_ids``, ``token_entry``, ``cu_q``): no
    value of the step is read on the host, so its decode steps may be recorded in a graph, and it says so."""

    class RunningMeanOnDevice(base):
        def capturable(self, batch):
            return True

        def plan(self, batch):
            pass

        def forward(self, x, batch, cache, store=True):
            H, T = self.hidden, x.shape[0]
            xs = x.float()
            entry = batch.token_entry.long()
            start = batch.cu_q.long()[entry]                       # first token of every token's entry
            slots = batch.slot_ids.long()
            csum = torch.cumsum(xs, 0)
            before = torch.where((start > 0)[:, None], csum[(start - 1).clamp(min=0)], torch.zeros_like(csum))
            state = cache.state[slots[entry]]                      # [T, H + 1]: the sums and the count before this step
            sums = csum - before + state[:, :H]
            cnt = state[:, H] + (torch.arange(T, device=x.device) - start + 1).float()
            if store:
                last = batch.cu_q.long()[1:] - 1
                cache.state.index_copy_(0, slots, torch.cat([sums[last], cnt[last][:, None]], 1))
            return (sums / cnt[:, None] * self.gain.float()).to(x.dtype)

    return RunningMeanOnDevice


@pytest.mark.parametrize("kind,head_dim", [("host", 16), ("device", 16), ("device", 64)])
def test_toy_with_state_through_the_entry_point_with_graphs(kind, head_dim, tmp_path):
    """The toy architecture with a running state behind ``LLMEngine`` with graphs allowed (the default): seven requests
    of different lengths, three at a time, so that slots and pages are handed out again.  The mixer that walks
    ``batch.entries`` on the host does not call itself capturable, so no step of its model is recorded; the same
    mixer written on the device arrays does, and its decode steps are replayed.  Greedy tokens equal the plain pass's
    either way: a replay with the slots of the recorded step would mix the requests' states."""
    from spyinfer_amd.config import register_architecture, unregister_architecture
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights import write_random_model
    import spyinfer_amd.parts.base as parts_base
    require_gpu()
    ToyConfig, build = _toy_parts(head_dim)
    if kind == "device":
        host_build = build

        def build(cfg):
            model = host_build(cfg)
            for layer in model.layers:
                if type(layer.mixer).__name__ == "RunningMean":
                    layer.mixer.__class__ = _running_mean_on_device(type(layer.mixer))
            return model
    register_architecture("ToyRunningMeanLM", ToyConfig, build)
    try:
        cfg = dict(architectures=["ToyRunningMeanLM"], hidden_size=64, num_hidden_layers=3, vocab_size=97, intermediate_size=80)
        folder = write_random_model(str(tmp_path / "toy"), cfg, 72, torch.bfloat16, **INIT)
        lengths, news = [70, 9, 41, 3, 33, 18, 55], [12, 20, 9, 25, 14, 17, 11]
        ps = prompts(97, lengths, 13)
        eng = LLMEngine(folder, dtype="float32", max_model_len=128, num_kvcache_blocks=14, max_num_seqs=3, max_num_batched_tokens=48)
        assert not eng.config.enforce_eager and eng.runner.use_graphs
        slots_seen = []
        admit = eng.runner.manager.admit
        eng.runner.manager.admit = lambda rid: (lambda rc: (slots_seen.append(rc.slot), rc)[1])(admit(rid))
        ids = [eng.add_request(p, SamplingParams(max_new_tokens=n, ignore_eos=True)) for p, n in zip(ps, news)]
        while eng.has_unfinished_requests():
            eng.step()
        got = [eng.get_generated_tokens(i) for i in ids]
        assert len(slots_seen) >= 7 and max(slots_seen.count(s) for s in set(slots_seen)) >= 2      # slots were used again
        if kind == "host":
            assert eng.runner.graph_replays == 0 and not eng.runner._graphs
        else:
            assert eng.runner.graph_replays >= 20 and eng.model.capturable(None)
        for p, n, g in zip(ps, news, got):
            toks = list(p)
            for t in g:
                logits = _plain_running_mean_lm(folder, toks, head_dim)[-1]
                best = int(torch.argmax(logits))
                assert t == best or float(logits[best] - logits[t]) < 1e-3, "request of %d tokens leaves the plain pass" % len(p)
                toks.append(t)
            assert len(g) == n
        eng.runner.manager.check()
        assert eng.runner.manager.slots.num_free == 3
        # a part that says nothing is taken to read the step on the host
        assert parts_base.Part().capturable(None) is False
    finally:
        unregister_architecture("ToyRunningMeanLM")


def test_matrices_in_tiles_only_in_a_captured_step_of_130_tokens():
    """``weight_copies="tiled"`` with more single tokens in a step than the products take from the tiles (130 > 128): every
    matrix's rows are restored ahead of its product into the device's one scratch tensor, inside a graph capture as
    outside.  Logits equal those of the runner that keeps both forms, step by step, and the captured step holds no
    restored rows of its own (one copy of every matrix would be 132 MB here)."""
    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, bind_weights
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.weights.random_init import random_tensors_on_device
    dev = require_gpu()
    V, R = 8192, 130
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=4, hidden_size=1024,
               num_attention_heads=8, num_key_value_heads=2, head_dim=128, intermediate_size=4096, vocab_size=V,
               rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=256)
    arch = architecture_of(raw)
    runners = {}
    for copies in ("both", "tiled"):
        model = arch.build(arch.config_cls.from_dict(raw))
        bind_weights(model, random_tensors_on_device(model.weight_specs(), 5, torch.bfloat16, dev, matrix_std=0.04), dev, copies)
        runners[copies] = ModelRunner(model, "bfloat16", dev, 16, 2 * R, R, enforce_eager=copies == "both", max_model_len=32)
    tiled = runners["tiled"]
    assert isinstance(tiled.model.layers[0].ffn.w_gate_up, ops.TiledOnly) and isinstance(tiled.model.lm_head.weight, ops.TiledOnly)
    one_copy_each = sum(m.tiled.numel() * 2 for layer in tiled.model.layers
                        for m in (layer.mixer.w_qkv, layer.mixer.w_o, layer.ffn.w_gate_up, layer.ffn.w_down)) + tiled.model.lm_head.weight.tiled.numel() * 2
    assert one_copy_each > (120 << 20)
    g = torch.Generator().manual_seed(2)
    caches = {k: [r.manager.admit(i) for i in range(R)] for k, r in runners.items()}
    base = None
    for step in range(6):
        toks = torch.randint(0, V, (R,), generator=g).tolist()
        out = {}
        for k, r in runners.items():
            for c in caches[k]:
                r.manager.reserve(c, 1)
            out[k] = r.step([StepEntry(c, [t], [0]) for c, t in zip(caches[k], toks)]).clone()
        assert torch.allclose(out["tiled"], out["both"], atol=8e-2, rtol=2e-2), "step %d: %g" % (step, (out["tiled"] - out["both"]).abs().max())
        if step == 0:
            torch.cuda.synchronize()
            base = torch.cuda.memory_reserved(dev)           # after the eager step: the scratch tensor and the activations exist
    torch.cuda.synchronize()
    assert tiled.graph_replays >= 4 and len(tiled._graphs) == 1
    grown = torch.cuda.memory_reserved(dev) - base
    # what does grow: the library's workspace of 76 MB, which a first product inside a capture takes from the graph's pool,
    # the logits tensor and a segment for the activations (94 MB were measured)
    assert grown <= (112 << 20), "the captured step holds %d MB more (one restored copy of every matrix: %d MB)" % (
        grown >> 20, one_copy_each >> 20)


LONG_N, SHORT_N, LONG_STEPS = 4200, 37, 40


def test_requests_of_uneven_lengths_decode_under_graphs(tmp_path):
    """Twenty requests of 1 to 1500 tokens decode 40 steps, recorded once and replayed: the host cuts every step's keys
    anew (long requests into parts, short ones whole; the cut changes as requests pass 32-key blocks), the recorded
    launch stays the same.  Logits of every step and request against the plain pass of the whole sequences."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.weights import write_random_model
    dev = require_gpu()
    raw = dict(TINY_E, max_position_embeddings=2048)
    folder = write_random_model(str(tmp_path), raw, 17, torch.bfloat16, **INIT)
    lengths = [1, 5, 31, 32, 33, 63, 64, 100, 129, 200, 255, 300, 450, 511, 700, 900, 1100, 1279, 1400, 1500]
    steps = 40
    g = torch.Generator().manual_seed(3)
    seqs = [torch.randint(0, raw["vocab_size"], (n + steps,), generator=g).tolist() for n in lengths]
    plain = PlainQwen3(folder)
    ref = [plain.forward(q) for q in seqs]
    R = len(lengths)
    runner = ModelRunner(load_model(folder, "bfloat16", dev), "bfloat16", dev, 16, sum(-(-(n + steps) // 16) for n in lengths) + 4, R,
                         enforce_eager=False, max_model_len=2048)
    caches = [runner.manager.admit(i) for i in range(R)]
    for c, q, n in zip(caches, seqs, lengths):
        runner.manager.reserve(c, n)
        runner.step([StepEntry(c, q[:n], [])])
    cuts = set()
    for i in range(steps):
        for c in caches:
            runner.manager.reserve(c, 1)
        got = runner.step([StepEntry(c, [q[n + i]], [0]) for c, q, n in zip(caches, seqs, lengths)]).cpu()
        want = torch.stack([r[n + i] for r, n in zip(ref, lengths)])
        assert torch.allclose(got, want, **TOL["bfloat16"]), "step %d: off by %s" % (i, (got - want).abs().max(1).values.tolist())
        rec = key_pieces.decode_pieces([n + i + 1 for n in lengths], raw["num_key_value_heads"], 0, head_dim=raw["head_dim"])
        cuts.add(tuple(rec[rec[:, 4] == 0][:, 5].tolist()))
    assert runner.graph_replays >= steps - 2 and len(runner._graphs) == 1
    assert len(cuts) > 1 and max(max(c) for c in cuts) > 1 and min(min(c) for c in cuts) == 1


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """Config E with 4608 positions and doubled q and k norm weights (single far keys carry most of a softmax's weight),
    a sequence of 4240 tokens and one of 77, and the plain pass's logits of both."""
    from safetensors.torch import load_file
    from spyinfer_amd.weights import write_file, write_random_model
    raw = dict(TINY_E, max_position_embeddings=4608)
    folder = write_random_model(str(tmp_path_factory.mktemp("long")), raw, 91, torch.bfloat16, **INIT)
    path = os.path.join(folder, "model.safetensors")
    w = {k: v.clone() for k, v in load_file(path).items()}
    for k in w:
        if k.endswith("q_norm.weight") or k.endswith("k_norm.weight"):
            w[k] = (w[k].float() * 2.0).to(torch.bfloat16)
    write_file(path, w)
    g = torch.Generator().manual_seed(8)
    seqs = [torch.randint(0, raw["vocab_size"], (n + LONG_STEPS,), generator=g).tolist() for n in (LONG_N, SHORT_N)]
    plain = PlainQwen3(folder)
    ref = [plain.forward(s) for s in seqs]
    # the construction does what it says: without the keys 1280..1535 (one of the 16 parts) the plain logits move visibly
    cut = plain.forward(seqs[0][:1280] + seqs[0][1536:])
    assert (cut[-LONG_STEPS:] - ref[0][-LONG_STEPS:]).abs().max() > 0.5
    return folder, seqs, ref


@pytest.mark.parametrize("dtype,cut", [("float32", "as measured"), ("bfloat16", "as measured"), ("bfloat16", "finest")])
def test_a_request_of_4200_tokens_decodes_under_graphs(dtype, cut, long_model, monkeypatch):
    """One long request beside a short one, decode steps recorded and replayed: block tables of the fixed width that
    4608 positions need (288 pages), the long request's keys in 16 parts (float32: the plain kernel reads them in one) or
    in the dozen and more pieces that the host cuts them into beside the short request, which stays whole ("finest": in
    more than sixteen, which the merging block takes in three and four rounds).  A part of the keys that is lost, read through
    a wrong page or merged wrongly moves the logits far beyond the tolerance (the fixture asserts it on the plain pass).
    Logits of every decode step against the plain pass of the whole sequences."""
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    folder, seqs, ref = long_model
    long_n, short_n, steps = LONG_N, SHORT_N, LONG_STEPS
    if cut == "finest":
        monkeypatch.setattr(key_pieces, "PIECE_MIN_BLOCKS", 4)
        monkeypatch.setattr(key_pieces, "PIECE_MERGE_MORE_US", 0.0)
    runner = ModelRunner(load_model(folder, dtype, dev), dtype, dev, 16, 300, 2, enforce_eager=False, max_model_len=4608)
    assert runner.fixed_max_blocks == 288
    caches = [runner.manager.admit(i) for i in range(2)]
    for lo in range(0, long_n, 2048):                               # the long prompt in portions
        n = min(2048, long_n - lo)
        runner.manager.reserve(caches[0], n)
        runner.step([StepEntry(caches[0], seqs[0][lo:lo + n], [])])
    runner.manager.reserve(caches[1], short_n)
    runner.step([StepEntry(caches[1], seqs[1][:short_n], [])])
    tol = dict(atol=1e-4, rtol=1e-4) if dtype == "float32" else dict(atol=0.28, rtol=0.02)
    parts = set()
    for i in range(steps):
        for c in caches:
            runner.manager.reserve(c, 1)
        got = runner.step([StepEntry(caches[0], [seqs[0][long_n + i]], [0]), StepEntry(caches[1], [seqs[1][short_n + i]], [0])]).cpu()
        parts.add(ops.key_parts_for(long_n + i + 1))
        if dtype == "bfloat16":
            # how the host cuts this step's keys: the long request in a dozen parts and more, the short one whole
            rec = key_pieces.decode_pieces([long_n + i + 1, short_n + i + 1], TINY_E["num_key_value_heads"], 0, head_dim=TINY_E["head_dim"])
            assert rec[rec[:, 0] == 0][0, 5] >= (20 if cut == "finest" else 12) and rec[rec[:, 0] == 1][0, 5] == 1
        want = torch.stack([ref[0][long_n + i], ref[1][short_n + i]])
        assert torch.allclose(got, want, **tol), "decode step %d (%s): off by %g / %g" % (
            i, "replayed" if i >= 2 else "eager or captured", (got[0] - want[0]).abs().max(), (got[1] - want[1]).abs().max())
    assert parts == {16} and runner.graph_replays >= steps - 2
