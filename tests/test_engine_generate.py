"""Generation through the entry point on the CPU stand-in for the kernels: greedy tokens equal
the plain implementation's whatever the budget, the pool or the company; temperature sampling
does not depend on the batch."""
import pytest
import torch

from spyinfer_amd.sampling import SamplingParams, uniform_for
from tests.configs import INIT, TINY_A, TINY_B
from tests.plain.qwen3_plain import PlainQwen3


@pytest.fixture(scope="module")
def folder_a(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    return write_random_model(str(tmp_path_factory.mktemp("gen_a")), TINY_A, 31, torch.bfloat16, **INIT)


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    return write_random_model(str(tmp_path_factory.mktemp("gen_b")), TINY_B, 32, torch.bfloat16, **INIT)


def prompts(vocab, lengths, seed=1):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


def test_greedy_equals_plain_under_every_schedule(folder_a, emu_ops):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    ps = prompts(256, [5, 17, 33, 60])
    plain = PlainQwen3(folder_a)
    want = [plain.greedy(p, 16) for p in ps]
    sp = SamplingParams(max_new_tokens=16, ignore_eos=True)
    for opts in (dict(), dict(max_num_batched_tokens=32), dict(max_num_batched_tokens=7, max_num_seqs=3),
                 dict(num_kvcache_blocks=7, max_num_batched_tokens=24)):      # 7 pages of 16: preemption
        kw = dict(dtype="float32", device="cpu", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=8)
        kw.update(opts)
        eng = LLMEngine(folder_a, **kw)
        got = eng.generate(ps, sp)
        assert got == want, opts
        assert eng.runner.manager.num_free_pages() == [kw["num_kvcache_blocks"]]
        if "num_kvcache_blocks" in opts:
            assert eng.scheduler.num_preemptions > 0
        eng.runner.manager.check()


def test_temperature_is_independent_of_the_batch(folder_b, emu_ops):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    ps = prompts(384, [1, 40, 130], seed=2)
    sp = SamplingParams(temperature=0.8, max_new_tokens=24, ignore_eos=True)
    kw = dict(dtype="float32", device="cpu", max_model_len=256, kvcache_block_size=8, num_kvcache_blocks=80, seed=9)
    together = LLMEngine(folder_b, max_num_batched_tokens=32, **kw).generate(ps, sp)
    alone = []
    for i, p in enumerate(ps):
        eng = LLMEngine(folder_b, **kw)
        eng._next_id = i                       # same request id -> same stream of uniform numbers
        alone.append(eng.generate([p], sp)[0])
    assert together == alone
    assert len({tuple(x) for x in together}) == 3


def test_finishing(folder_b, emu_ops):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    eng = LLMEngine(folder_b, dtype="float32", device="cpu", max_model_len=12, kvcache_block_size=8, num_kvcache_blocks=8)
    plain = PlainQwen3(folder_b)
    p = prompts(384, [6], seed=3)[0]
    first = plain.greedy(p, 1)[0]
    eng.eos_token_id = first                   # the first generated token ends the request and is kept
    rid = eng.add_request(p)
    while not eng.is_request_finished(rid):
        eng.step()
    assert eng.get_output_tokens(rid) == p + [first] and eng.finish_reason(rid) == "eos"
    rid = eng.add_request(p, SamplingParams(ignore_eos=True))
    while not eng.is_request_finished(rid):
        eng.step()
    assert len(eng.get_output_tokens(rid)) == 12 and eng.finish_reason(rid) == "max_model_len"
    # a further turn of a finished request
    eng.config.max_model_len = eng.scheduler.max_model_len = 40
    rid = eng.add_request(p, SamplingParams(max_new_tokens=3, ignore_eos=True))
    while not eng.is_request_finished(rid):
        eng.step()
    turn1 = eng.get_output_tokens(rid)
    eng.append_to_request(rid, [9, 8, 7], SamplingParams(max_new_tokens=2, ignore_eos=True))
    while not eng.is_request_finished(rid):
        eng.step()
    assert eng.get_output_tokens(rid)[:len(turn1) + 3] == turn1 + [9, 8, 7]
    assert eng.get_output_tokens(rid)[len(turn1) + 3:] == plain.greedy(turn1 + [9, 8, 7], 2)
    eng.remove_request(rid)
    assert not eng.has_unfinished_requests()
    with pytest.raises(TypeError, match="known"):
        LLMEngine(folder_b, device="cpu", page_size=4)
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([999])


def test_uniform_numbers():
    us = [uniform_for(3, i) for i in range(2000)]
    assert all(0.0 <= u < 1.0 for u in us) and abs(sum(us) / len(us) - 0.5) < 0.03
    assert uniform_for(3, 5) == uniform_for(3, 5) != uniform_for(4, 5)


def test_cli_usage(capsys):
    from spyinfer_amd.__main__ import main
    assert main([]) == 1
    assert main(["-m", "x", "-b", "cuda"]) == 1
    assert "Available backends: hip" in capsys.readouterr().err


def test_steps_run_ahead_change_nothing(folder_a, emu_ops):
    """Before a step of decoded tokens has handed its tokens to the host, the engine launches the next one for the same
    requests; not when a request ends by count or waits for admission; and when a request ends at its end token or is
    removed, its row in the step in flight is ignored.  The tokens that come out are those of an engine that never
    runs ahead, request by request; no page is lost."""
    from spyinfer_amd.engine.llm_engine import LLMEngine
    ps = prompts(256, [9, 30, 4, 21, 12], seed=7)
    plain = PlainQwen3(folder_a)
    # an end token that the second request really produces, so that it ends early
    g1 = plain.greedy(ps[1], 12)
    k = max(i for i in range(12) if g1[i] not in g1[:i])       # the last place where a token appears for the first time
    assert k >= 1
    eos = g1[k]

    def run(ahead):
        eng = LLMEngine(folder_a, dtype="float32", device="cpu", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=8)
        eng.eos_token_id = eos
        used = [0]
        eng.run_ahead = ahead
        real = eng._launch_ahead
        def counted(flight):
            got = real(flight)
            used[0] += got is not None
            return got
        eng._launch_ahead = counted
        ids = [eng.add_request(ps[0], SamplingParams(max_new_tokens=25, ignore_eos=True)),
               eng.add_request(ps[1], SamplingParams(max_new_tokens=25)),                   # ends at its end token
               eng.add_request(ps[2], SamplingParams(max_new_tokens=7, ignore_eos=True))]   # ends by count
        log = []
        for step in range(60):
            if step == 10:
                ids.append(eng.add_request(ps[3], SamplingParams(max_new_tokens=9, ignore_eos=True)))   # arrives in between
            if step == 16:
                eng.remove_request(ids[0])                                                   # leaves in between
                ids[0] = None
            if step == 20:
                ids.append(eng.add_request(ps[4], SamplingParams(temperature=0.7, max_new_tokens=8, ignore_eos=True, seed=5)))
            log.append(sorted(tuple(o) for o in eng.step()))
        assert not eng.has_unfinished_requests()
        eng.runner.manager.check()
        assert eng.runner.manager.num_free_pages() == [40]
        return log, [eng.get_generated_tokens(i) for i in ids if i is not None], used[0]

    log_a, out_a, used = run(True)
    log_b, out_b, _ = run(False)
    # a request that arrives while a step is in flight joins one step later: the calls differ, the requests' tokens do not
    per_request = lambda log: {rid: [t for step in log for r, t, _ in step if r == rid] for rid in range(5)}
    assert per_request(log_a) == per_request(log_b) and out_a == out_b
    assert [f for step in log_a for _, _, f in step].count(True) == [f for step in log_b for _, _, f in step].count(True) == 4
    assert used >= 15, "steps of decoded tokens alone must have been launched ahead (%d were)" % used
    assert out_a[0] == g1[:k + 1]                              # the second request ended at its end token
    assert out_a[1] == plain.greedy(ps[2], 7) and out_a[2] == plain.greedy(ps[3], 9)


def test_config_b_workload_against_plain_model_and_plain_sampler(folder_b, emu_ops):
    """Prompts of 1 / 40 / 130 tokens in portions of 32 beside decoding requests, pages of 8: greedy tokens equal the
    plain implementation's, and tokens sampled at temperature 0.8 equal the plain sampler's on the plain logits (so the
    index of a draw, run-ahead steps included, and the seed of a request are the stated ones)."""
    from tests.workloads import run_config_b_workload
    run_config_b_workload(folder_b, PlainQwen3(folder_b), "cpu", "float32")


def test_refused_turn_leaves_the_request_as_it_was_and_draws_go_on(folder_a, emu_ops):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from tests.workloads import check_sampled_against_plain
    plain = PlainQwen3(folder_a)
    p = prompts(256, [12])[0]
    sp = SamplingParams(temperature=0.9, max_new_tokens=5, ignore_eos=True, seed=77)
    for keep in (False, True):
        eng = LLMEngine(folder_a, dtype="float32", device="cpu", max_model_len=40, num_kvcache_blocks=8, keep_finished_cache=keep)
        rid = eng.add_request(p, sp)
        while not eng.is_request_finished(rid):
            eng.step()
        first = eng.get_generated_tokens(rid)
        history = eng.get_output_tokens(rid)
        with pytest.raises(ValueError, match="max_model_len"):
            eng.append_to_request(rid, [1] * 30)                       # 12 + 5 + 30 > 40
        with pytest.raises(ValueError, match="vocabulary"):
            eng.append_to_request(rid, [3, 999])
        assert eng.is_request_finished(rid) and eng.get_output_tokens(rid) == history and eng.get_generated_tokens(rid) == first
        prefill_before = eng.stats["prefill_tokens"]
        eng.append_to_request(rid, [7, 8, 9])
        while not eng.is_request_finished(rid):
            eng.step()
        second = eng.get_generated_tokens(rid)
        # the second turn computes its new tokens only if the cache was kept, the whole history otherwise
        assert eng.stats["prefill_tokens"] - prefill_before == (4 if keep else len(history) + 3)
        # its draws go on where the first turn's ended (indices 5..9 of the same seed), checked with the plain sampler
        check_sampled_against_plain(plain, [p], [first], 0.9, [77], 1e-4)
        compared, _ = check_sampled_against_plain(plain, [history + [7, 8, 9]], [second], 0.9, [77], 1e-4, first_draw=5)
        assert compared >= 4
        eng.remove_request(rid)
        eng.runner.manager.check()
        assert eng.runner.manager.num_free_pages() == [8] and eng.runner.manager.slots.num_free == eng.config.max_num_seqs


def test_a_turn_without_new_tokens_after_an_end_token_met_while_a_step_ran_ahead(folder_a, emu_ops):
    """A request ends at its end token while the next step is already in flight: that step has stored the end token's
    key and value, so a kept cache covers every token of the request.  A further turn that brings no tokens (the
    reference's append_to_request takes an empty message, src/engine/llm_engine.cpp:40-73) still has to sample from the
    last token's logits: the cache steps back by one token.  Tokens equal those of an engine that keeps nothing, the
    other requests go on, and nothing is lost."""
    from spyinfer_amd.engine.llm_engine import LLMEngine
    plain = PlainQwen3(folder_a)
    ps = prompts(256, [14, 6], seed=11)
    g0 = plain.greedy(ps[0], 10)
    k = max(i for i in range(10) if g0[i] not in g0[:i])
    assert k >= 2                                       # met after steps of decoded tokens alone: one was in flight
    eos = g0[k]

    def run(keep, turn):
        eng = LLMEngine(folder_a, dtype="float32", device="cpu", max_model_len=96, num_kvcache_blocks=24, keep_finished_cache=keep)
        eng.eos_token_id = eos
        rid = eng.add_request(ps[0], SamplingParams(max_new_tokens=20))
        other = eng.add_request(ps[1], SamplingParams(max_new_tokens=40, ignore_eos=True))
        while not eng.is_request_finished(rid):
            eng.step()
        assert eng.finish_reason(rid) == "eos" and eng.get_generated_tokens(rid) == g0[:k + 1]
        seq = eng._sequences[rid]
        if keep:
            assert seq.cache is not None and seq.cache.num_tokens == len(seq)      # the step in flight stored the end token
        eng.append_to_request(rid, turn, SamplingParams(max_new_tokens=4, ignore_eos=True))
        steps = 0
        while eng.has_unfinished_requests():
            eng.step()
            steps += 1
            assert steps < 200, "the engine is wedged"
        out = eng.get_generated_tokens(rid), eng.get_generated_tokens(other)
        eng.remove_request(rid)
        eng.remove_request(other)
        eng.runner.manager.check()
        assert eng.runner.manager.num_free_pages() == [24]
        return out

    for turn in ([], [9]):
        kept, fresh = run(True, turn), run(False, turn)
        assert kept == fresh
        assert kept[0] == plain.greedy(ps[0] + g0[:k + 1] + turn, 4)
        assert kept[1] == plain.greedy(ps[1], 40)
