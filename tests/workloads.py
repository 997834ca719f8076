"""Workloads shared by the CPU (stand-in kernels) and GPU tests of the entry point, and their checks against the
plain implementation."""
import torch

from tests.plain import sampler_plain


def prompts(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


def check_sampled_against_plain(plain, prompt_list, generated, temperature, seeds, margin, first_draw=0):
    """Every generated token against the plain sampler fed with the plain implementation's logits of the same prefix
    (the engine's own tokens so far, so one differing token does not hide the rest).  A draw whose uniform number lies
    within ``margin`` of an edge of the chosen token's interval of the cumulative distribution may fall either way under
    rounding and is not compared.  Returns (compared, skipped)."""
    compared = skipped = 0
    for r, (prompt, gen, seed) in enumerate(zip(prompt_list, generated, seeds)):
        logits = plain.forward(list(prompt) + list(gen))
        for i, tok in enumerate(gen):
            want, m = sampler_plain.choose(logits[len(prompt) - 1 + i].double().numpy(), temperature,
                                           sampler_plain.uniform(seed, first_draw + i))
            if m > margin:
                assert tok == want, "request %d, draw %d: engine %d, plain sampler %d (margin %.3g)" % (r, first_draw + i, tok, want, m)
                compared += 1
            else:
                skipped += 1
    return compared, skipped


def run_config_b_workload(folder, plain, device, dtype, **engine_options):
    """The workload of the second tiny configuration: prompts of 1 / 40 / 130 tokens, 24 tokens each, portions of at
    most 32 tokens mixed into the decode steps of the others, pages of 8; greedy, then temperature 0.8 with a seed.
    In bfloat16 the logits' rounding (0.04) moves the cumulative distribution by more than the width of a token's
    interval at temperature 0.8 (384 tokens of similar weight), so there the draws are compared at temperature 0.1,
    where few tokens hold most of the weight."""
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    ps = prompts(384, [1, 40, 130], seed=2)
    kw = dict(dtype=dtype, device=device, max_model_len=256, kvcache_block_size=8, num_kvcache_blocks=80, seed=9, prefill_chunk=32,
              max_num_batched_tokens=48)
    kw.update(engine_options)
    mixed = [0]

    def generate(params):
        eng = LLMEngine(folder, **kw)
        ids = [eng.add_request(p, params) for p in ps]
        real = eng.scheduler.schedule

        def watched():
            out = real()
            assert sum(x.num_tokens for x in out) <= kw["max_num_batched_tokens"] and all(x.num_tokens <= 32 for x in out)
            if any(x.num_tokens > 1 for x in out) and any(x.num_tokens == 1 and x.samples and x.seq.num_generated > 0 for x in out):
                mixed[0] += 1
            return out
        eng.scheduler.schedule = watched
        while eng.has_unfinished_requests():
            eng.step()
        eng.runner.manager.check()
        return [eng.get_generated_tokens(i) for i in ids], eng

    greedy, _ = generate(SamplingParams(max_new_tokens=24, ignore_eos=True))
    assert mixed[0] >= 3, "portions of the long prompt must share steps with decoding requests"
    if dtype == "float32":
        assert greedy == [plain.greedy(p, 24) for p in ps]
    temperature, margin, enough = (0.8, 2e-5, 68) if dtype == "float32" else (0.1, 0.08, 30)
    sampled, eng = generate(SamplingParams(temperature=temperature, max_new_tokens=24, ignore_eos=True))
    assert all(len(g) == 24 for g in sampled) and sampled != greedy
    seeds = [eng.config.seed + i for i in range(len(ps))]
    compared, skipped = check_sampled_against_plain(plain, ps, sampled, temperature, seeds, margin)
    assert compared >= enough, (compared, skipped)
    return sampled
