"""Random serving days through the entry point against the plain implementation: a tiny configuration, engine options
(page size, pool, most requests, token budget, portion size, graphs or not, kept caches, matrices in tiles only),
arrivals, endings (end token, count, removal) and further turns, all drawn from a seed; pools small enough for
preemption.  Every token is the plain implementation's wherever the plain logits' two largest are 1e-4 apart (float32)
or 0.3 (bfloat16), or the token agrees anyway; a request stops being compared at its first other token behind a
narrower margin.  (1800 further seeds in float32 and 2600 in bfloat16, run once: 168 000 tokens compared, 10 000
preemptions, 57 000 replayed graphs; one float32 day had another token, where two logits were 2e-6 apart.)"""
import random
from collections import Counter

import pytest
import torch

from tests.configs import INIT
from tests.gpu_util import require_gpu
from tests.plain.qwen3_plain import PlainQwen3

pytestmark = pytest.mark.gpu


def draw_model(rng):
    n_kv, group = rng.choice([1, 2, 3, 4, 8]), rng.choice([1, 2, 3, 4, 8])
    if rng.random() < 0.6:                  # widths that the tiled decode products take
        hidden, inter = rng.choice([128, 256, 384]), rng.choice([128, 256, 384, 640])
    else:
        hidden, inter = 8 * rng.randint(5, 40), 8 * rng.randint(6, 60)
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=rng.randint(1, 3),
                hidden_size=hidden, num_attention_heads=n_kv * group, num_key_value_heads=n_kv,
                head_dim=rng.choice([16, 32, 48, 64, 64, 128, 128, 80, 256]), intermediate_size=inter, vocab_size=rng.randint(90, 700),
                rope_theta=rng.choice([1e4, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5]), tie_word_embeddings=rng.random() < 0.5,
                max_position_embeddings=1024, bos_token_id=0, eos_token_id=1)


def plain_greedy(plain, tokens, n_new, wide):
    """[(token, whether the two largest logits are at least ``wide`` apart)] of a greedy continuation."""
    toks, out = list(tokens), []
    for _ in range(n_new):
        logits = plain.forward(toks)[-1]
        top = torch.topk(logits, 2).values
        out.append((int(torch.argmax(logits)), float(top[0] - top[1]) >= wide))
        toks.append(out[-1][0])
    return out


def compare(i, got, want, what):
    """Tokens compared: all of ``want``, or up to the first other token behind a narrow margin."""
    for k, (t, sure) in enumerate(want):
        assert k < len(got), "%s: request %d has %d tokens, %d wanted" % (what, i, len(got), len(want))
        if got[k] != t:
            assert not sure, "%s: request %d token %d is %d, plain says %d" % (what, i, k, got[k], t)
            return k
    assert len(got) == len(want), "%s: request %d has %d tokens, %d wanted" % (what, i, len(got), len(want))
    return len(want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_a_random_day(seed, dtype, tmp_path):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights import write_random_model
    require_gpu()
    rng = random.Random(9000 + seed)
    cfg = draw_model(rng)
    folder = write_random_model(str(tmp_path / "m"), cfg, 700 + seed, torch.bfloat16, **INIT)
    plain = PlainQwen3(folder)
    page, n_req = rng.choice([8, 16, 32]), rng.randint(4, 14)
    lengths = [rng.choice([rng.randint(1, 12), rng.randint(10, 90), rng.randint(60, 200)]) for _ in range(n_req)]
    news = [rng.randint(1, 14) for _ in range(n_req)]
    g = torch.Generator().manual_seed(seed)
    ps = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]
    wide = 1e-4 if dtype == "float32" else 0.3      # (float32: the logits' own tolerance; one day in 1400 had two logits 2e-6 apart)
    full = [plain_greedy(plain, p, n, wide) for p, n in zip(ps, news)]
    later = Counter(t for f in full for t, _ in f[1:])
    eos = later.most_common(1)[0][0] if later else 1
    use_eos = [rng.random() < 0.5 for _ in ps]
    longest = max(a + b for a, b in zip(lengths, news)) + 40
    pool = max(-(-longest // page) + 1, rng.randint(4, 40))
    opts = dict(dtype=dtype, max_model_len=min(1024, longest + 8), kvcache_block_size=page, num_kvcache_blocks=pool,
                max_num_seqs=rng.randint(1, 6), max_num_batched_tokens=rng.choice([16, 24, 48, 100, 4096]),
                prefill_chunk=rng.choice([2, 7, 32, 2048]), enforce_eager=rng.random() < 0.3,
                keep_finished_cache=rng.random() < 0.5, weight_copies=rng.choice(["both", "both", "tiled"]))
    print("seed %d: %s | %s | %d requests" % (seed, {k: cfg[k] for k in ("num_hidden_layers", "hidden_size", "num_attention_heads",
          "num_key_value_heads", "head_dim", "intermediate_size", "vocab_size")}, opts, n_req), flush=True)
    eng = LLMEngine(folder, **opts)
    eng.eos_token_id = eos
    arrival = sorted((rng.randint(0, 40), i) for i in range(n_req))
    removed_at = {i: rng.randint(2, 8) for i in rng.sample(range(n_req), 2)}        # steps after arrival
    second = {i: (torch.randint(0, cfg["vocab_size"], (rng.randint(0, 9),), generator=g).tolist(), rng.randint(1, 6))
              for i in rng.sample(range(n_req), 3) if i not in removed_at}          # a further turn: (new tokens, tokens to generate)

    def wanted(i):
        toks = [t for t, _ in full[i]]
        return full[i][:toks.index(eos) + 1] if use_eos[i] and eos in toks else full[i]

    ids, born, gone, turn2, step = {}, {}, {}, {}, 0
    while arrival or eng.has_unfinished_requests() or any(i in ids and i not in turn2 for i in second):
        while arrival and arrival[0][0] <= step:
            _, i = arrival.pop(0)
            ids[i] = eng.add_request(ps[i], SamplingParams(max_new_tokens=news[i], ignore_eos=not use_eos[i]))
            born[i] = step
        for i, after in removed_at.items():
            if i in ids and i not in gone and step == born[i] + after:
                gone[i] = eng.get_generated_tokens(ids[i])
                eng.remove_request(ids[i])
        for i, (more, n2) in second.items():
            if i in ids and i not in turn2 and eng.is_request_finished(ids[i]):
                first = eng.get_generated_tokens(ids[i])
                history = ps[i] + first + more
                if compare(i, first, wanted(i), "first turn") < len(wanted(i)) or len(history) + n2 + 2 >= opts["max_model_len"]:
                    turn2[i] = None                      # its tokens left the plain ones behind a narrow margin, or no room
                    continue
                turn2[i] = plain_greedy(plain, history, n2, wide)
                eng.append_to_request(ids[i], more, SamplingParams(max_new_tokens=n2, ignore_eos=True))
        eng.step()
        step += 1
        assert step < 4000
    for i in range(n_req):
        if i in gone:
            compare(i, gone[i], wanted(i)[:len(gone[i])], "removed early")
        elif turn2.get(i) is not None:
            compare(i, eng.get_generated_tokens(ids[i]), turn2[i], "second turn")
        elif i not in turn2:
            compare(i, eng.get_generated_tokens(ids[i]), wanted(i), "request")
    eng.runner.manager.check()
    for i in ids:
        if i not in gone:
            eng.remove_request(ids[i])
    assert eng.runner.manager.num_free_pages() == [pool]
