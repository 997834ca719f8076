"""Builds replay traces (whole, bulk + tail, changing portions, mixed) for given requests and
compares what a replay wrote with the plain implementation, position by position."""
import io
import json
import os
import random

import numpy as np
import torch


def whole(requests):
    """Every request alone, all its tokens in one step, logits everywhere."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def bulk_tail(requests, tail=32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        n = len(toks)
        cut = max(1, n - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:cut], "want": list(range(cut))}], "end": []})
        for i in range(cut, n):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == n - 1 else []})
        if cut == n:
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(7, 2, 13, 5, 3, 2, 29, 4, 2, 16, 11)):
    """Portions of changing size, down to two tokens, crossing page edges anywhere."""
    steps = []
    for rid, toks in requests.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            last = i + n == len(toks)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[i:i + n], "want": list(range(n))}],
                          "end": [rid] if last else []})
            i += n
    return steps


def mixed(requests, seed=0, max_live=4):
    """Up to ``max_live`` requests live at a time: portions of some beside single tokens of
    others, some left out of a step; a finished request makes room for the next."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0, rng.random() < 0.5]     # tokens, fed, decode-like after the first portion
        entries, end = [], []
        for rid in list(live):
            toks, fed, single = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step
            left = len(toks) - fed
            if fed == 0:
                n = min(left, rng.choice([2, 5, 9, 17, 31, 40]))
            elif single:
                n = 1
            else:
                n = min(left, rng.choice([1, 2, 3, 7, 12, 19]))
            want = list(range(n)) if n <= 4 else sorted(rng.sample(range(n), 3) + [n - 1])
            want = sorted(set(want))
            entries.append({"id": rid, "tokens": toks[fed:fed + n], "want": want})
            live[rid][1] = fed + n
            if fed + n == len(toks):
                end.append(rid)
        if not entries:
            continue
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def trace_properties(steps):
    """What a trace exercises: (steps that hold a portion of one request beside a single token of a request that has
    tokens in the cache already, requests admitted after another request ended, most requests live at once)."""
    fed, ended = {}, 0
    beside = late = most = 0
    for st in steps:
        portion = any(len(e["tokens"]) >= 2 for e in st["entries"])
        single = any(len(e["tokens"]) == 1 and fed.get(e["id"], 0) > 0 for e in st["entries"])
        beside += portion and single
        for e in st["entries"]:
            if e["id"] not in fed and e["tokens"]:
                late += ended > 0
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        most = max(most, len(fed))
        for rid in st["end"]:
            if fed.pop(rid, None) is not None:
                ended += 1
    return beside, late, most


def assert_mixed(steps, what=""):
    """A mixed trace must hold what it is for: at least 5 steps with a portion beside a decoded token, requests
    admitted after others ended (their pages are handed out again), at most four live."""
    beside, late, most = trace_properties(steps)
    assert beside >= 5 and late >= 1 and most <= 4, "%s: the mixed trace has %d steps with a portion beside a single token, " \
        "%d requests admitted after another ended, %d live at once" % (what, beside, late, most)


def max_live_tokens(steps, unit=64):
    """Most tokens held at any time, each live request rounded up to a multiple of ``unit``."""
    held, most = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // unit) * unit for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return most


def run_replay_inprocess(model_dir, dtype, out_dir, steps, max_tokens, extra=()):
    from spyinfer_amd.engine.replay import run
    stdin = io.StringIO("".join(json.dumps(s) + "\n" for s in steps))
    stdout = io.StringIO()
    rc = run(["--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)] + list(extra),
             stdin=stdin, stdout=stdout)
    assert rc == 0
    done = [l for l in stdout.getvalue().splitlines() if l.startswith("done ")]
    assert [d.split()[1] for d in done] == [str(s["step"]) for s in steps]


def collect(out_dir, steps, vocab):
    """{(request id, position): logits row} from the files of a replay."""
    fed, got = {}, {}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        path = os.path.join(out_dir, "%s.f32" % st["step"])
        if wanted == 0:
            assert not os.path.exists(path)
        else:
            data = np.fromfile(path, dtype="<f4").reshape(wanted, vocab)
            r = 0
            for e in st["entries"]:
                base = fed.get(e["id"], 0)
                for w in e["want"]:
                    got[(e["id"], base + w)] = data[r]
                    r += 1
        for e in st["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        for rid in st["end"]:
            fed.pop(rid, None)
    return got


def compare(got, plain_logits, atol, rtol, what=""):
    """``plain_logits``: {request id: [T, vocab] tensor}.  Reports the first wrong place."""
    assert got, "the replay wrote no logits"
    worst = 0.0
    for (rid, pos), row in sorted(got.items(), key=lambda kv: (str(kv[0][0]), kv[0][1])):
        ref = plain_logits[rid][pos].double().numpy()
        err = np.abs(row.astype(np.float64) - ref)
        lim = atol + rtol * np.abs(ref)
        if not np.all(np.isfinite(row)) or np.any(err > lim):
            j = int(np.argmax(err - lim))
            raise AssertionError("%s: request %r position %d differs from the plain implementation: logit %d is %r, expected %r "
                                 "(max abs err %.3g)" % (what, rid, pos, j, float(row[j]), float(ref[j]), float(err.max())))
        worst = max(worst, float(err.max()))
    return worst


def random_requests(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {"r%d" % i: torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
