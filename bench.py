#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

Default: the Qwen3-8B shape (36 layers, hidden 4096, 32 query and
8 key/value heads of 128, intermediate 12288, vocabulary 151936, untied head) with random
bfloat16 weights; 8 requests with 1024-token random prompts decode through the engine's own step
(scheduler, step function, cache, kernels, device sampling).  A "step" is one decode step.
The timed steps are centred on the workload's mean context: with 1024-token prompts and 256 generated tokens
(``--gen-len``) that is 1152 tokens, so untimed steps run up to context 1152 - steps / 2 first, whatever ``--steps`` is.
Prints ONE JSON line: decoded tokens per second, plus the prefill of 2048 tokens, the decode
step's HBM roofline, and decode at batch 1, 32 and 64 and at batch 32 with prompts of uneven lengths (128 to 2048
tokens, ``--uneven``) (tokens per second under "points"; their time per step,
mean context and share of the HBM roofline under "points_detail").  Beside the fractions of the published peaks
(8 TB/s, 2.5 PFLOP/s) the line gives fractions of rates measured at start-up on this GPU: a plain read of 2 GB
("measured_read_gbs", "frac_of_measured") and the library's product of 2048 rows with the model's gate/up matrix
("library_tflops", "frac_of_library").

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--dtype bfloat16|float32]

Other workloads, each again one JSON line:

    python bench.py --shape 14b --serve 64                 # Qwen3-14B shape: 64 requests at once until all have ended
    python bench.py --shape 32b --batch 64 --prompt-len 4096 --context 4608 --points "" --steps 32 --warmup 4   # long keys at the 32B shape
"""
import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

MODEL_8B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", num_hidden_layers=36, hidden_size=4096,
                num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960,
                bos_token_id=151643, eos_token_id=151645)
# the larger shapes; the default stays the 8B shape
SHAPES = {
    # the size of model that the reference's own run script names (run.sh:2): 28 narrow layers, where a step is many short kernels
    "0.6b": ("Qwen3-0.6B shape", dict(MODEL_8B, num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, intermediate_size=3072,
                                      tie_word_embeddings=True)),
    "1.7b": ("Qwen3-1.7B shape", dict(MODEL_8B, num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, intermediate_size=6144,
                                      tie_word_embeddings=True)),
    "4b": ("Qwen3-4B shape", dict(MODEL_8B, num_hidden_layers=36, hidden_size=2560, num_attention_heads=32, intermediate_size=9728,
                                  tie_word_embeddings=True)),
    "8b": ("Qwen3-8B shape", MODEL_8B),
    "14b": ("Qwen3-14B shape", dict(MODEL_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)),
    "32b": ("Qwen3-32B shape", dict(MODEL_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)),
}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--gen-len", type=int, default=256,
                    help="tokens that the workload generates per request: the timed steps are centred on its mean context")
    ap.add_argument("--context", type=int, default=4096, help="max_model_len")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,32,64", help="further decode batch sizes to report (empty: none)")
    ap.add_argument("--uneven", default="32", help="decode batch sizes to report with prompts of uneven lengths, uniform in "
                                                   "128 .. 2 x prompt-len (empty: none)")
    ap.add_argument("--spread", action="store_true", help="the headline batch's prompts too have uneven lengths (128 .. 2 x prompt-len)")
    ap.add_argument("--even-key-parts", action="store_true",
                    help="every request's keys in one number of parts instead of the host's cut by the step's lengths (for comparison)")
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--weight-copies", default="both", choices=["both", "tiled"], help="EngineConfig.weight_copies")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes of the model")
    ap.add_argument("--serve", type=int, default=0, metavar="N",
                    help="instead of the decode steps: N requests arriving at once, prompts of 128..2048 and outputs of 64..512 "
                         "tokens (uniform), run until all have ended; the value is generated tokens per second of the whole run")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    import torch

    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.engine.runner import bind_weights
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.sampling import SamplingParams
    from spyinfer_amd.weights.random_init import random_tensors_on_device

    ops.hip()
    if args.even_key_parts:
        ops.DECODE_PIECES = False
    dev = torch.device("cuda:0")
    shape_name, shape = SHAPES[args.shape]
    raw = dict(shape)
    model_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    arch = architecture_of(raw)
    cfg = arch.config_cls.from_dict(raw)
    model = arch.build(cfg)
    run_dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    weights = random_tensors_on_device(model.weight_specs(), args.seed, run_dtype, dev)
    bind_weights(model, weights, dev, args.weight_copies)
    del weights
    torch.cuda.empty_cache()

    points = [int(x) for x in args.points.split(",") if x.strip()]
    uneven = [int(x) for x in args.uneven.split(",") if x.strip()]
    max_batch = max([args.batch, args.serve] + points + uneven)
    page = 16
    pages_per_req = -(-args.context // page)
    eng = LLMEngine.__new__(LLMEngine)
    eng._init_with_model(model, dev, dtype=args.dtype, max_model_len=args.context, kvcache_block_size=page,
                         num_kvcache_blocks=max(pages_per_req * max_batch, -(-args.prefill_tokens // page)) + 8, max_num_seqs=max_batch,
                         max_num_batched_tokens=max(16384, args.prefill_tokens), enforce_eager=args.enforce_eager, seed=args.seed,
                         weight_copies=args.weight_copies)
    g = torch.Generator().manual_seed(args.seed)

    def prompts(n, length):
        return [torch.randint(0, cfg.vocab_size, (length,), generator=g).tolist() for _ in range(n)]

    act_bytes = 2 if args.dtype == "bfloat16" else 4
    L, H, I, V = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    nq, nkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    layer_params = H * (nq + 2 * nkv) * d + nq * d * H + 3 * H * I + 2 * H + 2 * d
    weight_bytes = (L * layer_params + H + V * H) * act_bytes              # every weight a decode step uses, once
    kv_bytes_per_token = sum(s.page_bytes(1, run_dtype) for s in model.cache_specs() if s is not None and s.paged)

    def decode_run(batch, steps, warmup, lengths=None):
        """tokens/s, ms/step, mean context over the timed steps.  Untimed steps first, ``warmup`` at least, until the
        timed window is centred on the workload's mean context (prompt + gen_len / 2).  ``lengths``: the prompts'
        lengths, if not all ``--prompt-len``."""
        lengths = [args.prompt_len] * batch if lengths is None else lengths
        untimed = max(warmup, min((args.gen_len - steps) // 2, args.context - max(lengths) - steps - 2))
        ids = [eng.add_request(prompts(1, n)[0], SamplingParams(temperature=0.0, max_new_tokens=untimed + steps + 64, ignore_eos=True))
               for n in lengths]
        while any(s.is_prefill or s.num_generated == 0 for s in (eng._sequences[i] for i in ids)):
            eng.step()                                                       # prompts, in portions under the budget
        for _ in range(untimed):
            eng.step()
        ctx0 = sum(len(eng._sequences[i]) for i in ids) / batch
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = eng.step()
            assert len(out) == batch
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        ctx1 = sum(len(eng._sequences[i]) for i in ids) / batch
        for i in ids:
            eng.remove_request(i)
        return batch * steps / dt, dt / steps * 1e3, (ctx0 + ctx1) / 2

    def prefill_run(tokens, repeats=3):
        best = None
        for _ in range(repeats + 1):
            rc = eng.runner.manager.admit("prefill")
            eng.runner.manager.reserve(rc, tokens)
            toks = prompts(1, tokens)[0]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = eng.runner.step([StepEntry(rc, toks, [tokens - 1])])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            eng.runner.manager.release(rc)
            assert logits.shape == (1, V)
            best = dt if best is None else min(best, dt)       # the first run also warms the library up
        return best

    def serve_run(n):
        """n requests at once through the scheduler until all have ended: (generated tokens/s, seconds, steps, mean number
        of requests in a step, preemptions, prompt tokens, generated tokens)."""
        lens = torch.randint(128, 2049, (n,), generator=g).tolist()
        outs = torch.randint(64, 513, (n,), generator=g).tolist()
        for length, new in zip(lens, outs):
            eng.add_request(prompts(1, length)[0], SamplingParams(temperature=0.0, max_new_tokens=new, ignore_eos=True))
        steps = rows = 0
        before = eng.scheduler.num_preemptions
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.has_unfinished_requests():
            rows += len(eng.step())
            steps += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        return sum(outs) / dt, dt, steps, rows / max(1, steps), eng.scheduler.num_preemptions - before, sum(lens), sum(outs)

    if args.serve:
        serve_run(min(args.serve, 4))                                        # warms the library and the graphs up
        v, dt, steps, mean_rows, pre, n_prompt, n_out = serve_run(args.serve)
        print(json.dumps({
            "metric": "generated tok/s, %d requests at once (%s, prompts 128..2048, outputs 64..512)" % (args.serve, shape_name),
            "value": round(v, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 0, "ms_per_step": round(dt / steps * 1e3, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights, uniform-random token ids and lengths)",
            "config": {"model": shape_name, "layers": cfg.num_hidden_layers, "layers_of_model": model_layers, "hidden": cfg.hidden_size,
                       "q_heads": nq, "kv_heads": nkv, "head_dim": d, "intermediate": I, "vocab": V, "global_batch": args.serve,
                       "seq_len": args.context, "prompt_tokens": n_prompt, "generated_tokens": n_out, "seconds": round(dt, 3),
                       "mean_rows_per_step": round(mean_rows, 2), "preemptions": pre, "page_size": page, "parallelism": "single GPU"}}))
        return 0

    # what this GPU gives a kernel that only reads, and the library a product of the prefill's shape: the rates that the
    # decode step and the prefill are held against beside the published peaks
    read_gbs = ops.measure_read_rate(dev) / 1e9
    lib_flops = None
    if args.dtype == "bfloat16":
        a = torch.randn((args.prefill_tokens, H), dtype=torch.bfloat16, device=dev)
        b = torch.randn((2 * I, H), dtype=torch.bfloat16, device=dev)
        best = None
        for _ in range(6):
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
            torch.matmul(a, b.t())
            t1.record()
            t1.synchronize()
            best = t0.elapsed_time(t1) if best is None else min(best, t0.elapsed_time(t1))
        lib_flops = 2.0 * args.prefill_tokens * 2 * I * H / (best * 1e-3)
        del a, b
    spread = lambda b: torch.randint(128, min(2 * args.prompt_len, args.context - args.gen_len) + 1, (b,), generator=g).tolist()
    value, ms, ctx = decode_run(args.batch, args.steps, args.warmup, spread(args.batch) if args.spread else None)
    step_bytes = weight_bytes + args.batch * ctx * kv_bytes_per_token
    achieved = step_bytes / (ms * 1e-3) / 1e9
    pf = prefill_run(args.prefill_tokens)
    T = args.prefill_tokens
    linear_flops = 2 * T * L * (H * (nq + 2 * nkv) * d + nq * d * H + 3 * H * I) + 2 * V * H
    attn_flops = L * 4 * d * nq * T * (T + 1) / 2
    pf_flops = linear_flops + attn_flops
    extra, detail = {}, {}
    for b in points:
        v, b_ms, b_ctx = decode_run(b, max(20, args.steps // 2), max(4, args.warmup // 2))
        extra["decode_b%d" % b] = round(v, 1)
        b_gbs = (weight_bytes + b * b_ctx * kv_bytes_per_token) / (b_ms * 1e-3) / 1e9
        detail["decode_b%d" % b] = {"ms_per_step": round(b_ms, 4), "mean_context": round(b_ctx, 1), "hbm_gbs": round(b_gbs, 1),
                                    "hbm_frac": round(b_gbs / PEAK_HBM_GBS, 4), "frac_of_measured": round(b_gbs / read_gbs, 4)}
    for b in uneven:
        lengths = spread(b)
        v, b_ms, b_ctx = decode_run(b, max(20, args.steps // 2), max(4, args.warmup // 2), lengths)
        extra["decode_b%d_uneven" % b] = round(v, 1)
        b_gbs = (weight_bytes + b * b_ctx * kv_bytes_per_token) / (b_ms * 1e-3) / 1e9
        detail["decode_b%d_uneven" % b] = {"ms_per_step": round(b_ms, 4), "mean_context": round(b_ctx, 1), "longest_prompt": max(lengths),
                                           "shortest_prompt": min(lengths), "hbm_gbs": round(b_gbs, 1),
                                           "hbm_frac": round(b_gbs / PEAK_HBM_GBS, 4), "frac_of_measured": round(b_gbs / read_gbs, 4)}
    line = {
        "metric": "decode tok/s at batch %d (%s, %d-token prompts)" % (args.batch, shape_name, args.prompt_len),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights, uniform-random token ids)",
        "config": {"model": shape_name, "layers": L, "layers_of_model": model_layers, "hidden": H, "q_heads": nq,
                   "kv_heads": nkv, "head_dim": d, "intermediate": I, "vocab": V, "global_batch": args.batch,
                   "seq_len": args.context, "prompt_len": args.prompt_len, "mean_context": round(ctx, 1), "page_size": page,
                   "graphs": not args.enforce_eager, "run_ahead": bool(eng.run_ahead), "parallelism": "single GPU",
                   "uneven_prompts": bool(args.spread), "keys_cut_by_host": bool(ops.DECODE_PIECES)},
        "prefill": {"value": round(T / pf, 1), "tokens": T, "ms": round(pf * 1e3, 3),
                    "frac": round(pf_flops / pf / PEAK_FLOPS[args.dtype], 4),
                    "library_tflops": None if lib_flops is None else round(lib_flops / 1e12, 1),
                    "frac_of_library": None if lib_flops is None else round(pf_flops / pf / lib_flops, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "measured_read_gbs": round(read_gbs, 1),
                     "frac_of_measured": round(achieved / read_gbs, 4)},
        "points": extra,
        "points_detail": detail,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
