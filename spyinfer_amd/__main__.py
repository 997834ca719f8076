"""Command line in the manner of the reference's ``main`` (main.cpp:10-125):

    python -m spyinfer_amd -m <model_path> [-b hip]

then a loop that reads a line, generates, and prints the answer as it is produced; ``/new``
starts a new conversation and ``/exit`` leaves.  A line holds token ids separated by blanks or
commas (the reference reads text and tokenises it; this engine works on token ids).  Further
options set the engine's configuration under the reference's names.
"""
from __future__ import annotations

import argparse
import sys

BACKENDS = ("hip",)


def parse_ids(line: str):
    return [int(x) for x in line.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="spyinfer_amd", usage="%(prog)s -m <model_path> [-b <backend_type>] [options]")
    ap.add_argument("-m", dest="model_path", help="model folder (config.json, model.safetensors)")
    ap.add_argument("-b", dest="backend_type", default="hip", help="backend; available: " + ", ".join(BACKENDS))
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--max-num-batched-tokens", type=int, default=16384)
    ap.add_argument("--prefill-chunk", type=int, default=2048, help="most tokens of one request in one step")
    ap.add_argument("--max-num-seqs", type=int, default=512)
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--kvcache-block-size", type=int, default=16)
    ap.add_argument("--num-kvcache-blocks", type=int, default=None)
    ap.add_argument("--weight-copies", default="both", choices=["both", "tiled"],
                    help="tiled: matrices are kept in tiles only (half the weights' memory, prompts a sixth slower)")
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--max-new-tokens", type=int, default=None)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--prompt-ids", action="append", default=[], help="generate for these token ids and leave (may repeat)")
    ap.add_argument("--prompt-file", metavar="FILE", help="generate for every line of token ids of this file and leave")
    ap.add_argument("--random-prompts", metavar="LENGTHS", help="generate for prompts of uniform-random token ids of these "
                    "lengths (e.g. 5,17,33), drawn with --seed, and leave")
    ap.add_argument("--random-model", metavar="CONFIG_JSON", help="write a random-weights model folder to -m from this "
                    "config.json and --seed, then leave")
    args = ap.parse_args(argv)
    if not args.model_path:
        ap.print_usage(sys.stderr)
        print("Use -h for help", file=sys.stderr)
        return 1
    if args.backend_type not in BACKENDS:
        print("Invalid backend type: %s\nAvailable backends: %s" % (args.backend_type, ", ".join(BACKENDS)), file=sys.stderr)
        return 1
    if args.random_model:
        import json

        from .weights import write_random_model
        with open(args.random_model) as f:
            write_random_model(args.model_path, json.load(f), args.seed)
        print("wrote", args.model_path)
        return 0

    from .engine.llm_engine import LLMEngine
    from .sampling import SamplingParams

    engine = LLMEngine(args.model_path, dtype=args.dtype, max_num_batched_tokens=args.max_num_batched_tokens,
                       prefill_chunk=args.prefill_chunk, max_num_seqs=args.max_num_seqs, max_model_len=args.max_model_len,
                       keep_finished_cache=False,
                       gpu_memory_utilization=args.gpu_memory_utilization, enforce_eager=args.enforce_eager,
                       kvcache_block_size=args.kvcache_block_size, num_kvcache_blocks=args.num_kvcache_blocks, seed=args.seed,
                       weight_copies=args.weight_copies)
    params = SamplingParams(temperature=args.temperature, max_new_tokens=args.max_new_tokens, ignore_eos=args.ignore_eos)

    def stream(rid):
        while not engine.is_request_finished(rid):
            for out in engine.step():
                if out.request_id == rid:
                    print(out.token, end=" ", flush=True)
        print()

    prompts = [parse_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [parse_ids(line) for line in f if line.strip()]
    if args.random_prompts:
        import torch
        g = torch.Generator().manual_seed(args.seed)
        vocab = engine.model.config.vocab_size
        prompts += [torch.randint(0, vocab, (n,), generator=g).tolist() for n in parse_ids(args.random_prompts)]
    if prompts:
        ids = [engine.add_request(p, params) for p in prompts]
        while engine.has_unfinished_requests():
            engine.step()
        for rid in ids:
            print(" ".join(str(t) for t in engine.get_generated_tokens(rid)))
        return 0

    engine.config.keep_finished_cache = True       # the conversation's further turns compute their new tokens only
    conversation = -1
    while True:
        print("\nUser: ", end="", flush=True)
        line = sys.stdin.readline()
        if not line or line.strip() == "/exit":
            if conversation != -1:
                engine.remove_request(conversation)
            break
        if line.strip() == "/new":
            if conversation != -1:
                engine.remove_request(conversation)
            conversation = -1
            print("Starting new conversation.")
            continue
        try:
            ids = parse_ids(line)
            if not ids:
                continue
            if conversation == -1:
                conversation = engine.add_request(ids, params)
            else:
                engine.append_to_request(conversation, ids)
        except ValueError as e:
            print("error: %s" % e)
            continue
        print("Assistant: ", end="", flush=True)
        stream(conversation)
    return 0


if __name__ == "__main__":
    sys.exit(main())
