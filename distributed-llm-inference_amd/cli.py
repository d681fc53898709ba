"""Command line: ``python -m dli_amd <command>``.

``generate`` runs prompts given as token ids (tokenisation is not the engine's business) and prints
the generated ids, one JSON list a line. ``random-weights`` writes a model folder from a
configuration and a seed. ``trace`` is the replay tool (same as ``bin/trace_run``).

Engine options carry the names and meanings of the reference's server
(src/dli/server/__main__.py:65-124): ``--model``, ``--dtype``, ``--num-blocks`` | ``--kv-cache-gb``,
``--block-size``, ``--no-prefix-caching``, ``--max-num-seqs``, ``--max-num-batched-tokens``.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Optional, Sequence


def _add_engine_options(p: argparse.ArgumentParser) -> None:
    p.add_argument("--model", required=True, help="model folder (config.json + *.safetensors)")
    p.add_argument("--device", default="cuda")
    p.add_argument("--dtype", default="auto", choices=["auto", "float32", "bfloat16"],
                   help="auto = bfloat16")
    kv = p.add_mutually_exclusive_group()
    kv.add_argument("--num-blocks", type=int, default=None)
    kv.add_argument("--kv-cache-gb", type=float, default=None,
                    help="cache pool size in GiB (with neither: as many pages as the live requests can fill, "
                         "within four fifths of the free device memory)")
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--no-prefix-caching", action="store_true",
                   help="no reuse of cached pages across requests")
    p.add_argument("--cuda-graphs", action=argparse.BooleanOptionalAction, default=None,
                   help="replay decode steps through HIP graphs (steps that fit no captured shape run eagerly); "
                        "with neither form: where the call decodes enough steps for recording them to pay")
    p.add_argument("--max-num-seqs", type=int, default=256,
                   help="most requests that are live at a time (the reference's server takes 64)")
    p.add_argument("--max-num-batched-tokens", type=int, default=4096,
                   help="tokens of a step, portions of prompts and decoded tokens together (the reference's "
                        "server takes 512; prompts run at twice the rate in steps of thousands of rows)")
    p.add_argument("--decode-weight-copy", action=argparse.BooleanOptionalAction, default=True,
                   help="keep a second copy of the bfloat16 matrices in the decode kernels' order "
                        "(faster decode steps, twice the weight memory)")
    p.add_argument("--decode-steps", type=int, default=8,
                   help="tokens of every request that one decoding step runs on the device before the host "
                        "looks (same tokens, fewer round trips; one without --cuda-graphs or in float32)")


def _read_prompts(args: argparse.Namespace) -> list[list[int]]:
    prompts: list[list[int]] = []
    for text in args.prompt_ids or []:
        prompts.append([int(t) for t in text.replace(",", " ").split()])
    if args.prompt_file:
        src = sys.stdin if args.prompt_file == "-" else open(args.prompt_file)
        for line in src:
            line = line.strip()
            if not line:
                continue
            prompts.append(json.loads(line) if line.startswith("[") else [int(t) for t in line.replace(",", " ").split()])
    if not prompts or any(not p for p in prompts):
        raise SystemExit("give at least one non-empty prompt with --prompt-ids or --prompt-file")
    return prompts


def cmd_generate(args: argparse.Namespace) -> int:
    from .engine.generate import generate
    from .sampling.params import SamplingParams

    params = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k,
                            top_p=args.top_p, seed=args.seed,
                            stop_token_ids=tuple(args.stop_token_ids or ()), ignore_eos=args.ignore_eos)
    out = generate(
        args.model, _read_prompts(args), params,
        dtype="bfloat16" if args.dtype == "auto" else args.dtype, num_blocks=args.num_blocks,
        kv_cache_gb=args.kv_cache_gb, block_size=args.block_size, max_num_seqs=args.max_num_seqs,
        max_num_batched_tokens=args.max_num_batched_tokens,
        enable_prefix_caching=not args.no_prefix_caching, eos_token_ids=tuple(args.eos_token_ids or ()),
        seed=args.engine_seed, cuda_graphs=args.cuda_graphs, device=args.device, decode_steps=args.decode_steps,
        decode_weight_copy=args.decode_weight_copy)
    for ids in out:
        print(json.dumps(ids))
    return 0


def cmd_random_weights(args: argparse.Namespace) -> int:
    from .weights.random_init import write_random_model

    config = json.loads(Path(args.config).read_text())
    out = write_random_model(args.out, config, seed=args.seed, std=args.std, norm_jitter=args.norm_jitter,
                             storage=args.storage, device=args.device)
    print(out)
    return 0


def main(argv: Optional[Sequence[str]] = None) -> int:
    top = argparse.ArgumentParser(prog="dli_amd", description=__doc__,
                                  formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = top.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate token ids for prompts given as token ids")
    _add_engine_options(g)
    g.add_argument("--prompt-ids", action="append", help="one prompt: token ids separated by spaces or commas")
    g.add_argument("--prompt-file", help="file with one prompt a line (ids or a JSON list); - for stdin")
    g.add_argument("--max-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=-1)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=None, help="seed of each request's random draws")
    g.add_argument("--engine-seed", type=int, default=0, help="seeds requests that have no --seed")
    g.add_argument("--stop-token-ids", type=int, nargs="*")
    g.add_argument("--eos-token-ids", type=int, nargs="*")
    g.add_argument("--ignore-eos", action="store_true")
    g.set_defaults(fn=cmd_generate)

    r = sub.add_parser("random-weights", help="write a model folder with random weights")
    r.add_argument("--config", required=True, help="a config.json")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--std", type=float, default=0.02)
    r.add_argument("--norm-jitter", type=float, default=0.0)
    r.add_argument("--storage", default="bfloat16", choices=["bfloat16", "float32"])
    r.add_argument("--device", default="cpu", help="where the values are drawn (cpu, or cuda for large models)")
    r.set_defaults(fn=cmd_random_weights)

    t = sub.add_parser("trace", help="replay a trace of token ids (see bin/trace_run)", add_help=False)
    t.set_defaults(fn=None)

    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] == "trace":
        from .trace import main as trace_main

        return trace_main(list(argv[1:]))
    args = top.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
