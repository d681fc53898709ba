"""Measures decode and prefill throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The default run is the Llama-3.2-1B shape with random weights in bfloat16: 8 requests decode
greedily at a context of about 4096 tokens through the engine's own step loop (schedule, one
batched step, sampling), W untimed steps and then exactly K timed ones between device
synchronisations. One JSON line reports decoded tokens a second, the time of a 2,048-token prefill
step, the decode step's memory roofline, and under ``points`` decode throughput at batch 1 and 64,
at the baseline's own context (2,048 growing to 2,304) and at 32,768 keys, a prompt of 16,384
tokens in portions of 2,048 and of 512, and the other
workloads that the baseline names: the Llama-3.2-3B sizes (decode at batch 8, a 2,048-token
prefill, 64 requests batched continuously under 2,048 tokens a step) and the SmolLM2-1.7B sizes
(decode at batch 8, 32 requests that share a prefix of 1,024 tokens). ``--no-other-shapes`` leaves
the other models out, ``--no-points`` everything but the headline.
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

# MI355X published peaks
HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

SLACK = 96  # decode steps that early requests may run before the timed ones (at least)


def slack_for(batch, context, budget):
    """Decode steps that the requests admitted first may run while the others' prompts are still
    computed ``budget`` tokens a step."""
    return max(SLACK, -(-batch * context // budget) + 8)

LLAMA_3_2_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 128256, "hidden_size": 2048,
    "intermediate_size": 8192, "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 64, "rms_norm_eps": 1e-5, "max_position_embeddings": 131072, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "tie_word_embeddings": True, "hidden_act": "silu",
}

# the other shapes that the baseline's configurations name, for measurements beside the default one
LLAMA_3_2_3B = dict(LLAMA_3_2_1B, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24, head_dim=128)
SMOLLM2_1_7B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 49152, "hidden_size": 2048,
    "intermediate_size": 8192, "num_hidden_layers": 24, "num_attention_heads": 32, "num_key_value_heads": 32,
    "head_dim": 64, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192, "rope_theta": 130000.0,
    "tie_word_embeddings": True, "hidden_act": "silu",
}
# the small members of the family (widths that are no multiple of 128), for --shape
SMOLLM2_135M = dict(SMOLLM2_1_7B, hidden_size=576, intermediate_size=1536, num_hidden_layers=30,
                    num_attention_heads=9, num_key_value_heads=3, rope_theta=100000.0)
SMOLLM2_360M = dict(SMOLLM2_1_7B, hidden_size=960, intermediate_size=2560, num_hidden_layers=32,
                    num_attention_heads=15, num_key_value_heads=5, rope_theta=100000.0)
SHAPES = {"Llama-3.2-1B": LLAMA_3_2_1B, "Llama-3.2-3B": LLAMA_3_2_3B, "SmolLM2-1.7B": SMOLLM2_1_7B,
          "SmolLM2-360M": SMOLLM2_360M, "SmolLM2-135M": SMOLLM2_135M}


def load_random_model(raw, dtype):
    """A model of the sizes ``raw`` with random weights, by the road that generation takes: a
    folder with config.json and model.safetensors (drawn on the GPU, a few seconds for a billion
    weights), read by the loader."""
    import tempfile

    from dli_amd.weights import load_model, write_random_model

    with tempfile.TemporaryDirectory(prefix="dli_amd_bench_") as folder:
        write_random_model(folder, raw, seed=0, std=0.02, device="cuda:0")
        return load_model(folder, dtype=dtype, device="cuda:0")


def engine_for(model, batch, context, block_size, budget, decode_steps=1, num_pages=None, prefix_caching=False):
    from dli_amd.engine import LLMEngine, SchedulerConfig

    pages = num_pages or batch * (-(-(context + slack_for(batch, context, budget)) // block_size) + 1) + 8
    pages += pages // 64  # room for the share of the pool that admission keeps back (1%)
    engine = LLMEngine.for_model(
        model, num_blocks=pages, block_size=block_size, enable_prefix_caching=prefix_caching,
        config=SchedulerConfig(max_num_seqs=max(batch, 1), max_num_batched_tokens=budget,
                               decode_steps=decode_steps))
    return engine, model.config


def make_engine(raw, dtype, batch, context, block_size, budget, decode_steps=1, num_pages=None,
                prefix_caching=False):
    return engine_for(load_random_model(raw, dtype), batch, context, block_size, budget, decode_steps, num_pages,
                      prefix_caching)


def decode_run(engine, cfg, batch, context, steps, warmup, decode_steps=1):
    """Tokens a second and milliseconds a step of ``steps`` decode steps at about ``context``."""
    import torch

    from dli_amd.sampling import SamplingParams

    gen = torch.Generator().manual_seed(batch)
    # Requests admitted first decode a token a step while the others still prefill; the prompts are
    # shortened by that many steps so that no request outgrows `context` while the clock runs.
    budget = engine.scheduler.config.max_num_batched_tokens
    slack = slack_for(batch, context, budget)
    # (the engine has brought this down to what its runner can do: the 32-bit path decodes one token a step)
    decode_steps = min(decode_steps, engine.scheduler.config.decode_steps)
    # An engine step may decode several tokens of every request (SchedulerConfig.decode_steps): the
    # clock runs over exactly `steps` decode steps of the model, cut into engine steps of 8, 4, 2 or 1
    # (the largest first), and the warm-up runs every such size once so that its graph exists (a
    # shape is recorded at once where no recorded shape of up to four times its rows can stand in:
    # measure batches that lie further apart on one engine).
    def chunks_of(n):
        out = []
        while n > 0:
            out.append(max(d for d in (8, 4, 2, 1) if d <= min(n, max(1, decode_steps))))
            n -= out[-1]
        return out

    timed = chunks_of(steps)
    warm_chunks = sorted(set(timed), reverse=True)
    while sum(warm_chunks) < warmup:
        warm_chunks.append(timed[0])
    warm, per = sum(warm_chunks), timed[0]
    prompt_len = context - steps - warm - per - 1   # an engine step reserves up to `per` slots ahead
    prompt_len -= -(-batch * prompt_len // budget) + 1
    ids = []
    for i in range(batch):
        prompt = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=gen).tolist()
        ids.append(f"b{batch}-{i}")
        # requests that were admitted first decode a few tokens while the others still prefill
        engine.add_request(ids[-1], prompt, SamplingParams(max_tokens=steps + warm + per + 1 + slack, ignore_eos=True))
    guard = 0
    while engine.scheduler.waiting or any(r.num_computed_tokens < prompt_len for r in engine.scheduler.running):
        engine.step()  # prefill, in portions under the token budget
        guard += 1
        assert guard < slack, "prefill took more steps than the pool has slack for"
    import dataclasses

    def advance(chunks):
        done = 0
        for n in chunks:
            engine.scheduler.config = dataclasses.replace(engine.scheduler.config, decode_steps=n)
            out = engine.step()
            assert len(out) == batch and all(len(o.new_token_ids) == n for o in out)
            done += n
        return done

    advance(warm_chunks)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    done = advance(timed)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert done == steps and len(engine.scheduler.running) == batch
    for rid in ids:
        engine.abort(rid)
    return batch * steps / dt, dt / steps * 1e3, per


def prefill_run(engine, cfg, tokens, repeats=3, portion=None):
    """Seconds for one prompt of ``tokens`` tokens (the best of ``repeats``, after one untimed run):
    in one step, or with ``portion`` in steps of at most that many tokens, each on top of the keys
    that the earlier ones left in the cache."""
    import dataclasses

    import torch

    from dli_amd.sampling import SamplingParams

    config = engine.scheduler.config
    assert (portion or tokens) <= config.max_num_batched_tokens, "the engine's buffers are made for its own budget"
    if portion:
        engine.scheduler.config = dataclasses.replace(config, max_num_batched_tokens=portion)
    gen = torch.Generator().manual_seed(99)
    best = float("inf")
    for r in range(repeats + 1):
        prompt = torch.randint(0, cfg.vocab_size, (tokens,), generator=gen).tolist()
        engine.add_request(f"p{r}", prompt, SamplingParams(max_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = 0
        while engine.has_unfinished():
            engine.step()
            steps += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert steps == -(-tokens // (portion or tokens))
        if r > 0:
            best = min(best, dt)
    engine.scheduler.config = config
    return best


def serving_run(raw, dtype, workload, budget, decode_steps, rounds=2, model=None):
    """Requests batched continuously under a budget of ``budget`` tokens a step. ``mixed``: 64 requests
    with prompts of 128 to 2,048 random tokens and 256 generated tokens each (the workload that the
    baseline names for the 3B sizes). ``shared-prefix``: 32 requests that share a prefix of 1,024 tokens
    and go on with 64 to 512 tokens of their own, 128 generated tokens each, with reuse of cached pages
    on (the one it names for SmolLM2-1.7B). The first round also captures the decode graphs (and, for
    the shared prefix, fills the cache with it); the last one is reported."""
    import random

    import torch

    from dli_amd.sampling import SamplingParams

    shared = workload == "shared-prefix"
    requests, longest, out_tokens = (32, 1024 + 512, 128) if shared else (64, 2048, 256)
    pages = requests * (-(-(longest + out_tokens) // 16) + 1) + 8
    engine, cfg = engine_for(model if model is not None else load_random_model(raw, dtype), requests,
                             longest + out_tokens - SLACK, 16, budget, decode_steps, num_pages=pages,
                             prefix_caching=shared)
    rng = random.Random(0)
    prefix = [rng.randrange(cfg.vocab_size) for _ in range(1024)] if shared else []
    result = {}
    for rnd in range(rounds):
        lens = [rng.randint(64, 512) if shared else rng.randint(128, 2048) for _ in range(requests)]
        before = engine.manager.stats()
        for i, n in enumerate(lens):
            engine.add_request(f"s{rnd}-{i}", prefix + [rng.randrange(cfg.vocab_size) for _ in range(n)],
                               SamplingParams(max_tokens=out_tokens, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        steps = generated = 0
        while engine.has_unfinished():
            generated += sum(len(o.new_token_ids) for o in engine.step())
            steps += 1
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        after = engine.manager.stats()
        prompt_tokens = sum(lens) + len(prefix) * requests
        result = {"requests": requests, "prompt_tokens": prompt_tokens, "generated_tokens": generated,
                  "prompt_tokens_from_cache": after.prompt_tokens_hit - before.prompt_tokens_hit,
                  "seconds": round(dt, 4), "engine_steps": steps, "generated_tok_s": round(generated / dt, 1),
                  "total_tok_s": round((prompt_tokens + generated) / dt, 1)}
    return result, cfg


def other_shapes(args, short, itemsize):
    """The baseline's other workloads, each on a model of its own sizes: flat entries for ``points``."""
    import gc

    import torch

    out = {}
    k = min(args.decode_steps, 8)
    steps, warm = min(args.steps, 32), min(args.warmup, 4)
    for key, shape in (("llama3b", "Llama-3.2-3B"), ("smollm2_1_7b", "SmolLM2-1.7B")):
        model = load_random_model(dict(SHAPES[shape]), args.dtype)
        engine, cfg = engine_for(model, 8, args.context, args.block_size, 8192, k)
        tok_s, ms, _ = decode_run(engine, cfg, 8, args.context, steps, warm, k)
        out[f"{key}_decode_b8"] = round(tok_s, 1)
        out[f"{key}_decode_b8_ms"] = round(ms, 4)
        out[f"{key}_decode_b8_frac"] = round(decode_bytes(cfg, 8, args.context, itemsize) / (ms * 1e-3) / 1e9 / HBM_GBPS, 4)
        if key == "llama3b":
            t = prefill_run(engine, cfg, 2048)
            out[f"{key}_prefill2048"] = round(2048 / t, 1)
            out[f"{key}_prefill2048_ms"] = round(t * 1e3, 3)
            out[f"{key}_prefill2048_frac"] = round(prefill_flops(cfg, 2048) / t / PEAK_FLOPS[short], 4)
        del engine
        gc.collect()
        workload, budget = ("mixed", 2048) if key == "llama3b" else ("shared-prefix", 4096)
        got, _ = serving_run(None, args.dtype, workload, budget, k, model=model)
        tag = f"{key}_serving_{workload.replace('-', '_')}_budget{budget}"
        out[f"{tag}_generated_tok_s"] = got["generated_tok_s"]
        out[f"{tag}_total_tok_s"] = got["total_tok_s"]
        out[f"{tag}_seconds"] = got["seconds"]
        out[f"{tag}_requests"] = got["requests"]
        if workload == "shared-prefix":
            out[f"{tag}_prompt_tokens"] = got["prompt_tokens"]
            out[f"{tag}_prompt_tokens_from_cache"] = got["prompt_tokens_from_cache"]
        del model
        gc.collect()
        torch.cuda.empty_cache()
    return out


def prefill_flops(cfg, tokens):
    h, d = cfg.hidden_size, cfg.head_dim
    q, kv = cfg.num_heads * d, cfg.num_kv_heads * d
    linear = cfg.num_layers * (h * (q + 2 * kv) + q * h + 3 * h * cfg.intermediate_size)
    attention = cfg.num_layers * 2 * cfg.num_heads * d * tokens * (tokens + 1)  # QK^T and PV, causal
    return 2.0 * linear * tokens + attention + 2.0 * cfg.vocab_size * h  # + the head for one row


def decode_bytes(cfg, batch, context, itemsize):
    weights = (cfg.num_parameters()) * itemsize
    kv_per_token = 2 * cfg.num_layers * cfg.num_kv_heads * cfg.head_dim * itemsize
    return weights + batch * context * kv_per_token


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--shape", default="Llama-3.2-1B", choices=sorted(SHAPES),
                    help="layer sizes (the default is the configuration that the headline number is quoted on)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has")
    ap.add_argument("--size", action="append", default=[], metavar="KEY=INT",
                    help="another value for a size of the shape's config.json, e.g. --size head_dim=80 "
                         "--size hidden_size=2560 (measurements at other sizes; the line's model name says so)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--decode-steps", type=int, default=8,
                    help="decode steps that one engine step runs on the device before the host looks "
                         "(the timed steps are cut into engine steps of at most this many)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill runs")
    ap.add_argument("--no-other-shapes", action="store_true",
                    help="skip the points on the Llama-3.2-3B and SmolLM2-1.7B sizes (each loads a model of its own)")
    ap.add_argument("--serving", nargs="?", const="mixed", default=None, choices=["mixed", "shared-prefix"],
                    help="instead of the decode steps, requests batched continuously under --budget tokens a "
                         "step. mixed: 64 requests, prompts of 128 to 2,048 tokens, 256 generated tokens each; "
                         "shared-prefix: 32 requests that share 1,024 tokens and add 64 to 512 of their own, "
                         "128 generated tokens each, with reuse of cached pages")
    ap.add_argument("--budget", type=int, default=4096, help="tokens a step for --serving")
    ap.add_argument("--only-prefill", action="store_true",
                    help="run only prefill steps of --prefill-tokens tokens (for profiling) and print their time")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="prompt length of --only-prefill (the line of the default run always has 2,048)")
    ap.add_argument("--portion", type=int, default=None,
                    help="with --only-prefill: the prompt runs in steps of at most this many tokens")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on one GPU)")
        return 2

    import torch

    raw = dict(SHAPES[args.shape])
    for item in args.size:
        key, _, value = item.partition("=")
        if key not in raw or not isinstance(raw[key], int) or isinstance(raw[key], bool):
            ap.error(f"--size {item}: {key!r} is no integer size of the shape's configuration")
        raw[key] = int(value)
    if args.size:
        args.shape += " with " + ", ".join(args.size)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    itemsize = 2 if short == "bf16" else 4
    if args.serving:
        got, cfg = serving_run(raw, args.dtype, args.serving, args.budget, min(args.decode_steps, 8))
        print(json.dumps({
            "metric": f"continuous batching ({args.serving}), {args.shape} shape: generated tok/s",
            "value": got["generated_tok_s"],
            "unit": "tok/s", "n_gpus": 1, "higher_is_better": True, "dtype": short,
            "data": "synthetic: random token ids, random-init weights N(0, 0.02)",
            "config": {"model": f"{args.shape} shape", "layers": cfg.num_layers, "budget_tokens_per_step": args.budget,
                       "workload": args.serving, "kv_block_size": 16,
                       "decode_steps_per_engine_step": min(args.decode_steps, 8)}, **got}))
        return 0
    max_batch = 1 if args.only_prefill else max(args.batch, 1 if args.no_points else 64)
    context = max(args.context, args.prefill_tokens + 64) if args.only_prefill else args.context
    engine, cfg = make_engine(raw, args.dtype, max_batch, context, args.block_size,
                              budget=max(8192, args.prefill_tokens if args.only_prefill else 0),
                              decode_steps=args.decode_steps)

    if args.only_prefill:
        n = args.prefill_tokens
        t = prefill_run(engine, cfg, n, repeats=args.steps, portion=args.portion)
        print(json.dumps({"prefill_ms": round(t * 1e3, 3), "tokens": n, "portion": args.portion or n,
                          "tok_s": round(n / t, 1),
                          "frac": round(prefill_flops(cfg, n) / t / PEAK_FLOPS[short], 4),
                          "attention_gflop_per_layer": round(2 * cfg.num_heads * cfg.head_dim * n * (n + 1) / 1e9, 2)}))
        return 0
    tok_s, ms, per_engine_step = decode_run(engine, cfg, args.batch, args.context, args.steps, args.warmup,
                                            args.decode_steps)
    achieved = decode_bytes(cfg, args.batch, args.context, itemsize) / (ms * 1e-3) / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {args.shape} shape",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: random token ids, random-init weights N(0, 0.02)",
        "config": {
            "model": f"{args.shape} shape", "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single GPU", "layers": cfg.num_layers, "layers_of_config": full_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_heads, "kv_heads": cfg.num_kv_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "rms_norm_eps": cfg.rms_norm_eps, "rope": f"{cfg.rope.rope_type} theta {cfg.rope.theta:g} factor {cfg.rope.factor:g}",
            "tied_head": cfg.tie_word_embeddings, "kv_block_size": args.block_size, "prefill_tokens": 2048,
            "sampling": "greedy", "decode_steps_per_engine_step": per_engine_step,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
    }
    if not args.no_points:
        t = prefill_run(engine, cfg, 2048)
        line["prefill"] = {"value": round(2048 / t, 1), "tokens": 2048, "ms": round(t * 1e3, 3),
                           "frac": round(prefill_flops(cfg, 2048) / t / PEAK_FLOPS[short], 4)}
        points = {}
        steps, warm = min(args.steps, 32), min(args.warmup, 4)

        def point(key, b, context, per_call):
            tok_s, ms, _ = decode_run(engine, cfg, b, context, steps, warm, per_call)
            points[key] = round(tok_s, 1)
            points[key + "_ms"] = round(ms, 4)
            points[key + "_frac"] = round(decode_bytes(cfg, b, context, itemsize) / (ms * 1e-3) / 1e9 / HBM_GBPS, 4)

        for b in (1, 64):   # the headline's context, other batch sizes
            point(f"decode_b{b}", b, args.context, args.decode_steps)
        for b in (1, 8, 64):
            # one token per engine step, an engine's own default (generate() and the command line take eight)
            point(f"decode_b{b}_one_token_per_call", b, args.context, 1)
            # prompts of 2,048 tokens with 256 generated: the context grows from 2,048 to 2,304
            point(f"decode_b{b}_context2304", b, 2304, args.decode_steps)
        if args.shape == "Llama-3.2-1B" and not args.layers:
            # a long context: 8 requests of 32,768 keys each (attention reads 8.6 GB a step beside 2.5 GB of weights)
            import gc

            model = engine.core.model
            del engine
            gc.collect()
            torch.cuda.empty_cache()
            engine, _ = engine_for(model, 8, 32768, args.block_size, 8192, args.decode_steps)
            point("decode_b8_context32768", 8, 32768, args.decode_steps)
            # a long prompt in portions, each on top of the keys of the earlier ones
            for portion in (2048, 512):   # 512 is the scheduler's own default budget
                t = prefill_run(engine, cfg, 16384, repeats=2, portion=portion)
                key = f"prefill16384_in_portions_of_{portion}"
                points[key] = round(16384 / t, 1)
                points[key + "_ms"] = round(t * 1e3, 3)
                points[key + "_frac"] = round(prefill_flops(cfg, 16384) / t / PEAK_FLOPS[short], 4)
            del engine, model
            gc.collect()
            torch.cuda.empty_cache()
            if not args.no_other_shapes:
                points.update(other_shapes(args, short, itemsize))
                line["config"]["other_shapes"] = (
                    "llama3b: Llama-3.2-3B sizes (28 layers, hidden 3072, 24 heads of 128, 8 kv heads, intermediate "
                    "8192, vocab 128256); smollm2_1_7b: SmolLM2-1.7B sizes (24 layers, hidden 2048, 32 heads of 64, "
                    "32 kv heads, intermediate 8192, vocab 49152); serving: continuous batching, 64 requests with "
                    "prompts of 128-2048 tokens and 256 generated (mixed) or 32 requests sharing 1024 tokens plus "
                    "64-512 of their own and 128 generated, page reuse on (shared_prefix)")
        line["points"] = points
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
