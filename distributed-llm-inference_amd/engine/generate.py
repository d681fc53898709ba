"""Single-call entry points: greedy decoding of one prompt, and ``generate`` for a folder.

``greedy_generate`` follows the reference's function of that name (src/dli/generate.py:21-87):
argmax each step, lowest id on ties, end-of-sequence ids included in the output. It drives the
same step function, cache manager and kernels as the engine, one request at a time.
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Collection, Optional, Sequence

from ..sampling.params import SamplingParams
from .engine import LLMEngine
from .scheduler import SchedulerConfig


def greedy_generate(model: Any, prompt_ids: Sequence[int], max_new_tokens: int, *,
                    eos_token_ids: Collection[int] = (), block_size: int = 16,
                    dtype: str = "bfloat16", cuda_graphs: bool = True) -> list[int]:
    """Generate up to ``max_new_tokens`` tokens by taking the argmax each step."""
    if not prompt_ids:
        raise ValueError("prompt_ids must be non-empty")
    if max_new_tokens <= 0:
        return []
    pages = -(-(len(prompt_ids) + max_new_tokens) // block_size) + 1
    engine = LLMEngine.for_model(
        model, num_blocks=pages, block_size=block_size, eos_token_ids=eos_token_ids, dtype=dtype,
        config=SchedulerConfig(max_num_seqs=1, max_num_batched_tokens=max(512, len(prompt_ids))),
        enable_prefix_caching=False, cuda_graphs=cuda_graphs)
    return engine.generate([prompt_ids], SamplingParams(max_tokens=max_new_tokens))[0]


def pages_for_requests(lengths: Sequence[int], block_size: int, max_num_seqs: int, most: int) -> int:
    """Pages of a pool for requests that will hold ``lengths`` tokens each at their end: enough for
    the ``max_num_seqs`` longest to be live together (a page more each for a step's look ahead,
    and the share that admission keeps back), at most ``most`` (what the memory holds: a request
    that this leaves no room for is refused by the engine, as with any pool)."""
    each = sorted((-(-n // block_size) + 1 for n in lengths), reverse=True)
    together = sum(each[:max(1, max_num_seqs)])
    wanted = together + together // 50 + 8
    return max(1, min(wanted, most)) if each else 1


GRAPHS_PAY_FROM = 128  # decode steps of a call from which recording its decode graphs pays


def graphs_pay(max_tokens: Sequence[int], max_num_seqs: int) -> bool:
    """Whether a call that builds its own engine should record decode graphs: the graphs of a
    call are recorded during it (a handful of them, some 10 ms each at the 1B sizes, and 30 ms
    once for collecting the engine of an earlier call: the shapes that a batch's tail asks for a
    few times are served by a recorded shape of more rows) and save up to a millisecond a decode
    step afterwards, so they pay from about a hundred steps on (calls in a row in one process, 64
    requests, prompts of 128 to 2,048 tokens, seconds without and with them: 64 tokens each 0.41
    and 0.48, 128 tokens 0.60 and 0.58, 256 tokens 0.99 and 0.85, 1,024 tokens 3.41 and 2.52; 8
    requests: 64 tokens 0.152 and 0.163, 128 tokens 0.28 and 0.22, 1,024 tokens 2.03 and 1.09).
    The steps are estimated as the longest generation times the rounds that the requests need at
    ``max_num_seqs`` a time."""
    if not max_tokens:
        return False
    rounds = -(-len(max_tokens) // max(1, max_num_seqs))
    return max(max_tokens) * rounds >= GRAPHS_PAY_FROM


def generate(model: str | Path | Any, prompts: Sequence[Sequence[int]],
             params: SamplingParams | Sequence[SamplingParams] | None = None, *,
             dtype: str = "bfloat16", num_blocks: Optional[int] = None, kv_cache_gb: Optional[float] = None,
             block_size: int = 16, max_num_seqs: int = 256, max_num_batched_tokens: int = 4096,
             enable_prefix_caching: bool = True, eos_token_ids: Collection[int] = (), seed: int = 0,
             cuda_graphs: Optional[bool] = None, device: str = "cuda", decode_steps: int = 8,
             decode_weight_copy: bool = True) -> list[list[int]]:
    """Load ``model`` (a folder or a loaded model), run ``prompts`` to completion, return token ids.

    All requests are known before the first step and nobody watches tokens arrive, so three
    defaults differ from an engine's own, which are the reference's
    (src/dli/engine/scheduler.py:46-47, src/dli/server/__main__.py:153):
    ``decode_steps``: decoding steps run up to that many tokens of every request on the device
    before the host looks (same tokens, fewer round trips; eight against one: 7.5 k against 6.8 k
    tokens/s at batch 8 and the 1B sizes). Without decode graphs (32-bit, ``cuda_graphs=False``)
    a step is one token.
    ``max_num_batched_tokens`` and ``max_num_seqs``: 4,096 tokens a step and up to 256 live
    requests against 512 and 64. A step of 512 rows leaves the products at a third of the rate
    they reach with 2,048 (64 requests of 128 to 2,048 prompt tokens and 256 generated ones at the
    1B sizes: 0.70 s against 1.37 s), and decoding 256 requests together yields 1.7 times the
    tokens a second of 64 (256 such requests: 2.0 s against 2.9 s).
    The pool: with neither ``num_blocks`` nor ``kv_cache_gb``, as many pages as the live requests
    can fill (:func:`pages_for_requests`), within four fifths of the device memory that is free
    once the weights are loaded; an engine's own default is 1 GiB.
    ``cuda_graphs``: None decides by :func:`graphs_pay` (an engine of its own records them always:
    it lives longer than a call)."""
    import torch

    from ..weights.loader import load_model
    from .core import pages_for_budget

    prompts = [list(p) for p in prompts]
    if params is None or isinstance(params, SamplingParams):
        per = [params or SamplingParams()] * len(prompts)
    else:
        per = list(params)
        if len(per) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
    if isinstance(model, (str, Path)):
        model = load_model(model, dtype=dtype, device=device, decode_weight_copy=decode_weight_copy)
    if cuda_graphs is None:
        cuda_graphs = graphs_pay([q.max_tokens for q in per], max_num_seqs)
    max_model_len = None
    if num_blocks is None and kv_cache_gb is None and prompts:
        lengths = [len(p) + q.max_tokens for p, q in zip(prompts, per)]
        free, _ = torch.cuda.mem_get_info(torch.device(device))
        num_blocks = pages_for_requests(lengths, block_size, max_num_seqs,
                                        pages_for_budget(model, block_size, free // 5 * 4))
        max_model_len = -(-max(lengths) // block_size) * block_size
    engine = LLMEngine.for_model(
        model, num_blocks=num_blocks, kv_cache_gb=kv_cache_gb, block_size=block_size, dtype=dtype,
        config=SchedulerConfig(max_num_seqs=max_num_seqs, max_num_batched_tokens=max_num_batched_tokens,
                               decode_steps=decode_steps),
        enable_prefix_caching=enable_prefix_caching, eos_token_ids=eos_token_ids, seed=seed,
        cuda_graphs=cuda_graphs, device=device, max_model_len=max_model_len)
    return engine.generate(prompts, per)
