"""Each part alone against the plain implementation's function for it, the cache store's page
copies, and the proof that another mixer plugs in: a toy mixer with state of its own is
registered, built and stepped here without a change to the framework's files."""

from __future__ import annotations

import math

import pytest
import torch

import plain_llama as P
from tiny_configs import TINY_A, TINY_B, model_folder

pytestmark = pytest.mark.gpu


def rt(dtype=torch.float32):
    from dli_amd.parts import Runtime

    return Runtime(torch.device("cuda"), dtype)


def test_norm_part_alone():
    from dli_amd.parts import PartSpec, build_part

    norm = build_part("norm", PartSpec("rms_norm", dict(width=192, eps=1e-6)), rt())
    w = (1 + 0.1 * torch.randn(192)).cuda()
    norm.load_weights({"weight": w})
    x = torch.randn(7, 192, device="cuda") * 3
    ref = P.rms_norm(x.cpu().double(), w.cpu().double(), 1e-6)
    assert (norm.forward(x.clone()).cpu().double() - ref).abs().max() < 1e-5
    delta = torch.randn_like(x)
    stream = x.clone()
    out = norm.forward(stream, delta)
    assert torch.allclose(stream, x + delta)  # the residual sum is made in place
    ref2 = P.rms_norm((x + delta).cpu().double(), w.cpu().double(), 1e-6)
    assert (out.cpu().double() - ref2).abs().max() < 1e-5
    assert norm.weight_specs()["weight"].role == "float32"


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_rotary_part_alone(raw):
    from dli_amd.architectures.llama import build_llama_spec
    from dli_amd.config import LlamaConfig
    from dli_amd.parts import build_part

    cfg = LlamaConfig.from_hf_dict(raw)
    spec = build_llama_spec(cfg).layers[0].parts["mixer"][1].params["position"]
    part = build_part("position", spec, rt())
    table, dim, pairing = part.rotary_table()
    assert dim == cfg.head_dim and pairing == "half"
    ref = P.inverse_frequencies(P.rope_settings(raw), cfg.head_dim)
    assert torch.allclose(table.cpu(), ref, rtol=2e-7, atol=0)


def test_feed_forward_part_alone():
    from dli_amd.parts import PartSpec, build_part

    for dtype, tol in ((torch.float32, 1e-4), (torch.bfloat16, 5e-2)):
        ff = build_part("feed_forward", PartSpec("gated_mlp", dict(hidden_size=64, intermediate_size=160, bias=True)), rt(dtype))
        w = {k: (torch.randn(*s.shape) / math.sqrt(s.shape[-1])).to(dtype) for k, s in ff.weight_specs().items()}
        ff.load_weights({k: v.cuda() for k, v in w.items()})
        x = torch.randn(5, 64).to(dtype)
        ref = P.swiglu_mlp(x.double(), {k: v.double() for k, v in w.items()}, "")
        got = ff.forward(x.cuda(), None)
        assert (got.cpu().double() - ref).abs().max() < tol * max(1.0, ref.abs().max().item())


def test_embedding_and_head_parts_alone():
    from dli_amd.parts import PartSpec, build_part

    emb = build_part("embedding", PartSpec("token_embedding", dict(vocab_size=301, hidden_size=72)), rt())
    table = torch.randn(301, 72).cuda()
    emb.load_weights({"weight": table})
    ids = torch.tensor([0, 300, 17], dtype=torch.int32, device="cuda")
    assert torch.equal(emb.forward(ids), table[ids.long()])
    for tied in (True, False):
        head = build_part("head", PartSpec("linear_head", dict(vocab_size=301, hidden_size=72, tied=tied)), rt())
        own = torch.randn(301, 72).cuda()
        head.load_weights({} if tied else {"weight": own})
        head.tie(table)
        x = torch.randn(4, 72, device="cuda")
        ref = x.cpu().double() @ (table if tied else own).cpu().double().T
        assert (head.forward(x).cpu().double() - ref).abs().max() < 1e-4
        assert bool(head.weight_specs()) == (not tied)


@pytest.mark.parametrize("name,dtype,page", [("A", "float32", 16), ("B", "float32", 8), ("B", "bfloat16", 16)])
def test_attention_part_alone(name, dtype, page):
    """The mixer of layer 0 with the model's own weights, fed rows directly: a fresh prompt, then
    a portion on top of it, against plain attention over the whole sequence."""
    from dli_amd.engine.batch import StepEntry
    from dli_amd.engine.core import build_core

    core = build_core(model_folder(name), num_pages=16, page_size=page, max_seqs=2, dtype=dtype,
                      enable_prefix_caching=False, watermark=0.0)
    cfg, w = P.load_folder(model_folder(name))
    sizes = P.model_sizes(cfg)
    mixer = core.model.layers[0].parts["mixer"]
    n = 23
    torch.manual_seed(1)
    x = torch.randn(n, cfg["hidden_size"]).to(core.model.rt.dtype)
    cos, sin = P.rope_cos_sin(P.inverse_frequencies(P.rope_settings(cfg), sizes["head_dim"]), torch.arange(n), torch.float64)
    ref = P.attention_block(x.double(), {k: v.double() for k, v in w.items()}, "model.layers.0.self_attn.", sizes, cos, sin)
    core.manager.allocate("r", list(range(n)), respect_watermark=False)
    outs = []
    for lo, hi in ((0, 14), (14, 23)):
        ctx = core.step.build_context([StepEntry("r", list(range(lo, hi)), lo, ())])
        outs.append(mixer.forward(x[lo:hi].cuda().contiguous(), ctx, core.step.caches[0]))
        core.manager.mark_computed("r", hi)
    got = torch.cat(outs).cpu().double()
    tol = 1e-4 if dtype == "float32" else 4e-2
    assert (got - ref).abs().max() < tol * max(1.0, ref.abs().max().item())


def test_page_copies_cover_every_layer():
    from dli_amd.cache.manager import CopyOp
    from dli_amd.engine.core import build_core

    core = build_core(model_folder("A"), num_pages=8, page_size=16, max_seqs=2, dtype="bfloat16")
    (pool,) = core.store.pools[0]
    pool.copy_(torch.randn(pool.shape, device="cuda").to(pool.dtype))
    before = pool.clone()
    core.store.copy_pages([CopyOp(src=2, dst=5), CopyOp(src=7, dst=0)])
    assert torch.equal(pool[:, :, 5], before[:, :, 2]) and torch.equal(pool[:, :, 0], before[:, :, 7])
    keep = [1, 2, 3, 4, 6, 7]
    assert torch.equal(pool[:, :, keep], before[:, :, keep])
    with pytest.raises(ValueError):
        core.store.copy_pages([CopyOp(src=1, dst=8)])


# ------------------------------------------------------------------ a toy mixer with state of its own

def test_a_toy_mixer_with_state_is_registered_built_and_stepped():
    """An exponential moving average over a request's rows: y_t = s_t W, s_t = a*s_{t-1} + x_t.
    Its state lives in the request's state slot. The model below alternates it with attention
    layers and runs one layer twice; stepping it in portions and mixed batches must equal running
    each request whole."""
    from typing import Any, Mapping

    from dli_amd.cache.manager import CacheManager
    from dli_amd.cache.store import CacheStore, group_specs
    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.engine.core import EngineCore
    from dli_amd.engine.step import StepFunction
    from dli_amd.parts import (LayerSpec, Mixer, ModelSpec, PartSpec, ScheduleEntry, StateSpec, WeightSpec,
                               register_part, unregister_part)
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model, write_random_model

    @register_part("mixer", "toy_ema")
    class ToyEMA(Mixer):
        def __init__(self, runtime, *, hidden_size: int, decay: float) -> None:
            super().__init__(runtime)
            self.hidden_size, self.decay = hidden_size, decay
            self.w = None

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.hidden_size, self.hidden_size))}

        def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
            self.w = tensors["mix.weight"]

        def cache_spec(self):
            return StateSpec((self.hidden_size,), torch.float32)

        def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
            out = torch.empty_like(x)
            for e in range(ctx.num_entries):  # a toy: plain torch, one request after the other
                r0, r1 = ctx.entry_rows(e)
                slot = int(ctx.state_slots_host[e])
                state = torch.zeros_like(cache.state[slot]) if ctx.is_fresh(e) else cache.state[slot].clone()
                for r in range(r0, r1):
                    state = self.decay * state + x[r].float()
                    out[r] = (state @ self.w.float().T).to(x.dtype)
                cache.state[slot] = state
            return out

    def parse(raw):
        return dict(raw)

    def build(cfg):
        h = cfg["hidden_size"]
        norm = dict(width=h, eps=cfg["eps"])
        pos = PartSpec("rotary", dict(dim=16, theta=10000.0))
        layers = []
        for i in range(3):
            p = f"layers.{i}."
            mixer = (PartSpec("toy_ema", dict(hidden_size=h, decay=0.5), p + "ema.") if i == 1 else
                     PartSpec("gqa_attention", dict(hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=16, position=pos,
                                                    window=9 if i == 2 else 0), p + "attn."))
            layers.append(LayerSpec(PartSpec("pre_norm"), {
                "mixer_norm": ("norm", PartSpec("rms_norm", norm, p + "n1.")), "mixer": ("mixer", mixer),
                "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, p + "n2.")),
                "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=48), p + "mlp."))}))
        return ModelSpec(
            architecture="ToyForCausalLM", vocab_size=cfg["vocab_size"], hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=cfg["vocab_size"], hidden_size=h), "embed."),
            layers=tuple(layers),
            # layer 0 runs twice (two caches), the windowed layer 2 and the stateful layer 1 between
            schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0)),
            final_norm=PartSpec("rms_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=cfg["vocab_size"], hidden_size=h, tied=True), "head."))

    register_architecture("ToyForCausalLM", parse, build)
    try:
        import tempfile

        raw = {"architectures": ["ToyForCausalLM"], "vocab_size": 61, "hidden_size": 32, "eps": 1e-5}
        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, raw, seed=3, std=0.2, norm_jitter=0.1)

            def make():
                model = load_model(folder, dtype="float32")
                specs = model.cache_specs()
                assert [type(s).__name__ for s in specs] == ["PagedKVSpec", "StateSpec", "PagedKVSpec", "PagedKVSpec"]
                store = CacheStore(model.rt, specs, num_pages=12, page_size=4, max_seqs=4)
                assert len(store.groups) == 2 and store.stateful  # full attention and the window of 9
                mgr = CacheManager(group_specs(store.groups), num_pages=12, page_size=4, max_seqs=4,
                                   stateful=store.stateful, watermark=0.0)
                assert not mgr.prefix_caching
                return EngineCore(model, mgr, store, StepFunction(model, mgr, store))

            toks = {"a": [5, 9, 2, 40, 33, 7, 7, 12, 60, 1, 18, 25, 3, 3, 44, 51, 9, 30, 2, 11, 17],
                    "b": [8, 8, 1, 50, 23, 4, 19, 36, 2, 45, 13, 27]}
            whole = {}
            for rid, t in toks.items():
                s = TraceSession(make())
                whole[rid] = s.step([{"id": rid, "tokens": t, "want": list(range(len(t)))}]).cpu()
            core = make()
            s = TraceSession(core)
            got = {"a": [], "b": []}
            plan = [{"a": 5}, {"a": 2, "b": 3}, {"a": 1, "b": 1}, {"b": 6}, {"a": 9, "b": 1}, {"a": 1, "b": 1}, {"a": 3}]
            fed = {"a": 0, "b": 0}
            for stepplan in plan:
                entries = []
                for rid, n in stepplan.items():
                    entries.append({"id": rid, "tokens": toks[rid][fed[rid]:fed[rid] + n], "want": list(range(n))})
                out = s.step(entries).cpu()
                row = 0
                for rid, n in stepplan.items():
                    got[rid].append(out[row:row + n])
                    row += n
                    fed[rid] += n
                core.manager.check_invariants()
            for rid in toks:
                assert fed[rid] == len(toks[rid])
                assert (torch.cat(got[rid]) - whole[rid]).abs().max() < 1e-4, rid
            assert core.manager.stats().window_pages_released > 0  # the window gave pages back
            s.step([], end=["a", "b"])
            assert core.manager.stats().used_pages == 0
    finally:
        unregister_architecture("ToyForCausalLM")
        unregister_part("mixer", "toy_ema")


def test_a_rotary_table_with_another_pairing_is_refused_and_any_role_may_own_the_cache():
    """The attention kernels rotate pairs (i, i + dim/2): a position encoding whose table names
    another pairing is refused when the mixer is finalized, not rotated wrongly. And the part of
    a layer that keeps a cache is found by what it answers to ``cache_spec()``, not by its role's
    name; two such parts in one layer are refused."""
    from dli_amd.kernels.ops import KernelArgumentError
    from dli_amd.parts import (LayerSpec, ModelSpec, PartSpec, PositionEncoding, RotaryTable, ScheduleEntry,
                               build_part, register_part, unregister_part)
    from dli_amd.parts.model import Model

    @register_part("position", "toy_adjacent_rotary")
    class Adjacent(PositionEncoding):
        def __init__(self, runtime, *, dim: int) -> None:
            super().__init__(runtime)
            self.dim = dim

        def rotary_table(self):
            return RotaryTable(torch.ones(self.dim // 2, device=self.rt.device), self.dim, "adjacent")

    try:
        attn = dict(hidden_size=32, num_heads=2, num_kv_heads=1, head_dim=16)
        bad = build_part("mixer", PartSpec("gqa_attention", dict(attn, position=PartSpec("toy_adjacent_rotary", dict(dim=16)))), rt())
        with pytest.raises(KernelArgumentError, match="adjacent"):
            bad.finalize()
        norm = dict(width=32, eps=1e-5)
        mixer = PartSpec("gqa_attention", dict(attn, position=PartSpec("rotary", dict(dim=16, theta=1e4))), "a.")

        def spec(parts):
            return ModelSpec(
                architecture="Toy", vocab_size=40, hidden_size=32,
                embedding=PartSpec("token_embedding", dict(vocab_size=40, hidden_size=32), "embed."),
                layers=(LayerSpec(PartSpec("pre_norm"), parts),), schedule=(ScheduleEntry(0),),
                final_norm=PartSpec("rms_norm", norm, "norm."),
                head=PartSpec("linear_head", dict(vocab_size=40, hidden_size=32, tied=True), "head."))

        base = {"mixer_norm": ("norm", PartSpec("rms_norm", norm, "n1.")), "mixer": ("mixer", mixer),
                "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, "n2.")),
                "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=32, intermediate_size=48), "mlp."))}
        model = Model(spec(base), rt())
        assert model.cache_owners() == [model.layers[0].parts["mixer"]]
        assert type(model.cache_specs()[0]).__name__ == "PagedKVSpec"
        two = dict(base, second_mixer=("mixer", PartSpec("gqa_attention", dict(attn), "b.")))
        with pytest.raises(ValueError, match="each keep a cache"):
            Model(spec(two), rt()).cache_specs()
    finally:
        unregister_part("position", "toy_adjacent_rotary")


# ------------------------------------------------------------------ toy feed-forward with routing, toy position encoding

def test_a_toy_routed_feed_forward_and_a_toy_position_encoding_are_registered_built_and_stepped():
    """Two more parts defined here and nowhere in the framework: a feed-forward that routes each
    row to one of three small experts (router logits and the choice in 32-bit), and a position
    encoding that is no rotation (q_i is scaled by s^i and k_j by s^-j, so a score decays with the
    distance i - j). A model that uses them in one layer and the built-in parts in the other steps
    in portions and mixed batches exactly as each request does whole."""
    from typing import Any, Mapping

    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.engine.core import build_core
    from dli_amd.parts import (FeedForward, LayerSpec, ModelSpec, PartSpec, PositionEncoding, ScheduleEntry,
                               WeightSpec, register_part, unregister_part)
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model, write_random_model

    @register_part("feed_forward", "toy_routed")
    class ToyRouted(FeedForward):
        def __init__(self, runtime, *, hidden_size: int, experts: int, expert_size: int) -> None:
            super().__init__(runtime)
            self.h, self.e, self.f = hidden_size, experts, expert_size
            self.t = {}

        def weight_specs(self):
            return {"router.weight": WeightSpec((self.e, self.h), role="float32"),
                    "up.weight": WeightSpec((self.e * self.f, self.h)),
                    "down.weight": WeightSpec((self.e * self.h, self.f))}

        def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
            self.t = dict(tensors)

        def forward(self, x: torch.Tensor, ctx: Any) -> torch.Tensor:
            scores = torch.softmax(x.float() @ self.t["router.weight"].float().T, dim=-1)
            weight, choice = scores.max(dim=-1)
            up = self.t["up.weight"].float().view(self.e, self.f, self.h)
            down = self.t["down.weight"].float().view(self.e, self.h, self.f)
            out = torch.empty_like(x)
            for r in range(x.shape[0]):  # a toy: one row after the other
                e = int(choice[r])
                out[r] = (weight[r] * (down[e] @ torch.relu(up[e] @ x[r].float()))).to(x.dtype)
            return out

    @register_part("position", "toy_decay")
    class ToyDecay(PositionEncoding):
        def __init__(self, runtime, *, base: float) -> None:
            super().__init__(runtime)
            self.base = base

        def apply(self, q, k, positions) -> None:
            s = torch.pow(torch.tensor(self.base, device=q.device), positions.float())[:, None, None]
            q.mul_(s.to(q.dtype))
            if k is not None:
                k.div_(s.to(k.dtype))

    def build(cfg):
        h = cfg["hidden_size"]
        norm = dict(width=h, eps=cfg["eps"])
        attn = dict(hidden_size=h, num_heads=4, num_kv_heads=2, head_dim=16)
        ffs = [PartSpec("toy_routed", dict(hidden_size=h, experts=3, expert_size=24), "layers.0.moe."),
               PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=40), "layers.1.mlp.")]
        poss = [PartSpec("toy_decay", dict(base=1.04)), PartSpec("rotary", dict(dim=16, theta=100.0))]
        layers = [LayerSpec(PartSpec("pre_norm"), {
            "mixer_norm": ("norm", PartSpec("rms_norm", norm, f"layers.{i}.n1.")),
            "mixer": ("mixer", PartSpec("gqa_attention", dict(attn, position=poss[i]), f"layers.{i}.attn.")),
            "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, f"layers.{i}.n2.")),
            "feed_forward": ("feed_forward", ffs[i])}) for i in range(2)]
        return ModelSpec(
            architecture="ToyRoutedForCausalLM", vocab_size=cfg["vocab_size"], hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=cfg["vocab_size"], hidden_size=h), "embed."),
            layers=tuple(layers), schedule=(ScheduleEntry(0), ScheduleEntry(1)),
            final_norm=PartSpec("rms_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=cfg["vocab_size"], hidden_size=h, tied=False), "head."))

    register_architecture("ToyRoutedForCausalLM", dict, build)
    try:
        import tempfile

        raw = {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 47, "hidden_size": 32, "eps": 1e-6}
        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, raw, seed=8, std=0.25, norm_jitter=0.1)
            make = lambda: build_core(load_model(folder, dtype="float32"), num_pages=14, page_size=4, max_seqs=4,
                                      enable_prefix_caching=False, watermark=0.0)
            toks = {"a": [5, 9, 2, 40, 33, 7, 7, 12, 46, 1, 18, 25, 3, 3, 44, 21, 9, 30, 2, 11, 17],
                    "b": [8, 8, 1, 30, 23, 4, 19, 36, 2, 45, 13, 27]}
            whole, routes = {}, set()
            for rid, t in toks.items():
                core = make()
                whole[rid] = TraceSession(core).step([{"id": rid, "tokens": t, "want": list(range(len(t)))}]).cpu()
                moe = core.model.layers[0].parts["feed_forward"]
                x = torch.randn(64, 32, device="cuda")
                routes |= set((x @ moe.t["router.weight"].float().T).argmax(-1).tolist())
            assert len(routes) > 1, "the router always picks the same expert: the test would prove little"
            core = make()
            s = TraceSession(core)
            got, fed = {"a": [], "b": []}, {"a": 0, "b": 0}
            for stepplan in [{"a": 5}, {"a": 2, "b": 3}, {"a": 1, "b": 1}, {"b": 6}, {"a": 9, "b": 1}, {"a": 1, "b": 1}, {"a": 3}]:
                entries = [{"id": rid, "tokens": toks[rid][fed[rid]:fed[rid] + n], "want": list(range(n))}
                           for rid, n in stepplan.items()]
                out = s.step(entries).cpu()
                row = 0
                for rid, n in stepplan.items():
                    got[rid].append(out[row:row + n])
                    row += n
                    fed[rid] += n
            for rid in toks:
                assert fed[rid] == len(toks[rid])
                assert (torch.cat(got[rid]) - whole[rid]).abs().max() < 1e-4, rid
    finally:
        unregister_architecture("ToyRoutedForCausalLM")
        unregister_part("feed_forward", "toy_routed")
        unregister_part("position", "toy_decay")


# ------------------------------------------------------------------ toy mixers whose cache is not keys and values of one size

def test_toy_mixers_with_smaller_values_and_with_keys_only_get_their_pages_and_step():
    """A mixer declares the size of its values beside that of its keys (``PagedKVSpec.value_dim``):
    a toy attention with keys of 16 and values of 8 numbers, and a toy that keeps one compressed
    vector per token and no values at all, defined here, get pages of their own sizes, step in
    portions and mixed batches as each request does whole, and their pages are copied on a fork."""
    from typing import Any, Mapping

    from dli_amd.cache.manager import CopyOp
    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.engine.core import build_core
    from dli_amd.parts import (LayerSpec, Mixer, ModelSpec, PagedKVSpec, PartSpec, ScheduleEntry, WeightSpec,
                               register_part, unregister_part)
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model, write_random_model

    class ToyPaged(Mixer):
        """Single-head attention in plain torch over the request's pages; ``vd`` 0: the cached
        vector serves as key and as value."""

        def __init__(self, runtime, *, hidden_size: int, kd: int, vd: int) -> None:
            super().__init__(runtime)
            self.h, self.kd, self.vd = hidden_size, kd, vd
            self.t = {}

        def weight_specs(self):
            specs = {"q.weight": WeightSpec((self.kd, self.h)), "k.weight": WeightSpec((self.kd, self.h)),
                     "o.weight": WeightSpec((self.h, self.vd or self.kd))}
            if self.vd:
                specs["v.weight"] = WeightSpec((self.vd, self.h))
            return specs

        def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
            self.t = {k: v.float() for k, v in tensors.items()}

        def cache_spec(self):
            return PagedKVSpec(1, self.kd, value_dim=self.vd)

        def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
            grp = ctx.groups[cache.group]
            bs = cache.k_pages.shape[2]
            assert (cache.v_pages is None) == (self.vd == 0)
            assert self.vd == 0 or cache.v_pages.shape[1:] == (1, self.vd, bs)
            xf = x.float()
            q, k = xf @ self.t["q.weight"].T, xf @ self.t["k.weight"].T
            slots = grp.slots.tolist()
            for r, slot in enumerate(slots):
                cache.k_pages[slot // bs, 0, slot % bs] = k[r].to(x.dtype)
                if self.vd:
                    cache.v_pages[slot // bs, 0, :, slot % bs] = (xf[r] @ self.t["v.weight"].T).to(x.dtype)
            out = torch.empty_like(x)
            tables = grp.block_tables.tolist()
            kv_len, q_start = ctx.kv_len.tolist(), ctx.q_start.tolist()
            for e in range(ctx.num_entries):
                r0, r1 = q_start[e], q_start[e + 1]
                pages = tables[e][:-(-kv_len[e] // bs)]
                keys = cache.k_pages[pages, 0].reshape(-1, self.kd)[:kv_len[e]].float()
                vals = (cache.v_pages[pages, 0].permute(0, 2, 1).reshape(-1, self.vd)[:kv_len[e]].float()
                        if self.vd else keys)
                for r in range(r0, r1):
                    seen = kv_len[e] - (r1 - 1 - r)
                    w = torch.softmax(keys[:seen] @ q[r] / self.kd ** 0.5, dim=0)
                    out[r] = ((w @ vals[:seen]) @ self.t["o.weight"].T).to(x.dtype)
            return out

    def build(cfg):
        h = cfg["hidden_size"]
        norm = dict(width=h, eps=cfg["eps"])
        mixers = [PartSpec("toy_paged", dict(hidden_size=h, kd=16, vd=8), "layers.0.mix."),
                  PartSpec("toy_paged", dict(hidden_size=h, kd=12, vd=0), "layers.1.mix."),
                  PartSpec("gqa_attention", dict(hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=16,
                                                 position=PartSpec("rotary", dict(dim=16, theta=100.0))), "layers.2.attn.")]
        layers = [LayerSpec(PartSpec("pre_norm"), {
            "mixer_norm": ("norm", PartSpec("rms_norm", norm, f"layers.{i}.n1.")), "mixer": ("mixer", mixers[i]),
            "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, f"layers.{i}.n2.")),
            "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=40),
                                                      f"layers.{i}.mlp."))}) for i in range(3)]
        return ModelSpec(
            architecture="ToyPagedForCausalLM", vocab_size=cfg["vocab_size"], hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=cfg["vocab_size"], hidden_size=h), "embed."),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(3)),
            final_norm=PartSpec("rms_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=cfg["vocab_size"], hidden_size=h, tied=True), "head."))

    register_part("mixer", "toy_paged")(ToyPaged)
    register_architecture("ToyPagedForCausalLM", dict, build)
    try:
        import tempfile

        raw = {"architectures": ["ToyPagedForCausalLM"], "vocab_size": 53, "hidden_size": 32, "eps": 1e-6}
        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, raw, seed=5, std=0.3, norm_jitter=0.1)
            make = lambda: build_core(load_model(folder, dtype="float32"), num_pages=14, page_size=4, max_seqs=4,
                                      enable_prefix_caching=False, watermark=0.0)
            core = make()
            store = core.store
            assert len(store.groups) == 3                      # three different needs, three block tables
            assert [[tuple(t.shape[1:]) for t in pools] for pools in store.pools] == [
                [(1, 14, 4 * 16), (1, 14, 4 * 8)], [(1, 14, 4 * 12)], [(2, 14, 4 * 16)]]
            assert store.bytes_per_page() == 4 * 4 * (16 + 8 + 12 + 16 + 16)
            toks = {"a": [5, 9, 2, 40, 33, 7, 7, 12, 46, 1, 18, 25, 3, 3, 44, 21, 9, 30, 2, 11, 17],
                    "b": [8, 8, 1, 30, 23, 4, 19, 36, 2, 45, 13, 27]}
            whole = {rid: TraceSession(make()).step([{"id": rid, "tokens": t, "want": list(range(len(t)))}]).cpu()
                     for rid, t in toks.items()}
            assert (whole["a"][5] - whole["a"][6]).abs().max() > 1e-3    # the same token twice: the context counts
            s = TraceSession(core)
            got, fed = {"a": [], "b": []}, {"a": 0, "b": 0}
            for stepplan in [{"a": 5}, {"a": 2, "b": 3}, {"a": 1, "b": 1}, {"b": 6}, {"a": 9, "b": 1}, {"a": 1, "b": 1}, {"a": 3}]:
                entries = [{"id": rid, "tokens": toks[rid][fed[rid]:fed[rid] + n], "want": list(range(n))}
                           for rid, n in stepplan.items()]
                out = s.step(entries).cpu()
                row = 0
                for rid, n in stepplan.items():
                    got[rid].append(out[row:row + n])
                    row += n
                    fed[rid] += n
            for rid in toks:
                assert (torch.cat(got[rid]) - whole[rid]).abs().max() < 1e-4, rid
            # a fork inside a partly filled page copies the keys-only pages and the small values too
            s.fork("a", "c")
            tail = [31, 6, 50]
            out_c = s.step([{"id": "c", "tokens": tail, "want": [0, 1, 2]}]).cpu()
            alone = TraceSession(make()).step([{"id": "x", "tokens": toks["a"] + tail,
                                                "want": list(range(len(toks["a"]), len(toks["a"]) + 3))}]).cpu()
            assert (out_c - alone).abs().max() < 1e-4
            before = [t.clone() for pools in store.pools for t in pools]
            store.copy_pages([CopyOp(src=1, dst=13, group=g) for g in range(3)])
            for t, b in zip([t for pools in store.pools for t in pools], before):
                assert torch.equal(t[:, :, 13], b[:, :, 1]) and torch.equal(t[:, :, :13], b[:, :, :13])
    finally:
        unregister_architecture("ToyPagedForCausalLM")
        unregister_part("mixer", "toy_paged")


# ------------------------------------------------------------------ a stateful toy mixer replayed from graphs

@pytest.mark.parametrize("capturable", [True, False])
def test_a_stateful_toy_mixer_that_says_it_can_be_recorded_is_replayed_from_graphs(capturable):
    """Decode graphs are not tied to attention: a model whose parts all answer
    ``graph_capturable`` with True is recorded and replayed, state slots included (padding rows of
    a replay write the slot that no request holds). The toy's decode form works on the step's
    device arrays only; with the answer False the same model decodes eagerly. Both equal each
    request run whole."""
    from typing import Any, Mapping

    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.engine.core import build_core
    from dli_amd.parts import (LayerSpec, Mixer, ModelSpec, PartSpec, ScheduleEntry, StateSpec, WeightSpec,
                               register_part, unregister_part)
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model, write_random_model

    @register_part("mixer", "toy_ema_device")
    class ToyEMADevice(Mixer):
        def __init__(self, runtime, *, hidden_size: int, decay: float) -> None:
            super().__init__(runtime)
            self.hidden_size, self.decay = hidden_size, decay
            self.w = None

        def weight_specs(self):
            return {"mix.weight": WeightSpec((self.hidden_size, self.hidden_size))}

        def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
            self.w = tensors["mix.weight"].float()

        def cache_spec(self):
            return StateSpec((self.hidden_size,), torch.float32)

        def graph_capturable(self, page_size: int) -> bool:
            return capturable

        def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
            if ctx.num_decode == ctx.num_tokens:  # one token a request: device arrays only, no waiting
                slots = ctx.state_slots.long()
                before = cache.state[slots]
                before = torch.where((ctx.positions == 0)[:, None], torch.zeros_like(before), before)
                state = self.decay * before + x.float()
                cache.state.index_copy_(0, slots, state)
                return (state @ self.w.T).to(x.dtype)
            out = torch.empty_like(x)
            for e in range(ctx.num_entries):
                r0, r1 = ctx.entry_rows(e)
                slot = int(ctx.state_slots_host[e])
                state = torch.zeros_like(cache.state[slot]) if ctx.is_fresh(e) else cache.state[slot].clone()
                for r in range(r0, r1):
                    state = self.decay * state + x[r].float()
                    out[r] = (state @ self.w.T).to(x.dtype)
                cache.state[slot] = state
            return out

    def build(cfg):
        h = cfg["hidden_size"]
        norm = dict(width=h, eps=cfg["eps"])
        mixers = [PartSpec("gqa_attention", dict(hidden_size=h, num_heads=4, num_kv_heads=2, head_dim=16,
                                                 position=PartSpec("rotary", dict(dim=16, theta=1e4))), "layers.0.attn."),
                  PartSpec("toy_ema_device", dict(hidden_size=h, decay=0.6), "layers.1.ema.")]
        layers = [LayerSpec(PartSpec("pre_norm"), {
            "mixer_norm": ("norm", PartSpec("rms_norm", norm, f"layers.{i}.n1.")), "mixer": ("mixer", mixers[i]),
            "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, f"layers.{i}.n2.")),
            "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=96),
                                                      f"layers.{i}.mlp."))}) for i in range(2)]
        return ModelSpec(
            architecture="ToyStatefulForCausalLM", vocab_size=cfg["vocab_size"], hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=cfg["vocab_size"], hidden_size=h), "embed."),
            layers=tuple(layers), schedule=(ScheduleEntry(0), ScheduleEntry(1)),
            final_norm=PartSpec("rms_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=cfg["vocab_size"], hidden_size=h, tied=True), "head."))

    register_architecture("ToyStatefulForCausalLM", dict, build)
    try:
        import tempfile

        raw = {"architectures": ["ToyStatefulForCausalLM"], "vocab_size": 96, "hidden_size": 64, "eps": 1e-5}
        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, raw, seed=21, std=0.12, norm_jitter=0.1)

            def make(graphs):
                core = build_core(load_model(folder, dtype="bfloat16"), num_pages=12, page_size=16, max_seqs=4,
                                  enable_prefix_caching=False, watermark=0.0)
                if graphs:
                    core.step.enable_decode_graphs(4, 12 * 16)
                return core

            toks = {"a": [5, 9, 2, 40, 33, 7, 7, 12, 60, 1, 18, 25, 3, 3, 44, 51, 9, 30, 2, 11, 17],
                    "b": [8, 8, 1, 50, 23, 4, 19, 36, 2, 45, 13, 27, 90, 6], "c": [70, 3, 3, 15, 81, 22, 9]}
            whole = {rid: TraceSession(make(False)).step([{"id": rid, "tokens": t, "want": list(range(len(t)))}]).float().cpu()
                     for rid, t in toks.items()}
            core = make(True)
            assert (core.step.graphs is not None) == capturable
            s = TraceSession(core)
            heads = {"a": 15, "b": 8, "c": 1}     # c decodes from its first token on: its state starts in a replay
            s.step([{"id": rid, "tokens": toks[rid][:n], "want": []} for rid, n in heads.items() if n > 1])
            s.step([{"id": "c", "tokens": toks["c"][:1], "want": [0]}])
            fed = dict(heads)
            worst = 0.0
            for stepno in range(6):
                live = [rid for rid in toks if fed[rid] < len(toks[rid])]
                out = s.step([{"id": rid, "tokens": [toks[rid][fed[rid]]], "want": [0]} for rid in live]).float().cpu()
                for row, rid in enumerate(live):
                    ref = whole[rid][fed[rid]]
                    worst = max(worst, ((out[row] - ref).abs().max() / max(1.0, ref.abs().max().item())).item())
                    fed[rid] += 1
            assert worst < 4e-2, worst
            assert not capturable or core.step.graphs.replays >= 6
    finally:
        unregister_architecture("ToyStatefulForCausalLM")
        unregister_part("mixer", "toy_ema_device")


# ------------------------------------------------------------------ a toy block arrangement

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_block_arrangement_is_registered_built_and_stepped(dtype):
    """Another arrangement of a layer's parts, defined here and nowhere in the framework: one norm,
    and mixer and feed-forward side by side, ``x + attention(norm(x)) + mlp(norm(x))``. It
    implements ``forward`` only (no description for the loop in C, no fused decode form), so every
    optional route must step aside by itself, in both precisions: the model below has such a
    layer, a pre-norm layer, and such a layer again, and runs whole, in portions, mixed and token
    by token (through decode graphs in bfloat16) against a plain float64 model of that
    arrangement written with the plain implementation's parts."""
    import tempfile
    from typing import Any, Mapping

    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.engine.core import build_core
    from dli_amd.parts import Block, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_part, unregister_part
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model, write_random_model

    @register_part("block", "toy_parallel")
    class ToyParallel(Block):
        roles = ("norm", "mixer", "feed_forward")

        def __init__(self, runtime) -> None:
            super().__init__(runtime)

        def graph_capturable(self, page_size: int) -> bool:
            return True  # nothing here reads the host's arrays

        def forward(self, x, delta, ctx: Any, cache: Any, parts: Mapping[str, Any]):
            h = parts["norm"].forward(x, delta)  # x <- x + delta
            return x, parts["mixer"].forward(h, ctx, cache) + parts["feed_forward"].forward(h, ctx)

    h, heads, kv_heads, d, inter, vocab, eps, theta = 48, 3, 1, 16, 80, 53, 1e-5, 1000.0

    def build(cfg):
        norm = dict(width=h, eps=eps)
        pos = PartSpec("rotary", dict(dim=d, theta=theta))
        layers = []
        for i, kind in enumerate(("toy_parallel", "pre_norm", "toy_parallel")):
            p = f"layers.{i}."
            parts = {"mixer": ("mixer", PartSpec("gqa_attention", dict(hidden_size=h, num_heads=heads, num_kv_heads=kv_heads,
                                                                      head_dim=d, position=pos), p + "attn.")),
                     "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=inter),
                                                               p + "mlp."))}
            if kind == "toy_parallel":
                parts["norm"] = ("norm", PartSpec("rms_norm", norm, p + "n."))
            else:
                parts["mixer_norm"] = ("norm", PartSpec("rms_norm", norm, p + "n1."))
                parts["feed_forward_norm"] = ("norm", PartSpec("rms_norm", norm, p + "n2."))
            layers.append(LayerSpec(PartSpec(kind), parts))
        return ModelSpec(
            architecture="ToyParallelForCausalLM", vocab_size=vocab, hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=vocab, hidden_size=h), "embed."),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(3)),
            final_norm=PartSpec("rms_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=vocab, hidden_size=h, tied=True), "head."))

    def plain(w, tokens):
        """The same model in float64: the arrangement above, part by part."""
        w = {k: v.double() for k, v in w.items()}
        sizes = dict(num_heads=heads, num_kv_heads=kv_heads, head_dim=d)
        inv_freq = P.inverse_frequencies({"rope_type": "default", "theta": theta}, d)
        cos, sin = P.rope_cos_sin(inv_freq, torch.arange(len(tokens)), torch.float64)
        x = w["embed.weight"][torch.tensor(tokens)]
        for i, kind in enumerate(("toy_parallel", "pre_norm", "toy_parallel")):
            p = f"layers.{i}."
            if kind == "toy_parallel":
                n = P.rms_norm(x, w[p + "n.weight"], eps)
                x = x + P.attention_block(n, w, p + "attn.", sizes, cos, sin) + P.swiglu_mlp(n, w, p + "mlp.")
            else:
                x = x + P.attention_block(P.rms_norm(x, w[p + "n1.weight"], eps), w, p + "attn.", sizes, cos, sin)
                x = x + P.swiglu_mlp(P.rms_norm(x, w[p + "n2.weight"], eps), w, p + "mlp.")
        return P.linear(P.rms_norm(x, w["norm.weight"], eps), w["embed.weight"])

    register_architecture("ToyParallelForCausalLM", dict, build)
    try:
        from test_model_gpu import check

        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, {"architectures": ["ToyParallelForCausalLM"]}, seed=12, std=0.15,
                                        norm_jitter=0.1)
            _, weights = P.load_folder(folder)
            rng = torch.Generator().manual_seed(3)
            toks = {rid: torch.randint(0, vocab, (n,), generator=rng).tolist() for rid, n in (("a", 45), ("b", 23))}
            ref = {rid: plain(weights, t) for rid, t in toks.items()}
            model = load_model(folder, dtype=dtype)
            core = build_core(model, num_pages=12, page_size=16, max_seqs=4, enable_prefix_caching=False, watermark=0.0)
            core.step.enable_decode_graphs(4, 12 * 16)
            assert (core.step.graphs is not None) == (dtype == "bfloat16")
            s = TraceSession(core)
            for rid, t in toks.items():  # whole
                got = s.step([{"id": rid, "tokens": t, "want": list(range(len(t)))}], end=[rid])
                check(got, ref[rid], dtype, f"toy block, {rid} whole")
            # portions of changing size beside the other request's portions, then token by token together
            fed = {"a": 0, "b": 0}
            for plan in ({"a": 16}, {"a": 7, "b": 5}, {"a": 2, "b": 9}, {"a": 5, "b": 2}, {"a": 3}):
                entries = [{"id": rid, "tokens": toks[rid][fed[rid]:fed[rid] + n], "want": list(range(n))}
                           for rid, n in plan.items()]
                got = s.step(entries)
                want = torch.cat([ref[rid][fed[rid]:fed[rid] + n] for rid, n in plan.items()])
                check(got, want, dtype, f"toy block, portions {plan} at {fed}")
                for rid, n in plan.items():
                    fed[rid] += n
            assert model.native_runs == 0, "the loop in C knows the pre-norm arrangement only"
            while fed["b"] < len(toks["b"]):
                got = s.step([{"id": rid, "tokens": [toks[rid][fed[rid]]], "want": [0]} for rid in ("a", "b")])
                check(got, torch.stack([ref[rid][fed[rid]] for rid in ("a", "b")]), dtype, f"toy block, decode at {fed}")
                fed = {rid: n + 1 for rid, n in fed.items()}
            if dtype == "bfloat16":
                assert core.step.graphs.replays > 0
            core.manager.check_invariants()
    finally:
        unregister_architecture("ToyParallelForCausalLM")
        unregister_part("block", "toy_parallel")


def test_a_subclass_of_a_built_in_part_is_not_taken_for_it_by_the_loop_in_c():
    """The loop in C that issues a step's launches hard-codes what the built-in parts compute. A
    part that inherits from one of them and changes its arithmetic (here: attention whose output is
    halved) inherits ``native_fields`` too; it must not be run as its parent. The same weights in
    Llama's own arrangement go through the loop, and give other logits."""
    import dataclasses

    from dli_amd.architectures.llama import build_llama_spec
    from dli_amd.config import LlamaConfig, register_architecture, unregister_architecture
    from dli_amd.engine.core import build_core
    from dli_amd.parts import PartSpec, register_part, unregister_part
    from dli_amd.parts.attention import GQAttention
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model

    @register_part("mixer", "toy_halved_attention")
    class Halved(GQAttention):
        def forward(self, x, ctx, cache):
            return super().forward(x, ctx, cache) * 0.5

    def build(cfg):
        spec = build_llama_spec(cfg)
        layers = []
        for ls in spec.layers:
            family, mixer = ls.parts["mixer"]
            layers.append(dataclasses.replace(ls, parts={**ls.parts, "mixer": (
                family, dataclasses.replace(mixer, kind="toy_halved_attention"))}))
        return dataclasses.replace(spec, layers=tuple(layers))

    register_architecture("LlamaForCausalLM", LlamaConfig.from_hf_dict, build, model_types=("llama",), replace=True)
    try:
        halved = load_model(model_folder("D"), dtype="bfloat16")
    finally:
        register_architecture("LlamaForCausalLM", LlamaConfig.from_hf_dict, build_llama_spec, model_types=("llama",),
                              replace=True)
        unregister_part("mixer", "toy_halved_attention")
    plain_model = load_model(model_folder("D"), dtype="bfloat16")
    toks = list(range(3, 93))
    outs = []
    for model in (halved, plain_model):
        core = build_core(model, num_pages=8, page_size=16, max_seqs=2, enable_prefix_caching=False, watermark=0.0)
        outs.append(TraceSession(core).step([{"id": "r", "tokens": toks, "want": [89]}]).clone())
    assert halved.native_runs == 0 and plain_model.native_runs == 1
    assert not torch.allclose(outs[0], outs[1], atol=1e-3)


# ------------------------------------------------------------------ a toy norm

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_norm_is_registered_built_and_stepped(dtype):
    """Another norm, defined here and nowhere in the framework: a layer norm with mean, variance,
    weight and bias, as the three norms of a pre-norm model. It has no ``fused_params`` (the fused
    decode kernels and the loop in C compute an RMS norm), so every step must take the parts' plain
    ``forward``; its ``forward(x, delta)`` makes the residual sum in place as the interface asks.
    Whole, in portions, mixed and token by token against a plain float64 model."""
    import tempfile
    from typing import Mapping, Optional

    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.engine.core import build_core
    from dli_amd.parts import LayerSpec, ModelSpec, Norm, PartSpec, ScheduleEntry, WeightSpec, register_part, unregister_part
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model, write_random_model

    @register_part("norm", "toy_layer_norm")
    class ToyLayerNorm(Norm):
        def __init__(self, runtime, *, width: int, eps: float) -> None:
            super().__init__(runtime)
            self.width, self.eps = width, eps
            self.w = self.b = None

        def weight_specs(self):
            return {"weight": WeightSpec((self.width,), role="float32", init="norm"),
                    "bias": WeightSpec((self.width,), role="float32")}

        def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
            self.w, self.b = tensors["weight"], tensors["bias"]

        def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
            if delta is not None:
                x.copy_((x.float() + delta.float()).to(x.dtype))  # the residual sum, in place, 32-bit
            h = x.float()
            h = (h - h.mean(-1, keepdim=True)) * torch.rsqrt(h.var(-1, unbiased=False, keepdim=True) + self.eps)
            return (h * self.w + self.b).to(x.dtype)

    h, heads, kv_heads, d, inter, vocab, eps, theta, n_layers = 40, 2, 2, 16, 56, 45, 1e-5, 10000.0, 2

    def build(cfg):
        norm = dict(width=h, eps=eps)
        pos = PartSpec("rotary", dict(dim=d, theta=theta))
        layers = []
        for i in range(n_layers):
            p = f"layers.{i}."
            layers.append(LayerSpec(PartSpec("pre_norm"), {
                "mixer_norm": ("norm", PartSpec("toy_layer_norm", norm, p + "n1.")),
                "mixer": ("mixer", PartSpec("gqa_attention", dict(hidden_size=h, num_heads=heads, num_kv_heads=kv_heads,
                                                                 head_dim=d, position=pos), p + "attn.")),
                "feed_forward_norm": ("norm", PartSpec("toy_layer_norm", norm, p + "n2.")),
                "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=inter), p + "mlp."))}))
        return ModelSpec(
            architecture="ToyLayerNormForCausalLM", vocab_size=vocab, hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=vocab, hidden_size=h), "embed."),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(n_layers)),
            final_norm=PartSpec("toy_layer_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=vocab, hidden_size=h, tied=False), "head."))

    def layer_norm(x, w, b):
        return (x - x.mean(-1, keepdim=True)) / torch.sqrt(x.var(-1, unbiased=False, keepdim=True) + eps) * w + b

    def plain(w, tokens):
        w = {k: v.double() for k, v in w.items()}
        sizes = dict(num_heads=heads, num_kv_heads=kv_heads, head_dim=d)
        cos, sin = P.rope_cos_sin(P.inverse_frequencies({"rope_type": "default", "theta": theta}, d),
                                  torch.arange(len(tokens)), torch.float64)
        x = w["embed.weight"][torch.tensor(tokens)]
        for i in range(n_layers):
            p = f"layers.{i}."
            x = x + P.attention_block(layer_norm(x, w[p + "n1.weight"], w[p + "n1.bias"]), w, p + "attn.", sizes, cos, sin)
            x = x + P.swiglu_mlp(layer_norm(x, w[p + "n2.weight"], w[p + "n2.bias"]), w, p + "mlp.")
        return P.linear(layer_norm(x, w["norm.weight"], w["norm.bias"]), w["head.weight"])

    register_architecture("ToyLayerNormForCausalLM", dict, build)
    try:
        from test_model_gpu import check

        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, {"architectures": ["ToyLayerNormForCausalLM"]}, seed=14, std=0.2,
                                        norm_jitter=0.1)
            _, weights = P.load_folder(folder)
            rng = torch.Generator().manual_seed(4)
            toks = {rid: torch.randint(0, vocab, (n,), generator=rng).tolist() for rid, n in (("a", 41), ("b", 19))}
            ref = {rid: plain(weights, t) for rid, t in toks.items()}
            model = load_model(folder, dtype=dtype)
            core = build_core(model, num_pages=10, page_size=8, max_seqs=4, enable_prefix_caching=False, watermark=0.0)
            core.step.enable_decode_graphs(4, 80)
            assert core.step.graphs is None, "a part that does not say so is not recorded into graphs"
            s = TraceSession(core)
            for rid, t in toks.items():
                got = s.step([{"id": rid, "tokens": t, "want": list(range(len(t)))}], end=[rid])
                check(got, ref[rid], dtype, f"toy norm, {rid} whole")
            fed = {"a": 0, "b": 0}
            for plan in ({"a": 13}, {"a": 7, "b": 5}, {"a": 2, "b": 9}, {"a": 5, "b": 2}):
                entries = [{"id": rid, "tokens": toks[rid][fed[rid]:fed[rid] + n], "want": list(range(n))}
                           for rid, n in plan.items()]
                got = s.step(entries)
                check(got, torch.cat([ref[rid][fed[rid]:fed[rid] + n] for rid, n in plan.items()]), dtype,
                      f"toy norm, portions {plan} at {fed}")
                for rid, n in plan.items():
                    fed[rid] += n
            while fed["b"] < len(toks["b"]):
                got = s.step([{"id": rid, "tokens": [toks[rid][fed[rid]]], "want": [0]} for rid in ("a", "b")])
                check(got, torch.stack([ref[rid][fed[rid]] for rid in ("a", "b")]), dtype, f"toy norm, decode at {fed}")
                fed = {rid: n + 1 for rid, n in fed.items()}
            assert model.native_runs == 0
            core.manager.check_invariants()
    finally:
        unregister_architecture("ToyLayerNormForCausalLM")
        unregister_part("norm", "toy_layer_norm")
