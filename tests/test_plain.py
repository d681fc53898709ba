"""Pins of the plain implementation beside the reference's text: library routines that special
cases reduce to, invariants, and vectors from the reference's own tests. Each is chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, a wrong band) fails it.
"""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
from tiny_configs import TINY_A, TINY_B, TINY_C, model_folder

torch.manual_seed(0)
F64 = torch.float64


# ------------------------------------------------------------------ rotary frequencies

def test_default_frequencies_are_the_geometric_progression():
    f = P.inverse_frequencies({"theta": 10000.0, "rope_type": "default"}, 16)
    assert f.dtype == torch.float32 and f.shape == (8,)
    assert f[0] == 1.0
    for i in range(8):
        assert abs(f[i].item() - 10000.0 ** (-2 * i / 16)) < 1e-7


def test_linear_divides_and_llama3_with_factor_one_is_default():
    base = P.inverse_frequencies({"theta": 5e5, "rope_type": "default"}, 32)
    lin = P.inverse_frequencies({"theta": 5e5, "rope_type": "linear", "factor": 2.0}, 32)
    assert torch.allclose(lin, base / 2)
    same = P.inverse_frequencies({"theta": 5e5, "rope_type": "llama3", "factor": 1.0, "low_freq_factor": 1.0,
                                  "high_freq_factor": 4.0, "original_max_position_embeddings": 64}, 32)
    assert torch.allclose(same, base, rtol=1e-6)


def test_llama3_bands_of_config_b():
    """Original context 64, low 1, high 4: wavelengths under 16 stay, over 64 are divided by 8,
    between they blend, continuously at both ends."""
    rope = P.rope_settings(TINY_B)
    base = P.inverse_frequencies({"theta": rope["theta"], "rope_type": "default"}, 32).double()
    got = P.inverse_frequencies(rope, 32).double()
    wavelen = 2 * math.pi / base
    assert (wavelen < 16).any() and (wavelen > 64).any() and ((wavelen >= 16) & (wavelen <= 64)).any()
    for b, g, wl in zip(base.tolist(), got.tolist(), wavelen.tolist()):
        if wl < 16:
            assert g == pytest.approx(b, rel=1e-6)
        elif wl > 64:
            assert g == pytest.approx(b / 8, rel=1e-6)
        else:
            s = (64 / wl - 1) / (4 - 1)
            assert g == pytest.approx((1 - s) * b / 8 + s * b, rel=1e-5)
            assert b / 8 <= g <= b
    # continuity: at the band edges the blend meets its neighbours
    edge = lambda wl: (1 - (64 / wl - 1) / 3) / 8 + (64 / wl - 1) / 3
    assert edge(16.0) == pytest.approx(1.0) and edge(64.0) == pytest.approx(1 / 8)


def test_rope_settings_defaults_and_precedence():
    assert P.rope_settings({})["theta"] == 10000.0
    r = P.rope_settings({"rope_scaling": {"type": "linear", "factor": 2}, "rope_theta": 7.0})
    assert r["rope_type"] == "linear" and r["theta"] == 7.0
    r = P.rope_settings({"max_position_embeddings": 99, "rope_scaling": {"rope_type": "llama3", "factor": 8},
                         "rope_parameters": {"rope_theta": 3.0}})
    assert r["theta"] == 3.0 and r["original_max_position_embeddings"] == 99
    assert (r["low_freq_factor"], r["high_freq_factor"]) == (1.0, 4.0)


# ------------------------------------------------------------------ rotation

def test_rotation_is_the_complex_product_on_pairs_i_and_i_plus_half():
    d, n = 16, 5
    inv = P.inverse_frequencies({"theta": 10000.0, "rope_type": "default"}, d)
    pos = torch.tensor([0, 1, 2, 7, 100])
    cos, sin = P.rope_cos_sin(inv, pos, F64)
    x = torch.randn(3, n, d, dtype=F64)
    y = P.apply_rope(x, cos, sin)
    z = torch.complex(x[..., :d // 2], x[..., d // 2:]) * torch.polar(
        torch.ones(n, d // 2, dtype=F64), pos.double()[:, None] * inv.double()[None, :])
    assert torch.allclose(y[..., :d // 2], z.real, atol=1e-6) and torch.allclose(y[..., d // 2:], z.imag, atol=1e-6)
    assert torch.equal(y[:, 0], x[:, 0])  # position 0 is the identity
    pair_norm = lambda t: t[..., :d // 2] ** 2 + t[..., d // 2:] ** 2
    assert torch.allclose(pair_norm(y), pair_norm(x), atol=1e-9)
    # adjacent pairing (2i, 2i+1) would be a different function
    adj = x.clone()
    z2 = torch.view_as_complex(x.reshape(3, n, d // 2, 2).contiguous()) * torch.polar(
        torch.ones(n, d // 2, dtype=F64), pos.double()[:, None] * inv.double()[None, :])
    assert not torch.allclose(torch.view_as_real(z2).reshape(3, n, d), y, atol=1e-3)


def test_scores_depend_on_distance_only():
    d = 32
    inv = P.inverse_frequencies(P.rope_settings(TINY_B), d)
    q, k = torch.randn(1, 1, d, dtype=F64), torch.randn(1, 1, d, dtype=F64)
    def score(m, n):
        cq, sq = P.rope_cos_sin(inv, torch.tensor([m]), F64)
        ck, sk = P.rope_cos_sin(inv, torch.tensor([n]), F64)
        return (P.apply_rope(q, cq, sq) * P.apply_rope(k, ck, sk)).sum().item()
    assert score(5, 3) == pytest.approx(score(105, 103), abs=1e-4)
    assert score(5, 3) != pytest.approx(score(3, 5), abs=1e-3)  # the sign of the distance counts


# ------------------------------------------------------------------ norm, attention, feed-forward

def test_rms_norm_against_the_library_and_its_properties():
    x, w = torch.randn(4, 50, dtype=F64) * 3, torch.randn(50, dtype=F64)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (50,), w, 1e-5), atol=1e-12)
    ones = torch.ones(50, dtype=F64)
    y = P.rms_norm(x, ones, 1e-5)
    ms = x.pow(2).mean(-1)
    assert torch.allclose(y.pow(2).mean(-1), ms / (ms + 1e-5), atol=1e-12)  # eps inside the root
    assert torch.allclose(P.rms_norm(7 * x, w, 0.0), P.rms_norm(x, w, 0.0), atol=1e-9)
    tiny = x * 1e-4
    assert not torch.allclose(P.rms_norm(tiny, w, 1e-5), P.rms_norm(tiny, w, 1e-6), rtol=1e-2)
    assert not torch.allclose(P.rms_norm(x, w, 1e-5), (x - x.mean(-1, keepdim=True)) /
                              x.std(-1, keepdim=True) * w, atol=1e-2)  # not a layer norm


def test_attention_reduces_to_the_library_routine():
    heads, kvh, n, d = 6, 2, 9, 8
    q, k, v = torch.randn(heads, n, d, dtype=F64), torch.randn(kvh, n, d, dtype=F64), torch.randn(kvh, n, d, dtype=F64)
    lib = F.scaled_dot_product_attention(q, k.repeat_interleave(3, 0), v.repeat_interleave(3, 0), is_causal=True)
    assert torch.allclose(P.causal_attention(q, k, v), lib, atol=1e-12)
    # grouping is contiguous: head h reads kv head h // 3, not h % 2
    wrong = F.scaled_dot_product_attention(q, k.repeat(3, 1, 1), v.repeat(3, 1, 1), is_causal=True)
    assert not torch.allclose(P.causal_attention(q, k, v), wrong, atol=1e-3)
    one = P.causal_attention(q[:, :1], k[:, :1], v[:, :1])  # a single key: the output is its value
    assert torch.allclose(one, v[:, :1].repeat_interleave(3, 0), atol=1e-12)
    same_k = k[:, :1].expand(kvh, n, d)  # equal keys: the running mean of the values
    mean = P.causal_attention(q, same_k, v)
    assert torch.allclose(mean[0, 3], v[0, :4].mean(0), atol=1e-12)
    mha = P.causal_attention(q[:2], k, v)  # as many kv heads as heads
    assert torch.allclose(mha, F.scaled_dot_product_attention(q[:2], k, v, is_causal=True), atol=1e-12)


def test_swiglu_against_the_library_and_its_limits():
    h, i = 12, 20
    w = {"gate_proj.weight": torch.randn(i, h, dtype=F64), "up_proj.weight": torch.randn(i, h, dtype=F64),
         "down_proj.weight": torch.randn(h, i, dtype=F64)}
    x = torch.randn(5, h, dtype=F64)
    lib = F.linear(F.silu(F.linear(x, w["gate_proj.weight"])) * F.linear(x, w["up_proj.weight"]), w["down_proj.weight"])
    assert torch.allclose(P.swiglu_mlp(x, w, ""), lib, atol=1e-10)
    assert P.silu(torch.tensor(0.0)) == 0 and P.silu(torch.tensor(40.0, dtype=F64)) == pytest.approx(40.0)
    swapped = {**w, "gate_proj.weight": w["up_proj.weight"], "up_proj.weight": w["gate_proj.weight"]}
    assert not torch.allclose(P.swiglu_mlp(x, swapped, ""), lib, atol=1e-3)  # gate and up are not symmetric


# ------------------------------------------------------------------ whole model

@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_properties(name):
    cfg, w = P.load_folder(model_folder(name))
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5]
    logits = P.forward_logits(w, cfg, toks)
    assert logits.shape == (len(toks), cfg["vocab_size"])
    # causal: a prefix gives the same logits at its positions
    assert torch.allclose(P.forward_logits(w, cfg, toks[:6]), logits[:6], atol=1e-9)
    # head: tied models read the embedding, untied ones their own matrix
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    assert ("lm_head.weight" in w) == (not cfg["tie_word_embeddings"])
    # a shift of all positions changes nothing where only distances count (default and linear rope)
    shifted = P.forward_logits(w, cfg, toks, first_position=37)
    if name in ("A", "C"):
        assert torch.allclose(shifted, logits, atol=1e-4)
    # float32 evaluation tracks float64
    assert (P.forward_logits(w, cfg, toks, dtype=torch.float32).double() - logits).abs().max() < 1e-4
    assert head.shape == (cfg["vocab_size"], cfg["hidden_size"])


# ------------------------------------------------------------------ layer composition
# The arrangement of a block (which norm feeds which branch, where the two sums sit, the final norm
# and the head; model/llama.py:194-213,299-305) pinned by library routines and by what a wrong
# arrangement would change.

def _library_rotate(x, positions, inv_freq):
    """Rotation of ``x [heads, n, d]`` written as a complex product on pairs (i, i + d/2)."""
    half = x.shape[-1] // 2
    z = torch.complex(x[..., :half], x[..., half:]) * torch.polar(
        torch.ones(len(positions), half, dtype=x.dtype), positions[:, None].to(x.dtype) * inv_freq.to(x.dtype))
    return torch.cat([z.real, z.imag], dim=-1)


def _library_layer(h, w, i, cfg, positions):
    """One block composed from library routines, every sum written out."""
    s = P.model_sizes(cfg)
    nh, nkv, d, eps = s["num_heads"], s["num_kv_heads"], s["head_dim"], s["eps"]
    n, p = h.shape[0], f"model.layers.{i}."
    inv_freq = P.inverse_frequencies(P.rope_settings(cfg), d)
    a = F.rms_norm(h, (h.shape[-1],), w[p + "input_layernorm.weight"], eps)
    q = F.linear(a, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias"))
    k = F.linear(a, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias"))
    v = F.linear(a, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
    q = _library_rotate(q.view(n, nh, d).transpose(0, 1), positions, inv_freq)
    k = _library_rotate(k.view(n, nkv, d).transpose(0, 1), positions, inv_freq)
    v = v.view(n, nkv, d).transpose(0, 1)
    k, v = (t.repeat_interleave(nh // nkv, dim=0) for t in (k, v))
    o = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    o = F.linear(o.transpose(0, 1).reshape(n, nh * d), w[p + "self_attn.o_proj.weight"],
                 w.get(p + "self_attn.o_proj.bias"))
    h = h + o
    m = F.rms_norm(h, (h.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
    gate = F.linear(m, w[p + "mlp.gate_proj.weight"], w.get(p + "mlp.gate_proj.bias"))
    up = F.linear(m, w[p + "mlp.up_proj.weight"], w.get(p + "mlp.up_proj.bias"))
    return h + F.linear(F.silu(gate) * up, w[p + "mlp.down_proj.weight"], w.get(p + "mlp.down_proj.bias"))


def _without_branches(w, keep=()):
    """The weights with every layer's o_proj and down_proj (and their biases) zeroed, except the
    layers in ``keep``: such a layer adds nothing to the residual stream."""
    out = dict(w)
    for name, t in w.items():
        if ("o_proj" in name or "down_proj" in name) and not any(f"layers.{i}." in name for i in keep):
            out[name] = torch.zeros_like(t)
    return out


def _head(w, cfg):
    return w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_dead_branches_leave_embedding_final_norm_and_head(name):
    cfg, w = P.load_folder(model_folder(name))
    w = {k: t.to(F64) for k, t in w.items()}
    toks = [7, 2, 9, 9, 30, 1, 17]
    dead = _without_branches(w)
    e = w["model.embed_tokens.weight"][torch.tensor(toks)]
    want = F.linear(F.rms_norm(e, (e.shape[-1],), w["model.norm.weight"], cfg["rms_norm_eps"]), _head(w, cfg))
    got = P.forward_logits(dead, cfg, toks)
    assert torch.allclose(got, want, atol=1e-10)
    # the final norm is there: a scale of the embedding rows cancels (up to eps) ...
    scaled = dict(dead)
    scaled["model.embed_tokens.weight"] = dead["model.embed_tokens.weight"] * 3.0
    if not cfg["tie_word_embeddings"]:
        assert torch.allclose(P.forward_logits(scaled, cfg, toks), got, rtol=2e-3, atol=1e-3)
        assert not torch.allclose(P.forward_logits(scaled, cfg, toks), 3.0 * got, rtol=2e-3, atol=1e-3)
    else:  # ... and with a tied head it is the head that scales
        assert torch.allclose(P.forward_logits(scaled, cfg, toks), 3.0 * got, rtol=2e-3, atol=1e-3)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_one_live_layer_equals_the_library_composition(name):
    cfg, w = P.load_folder(model_folder(name))
    w = {k: t.to(F64) for k, t in w.items()}
    toks = [4, 250, 3, 3, 91, 18, 5, 77, 6]
    positions = torch.arange(len(toks))
    e = w["model.embed_tokens.weight"][torch.tensor(toks)]
    for i in range(cfg["num_hidden_layers"]):
        live = _without_branches(w, keep=(i,))
        h = _library_layer(e, live, i, cfg, positions)
        want = F.linear(F.rms_norm(h, (h.shape[-1],), w["model.norm.weight"], cfg["rms_norm_eps"]), _head(w, cfg))
        got = P.forward_logits(live, cfg, toks)
        assert torch.allclose(got, want, atol=1e-6), (name, i)
        assert not torch.allclose(got, P.forward_logits(_without_branches(w), cfg, toks), atol=1e-3)
    # all layers live: the blocks chained (the plain rotation takes its angles in 32-bit as the
    # reference does, rope.py:58-60; the library composition here takes them in 64-bit)
    h = e
    for i in range(cfg["num_hidden_layers"]):
        h = _library_layer(h, w, i, cfg, positions)
    want = F.linear(F.rms_norm(h, (h.shape[-1],), w["model.norm.weight"], cfg["rms_norm_eps"]), _head(w, cfg))
    assert torch.allclose(P.forward_logits(w, cfg, toks), want, atol=1e-6)


@pytest.mark.parametrize("name", ["A", "B"])
def test_each_norm_feeds_its_own_branch(name):
    cfg, w = P.load_folder(model_folder(name))
    toks = [4, 250, 3, 3, 91, 18]
    base = P.forward_logits(w, cfg, toks)
    a, b = "model.layers.0.input_layernorm.weight", "model.layers.0.post_attention_layernorm.weight"
    swapped = dict(w)
    swapped[a], swapped[b] = w[b], w[a]
    assert (P.forward_logits(swapped, cfg, toks) - base).abs().max() > 1e-3
    # with the feed-forward dead, only the norm before the attention matters, and the other way round
    for dead, silent, heard in (("down_proj", b, a), ("o_proj", a, b)):
        part = {k: (torch.zeros_like(t) if f"layers.0." in k and dead in k else t) for k, t in w.items()}
        ref = P.forward_logits(part, cfg, toks)
        for which, changes in ((silent, False), (heard, True)):
            mod = dict(part)
            mod[which] = part[which] * 1.5
            assert ((P.forward_logits(mod, cfg, toks) - ref).abs().max() > 1e-3) == changes, (dead, which)


def test_greedy_generation_recomputes_and_breaks_ties_low():
    cfg, w = P.load_folder(model_folder("A"))
    out = P.greedy_generate(w, cfg, [5, 6, 7], 6)
    assert len(out) == 6
    logits = P.forward_logits(w, cfg, [5, 6, 7] + out[:3])
    assert int(torch.argmax(logits[-1])) == out[3]
    assert int(torch.argmax(torch.tensor([0.1, 2.0, 2.0, -1.0]))) == 1


# ------------------------------------------------------------------ sampling distribution

def test_sampling_probabilities_vectors():
    """tests/unit/test_sampling.py:13-44 of the reference."""
    logits = torch.log(torch.tensor([0.5, 0.3, 0.15, 0.05]))
    p = P.sampling_probabilities(logits, 1.0, -1, 1.0)
    assert torch.allclose(p, torch.tensor([0.5, 0.3, 0.15, 0.05], dtype=F64), atol=1e-7)
    pk = P.sampling_probabilities(logits, 1.0, 2, 1.0)
    assert pk[2] == 0 and pk[3] == 0 and pk[0] == pytest.approx(0.625)
    pp = P.sampling_probabilities(logits, 1.0, -1, 0.6)
    assert set(torch.nonzero(pp).flatten().tolist()) == {0, 1}  # preceding mass 0 and 0.5 < 0.6
    assert torch.nonzero(P.sampling_probabilities(logits, 1.0, -1, 1e-6)).flatten().tolist() == [0]
    hot = P.sampling_probabilities(logits, 0.5, -1, 1.0)
    assert hot[0] == pytest.approx(0.25 / (0.25 + 0.09 + 0.0225 + 0.0025))
