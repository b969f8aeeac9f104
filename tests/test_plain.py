"""Pins of the plain implementation: what fixes each formula besides reading the reference.

Each check is chosen so that a plausible mistake fails it: a wrong sign or pairing in the
rotation, a norm in the wrong place or with 1 + w, a head grouping by modulo, a swapped gate.
"""

import math

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from conftest import TINY_A, TINY_B

F64 = torch.float64


def rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=F64) * scale


def test_rms_norm_is_the_library_routine():
    x, w = rand(5, 64, seed=1, scale=3.0), rand(64, seed=2)
    got = plain.rms_norm(x, w, 1e-6)
    want = torch.nn.functional.rms_norm(x, (64,), w, 1e-6)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    # the weight is plain w, not 1 + w: with w = 1 rows have mean square 1
    ones = plain.rms_norm(x, torch.ones(64, dtype=F64), 1e-12)
    assert torch.allclose((ones * ones).mean(-1), torch.ones(5, dtype=F64), atol=1e-9)
    # eps sits inside the square root: a zero row stays zero and finite
    assert torch.equal(plain.rms_norm(torch.zeros(1, 8, dtype=F64), torch.ones(8, dtype=F64), 1e-5),
                       torch.zeros(1, 8, dtype=F64))


def test_rope_formula_identity_and_pairing():
    # vectors of the reference's test: tests/backend/test_cpu_ops.cpp:50-74 (2 heads of 8, positions 0 and 7)
    heads, dim, theta = 2, 8, 10000.0
    x = rand(2, heads, dim, seed=4)
    out = plain.rope_neox(x, [0, 7], theta)
    assert torch.allclose(out[0], x[0], atol=1e-12)                    # position 0 is the identity
    for h in range(heads):
        for i in range(dim // 2):
            angle = 7.0 * theta ** (-2.0 * i / dim)
            x1, x2 = float(x[1, h, i]), float(x[1, h, i + dim // 2])    # pairs (i, i + d/2), not (2i, 2i+1)
            assert float(out[1, h, i]) == pytest.approx(x1 * math.cos(angle) - x2 * math.sin(angle), rel=1e-5, abs=1e-6)
            assert float(out[1, h, i + dim // 2]) == pytest.approx(x2 * math.cos(angle) + x1 * math.sin(angle), rel=1e-5, abs=1e-6)
    # a rotation keeps the length of every pair
    assert torch.allclose(out.norm(dim=-1), x.norm(dim=-1), atol=1e-9)


def test_rope_scores_depend_on_distance_only():
    # tests/backend/test_cpu_ops.cpp:76-90: score(5, 3) == score(12, 10)
    q0, k0 = rand(1, 1, 8, seed=5), rand(1, 1, 8, seed=6)

    def score(qp, kp):
        return float((plain.rope_neox(q0, [qp], 10000.0) * plain.rope_neox(k0, [kp], 10000.0)).sum())

    assert score(5, 3) == pytest.approx(score(12, 10), rel=1e-4)
    assert abs(score(5, 3) - score(5, 4)) > 1e-3                        # and it does depend on the distance


def test_inv_freq_is_float32_of_the_formula():
    f = plain.rope_inv_freq(1e6, 32)
    assert f.dtype == np.float32 and f[0] == 1.0
    assert f[5] == pytest.approx(1e6 ** (-10 / 32), rel=1e-6)


def test_attention_without_mask_or_rotation_is_softmax_attention():
    # The last row of a causal pass sees every key: it must equal plain softmax attention.
    T, H, Dh = 9, 4, 16
    q, k, v = rand(T, H, Dh, seed=7), rand(T, H, Dh, seed=8), rand(T, H, Dh, seed=9)
    out = plain.causal_attention(q, k, v, 0.25)
    for h in range(H):
        p = torch.softmax(0.25 * (q[-1, h] @ k[:, h].T), dim=-1)
        assert torch.allclose(out[-1, h], p @ v[:, h], atol=1e-12)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True, scale=0.25).transpose(0, 1)
    assert torch.allclose(out, lib, atol=1e-10)
    # the first row sees only itself
    assert torch.allclose(out[0], v[0], atol=1e-12)


def test_attention_head_grouping_and_constant_values():
    T, H, KVH, Dh = 6, 6, 2, 8
    q, k, v = rand(T, H, Dh, seed=10), rand(T, KVH, Dh, seed=11), rand(T, KVH, Dh, seed=12)
    out = plain.causal_attention(q, k, v, 0.3)
    # consecutive groups of H / KVH query heads share a KV head: repeat_interleave, not repeat
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.repeat_interleave(3, 1).transpose(0, 1), v.repeat_interleave(3, 1).transpose(0, 1),
        is_causal=True, scale=0.3).transpose(0, 1)
    assert torch.allclose(out, lib, atol=1e-10)
    wrong = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.repeat(1, 3, 1).transpose(0, 1), v.repeat(1, 3, 1).transpose(0, 1),
        is_causal=True, scale=0.3).transpose(0, 1)
    assert not torch.allclose(out, wrong, atol=1e-3)
    # probabilities sum to one: constant values come back unchanged
    const = torch.full_like(v, 0.7)
    assert torch.allclose(plain.causal_attention(q, k, const, 0.3), torch.full_like(q, 0.7), atol=1e-12)


def test_attention_window_limits_the_keys():
    T, H, Dh = 10, 2, 8
    q, k, v = rand(T, H, Dh, seed=13), rand(T, H, Dh, seed=14), rand(T, H, Dh, seed=15)
    out = plain.causal_attention(q, k, v, 0.5, window=3)
    t = 7
    p = torch.softmax(0.5 * (q[t, 0] @ k[t - 2:t + 1, 0].T), dim=-1)    # keys t-2 .. t
    assert torch.allclose(out[t, 0], p @ v[t - 2:t + 1, 0], atol=1e-12)
    assert torch.allclose(plain.causal_attention(q, k, v, 0.5, window=T), plain.causal_attention(q, k, v, 0.5))


@pytest.mark.parametrize("window", [None, 1, 4, 9])
def test_attention_tail_is_the_last_rows_of_the_whole(window):
    T, H, KVH, Dh, n = 23, 6, 2, 8, 5
    q, k, v = rand(T, H, Dh, seed=31), rand(T, KVH, Dh, seed=32), rand(T, KVH, Dh, seed=33)
    whole = plain.causal_attention(q, k, v, 0.4, window)
    assert torch.allclose(plain.causal_attention_tail(q[-n:], k, v, 0.4, window), whole[-n:], atol=1e-12)
    assert torch.allclose(plain.causal_attention_tail(q[-1:], k, v, 0.4, window), whole[-1:], atol=1e-12)


def test_swiglu_is_silu_times_up():
    h = rand(3, 16, seed=16)
    wg, wu, wd = rand(24, 16, seed=17), rand(24, 16, seed=18), rand(16, 24, seed=19)
    got = plain.swiglu(h, wg, wu, wd)
    want = (torch.nn.functional.silu(h @ wg.T) * (h @ wu.T)) @ wd.T
    assert torch.allclose(got, want, atol=1e-12)
    swapped = plain.swiglu(h, wu, wg, wd)
    assert not torch.allclose(got, swapped, atol=1e-3)
    # one value by hand: src/backend/cpu/cpu_backend.cpp:205 gate / (1 + exp(-gate)) * up
    one = plain.swiglu(torch.tensor([[1.0]], dtype=F64), torch.tensor([[2.0]], dtype=F64),
                       torch.tensor([[3.0]], dtype=F64), torch.tensor([[1.0]], dtype=F64))
    assert float(one) == pytest.approx(2.0 / (1 + math.exp(-2.0)) * 3.0)


def _weights(cfg, seed):
    from tie_amd.models import expected_tensors_for_config
    from tie_amd.weights.random_init import random_tensors

    specs = [s for s in expected_tensors_for_config(cfg) if not s.optional]
    return {n: t.to(F64) for n, t in random_tensors(specs, seed, torch.float32)}


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B], ids=["A", "B"])
def test_whole_model_properties(cfg):
    w = _weights(cfg, 3)
    tokens = [(i * 7 + 3) % cfg["vocab_size"] for i in range(12)]
    logits = plain.forward(w, cfg, tokens)
    assert logits.shape == (12, cfg["vocab_size"])
    # causality: a prefix gives the same logits at its positions
    assert torch.allclose(plain.forward(w, cfg, tokens[:7]), logits[:7], atol=1e-10)
    # the q/k norm sits before the rotation and matters: scaling q_norm's weight changes the logits,
    # scaling q_proj does not (a per-head RMSNorm removes the scale of its input)
    w2 = dict(w)
    w2["model.layers.0.self_attn.q_proj.weight"] = w["model.layers.0.self_attn.q_proj.weight"] * 3.0
    assert torch.allclose(plain.forward(w2, cfg, tokens), logits, atol=1e-4)
    w3 = dict(w)
    w3["model.layers.0.self_attn.q_norm.weight"] = w["model.layers.0.self_attn.q_norm.weight"] * 3.0
    assert not torch.allclose(plain.forward(w3, cfg, tokens), logits, atol=1e-4)
    # tied or separate head
    if cfg["tie_word_embeddings"]:
        assert "lm_head.weight" not in w
    else:
        w4 = dict(w)
        w4["lm_head.weight"] = w["lm_head.weight"] * 2.0
        assert torch.allclose(plain.forward(w4, cfg, tokens), logits * 2.0, atol=1e-9)


def test_one_layer_one_head_by_hand():
    """A one-layer, one-head model written out with library calls only."""
    cfg = {"num_hidden_layers": 1, "hidden_size": 8, "num_attention_heads": 1, "num_key_value_heads": 1,
           "head_dim": 8, "intermediate_size": 12, "vocab_size": 10, "rope_theta": 100.0, "rms_norm_eps": 1e-5,
           "tie_word_embeddings": True, "max_position_embeddings": 16}
    w = {"model.embed_tokens.weight": rand(10, 8, seed=30),
         "model.layers.0.input_layernorm.weight": rand(8, seed=31).abs() + 0.5,
         "model.layers.0.self_attn.q_proj.weight": rand(8, 8, seed=32), "model.layers.0.self_attn.k_proj.weight": rand(8, 8, seed=33),
         "model.layers.0.self_attn.v_proj.weight": rand(8, 8, seed=34), "model.layers.0.self_attn.o_proj.weight": rand(8, 8, seed=35),
         "model.layers.0.self_attn.q_norm.weight": rand(8, seed=36).abs() + 0.5, "model.layers.0.self_attn.k_norm.weight": rand(8, seed=37).abs() + 0.5,
         "model.layers.0.post_attention_layernorm.weight": rand(8, seed=38).abs() + 0.5,
         "model.layers.0.mlp.gate_proj.weight": rand(12, 8, seed=39), "model.layers.0.mlp.up_proj.weight": rand(12, 8, seed=40),
         "model.layers.0.mlp.down_proj.weight": rand(8, 12, seed=41), "model.norm.weight": rand(8, seed=42).abs() + 0.5}
    tokens = [3, 1, 4, 1, 5]
    F = torch.nn.functional
    x = w["model.embed_tokens.weight"][tokens]
    h = F.rms_norm(x, (8,), w["model.layers.0.input_layernorm.weight"], 1e-5)
    q = F.rms_norm(h @ w["model.layers.0.self_attn.q_proj.weight"].T, (8,), w["model.layers.0.self_attn.q_norm.weight"], 1e-5)
    k = F.rms_norm(h @ w["model.layers.0.self_attn.k_proj.weight"].T, (8,), w["model.layers.0.self_attn.k_norm.weight"], 1e-5)
    v = h @ w["model.layers.0.self_attn.v_proj.weight"].T

    def rot(t):  # rotate-half with complex numbers: (x1 + i x2) * e^{i angle}
        ang = torch.arange(5, dtype=F64)[:, None] * (100.0 ** (-torch.arange(4, dtype=F64) / 4))[None, :]
        z = torch.complex(t[:, :4], t[:, 4:]) * torch.polar(torch.ones_like(ang), ang)
        return torch.cat([z.real, z.imag], dim=-1)

    a = F.scaled_dot_product_attention(rot(q)[None], rot(k)[None], v[None], is_causal=True, scale=8 ** -0.5)[0]
    x = x + a @ w["model.layers.0.self_attn.o_proj.weight"].T
    h = F.rms_norm(x, (8,), w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
    x = x + (F.silu(h @ w["model.layers.0.mlp.gate_proj.weight"].T) * (h @ w["model.layers.0.mlp.up_proj.weight"].T)) @ w["model.layers.0.mlp.down_proj.weight"].T
    want = F.rms_norm(x, (8,), w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    got = plain.forward(w, cfg, tokens)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_mersenne_twister_known_value():
    # The C++ standard fixes the 10000th output of a default-seeded mt19937_64.
    rng = plain.MT19937_64(5489)
    for _ in range(9999):
        rng()
    assert rng() == 9981545732273789042


def test_plain_sampler_vectors_of_the_reference():
    # tests/sampling/test_sampler.cpp:27-178
    rng = plain.MT19937_64(0)
    assert plain.sample([0.1, 2.0, -1.0], 0.0, 0, 1.0, rng) == 1
    assert plain.sample([3.0, 1.0, 3.0], 0.0, 0, 1.0, rng) == 0
    logits = [math.log(0.7), math.log(0.2), math.log(0.1)]

    def freq(seed, draws, **kw):
        r = plain.MT19937_64(seed)
        f = [0.0] * 3
        for _ in range(draws):
            f[plain.sample(logits, 1.0, kw.get("top_k", 0), kw.get("top_p", 1.0), r)] += 1.0 / draws
        return f

    f = freq(42, 20000)
    assert f[0] == pytest.approx(0.7, rel=0.03) and f[1] == pytest.approx(0.2, rel=0.1) and f[2] == pytest.approx(0.1, rel=0.15)
    f = freq(7, 5000, top_k=2)
    assert f[2] == 0.0 and f[0] == pytest.approx(0.7 / 0.9, rel=0.05)
    f = freq(7, 5000, top_p=0.75)
    assert f[2] == 0.0 and f[1] > 0.0
    f = freq(7, 500, top_p=0.01)
    assert f[0] == pytest.approx(1.0) and f[1] == 0.0
    assert freq(3, 200) == freq(3, 200)
    inf = math.inf
    assert plain.sample([1.0, inf, 2.0, inf], 1.0, 0, 1.0, rng) == 1
    assert plain.sample([-inf, 0.0, -inf], 1.0, 0, 1.0, rng) == 1
    assert plain.sample([0.0, 1.0, -2.0], 1e-40, 0, 1.0, rng) == 1
    for seed in range(50):
        r = plain.MT19937_64(seed)
        assert plain.sample([5.0, 6.0], 2e-38, 0, 1.0, r) == 1
        assert plain.sample([-17.0, -13.0, -15.0], 2e-38, 0, 1.0, r) == 1
    with pytest.raises(ValueError):
        plain.sample([1.0, math.nan], 0.0, 0, 1.0, rng)
    with pytest.raises(ValueError):
        plain.sample([-inf, -inf], 1.0, 0, 1.0, rng)
