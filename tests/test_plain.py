"""Pins the plain implementation by facts other than the reference's text."""
import json
import math
import os

import numpy as np
import pytest

from tests.plain import qwen2_plain as P


# ---- vectors the reference's own tests hold (test/qwen.test.ts:15-46) -------------------------

def test_plain_matches_reference_fixture_logits(reference_fixture):
    cfg, w = P.load_folder(reference_fixture)
    ref = json.load(open(os.path.join(reference_fixture, "reference.json")))
    worst = 0.0
    for case in ref["cases"]:
        history = list(case["tokens"])
        for step, name in enumerate(case["logits"]):
            want = np.fromfile(os.path.join(reference_fixture, name), dtype="<f4")
            got = P.forward_logits(w, cfg, history)[-1]
            worst = max(worst, float(np.abs(got - want).max()))
            assert int(np.argmax(got)) == case["output"][step]
            history.append(case["output"][step])
    assert worst < 2e-6  # the reference's own bound (test/qwen.test.ts:35)


# ---- RMSNorm ---------------------------------------------------------------------------------

def test_rms_norm_constant_and_library_form():
    x = np.full((1, 24), 3.0, dtype=np.float32)
    y = P.rms_norm(x, np.ones(24, dtype=np.float32), 1e-5)
    assert np.allclose(y, 3.0 / math.sqrt(9.0 + 1e-5), atol=1e-7)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 24)).astype(np.float32)
    wt = rng.uniform(0.5, 1.5, 24).astype(np.float32)
    lib = x * (1.0 / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6)) * wt
    assert np.allclose(P.rms_norm(x, wt, 1e-6), lib, atol=1e-6)
    # the weight multiplies as it is (a "1 + w" norm would double this)
    assert np.allclose(P.rms_norm(x, 2 * wt, 1e-6), 2 * lib, atol=2e-6)
    # eps stands inside the root: zero input gives zero, not NaN
    assert np.all(P.rms_norm(np.zeros((1, 24), np.float32), wt, 1e-6) == 0)
    big = P.rms_norm(x * 1e-3, wt, 1e-2)
    assert np.abs(big).max() < 0.1 * np.abs(lib).max()


# ---- linear ----------------------------------------------------------------------------------

def test_linear_layout_is_out_by_in():
    rng = np.random.default_rng(1)
    wt = rng.standard_normal((7, 5)).astype(np.float32)
    b = rng.standard_normal(7).astype(np.float32)
    e2 = np.zeros((1, 5), np.float32)
    e2[0, 2] = 1
    assert np.allclose(P.linear(e2, wt, b)[0], wt[:, 2] + b)
    x = rng.standard_normal((3, 5)).astype(np.float32)
    assert np.allclose(P.linear(x, wt, b), x @ wt.T + b, atol=1e-6)


# ---- RoPE ------------------------------------------------------------------------------------

def test_rope_pairing_sign_and_shift():
    hd, theta = 8, 10000.0
    x = np.zeros((1, hd), np.float32)
    x[0, 1] = 1.0
    y = P.rope_neox(x, [3], hd, theta)[0]
    ang = 3 / theta ** (2 * 1 / hd)
    # neox pairing: index d pairs with d + hd/2 (interleaved pairing would light index 0 or 2)
    want = np.zeros(hd)
    want[1], want[1 + hd // 2] = math.cos(ang), math.sin(ang)
    assert np.allclose(y, want, atol=1e-7)
    # pair 0 turns by exactly the position
    x = np.zeros((1, hd), np.float32)
    x[0, 0] = 1.0
    y = P.rope_neox(x, [2], hd, theta)[0]
    assert np.allclose([y[0], y[hd // 2]], [math.cos(2), math.sin(2)], atol=1e-7)
    rng = np.random.default_rng(2)
    q = rng.standard_normal((1, 2 * hd)).astype(np.float32)
    k = rng.standard_normal((1, 2 * hd)).astype(np.float32)
    assert np.array_equal(P.rope_neox(q, [0], hd, theta), q)  # position 0 is the identity
    # only distances count; norms of pairs are kept
    d1 = (P.rope_neox(q, [5], hd, theta) * P.rope_neox(k, [2], hd, theta)).reshape(2, hd).sum(-1)
    d2 = (P.rope_neox(q, [45], hd, theta) * P.rope_neox(k, [42], hd, theta)).reshape(2, hd).sum(-1)
    assert np.allclose(d1, d2, atol=1e-5)
    d3 = (P.rope_neox(q, [2], hd, theta) * P.rope_neox(k, [5], hd, theta)).reshape(2, hd).sum(-1)
    assert not np.allclose(d1, d3, atol=1e-3)
    assert np.allclose(np.linalg.norm(P.rope_neox(q, [17], hd, theta)), np.linalg.norm(q), atol=1e-6)


# ---- attention -------------------------------------------------------------------------------

def _library_attention(q, k, v, heads, kv_heads, hd, window=None):
    t = q.shape[0]
    qh = q.reshape(t, heads, hd).transpose(1, 0, 2).astype(np.float64)
    kh = np.repeat(k.reshape(t, kv_heads, hd).transpose(1, 0, 2), heads // kv_heads, axis=0).astype(np.float64)
    vh = np.repeat(v.reshape(t, kv_heads, hd).transpose(1, 0, 2), heads // kv_heads, axis=0).astype(np.float64)
    s = qh @ kh.transpose(0, 2, 1) / math.sqrt(hd)
    i, j = np.arange(t)[:, None], np.arange(t)[None, :]
    mask = j > i
    if window is not None:
        mask |= (i - j) >= window
    s = np.where(mask, -np.inf, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return (p @ vh).transpose(1, 0, 2).reshape(t, heads * hd)


def test_attention_against_library_form_and_special_cases():
    rng = np.random.default_rng(3)
    heads, kv_heads, hd, t = 6, 2, 8, 11
    q = rng.standard_normal((t, heads * hd)).astype(np.float32)
    k = rng.standard_normal((t, kv_heads * hd)).astype(np.float32)
    v = rng.standard_normal((t, kv_heads * hd)).astype(np.float32)
    got = P.causal_gqa_attention(q, k, v, heads, kv_heads, hd)
    assert np.allclose(got, _library_attention(q, k, v, heads, kv_heads, hd), atol=2e-6)
    # the first token sees only itself: output is v of its group (pins the head -> group map)
    for h in range(heads):
        g = h // (heads // kv_heads)
        assert np.allclose(got[0, h * hd:(h + 1) * hd], v[0, g * hd:(g + 1) * hd], atol=1e-7)
    # all keys equal -> running mean of v
    same = P.causal_gqa_attention(q, np.tile(k[:1], (t, 1)), v, heads, kv_heads, hd)
    means = np.cumsum(v.astype(np.float64), 0) / np.arange(1, t + 1)[:, None]
    assert np.allclose(same[:, :hd], means[:, :hd], atol=1e-6)
    # causal: a later token never changes an earlier row
    k2, v2 = k.copy(), v.copy()
    k2[7:] += 1.0
    v2[7:] -= 2.0
    assert np.array_equal(P.causal_gqa_attention(q, k2, v2, heads, kv_heads, hd)[:7], got[:7])
    # a window of w keeps keys p-w+1..p
    win = P.causal_gqa_attention(q, k, v, heads, kv_heads, hd, window=4)
    assert np.allclose(win, _library_attention(q, k, v, heads, kv_heads, hd, window=4), atol=2e-6)
    assert np.allclose(win[:4], got[:4], atol=1e-7) and not np.allclose(win[6], got[6], atol=1e-4)


def test_single_head_no_rotation_is_plain_softmax_attention():
    rng = np.random.default_rng(4)
    t, hd = 5, 4
    q, k, v = (rng.standard_normal((t, hd)).astype(np.float32) for _ in range(3))
    got = P.causal_gqa_attention(q, k, v, 1, 1, hd)
    assert np.allclose(got, _library_attention(q, k, v, 1, 1, hd), atol=1e-6)
    # the scale is 1/sqrt(head_dim): scaling q by sqrt(hd) equals unscaled scores
    s = (q[-1].astype(np.float64) * math.sqrt(hd)) @ k.T.astype(np.float64) / math.sqrt(hd)
    p = np.exp(s - s.max())
    assert np.allclose(P.causal_gqa_attention(q * math.sqrt(hd), k, v, 1, 1, hd)[-1], (p / p.sum()) @ v, atol=1e-5)


# ---- SwiGLU ----------------------------------------------------------------------------------

def test_swiglu_gate_is_the_activated_operand():
    g = np.array([[0.0, 30.0, -30.0, 1.0]], np.float32)
    u = np.array([[5.0, 2.0, 2.0, 3.0]], np.float32)
    y = P.swiglu(g, u)[0]
    assert y[0] == 0 and abs(y[1] - 60.0) < 1e-4 and abs(y[2]) < 1e-8
    assert abs(y[3] - (1 / (1 + math.exp(-1))) * 3) < 1e-6
    assert not np.allclose(P.swiglu(u, g), P.swiglu(g, u))


# ---- whole model -----------------------------------------------------------------------------

def _tiny(seed=0, tied=True):
    cfg = dict(hidden_size=24, intermediate_size=40, num_hidden_layers=2, num_attention_heads=3,
               num_key_value_heads=1, vocab_size=50, rms_norm_eps=1e-5, rope_theta=1e4,
               tie_word_embeddings=tied)
    rng = np.random.default_rng(seed)
    h, i, kv = 24, 40, 8
    w = {"model.embed_tokens.weight": rng.standard_normal((50, h)).astype(np.float32) * 0.5,
         "model.norm.weight": rng.uniform(0.7, 1.3, h).astype(np.float32),
         "lm_head.weight": rng.standard_normal((50, h)).astype(np.float32) * 0.5}
    for l in range(2):
        p = f"model.layers.{l}."
        for name, shape in [("self_attn.q_proj", (h, h)), ("self_attn.k_proj", (kv, h)), ("self_attn.v_proj", (kv, h)),
                            ("self_attn.o_proj", (h, h)), ("mlp.gate_proj", (i, h)), ("mlp.up_proj", (i, h)),
                            ("mlp.down_proj", (h, i))]:
            w[p + name + ".weight"] = rng.standard_normal(shape).astype(np.float32) * 0.3
        for name, n in [("self_attn.q_proj", h), ("self_attn.k_proj", kv), ("self_attn.v_proj", kv)]:
            w[p + name + ".bias"] = rng.uniform(-0.3, 0.3, n).astype(np.float32)
        w[p + "input_layernorm.weight"] = rng.uniform(0.7, 1.3, h).astype(np.float32)
        w[p + "post_attention_layernorm.weight"] = rng.uniform(0.7, 1.3, h).astype(np.float32)
    return cfg, w


def test_model_causality_and_head_choice():
    cfg, w = _tiny()
    toks = [3, 14, 15, 9, 2, 6]
    full = P.forward_logits(w, cfg, toks)
    assert np.allclose(P.forward_logits(w, cfg, toks[:4]), full[:4], atol=1e-6)
    changed = P.forward_logits(w, cfg, toks[:4] + [40, 41])
    assert np.allclose(changed[:4], full[:4], atol=1e-6) and not np.allclose(changed[4:], full[4:], atol=1e-3)
    cfg2 = dict(cfg, tie_word_embeddings=False)
    assert not np.allclose(P.forward_logits(w, cfg2, toks), full, atol=1e-3)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"]
    assert np.array_equal(P.forward_logits(w2, cfg2, toks), full)
    # biases matter (a loader that dropped them would pass a bias-free check)
    w3 = dict(w)
    w3["model.layers.0.self_attn.k_proj.bias"] = np.zeros(8, np.float32)
    assert not np.allclose(P.forward_logits(w3, cfg, toks), full, atol=1e-4)


def test_bf16_round_matches_torch():
    import torch
    x = np.random.default_rng(5).standard_normal(1000).astype(np.float32) * 3
    x[:4] = [1.00390625, 1.01171875, -1.00390625, 0.0]  # ties round to even
    assert np.array_equal(P.bf16_round(x), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
