"""Plain Qwen2 forward pass: whole sequence, no cache, float64 arithmetic.

Every function follows one formula of the reference (LandoWang/sprout-lm,
paths relative to its root) and cites it.  Storage is float32 and sums run in
float64, as the reference's JavaScript numbers do (src/qwen.ts:59-92).

`store` is an optional rounding function applied wherever the bfloat16 engine
keeps a tensor in bfloat16 (projection outputs, normed activations, cached
keys and values, the attention output, the gated product).  With the default
(float32 rounding) the functions are the reference's float32 arithmetic.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


def f32(x):
    return np.asarray(x, dtype=np.float64).astype(np.float32)


def bf16_round(x):
    """Round-to-nearest-even float32 -> bfloat16 -> float32 (numpy only)."""
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(a.shape)


def rms_norm(x, weight, eps):
    """src/qwen.ts:72-77: s = 1/sqrt(mean(x^2)+eps); y = f32(x*s) * w."""
    x64 = np.asarray(x, dtype=np.float64)
    scale = 1.0 / np.sqrt((x64 * x64).mean(axis=-1, keepdims=True) + eps)
    normed = f32(x64 * scale)
    return f32(normed.astype(np.float64) * np.asarray(weight, dtype=np.float64))


def linear(x, weight, bias=None):
    """src/qwen.ts:59-70: y[row] = sum_col W[row, col] * x[col] + b[row]; W is [out, in]."""
    y = np.asarray(x, dtype=np.float64) @ np.asarray(weight, dtype=np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return f32(y)


def rope_neox(x, positions, head_dim, theta):
    """src/qwen.ts:81-92: pair (d, d+half) of every head turns by pos / theta^(2d/head_dim)."""
    x = np.asarray(x, dtype=np.float64)
    tokens, width = x.shape
    half = head_dim // 2
    out = x.copy().reshape(tokens, width // head_dim, head_dim)
    src = x.reshape(tokens, width // head_dim, head_dim)
    d = np.arange(half, dtype=np.float64)
    angle = np.asarray(positions, dtype=np.float64)[:, None] / theta ** (2.0 * d / head_dim)
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    a, b = src[..., :half], src[..., half:]
    out[..., :half] = a * cos - b * sin
    out[..., half:] = b * cos + a * sin
    return f32(out.reshape(tokens, width))


def causal_gqa_attention(q, k, v, n_heads, n_kv_heads, head_dim, window=None, positions=None):
    """src/qwen.ts:173-194: head h reads kv head floor(h / (n_heads/n_kv_heads));
    score = q.k / sqrt(head_dim) over keys j <= p; softmax with max subtraction; sum_j P_j v_j.

    `window` (not in the reference, which rejects sliding windows at
    src/qwen.ts:18) keeps only keys with p - j < window.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    tokens = q.shape[0]
    group = n_heads // n_kv_heads
    out = np.zeros((tokens, n_heads * head_dim), dtype=np.float32)
    for h in range(n_heads):
        g = h // group
        qh = q[:, h * head_dim:(h + 1) * head_dim]
        kh = k[:, g * head_dim:(g + 1) * head_dim]
        vh = v[:, g * head_dim:(g + 1) * head_dim]
        for p in range(tokens):
            first = 0 if window is None else max(0, p - window + 1)
            scores = f32(kh[first:p + 1] @ qh[p] / math.sqrt(head_dim)).astype(np.float64)
            e = f32(np.exp(scores - scores.max())).astype(np.float64)
            probs = f32(e / e.sum()).astype(np.float64)
            out[p, h * head_dim:(h + 1) * head_dim] = f32(probs @ vh[first:p + 1])
    return out


def swiglu(gate, up):
    """src/qwen.ts:199: f32(g / (1 + exp(-g))) * u."""
    g = np.asarray(gate, dtype=np.float64)
    silu = f32(g / (1.0 + np.exp(-g)))
    return f32(silu.astype(np.float64) * np.asarray(up, dtype=np.float64))


def attention_block(x, w, prefix, cfg, positions, store=f32, window=None):
    """src/qwen.ts:166-195: norm, q/k/v with bias, rope on q and k, attention, o_proj."""
    heads, kv_heads = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    head_dim = cfg["hidden_size"] // heads
    n = store(rms_norm(x, w[prefix + "input_layernorm.weight"], cfg["rms_norm_eps"]))
    q = store(linear(n, w[prefix + "self_attn.q_proj.weight"], w[prefix + "self_attn.q_proj.bias"]))
    k = store(linear(n, w[prefix + "self_attn.k_proj.weight"], w[prefix + "self_attn.k_proj.bias"]))
    v = store(linear(n, w[prefix + "self_attn.v_proj.weight"], w[prefix + "self_attn.v_proj.bias"]))
    q = store(rope_neox(q, positions, head_dim, cfg["rope_theta"]))
    k = store(rope_neox(k, positions, head_dim, cfg["rope_theta"]))
    a = store(causal_gqa_attention(q, k, v, heads, kv_heads, head_dim, window=window))
    return linear(a, w[prefix + "self_attn.o_proj.weight"])


def feed_forward_block(x, w, prefix, cfg, store=f32):
    """src/qwen.ts:196-200: norm, gate and up, SwiGLU, down."""
    n = store(rms_norm(x, w[prefix + "post_attention_layernorm.weight"], cfg["rms_norm_eps"]))
    gate = linear(n, w[prefix + "mlp.gate_proj.weight"])
    up = linear(n, w[prefix + "mlp.up_proj.weight"])
    return linear(store(swiglu(gate, up)), w[prefix + "mlp.down_proj.weight"])


def decoder_layer(x, w, layer, cfg, positions, store=f32):
    """src/qwen.ts:164-202: x += attention(norm(x)); x += mlp(norm(x)); float32 adds (src/qwen.ts:79)."""
    prefix = f"model.layers.{layer}."
    x = f32(x.astype(np.float64) + attention_block(x, w, prefix, cfg, positions, store))
    x = f32(x.astype(np.float64) + feed_forward_block(x, w, prefix, cfg, store))
    return x


def forward_logits(w, cfg, tokens, store=f32, first_position=0, rows=None):
    """Logits [len(tokens), vocab] at every position (src/qwen.ts:158-204 over a whole sequence), or at the
    positions `rows` only (the reference computes them where they are asked for, src/qwen.ts:203).

    The output matrix is the embedding when tie_word_embeddings (src/qwen.ts:152).
    """
    tokens = np.asarray(tokens, dtype=np.int64)
    positions = np.arange(len(tokens)) + first_position
    x = f32(np.asarray(w["model.embed_tokens.weight"])[tokens])
    for layer in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, layer, cfg, positions, store)
    if rows is not None:
        x = x[np.asarray(rows, dtype=np.int64)]
    n = store(rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]))
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(n, head)


def greedy(w, cfg, prompt, steps, store=f32):
    """scripts/reference.py:20-44: recompute the whole history, take argmax of the last row, append."""
    history, out = list(prompt), []
    for _ in range(steps):
        token = int(np.argmax(forward_logits(w, cfg, history, store)[-1]))
        history.append(token)
        out.append(token)
    return out


def load_folder(folder, dtype="float32"):
    """Read config.json and model.safetensors of a model folder with the safetensors library.

    Returns (config dict, {name: float32 array}).  bfloat16 tensors widen
    exactly; with dtype == "bfloat16" float32 tensors are rounded to bfloat16
    first, which is what the engine's bfloat16 loader keeps.
    """
    import torch
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    weights = {}
    for name, t in tensors.items():
        if dtype == "bfloat16":
            t = t.to(torch.bfloat16)
        weights[name] = t.to(torch.float32).numpy()
    return cfg, weights
