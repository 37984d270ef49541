"""Plain, slow Llama forward pass: whole sequences, no cache, float64 NumPy.

Written from the formulas of the reference runtime (file:line citations are
paths under the reference checkout).  One function per part; nothing here is
shared with the engine: it reads the model folder with the `safetensors`
library and `json`, never through the engine's loader, and it never touches a
GPU.  Every engine path is compared with `forward()`.
"""
import json
from pathlib import Path

import numpy as np


def rmsnorm(x, weight, eps):
    """y = x * 1/sqrt(mean(x^2) + eps) * w, weight multiplies after
    normalisation, eps inside the root (runtime/reference.py:5-6,
    kernels/ops.cu:3-19)."""
    x = np.asarray(x, np.float64)
    scale = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return x * scale * np.asarray(weight, np.float64)


def rope(x, positions, theta):
    """Split-half rotary embedding on [T, heads, D]: pair (i, i + D/2) turns by
    pos * theta^(-2i/D) (runtime/reference.py:9-15, kernels/ops.cu:21-33)."""
    x = np.asarray(x, np.float64)
    d = x.shape[-1]
    if d % 2:
        raise ValueError("rotary embedding needs an even head size")
    half = d // 2
    inv_freq = np.float64(theta) ** (-np.arange(half, dtype=np.float64) * 2.0 / d)
    angle = np.asarray(positions, np.float64)[:, None] * inv_freq[None, :]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return np.concatenate((a * cos - b * sin, b * cos + a * sin), axis=-1)


def attention_one_query(q, k, v):
    """One query position over T visible keys.  q [Hq, D]; k, v [T, Hkv, D].
    Consecutive query heads share a KV head; scale 1/sqrt(D); softmax with the
    maximum subtracted (runtime/reference.py:18-27)."""
    q, k, v = (np.asarray(t, np.float64) for t in (q, k, v))
    heads, kv_heads = q.shape[0], k.shape[1]
    if heads % kv_heads:
        raise ValueError("query heads must be a multiple of KV heads")
    kv_of_head = np.arange(heads) // (heads // kv_heads)
    scores = np.einsum("hd,thd->ht", q, k[:, kv_of_head]) / np.sqrt(q.shape[-1])
    scores = scores - scores.max(axis=-1, keepdims=True)
    p = np.exp(scores)
    p = p / p.sum(axis=-1, keepdims=True)
    return np.einsum("ht,thd->hd", p, v[:, kv_of_head])


def causal_attention(q, k, v, window=None):
    """Position t sees keys 0..t (runtime/reference.py:30-31;
    docs/ARCHITECTURE.md:20-21).  `window` keeps only the last `window` keys
    (t-window+1..t); the reference has no window, None means all keys."""
    out = []
    for t in range(len(q)):
        lo = 0 if window is None else max(0, t + 1 - window)
        out.append(attention_one_query(q[t], k[lo:t + 1], v[lo:t + 1]))
    return np.stack(out)


def swiglu(gate, up):
    """a = g * sigmoid(g) * u (runtime/model.py:117-119,
    kernels/execution.cu:7-10; the form without a clamp, as in
    tests/test_model.py:22)."""
    gate = np.asarray(gate, np.float64)
    return gate / (1.0 + np.exp(-gate)) * np.asarray(up, np.float64)


def linear(x, weight):
    """y = x . W^T with W stored [out, in], no bias (runtime/model.py:108)."""
    return np.asarray(x, np.float64) @ np.asarray(weight, np.float64).T


def read_folder(folder):
    """config.json as a dict and every tensor of model.safetensors as float64."""
    import torch
    from safetensors import safe_open
    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float64).numpy()
    return config, weights


def head_dim_of(config):
    return config.get("head_dim") or config["hidden_size"] // config["num_attention_heads"]


def forward(config, weights, tokens, upto_layer=None):
    """Logits [T, vocab] for one whole sequence (runtime/model.py:105-120 run
    on all positions at once, as tests/test_model.py:10-23 does)."""
    c = config
    heads, kv_heads, dim = c["num_attention_heads"], c["num_key_value_heads"], head_dim_of(c)
    eps, theta = c["rms_norm_eps"], c["rope_theta"]
    positions = np.arange(len(tokens))
    x = np.asarray(weights["model.embed_tokens.weight"], np.float64)[np.asarray(tokens)]
    layers = c["num_hidden_layers"] if upto_layer is None else upto_layer
    for layer in range(layers):
        p = f"model.layers.{layer}."
        h = rmsnorm(x, weights[p + "input_layernorm.weight"], eps)
        q = rope(linear(h, weights[p + "self_attn.q_proj.weight"]).reshape(-1, heads, dim), positions, theta)
        k = rope(linear(h, weights[p + "self_attn.k_proj.weight"]).reshape(-1, kv_heads, dim), positions, theta)
        v = linear(h, weights[p + "self_attn.v_proj.weight"]).reshape(-1, kv_heads, dim)
        attended = causal_attention(q, k, v).reshape(len(tokens), heads * dim)
        x = x + linear(attended, weights[p + "self_attn.o_proj.weight"])
        h = rmsnorm(x, weights[p + "post_attention_layernorm.weight"], eps)
        act = swiglu(linear(h, weights[p + "mlp.gate_proj.weight"]), linear(h, weights[p + "mlp.up_proj.weight"]))
        x = x + linear(act, weights[p + "mlp.down_proj.weight"])
    if upto_layer is not None:
        return x
    head = weights["model.embed_tokens.weight"] if c.get("tie_word_embeddings", False) else weights["lm_head.weight"]
    return linear(rmsnorm(x, weights["model.norm.weight"], eps), head)


def greedy(config, weights, prompt, steps):
    """Greedy continuation by recomputing the whole sequence each step; the
    lowest index wins a tie (np.argmax; runtime/engine.py:99)."""
    tokens = list(prompt)
    out = []
    for _ in range(steps):
        nxt = int(np.argmax(forward(config, weights, tokens)[-1]))
        out.append(nxt)
        tokens.append(nxt)
    return out
