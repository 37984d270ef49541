"""Pins of the plain implementation: vectors the reference's own tests hold,
special cases that reduce to a library routine, and invariants, each chosen so
that a plausible mistake fails it."""
import numpy as np
import torch

import plain_llama as P


def test_attention_large_equal_scores_give_mean_of_values():
    # reference tests/test_reference.py:7-13: 1e3-magnitude scores stay finite and
    # equal scores give the mean of the value rows
    q = np.full((4, 8), 1e3)
    k = np.full((3, 2, 8), 1e3)
    v = np.arange(48, dtype=np.float64).reshape(3, 2, 8)
    out = P.attention_one_query(q, k, v)
    assert np.isfinite(out).all()
    np.testing.assert_allclose(out[0], v[:, 0].mean(axis=0))
    np.testing.assert_allclose(out[3], v[:, 1].mean(axis=0))  # heads 2,3 read kv head 1


def test_rope_preserves_norm_and_position_zero_is_identity():
    # reference tests/test_reference.py:15-18
    x = np.random.default_rng(4).normal(size=(3, 2, 10))
    y = P.rope(x, [0, 7, 100], 10000.0)
    np.testing.assert_allclose((x * x).sum(-1), (y * y).sum(-1), rtol=1e-12)
    np.testing.assert_allclose(y[0], x[0], atol=0)


def test_rmsnorm_of_zero_is_zero_and_unit_rms():
    # reference tests/test_reference.py:20-21
    assert (P.rmsnorm(np.zeros((2, 8)), np.ones(8), 1e-5) == 0).all()
    x = np.random.default_rng(0).normal(size=(5, 33)) * 7
    y = P.rmsnorm(x, np.ones(33), 0.0)
    np.testing.assert_allclose(np.sqrt((y * y).mean(-1)), 1.0, rtol=1e-12)
    # the weight multiplies after the normalisation (a norm in the wrong place fails this)
    w = np.random.default_rng(1).normal(size=33)
    np.testing.assert_allclose(P.rmsnorm(x, w, 0.0), y * w, rtol=1e-12)
    # eps sits inside the root: with a huge eps the output is x / sqrt(eps)
    np.testing.assert_allclose(P.rmsnorm(x, np.ones(33), 1e12), x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e12))


def test_rope_is_a_complex_rotation_with_split_half_pairing():
    # (x[i] + j x[i + D/2]) * exp(j * pos * theta^(-2i/D)); interleaved pairing or a
    # wrong sign of the sine fails this
    rng = np.random.default_rng(2)
    d, theta = 12, 500000.0
    x = rng.normal(size=(4, 3, d))
    pos = np.array([0, 1, 17, 250])
    y = P.rope(x, pos, theta)
    z = x[..., :d // 2] + 1j * x[..., d // 2:]
    ang = pos[:, None] * theta ** (-np.arange(d // 2) * 2.0 / d)
    zr = z * np.exp(1j * ang)[:, None, :]
    np.testing.assert_allclose(y[..., :d // 2], zr.real, atol=1e-12)
    np.testing.assert_allclose(y[..., d // 2:], zr.imag, atol=1e-12)


def test_rope_of_one_head_worked_by_hand_from_the_references_kernel():
    """The reference states the rotation twice, independently: as NumPy (runtime/reference.py:9-15) and as a CUDA
    kernel that its own tests hold against the former (kernels/ops.cu:21-33, tests/test_cuda.py:28-39).  This is the
    kernel's arithmetic walked through by hand for one head of four coordinates at position 3 with theta 100:
    thread d of `half = 2` reads a = x[d], b = x[d + half], turns them by 3 * 100^(-2 d / 4), so the pairs are
    (0, 2) and (1, 3) and the angles 3 and 0.3.  Neighbouring pairs (0, 1), (2, 3), the angle schedule
    theta^(-d / dim), or the sine's sign the other way round each change these four numbers.  (The installed
    `transformers` package is no source for this repository, so its Llama is not imported here; the pairing is that
    of the reference's two texts.)"""
    from math import cos, sin
    x = np.array([[[1.0, 2.0, 3.0, 4.0]]])
    want = [1 * cos(3.0) - 3 * sin(3.0), 2 * cos(0.3) - 4 * sin(0.3), 3 * cos(3.0) + 1 * sin(3.0), 4 * cos(0.3) + 2 * sin(0.3)]
    np.testing.assert_allclose(P.rope(x, [3], 100.0)[0, 0], want, rtol=1e-14)
    np.testing.assert_allclose(want, [-1.4133525208, 0.7285921516, -2.8288574817, 4.4123863698], rtol=1e-9)


def test_rope_scores_depend_on_distance_only():
    rng = np.random.default_rng(3)
    q, k = rng.normal(size=(1, 1, 16)), rng.normal(size=(1, 1, 16))
    def score(pq, pk, theta=10000.0):
        return float((P.rope(q, [pq], theta) * P.rope(k, [pk], theta)).sum())
    assert abs(score(5, 2) - score(105, 102)) < 1e-9
    assert abs(score(5, 2) - score(2, 5)) > 1e-6           # direction matters
    assert abs(score(5, 2) - score(5, 2, 500000.0)) > 1e-6  # theta matters


def test_attention_reduces_to_library_softmax_attention():
    # no rotation, one KV head per query head: torch's scaled_dot_product_attention
    rng = np.random.default_rng(5)
    T, H, D = 9, 3, 8
    q, k, v = (rng.normal(size=(T, H, D)) for _ in range(3))
    ours = P.causal_attention(q, k, v)
    tq, tk, tv = (torch.from_numpy(t).permute(1, 0, 2)[None] for t in (q, k, v))
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)[0].permute(1, 0, 2).numpy()
    np.testing.assert_allclose(ours, ref, atol=1e-12)
    # one visible key: the output is that value row
    np.testing.assert_allclose(ours[0], v[0], atol=1e-12)


def test_grouped_heads_equal_repeated_kv_heads():
    rng = np.random.default_rng(6)
    q = rng.normal(size=(6, 4, 8))
    k, v = rng.normal(size=(6, 2, 8)), rng.normal(size=(6, 2, 8))
    grouped = P.causal_attention(q, k, v)
    repeated = P.causal_attention(q, np.repeat(k, 2, axis=1), np.repeat(v, 2, axis=1))
    np.testing.assert_allclose(grouped, repeated, atol=1e-12)
    # consecutive (not strided) query heads share a KV head
    assert not np.allclose(grouped, P.causal_attention(q, np.tile(k, (1, 2, 1)), np.tile(v, (1, 2, 1))))


def test_window_limits_visible_keys():
    rng = np.random.default_rng(7)
    q, k, v = (rng.normal(size=(10, 2, 4)) for _ in range(3))
    full = P.causal_attention(q, k, v)
    win = P.causal_attention(q, k, v, window=3)
    np.testing.assert_allclose(win[:3], full[:3], atol=1e-12)  # fewer than 3 keys so far
    np.testing.assert_allclose(win[7], P.attention_one_query(q[7], k[5:8], v[5:8]), atol=1e-12)
    np.testing.assert_allclose(P.causal_attention(q, k, v, window=100), full, atol=1e-12)


def test_swiglu_is_library_silu_times_up():
    g = np.linspace(-30, 30, 41)
    u = np.linspace(1, 2, 41)
    ref = (torch.nn.functional.silu(torch.from_numpy(g)) * torch.from_numpy(u)).numpy()
    np.testing.assert_allclose(P.swiglu(g, u), ref, rtol=1e-12, atol=1e-300)
    assert P.swiglu(np.zeros(3), np.ones(3)).tolist() == [0, 0, 0]


def test_forward_matches_an_independent_torch_composition(folders):
    # the same model composed from torch library routines (embedding, rms_norm,
    # linear, sdpa); only the rotary embedding is taken from the plain module
    cfg, w = P.read_folder(folders["a"])
    tokens = [3, 250, 17, 17, 99, 4, 8]
    ours = P.forward(cfg, w, tokens)
    F = torch.nn.functional
    tw = {k: torch.from_numpy(v) for k, v in w.items()}
    nh, nkv, D, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    x = F.embedding(torch.tensor(tokens), tw["model.embed_tokens.weight"])
    pos = np.arange(len(tokens))
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = F.rms_norm(x, (x.shape[-1],), tw[p + "input_layernorm.weight"], eps)
        q = torch.from_numpy(P.rope(F.linear(h, tw[p + "self_attn.q_proj.weight"]).view(-1, nh, D).numpy(), pos, cfg["rope_theta"]))
        k = torch.from_numpy(P.rope(F.linear(h, tw[p + "self_attn.k_proj.weight"]).view(-1, nkv, D).numpy(), pos, cfg["rope_theta"]))
        v = F.linear(h, tw[p + "self_attn.v_proj.weight"]).view(-1, nkv, D)
        k, v = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
        a = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None], k.permute(1, 0, 2)[None], v.permute(1, 0, 2)[None],
                                           is_causal=True)[0].permute(1, 0, 2).reshape(len(tokens), nh * D)
        x = x + F.linear(a, tw[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (x.shape[-1],), tw[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, tw[p + "mlp.gate_proj.weight"])) * F.linear(h, tw[p + "mlp.up_proj.weight"]),
                         tw[p + "mlp.down_proj.weight"])
    ref = F.linear(F.rms_norm(x, (x.shape[-1],), tw["model.norm.weight"], eps), tw["model.embed_tokens.weight"])
    np.testing.assert_allclose(ours, ref.numpy(), rtol=1e-9, atol=1e-12)


def test_forward_is_causal_and_prefix_stable(folders):
    cfg, w = P.read_folder(folders["b"])
    tokens = [5, 400, 33, 8, 120, 7]
    full = P.forward(cfg, w, tokens)
    np.testing.assert_allclose(P.forward(cfg, w, tokens[:4]), full[:4], atol=1e-12)
    changed = P.forward(cfg, w, tokens[:5] + [9])
    np.testing.assert_allclose(changed[:5], full[:5], atol=1e-12)
    assert not np.allclose(changed[5], full[5])


def test_reference_toy_weights_vector(folders):
    # the reference's own model test (tests/test_model.py:8-26) feeds tokens
    # [1,9,5,7,3] through its default toy configuration; its weights come from
    # numpy's default_rng(42) (runtime/model.py:38-55).  Rebuilt here, the plain
    # forward must agree with the computation of that test written out a second time.
    c = dict(vocab_size=128, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
             num_key_value_heads=2, rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=False)
    rng = np.random.default_rng(42)
    w = {}
    def matrix(name, out, inp):
        w[name] = (rng.normal(size=(out, inp)) / np.sqrt(inp)).astype(np.float32)
    dim = 16
    matrix("model.embed_tokens.weight", 128, 64)
    matrix("lm_head.weight", 128, 64)
    w["model.norm.weight"] = np.ones(64, np.float32)
    for layer in range(2):
        p = f"model.layers.{layer}."
        for n in ("input_layernorm", "post_attention_layernorm"):
            w[p + n + ".weight"] = np.ones(64, np.float32)
        for proj, out in (("q_proj", 64), ("k_proj", 2 * dim), ("v_proj", 2 * dim), ("o_proj", 64)):
            matrix(p + "self_attn." + proj + ".weight", out, 64)
        for proj in ("gate_proj", "up_proj"):
            matrix(p + "mlp." + proj + ".weight", 128, 64)
        matrix(p + "mlp.down_proj.weight", 64, 128)
    tokens = [1, 9, 5, 7, 3]
    got = P.forward(c, w, tokens)
    # the same computation written a second time from the formulas, sharing nothing with the plain module: the norm
    # spelled out, the rotary embedding as a complex rotation, attention as one masked softmax matrix per head
    def norm(z, weight):
        return z / np.sqrt((z * z).mean(-1, keepdims=True) + 1e-5) * weight.astype(np.float64)

    def turn(z):   # z [T, heads, dim]: coordinates (i, i + dim/2) are the real and imaginary part of one number
        half = dim // 2
        angle = np.arange(5)[:, None] * 10000.0 ** (-2.0 * np.arange(half) / dim)[None, :]
        zc = (z[..., :half] + 1j * z[..., half:]) * np.exp(1j * angle)[:, None, :]
        return np.concatenate([zc.real, zc.imag], axis=-1)

    def attend(q, k, v):   # q [T, 4, dim], k and v [T, 2, dim]: query head h reads key head h // 2
        out = np.zeros_like(q)
        for h in range(4):
            scores = q[:, h] @ k[:, h // 2].T / np.sqrt(dim)
            scores[np.triu_indices(5, 1)] = -np.inf
            weights = np.exp(scores - scores.max(-1, keepdims=True))
            out[:, h] = (weights / weights.sum(-1, keepdims=True)) @ v[:, h // 2]
        return out

    x = w["model.embed_tokens.weight"][tokens].astype(np.float64)
    for layer in range(2):
        p = f"model.layers.{layer}."
        lin = lambda z, n: z @ w[p + n + ".weight"].astype(np.float64).T
        h = norm(x, w[p + "input_layernorm.weight"])
        q = turn(lin(h, "self_attn.q_proj").reshape(-1, 4, dim))
        k = turn(lin(h, "self_attn.k_proj").reshape(-1, 2, dim))
        v = lin(h, "self_attn.v_proj").reshape(-1, 2, dim)
        x = x + lin(attend(q, k, v).reshape(-1, 64), "self_attn.o_proj")
        h = norm(x, w[p + "post_attention_layernorm.weight"])
        g = lin(h, "mlp.gate_proj")
        x = x + lin(g / (1 + np.exp(-g)) * lin(h, "mlp.up_proj"), "mlp.down_proj")
    expected = norm(x, w["model.norm.weight"]) @ w["lm_head.weight"].astype(np.float64).T
    np.testing.assert_allclose(got, expected, atol=1e-12)
    assert got.shape == (5, 128) and np.abs(got).max() > 0.5  # real-sized logits, not a degenerate case
