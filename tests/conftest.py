"""Shared fixtures: tiny configurations of the architecture, model folders with
random weights written with the `safetensors` library (not the engine's writer),
and the comparison helpers.  Tests marked `gpu` need an MI355X; all others run
on the CPU."""
import json
import os
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(Path(__file__).resolve().parent))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


# Four tiny configurations that differ in every size and option: head counts and
# grouping, head size (16 / 24 / 64, the last not hidden/heads), widths and
# vocabularies that are no power of two, number of layers, eps, theta, tied head.
TINY = {
    "a": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              intermediate_size=172, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-5,
              tie_word_embeddings=True, max_position_embeddings=320),
    "b": dict(num_hidden_layers=3, hidden_size=144, num_attention_heads=6, num_key_value_heads=6, head_dim=24,
              intermediate_size=384, vocab_size=509, rope_theta=500000.0, rms_norm_eps=1e-6,
              tie_word_embeddings=False, max_position_embeddings=512),
    "c": dict(num_hidden_layers=2, hidden_size=200, num_attention_heads=6, num_key_value_heads=2, head_dim=64,
              intermediate_size=264, vocab_size=1003, rope_theta=100000.0, rms_norm_eps=1e-5,
              tie_word_embeddings=False, max_position_embeddings=640),
    # sizes that fit none of the fast paths: width and head size that are no multiples of 8
    "d": dict(num_hidden_layers=2, hidden_size=100, num_attention_heads=5, num_key_value_heads=1, head_dim=20,
              intermediate_size=90, vocab_size=257, rope_theta=20000.0, rms_norm_eps=1e-4,
              tie_word_embeddings=True, max_position_embeddings=384),
}
SEEDS = {"a": 0, "b": 1, "c": 2, "d": 3}


def tensor_shapes(c):
    H, D, nh, nkv, I, V = (c["hidden_size"], c["head_dim"], c["num_attention_heads"], c["num_key_value_heads"],
                           c["intermediate_size"], c["vocab_size"])
    shapes = {"model.embed_tokens.weight": (V, H), "model.norm.weight": (H,)}
    if not c["tie_word_embeddings"]:
        shapes["lm_head.weight"] = (V, H)
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        shapes.update({p + "input_layernorm.weight": (H,), p + "post_attention_layernorm.weight": (H,),
                       p + "self_attn.q_proj.weight": (nh * D, H), p + "self_attn.k_proj.weight": (nkv * D, H),
                       p + "self_attn.v_proj.weight": (nkv * D, H), p + "self_attn.o_proj.weight": (H, nh * D),
                       p + "mlp.gate_proj.weight": (I, H), p + "mlp.up_proj.weight": (I, H),
                       p + "mlp.down_proj.weight": (H, I)})
    return shapes


def make_weights(c, seed, sharp=True):
    """N(0, 0.02) matrices, norms 1 + N(0, 0.02); with `sharp` the query and key
    projections are scaled up so that attention scores have a spread of one to
    three units (as in a trained model) instead of near zero, and a wrong key,
    position or page changes the logits; the other matrices are scaled so that
    the layers' contributions are as large as the embedding.  `sharp` may also be the two
    factors themselves, (queries and keys, the other matrices)."""
    import torch
    rng = np.random.default_rng(seed)
    qk, rest = (6.0, 4.0) if sharp is True else sharp if sharp else (1.0, 1.0)
    sharp = bool(sharp)
    out = {}
    for name, shape in sorted(tensor_shapes(c).items()):
        w = rng.standard_normal(size=shape).astype(np.float32) * 0.02
        if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
            w = 1.0 + w
        elif sharp and ("q_proj" in name or "k_proj" in name):
            w = w * qk
        elif sharp and ("v_proj" in name or "o_proj" in name or "mlp" in name):
            w = w * rest
        out[name] = torch.from_numpy(w).to(torch.bfloat16)
    return out


def write_folder(folder, c, seed, sharp=True):
    from safetensors.torch import save_file
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    raw = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", **c}
    (folder / "config.json").write_text(json.dumps(raw))
    save_file(make_weights(c, seed, sharp), str(folder / "model.safetensors"))
    return folder


@pytest.fixture(scope="session")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("models")
    return {name: write_folder(base / name, TINY[name], SEEDS[name]) for name in TINY}


_PLAIN = {}


def plain_logits(folder, tokens):
    """float64 logits [T, V] of the plain implementation, cached per (folder, tokens)."""
    import plain_llama
    key = (str(folder), tuple(tokens))
    if key not in _PLAIN:
        cfg, w = _PLAIN.setdefault(("folder", str(folder)), plain_llama.read_folder(folder))
        _PLAIN[key] = plain_llama.forward(cfg, w, list(tokens))
    return _PLAIN[key]


@pytest.fixture
def no_gemv():
    """Products of one or two rows against large weights run the matrix-vector kernel; a test about the kernels that
    take every other product switches it off for its duration."""
    from runtime.kernels import ops
    ops.set_gemv(0)
    yield
    ops.set_gemv()


def tune_attention(model, **settings):
    """Give every attention mixer of `model` launch rules that are told `settings` (kernels.attention.AttentionTuning)."""
    from runtime.kernels.attention import AttentionTuning
    tuning = AttentionTuning(**settings)
    for layer in model.layers:
        if hasattr(getattr(layer, "mixer", None), "tuning"):
            layer.mixer.tuning = tuning
    return tuning


def random_tokens(seed, n, vocab):
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


# Bounds of the comparisons with the plain implementation.  float32: largest
# difference over largest magnitude (the target is 1e-4; this is tighter).
# bfloat16: relative root-mean-square error of a request's logits, the measure
# and the bound the reference holds for bfloat16 against its float32 oracle
# (tests/test_precision.py:27-28: < 0.04).
F32_TOL = 2e-5
BF16_RMSE = 0.04


ACHIEVED = {}    # (test file, dtype) -> the largest error that a comparison of that file came to


def _record(dtype, err):
    name = os.environ.get("PYTEST_CURRENT_TEST", "?").split("::")[0]
    ACHIEVED[(name, dtype)] = max(ACHIEVED.get((name, dtype), 0.0), float(err))


def pytest_terminal_summary(terminalreporter):
    """What the comparisons with the plain implementation came to, beside their bounds."""
    if ACHIEVED:
        terminalreporter.write_line(f"largest errors against the plain implementation (bounds: float32 {F32_TOL}, bfloat16 rmse {BF16_RMSE})")
        for (name, dtype), err in sorted(ACHIEVED.items()):
            terminalreporter.write_line(f"  {name:40s} {dtype:9s} {err:.2e}")


def assert_close(got, ref, dtype, what=""):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, f"{what}: shape {got.shape} vs {ref.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite logits"
    if dtype == "float32":
        err = np.abs(got - ref).max() / np.abs(ref).max()
        _record(dtype, err)
        assert err < F32_TOL, f"{what}: float32 differs by {err:.3e} (bound {F32_TOL})"
    else:
        err = np.linalg.norm(got - ref) / np.linalg.norm(ref)
        _record(dtype, err)
        assert err < BF16_RMSE, f"{what}: bfloat16 relative rmse {err:.3e} (bound {BF16_RMSE})"
        rows = np.linalg.norm(got - ref, axis=-1) / np.linalg.norm(ref, axis=-1)
        assert rows.max() < 3 * BF16_RMSE, f"{what}: bfloat16 worst row {rows.max():.3e}"
