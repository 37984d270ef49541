"""The layer sizes of the real family members (SmolLM2-135M, SmolLM2-1.7B, Llama-3-8B) with few
layers and a small vocabulary, so that the plain implementation stays fast: prompt in portions,
then single tokens, in float32 and bfloat16, against the plain implementation.  These sizes take
other kernel paths than the tiny configurations (head size 128, inner sizes of 4096 and 14336,
sixteen-wave and four-wave products, the 128 x 128 tile)."""
import numpy as np
import pytest

from conftest import assert_close, plain_logits, random_tokens, write_folder

pytestmark = pytest.mark.gpu

FAMILY = {
    "smollm2-135m": dict(num_hidden_layers=2, hidden_size=576, num_attention_heads=9, num_key_value_heads=3, head_dim=64,
                         intermediate_size=1536, vocab_size=3001, rope_theta=100000.0, rms_norm_eps=1e-5,
                         tie_word_embeddings=True, max_position_embeddings=512),
    "smollm2-1.7b": dict(num_hidden_layers=1, hidden_size=2048, num_attention_heads=32, num_key_value_heads=32, head_dim=64,
                         intermediate_size=8192, vocab_size=2003, rope_theta=130000.0, rms_norm_eps=1e-5,
                         tie_word_embeddings=True, max_position_embeddings=512),
    "llama-3-8b": dict(num_hidden_layers=1, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                       intermediate_size=14336, vocab_size=2001, rope_theta=500000.0, rms_norm_eps=1e-5,
                       tie_word_embeddings=False, max_position_embeddings=512),
}


@pytest.fixture(scope="module")
def family_folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("family")
    # plain N(0, 0.02) weights except sharper queries and keys: wide layers keep activations moderate
    return {name: write_folder(base / name, cfg, seed=11 + i, sharp=False) for i, (name, cfg) in enumerate(FAMILY.items())}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(FAMILY))
def test_family_layer_sizes(family_folders, name, dtype):
    from runtime.engine import load_model, ModelRunner, StepEntry
    folder = family_folders[name]
    V = FAMILY[name]["vocab_size"]
    a, b = random_tokens(1, 150, V), random_tokens(2, 70, V)
    model = load_model(folder, dtype=dtype)
    runner = ModelRunner(model, n_pages=24, page_size=16, max_requests=4)
    runner.create("a"); runner.create("b")
    got = {"a": [], "b": []}
    plan = [[("a", 100), ("b", 3)], [("a", 30), ("b", 1)], [("a", 1), ("b", 66)]] + [[("a", 1)]] * 19
    fed = {"a": 0, "b": 0}
    seqs = {"a": a, "b": b}
    for step in plan:
        entries = [StepEntry(k, seqs[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
        out = runner.step(entries).cpu().numpy()
        row = 0
        for k, n in step:
            got[k].append(out[row:row + n]); row += n; fed[k] += n
    for k in seqs:
        assert fed[k] == len(seqs[k])
        assert_close(np.concatenate(got[k]), plain_logits(folder, seqs[k]), dtype, what=f"{name} request {k}")
    runner.cache.check()
