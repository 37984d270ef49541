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
                         tie_word_embeddings=True, max_position_embeddings=768),
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
    # (portions, then six steps of two single tokens and thirteen of one: the products of one and of two rows)
    plan = [[("a", 100), ("b", 3)], [("a", 30), ("b", 1)], [("a", 1), ("b", 60)]] + [[("a", 1), ("b", 1)]] * 6 + [[("a", 1)]] * 13
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


@pytest.mark.parametrize("name", ["smollm2-1.7b", "llama-3-8b"])
def test_a_cut_across_the_library_threshold_changes_rounding_only(family_folders, name):
    """With large weights a portion of more than 64 rows takes the vendor library's bf16 product, whose output
    projection and down projection are rounded to bfloat16 before they are added to the float residual; 64 rows
    and fewer add the float accumulator.  The same prompt cut at 65 + 35 and at 64 + 36 rows therefore differs by
    that rounding, and by nothing more: the difference between the two runs stays far inside the bound that
    either holds against the plain implementation."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.kernels import ops
    from conftest import BF16_RMSE
    folder = family_folders[name]
    V = FAMILY[name]["vocab_size"]
    tokens = random_tokens(5, 100, V)
    model = load_model(folder, dtype="bfloat16")
    assert ops.library_ok(65, model.layers[0].mixer.w_out) and not ops.library_ok(64, model.layers[0].mixer.w_out)
    runs = []
    for first in (65, 64):
        runner = ModelRunner(model, n_pages=16, page_size=16, max_requests=2)
        runner.create("p")
        out = [runner.step([StepEntry("p", tokens[:first], list(range(first)))]).float().cpu().numpy(),
               runner.step([StepEntry("p", tokens[first:], list(range(100 - first)))]).float().cpu().numpy()]
        runs.append(np.concatenate(out))
    ref = plain_logits(folder, tokens)
    for got in runs:
        assert_close(got, ref, "bfloat16", what=name)
    between = np.linalg.norm(runs[0] - runs[1]) / np.linalg.norm(ref)
    assert between < BF16_RMSE / 4, f"the two cuts differ by {between:.3e}"


@pytest.mark.parametrize("execution", ["eager", "graph"])
def test_decoding_at_a_context_whose_keys_are_split_over_blocks(family_folders, execution, monkeypatch):
    """From a context of about 550 keys on (more than two 32-key steps a wave), a decode step of few rows splits every row's keys over blocks; at the
    135M sizes the output projection then merges the blocks' partial results itself (no merge kernel).  Three requests
    of very different lengths decode together (the short one's later splits see no key at all), then one alone."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    name = "smollm2-135m"
    folder = family_folders[name]
    V = FAMILY[name]["vocab_size"]
    seqs = {"long": random_tokens(11, 700, V), "mid": random_tokens(12, 310, V), "short": random_tokens(13, 20, V)}
    model = load_model(folder, dtype="bfloat16")
    runner = ModelRunner(model, n_pages=80, page_size=16, max_requests=4, execution=execution)
    fed, got = {}, {k: [] for k in seqs}
    for k, toks in seqs.items():
        runner.create(k)
        fed[k] = len(toks) - 12
        runner.step([StepEntry(k, toks[:fed[k]], [])])
    from runtime.kernels import ops
    seen = []
    real = ops.gemm_merged

    def spy(partials, *args, **kwargs):
        seen.append(partials[2])
        return real(partials, *args, **kwargs)

    monkeypatch.setattr(ops, "gemm_merged", spy)
    for step in range(12):
        live = [k for k in seqs if step < 8 or k == "long"]          # the last four steps: one row
        out = runner.step([StepEntry(k, [seqs[k][fed[k]]], [0]) for k in live]).float().cpu().numpy()
        for row, k in zip(out, live):
            got[k].append(row); fed[k] += 1
    assert any(n is not None and n >= 2 for n in seen), "no decode step left its partial results to the output projection"
    for k, toks in seqs.items():
        ref = plain_logits(folder, toks)
        assert_close(np.stack(got[k]), ref[len(toks) - 12:len(toks) - 12 + len(got[k])], "bfloat16", what=f"request {k}")
    runner.cache.check()
