"""The configuration that the benchmark measures, whole: the SmolLM2-135M preset with all of its 30 layers and its
vocabulary of 49,152, random weights.  A 300-token prompt in three portions, then 8 single tokens, in float32 and
in bfloat16, launched kernel by kernel and as captured programs, against the plain implementation (which takes the
whole sequence at once in float64).  Thirty layers of bfloat16 rounding are held to the same bound as two."""
import numpy as np
import pytest

from conftest import assert_close, plain_logits, random_tokens, write_folder

pytestmark = pytest.mark.gpu

KEYS = ("num_hidden_layers", "hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
        "vocab_size", "rope_theta", "rms_norm_eps", "tie_word_embeddings")


@pytest.fixture(scope="module")
def full_folder(tmp_path_factory):
    from runtime.config import preset
    raw = preset("smollm2-135m")
    cfg = {k: raw[k] for k in KEYS if k in raw}
    cfg.setdefault("head_dim", raw["hidden_size"] // raw["num_attention_heads"])
    cfg["max_position_embeddings"] = 512
    assert (cfg["num_hidden_layers"], cfg["vocab_size"], cfg["hidden_size"]) == (30, 49152, 576)
    # Queries, keys and the other matrices at twice the width of N(0, 0.02): attention is not uniform (scores spread
    # over about one unit) and every layer adds to the residual stream what the embedding brought.  Sharper weights
    # are of no use at this depth: rounding then grows from layer to layer, evenly over all rows, in float32 (2 layers
    # 9e-6, 8 layers 5e-5, 30 layers 3e-4 of the largest logit with the factors 6 and 4 that the tiny models take)
    # as in bfloat16 (rmse 0.03, 0.15, 0.48), until the bound measures the weights and not the engine.
    return write_folder(tmp_path_factory.mktemp("full") / "smollm2-135m", cfg, seed=5, sharp=(2.0, 2.0)), cfg


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_all_layers_and_the_whole_vocabulary(full_folder, dtype, execution):
    from runtime.engine import load_model, ModelRunner, StepEntry
    folder, cfg = full_folder
    tokens = random_tokens(3, 308, cfg["vocab_size"])
    model = load_model(folder, dtype=dtype)
    runner = ModelRunner(model, n_pages=24, page_size=16, max_requests=2, execution=execution)
    ref = plain_logits(folder, tokens)
    # twice: a captured program is recorded at the second step of its shape, so the second pass replays them all
    for request in ("first", "second") if execution == "graph" else ("first",):
        runner.create(request)
        got, at = [], 0
        for n in (100, 37, 163) + (1,) * 8:
            got.append(runner.step([StepEntry(request, tokens[at:at + n], list(range(n)))]).float().cpu().numpy())
            at += n
        assert at == len(tokens)
        assert_close(np.concatenate(got), ref, dtype, what=f"{dtype}/{execution}/{request} pass")
        runner.release(request)
    runner.cache.check()
