"""Seeded random configurations of the architecture (head counts and grouping, head sizes in
steps of 4, widths and vocabularies of any parity, one to three layers, tied or not): a short
mixed trace in float32 and bfloat16 against the plain implementation.  What the fixed tiny
configurations do not happen to cover shows here."""
import numpy as np
import pytest

from conftest import assert_close, plain_logits, random_tokens, write_folder

pytestmark = pytest.mark.gpu


def random_config(seed):
    rng = np.random.default_rng(1000 + seed)
    kv = int(rng.choice([1, 2, 3, 4]))
    heads = kv * int(rng.choice([1, 2, 3, 5, 8]))
    head_dim = int(rng.choice([4, 8, 12, 16, 20, 24, 32, 40, 48, 64, 80, 96, 128]))
    hidden = int(rng.choice([2, 4, 6, 8])) * int(rng.integers(5, 40))
    return dict(num_hidden_layers=int(rng.integers(1, 4)), hidden_size=hidden, num_attention_heads=heads,
                num_key_value_heads=kv, head_dim=head_dim, intermediate_size=int(rng.integers(9, 200)) * int(rng.choice([1, 2, 8])),
                vocab_size=int(rng.integers(50, 700)), rope_theta=float(rng.choice([1e4, 5e5, 1e6, 777.0])),
                rms_norm_eps=float(rng.choice([1e-5, 1e-6, 1e-3])), tie_word_embeddings=bool(rng.integers(0, 2)),
                max_position_embeddings=256)


@pytest.mark.parametrize("seed", range(10))
def test_random_configuration(tmp_path, seed):
    from runtime.engine import load_model, ModelRunner, StepEntry
    cfg = random_config(seed)
    folder = write_folder(tmp_path / "m", cfg, seed=seed)
    V = cfg["vocab_size"]
    seqs = {"a": random_tokens(seed, 96, V), "b": random_tokens(seed + 50, 41, V), "c": random_tokens(seed + 90, 66, V)}
    plan = [[("a", 37), ("b", 2)], [("a", 1), ("b", 30), ("c", 5)], [("a", 20), ("b", 1), ("c", 1)],
            [("a", 2), ("b", 8), ("c", 59)], [("a", 30), ("c", 1)]]
    for dtype in ("float32", "bfloat16"):
        model = load_model(folder, dtype=dtype)
        runner = ModelRunner(model, n_pages=14, page_size=16, max_requests=4, execution="graph")
        got, fed = {k: [] for k in seqs}, {k: 0 for k in seqs}
        for k in seqs:
            runner.create(k)
        for step in plan:
            entries = [StepEntry(k, seqs[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for _ in range(6):   # decode-only steps (captured programs in graph mode)
            entries = [StepEntry("a", [seqs["a"][fed["a"]]], [0])]
            got["a"].append(runner.step(entries).cpu().numpy()); fed["a"] += 1
        for k in seqs:
            done = fed[k]
            assert_close(np.concatenate(got[k]), plain_logits(folder, seqs[k][:done])[:done], dtype, what=f"{cfg} request {k}")
        runner.cache.check()
