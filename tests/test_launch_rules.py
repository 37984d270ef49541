"""The rules that pick a kernel's form are plain functions of sizes: their decisions at the points where
measurements settled them (profiles/prompt_attention_forms_and_the_rule_that_picks.txt and
profiles/decode_attention_launch_shapes_and_the_rule_that_picks.txt), so that a change of a rule shows."""
import pytest

from runtime.kernels.attention import fused_merge_splits, prompt_form, rows_launch, rows_stream_loads


@pytest.mark.parametrize("heads, kv_heads, dim, rows, form", [
    (9, 3, 64, 2048, ("square", 1, 2)),       # about one block a compute unit: two halves a block
    (9, 3, 64, 3072, ("square", 1, 2)),       # 441 blocks, a long chain: still halves
    (9, 3, 64, 6144, ("square", 2, 2)),       # 440 blocks of 128 items from 3,072 keys on
    (9, 3, 64, 8192, ("square", 2, 1)),
    (32, 32, 64, 2048, ("square", 2, 1)),
    (32, 32, 64, 4096, ("square", 3, 1)),     # 2,048 blocks of 64 items: 192 items a block
    (32, 8, 128, 2048, ("square", 2, 1)),
    (32, 8, 128, 3072, ("square", 3, 1)),     # large heads: 192 items from 1,100 blocks on
    (16, 4, 64, 3072, ("square", 2, 2)),
    (16, 4, 64, 6144, ("square", 2, 1)),      # 768 blocks of 128 items: the halves would crowd the compute units
])
def test_prompt_attention_form_at_measured_points(heads, kv_heads, dim, rows, form):
    assert tuple(prompt_form(rows, 1, rows, heads, kv_heads, dim, 16)) == form


def test_prompt_attention_form_needs_long_portions_and_pages_of_eight_keys():
    assert prompt_form(40, 8, 3000, 9, 3, 64, 16)[0] == "tiles"        # many short portions
    assert prompt_form(2048, 1, 2048, 9, 3, 64, 4)[0] != "square"      # the copying waves take 8 keys of a page
    assert prompt_form(2048, 1, 2048, 2, 2, 256, 16)[0] == "tiles"     # heads of more than 128 coordinates


@pytest.mark.parametrize("blocks, keys, group, dim, launch", [
    (3, 2048, 3, 64, (8, 8)),          # one request of the 135M sizes
    (24, 2048, 3, 64, (8, 8)),         # eight
    (192, 2048, 3, 64, (8, 1)),        # 64: one block of eight waves a compute unit, no split
    (24, 8192, 3, 64, (8, 10)),        # eight waves at long contexts too
    (3, 8192, 3, 64, (8, 16)),         # one request at 8k: 16 splits of two steps a wave, not 31 of one
    (12, 8192, 3, 64, (8, 16)),
    (3, 32768, 3, 64, (8, 32)),        # at 32k a wave has steps enough for 32 splits
    (12, 32768, 3, 64, (8, 21)),
    (96, 8192, 3, 64, (4, 16)),        # but from 16 rows on four waves and about 1,536 blocks in all (non-temporal loads)
    (192, 32768, 3, 64, (4, 8)),
    (48, 8192, 3, 64, (8, 5)),         # 16 rows at 8k stay
    (48, 32768, 3, 64, (4, 16)),
    (24, 512, 3, 64, (8, 1)),          # two steps a wave: nothing to split
    (384, 512, 3, 64, (4, 1)),
    (8, 8192, 4, 128, (4, 32)),        # at most 32 splits
    (64, 2048, 4, 128, (4, 8)),
    (512, 2048, 4, 128, (4, 1)),
])
def test_decode_attention_launch_at_measured_points(blocks, keys, group, dim, launch):
    assert tuple(rows_launch(blocks, keys, group, dim)) == launch


@pytest.mark.parametrize("blocks, keys, group, dim, streams", [
    (24, 2048, 3, 64, True),           # eight requests of the 135M sizes: 192 blocks of eight waves, one step a wave
    (3, 2048, 3, 64, False),           # one request: few blocks
    (192, 2048, 3, 64, False),         # 64 requests unsplit: a wave walks eight steps
    (24, 8192, 3, 64, False),
    (12, 8192, 3, 64, True),           # 4 requests at 8k: 21 splits, a step and a half a wave
    (2048, 2048, 1, 64, True),         # four waves a block: always
    (8, 8192, 4, 128, True),           # large heads: always
    (512, 512, 4, 128, True),
])
def test_decode_attention_streams_keys_and_values_at_measured_points(blocks, keys, group, dim, streams):
    waves, splits = rows_launch(blocks, keys, group, dim)
    assert rows_stream_loads(blocks, keys, waves, splits, dim) is streams


@pytest.mark.parametrize("splits, rows, fused", [
    (8, 8, 8),         # eight requests of the 135M sizes at 2k: the output projection merges all eight
    (10, 8, 8),        # at 8k the rule asks for ten: eight merged there still beat ten and a merge kernel
    (8, 16, 4),        # more than 8 rows bring at most four each
    (4, 16, 4),
    (32, 1, None),     # one row at 8k to 32k keeps its 32 splits: a quarter of the blocks would cost more than the merge kernel
    (24, 1, None),
    (3, 4, 2),
    (1, 8, None),
])
def test_splits_that_the_output_projection_merges_itself(splits, rows, fused):
    assert fused_merge_splits(splits, rows, lambda n: True) == fused
    assert fused_merge_splits(splits, rows, lambda n: False) is None
