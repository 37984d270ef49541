"""The order of layers as data: what a model checks when an entry of the order reads another entry's cache."""
import pytest


def build(schedule, second=None, first=None):
    from runtime import make_part
    from runtime.models import Model
    from runtime.parts import TokenEmbedding, LMHead
    position = make_part("position", "none", head_dim=16, max_positions=32)

    def block(n, **attention):
        args = dict(hidden=24, heads=4, kv_heads=2, head_dim=16, position=position)
        args.update(attention)
        return make_part("block", "prenorm", mixer_norm=make_part("norm", "rmsnorm", name=n + ".n1", dim=24, eps=1e-5),
                         mixer=make_part("mixer", "attention", name=n + ".attn", **args),
                         ffn_norm=make_part("norm", "rmsnorm", name=n + ".n2", dim=24, eps=1e-5),
                         ffn=make_part("ffn", "gated_mlp", name=n + ".mlp", hidden=24, intermediate=32))
    layers = [block("l0", **(first or {})), block("l1", **(second or {"own_kv": False}))]
    return Model(None, TokenEmbedding("embed", 50, 24), layers, make_part("norm", "rmsnorm", name="final", dim=24, eps=1e-5),
                 LMHead("head", 50, 24), schedule=schedule, max_positions=32, vocab_size=50)


def test_a_layer_may_read_the_cache_of_an_earlier_one():
    from runtime.models import ScheduleEntry
    model = build([ScheduleEntry(0), ScheduleEntry(1, reads=0)])
    assert set(model.cache_needs()) == {0} and model.site_of(1) == 0
    # twice: each reading run names the entry whose cache it reads
    model = build([ScheduleEntry(0), ScheduleEntry(1, reads=0), ScheduleEntry(0), ScheduleEntry(1, reads=2)])
    assert set(model.cache_needs()) == {0, 2} and [model.site_of(i) for i in range(4)] == [0, 0, 2, 2]


def test_what_a_reading_layer_expects_is_checked_against_what_is_kept():
    from runtime.models import ScheduleEntry
    order = [ScheduleEntry(0), ScheduleEntry(1, reads=0)]
    with pytest.raises(ValueError, match="keeps 2 x 16"):
        build(order, second={"own_kv": False, "kv_heads": 1})
    with pytest.raises(ValueError, match="keeps the last 8"):
        build(order, first={"window": 8})                                  # the reader looks back over all keys
    with pytest.raises(ValueError, match="keeps the last 8"):
        build(order, first={"window": 8}, second={"own_kv": False, "window": 12})
    build(order, first={"window": 8}, second={"own_kv": False, "window": 8})
    build(order, first={"window": 8}, second={"own_kv": False, "window": 5})
    with pytest.raises(ValueError, match="keeps one"):
        build(order, second={"own_kv": True})                              # a mixer with a cache of its own reads no other
    with pytest.raises(ValueError, match="earlier entry"):
        build([ScheduleEntry(1, reads=1), ScheduleEntry(0)])
    with pytest.raises(ValueError, match="earlier entry"):
        build([ScheduleEntry(0), ScheduleEntry(1, reads=0), ScheduleEntry(1, reads=1)])   # the entry it names keeps none
