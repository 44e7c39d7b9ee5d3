"""The Gusedra configuration: parser, round trip, errors, the parts it turns into, and the cache's
bookkeeping for windows with first positions that stay (no GPU)."""
import pytest
import torch

import plain_gusedra as P
from agave_amd.cache import PAGE, GroupKey, GroupPages, KVCache, pages_in_reach
from agave_amd.config import ConfigError, GusedraConfig, find_architecture
from agave_amd.engine.model import tensor_needs
from agave_amd.parts.biased_attention import bucket_of_distance, distance_table


def small():
    return P.config([P.attention2_layer(4, 2, 16, 8, 40, 5, 100, mlp=P.dense(48), buckets=16),
                     P.attention_layer(6, 3, 8, 24, 70, mlp=P.moe(6, 2, 3, 4, 2, 1.5, 20, shared_ff=12)),
                     P.attention_layer(6, 3, 8, 24, 30, kv_from=1),
                     P.attention2_layer(2, 1, 16, 16, None, 0, 50, mlp=P.moe(4, 0, 2, 1, 1, 1.0, 8))], vocab=50, width=32)


def test_parse_round_trip_and_spec():
    cfg = small()
    raw = P.public(cfg)
    arch = find_architecture(raw)
    assert arch.name == "Gusedra"
    c = arch.parse(raw)
    assert isinstance(c, GusedraConfig) and arch.parse(c.to_dict()) == c
    assert c.layers[0].mixer.keep_first == 5 and c.layers[2].mixer.kv_from == 1 and c.layers[3].mixer.window is None
    w = P.random_weights(cfg, 1)
    spec = arch.spec(c, {k: tuple(v.shape) for k, v in w.items()})
    assert [(e.layer, e.memory, e.writes) for e in spec.order] == [(0, 0, True), (1, 1, True), (2, 1, False), (3, 3, True)]
    assert spec.layers[0].mixer.bias.buckets == 16 and spec.layers[0].mixer.bias.max_distance == 100
    assert spec.layers[1].mixer.sink == "l1.mix.sink" and spec.layers[2].mixer.k_proj == ""
    assert spec.layers[1].ffn.n_identity == 2 and spec.layers[1].ffn.shared.intermediate == 12 and spec.layers[2].ffn is None
    assert spec.layers[0].post_mixer_norm.scale_by == "l0.ls1" and spec.layers[0].post_mixer_norm.mult == cfg["residual_mult"]
    needs = {n.name: tuple(n.shape) for n in tensor_needs(spec)}
    # every tensor the model reads is one the plain implementation made, with its shape (the norms and the layer
    # scale of a layer without a feed-forward are not read)
    assert set(w) - set(needs) == {"l2.norm2", "l2.norm2.b", "l2.norm2b", "l2.norm2b.b", "l2.ls2"}
    assert all(tuple(w[n].shape) == s for n, s in needs.items())


@pytest.mark.parametrize("change, message", [
    (lambda r: r["layers"][0].update(type="attention_3"), "unknown layer type"),
    (lambda r: r["layers"][0]["mixer"].pop("bias_max"), "bias_max"),
    (lambda r: r["layers"][0]["mixer"].update(heads=3), "multiple of kv_heads"),
    (lambda r: r["layers"][2]["mixer"].update(kv_from=2), "earlier layer"),
    (lambda r: r["layers"][2]["mixer"].update(kv_from=1, dim=16), "must equal those of layer 1"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=5), "top (5) exceeds"),
    (lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=3), "equal"),
    (lambda r: r["layers"][1]["mlp"].update(kind="sparse"), "unknown kind"),
    (lambda r: r.pop("norm"), "'norm' must be an object"),
])
def test_errors_name_the_key(change, message):
    raw = P.public(small())
    change(raw)
    with pytest.raises(ConfigError) as e:
        GusedraConfig.from_dict(raw)
    assert message in str(e.value)


def test_a_layer_may_not_read_a_layer_that_reads():
    cfg = P.config([P.attention_layer(2, 2, 8, 8, 10), P.attention_layer(2, 2, 8, 8, 10, kv_from=0),
                    P.attention_layer(2, 2, 8, 8, 10, kv_from=1)])
    with pytest.raises(ConfigError) as e:
        GusedraConfig.from_dict(P.public(cfg))
    assert "without keys and values of its own" in str(e.value)


def test_buckets_of_distances():
    # below half the buckets every distance has its own; the last bucket starts at the largest distance at the latest
    for B, D in ((32, 120), (16, 100), (9, 40), (64, 128), (8, 5000)):
        half = B // 2
        got = [bucket_of_distance(n, B, D) for n in range(D + 50)]
        assert got[:half] == list(range(half)) and got[half] == half
        assert all(a <= b for a, b in zip(got, got[1:])) and got[D] == B - 1 and max(got) == B - 1
        assert got == [P.bucket(n, B, D) for n in range(D + 50)]
    # where the logarithms' quotient is a whole number in exact arithmetic, it counts as that number
    assert bucket_of_distance(64, 64, 128) == 32 + 16 and bucket_of_distance(63, 64, 128) == 32 + 15
    rel = torch.randn(16, 3)
    table = distance_table(rel, 16, 100)
    assert table.shape[0] == 3 and torch.equal(table[:, -1], rel[15]) and table.shape[1] <= 101
    for n in (0, 7, 8, 30, table.shape[1] - 1):
        assert torch.equal(table[:, n], rel[bucket_of_distance(n, 16, 100)])
    with pytest.raises(ValueError):
        distance_table(rel, 16, 8)


def test_first_pages_are_kept_and_stand_first_in_the_table():
    key = GroupKey(100, 2, 16, v_head_dim=8, layout="rows_vt", keep_first=70)        # two kept pages
    assert key.kept_pages == 2 and GroupKey(None, 2, 16, keep_first=70).kept_pages == 0
    g = GroupPages(key, 12, 2)
    base, pages = g.plan(0, 0, 50)
    assert base == 2 and len(pages) == 1                     # a short sequence: only the page it has
    g.commit(0, 50)
    base, pages = g.plan(0, 50, 400)                         # positions 50 .. 449: pages 0 .. 7
    assert base == 2 and len(pages) == 8 and len(set(pages)) == 8
    first_two = pages[:2]
    g.commit(0, 450)
    held = g.held(0)
    assert sorted(held) == [0, 1, 5, 6, 7]                   # the window reaches back to 351 = page 5; 0 and 1 stay
    base, pages = g.plan(0, 450, 1)
    assert base == 5 and pages[:2] == first_two and pages[2:] == [held[5], held[6], held[7]]
    for n in range(451, 900):                                # decoding on: never more than kept + window pages
        g.commit(0, n)
        base, pages = g.plan(0, n, 1)
        assert pages[:2] == first_two and base >= 2 and len(pages) <= 2 + pages_in_reach(100, 4096, 1)
        assert len(g.held(0)) <= pages_in_reach(100, 4096, 1, 2)
    g.release(0)
    assert g.pool.n_free == 12
    # the window still overlaps the kept pages: the columns are the pages in order
    g2 = GroupPages(GroupKey(100, 1, 8, layout="rows_vt", keep_first=10), 8, 1)
    base, pages = g2.plan(0, 0, 130)
    assert base == 1 and len(pages) == 3


def test_readers_with_different_windows_share_the_wider_need():
    a = GroupKey(72, 2, 8, v_head_dim=4, layout="rows_vt")
    b = GroupKey(200, 2, 8, v_head_dim=4, layout="rows_vt", keep_first=3)
    both = a.covering(b)
    assert both.window == 200 and both.keep_first == 3 and a.covering(GroupKey(None, 2, 8, v_head_dim=4, layout="rows_vt")).window is None
    assert a.covering(GroupKey(72, 2, 16, v_head_dim=4, layout="rows_vt")) is None
    cache = KVCache({0: both}, {}, 2, {both: 10}, torch.float32, None, 1024)
    s = cache.alloc_slot()
    cache.check_pieces([s], [[300], [300]])
    cache.plan_step([s], [300])
    cache.commit_step([s], [300])
    assert sorted(cache.groups[0].held(s)) == [0, 1, 2, 3, 4]     # 300 - 200 + 1 = 101: page 1 on, and page 0 kept
    cache.free_slot(s)
