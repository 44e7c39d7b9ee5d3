"""Rilenex without a GPU: the configuration's parser, the model spec it turns into, the tensors
the parts ask for, and the cache's bookkeeping for a group whose queries see their own chunk only."""
import copy

import pytest
import torch

import plain_rilenex as P
from agave_amd.cache import PAGE, GroupKey, GroupPages, KVCache, StateNeed, pages_in_reach
from agave_amd.config import ConfigError, RilenexConfig, find_architecture
from agave_amd.config.spec import (DenseFfnSpec, GatedDeltaSpec, Hgrn2Spec, ParallelMixerSpec, TalkingAttentionSpec)
from agave_amd.engine.model import tensor_needs
from agave_amd.weights.loader import WeightError, check_tensors


def small_config():
    return P.config([P.parallel_layer((4, 2, 24, 16, 2, 48, 16, 10000.0), (4, 2, 16, 24, 3), ff=96),
                     P.hgrn2_layer(3, 20, 12),
                     P.hgrn2_layer(2, 16, 16, ff=80)], vocab=131, width=64)


def test_found_by_its_single_name_and_parsed():
    raw = small_config()
    arch = find_architecture(raw)
    assert arch.name == "Rilenex"
    cfg = arch.parse(raw)
    assert isinstance(cfg, RilenexConfig) and cfg.vocab == 131 and cfg.width == 64 and len(cfg.layers) == 3
    assert cfg.layers[0].ff == 96 and cfg.layers[1].ff is None
    assert cfg.layers[0].mixer.left.chunk == 48 and cfg.layers[0].mixer.right.conv == 3
    assert arch.parse(cfg.to_dict()) == cfg


def test_spec_names_the_parts_with_their_constants():
    raw = small_config()
    arch = find_architecture(raw)
    spec = arch.spec(arch.parse(raw), None)
    assert spec.embed_scale == 1.0 and spec.head_weight == "head" and spec.final_norm.weight == "final.norm"
    assert not spec.final_norm.add_one
    l0, l1, l2 = spec.layers
    assert l0.kind == "prenorm" and isinstance(l0.mixer, ParallelMixerSpec) and l0.mixer.scales == (0.7, 1.2)
    left, right = l0.mixer.branches
    assert isinstance(left, TalkingAttentionSpec) and left.chunk == 48 and left.v_head_dim == 16 and left.conv_taps == 2
    assert left.position.interleaved and left.position.rotary_dim == 16 and left.talk == "l0.mix.left.talk"
    assert isinstance(right, GatedDeltaSpec) and right.n_kv_heads == 2 and right.unit_eps == 1e-6
    assert isinstance(l0.ffn, DenseFfnSpec) and l0.ffn.activation == "xielu" and l0.ffn.act_params == "l0.mlp.act"
    assert isinstance(l1.mixer, Hgrn2Spec) and l1.ffn is None and l1.pre_ffn_norm is None
    assert isinstance(l2.ffn, DenseFfnSpec)


def test_inner_sizes_come_from_the_checkpoint():
    raw = small_config()
    arch = find_architecture(raw)
    w = P.random_weights(raw, 1, ranks=(7, 9))
    spec = arch.spec(arch.parse(raw), {k: tuple(v.shape) for k, v in w.items()})
    right = spec.layers[0].mixer.branches[1]
    assert (right.decay_rank, right.gate_rank) == (7, 9)
    assert check_tensors({k: tuple(v.shape) for k, v in w.items()}, tensor_needs(spec)) == []
    # a wrong shape and a missing tensor are named together
    bad = {k: tuple(v.shape) for k, v in w.items() if k != "l1.mix.lower"}
    bad["l0.mix.left.talk"] = (4, 3)
    with pytest.raises(WeightError) as e:
        check_tensors(bad, tensor_needs(spec))
    assert "l1.mix.lower" in str(e.value) and "l0.mix.left.talk" in str(e.value)


def test_a_side_without_mask_or_convolution():
    raw = copy.deepcopy(small_config())
    left = raw["layers"][0]["mixer"]["left"]
    left["mask"] = None
    left.pop("conv")
    cfg = RilenexConfig.from_dict(raw)
    assert cfg.layers[0].mixer.left.chunk is None and cfg.layers[0].mixer.left.conv == 0
    spec = cfg.model_spec(None)
    talk = spec.layers[0].mixer.branches[0]
    assert talk.chunk is None and talk.conv_taps == 0
    assert not any(n.name.endswith("left.q.conv") for n in tensor_needs(spec))
    assert RilenexConfig.from_dict(cfg.to_dict()) == cfg


@pytest.mark.parametrize("edit, word", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0].__setitem__("type", "other"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 26), "rot"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].pop("size"), "size"),
    (lambda c: c["layers"][0]["mixer"]["right"].pop("conv"), "conv"),
    (lambda c: c["layers"][2].__setitem__("mlp", {"kind": "routed", "ff": 8}), "dense"),
    (lambda c: c["norm"].__setitem__("eps", 0), "eps"),
])
def test_bad_configurations_are_named(edit, word):
    raw = copy.deepcopy(small_config())
    edit(raw)
    with pytest.raises(ConfigError) as e:
        RilenexConfig.from_dict(raw)
    assert word in str(e.value)


# ---------------------------------------------------------------- the cache for chunks
def test_chunk_reach_and_first_needed():
    key = GroupKey(None, 2, 24, chunk=48, v_head_dim=16, layout="rows")
    assert key.reach == 48
    assert [key.first_needed(n) for n in (0, 47, 48, 95, 96, 200)] == [0, 0, 48, 48, 96, 192]
    both = GroupKey(10, 2, 24, chunk=48)
    assert both.reach == 10 and both.first_needed(50) == 48 and both.first_needed(70) == 61
    assert pages_in_reach(key.reach, 4096, 1) == 2          # a chunk of 48 touches at most two pages
    assert pages_in_reach(GroupKey(None, 1, 8, chunk=200).reach, 4096, 1) == 5


def test_pages_of_finished_chunks_are_given_back_and_used_again():
    key = GroupKey(None, 1, 8, chunk=100, v_head_dim=4, layout="rows")
    g = GroupPages(key, n_pages=4, max_slots=2)
    base, pages = g.plan(0, 0, 90)                           # positions 0..89: pages 0 and 1
    assert base == 0 and len(pages) == 2
    g.commit(0, 90)
    assert sorted(g.held(0)) == [0, 1]
    base, pages = g.plan(0, 90, 20)                          # 90..109: chunk 1 starts at 100, inside page 1
    g.commit(0, 110)
    assert sorted(g.held(0)) == [1]                          # page 0 holds nothing a later query sees
    base, pages = g.plan(0, 110, 150)                        # up to 259: pages 1..4; three new ones, and page 0's id is free for one of them
    assert base == 1 and len(pages) == 4
    g.commit(0, 260)                                         # chunk 2 starts at 200: page 3
    assert sorted(g.held(0)) == [3, 4]
    g.release(0)
    assert g.pool.n_free == 4


def test_row_layout_and_named_state_bookkeeping():
    key = GroupKey(None, 2, 24, chunk=48, v_head_dim=16, layout="rows")
    needs = {0: {"b0.conv": StateNeed((1, 10)), "b1.S": StateNeed((2, 3, 4))}, 1: StateNeed((5,))}
    cache = KVCache({0: key}, needs, max_slots=2, pages_per_group={key: 6}, dtype=torch.float32, device=None,
                    max_context=512)
    assert set(cache.state[0]) == {"b0.conv", "b1.S"} and cache.state[1] is None
    s = cache.alloc_slot()
    pos0, plans = cache.plan_step([s], [130])
    assert pos0 == [0] and len(plans[0].rows[0]) == 3
    cache.commit_step([s], [130])
    assert sorted(cache.groups[0].held(s)) == [1, 2]         # the chunk of position 130 starts at 96
    cache.free_slot(s)
    with pytest.raises(Exception):
        KVCache({0: GroupKey(None, 2, 24, v_head_dim=16)}, {}, 1, {GroupKey(None, 2, 24, v_head_dim=16): 1}, torch.float32, None, 64)
