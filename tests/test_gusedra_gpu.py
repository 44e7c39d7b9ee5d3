"""The Gusedra decoder through the engine, against ``plain_gusedra``: whole prompts, decoding token by token,
prompts in pieces down to two tokens, batches of unequal requests, slots and pages used again, long decoding
across the windows' and the pages' borders, other sizes, a layer that reads another layer's keys through a
window of its own, greedy generation through the engine's entry point, the command line and the trace replay
tool."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import engine_utils as U
import plain_gusedra as P

pytestmark = pytest.mark.gpu

def reading(layer, source):
    """The layer without keys and values of its own, reading those of layer ``source``."""
    layer["mixer"]["kv_from"] = source
    return layer


CONFIGS = {
    # both mixers, grouped heads, values wider and narrower than keys, windows that are no multiples of a page and
    # differ from layer to layer, a reader with a wider window than the layer it reads, both feed-forwards
    "mixed": lambda: P.config([
        P.attention2_layer(4, 2, 16, 24, 40, 5, 100, mlp=P.dense(96), buckets=16),
        P.attention_layer(6, 3, 24, 8, 50, mlp=P.moe(6, 2, 3, 4, 2, 1.5, 24, shared_ff=16)),
        P.attention_layer(6, 3, 24, 8, 90, kv_from=1, mlp=P.dense(40)),
        P.attention2_layer(2, 1, 32, 32, 70, 66, 60, mlp=P.moe(5, 0, 2, 1, 1, 0.8, 40), buckets=9),
        P.attention_layer(3, 3, 24, 8, 64, kv_from=1)], vocab=131, width=64),
    # a width that is no multiple of 8 (no matrix-core packing), heads of 20 and 12, no masks at all, one key head,
    # a reader with a narrower window than its source, a router without identity experts or groups, no shared expert
    "odd": lambda: P.config([
        P.attention_layer(5, 1, 20, 12, None, mlp=P.moe(3, 0, 1, 1, 1, 1.0, 30)),
        P.attention2_layer(3, 3, 12, 20, None, 0, 300, mlp=None, buckets=20),
        P.attention_layer(5, 1, 20, 12, 17, kv_from=0, mlp=P.dense(50))], vocab=97, width=60, residual_mult=1.0),
    # readers of the other kind than their source: slopes and sinks over the keys of a layer with a learned bias and kept
    # positions (the pages then serve the reader's wider window and keep the source's first positions), and the reverse;
    # a single layer of each kind without a feed-forward at the end; one router output more than experts, all chosen
    "cross": lambda: P.config([
        P.attention2_layer(4, 2, 16, 32, 40, 5, 64, mlp=P.moe(3, 1, 4, 1, 1, 1.0, 16), buckets=10),
        P.attention_layer(6, 2, 16, 32, 60, kv_from=0, mlp=P.dense(48)),
        P.attention_layer(2, 2, 32, 16, 100, mlp=None),
        reading(P.attention2_layer(4, 2, 32, 16, 30, 70, 200, mlp=None, buckets=14), 2),
    ], vocab=77, width=48, eps=1e-3, residual_mult=1.5),
    # sizes the matrix cores take, several pages of kept positions, everything a multiple of 16
    "even": lambda: P.config([
        P.attention2_layer(8, 2, 64, 64, 128, 130, 500, mlp=P.moe(8, 0, 2, 4, 2, 2.5, 64, shared_ff=64), buckets=32),
        P.attention_layer(4, 4, 32, 64, 96, mlp=P.dense(256))], vocab=256, width=128, residual_mult=0.6),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(name, decided=False):
        if (name, decided) not in made:
            cfg = CONFIGS[name]()
            w = P.random_weights(cfg, seed=len(name), decided_routing=decided)
            folder = U.write_model(str(tmp_path_factory.mktemp(name)), P.public(cfg), w)
            made[(name, decided)] = (cfg, w, folder)
        return made[(name, decided)]
    return get


def engine(folder, dtype, **kw):
    from agave_amd.engine import Engine
    kw.setdefault("max_slots", 4)
    kw.setdefault("max_context", 512)
    return Engine.from_folder(folder, dtype=dtype, **kw)


def close(got, ref, dtype, what):
    scale = float(ref.abs().max())
    err = (got.double() - ref).abs().max(dim=-1).values
    tol = 3e-5 if dtype == "float32" else 0.04
    assert float(err.max()) <= tol * scale, f"{what}: error {float(err.max()):.3e} of {scale:.3e} at row {int(err.argmax())}"


def model_for(models, name, dtype):
    # in bfloat16 the choice of experts is decided by the corrections (a close call would go either way)
    return models(name, decided=(dtype == "bfloat16"))


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_and_pieces(models, name, dtype):
    cfg, w, folder = model_for(models, name, dtype)
    eng = engine(folder, dtype)
    toks = U.random_tokens(260, cfg["vocab"], 1)
    ref = P.forward(cfg, w, toks)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 150), ref, dtype, "the last 150 one by one, across windows and page borders")
    close(U.run_tail(eng, toks, 259), ref, dtype, "token by token from the first")
    for piece in (2, 7, 64, 100):                 # the prompt enters in pieces of this many tokens
        eng.prefill_chunk = piece
        close(U.run_whole(eng, toks[:170]), ref[:170], dtype, f"pieces of {piece}")
    eng.prefill_chunk = 0
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_streams_after_every_layer(models):
    """The residual stream after each layer, read off the engine between its blocks."""
    from agave_amd.parts.norm import add_branch
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    eng.use_graphs = False
    toks = U.random_tokens(90, cfg["vocab"], 4)
    want = []
    P.forward(cfg, w, toks, streams=want)
    seen = []
    for b in eng.model.blocks[1:]:
        def wrapped(h, pending, step, memory, writes, inner=b.forward):
            copy = h.clone()
            add_branch(copy, pending)
            seen.append(copy.cpu())
            return inner(h, pending, step, memory, writes)
        b.forward = wrapped
    U.run_whole(eng, toks)
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert float((got.double() - ref).abs().max()) < 3e-5 * float(ref.abs().max()), f"after layer {i}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(models, dtype):
    cfg, w, folder = model_for(models, "mixed", dtype)
    eng = engine(folder, dtype, max_slots=3, max_context=256, cache_tokens=448)
    for b, (lens, first) in enumerate([((50, 1, 130), (30, 1, 2)), ((70, 33), (69, 1)), ((90, 9, 140), (5, 9, 101))]):
        reqs = [U.random_tokens(n, cfg["vocab"], 10 * b + i) for i, n in enumerate(lens)]
        outs = U.run_batched(eng, reqs, first)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            close(o, P.forward(cfg, w, r), dtype, f"batch {b} request {i}")
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_the_cache_as_the_mixers_asked(models):
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    keys = {eng.cache.group_keys[g] for g in eng.cache.group_of_memory.values()}
    assert set(eng.cache.group_of_memory) == {0, 1, 3}            # layers 2 and 4 read layer 1's memory
    by_mem = {m: eng.cache.group_keys[g] for m, g in eng.cache.group_of_memory.items()}
    assert by_mem[1].window == 90 and by_mem[0].keep_first == 5 and by_mem[3].kept_pages == 2      # the widest reader's window
    assert all(k.layout == "rows_vt" for k in keys) and by_mem[1].v_head_dim == 8
    from agave_amd.ops import library
    slot = eng.alloc_slot()
    eng.step([slot], [[1, 2]])
    eng.free_slot(slot)
    loaded = library.loaded_paths()
    assert any(p.endswith("attention_biased.so") for p in loaded) and any(p.endswith("routed_ffn.so") for p in loaded)


def test_long_decoding_holds_few_pages(models):
    """Decoding far past the windows: a sequence holds the kept pages and the window's, and the logits stay right."""
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32", max_slots=1, max_context=1024, cache_tokens=64 * 7)
    toks = U.random_tokens(700, cfg["vocab"], 9)
    ref = P.forward(cfg, w, toks)
    close(U.run_tail(eng, toks, 500), ref, "float32", "500 tokens decoded through a pool of seven pages")


def test_an_early_token_that_stays_visible_moves_late_logits(models):
    """A change of the third token (one of the kept first positions of layer 0) moves the logits 300 tokens later,
    where no window reaches it; a change of the token just behind the kept ones does not reach that far."""
    cfg = P.config([P.attention2_layer(2, 1, 16, 16, 20, 5, 400, mlp=None, buckets=8)], vocab=60, width=32)
    w = P.random_weights(cfg, 3)
    from agave_amd.engine import Engine
    eng = Engine.from_tensors(P.public(cfg), {k: v.bfloat16() for k, v in w.items()}, dtype="float32", max_slots=2, max_context=512)
    toks = U.random_tokens(330, 60, 3)
    kept, behind = list(toks), list(toks)
    kept[2] = (toks[2] + 11) % 60
    behind[5] = (toks[5] + 11) % 60
    ref, ref_kept, ref_behind = (P.forward(cfg, w, t) for t in (toks, kept, behind))
    moved = float((ref[-1] - ref_kept[-1]).abs().max())
    assert moved > 1e-3 * float(ref.abs().max()) and float((ref[-1] - ref_behind[-1]).abs().max()) < 1e-9
    for t, r in ((toks, ref), (kept, ref_kept)):
        got = U.run_tail(eng, t, 40)
        assert float((got[-1].double() - r[-1]).abs().max()) < 0.02 * moved
        close(got, r, "float32", "kept first positions")


@pytest.mark.parametrize("dtype", ["float32"])
def test_greedy_generation_through_the_entry_point(models, dtype):
    from agave_amd.sampling import SamplingParams
    cfg, w, folder = models("mixed")
    eng = engine(folder, dtype, max_slots=2, max_context=128)
    prompts = [U.random_tokens(7, cfg["vocab"], 50), U.random_tokens(45, cfg["vocab"], 51), U.random_tokens(1, cfg["vocab"], 52)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8))      # three requests, two slots: a slot is used again
    for p, r in zip(prompts, res):
        seq = list(p)
        for _ in range(8):
            seq.append(P.argmax_first(P.forward(cfg, w, seq)[-1]))
        assert list(r.tokens) == seq[len(p):]


def test_command_line_and_trace_replay(models, tmp_path):
    cfg, w, folder = models("odd", decided=True)
    root = U.ROOT
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "agave_amd"), folder, "3 17 5 80 2", "-n", "5", "--dtype", "float32",
                          "--json"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    seq = [3, 17, 5, 80, 2]
    for _ in range(5):
        seq.append(P.argmax_first(P.forward(cfg, w, seq)[-1]))
    got = json.loads(out.stdout.strip().splitlines()[-1])
    assert got["outputs"][0]["tokens"] == seq[5:] and got["outputs"][0]["prompt_tokens"] == 5
    batches = [[U.random_tokens(n, cfg["vocab"], 70 + n) for n in (40, 3, 110)], [U.random_tokens(n, cfg["vocab"], 90 + n) for n in (25, 60)]]
    firsts = [(8, 3, 78), (1, 59)]
    records, where = U.trace_steps_batched(batches, firsts)
    for dtype in ("float32", "bfloat16"):
        steps = U.run_trace_tool(folder, dtype, records, str(tmp_path / dtype), 256, cfg["vocab"])
        for bi, reqs in enumerate(batches):
            for i, r in enumerate(reqs):
                got = torch.from_numpy(np.stack([steps[s][row] for s, row in where[(bi, i)]]))
                close(got, P.forward(cfg, w, r), dtype, f"replay {dtype} batch {bi} request {i}")
