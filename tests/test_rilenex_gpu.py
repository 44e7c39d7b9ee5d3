"""The Rilenex decoder through the engine, against ``plain_rilenex``: mixers alone and together,
whole prompts, decoding token by token, prompts in pieces down to two tokens, batches of unequal
requests, slots and pages used again, long decoding across chunk and page borders, other sizes,
greedy generation through the engine's entry point, the command line and the trace replay tool."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import engine_utils as U
import plain_rilenex as P

pytestmark = pytest.mark.gpu

# (heads, kv_heads, dim, vdim, conv, chunk, rot_dims, rot_base) and (heads, kv_heads, dim, vdim, conv)
CONFIGS = {
    # both mixers, grouped heads on both sides, a chunk that is no multiple of a page, partial rotation
    "mixed": lambda: P.config([P.parallel_layer((4, 2, 24, 16, 2, 48, 16, 10000.0), (4, 2, 16, 24, 3), ff=96),
                               P.hgrn2_layer(3, 20, 12),
                               P.parallel_layer((2, 2, 16, 16, 4, 64, 16, 500.0), (2, 2, 8, 8, 2), 1.3, 0.6, ff=40),
                               P.hgrn2_layer(2, 16, 16, ff=80)], vocab=131, width=64),
    # a width that is no multiple of 8 (no matrix-core packing), one key head, a chunk longer than a page, taps of 1
    "odd": lambda: P.config([P.hgrn2_layer(5, 12, 28, ff=50),
                             P.parallel_layer((6, 1, 20, 10, 1, 100, 8, 77.0), (3, 1, 24, 20, 4), ff=None)], vocab=97, width=60),
    # the attention side without a mask (every earlier key) and without a convolution, no rotation, heads of 18
    "no_mask": lambda: P.config([P.parallel_layer((3, 3, 18, 14, 0, None, 0, 10.0), (2, 1, 12, 18, 3), ff=44)], vocab=89, width=48),
    "hgrn2_alone": lambda: P.config([P.hgrn2_layer(6, 40, 24)], vocab=101, width=72),
    "parallel_alone": lambda: P.config([P.parallel_layer((8, 4, 32, 32, 3, 32, 32, 250.0), (4, 4, 32, 48, 4))], vocab=101, width=72),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            cfg = CONFIGS[name]()
            w = P.random_weights(cfg, seed=len(name))
            folder = U.write_model(str(tmp_path_factory.mktemp(name)), cfg, w)
            made[name] = (cfg, w, folder)
        return made[name]
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


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_and_pieces(models, name, dtype):
    cfg, w, folder = models(name)
    eng = engine(folder, dtype)
    toks = U.random_tokens(230, cfg["vocab"], 1)
    ref = P.forward(cfg, w, toks)
    close(U.run_whole(eng, toks), ref, dtype, "whole")
    close(U.run_tail(eng, toks, 120), ref, dtype, "the last 120 one by one, across chunk and page borders")
    for piece in (2, 7, 64, 100):                 # the prompt enters in pieces of this many tokens
        eng.prefill_chunk = piece
        close(U.run_whole(eng, toks[:150]), ref[:150], dtype, f"pieces of {piece}")
    eng.prefill_chunk = 0
    assert eng.cache.slots.n_free == eng.cache.max_slots


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_unequal_requests_and_slots_used_again(models, dtype):
    cfg, w, folder = models("mixed")
    eng = engine(folder, dtype, max_slots=3, max_context=256, cache_tokens=448)
    for b, (lens, first) in enumerate([((50, 1, 130), (30, 1, 2)), ((70, 33), (69, 1)), ((90, 9, 140), (5, 9, 101))]):
        reqs = [U.random_tokens(n, cfg["vocab"], 10 * b + i) for i, n in enumerate(lens)]
        outs = U.run_batched(eng, reqs, first)
        for i, (r, o) in enumerate(zip(reqs, outs)):
            close(o, P.forward(cfg, w, r), dtype, f"batch {b} request {i}")
    assert eng.cache.slots.n_free == eng.cache.max_slots
    assert all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


def test_state_and_cache_as_the_mixers_asked(models):
    cfg, w, folder = models("mixed")
    eng = engine(folder, "float32")
    assert set(eng.cache.state) == {0, 1, 2, 3}
    assert set(eng.cache.state[0]) == {"b0.conv", "b1.S", "b1.conv"} and set(eng.cache.state[1]) == {"S"}
    assert tuple(eng.cache.state[0]["b1.S"].shape[1:]) == (4, 24, 16) and tuple(eng.cache.state[0]["b0.conv"].shape[1:]) == (1, 4 * 24 + 2 * 24 + 2 * 16)
    keys = eng.cache.group_keys
    assert len(keys) == 2 and {k.chunk for k in keys} == {48, 64} and all(k.layout == "rows" for k in keys)
    assert not eng._prompt_graphs_ok           # mixers with a state run their prompts as they are, never padded
    from agave_amd.ops import library
    slot = eng.alloc_slot()
    eng.step([slot], [[1, 2]])
    eng.free_slot(slot)
    assert any(p.endswith("sequence.so") for p in library.loaded_paths())     # the HIP kernels ran, nothing else could


def test_long_memory_shows_in_the_logits(models):
    """With forget gates that hardly forget and decays near one, a change of the second token moves the
    logits 400 tokens later, and the engine follows the plain model there (decoded token by token)."""
    cfg = P.config([P.hgrn2_layer(2, 16, 16, ff=None), P.parallel_layer((2, 1, 16, 8, 2, 32, 16, 100.0), (2, 1, 16, 16, 2))],
                   vocab=50, width=32)
    w = P.random_weights(cfg, 5)
    w["l0.mix.lower"] = torch.full_like(w["l0.mix.lower"], 0.996).bfloat16().float()
    w["l1.mix.right.dt_bias"] = torch.full_like(w["l1.mix.right.dt_bias"], -9.0)
    w["l1.mix.right.a2"] = (0.05 * w["l1.mix.right.a2"]).bfloat16().float()
    from agave_amd.engine import Engine
    eng = Engine.from_tensors(cfg, {k: v.bfloat16() for k, v in w.items()}, dtype="float32", max_slots=2, max_context=512)
    toks = U.random_tokens(420, 50, 3)
    other = list(toks)
    other[1] = (toks[1] + 7) % 50
    ref, ref_other = P.forward(cfg, w, toks), P.forward(cfg, w, other)
    moved = float((ref[-1] - ref_other[-1]).abs().max())
    assert moved > 1e-3 * float(ref.abs().max()), "the test's weights do not carry the early token that far"
    for t, r in ((toks, ref), (other, ref_other)):
        got = U.run_tail(eng, t, 60)
        assert float((got[-1].double() - r[-1]).abs().max()) < 0.05 * moved
        close(got, r, "float32", "long memory")


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
    cfg, w, folder = models("odd")
    root = U.ROOT
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "agave_amd"), folder, "3 17 5 80 2", "-n", "5", "--dtype", "float32",
                          "--json"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    seq = [3, 17, 5, 80, 2]
    for _ in range(5):
        seq.append(P.argmax_first(P.forward(cfg, w, seq)[-1]))
    got = json.loads(out.stdout.strip().splitlines()[-1])
    assert got["outputs"][0]["tokens"] == seq[5:] and got["outputs"][0]["prompt_tokens"] == 5
    # the replay tool: two batches one after another, unequal lengths
    batches = [[U.random_tokens(n, cfg["vocab"], 70 + n) for n in (40, 3, 110)], [U.random_tokens(n, cfg["vocab"], 90 + n) for n in (25, 60)]]
    firsts = [(8, 3, 78), (1, 59)]
    records, where = U.trace_steps_batched(batches, firsts)
    for dtype in ("float32", "bfloat16"):
        steps = U.run_trace_tool(folder, dtype, records, str(tmp_path / dtype), 256, cfg["vocab"])
        for bi, reqs in enumerate(batches):
            for i, r in enumerate(reqs):
                got = torch.from_numpy(np.stack([steps[s][row] for s, row in where[(bi, i)]]))
                close(got, P.forward(cfg, w, r), dtype, f"replay {dtype} batch {bi} request {i}")
