"""Every kernel of ``csrc/sequence.hip`` alone, and the activation of the dense feed-forward, against
the plain functions of ``plain_rilenex``: sizes that are no powers of two, sequences fed whole, in
pieces and token by token through the framework's own cache and step planner, inputs made so that
a fault would show (a key just inside or just outside a chunk, at a page's border, far back)."""
import math

import pytest
import torch

import plain_rilenex as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def planner_for(kv=None, state=None, slots=3, pages=24, dtype=torch.float32, context=1024):
    from agave_amd.cache import KVCache
    from agave_amd.engine.step import StepPlanner
    cache = KVCache(kv or {}, state or {}, slots, {k: pages for k in (kv or {}).values()}, dtype, torch.device(DEV), context)
    return cache, StepPlanner(cache, 1000, torch.device(DEV))


def feed(cache, planner, slots, counts):
    """One step that brings ``counts[i]`` tokens to ``slots[i]``; commit is the caller's."""
    return planner.plan(slots, [[0] * c for c in counts], "all")


def cuts(total, first, piece):
    """Row ranges: ``first`` rows, then pieces of ``piece`` rows (1: token by token)."""
    out, at = [(0, first)], first
    while at < total:
        n = min(piece, total - at)
        out.append((at, at + n))
        at += n
    return out


# ---------------------------------------------------------------- short convolution
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("silu", [False, True])
def test_short_conv_whole_pieces_and_tokens(taps, silu):
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    C, T = 37, 29
    g = torch.Generator().manual_seed(taps)
    u = torch.randn(T, C, generator=g)
    w = torch.randn(C, taps, generator=g)
    ref = P.short_conv(u.to(F64), w.to(F64))
    ref = P.silu(ref) if silu else ref
    for first, piece in ((T, 1), (11, 1), (5, 2), (1, 3), (2, 9)):        # also fewer new tokens than taps
        cache, planner = planner_for(state={0: StateNeed((taps - 1, C))})
        cache.alloc_slot()                                                # slot 0 stays unused: slot 1's state is not the first
        slot = cache.alloc_slot()
        got = torch.zeros(T, C)
        for lo, hi in cuts(T, first, piece):
            step = feed(cache, planner, [slot], [hi - lo])
            x = u[lo:hi].to(DEV).contiguous()
            y = torch.empty_like(x)
            S.short_conv(x, w.to(DEV), y, cache.state[0], step, silu)
            planner.commit(step)
            got[lo:hi] = y.cpu()
        assert torch.allclose(got.to(F64), ref, atol=2e-5, rtol=1e-5), (first, piece)


def test_short_conv_batch_of_unequal_sequences_and_a_slot_used_again():
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    C, taps = 20, 4
    g = torch.Generator().manual_seed(3)
    w = torch.randn(C, taps, generator=g)
    cache, planner = planner_for(state={0: StateNeed((taps - 1, C))})
    for round_ in range(2):                                               # the second round reuses the slots: state starts at zero again
        seqs = [torch.randn(n, C, generator=g) for n in (9, 1, 17)]
        slots = [cache.alloc_slot() for _ in seqs]
        first = [4, 1, 2]
        outs = [[] for _ in seqs]
        step = feed(cache, planner, slots, first)
        x = torch.cat([s[:f] for s, f in zip(seqs, first)]).to(DEV)
        y = torch.empty_like(x)
        S.short_conv(x, w.to(DEV), y, cache.state[0], step, False)
        planner.commit(step)
        at = 0
        for i, f in enumerate(first):
            outs[i].append(y[at:at + f].cpu())
            at += f
        used = list(first)
        live = [i for i in range(3) if used[i] < len(seqs[i])]
        while live:
            step = feed(cache, planner, [slots[i] for i in live], [1] * len(live))
            x = torch.stack([seqs[i][used[i]] for i in live]).to(DEV)
            y = torch.empty_like(x)
            S.short_conv(x, w.to(DEV), y, cache.state[0], step, False)
            planner.commit(step)
            for j, i in enumerate(live):
                outs[i].append(y[j:j + 1].cpu())
                used[i] += 1
            live = [i for i in live if used[i] < len(seqs[i])]
        for i, s in enumerate(seqs):
            assert torch.allclose(torch.cat(outs[i]).to(F64), P.short_conv(s.to(F64), w.to(F64)), atol=2e-5), (round_, i)
        for s in slots:
            cache.free_slot(s)


# ---------------------------------------------------------------- head norm, rotation, cache rows
def plain_rotate_halves(x, pos, dims, base):
    out = x.clone()
    half = dims // 2
    for i in range(half):
        a = pos * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("dk, dv, rot", [(24, 16, 24), (40, 8, 12), (70, 70, 0), (130, 36, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_rotation_and_rows_in_the_cache(interleaved, dk, dv, rot, dtype):
    from agave_amd.cache import GroupKey
    from agave_amd.ops import sequence as S
    H, G, T, base, eps = 3, 1, 150, 777.0, 1e-5
    key = GroupKey(None, G, dk, chunk=None, v_head_dim=dv, layout="rows")
    cache, planner = planner_for(kv={0: key}, dtype=dtype)
    cache.alloc_slot()
    slot = cache.alloc_slot()
    g = torch.Generator().manual_seed(dk)
    q, k, v = torch.randn(T, H * dk, generator=g), torch.randn(T, G * dk, generator=g), torch.randn(T, G * dv, generator=g)
    qg, kg = 1 + 0.2 * torch.randn(dk, generator=g), 1 + 0.2 * torch.randn(dk, generator=g)
    freq = None
    if rot:
        freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64, device=DEV)
    k_pages, v_pages, _ = cache.pages_of(0)
    q_out = torch.empty(T, H * dk, device=DEV)
    for lo, hi in cuts(T, 70, 33):
        step = feed(cache, planner, [slot], [hi - lo])
        table, tbase = step.tables[0]
        S.head_norm_rope_rows(q[lo:hi].to(DEV), k[lo:hi].to(DEV), v[lo:hi].to(DEV), q_out[lo:hi], qg.to(DEV), kg.to(DEV),
                              eps, eps, freq, interleaved, step, k_pages, v_pages, table, tbase, H, G, dk, dv)
        planner.commit(step)
    pos = torch.arange(T, dtype=F64)
    turn = P.rotate_interleaved if interleaved else plain_rotate_halves
    q_ref = P.rms_norm(q.to(F64).view(T, H, dk), qg.to(F64), eps)
    k_ref = P.rms_norm(k.to(F64).view(T, G, dk), kg.to(F64), eps)
    if rot:
        q_ref, k_ref = turn(q_ref, pos, rot, base), turn(k_ref, pos, rot, base)
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(q_out.cpu().to(F64).view(T, H, dk), q_ref, atol=3e-5, rtol=1e-5)
    held = cache.groups[0].held(slot)
    for page, pid in held.items():
        n = min(64, T - page * 64)
        kk = k_pages[pid, :, :n].float().cpu().to(F64).transpose(0, 1)           # [n, G, dk]
        vv = v_pages[pid, :, :n].float().cpu().to(F64).transpose(0, 1)
        assert torch.allclose(kk, k_ref[page * 64:page * 64 + n], atol=tol, rtol=tol), page
        assert torch.allclose(vv, v.to(F64).view(T, G, dv)[page * 64:page * 64 + n], atol=tol, rtol=tol), page


# ---------------------------------------------------------------- attention with talking heads
def run_talk_attention(q, k, v, talk, gate, scale, chunk, dtype, plan, out_scale=1.0, split=False):
    """Feed one sequence as ``plan`` (row ranges) through the cache; returns [T, H * dv] (float64 on the host)."""
    from agave_amd.cache import GroupKey
    from agave_amd.ops import sequence as S
    T, H, dk = q.shape
    G, dv = k.shape[1], v.shape[2]
    key = GroupKey(None, G, dk, chunk=chunk, v_head_dim=dv, layout="rows")
    cache, planner = planner_for(kv={0: key}, dtype=dtype)
    cache.alloc_slot()
    slot = cache.alloc_slot()
    k_pages, v_pages, _ = cache.pages_of(0)
    out = torch.zeros(T, H * dv, dtype=dtype, device=DEV)
    for lo, hi in plan:
        step = feed(cache, planner, [slot], [hi - lo])
        table, tbase = step.tables[0]
        q_rows = torch.empty(hi - lo, H * dk, device=DEV)
        S.head_norm_rope_rows(q[lo:hi].reshape(hi - lo, -1).float().to(DEV), k[lo:hi].reshape(hi - lo, -1).float().to(DEV),
                              v[lo:hi].reshape(hi - lo, -1).float().to(DEV), q_rows, None, None, 0.0, 0.0, None, False, step,
                              k_pages, v_pages, table, tbase, H, G, dk, dv)
        parts = None
        if split and chunk is not None:         # a workgroup per token and tile of 64 keys, then the merge
            parts = torch.full((hi - lo, (chunk + 63) // 64, H, dv + 2), float("nan"), device=DEV)
        S.talk_attention(q_rows, None if gate is None else gate[lo:hi].float().to(DEV).contiguous(), out[lo:hi], k_pages,
                         v_pages, table, tbase, step, None if talk is None else talk.float().to(DEV), H, G, dk, dv, scale,
                         chunk, out_scale, parts=parts)
        planner.commit(step)
    return out.float().cpu().to(F64), cache, slot


@pytest.mark.parametrize("H, G, dk, dv, chunk", [(4, 2, 24, 16, 48), (3, 3, 40, 40, 64), (6, 1, 16, 20, 100), (2, 1, 72, 8, None),
                                                 (5, 5, 8, 130, 7), (9, 3, 18, 6, 200)])      # (18: no 16-byte loads of a key row)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_talk_attention_prompt_pieces_and_decoding(H, G, dk, dv, chunk, dtype):
    T = 215
    g = torch.Generator().manual_seed(H * 100 + dk)
    rnd = lambda *s: torch.randn(*s, generator=g)
    q, k, v = rnd(T, H, dk), rnd(T, G, dk), rnd(T, G, dv)
    if dtype == torch.bfloat16:
        k, v = k.bfloat16().float(), v.bfloat16().float()
    talk = torch.eye(H) + 0.4 * rnd(H, H)
    gate = rnd(T, H)
    scale = 1.3 / math.sqrt(dk)
    ref = P.talk_attention_core(q.to(F64), k.to(F64), v.to(F64), talk.to(F64), scale, chunk) * P.sigmoid(gate.to(F64))[:, :, None]
    ref = (0.8 * ref).reshape(T, -1)
    tol = 3e-5 if dtype == torch.float32 else 1.5e-2
    for plan, split in ((cuts(T, T, 1), False), (cuts(T, 130, 1), False), (cuts(T, 130, 1), True), (cuts(T, 3, 2), False),
                        (cuts(T, 50, 47), True)):
        got, cache, slot = run_talk_attention(q, k, v, talk, gate, scale, chunk, dtype, plan, out_scale=0.8, split=split)
        err = (got - ref).abs().max(-1).values
        assert float(err.max()) <= tol * max(1.0, float(ref.abs().max())), (plan[0], int(err.argmax()), float(err.max()))
        if chunk is not None:                                       # only the pages of the running chunk are still held
            first = ((T // chunk) * chunk) // 64
            assert min(cache.groups[0].held(slot)) == first


@pytest.mark.parametrize("chunk", [48, 64, 100])
@pytest.mark.parametrize("decode", [False, True])
def test_a_key_just_inside_and_just_outside_the_chunk_stands_out(chunk, decode):
    """Queries late in their chunk, with one key made to dominate: the chunk's first key must be seen,
    the key before it must not, wherever the page's border lies.  No mixing, so a head's output is its
    own softmax and the dominant key's value shows."""
    H, G, dk, dv, T = 2, 1, 16, 4, 3 * 100 + 5
    g = torch.Generator().manual_seed(chunk)
    q, k = 0.1 * torch.randn(T, H, dk, generator=g), 0.1 * torch.randn(T, G, dk, generator=g)
    v = torch.zeros(T, G, dv)
    v[:, 0, 0] = torch.arange(T, dtype=torch.float32)                # a value says which key it came from
    probes = []
    for c in range(1, T // chunk):
        start, last = c * chunk, min(T - 1, c * chunk + chunk - 1)
        for loud, seen in ((start, True), (start - 1, False)):
            probes.append((last, loud, seen))
    for last, loud, seen in probes:
        kk, qq = k.clone(), q.clone()
        kk[loud, 0] = 0
        kk[loud, 0, 3] = 30.0
        qq[last, :, 3] = 30.0                                        # score 900 * scale on the loud key
        plan = cuts(T, last, 1) if decode else cuts(T, T, 1)
        got, _, _ = run_talk_attention(qq, kk, v, None, None, 1.0, chunk, torch.float32, [p for p in plan if p[0] <= last],
                                       split=decode)
        ref = P.talk_attention_core(qq.to(F64), kk.to(F64), v.to(F64), None, 1.0, chunk).reshape(T, -1)
        assert torch.allclose(got[last], ref[last], atol=1e-3), (last, loud)
        assert (abs(float(got[last, 0]) - loud) < 1e-3) == seen, (last, loud, float(got[last, 0]))


def test_talk_attention_first_tokens_and_batches_share_nothing():
    """Sequences of 1, 2 and 70 tokens in one step give what each gives alone."""
    from agave_amd.cache import GroupKey
    from agave_amd.ops import sequence as S
    H, G, dk, dv, chunk = 4, 2, 24, 16, 48
    g = torch.Generator().manual_seed(9)
    lens = [1, 2, 70]
    qs = [torch.randn(n, H, dk, generator=g) for n in lens]
    ks = [torch.randn(n, G, dk, generator=g) for n in lens]
    vs = [torch.randn(n, G, dv, generator=g) for n in lens]
    talk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    key = GroupKey(None, G, dk, chunk=chunk, v_head_dim=dv, layout="rows")
    cache, planner = planner_for(kv={0: key})
    slots = [cache.alloc_slot() for _ in lens]
    step = feed(cache, planner, slots, lens)
    table, tbase = step.tables[0]
    k_pages, v_pages, _ = cache.pages_of(0)
    n = sum(lens)
    cat = lambda xs: torch.cat([x.reshape(x.shape[0], -1) for x in xs]).to(DEV)
    q_rows, out = torch.empty(n, H * dk, device=DEV), torch.empty(n, H * dv, device=DEV)
    S.head_norm_rope_rows(cat(qs), cat(ks), cat(vs), q_rows, None, None, 0.0, 0.0, None, True, step, k_pages, v_pages, table,
                          tbase, H, G, dk, dv)
    S.talk_attention(q_rows, None, out, k_pages, v_pages, table, tbase, step, talk.to(DEV), H, G, dk, dv, 0.2, chunk)
    at = 0
    for q, k, v in zip(qs, ks, vs):
        ref = P.talk_attention_core(q.to(F64), k.to(F64), v.to(F64), talk.to(F64), 0.2, chunk).reshape(q.shape[0], -1)
        assert torch.allclose(out[at:at + q.shape[0]].cpu().to(F64), ref, atol=3e-5)
        at += q.shape[0]


# ---------------------------------------------------------------- the gated linear recurrence
def run_recurrence(mode, tensors, sizes, plan_rows, vectors):
    """One sequence fed as ``plan_rows``; returns the read-outs [T, H * dv] and the final state."""
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    H, G, dk, dv = sizes
    cache, planner = planner_for(state={0: StateNeed((H, dv, dk))})
    cache.alloc_slot()
    slot = cache.alloc_slot()
    T = tensors["v"].shape[0]
    out = torch.zeros(T, H * dv, device=DEV)
    for lo, hi in plan_rows:
        step = feed(cache, planner, [slot], [hi - lo])
        t = {n: x[lo:hi].to(DEV).contiguous() for n, x in tensors.items()}
        S.gated_recurrence(mode, t["q"], t["k"], t["v"], out[lo:hi], cache.state[0], step, H, G, dk, dv,
                           dt_in=t.get("dt"), beta=t.get("beta"), **{n: x.to(DEV) for n, x in vectors.items()})
        planner.commit(step)
    return out.cpu().to(F64), cache.state[0][slot].cpu().to(F64).transpose(1, 2)


@pytest.mark.parametrize("H, G, dk, dv", [(4, 2, 16, 24), (3, 3, 20, 12), (2, 1, 64, 64), (2, 2, 100, 70), (1, 1, 130, 8), (5, 1, 8, 3)])
def test_delta_rule_whole_pieces_and_tokens(H, G, dk, dv):
    from agave_amd.ops import sequence as S
    T = 90
    g = torch.Generator().manual_seed(dk + dv)
    rnd = lambda *s: torch.randn(*s, generator=g)
    q, k, v, beta, dt = rnd(T, G * dk), rnd(T, G * dk), rnd(T, H * dv), rnd(T, H), rnd(T, H * dk)
    a_log, dt_bias = 0.5 * rnd(H) - 1.0, rnd(H * dk) - 1.0
    qd, kd = q.to(F64).view(T, G, dk), k.to(F64).view(T, G, dk)
    qn = qd / torch.sqrt((qd * qd).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    kn = kd / torch.sqrt((kd * kd).sum(-1, keepdim=True) + 1e-6)
    decay = torch.exp(-torch.exp(a_log.to(F64))[None, :, None] * P.softplus(dt.to(F64) + dt_bias.to(F64)).view(T, H, dk))
    ref, S_ref = P.delta_steps(qn, kn, v.to(F64).view(T, H, dv), P.sigmoid(beta.to(F64)), decay)
    for plan in (cuts(T, T, 1), cuts(T, 40, 1), cuts(T, 1, 2), cuts(T, 17, 16), cuts(T, 33, 31)):
        got, S_got = run_recurrence(S.DELTA, {"q": q, "k": k, "v": v, "beta": beta, "dt": dt}, (H, G, dk, dv), plan,
                                    {"a_log": a_log, "dt_bias": dt_bias})
        assert torch.allclose(got, ref.reshape(T, -1), atol=3e-5, rtol=1e-4), plan[:2]
        assert torch.allclose(S_got, S_ref, atol=3e-5, rtol=1e-4), plan[:2]


@pytest.mark.parametrize("H, dk, dv", [(3, 20, 12), (6, 48, 16), (2, 16, 16), (1, 200, 90)])
def test_forget_gate_recurrence_whole_pieces_and_tokens(H, dk, dv):
    from agave_amd.ops import sequence as S
    T = 90
    g = torch.Generator().manual_seed(dk * dv)
    rnd = lambda *s: torch.randn(*s, generator=g)
    q, f_in, v = rnd(T, H * dk), rnd(T, H * dk), rnd(T, H * dv)
    lower, f_bias = torch.rand(H * dk, generator=g), 0.5 * rnd(H * dk)
    f = lower.to(F64) + (1 - lower.to(F64)) * P.sigmoid(f_in.to(F64) + f_bias.to(F64))
    ref, S_ref = P.forget_steps(P.silu(q.to(F64)).view(T, H, dk), f.view(T, H, dk), v.to(F64).view(T, H, dv))
    for plan in (cuts(T, T, 1), cuts(T, 40, 1), cuts(T, 2, 2), cuts(T, 17, 16)):
        got, S_got = run_recurrence(S.FORGET, {"q": q, "k": f_in, "v": v}, (H, H, dk, dv), plan,
                                    {"lower": lower, "f_bias": f_bias})
        assert torch.allclose(got, ref.reshape(T, -1), atol=3e-5, rtol=1e-4), plan[:2]
        assert torch.allclose(S_got, S_ref, atol=3e-5, rtol=1e-4), plan[:2]


def test_a_write_far_back_is_still_read():
    """What token 100 wrote is read 600 tokens later, among hundreds of small writes, as long as the
    forget gate stays open in between; with the gate at one half it is gone."""
    from agave_amd.ops import sequence as S
    H, dk, dv, T = 1, 8, 4, 700
    g = torch.Generator().manual_seed(1)
    q = torch.zeros(T, dk)
    q[-1, 2] = 5.0
    v = 0.01 * torch.randn(T, dv, generator=g)
    v[100] = torch.tensor([7.0, -3.0, 2.0, 1.0])
    lower = torch.zeros(dk)
    for between, kept in ((20.0, True), (0.0, False)):
        f_in = torch.full((T, dk), between)                     # sigmoid(20): the gate keeps everything and writes nothing
        f_in[100, 2] = -20.0                                    # once, channel 2 forgets all and takes token 100's values
        f = P.sigmoid(f_in.to(F64))
        ref, _ = P.forget_steps(P.silu(q.to(F64)).view(T, H, dk), f.view(T, H, dk), v.to(F64).view(T, H, dv))
        got, _ = run_recurrence(S.FORGET, {"q": q, "k": f_in, "v": v}, (H, H, dk, dv), cuts(T, 650, 1), {"lower": lower})
        assert torch.allclose(got[-1], ref[-1].reshape(-1), atol=1e-4, rtol=1e-4)
        assert (float(got[-1, 0].abs()) > 10.0) == kept


def test_recurrence_batch_of_unequal_sequences_against_each_alone():
    from agave_amd.cache import StateNeed
    from agave_amd.ops import sequence as S
    H, dk, dv = 3, 20, 12
    g = torch.Generator().manual_seed(4)
    lens = [1, 33, 2, 18]
    mk = lambda n: {"q": torch.randn(n, H * dk, generator=g), "k": torch.randn(n, H * dk, generator=g), "v": torch.randn(n, H * dv, generator=g)}
    seqs = [mk(n) for n in lens]
    lower = torch.rand(H * dk, generator=g)
    cache, planner = planner_for(state={0: StateNeed((H, dv, dk))}, slots=4)
    slots = [cache.alloc_slot() for _ in lens]
    step = feed(cache, planner, slots, lens)
    cat = {n: torch.cat([s[n] for s in seqs]).to(DEV) for n in ("q", "k", "v")}
    out = torch.empty(sum(lens), H * dv, device=DEV)
    S.gated_recurrence(S.FORGET, cat["q"], cat["k"], cat["v"], out, cache.state[0], step, H, H, dk, dv, lower=lower.to(DEV))
    at = 0
    for s, n in zip(seqs, lens):
        alone, _ = run_recurrence(S.FORGET, s, (H, H, dk, dv), [(0, n)], {"lower": lower})
        assert torch.allclose(out[at:at + n].cpu().to(F64), alone, atol=1e-6)
        at += n


# ---------------------------------------------------------------- read-out norm, activation, sum
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H, dv, gated", [(4, 24, True), (3, 70, False), (1, 130, True)])
def test_head_norm_gate(dtype, H, dv, gated):
    from agave_amd.ops import sequence as S
    g = torch.Generator().manual_seed(dv)
    n = 19
    o, w, gate = torch.randn(n, H * dv, generator=g), 1 + 0.2 * torch.randn(dv, generator=g), torch.randn(n, H * dv, generator=g)
    out = torch.empty(n, H * dv, dtype=dtype, device=DEV)
    S.head_norm_gate(o.to(DEV), w.to(DEV), gate.to(DEV) if gated else None, out, H, dv, 1e-5, 1.1)
    ref = P.rms_norm(o.to(F64).view(n, H, dv), w.to(F64), 1e-5)
    if gated:
        ref = ref * P.sigmoid(gate.to(F64)).view(n, H, dv)
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.float().cpu().to(F64), 1.1 * ref.reshape(n, -1), atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cols", [77, 96])            # rows that 16-byte loads do not divide, and rows that they do
def test_xielu_and_scaled_sum(dtype, cols):
    from agave_amd.ops import kernels, sequence as S
    g = torch.Generator().manual_seed(0)
    x = (3 * torch.randn(13, cols, generator=g)).to(dtype)
    out = torch.empty_like(x, device=DEV)
    p, q = 0.37, -0.61
    kernels.unary_act(x.to(DEV), out, "xielu", math.log1p(math.exp(p)), 0.5 + math.log1p(math.exp(q)))
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.float().cpu().to(F64), P.xielu(x.float().to(F64), p, q), atol=tol, rtol=tol)
    y = torch.randn(13, cols, generator=g).to(dtype)
    S.scaled_sum(x.to(DEV), 0.8, y.to(DEV), 1.1, out)
    assert torch.allclose(out.float().cpu(), 0.8 * x.float() + 1.1 * y.float(), atol=tol * 4, rtol=tol)
