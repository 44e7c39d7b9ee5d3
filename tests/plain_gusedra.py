"""A plain, slow implementation of the Gusedra decoder: float64, whole sequences at once, one function
per mechanism, nothing shared with the package.  The GPU tests compare the engine with it.

Notation: rows are tokens; ``i`` is a query's position, ``j`` a key's, ``n = i - j`` their distance.

* layer norm        ``ln(x) = (x - mean x) / sqrt(mean (x - mean x)^2 + eps) * w + b``
* a layer           ``x += m * ls1 * ln1b(mix(ln1(x)));  x += m * ls2 * ln2b(ff(ln2(x)))``
* visibility        ``j <= i and (n < window or j < keep_first)``  (no window: every ``j <= i``)
* slope bias        ``-2^(-8 (h + 1) / H) * n`` for head h of H
* bucket bias       ``rel[bucket(n), h]``; with B buckets, half = B // 2 and D the largest distance:
                    ``bucket(n) = n`` below half, else ``min(B - 1, half + floor(log(n / half) / log(D / half) * (B - half)))``
* sink              one more term ``exp(sink_h)`` in the softmax's denominator, with no value
* gate              heads side by side, times ``sigmoid(W_g x)``, before the output matrix
* dense ff          ``W_down relu(W_up x)^2``
* routed ff         scores ``s = softmax(W_r x)``; choice by ``s + correction`` within the best groups (a group counts by
                    its largest ``s + correction``); weights ``s * scale``; the last outputs are identity experts; a
                    shared expert is added.  Expert: ``W_down (silu(W_gate x) * (W_up x))``.
"""
import math
from typing import Dict, List, Optional, Sequence

import torch

F = torch.float64


# ---------------------------------------------------------------- configurations
def attention_layer(heads, kv_heads, dim, vdim, window, scale=None, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window is not None:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def attention2_layer(heads, kv_heads, dim, vdim, window, keep_first, bias_max, scale=None, mlp=None, buckets=32):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5,
         "bias_max": bias_max}
    if window is not None:
        m["mask"] = {"size": window, "keep_first": keep_first}
    return {"type": "attention_2", "mixer": m, "mlp": mlp, "_buckets": buckets}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, groups, keep, scale, ff, shared_ff=None):
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}}
    if shared_ff is not None:
        out["shared"] = {"ff": shared_ff}
    return out


def config(layers, vocab=97, width=64, eps=1e-5, residual_mult=0.7):
    """(config.json content, {layer: buckets of its learned bias})."""
    buckets = {i: l.pop("_buckets") for i, l in enumerate(layers) if "_buckets" in l}
    cfg = {"architecture": "Gusedra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": residual_mult,
           "layers": layers}
    cfg["_buckets"] = buckets
    return cfg


def public(cfg):
    """The configuration without the test's own notes (what goes into config.json)."""
    return {k: v for k, v in cfg.items() if not k.startswith("_")}


def random_weights(cfg, seed=0, std=None, decided_routing=False) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names, rounded to bfloat16 (so every engine reads the same numbers).
    ``decided_routing``: the corrections lie 1.5 apart, more than two scores can differ, so the choice of experts
    is the same for every token and no rounding can change it (for comparisons in bfloat16, where a close call
    between two experts would otherwise go either way; the weights still follow the scores)."""
    g = torch.Generator().manual_seed(seed)
    e = cfg["width"]
    w: Dict[str, torch.Tensor] = {}

    def mat(name, out, inp, s=None):
        w[name] = torch.randn(out, inp, generator=g) * (s if s is not None else (std or inp ** -0.5))

    def vec(name, n, mean=0.0, s=0.2):
        w[name] = mean + torch.randn(n, generator=g) * s

    def norm(name):
        vec(name, e, 1.0, 0.2)
        vec(name + ".b", e, 0.0, 0.1)

    mat("embed", cfg["vocab"], e, 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        for n in ("norm1", "norm2", "norm1b", "norm2b"):
            norm(p + n)
        vec(p + "ls1", e, 0.8, 0.3)
        vec(p + "ls2", e, 0.8, 0.3)
        m = layer["mixer"]
        H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        mat(p + "mix.q", H * d, e)
        if m.get("kv_from") is None:
            mat(p + "mix.k", G * d, e)
            mat(p + "mix.v", G * vd, e)
        if layer["type"] == "attention":
            vec(p + "mix.sink", H, 0.5, 1.0)
        else:
            w[p + "mix.rel"] = torch.randn(cfg["_buckets"][i], H, generator=g) * 0.7
            mat(p + "mix.g", H * vd, e)
        mat(p + "mix.o", e, H * vd)
        f = layer["mlp"]
        if f is None:
            continue
        if f["kind"] == "dense":
            mat(p + "mlp.up", f["ff"], e)
            mat(p + "mlp.down", e, f["ff"])
        else:
            r = f["router"]
            for x in range(r["experts"]):
                mat(p + f"mlp.e{x}.gate", f["expert"]["ff"], e)
                mat(p + f"mlp.e{x}.up", f["expert"]["ff"], e)
                mat(p + f"mlp.e{x}.down", e, f["expert"]["ff"])
            mat(p + "mlp.router", r["experts"] + r.get("identity", 0), e, 1.5 * e ** -0.5)
            n_out = r["experts"] + r.get("identity", 0)
            vec(p + "mlp.correction", n_out, 0.0, 0.05)
            if decided_routing:
                w[p + "mlp.correction"] = 1.5 * torch.randperm(n_out, generator=g).float() - 0.75 * n_out
            if f.get("shared"):
                mat(p + "mlp.shared.gate", f["shared"]["ff"], e)
                mat(p + "mlp.shared.up", f["shared"]["ff"], e)
                mat(p + "mlp.shared.down", e, f["shared"]["ff"])
    norm("final.norm")
    mat("head", cfg["vocab"], e)
    return {k: v.bfloat16().float() for k, v in w.items()}


# ---------------------------------------------------------------- mechanisms
def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def visible(T: int, window: Optional[int], keep_first: int = 0) -> torch.Tensor:
    """[T, T] bool: may the query in row i see the key in column j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def slope_bias(T: int, H: int) -> torch.Tensor:
    """[H, T, T]: what is added to the scores of head h (a negative multiple of the distance)."""
    n = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F)
    return -slopes[:, None, None] * n


def bucket(n: int, B: int, D: int) -> int:
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + math.floor(math.log(n / half) / math.log(D / half) * (B - half) + 1e-12))


def bucket_bias(T: int, rel: torch.Tensor, D: int) -> torch.Tensor:
    """[H, T, T] from the learned table rel [B, H] (entries above the diagonal are never used)."""
    B, H = rel.shape
    by_distance = torch.stack([rel[bucket(n, B, D)] for n in range(T)])           # [T, H]
    n = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp(min=0)
    return by_distance[n].permute(2, 0, 1).to(F)


def softmax_attention(q, k, v, scale, bias, mask, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, vd], bias [H, T, T], mask [T, T] -> [T, H, vd]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale + bias[h]
        s = s.masked_fill(~mask, -math.inf)
        top = s.max(-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].expand_as(top))
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - top)
        out[:, h] = (e / den) @ v[:, g]
    return out


def mixer(layer, w, p, x, kv):
    """One attention mixer on the normalised rows x; ``kv`` maps a layer to its (k, v) (filled by layers with projections)."""
    m = layer["mixer"]
    T = x.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (x @ w[p + "q"].T).view(T, H, d)
    if m.get("kv_from") is not None:
        k, v = kv[m["kv_from"]]
    else:
        k, v = (x @ w[p + "k"].T).view(T, G, d), (x @ w[p + "v"].T).view(T, G, vd)
    window = m["mask"]["size"] if m.get("mask") else None
    if layer["type"] == "attention":
        ctx = softmax_attention(q, k, v, m["scale"], slope_bias(T, H), visible(T, window), sink=w[p + "sink"])
        ctx = ctx.reshape(T, H * vd)
    else:
        keep = m["mask"].get("keep_first", 0) if m.get("mask") else 0
        ctx = softmax_attention(q, k, v, m["scale"], bucket_bias(T, w[p + "rel"], m["bias_max"]), visible(T, window, keep))
        ctx = ctx.reshape(T, H * vd) * torch.sigmoid(x @ w[p + "g"].T)
    return ctx @ w[p + "o"].T, (k, v)


def dense_ff(w, p, x):
    return torch.relu(x @ w[p + "up"].T) ** 2 @ w[p + "down"].T


def gated_expert(w, p, x):
    a = x @ w[p + "gate"].T
    return (a * torch.sigmoid(a) * (x @ w[p + "up"].T)) @ w[p + "down"].T


def route(z, correction, groups, keep, top, scale):
    """Router logits z [T, R] -> (chosen outputs [T, top], their weights [T, top])."""
    T, R = z.shape
    s = torch.softmax(z, -1)
    c = s + correction
    size = R // groups
    best_groups = c.view(T, groups, size).max(-1).values.topk(keep, dim=-1).indices          # [T, keep]
    open_ = torch.zeros(T, groups, dtype=torch.bool)
    open_.scatter_(1, best_groups, True)
    c = c.masked_fill(~open_.repeat_interleave(size, dim=1), -math.inf)
    chosen = c.topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen) * scale


def routed_ff(f, w, p, x):
    r = f["router"]
    E, I = r["experts"], r.get("identity", 0)
    g = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weight = route(x @ w[p + "router"].T, w[p + "correction"], g["count"], g["keep"], r["top"], r.get("scale", 1.0))
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e, a in zip(chosen[t].tolist(), weight[t]):
            out[t] += a * (x[t] if e >= E else gated_expert(w, p + f"e{e}.", x[t:t + 1])[0])
    if f.get("shared"):
        out = out + gated_expert(w, p + "shared.", x)
    return out


# ---------------------------------------------------------------- the model
def forward(cfg, weights, tokens: Sequence[int], streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of a whole sequence; ``streams`` collects the residual stream after every layer."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = w["embed"][torch.tensor(list(tokens))]
    kv = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        a, own = mixer(layer, w, p + "mix.", layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), kv)
        if layer["mixer"].get("kv_from") is None:
            kv[i] = own
        x = x + m * w[p + "ls1"] * layer_norm(a, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        f = layer["mlp"]
        if f is not None:
            y = layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps)
            y = dense_ff(w, p + "mlp.", y) if f["kind"] == "dense" else routed_ff(f, w, p + "mlp.", y)
            x = x + m * w[p + "ls2"] * layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T


def argmax_first(row: torch.Tensor) -> int:
    return int(torch.nonzero(row == row.max())[0])
