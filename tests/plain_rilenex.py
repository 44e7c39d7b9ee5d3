"""A plain, slow statement of the Rilenex decoder: float64, whole sequences, token by token where
the design is recurrent, one function per mechanism.  It shares no code with the framework; the
tests compare the framework with it.

Notation: ``x`` is [T, width]; a linear map stored [out, in] is applied as ``x @ W.T``; positions
count from 0; ``rms(x) = x / sqrt(mean(x^2) + eps)`` over the last axis.
"""
import math
from typing import Dict, List, Optional, Sequence

import torch

F = torch.float64


# ---------------------------------------------------------------- small functions
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * w


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def xielu(z: torch.Tensor, p: float, q: float) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    sp = math.log1p(math.exp(p))
    sq = math.log1p(math.exp(q))
    neg = (0.5 + sq) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    pos = sp * z * z + 0.5 * z
    return torch.where(z > 0, pos, neg)


def short_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y[t, c] = sum_j w[c, j] u[t - taps + 1 + j, c], zeros before the start (u is [T, C])."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotate_interleaved(x: torch.Tensor, pos: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x is [T, heads, dim]; the pairs (2i, 2i+1), i < dims/2, turn by pos * base^(-2i/dims)."""
    out = x.clone()
    for i in range(dims // 2):
        a = pos * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


# ---------------------------------------------------------------- mixers
def chunk_talk_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The softmax side of the parallel mixer: convolved q/k/v, head norms, rotation, scores mixed
    across heads, keys of the query's own chunk only, a gate per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T, dtype=F)
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if p + "q.conv" in W:                                            # a side without a convolution has none
        q, k, v = short_conv(q, W[p + "q.conv"]), short_conv(k, W[p + "k.conv"]), short_conv(v, W[p + "v.conv"])
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, V)
    q = rms_norm(q, W[p + "q.norm"], eps)
    k = rms_norm(k, W[p + "k.norm"], eps)
    q = rotate_interleaved(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_interleaved(k, pos, m["rot"]["dims"], m["rot"]["base"])
    gate = sigmoid(h @ W[p + "g"].T)                                    # [T, H]
    out = talk_attention_core(q, k, v, W[p + "talk"], m["scale"], (m.get("mask") or {}).get("size")) * gate[:, :, None]
    return out.reshape(T, H * V) @ W[p + "o"].T


def talk_attention_core(q, k, v, talk, scale, chunk, pos0: int = 0):
    """q [T, H, D], k [T, G, D], v [T, G, V] of positions pos0 .. pos0 + T - 1 (only keys inside this
    stretch exist).  Scores are mixed across heads by ``talk`` [H, H] (None: not mixed); position i
    sees j <= i with j // chunk == i // chunk (``chunk`` None: all j <= i).  Returns [T, H, V]."""
    T, H, _ = q.shape
    G, V = k.shape[1], v.shape[2]
    rep = H // G
    out = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        lo = 0 if chunk is None else max(0, ((pos0 + t) // chunk) * chunk - pos0)
        raw = torch.stack([(k[lo:t + 1, hh // rep] @ q[t, hh]) * scale for hh in range(H)])   # [H, keys]
        mixed = raw if talk is None else talk @ raw
        w = torch.softmax(mixed, dim=-1)
        for hh in range(H):
            out[t, hh] = w[hh] @ v[lo:t + 1, hh // rep]
    return out


def gated_delta(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """The recurrent side of the parallel mixer: a delta rule whose state decays per key channel."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rep = H // G
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ W[p + "b"].T)                                    # [T, H]
    dt = softplus((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * dt)   # [T, H, D]
    gate = sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).view(T, H, V)
    o, _ = delta_steps(q, k, v, beta, decay)
    o = rms(o, eps) * W[p + "norm"] * gate
    return o.reshape(T, H * V) @ W[p + "o"].T


def delta_steps(q, k, v, beta, decay, S=None):
    """q, k [T, G, D] (already unit vectors), v [T, H, V], beta [T, H], decay [T, H, D]; per head
    S <- diag(decay) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.  Returns (o [T, H, V], S)."""
    T, H, V = v.shape
    G, D = k.shape[1], k.shape[2]
    rep = H // G
    S = torch.zeros(H, D, V, dtype=F) if S is None else S.clone()
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        for hh in range(H):
            kk, qq = k[t, hh // rep], q[t, hh // rep]
            S[hh] = decay[t, hh][:, None] * S[hh]
            u = beta[t, hh] * (v[t, hh] - S[hh].T @ kk)
            S[hh] = S[hh] + torch.outer(kk, u)
            o[t, hh] = S[hh].T @ qq
    return o, S


def forget_steps(q, f, v, S=None):
    """q, f [T, H, D], v [T, H, V]:  S <- diag(f) S + (1 - f) v^T;  o = S^T q.  Returns (o, S)."""
    T, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=F) if S is None else S.clone()
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def parallel_mixer(h, W, p, m, eps):
    left = chunk_talk_attention(h, W, p + "left.", m["left"], eps)
    right = gated_delta(h, W, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def hgrn2(h: torch.Tensor, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Linear attention whose forget gate f also sets what is written: S = diag(f) S + (1 - f) v^T."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, V)
    low = W[p + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).view(T, H, D)
    o, _ = forget_steps(q, f, v)
    o = rms_norm(o, W[p + "norm"], eps)
    return o.reshape(T, H * V) @ W[p + "o"].T


MIXERS = {"parallel": parallel_mixer, "hgrn2": hgrn2}


# ---------------------------------------------------------------- feed-forward and the model
def dense_ffn(h, W, p):
    act = W[p + "act"]
    return xielu(h @ W[p + "up"].T, float(act[0]), float(act[1])) @ W[p + "down"].T


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: Sequence[int],
            layers_out: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  ``layers_out`` receives the residual stream after each layer."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + MIXERS[layer["type"]](rms_norm(x, W[p + "norm1"], eps), W, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + dense_ffn(rms_norm(x, W[p + "norm2"], eps), W, p + "mlp.")
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T


# ---------------------------------------------------------------- random models for the tests
def random_weights(cfg: dict, seed: int, ranks=(6, 5)) -> Dict[str, torch.Tensor]:
    """Weights for ``cfg`` as bfloat16-representable float32 tensors, drawn so that every mechanism
    matters: lower bounds and decays spread over (0, 1), gates away from saturation."""
    g = torch.Generator().manual_seed(seed)
    E = cfg["width"]

    def mat(o, i, std=None):
        return torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)

    def vec(n, mean=1.0, std=0.1):
        return mean + torch.randn(n, generator=g) * std

    W = {"embed": torch.randn(cfg["vocab"], E, generator=g), "final.norm": vec(E), "head": mat(cfg["vocab"], E)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        W[p + "norm1"] = vec(E)
        if layer["type"] == "hgrn2":
            H, D, V = m["heads"], m["dim"], m["vdim"]
            W.update({p + "mix.q": mat(H * D, E), p + "mix.f": mat(H * D, E), p + "mix.f.b": vec(H * D, 0.0, 0.5),
                      p + "mix.lower": torch.rand(H * D, generator=g) * 0.9, p + "mix.v": mat(H * V, E),
                      p + "mix.norm": vec(V), p + "mix.o": mat(E, H * V)})
        else:
            l, r = m["left"], m["right"]
            q = p + "mix.left."
            H, G, D, V = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            W.update({q + "q": mat(H * D, E), q + "k": mat(G * D, E), q + "v": mat(G * V, E),
                      q + "q.norm": vec(D), q + "k.norm": vec(D), q + "talk": torch.eye(H) + mat(H, H, 0.3),
                      q + "g": mat(H, E), q + "o": mat(E, H * V)})
            if l.get("conv"):
                W.update({q + "q.conv": mat(H * D, l["conv"], 0.6), q + "k.conv": mat(G * D, l["conv"], 0.6),
                          q + "v.conv": mat(G * V, l["conv"], 0.6)})
            q = p + "mix.right."
            H, G, D, V = r["heads"], r["kv_heads"], r["dim"], r["vdim"]
            ra, rg = r.get("decay_rank", ranks[0]), r.get("gate_rank", ranks[1])
            W.update({q + "q": mat(G * D, E), q + "k": mat(G * D, E), q + "v": mat(H * V, E),
                      q + "q.conv": mat(G * D, r["conv"], 0.6), q + "k.conv": mat(G * D, r["conv"], 0.6),
                      q + "v.conv": mat(H * V, r["conv"], 0.6), q + "b": mat(H, E),
                      q + "A_log": torch.randn(H, generator=g) * 0.5 - 1.0, q + "norm": vec(V),
                      q + "a1": mat(ra, E), q + "a2": mat(H * D, ra), q + "dt_bias": vec(H * D, -1.0, 1.0),
                      q + "g1": mat(rg, E), q + "g2": mat(H * V, rg), q + "o": mat(E, H * V)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            W.update({p + "norm2": vec(E), p + "mlp.up": mat(ff, E), p + "mlp.down": mat(E, ff),
                      p + "mlp.act": torch.tensor([0.3, -0.4]) + torch.randn(2, generator=g) * 0.2})
    return {k: v.bfloat16().float() for k, v in W.items()}


def hgrn2_layer(heads, dim, vdim, ff=None):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def parallel_layer(left, right, left_scale=0.7, right_scale=1.2, ff=None):
    """``left``: (heads, kv_heads, dim, vdim, conv, chunk, rot_dims, rot_base); ``right``: (heads, kv_heads, dim, vdim, conv)."""
    lh, lg, ld, lv, lc, chunk, rot, base = left
    rh, rg, rd, rv, rc = right
    return {"type": "parallel", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"left": {"heads": lh, "kv_heads": lg, "dim": ld, "vdim": lv, **({"conv": lc} if lc else {}),
                               "scale": ld ** -0.5, "mask": None if chunk is None else {"size": chunk},
                               "rot": {"dims": rot, "base": base}},
                      "right": {"heads": rh, "kv_heads": rg, "dim": rd, "vdim": rv, "conv": rc},
                      "left_scale": left_scale, "right_scale": right_scale}}


def config(layers, vocab=131, width=64, eps=1e-5):
    return {"architecture": "Rilenex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}


def argmax_first(row: torch.Tensor) -> int:
    return int(torch.argmax(row))
