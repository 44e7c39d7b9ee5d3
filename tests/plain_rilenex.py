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
    q = short_conv(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, H, D)
    k = short_conv(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, D)
    v = short_conv(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, G, V)
    q = rms_norm(q, W[p + "q.norm"], eps)
    k = rms_norm(k, W[p + "k.norm"], eps)
    q = rotate_interleaved(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_interleaved(k, pos, m["rot"]["dims"], m["rot"]["base"])
    rep = H // G
    size = m["mask"]["size"]
    gate = sigmoid(h @ W[p + "g"].T)                                    # [T, H]
    out = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        lo = (t // size) * size
        raw = torch.stack([(k[lo:t + 1, hh // rep] @ q[t, hh]) * m["scale"] for hh in range(H)])   # [H, keys]
        mixed = W[p + "talk"] @ raw
        w = torch.softmax(mixed, dim=-1)
        for hh in range(H):
            out[t, hh] = w[hh] @ v[lo:t + 1, hh // rep]
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ W[p + "o"].T


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
    S = torch.zeros(H, D, V, dtype=F)
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        for hh in range(H):
            kk, qq = k[t, hh // rep], q[t, hh // rep]
            S[hh] = decay[t, hh][:, None] * S[hh]
            u = beta[t, hh] * (v[t, hh] - S[hh].T @ kk)
            S[hh] = S[hh] + torch.outer(kk, u)
            o[t, hh] = S[hh].T @ qq
    o = rms(o, eps) * W[p + "norm"] * gate
    return o.reshape(T, H * V) @ W[p + "o"].T


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
    S = torch.zeros(H, D, V, dtype=F)
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
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


def argmax_first(row: torch.Tensor) -> int:
    return int(torch.argmax(row))
