"""Python faces of ``csrc/routed_ffn.hip``: the router's choice of experts and the experts' products."""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _F, _dev, _f32vec, _i32, _rows, dt, ptr, stream

LIBRARY = "routed_ffn"
MAX_OUTPUTS = 1024

kernels.register_signatures(LIBRARY, {
    "agave_route_topk": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _F, _P, _P, _P],
    "agave_routed_experts_plain": [_I, _P, _L, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P],
    "agave_routed_combine": [_I, _P, _P, _P, _P, _P, _L, _P, _L, _P, _L, _I, _I, _I, _I, _P],
})


def _lib():
    return kernels.lib(LIBRARY)


def route_topk(logits: torch.Tensor, correction: Optional[torch.Tensor], scratch: torch.Tensor, groups: int, keep: int,
               top: int, scale: float, choice: torch.Tensor, weight: torch.Tensor) -> None:
    """For every row of 32-bit router logits [N, R]: s = softmax; among the outputs of the ``keep`` groups (of
    ``groups`` equal groups of neighbours) whose largest ``s + correction`` is largest, the ``top`` outputs with the
    largest ``s + correction`` go to ``choice`` [N, top] (int32) and ``s * scale`` to ``weight`` [N, top]."""
    _dev(logits, correction, scratch, choice, weight)
    n, r = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise TypeError("route_topk: router logits must be float32 rows")
    _f32vec(correction, "correction", r)
    if scratch.dtype != torch.float32 or not scratch.is_contiguous() or scratch.numel() < n * r:
        raise ValueError("route_topk: scratch must hold a float32 value per logit")
    _i32(choice, "choice", n * top)
    if weight.dtype != torch.float32 or not weight.is_contiguous() or weight.numel() < n * top:
        raise ValueError("route_topk: weight must be contiguous float32 [N, top]")
    library.call(_lib(), "agave_route_topk", ptr(logits), logits.stride(0), ptr(correction), ptr(scratch), n, r, groups, keep,
                 top, float(scale), ptr(choice), ptr(weight), stream())


def experts_plain(x: torch.Tensor, choice: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                  act_rows: torch.Tensor, y: torch.Tensor, top: int, activation: int) -> None:
    """y[p] = W_down[e] (act(W_gate[e] x_t) * (W_up[e] x_t)) for every pair p = t * top + slot whose choice e is an
    expert with weights (e < E); rows of other pairs are left alone.  ``y`` is float32 [N * top, hidden]."""
    _dev(x, choice, w_gate, w_up, w_down, act_rows, y)
    n, hidden = x.shape
    ldx = _rows(x, "x")
    e, ff, k = w_gate.shape
    if k != hidden or w_up.shape != w_gate.shape or w_down.shape != (e, hidden, ff):
        raise ValueError("experts: weights must be [E, ff, hidden], [E, ff, hidden] and [E, hidden, ff]")
    for w in (w_gate, w_up, w_down):
        if w.dtype != x.dtype or not w.is_contiguous():
            raise TypeError("experts: weights must be contiguous and of the rows' dtype")
    _i32(choice, "choice", n * top)
    if act_rows.dtype != x.dtype or not act_rows.is_contiguous() or act_rows.shape != (n * top, ff):
        raise ValueError(f"experts: inner rows must be [{n * top}, {ff}] of the rows' dtype")
    if y.dtype != torch.float32 or not y.is_contiguous() or y.shape != (n * top, hidden):
        raise ValueError(f"experts: y must be float32 [{n * top}, {hidden}]")
    library.call(_lib(), "agave_routed_experts_plain", dt(x), ptr(x), ldx, ptr(choice), ptr(w_gate), ptr(w_up), ptr(w_down),
                 ptr(act_rows), ptr(y), n, top, e, ff, hidden, activation, stream())


def combine(y: Optional[torch.Tensor], place: Optional[torch.Tensor], choice: torch.Tensor, weight: torch.Tensor,
            x: torch.Tensor, shared: Optional[torch.Tensor], out: torch.Tensor, top: int, n_experts: int) -> None:
    """out[t] = sum over the token's pairs of weight * (the pair's expert row of ``y``, or ``x[t]`` itself where the
    choice is an identity expert, e >= n_experts) + shared[t]."""
    _dev(y, place, choice, weight, x, shared, out)
    n, hidden = x.shape
    ldx, ldo = _rows(x, "x"), _rows(out, "out")
    if out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError("combine: out must have the input's shape and dtype")
    lds = 0
    if shared is not None:
        lds = _rows(shared, "shared")
        if shared.shape != x.shape or shared.dtype != x.dtype:
            raise ValueError("combine: the shared expert's rows must have the input's shape and dtype")
    if y is not None and (y.dtype != torch.float32 or not y.is_contiguous() or y.shape[1] != hidden or y.shape[0] < n * top):
        raise ValueError("combine: y must be float32 [>= N * top, hidden]")
    _i32(choice, "choice", n * top)
    _i32(place, "place", n * top)
    library.call(_lib(), "agave_routed_combine", dt(x), ptr(y), ptr(place), ptr(choice), ptr(weight), ptr(x), ldx, ptr(shared),
                 lds, ptr(out), ldo, n, top, n_experts, hidden, stream())
