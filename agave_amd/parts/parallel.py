"""Mixers side by side: every branch reads the same rows, and the result is the sum of
``scales[i] * branch_i(x)``.

Branches that can hand over the rows their output product reads (``context_into`` with
``context_width``, ``o_weight`` and ``input_matrices``: the built-in mixers with a state do) share
their first product too (all their matrices stacked, one launch, the 32-bit rows shared out by
columns) and write their rows, already times their scale, side by side into one buffer; one product
with the branches' output matrices put next to each other along the columns makes the weighted
sum: ``[W_1 W_2] [s_1 c_1; s_2 c_2]``.  Any other pair of branches runs its own ``forward`` and a
small kernel adds the two results.

At most one branch may keep keys and values in the cache (a memory has one group of pages); every
branch's fixed-size state lives in the memory under the branch's own prefix (``b0.``, ``b1.``, ...).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import ParallelMixerSpec
from ..ops import sequence as seq_ops
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, mixer_libraries, register
from .linear import Linear


class ParallelMixer:
    def __init__(self, spec: ParallelMixerSpec, weights, env: BuildEnv):
        if len(spec.branches) < 2 or len(spec.branches) != len(spec.scales):
            raise ValueError("a parallel mixer has at least two branches and a scale for each")
        self.spec, self.env = spec, env
        classes = [lookup("mixer", b.kind) for b in spec.branches]
        self.fused = all(hasattr(c, "context_into") for c in classes)
        if not self.fused and len(classes) != 2:
            raise ValueError("branches that do not hand over their output product's rows are summed in pairs only")
        self.branches = []
        for i, (b, c) in enumerate(zip(spec.branches, classes)):
            part = c(b, weights, env, own_output=False, own_input=False) if self.fused else c(b, weights, env)
            part.state_prefix = f"b{i}."
            self.branches.append(part)
        if sum(1 for p in self.branches if p.kv_need() is not None) > 1:
            raise ValueError("a parallel mixer: at most one branch may keep keys and values in the cache")
        self.o = self.inp = None
        if self.fused:
            # every branch reads the same rows: their first products are one, its 32-bit rows shared out by columns
            firsts = [m for p in self.branches for m in p.input_matrices]
            for p in self.branches:
                p.input_matrices = None
            self.inp = Linear(firsts, env, "parallel_in")
            self.in_bounds = [0]
            for p in self.branches:
                self.in_bounds.append(self.in_bounds[-1] + p.input_width)
            mats = [p.o_weight for p in self.branches]
            for p in self.branches:
                p.o_weight = None
            # the same type rule as every matrix, then side by side along the columns
            keep = {env.weight_dtype(m.dtype) for m in mats}
            to = keep.pop() if len(keep) == 1 else torch.float32
            self.o = Linear([torch.cat([m.to(to) for m in mats], dim=1)], env, "parallel_o")
            self.bounds = [0]
            for p in self.branches:
                self.bounds.append(self.bounds[-1] + p.context_width)

    @staticmethod
    def kernel_libraries(spec: ParallelMixerSpec, dtype):
        libs = {"sequence"}
        for b in spec.branches:
            libs |= mixer_libraries(b, dtype)
        return tuple(sorted(libs))

    @staticmethod
    def tensor_needs(spec: ParallelMixerSpec) -> List[TensorNeed]:
        needs: List[TensorNeed] = []
        for b in spec.branches:
            needs += lookup("mixer", b.kind).tensor_needs(b)
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        for p in self.branches:
            need = p.kv_need()
            if need is not None:
                return need
        return None

    def state_need(self) -> Optional[Dict[str, StateNeed]]:
        out: Dict[str, StateNeed] = {}
        for i, p in enumerate(self.branches):
            need = p.state_need()
            if need is None:
                continue
            if not isinstance(need, dict):
                need = {p.state_prefix + "state": need}
            out.update(need)
        return out or None

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        ws, n = self.env.workspace, x.shape[0]
        if self.fused:
            ctx = ws.get("parallel_ctx", n, self.bounds[-1], self.env.dtype)
            first = self.inp.forward(x, out_dtype=torch.float32, tag="parallel_in")
            for p, view, rows, scale in zip(self.branches, ws.columns(ctx, tuple(self.bounds)),
                                            ws.columns(first, tuple(self.in_bounds)), self.spec.scales):
                p.context_into(x, step, memory, writes, view, scale, proj=rows)
            return self.o.forward(ctx, tag="parallel_o", slices_ok=True)
        a = self.branches[0].forward(x, step, memory, writes)
        b = self.branches[1].forward(x, step, memory, writes)
        if a.dim() != 2 or b.dim() != 2:
            raise ValueError("a branch of a parallel mixer returns plain rows [N, hidden], not slices that add up")
        out = ws.get("parallel_sum", n, a.shape[1], self.env.dtype)
        seq_ops.scaled_sum(a, self.spec.scales[0], b, self.spec.scales[1], out)
        return out


register("mixer", "parallel", ParallelMixer)
