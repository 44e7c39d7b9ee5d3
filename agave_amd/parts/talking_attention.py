"""Softmax attention whose heads talk to each other, as a mixer.

In the order of its steps: q, k, v (and a gate's logit per head) in one product; an optional short
causal convolution on every channel of q, k and v; an RMS norm per head on q and k with one gain
vector each; a rotation of the first ``rotary_dim`` elements of every head; k and v appended to the
cache (rows of ``head_dim`` and ``v_head_dim`` elements); scores ``scale * q.k`` mixed across the
heads, ``s_h <- sum_g talk[h, g] s_g``; softmax over the keys ``j <= i`` of the query's own chunk
(``j // chunk == i // chunk``, chunks counted from the sequence's first position), or over all
earlier keys; head h's output times ``sigmoid(gate_h)``; the output product.

Between the first product and the rows of the output product everything is 32-bit; the cache
holds the engine's element type.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import TalkingAttentionSpec
from ..ops import sequence as seq_ops
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, register, state_tensor
from .linear import Linear
from .short_conv import ShortConv


SPLIT_TILES_UP_TO = 64       # steps of up to this many tokens share a token's keys among workgroups


class TalkingAttention:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("sequence",)

    def __init__(self, spec: TalkingAttentionSpec, weights, env: BuildEnv, own_output: bool = True, own_input: bool = True):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        self.spec, self.env = spec, env
        self.state_prefix = ""
        s = spec
        self.qd, self.kd, self.vd = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim, s.n_kv_heads * s.v_head_dim
        self.context_width = s.n_heads * s.v_head_dim
        mats = [weights.get(s.q_proj), weights.get(s.k_proj), weights.get(s.v_proj)]
        if s.gate_proj:
            mats.append(weights.get(s.gate_proj))
        # (side by side with other mixers, the first products of all of them are one: the parent takes the matrices)
        self.input_matrices = None if own_input else mats
        self.input_width = sum(int(m.shape[0]) for m in mats)
        self.proj = Linear(mats, env, "talk_qkvg") if own_input else None
        self.conv = (ShortConv([weights.get(s.q_conv), weights.get(s.k_conv), weights.get(s.v_conv)], env, silu=False,
                               name="talk_conv") if s.conv_taps else None)
        self.q_norm = lookup("norm", s.q_norm.kind)(s.q_norm, weights, env) if s.q_norm else None
        self.k_norm = lookup("norm", s.k_norm.kind)(s.k_norm, weights, env) if s.k_norm else None
        for name, part in (("q_norm", self.q_norm), ("k_norm", self.k_norm)):
            if part is not None and not (hasattr(part, "gain") and hasattr(part, "eps")):
                raise ValueError(f"talking attention: {name} must be an RMS norm (the kernel takes a gain and an eps)")
        self.position = lookup("position", s.position.kind)(s.position, env)
        table = getattr(self.position, "rotation_table", None)
        if table is None:
            raise ValueError(f"talking attention: the position encoding {s.position.kind!r} is no rotation of pairs")
        self.freq, self.interleaved = table()
        self.talk = weights.get(s.talk).to(torch.float32).contiguous().to(env.device) if s.talk else None
        self.o_weight = weights.get(s.o_proj)
        self.o = Linear([self.o_weight], env, "talk_o") if own_output else None
        if own_output:
            self.o_weight = None

    @staticmethod
    def tensor_needs(spec: TalkingAttentionSpec) -> List[TensorNeed]:
        s = spec
        qd, kd, vd = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim, s.n_kv_heads * s.v_head_dim
        needs = [TensorNeed(s.q_proj, (qd, s.hidden)), TensorNeed(s.k_proj, (kd, s.hidden)),
                 TensorNeed(s.v_proj, (vd, s.hidden)), TensorNeed(s.o_proj, (s.hidden, s.n_heads * s.v_head_dim))]
        if s.conv_taps:
            needs += [TensorNeed(s.q_conv, (qd, s.conv_taps)), TensorNeed(s.k_conv, (kd, s.conv_taps)),
                      TensorNeed(s.v_conv, (vd, s.conv_taps))]
        if s.talk:
            needs.append(TensorNeed(s.talk, (s.n_heads, s.n_heads)))
        if s.gate_proj:
            needs.append(TensorNeed(s.gate_proj, (s.n_heads, s.hidden)))
        for n in (s.q_norm, s.k_norm):
            if n is not None:
                needs += lookup("norm", n.kind).tensor_needs(n)
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        s = self.spec
        return GroupKey(None, s.n_kv_heads, s.head_dim, chunk=s.chunk, v_head_dim=s.v_head_dim, layout="rows")

    def state_need(self) -> Optional[Dict[str, StateNeed]]:
        return {self.state_prefix + "conv": self.conv.state_need()} if self.conv is not None else None

    def context_into(self, x: torch.Tensor, step, memory: int, writes: bool, out: torch.Tensor, scale: float = 1.0,
                     proj: Optional[torch.Tensor] = None) -> None:
        """The rows that the output product reads, times ``scale``, into ``out`` [N, context_width].
        ``proj``: the first product's 32-bit rows [N, input_width], if the caller made them."""
        s, ws, pre = self.spec, self.env.workspace, self.state_prefix
        n = x.shape[0]
        if not writes:
            raise ValueError("talking attention keeps a convolution state and a cache of its own; it cannot read another run's")
        k_pages, v_pages, _ = step.cache.pages_of(memory)
        table, base = step.tables[step.cache.group_of_memory[memory]]
        if proj is None:
            proj = self.proj.forward(x, out_dtype=torch.float32, tag=pre + "talk_qkvg")
        lo = self.qd + self.kd + self.vd
        qkv = proj[:, :lo]
        gate = proj[:, lo:lo + s.n_heads] if s.gate_proj else None
        if self.conv is not None:
            conved = ws.get(pre + "talk_conved", n, lo, torch.float32)
            self.conv.forward(qkv, conved, state_tensor(step, memory, pre + "conv"), step)
            qkv = conved
        q, k, v = ws.columns(qkv, (0, self.qd, self.qd + self.kd, lo))
        q_rot = ws.get(pre + "talk_q", n, self.qd, torch.float32)
        seq_ops.head_norm_rope_rows(q, k, v, q_rot, self.q_norm.gain if self.q_norm else None,
                                    self.k_norm.gain if self.k_norm else None, self.q_norm.eps if self.q_norm else 0.0,
                                    self.k_norm.eps if self.k_norm else 0.0, self.freq, self.interleaved, step,
                                    k_pages, v_pages, table, base, s.n_heads, s.n_kv_heads, s.head_dim, s.v_head_dim)
        # few tokens (decode steps): a workgroup per token and tile of 64 keys, merged by a second kernel
        parts = None
        if s.chunk is not None and n <= SPLIT_TILES_UP_TO and s.chunk > 64:
            tiles = (s.chunk + 63) // 64
            parts = ws.get(pre + "talk_parts", n * tiles, s.n_heads * (s.v_head_dim + 2), torch.float32).view(
                n, tiles, s.n_heads, s.v_head_dim + 2)
        seq_ops.talk_attention(q_rot, gate, out, k_pages, v_pages, table, base, step, self.talk, s.n_heads, s.n_kv_heads,
                               s.head_dim, s.v_head_dim, s.scale, s.chunk, scale, parts=parts)

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        ctx = self.env.workspace.get(self.state_prefix + "talk_ctx", x.shape[0], self.context_width, self.env.dtype)
        self.context_into(x, step, memory, writes, ctx)
        return self.o.forward(ctx, tag="talk_o", slices_ok=True)


register("mixer", "talking_attention", TalkingAttention)
