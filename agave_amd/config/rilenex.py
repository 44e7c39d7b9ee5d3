"""Typed configuration of the Rilenex decoder, read from config.json's own keys.

config.json: ``architecture`` ("Rilenex"), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a
list whose entries give ``type`` (the mixer: ``parallel`` or ``hgrn2``), ``mixer`` (its sizes and
constants) and ``mlp`` (``{"kind": "dense", "ff": n}`` or null).  Tensor names: ``embed``,
``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.up|down|act``, ``final.norm``, ``head``.

A layer is pre-norm: ``x += mixer(norm1(x)); x += ff(norm2(x))`` with plain RMS norms.

``parallel``: two mixers on the same input, summed with ``left_scale`` and ``right_scale``.  The
left one is softmax attention with a short convolution behind q, k and v, per-head RMS norms of q
and k, an interleaved rotation of the first ``rot.dims`` elements, scores mixed across heads by
``talk``, keys of the query's own chunk of ``mask.size`` positions, and a sigmoid gate per head.
The right one is a delta rule with a decay per head and key channel.  ``hgrn2`` is linear
attention whose forget gate (bounded below by ``lower``) also sets what is written.  The
feed-forward is ``W_down xielu(W_up x)``.

The design has no bound on positions; :data:`POSITIONS` is what the engine is told.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Iterable, List, Mapping, Optional, Tuple

from .errors import ConfigError
from .spec import (DenseFfnSpec, GatedDeltaSpec, Hgrn2Spec, LayerSpec, ModelSpec, NormSpec, ParallelMixerSpec,
                   PositionSpec, RunEntry, TalkingAttentionSpec)

POSITIONS = 1 << 20           # the longest sequence the engine is told of (no tensor or constant depends on it)
DELTA_UNIT_EPS = 1e-6         # inside the root of the delta rule's unit vectors (the design fixes it)


def _int(d: dict, key: str, where: str, least: int = 1) -> int:
    v = d.get(key)
    if v is None:
        raise ConfigError(f"config.json: {where}: required key '{key}' is missing")
    if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v or int(v) < least:
        raise ConfigError(f"config.json: {where}: '{key}' must be an integer >= {least}, got {v!r}")
    return int(v)


def _num(d: dict, key: str, where: str, positive: bool = False) -> float:
    v = d.get(key)
    if v is None:
        raise ConfigError(f"config.json: {where}: required key '{key}' is missing")
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or (positive and v <= 0):
        raise ConfigError(f"config.json: {where}: '{key}' must be a {'positive ' if positive else ''}number, got {v!r}")
    return float(v)


def _obj(d: dict, key: str, where: str) -> dict:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}: '{key}' must be an object")
    return v


@dataclass(frozen=True)
class TalkSide:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    scale: float
    chunk: Optional[int]               # None: every earlier key
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class DeltaSide:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: Optional[int] = None   # inner sizes of the two-step projections: config.json need not give them
    gate_rank: Optional[int] = None    # (the checkpoint's tensor shapes do); optional keys for random weights


@dataclass(frozen=True)
class ParallelLayer:
    left: TalkSide
    right: DeltaSide
    left_scale: float
    right_scale: float
    type = "parallel"


@dataclass(frozen=True)
class Hgrn2Layer:
    heads: int
    dim: int
    vdim: int
    type = "hgrn2"


@dataclass(frozen=True)
class RilenexLayer:
    mixer: object                      # ParallelLayer | Hgrn2Layer
    ff: Optional[int]                  # None: no feed-forward


@dataclass(frozen=True)
class RilenexConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[RilenexLayer, ...]

    architecture = "Rilenex"

    # ------------------------------------------------------------------ parse
    @classmethod
    def from_dict(cls, raw: dict) -> "RilenexConfig":
        vocab, width = _int(raw, "vocab", "top level"), _int(raw, "width", "top level")
        eps = _num(_obj(raw, "norm", "top level"), "eps", "norm", positive=True)
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers: List[RilenexLayer] = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            m = _obj(e, "mixer", where)
            if kind == "hgrn2":
                mixer = Hgrn2Layer(_int(m, "heads", where), _int(m, "dim", where), _int(m, "vdim", where))
            elif kind == "parallel":
                lw, rw = where + ".mixer.left", where + ".mixer.right"
                l, r = _obj(m, "left", where + ".mixer"), _obj(m, "right", where + ".mixer")
                rot = _obj(l, "rot", lw)
                # (a side without a mask sees every earlier key; one without a convolution has none)
                chunk = _int(_obj(l, "mask", lw), "size", lw + ".mask") if l.get("mask") is not None else None
                left = TalkSide(_int(l, "heads", lw), _int(l, "kv_heads", lw), _int(l, "dim", lw), _int(l, "vdim", lw),
                                _int(l, "conv", lw, least=0) if l.get("conv") is not None else 0, _num(l, "scale", lw), chunk,
                                _int(rot, "dims", lw + ".rot", least=0), _num(rot, "base", lw + ".rot", positive=True))
                right = DeltaSide(_int(r, "heads", rw), _int(r, "kv_heads", rw), _int(r, "dim", rw), _int(r, "vdim", rw),
                                  _int(r, "conv", rw),
                                  _int(r, "decay_rank", rw) if r.get("decay_rank") is not None else None,
                                  _int(r, "gate_rank", rw) if r.get("gate_rank") is not None else None)
                for side, sw in ((left, lw), (right, rw)):
                    if side.heads % side.kv_heads:
                        raise ConfigError(f"config.json: {sw}: heads ({side.heads}) is not a multiple of kv_heads ({side.kv_heads})")
                if left.rot_dims % 2 or left.rot_dims > left.dim:
                    raise ConfigError(f"config.json: {lw}.rot: dims ({left.rot_dims}) must be even and at most dim ({left.dim})")
                mixer = ParallelLayer(left, right, _num(m, "left_scale", where + ".mixer"), _num(m, "right_scale", where + ".mixer"))
            else:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r} (parallel, hgrn2)")
            mlp = e.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}: mlp must be null or of kind 'dense', got {mlp!r}")
                ff = _int(mlp, "ff", where + ".mlp")
            layers.append(RilenexLayer(mixer, ff))
        return cls(vocab, width, eps, tuple(layers))

    # ------------------------------------------------------------------ export
    def to_dict(self) -> dict:
        """config.json content that parses back to this configuration."""
        out = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, Hgrn2Layer):
                mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim}
            else:
                l, r = m.left, m.right
                mixer = {"left": {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "conv": l.conv,
                                  "scale": l.scale, "mask": None if l.chunk is None else {"size": l.chunk},
                                  "rot": {"dims": l.rot_dims, "base": l.rot_base}},
                         "right": {"heads": r.heads, "kv_heads": r.kv_heads, "dim": r.dim, "vdim": r.vdim, "conv": r.conv},
                         "left_scale": m.left_scale, "right_scale": m.right_scale}
                for key, val in (("decay_rank", r.decay_rank), ("gate_rank", r.gate_rank)):
                    if val is not None:
                        mixer["right"][key] = val
            out.append({"type": m.type, "mixer": mixer,
                        "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.eps}, "layers": out}

    # ------------------------------------------------------------------ spec
    def model_spec(self, tensor_names: Optional[Iterable[str]] = None) -> ModelSpec:
        """The architecture as parts.  ``tensor_names`` may map names to shapes: the inner sizes of
        the decay's and the output gate's two projections are the checkpoint's (config.json need not
        hold them); without a checkpoint they are the optional keys, else a quarter of the head's
        key (value) size, at least 8."""
        e, eps = self.width, self.eps
        shapes = tensor_names if isinstance(tensor_names, Mapping) else {}

        def rank(name: str, given: Optional[int], size: int) -> int:
            if name in shapes and len(shapes[name]) == 2:
                return int(shapes[name][0])
            return int(given) if given is not None else max(8, size // 4)

        def norm(name: str, size: int) -> NormSpec:
            return NormSpec("rmsnorm", size, eps, name, add_one=False)

        layers: List[LayerSpec] = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}.mix."
            m = layer.mixer
            if isinstance(m, Hgrn2Layer):
                mixer = Hgrn2Spec(kind="hgrn2", hidden=e, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, norm_eps=eps,
                                  q_proj=p + "q", f_proj=p + "f", f_bias=p + "f.b", lower=p + "lower", v_proj=p + "v",
                                  o_proj=p + "o", out_norm=p + "norm")
            else:
                l, r = m.left, m.right
                lp, rp = p + "left.", p + "right."
                left = TalkingAttentionSpec(
                    kind="talking_attention", hidden=e, n_heads=l.heads, n_kv_heads=l.kv_heads, head_dim=l.dim,
                    v_head_dim=l.vdim, scale=l.scale, chunk=l.chunk, conv_taps=l.conv,
                    position=(PositionSpec("rope", rotary_dim=l.rot_dims, theta=l.rot_base, interleaved=True)
                              if l.rot_dims else PositionSpec("none")),
                    q_norm=norm(lp + "q.norm", l.dim), k_norm=norm(lp + "k.norm", l.dim),
                    q_proj=lp + "q", k_proj=lp + "k", v_proj=lp + "v", o_proj=lp + "o",
                    q_conv=lp + "q.conv", k_conv=lp + "k.conv", v_conv=lp + "v.conv", talk=lp + "talk", gate_proj=lp + "g")
                right = GatedDeltaSpec(
                    kind="gated_delta", hidden=e, n_heads=r.heads, n_kv_heads=r.kv_heads, head_dim=r.dim,
                    v_head_dim=r.vdim, conv_taps=r.conv, norm_eps=eps, unit_eps=DELTA_UNIT_EPS,
                    decay_rank=rank(rp + "a1", r.decay_rank, r.dim), gate_rank=rank(rp + "g1", r.gate_rank, r.vdim),
                    q_proj=rp + "q", k_proj=rp + "k", v_proj=rp + "v", o_proj=rp + "o",
                    q_conv=rp + "q.conv", k_conv=rp + "k.conv", v_conv=rp + "v.conv", beta_proj=rp + "b",
                    decay_in=rp + "a1", decay_out=rp + "a2", decay_bias=rp + "dt_bias", decay_log=rp + "A_log",
                    gate_in=rp + "g1", gate_out=rp + "g2", out_norm=rp + "norm")
                mixer = ParallelMixerSpec(kind="parallel", branches=(left, right), scales=(m.left_scale, m.right_scale))
            ffn = None
            if layer.ff is not None:
                fp = f"l{i}.mlp."
                ffn = DenseFfnSpec(kind="dense", hidden=e, intermediate=layer.ff, activation="xielu",
                                   up_proj=fp + "up", down_proj=fp + "down", act_params=fp + "act")
            layers.append(LayerSpec(kind="prenorm", mixer=mixer, ffn=ffn, pre_mixer_norm=norm(f"l{i}.norm1", e),
                                    pre_ffn_norm=norm(f"l{i}.norm2", e) if ffn is not None else None))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden=e, embed_weight="embed", embed_scale=1.0,
            layers=layers, order=[RunEntry(i, i, True) for i in range(len(layers))],
            final_norm=norm("final.norm", e), head_weight="head", max_context=POSITIONS,
            bos_token_id=None, eos_token_ids=(),
            # a tensor that no part asks for (the second norm of a layer without a feed-forward, say) is passed over
            tensor_scope=())
