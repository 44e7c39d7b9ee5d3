"""Typed configuration of the Gusedra decoder, read from config.json's own keys.

config.json: ``architecture`` ("Gusedra"), ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` and
``layers``, a list whose entries give ``type`` (the mixer: ``attention`` or ``attention_2``), ``mixer``
(its sizes and constants) and ``mlp`` (``{"kind": "dense", "ff": n}``, ``{"kind": "moe", ...}`` or null).
Tensor names: ``embed``, ``l<i>.norm1|norm2|norm1b|norm2b`` (each with ``.b``), ``l<i>.ls1|ls2``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm`` (with ``.b``), ``head``.

A layer has a layer norm before and after each sublayer and a layer scale on each branch:
``x += m ls1 * norm1b(mixer(norm1(x)));  x += m ls2 * norm2b(ff(norm2(x)))`` with ``m = residual_mult``.

Both mixers are softmax attention with grouped query heads, keys of size ``dim`` and values of size
``vdim``, no rotation, ``scale`` on q.k and a sliding window ``mask.size``:

``attention``    the score of (i, j) loses ``slope_h (i - j)`` with ``slope_h = 2^(-8 (h + 1) / heads)``; every
                 head has a sink ``exp(sink_h)`` in the softmax's denominator; with ``kv_from: j`` the layer has
                 no key and value projections and reads layer j's cache through its own mask.
``attention_2``  a learned bias ``rel[bucket(i - j), h]`` over logarithmic buckets of distances up to
                 ``bias_max``; the first ``mask.keep_first`` positions stay visible beyond the window; the
                 concatenated heads are multiplied by ``sigmoid(W_g x)`` before the output product.

Feed-forwards: ``dense``: ``W_down relu(W_up x)^2``; ``moe``: ``router.experts`` gated SiLU experts of size
``expert.ff`` plus ``router.identity`` identity experts, ``router.top`` of them per token chosen by softmax
score + ``correction`` within the best ``groups.keep`` of ``groups.count`` groups, weighted by score times
``router.scale``, and a shared expert of size ``shared.ff``.

The design has no bound on positions; :data:`POSITIONS` is what the engine is told.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, List, Optional, Tuple

from .errors import ConfigError
from .rilenex import _int, _num, _obj
from .spec import (BiasedAttentionSpec, DenseFfnSpec, GatedFfnSpec, LayerSpec, ModelSpec, NormSpec, RoutedFfnSpec, RunEntry,
                   ScoreBiasSpec)

POSITIONS = 1 << 20           # the longest sequence the engine is told of (no tensor or constant depends on it)
SLOPE_LOG2 = 8.0              # slope_h = 2^(-SLOPE_LOG2 (h + 1) / heads): the design fixes it


@dataclass(frozen=True)
class GusedraMixer:
    type: str                          # "attention" | "attention_2"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]              # None: every earlier key
    keep_first: int = 0                # attention_2
    bias_max: Optional[int] = None     # attention_2
    kv_from: Optional[int] = None      # attention


@dataclass(frozen=True)
class GusedraMoe:
    experts: int
    identity: int
    top: int
    groups: int
    keep_groups: int
    scale: float
    ff: int
    shared_ff: Optional[int]


@dataclass(frozen=True)
class GusedraLayer:
    mixer: GusedraMixer
    mlp: object                        # None | int (dense: ff) | GusedraMoe


@dataclass(frozen=True)
class GusedraConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    layers: Tuple[GusedraLayer, ...]

    architecture = "Gusedra"

    # ------------------------------------------------------------------ parse
    @classmethod
    def from_dict(cls, raw: dict) -> "GusedraConfig":
        vocab, width = _int(raw, "vocab", "top level"), _int(raw, "width", "top level")
        eps = _num(_obj(raw, "norm", "top level"), "eps", "norm", positive=True)
        mult = _num(raw, "residual_mult", "top level") if raw.get("residual_mult") is not None else 1.0
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers: List[GusedraLayer] = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            if kind not in ("attention", "attention_2"):
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r} (attention, attention_2)")
            m = _obj(e, "mixer", where)
            mw = where + ".mixer"
            heads, kv_heads = _int(m, "heads", mw), _int(m, "kv_heads", mw)
            if heads % kv_heads:
                raise ConfigError(f"config.json: {mw}: heads ({heads}) is not a multiple of kv_heads ({kv_heads})")
            window, keep_first = None, 0
            if m.get("mask") is not None:
                mask = _obj(m, "mask", mw)
                window = _int(mask, "size", mw + ".mask")
                if kind == "attention_2" and mask.get("keep_first") is not None:
                    keep_first = _int(mask, "keep_first", mw + ".mask", least=0)
            bias_max = kv_from = None
            if kind == "attention_2":
                bias_max = _int(m, "bias_max", mw)
            if m.get("kv_from") is not None:
                kv_from = _int(m, "kv_from", mw, least=0)
            mixer = GusedraMixer(kind, heads, kv_heads, _int(m, "dim", mw), _int(m, "vdim", mw), _num(m, "scale", mw),
                                 window, keep_first, bias_max, kv_from)
            layers.append(GusedraLayer(mixer, cls._mlp(e.get("mlp"), where + ".mlp")))
        for i, layer in enumerate(layers):
            j = layer.mixer.kv_from
            if j is None:
                continue
            mw = f"layers[{i}].mixer"
            if not 0 <= j < len(layers) or j >= i:
                raise ConfigError(f"config.json: {mw}: kv_from ({j}) must name an earlier layer")
            src = layers[j].mixer
            if src.kv_from is not None:
                raise ConfigError(f"config.json: {mw}: kv_from ({j}) names a layer without keys and values of its own")
            mine, its = layer.mixer, src
            if (mine.kv_heads, mine.dim, mine.vdim) != (its.kv_heads, its.dim, its.vdim):
                raise ConfigError(f"config.json: {mw}: kv_heads, dim and vdim must equal those of layer {j}, whose keys "
                                  f"and values it reads")
        return cls(vocab, width, eps, mult, tuple(layers))

    @staticmethod
    def _mlp(mlp, where: str):
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json: {where} must be null or an object")
        kind = mlp.get("kind")
        if kind == "dense":
            return _int(mlp, "ff", where)
        if kind != "moe":
            raise ConfigError(f"config.json: {where}: unknown kind {kind!r} (dense, moe)")
        r = _obj(mlp, "router", where)
        rw = where + ".router"
        experts = _int(r, "experts", rw, least=0)
        identity = _int(r, "identity", rw, least=0) if r.get("identity") is not None else 0
        outputs = experts + identity
        if outputs < 1:
            raise ConfigError(f"config.json: {rw}: no experts")
        groups, keep = 1, 1
        if r.get("groups") is not None:
            g = _obj(r, "groups", rw)
            groups, keep = _int(g, "count", rw + ".groups"), _int(g, "keep", rw + ".groups")
        if outputs % groups or keep > groups:
            raise ConfigError(f"config.json: {rw}: {outputs} experts (identity experts included) must form {groups} equal "
                              f"groups, of which {keep} are kept")
        top = _int(r, "top", rw)
        if top > keep * (outputs // groups):
            raise ConfigError(f"config.json: {rw}: top ({top}) exceeds the {keep * (outputs // groups)} experts of the kept groups")
        scale = _num(r, "scale", rw) if r.get("scale") is not None else 1.0
        ff = _int(_obj(mlp, "expert", where), "ff", where + ".expert") if experts else 0
        shared_ff = _int(_obj(mlp, "shared", where), "ff", where + ".shared") if mlp.get("shared") is not None else None
        return GusedraMoe(experts, identity, top, groups, keep, scale, ff, shared_ff)

    # ------------------------------------------------------------------ export
    def to_dict(self) -> dict:
        """config.json content that parses back to this configuration."""
        out = []
        for layer in self.layers:
            m = layer.mixer
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
            if m.window is not None:
                mixer["mask"] = {"size": m.window}
                if m.type == "attention_2":
                    mixer["mask"]["keep_first"] = m.keep_first
            if m.bias_max is not None:
                mixer["bias_max"] = m.bias_max
            if m.kv_from is not None:
                mixer["kv_from"] = m.kv_from
            f = layer.mlp
            if f is None:
                mlp = None
            elif isinstance(f, int):
                mlp = {"kind": "dense", "ff": f}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.ff},
                       "router": {"experts": f.experts, "identity": f.identity, "top": f.top, "scale": f.scale,
                                  "groups": {"count": f.groups, "keep": f.keep_groups}}}
                if f.shared_ff is not None:
                    mlp["shared"] = {"ff": f.shared_ff}
            out.append({"type": m.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "residual_mult": self.residual_mult, "layers": out}

    # ------------------------------------------------------------------ spec
    def model_spec(self, tensor_names: Optional[Iterable[str]] = None) -> ModelSpec:
        """The architecture as parts.  The number of buckets of a learned bias is the checkpoint's (the rows
        of its table); without a checkpoint it is 32."""
        e, eps = self.width, self.eps
        shapes = tensor_names if hasattr(tensor_names, "get") else {}

        def norm(name: str, scale_by: str = "", mult: float = 1.0) -> NormSpec:
            return NormSpec("layernorm", e, eps, name, bias=name + ".b", scale_by=scale_by, mult=mult)

        layers: List[LayerSpec] = []
        order: List[RunEntry] = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}.mix."
            m = layer.mixer
            own = m.kv_from is None
            if m.type == "attention":
                bias = ScoreBiasSpec(kind="slopes", slope_log2=SLOPE_LOG2)
            else:
                rows = shapes.get(p + "rel")
                bias = ScoreBiasSpec(kind="buckets", table=p + "rel", buckets=int(rows[0]) if rows else 32,
                                     max_distance=int(m.bias_max))
            mixer = BiasedAttentionSpec(
                kind="biased_attention", hidden=e, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                v_head_dim=m.vdim, scale=m.scale, window=m.window, keep_first=m.keep_first, bias=bias,
                sink=p + "sink" if m.type == "attention" else "", gate_proj=p + "g" if m.type == "attention_2" else "",
                q_proj=p + "q", k_proj=p + "k" if own else "", v_proj=p + "v" if own else "", o_proj=p + "o")
            f = layer.mlp
            fp = f"l{i}.mlp."
            if f is None:
                ffn = None
            elif isinstance(f, int):
                ffn = DenseFfnSpec(kind="dense", hidden=e, intermediate=f, activation="relu2", up_proj=fp + "up",
                                   down_proj=fp + "down")
            else:
                shared = None
                if f.shared_ff is not None:
                    shared = GatedFfnSpec(kind="gated_dense", hidden=e, intermediate=f.shared_ff, activation="silu",
                                          gate_proj=fp + "shared.gate", up_proj=fp + "shared.up", down_proj=fp + "shared.down")
                ffn = RoutedFfnSpec(kind="routed", hidden=e, intermediate=f.ff, n_experts=f.experts, n_identity=f.identity,
                                    top=f.top, groups=f.groups, keep_groups=f.keep_groups, route_scale=f.scale,
                                    activation="silu", router=fp + "router", correction=fp + "correction",
                                    expert_prefix=fp + "e", shared=shared)
            mult = self.residual_mult
            layers.append(LayerSpec(
                kind="sandwich", mixer=mixer, ffn=ffn, pre_mixer_norm=norm(f"l{i}.norm1"),
                post_mixer_norm=norm(f"l{i}.norm1b", scale_by=f"l{i}.ls1", mult=mult),
                pre_ffn_norm=norm(f"l{i}.norm2") if ffn is not None else None,
                post_ffn_norm=norm(f"l{i}.norm2b", scale_by=f"l{i}.ls2", mult=mult) if ffn is not None else None))
            # a layer without keys and values reads the memory of the layer it names, and appends nothing
            order.append(RunEntry(i, i, True) if own else RunEntry(i, m.kv_from, False))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden=e, embed_weight="embed", embed_scale=1.0,
            layers=layers, order=order, final_norm=norm("final.norm"), head_weight="head", max_context=POSITIONS,
            bos_token_id=None, eos_token_ids=(),
            # a tensor that no part asks for (the second norms of a layer without a feed-forward, say) is passed over
            tensor_scope=())
