"""The Gokolix architecture's configuration, typed, from its own ``config.json`` keys.

A Gokolix file gives the width (``width``), the vocabulary (``vocab``), the norms' epsilon
(``norm.eps``), the factor on the token table's rows (``embedding.scale``), its layers one by
one (``layers``: each with ``type`` = which mixer, the mixer's sizes and constants under
``mixer`` and its feed-forward under ``mlp`` or null) and, under ``loop``, a run of layers that
is passed through several times with the same weights. Every size and constant is read from
there; a key this parser does not know raises, because a rule dropped without a word would load
and then compute something else.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping

from .llama import UnsupportedModelError
from .radivik import YarnScaling, _only

ARCHITECTURE = "Gokolix"
# No position limit is part of the design; the engine's own ``max_seq_len`` bounds the tables.
MAX_POSITION = 1 << 20


def _window(m: Mapping[str, Any], where: str) -> int | None:
    mask = m.get("mask")
    if mask is None:
        return None
    _only(mask, ("size",), where + ".mask")
    size = int(mask["size"])
    if size < 1:
        raise UnsupportedModelError(f"{where}.mask.size must be at least 1, got {size}")
    return size


@dataclass(frozen=True)
class BiasedAttention:
    """Grouped-query attention without rotation: biases on q and k, a weighted norm per head,
    values that are the un-normed keys, a learned bias per bucket of the distance, a sink."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: float          # the distance from which on the bias table's last row is used
    window: int | None
    # Rows of the bias table. config.json does not have to say: the table's shape in the checkpoint does
    # (``GokolixConfig.fitted_to_checkpoint``); a file written without a checkpoint to look at names it.
    buckets: int | None = None

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "BiasedAttention":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "bias_max", "mask", "buckets"), where)
        heads, kv_heads = int(m["heads"]), int(m["kv_heads"])
        if kv_heads < 1 or heads % kv_heads:
            raise UnsupportedModelError(f"{where}: {heads} heads cannot share {kv_heads} key/value heads")
        dim, vdim = int(m["dim"]), int(m.get("vdim", m["dim"]))
        if vdim != dim:
            raise UnsupportedModelError(f"{where}: the values are the keys, so vdim {vdim} must equal dim {dim}")
        buckets = m.get("buckets")
        return cls(heads, kv_heads, dim, vdim, float(m["scale"]), float(m["bias_max"]), _window(m, where),
                   None if buckets is None else int(buckets))

    def to_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "bias_max": self.bias_max}
        if self.buckets is not None:
            out["buckets"] = self.buckets
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class LatentAttention:
    """Attention whose keys and values are made from one compressed vector per token."""

    heads: int
    dim: int                 # un-rotated query/key dimensions per head
    rot_dim: int             # rotated ones
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_scaling: YarnScaling | None
    window: int | None

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "LatentAttention":
        _only(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot", "mask"), where)
        rot_dim = int(m.get("rot_dim", 0))
        rot = m.get("rot") or {"base": 10000.0, "dims": rot_dim}       # a mixer without a rotated part need not describe a rotation
        _only(rot, ("base", "dims", "scaling"), where + ".rot")
        if int(rot.get("dims", rot_dim)) != rot_dim or rot_dim % 2 or rot_dim < 0:
            raise UnsupportedModelError(f"{where}: the rotated part is rot_dim = {rot_dim} wide and even; rot.dims says {rot.get('dims')}")
        if int(m["heads"]) < 1 or int(m["kv_rank"]) < 1:
            raise UnsupportedModelError(f"{where}: heads and kv_rank must be positive")
        return cls(int(m["heads"]), int(m["dim"]), rot_dim, int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]),
                   float(rot["base"]), YarnScaling.from_json(rot.get("scaling")), _window(m, where))

    def to_json(self) -> dict[str, Any]:
        rot: dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dim}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_json()
        out: dict[str, Any] = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "scale": self.scale, "rot": rot}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class GatedRecurrence:
    """A gated linear recurrence behind a short causal convolution."""

    width: int
    blocks: int              # the gates' matrices are block-diagonal with this many blocks
    conv: int                # taps of the convolution

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "GatedRecurrence":
        _only(m, ("width", "blocks", "conv"), where)
        width, blocks, conv = int(m["width"]), int(m["blocks"]), int(m["conv"])
        if blocks < 1 or width % blocks or conv < 1:
            raise UnsupportedModelError(f"{where}: width {width} in {blocks} blocks, {conv} taps")
        return cls(width, blocks, conv)

    def to_json(self) -> dict[str, Any]:
        return {"width": self.width, "blocks": self.blocks, "conv": self.conv}


MIXERS = {"attention": BiasedAttention, "latent_attention": LatentAttention, "rglru": GatedRecurrence}


@dataclass(frozen=True)
class GokolixLayer:
    type: str
    mixer: Any
    ff: int | None           # inner size of the dense gated feed-forward; None: the layer has none


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class GokolixConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    embedding_scale: float
    layers: tuple[GokolixLayer, ...]
    loop: Loop | None
    stop_token_ids: frozenset[int] = frozenset()

    @classmethod
    def from_dicts(cls, raw: Mapping[str, Any], gen: Mapping[str, Any] | None = None) -> "GokolixConfig":
        _only(raw, ("architecture", "architectures", "embedding", "layers", "loop", "norm", "vocab", "width"), "config.json")
        _only(raw["norm"], ("eps",), "norm")
        emb = raw.get("embedding") or {}
        _only(emb, ("scale",), "embedding")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = entry.get("type")
            if kind not in MIXERS:
                raise UnsupportedModelError(f"{where}: mixer type {kind!r}; implemented: {sorted(MIXERS)}")
            mixer = MIXERS[kind].from_json(entry["mixer"], where + ".mixer")
            ff = None
            if entry.get("mlp") is not None:
                f = entry["mlp"]
                _only(f, ("kind", "ff"), where + ".mlp")
                if f.get("kind") != "dense":
                    raise UnsupportedModelError(f"{where}.mlp: feed-forward kind {f.get('kind')!r}; only 'dense' is implemented")
                ff = int(f["ff"])
            layers.append(GokolixLayer(kind, mixer, ff))
        loop = None
        if raw.get("loop") is not None:
            lp = raw["loop"]
            _only(lp, ("start", "stop", "times"), "loop")
            loop = Loop(int(lp["start"]), int(lp["stop"]), int(lp["times"]))
            if not 0 <= loop.start < loop.stop <= len(layers) or loop.times < 1:
                raise UnsupportedModelError(f"loop {lp} does not fit {len(layers)} layers")
        return cls(int(raw["vocab"]), int(raw["width"]), float(raw["norm"]["eps"]), float(emb.get("scale", 1.0)),
                   tuple(layers), loop)

    def fitted_to_checkpoint(self, shapes: Mapping[str, tuple[int, ...]]) -> "GokolixConfig":
        """The configuration with what the checkpoint's tensor shapes decide: the rows of every
        attention layer's bias table."""
        layers = []
        for i, layer in enumerate(self.layers):
            shape = shapes.get(f"l{i}.mix.rel") if layer.type == "attention" else None
            if shape is not None:
                layer = replace(layer, mixer=replace(layer.mixer, buckets=int(shape[0])))
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    def to_config_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
            "layers": [{"type": l.type, "mixer": l.mixer.to_json(),
                        "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}} for l in self.layers],
            "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size, "width": self.hidden_size,
        }
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out
