"""The Radivik architecture's configuration, typed, from its own ``config.json`` keys.

A Radivik file lists its layers one by one (``layers``: each with ``type``, the mixer's
sizes under ``mixer`` and its feed-forward under ``mlp`` or null), and gives the width
(``width``), the vocabulary (``vocab``), the norms' epsilon (``norm.eps``) and the factor on
the stream in front of every sum (``postln_alpha``). Every size and constant is read from
there; a key this parser does not know raises, because a rule dropped without a word would
load and then compute something else.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Mapping

from .llama import UnsupportedModelError

ARCHITECTURE = "Radivik"
# No position limit is part of the design; the engine's own ``max_seq_len`` bounds the tables.
MAX_POSITION = 1 << 20


def _only(entry: Mapping[str, Any], known: tuple[str, ...], where: str) -> None:
    extra = sorted(set(entry) - set(known))
    if extra:
        raise UnsupportedModelError(f"{where}: keys {extra} are not understood")


@dataclass(frozen=True)
class YarnScaling:
    """Frequencies slowed by ``factor`` for waves that make fewer than ``slow`` turns over the
    ``original`` length, kept for those that make more than ``fast``, blended in between."""

    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def from_json(cls, entry: Mapping[str, Any] | None) -> "YarnScaling | None":
        if entry is None:
            return None
        _only(entry, ("factor", "original", "fast", "slow"), "rot.scaling")
        return cls(float(entry["factor"]), float(entry["original"]), float(entry["fast"]), float(entry["slow"]))

    def to_json(self) -> dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class RadivikAttention:
    heads: int
    kv_heads: int
    dim: int                 # per-head size of queries and keys
    vdim: int                # per-head size of values
    scale: float             # factor on q.k
    rot_dims: int            # leading dimensions of a head that are rotated
    rot_base: float
    rot_scaling: YarnScaling | None
    kv_from: int | None      # the layer whose keys and values this layer reads; None: its own

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "RadivikAttention":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "rot", "kv_from"), where)
        rot = m["rot"]
        _only(rot, ("base", "dims", "scaling"), where + ".rot")
        heads, kv_heads = int(m["heads"]), int(m["kv_heads"])
        if kv_heads < 1 or heads % kv_heads:
            raise UnsupportedModelError(f"{where}: {heads} heads cannot share {kv_heads} key/value heads")
        dim, dims = int(m["dim"]), int(rot["dims"])
        if dims % 2 or not 0 <= dims <= dim:
            raise UnsupportedModelError(f"{where}: rot.dims must be even and at most dim, got {dims} of {dim}")
        kv_from = m.get("kv_from")
        return cls(heads, kv_heads, dim, int(m["vdim"]), float(m["scale"]), dims, float(rot["base"]),
                   YarnScaling.from_json(rot.get("scaling")), None if kv_from is None else int(kv_from))

    def to_json(self) -> dict[str, Any]:
        rot: dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = self.rot_scaling.to_json()
        out: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "rot": rot}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class RadivikExperts:
    experts: int
    top: int
    ff: int                  # inner size of one expert
    limit: float             # bound on the gate (from above) and on the linear branch (both sides)

    @classmethod
    def from_json(cls, f: Mapping[str, Any], where: str) -> "RadivikExperts":
        _only(f, ("kind", "router", "expert"), where)
        if f.get("kind") != "moe":
            raise UnsupportedModelError(f"{where}: feed-forward kind {f.get('kind')!r}; only 'moe' is implemented")
        _only(f["router"], ("experts", "top"), where + ".router")
        _only(f["expert"], ("ff", "limit"), where + ".expert")
        experts, top = int(f["router"]["experts"]), int(f["router"]["top"])
        if not 1 <= top <= experts:
            raise UnsupportedModelError(f"{where}: top {top} of {experts} experts")
        return cls(experts, top, int(f["expert"]["ff"]), float(f["expert"]["limit"]))

    def to_json(self) -> dict[str, Any]:
        return {"kind": "moe", "router": {"experts": self.experts, "top": self.top},
                "expert": {"ff": self.ff, "limit": self.limit}}


@dataclass(frozen=True)
class RadivikLayer:
    mixer: RadivikAttention
    mlp: RadivikExperts | None
    # A layer without a feed-forward has no second half; if its checkpoint nevertheless brings a
    # second norm, that norm is applied to the stream alone: x <- norm2(alpha x).
    lone_second_norm: bool = False


@dataclass(frozen=True)
class RadivikConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    postln_alpha: float
    layers: tuple[RadivikLayer, ...]
    stop_token_ids: frozenset[int] = frozenset()

    @classmethod
    def from_dicts(cls, raw: Mapping[str, Any], gen: Mapping[str, Any] | None = None) -> "RadivikConfig":
        _only(raw, ("architecture", "architectures", "layers", "norm", "postln_alpha", "vocab", "width"), "config.json")
        _only(raw["norm"], ("eps",), "norm")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            if entry.get("type") != "attention":
                raise UnsupportedModelError(f"{where}: mixer type {entry.get('type')!r}; only 'attention' is implemented")
            mixer = RadivikAttention.from_json(entry["mixer"], where + ".mixer")
            mlp = None if entry.get("mlp") is None else RadivikExperts.from_json(entry["mlp"], where + ".mlp")
            layers.append(RadivikLayer(mixer, mlp))
        for i, layer in enumerate(layers):
            j = layer.mixer.kv_from
            if j is None:
                continue
            if not 0 <= j < i or layers[j].mixer.kv_from is not None:
                raise UnsupportedModelError(f"layers[{i}].mixer.kv_from = {j}: must name an earlier layer with keys of its own")
            a, b = layer.mixer, layers[j].mixer
            if (a.kv_heads, a.dim, a.vdim) != (b.kv_heads, b.dim, b.vdim):
                raise UnsupportedModelError(f"layers[{i}] reads layer {j}'s keys and values but has other sizes")
        return cls(int(raw["vocab"]), int(raw["width"]), float(raw["norm"]["eps"]), float(raw["postln_alpha"]), tuple(layers))

    def fitted_to_checkpoint(self, names: "Mapping[str, tuple[int, ...]] | frozenset[str]") -> "RadivikConfig":
        """The configuration with what the checkpoint's tensor names decide."""
        layers = tuple(replace(layer, lone_second_norm=layer.mlp is None and f"l{i}.norm2" in names)
                       for i, layer in enumerate(self.layers))
        return replace(self, layers=layers)

    def to_config_json(self) -> dict[str, Any]:
        return {
            "architecture": ARCHITECTURE,
            "layers": [{"type": "attention", "mixer": l.mixer.to_json(), "mlp": None if l.mlp is None else l.mlp.to_json()}
                       for l in self.layers],
            "norm": {"eps": self.norm_eps}, "postln_alpha": self.postln_alpha,
            "vocab": self.vocab_size, "width": self.hidden_size,
        }
