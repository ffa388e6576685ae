"""One registry from an architecture's name to its configuration class and model builder.

``config.json["architectures"][0]`` (or its ``"architecture"``, a plain name) picks the entry; the entry's configuration class
parses the architecture's own keys and its builder turns the typed configuration into a
``ModelSpec``. An unknown name is an error that lists what is registered.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Mapping

from prefixserve_amd.parts.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Any                              # needs from_dicts(raw, gen) -> config
    build_spec: Callable[[Any], ModelSpec]


_ARCHITECTURES: dict[str, Architecture] = {}


class UnknownArchitectureError(ValueError):
    pass


def register_architecture(name: str, config_cls: Any, build_spec: Callable[[Any], ModelSpec]) -> None:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_cls, build_spec)


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def architecture_of(raw: Mapping[str, Any]) -> Architecture:
    archs = raw.get("architectures")
    if isinstance(raw.get("architecture"), str) and not archs:
        archs = [raw["architecture"]]            # files that name their one architecture in the singular
    if not archs or not isinstance(archs, list):
        raise UnknownArchitectureError(
            f"config.json has no 'architectures' entry; registered: {registered_architectures()}")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise UnknownArchitectureError(
            f"architecture {name!r} is not registered; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def read_model_dir(model_dir: str | Path) -> tuple[Architecture, Any, dict[str, Any]]:
    """(architecture entry, typed configuration, raw config.json) of a model folder."""
    model_dir = Path(model_dir)
    cfg_path = model_dir / "config.json"
    if not cfg_path.exists():
        raise FileNotFoundError(f"{cfg_path} not found")
    raw = json.loads(cfg_path.read_text())
    gen_path = model_dir / "generation_config.json"
    gen = json.loads(gen_path.read_text()) if gen_path.exists() else {}
    arch = architecture_of(raw)
    cfg = arch.config_cls.from_dicts(raw, gen)
    # A configuration class may look at which tensors the checkpoint holds (names and shapes, from
    # the files' headers) where its config.json leaves something to the checkpoint.
    fit = getattr(cfg, "fitted_to_checkpoint", None)
    if fit is not None:
        names = _tensor_names(model_dir)
        if names is not None:
            cfg = fit(names)
    return arch, cfg, raw


def _tensor_names(model_dir: Path) -> dict[str, tuple[int, ...]] | None:
    """Name -> shape of the tensors in the folder's safetensors files, read from their headers; None if there are none."""
    import struct

    files = sorted(model_dir.glob("*.safetensors"))
    if not files:
        return None
    names: dict[str, tuple[int, ...]] = {}
    for f in files:
        with open(f, "rb") as fh:
            (n,) = struct.unpack("<Q", fh.read(8))
            names.update((k, tuple(v["shape"])) for k, v in json.loads(fh.read(n)).items() if k != "__metadata__")
    return names
