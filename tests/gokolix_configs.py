"""Tiny Gokolix configurations for the tests. They differ from each other in what the design
lets differ: width, vocabulary, the factor on the token table, the order and kinds of layers,
head counts and groups (4/4, 6/2, 3/1, 1/1), head sizes (also ones that are no multiple of 16),
windows (none, 1, a few tokens, longer than the prompts), the bias table's rows and reach, the
latent size against the head size (larger and smaller), how many dimensions rotate, the
rotation's scaling (present, absent), the recurrence's width, blocks (1 to several) and taps
(1 to 5), layers without a feed-forward, and the repeated stretch: none, the whole model once,
a middle stretch three times."""

from __future__ import annotations

import copy
import json
from pathlib import Path


def attention(heads, kv_heads, dim, scale, bias_max, buckets, window=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "bias_max": bias_max, "buckets": buckets}
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "attention", "mixer": m}


def latent(heads, dim, rot_dim, vdim, rank, scale, base, scaling=None, window=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def recurrence(width, blocks, taps):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": taps}}


def layer(mixer, ff):
    return {**mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def model(vocab, width, eps, scale, layers, loop=None):
    out = {"architecture": "Gokolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
           "layers": layers}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


_YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}

GOKOLIX = {
    # a middle stretch passed through three times: recurrence and latent attention inside it
    "A": model(96, 64, 1e-5, 3.0, [
        layer(attention(4, 4, 16, 0.4, 20, 12, window=8), 80),
        layer(recurrence(48, 3, 3), 40),
        layer(latent(2, 24, 8, 16, 40, 0.3, 500.0, _YARN, window=24), None),
        layer(attention(6, 2, 8, 0.9, 9, 6, window=5), 56),
    ], loop=(1, 3, 3)),
    # no repeated stretch, a layer without a window, one tap, one block, one kv head, one latent head
    "B": model(130, 72, 1e-6, 1.0, [
        layer(latent(1, 12, 4, 20, 16, 0.5, 10000.0), 48),
        layer(recurrence(40, 1, 1), None),
        layer(attention(3, 1, 24, 0.25, 40, 16), 64),
        layer(recurrence(56, 7, 5), 32),
    ]),
    # the whole model as one pass, a window of one token, the latent smaller than a head
    "C": model(70, 48, 1e-5, 7.5, [
        layer(attention(1, 1, 40, 0.2, 6, 4, window=1), 24),
        layer(latent(4, 32, 16, 8, 24, 0.15, 50.0, {"factor": 16.0, "original": 16, "fast": 4.0, "slow": 0.5}, window=300), 72),
        layer(recurrence(32, 4, 2), 16),
    ], loop=(0, 3, 1)),
}

STD = 0.15      # projections of unit-size rows come out near 1: the softmax, the gates and the ReLU all bite


def write_gokolix(folder, name_or_config, seed: int = 3, std: float = STD, keep_buckets: bool = False, edit=None) -> Path:
    """A model folder with random weights. config.json does not say how many rows the bias tables
    have (unless ``keep_buckets``): the loader takes that from the checkpoint, as for a file that
    never had the key. ``edit(tensors)`` may change the tensors before they are written."""
    from safetensors.torch import save_file

    import prefixserve_amd.models  # noqa: F401
    from prefixserve_amd.config.registry import architecture_of
    from prefixserve_amd.parts.model import DecoderModel
    from prefixserve_amd.weights import random_tensors

    config = copy.deepcopy(GOKOLIX[name_or_config] if isinstance(name_or_config, str) else name_or_config)
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    arch = architecture_of(config)
    want = DecoderModel(arch.build_spec(arch.config_cls.from_dicts(config, {}))).weights()
    tensors = random_tensors(want, seed=seed, std=std)
    if edit is not None:
        edit(tensors)
    if not keep_buckets:
        for entry in config["layers"]:
            entry["mixer"].pop("buckets", None)
    (folder / "config.json").write_text(json.dumps(config, indent=1))
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
