"""Tiny Radivik configurations for the tests. They differ from each other in every size and
option the design has: width, vocabulary, head counts and groups (6/2, 4/4, 8/1), query/key and
value sizes (value larger, smaller and equal; 24 is no multiple of 16), how much of a head
rotates (a part, all of it), the rotation's base and scaling (present with a blend band inside
the rotated dimensions, absent), the score scale, which layers read another layer's keys and
values (and how many read the same one), layers without a feed-forward, the number of experts
and how many a token uses (1, 2, 3), the experts' inner size and clamp (tight and loose), the
factor on the stream (other than 1 and equal to 1), and the norms' eps."""

from __future__ import annotations


def _mixer(heads, kv_heads, dim, vdim, scale, dims, base, scaling=None, kv_from=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts, top, ff, limit):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


_S1 = {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0}
_M1 = dict(heads=6, kv_heads=2, dim=32, vdim=48, scale=0.35, dims=12, base=900.0, scaling=_S1)
_M2 = dict(heads=4, kv_heads=4, dim=24, vdim=16, scale=0.6, dims=24, base=10000.0)
_M3 = dict(heads=8, kv_heads=1, dim=16, vdim=16, scale=1.5, dims=4, base=50.0,
           scaling={"factor": 16.0, "original": 16, "fast": 4.0, "slow": 0.5})

RADIVIK = {
    # own keys, a reader without feed-forward, own keys again, two readers of the same layer
    "P": {"architecture": "Radivik", "vocab": 120, "width": 96, "norm": {"eps": 1e-5}, "postln_alpha": 1.5, "layers": [
        _layer(_mixer(**_M1), _moe(5, 2, 40, 0.7)),
        _layer(_mixer(**_M1, kv_from=0), None),
        _layer(_mixer(**_M1), _moe(5, 2, 40, 0.7)),
        _layer(_mixer(**_M1, kv_from=2), _moe(7, 3, 24, 0.7)),
        _layer(_mixer(**_M1, kv_from=2), _moe(5, 2, 40, 0.7)),
    ]},
    # every head its own keys, the whole head rotates, no scaling, loose clamp, alpha 1
    "Q": {"architecture": "Radivik", "vocab": 90, "width": 64, "norm": {"eps": 1e-6}, "postln_alpha": 1.0, "layers": [
        _layer(_mixer(**_M2), _moe(4, 3, 56, 6.0)),
        _layer(_mixer(**_M2), None),
        _layer(_mixer(**_M2, kv_from=1), _moe(4, 1, 56, 6.0)),
    ]},
    # one kv head for eight query heads, layers of different shapes in one model (two layer groups)
    "R": {"architecture": "Radivik", "vocab": 200, "width": 128, "norm": {"eps": 1e-5}, "postln_alpha": 3.0, "layers": [
        _layer(_mixer(**_M3), _moe(9, 1, 32, 1.2)),
        _layer(_mixer(**_M1), _moe(3, 2, 64, 0.4)),
        _layer(_mixer(**_M3, kv_from=0), _moe(9, 1, 32, 1.2)),
    ]},
}

RADIVIK_STD = 0.12     # projections of unit-size rows come out near 1: clamps and the softmax both bite


def write_radivik(folder, name: str, seed: int = 3, std: float = RADIVIK_STD, config=None):
    from prefixserve_amd.weights import write_random_model

    return write_random_model(folder, config if config is not None else RADIVIK[name], seed=seed, std=std)
