"""The Radivik decoder as a ``ModelSpec``.

Every layer keeps its norm behind the sum (block "postnorm" with the configuration's factor on
the stream); its mixer is paged grouped-query attention with a value size of its own, a
YaRN-scaled rotation of the head's leading dimensions, queries and keys brought to unit root
mean square behind the rotation and the score scale the file gives; its feed-forward, where
it has one, a mixture of experts. A layer that names another layer under ``kv_from`` has no
key and value projections: its run reads the cache entry that layer's run writes. Layers
may differ in all of this; weight names are the checkpoint's own (``l<i>.mix.q`` ...).
"""

from __future__ import annotations

from prefixserve_amd.config.radivik import MAX_POSITION, RadivikAttention, RadivikConfig
from prefixserve_amd.config.registry import register_architecture
from prefixserve_amd.parts.attention import slot_size
from prefixserve_amd.parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

MIXER_NAMES = {"q": "mix.q", "k": "mix.k", "v": "mix.v", "o": "mix.o"}
EXPERT_NAMES = {"router": "mlp.router", "gate": "mlp.e{e}.gate", "up": "mlp.e{e}.up", "down": "mlp.e{e}.down"}
# Fixed by the design, not by a file: the gate's sigmoid is taken at 1.702 g, the linear branch is shifted by 1.
GATE_ALPHA = 1.702
UP_SHIFT = 1.0


def _rotation(m: RadivikAttention) -> PartSpec:
    scaling = None
    if m.rot_scaling is not None:
        s = m.rot_scaling
        scaling = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
    return PartSpec("yarn", {"head_dim": slot_size(m.dim, m.vdim), "rotary_dim": m.rot_dims, "base": m.rot_base,
                             "scaling": scaling})


def build_radivik_spec(cfg: RadivikConfig) -> ModelSpec:
    positions: dict[str, PartSpec] = {}
    by_params: dict[str, str] = {}
    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        # Layers whose rotation is the same share one table.
        rot = _rotation(m)
        key = repr(sorted(rot.params.items(), key=lambda kv: kv[0]))
        name = by_params.setdefault(key, f"rot{len(by_params)}")
        positions[name] = rot
        mixer = PartSpec("paged_attention", {
            "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim,
            "names": MIXER_NAMES, "position": name, "scale": m.scale, "qk_norm_eps": cfg.norm_eps,
            "own_kv": m.kv_from is None, "exact_weights": True,
        })
        ff = ff_norm = None
        if layer.mlp is not None:
            f = layer.mlp
            ff = PartSpec("routed_experts", {
                "num_experts": f.experts, "top_k": f.top, "intermediate_size": f.ff, "names": EXPERT_NAMES,
                "limit": f.limit, "gate_alpha": GATE_ALPHA, "up_shift": UP_SHIFT,
            })
            ff_norm = PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "norm2"})
        elif layer.lone_second_norm:
            ff_norm = PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "norm2"})
        layers.append(LayerSpec(
            prefix=f"l{i}.", mixer=mixer, feed_forward=ff,
            mixer_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "norm1"}), feed_forward_norm=ff_norm,
            block="postnorm", block_params={"alpha": cfg.postln_alpha},
        ))
        order.append(LayerRun(i, i, True) if m.kv_from is None else LayerRun(i, m.kv_from, False))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embedding="embed", layers=tuple(layers),
        order=tuple(order), final_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "final.norm"}),
        final_norm_prefix="", head="head", positions=positions, max_position=MAX_POSITION,
        stop_token_ids=cfg.stop_token_ids,
    )


register_architecture("Radivik", RadivikConfig, build_radivik_spec)
