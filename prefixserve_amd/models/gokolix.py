"""The Gokolix decoder as a ``ModelSpec``.

Every layer is a parallel block (one norm whose weight is stored as its distance from one; mixer
and feed-forward both read it and both add to the stream). The mixer is, layer by layer, one of:
paged grouped-query attention without rotation, with biases on q and k, a weighted norm per
head, the un-normed keys as values, a learned bias by bucketed distance, a window and a sink;
latent attention with a YaRN-scaled rotation of the shared key part; a gated linear recurrence.
The feed-forward, where a layer has one, is a dense gated one with ReLU on the gate. The token
table's rows are scaled, and it is the output matrix too, unscaled.

A stretch of layers may be passed through several times with the same weights: the order then
lists those layers once per pass, every run with a cache entry (or state) of its own, and the
first run of every pass is preceded by the re-entry transform (the stream mixed with the token
table's output again, plus a learned row per pass). Weight names are the checkpoint's own
(``l<i>.mix.q`` ...).
"""

from __future__ import annotations

from prefixserve_amd.config.gokolix import MAX_POSITION, GokolixConfig
from prefixserve_amd.config.llama import UnsupportedModelError
from prefixserve_amd.config.registry import register_architecture
from prefixserve_amd.parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

ATTENTION_NAMES = {"q": "mix.q", "k": "mix.k", "o": "mix.o", "q_bias": "mix.q.b", "k_bias": "mix.k.b",
                   "q_norm": "mix.q.norm", "k_norm": "mix.k.norm", "rel": "mix.rel", "sink": "mix.sink"}
LATENT_NAMES = {"q": "mix.q", "down": "mix.dkv", "down_norm": "mix.dkv.norm", "up_k": "mix.uk", "up_v": "mix.uv",
                "o": "mix.o", "sink": "mix.sink"}
RECURRENCE_NAMES = {"y": "mix.y", "y_bias": "mix.y.b", "x": "mix.x", "x_bias": "mix.x.b", "conv": "mix.conv",
                    "conv_bias": "mix.conv.b", "gate_r": "mix.ra", "gate_r_bias": "mix.ra.b", "gate_i": "mix.ri",
                    "gate_i_bias": "mix.ri.b", "lam": "mix.lam", "o": "mix.o"}
FEED_FORWARD_NAMES = {"gate": "mlp.gate", "up": "mlp.up", "down": "mlp.down"}
# Fixed by the design, not by a file: the recurrence's decay is exp(-8 r softplus(lam)).
DECAY_SCALE = 8.0


def build_gokolix_spec(cfg: GokolixConfig) -> ModelSpec:
    positions: dict[str, PartSpec] = {}
    by_params: dict[str, str] = {}
    layers = []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "attention":
            if m.buckets is None:
                raise UnsupportedModelError(f"layers[{i}]: the number of rows of the bias table is not known "
                                            "(neither a checkpoint's l<i>.mix.rel nor a 'buckets' key says)")
            mixer = PartSpec("paged_attention", {
                "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "names": ATTENTION_NAMES,
                "scale": m.scale, "window": m.window, "qk_norm_eps": cfg.norm_eps, "qk_norm_weights": True,
                "qk_bias": True, "values_are_keys": True, "sink": True, "exact_weights": True,
                "distance_bias": {"buckets": m.buckets, "far": m.bias_max},
            })
        elif layer.type == "latent_attention":
            name = None
            if m.rot_dim:
                s = m.rot_scaling
                scaling = None if s is None else {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
                rot = PartSpec("yarn", {"head_dim": m.rot_dim, "rotary_dim": m.rot_dim, "base": m.rot_base, "scaling": scaling})
                key = repr(sorted(rot.params.items(), key=lambda kv: kv[0]))
                name = by_params.setdefault(key, f"rot{len(by_params)}")          # equal rotations share one table
                positions[name] = rot
            mixer = PartSpec("latent_attention", {
                "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim, "rank": m.kv_rank,
                "names": LATENT_NAMES, "norm_eps": cfg.norm_eps, "position": name, "scale": m.scale, "window": m.window,
                "sink": True,
            })
        else:
            mixer = PartSpec("gated_linear_recurrence", {"width": m.width, "blocks": m.blocks, "taps": m.conv,
                                                         "names": RECURRENCE_NAMES, "decay_scale": DECAY_SCALE})
        ff = None
        if layer.ff is not None:
            ff = PartSpec("swiglu", {"intermediate_size": layer.ff, "names": FEED_FORWARD_NAMES, "activation": "relu"})
        layers.append(LayerSpec(
            prefix=f"l{i}.", mixer=mixer, feed_forward=ff,
            mixer_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "norm1", "unit_offset": True}),
            feed_forward_norm=None, block="parallel",
        ))

    # The order: layers in front of the repeated stretch, the stretch once per pass, the rest.
    order: list[LayerRun] = []
    transforms: dict[str, PartSpec] = {}
    n, loop = len(cfg.layers), cfg.loop
    if loop is None:
        sequence = [(i, 0, False) for i in range(n)]
    else:
        transforms["reentry"] = PartSpec("reentry", {"passes": loop.times, "names": {"in": "loop.in", "step": "loop.step"}})
        sequence = [(i, 0, False) for i in range(loop.start)]
        for p in range(loop.times):
            sequence += [(i, p, i == loop.start) for i in range(loop.start, loop.stop)]
        sequence += [(i, 0, False) for i in range(loop.stop, n)]
    for entry, (i, p, opens) in enumerate(sequence):
        order.append(LayerRun(i, entry, True, before=("reentry",) if opens else (), pass_index=p))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embedding="embed", layers=tuple(layers),
        order=tuple(order), final_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "final.norm", "unit_offset": True}),
        final_norm_prefix="", head=None, positions=positions, max_position=MAX_POSITION,
        stop_token_ids=cfg.stop_token_ids,
        embedding_transforms=(PartSpec("scale", {"factor": cfg.embedding_scale}),),
        stream_transforms=transforms,
    )


register_architecture("Gokolix", GokolixConfig, build_gokolix_spec)
