"""Radivik on the host: its configuration, the model built from it, and the whole engine path
(packing, pages, shared cache entries, replay, scheduler, generation) with the kernel library's
CPU stand-in, against the plain implementation in tests/plain/radivik_plain.py."""

from __future__ import annotations

import copy
import json
import math

import numpy as np
import pytest
import torch

import traces
from emulated_ops import EmulatedOps
from plain import radivik_plain as plain
from prefixserve_amd.config import RadivikConfig, UnsupportedModelError, read_model_dir
from prefixserve_amd.engine.batch import StepItem
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner
from prefixserve_amd.models.radivik import build_radivik_spec
from prefixserve_amd.parts.attention import head_slots, slot_size
from prefixserve_amd.parts.base import Runtime, Workspace
from prefixserve_amd.parts.rope import YarnRotary
from radivik_configs import RADIVIK, write_radivik


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_radivik(tmp_path_factory.mktemp(f"radivik-{name}"), name) for name in RADIVIK}


def test_configuration_reads_every_key_and_refuses_what_it_does_not_know():
    cfg = RadivikConfig.from_dicts(RADIVIK["P"])
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.postln_alpha) == (120, 96, 1e-5, 1.5)
    m = cfg.layers[3].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.rot_dims, m.rot_base, m.kv_from) == (6, 2, 32, 48, 0.35, 12, 900.0, 2)
    assert m.rot_scaling.factor == 4.0 and m.rot_scaling.original == 48 and (m.rot_scaling.fast, m.rot_scaling.slow) == (8.0, 1.0)
    assert cfg.layers[1].mlp is None and cfg.layers[0].mixer.kv_from is None
    f = cfg.layers[3].mlp
    assert (f.experts, f.top, f.ff, f.limit) == (7, 3, 24, 0.7)
    assert RadivikConfig.from_dicts(cfg.to_config_json()) == cfg
    for path, value in [(("layers", 0, "mixer", "window"), 8), (("layers", 0, "mlp", "kind"), "dense"),
                        (("layers", 0, "type"), "recurrent"), (("layers", 0, "mixer", "rot", "kind"), "x"),
                        (("sink",), True), (("layers", 1, "mixer", "kv_from"), 1), (("layers", 1, "mixer", "kv_from"), 3),
                        (("layers", 3, "mixer", "kv_from"), 1), (("layers", 0, "mlp", "router", "top"), 6)]:
        raw = copy.deepcopy(RADIVIK["P"])
        at = raw
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(UnsupportedModelError):
            RadivikConfig.from_dicts(raw)


def test_spec_shares_cache_entries_and_tables(folders):
    arch, cfg, _ = read_model_dir(folders["P"])
    assert arch.name == "Radivik"
    spec = build_radivik_spec(cfg)
    assert [(r.layer, r.cache, r.writes_cache) for r in spec.order] == [
        (0, 0, True), (1, 0, False), (2, 2, True), (3, 2, False), (4, 2, False)]
    assert len(spec.positions) == 1                       # one rotation for all five layers
    assert spec.layers[1].feed_forward is None and spec.layers[1].feed_forward_norm is None
    assert "k" not in spec.layers[1].mixer.params["names"] or not spec.layers[1].mixer.params["own_kv"]
    spec_r = build_radivik_spec(RadivikConfig.from_dicts(RADIVIK["R"]))
    assert len(spec_r.positions) == 2


def test_reader_layers_have_no_key_and_value_tensors(folders):
    from safetensors import safe_open

    with safe_open(str(folders["P"] / "model.safetensors"), framework="pt") as f:
        names = set(f.keys())
    assert {"l0.mix.k", "l0.mix.v", "l2.mix.k", "l1.mix.q", "l1.mix.o", "l0.norm2", "l3.mlp.e6.down", "l3.mlp.router",
            "final.norm", "head", "embed"} <= names
    assert not {"l1.mix.k", "l1.mix.v", "l3.mix.k", "l4.mix.v", "l1.norm2", "l1.mlp.router"} & names


@pytest.mark.parametrize("dims,base,scaling", [(12, 900.0, {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0}),
                                               (24, 10000.0, None), (4, 50.0, {"factor": 16.0, "original": 16, "fast": 4.0, "slow": 0.5}),
                                               (16, 1e5, {"factor": 2.0, "original": 4096, "fast": 32.0, "slow": 1.0})])
def test_rotation_table_against_the_plain_frequencies(dims, base, scaling):
    pos = YarnRotary(32, dims, base, scaling)
    pos.bind({}, Runtime(torch.device("cpu"), torch.float32, None, Workspace(torch.device("cpu"))))
    pos.prepare(300)
    freq, gain = plain.yarn_frequencies(dims, base, scaling)
    if scaling is not None:
        assert gain == pytest.approx(0.1 * math.log(scaling["factor"]) + 1.0)
        plain_f = base ** (-2.0 * np.arange(dims // 2) / dims)
        assert np.all(freq <= plain_f * (1 + 1e-12)) and np.all(freq >= plain_f / scaling["factor"] * (1 - 1e-12))
    ang = np.arange(300)[:, None] * freq[None, :]
    t = pos.table.numpy()
    np.testing.assert_allclose(t[:, : dims // 2, 0], np.cos(ang) * gain, atol=2e-7)
    np.testing.assert_allclose(t[:, : dims // 2, 1], np.sin(ang) * gain, atol=2e-7)
    assert np.all(t[:, dims // 2:, 0] == 1.0) and np.all(t[:, dims // 2:, 1] == 0.0)


@pytest.mark.parametrize("dim,vdim,dims", [(32, 48, 12), (24, 16, 24), (16, 16, 4), (64, 80, 16), (130, 8, 2), (20, 20, 0)])
def test_head_slots_put_partners_half_a_head_apart(dim, vdim, dims):
    slots = slot_size(dim, vdim)
    assert slots >= max(dim, vdim) and slots % 16 == 0
    index = head_slots(dim, dims, slots)
    assert sorted(set(index)) == sorted(index) and max(index) < slots
    for i in range(dims // 2):
        assert index[i] == i and index[i + dims // 2] == i + slots // 2
    for j in range(dims, dim):                              # what does not rotate meets identity entries
        assert index[j] % (slots // 2) >= dims // 2


def runner_for(folder, pages, dtype="float32"):
    return ModelRunner(folder, dtype=dtype, device="cpu", num_blocks=pages, max_seq_len=pages * 16, max_num_seqs=8,
                       use_graphs=False, ops=EmulatedOps())


LENGTHS = [70, 33, 97, 18, 64, 45, 52, 81, 29]


@pytest.mark.parametrize("name", list(RADIVIK))
def test_every_cutting_matches_the_plain_model_on_the_host(name, folders):
    rng = np.random.default_rng(4)
    reqs = [rng.integers(0, RADIVIK[name]["vocab"], n).tolist() for n in LENGTHS]
    model = plain.PlainRadivik(folders[name])
    truth = [model.logits(t) for t in reqs]
    runner = runner_for(folders[name], 32)
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        assert traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, 2e-5) < 2e-5
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=2)
    assert sum(len(r) for r in reqs) > 1.3 * peak
    small = runner_for(folders[name], peak // 16)
    for t in small.pools.tensors:
        t.fill_(1e30)                                       # a page that is used again never holds zeros
    rp = TraceReplayer(small)
    assert traces.compare(rp.run_step, steps, expect, truth, 2e-5) < 2e-5
    assert all(rp.cache.num_free(g) == peak // 16 for g in range(rp.cache.num_groups))


def test_layers_follow_the_plain_model_one_by_one(folders):
    """The stream behind every layer: a fault shows in the layer that makes it."""
    rng = np.random.default_rng(9)
    toks = rng.integers(0, 120, 21).tolist()
    want = plain.PlainRadivik(folders["P"]).hidden(toks, every_layer=True)
    runner = runner_for(folders["P"], 8)
    seen = []
    for blk in runner.model.blocks:
        inner = blk.forward

        def forward(residual, *a, _inner=inner, **kw):
            out = _inner(residual, *a, **kw)
            seen.append(residual.clone().numpy())
            return out

        blk.forward = forward
    runner.step([StepItem(key="a", tokens=toks, start=0, block_tables=[[0, 1]], slot=0, want=[20])])
    assert len(seen) == len(want)
    for i, (got, exp) in enumerate(zip(seen, want)):
        assert np.abs(got - exp).max() < 2e-5 * np.abs(exp).max(), f"layer {i}"


def test_greedy_generation_through_the_engine_and_scheduler(folders):
    """The package's entry point: prompts in portions of 16 under a budget, three requests at a
    time, so few pages that requests wait and pages come back; prefix cache on (no state here)."""
    from prefixserve_amd.engine.engine import Engine, EngineConfig
    from prefixserve_amd.generation import generate

    model = plain.PlainRadivik(folders["Q"])
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, 90, n).tolist() for n in (5, 23, 40, 9, 31)]
    prompts.append(prompts[2][:33] + [7, 8])                # shares two pages of prefix with another request
    eng = Engine(EngineConfig(model_path=str(folders["Q"]), dtype="float32", device="cpu", max_num_seqs=3,
                              max_prefill_tokens=16, max_seq_len=128, num_blocks=14, use_graphs=False), ops=EmulatedOps())
    outs, stats = generate(eng, prompts, 12, temperature=0.0, ignore_eos=True)
    for p, o in zip(prompts, outs):
        assert list(o.tokens) == model.greedy(p, 12)
    assert outs[5].cached_tokens >= 16


def test_a_second_norm_without_a_feed_forward_is_applied_if_the_checkpoint_brings_one(folders, tmp_path):
    """config.json does not say whether a layer without a feed-forward has a second norm: the
    checkpoint does. Without the tensor the layer ends behind its first norm; with it, the
    second norm is applied to alpha x alone."""
    import shutil

    from safetensors.torch import load_file, save_file

    folder = tmp_path / "m"
    shutil.copytree(folders["P"], folder)
    tensors = load_file(str(folder / "model.safetensors"))
    assert "l1.norm2" not in tensors
    tensors["l1.norm2"] = (1.0 + 0.2 * torch.randn(96, generator=torch.Generator().manual_seed(1))).to(torch.bfloat16)
    save_file(tensors, str(folder / "model.safetensors"))
    _, cfg, _ = read_model_dir(folder)
    assert cfg.layers[1].lone_second_norm and not cfg.layers[0].lone_second_norm
    assert not read_model_dir(folders["P"])[1].layers[1].lone_second_norm
    toks = np.random.default_rng(3).integers(0, 120, 30).tolist()
    model = plain.PlainRadivik(folder)
    pos, kept = np.arange(len(toks)), {}
    x = model.w["embed"][np.asarray(toks)]
    for i, layer in enumerate(model.cfg["layers"]):
        x = plain.rms_norm(model.alpha * x + model.mixer(i, x, pos, kept), model.w[f"l{i}.norm1"], model.eps)
        if layer["mlp"] is not None:
            x = plain.rms_norm(model.alpha * x + model.feed_forward(i, x), model.w[f"l{i}.norm2"], model.eps)
        elif i == 1:
            x = plain.rms_norm(model.alpha * x, model.w["l1.norm2"], model.eps)
    want = plain.rms_norm(x, model.w["final.norm"], model.eps) @ model.w["head"].T
    rp = TraceReplayer(runner_for(folder, 8))
    got = rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": toks, "want": list(range(30))}], "end": ["a"]})
    assert np.abs(got - want).max() < 2e-5 * np.abs(want).max()
    assert np.abs(got - model.logits(toks)).max() > 1e-3 * np.abs(want).max()      # and it is not a no-op
