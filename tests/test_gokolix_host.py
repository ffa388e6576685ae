"""Gokolix on the host: its configuration, the model built from it, and the whole engine path
(packing, pages, windows, state slots, the repeated stretch, replay, scheduler, generation) with
the kernel library's CPU stand-in, against the plain implementation in tests/plain/gokolix_plain.py."""

from __future__ import annotations

import copy
import json

import numpy as np
import pytest
import torch

import traces
from emulated_ops import EmulatedOps
from gokolix_configs import GOKOLIX, attention, latent, layer, model, recurrence, write_gokolix
from plain import gokolix_plain as plain
from prefixserve_amd.config import GokolixConfig, UnsupportedModelError, read_model_dir
from prefixserve_amd.engine.batch import StepItem
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner
from prefixserve_amd.models.gokolix import build_gokolix_spec
from prefixserve_amd.parts.attention import distance_table
from prefixserve_amd.parts.base import Runtime, Workspace
from prefixserve_amd.parts.rope import YarnRotary

TOL = 3e-5


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_gokolix(tmp_path_factory.mktemp(f"gokolix-{name}"), name) for name in GOKOLIX}


def runner_for(folder, pages, dtype="float32", slots=4):
    return ModelRunner(folder, dtype=dtype, device="cpu", num_blocks=pages, max_seq_len=pages * 16, max_num_seqs=slots,
                       use_graphs=False, ops=EmulatedOps())


def whole(runner, toks, want=None):
    want = list(range(len(toks))) if want is None else want
    rp = TraceReplayer(runner)
    return rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": list(toks), "want": want}], "end": ["a"]})


def close(got, want, tol=TOL):
    return float(np.abs(got - want).max()) <= tol * float(np.abs(want).max())


# ------------------------------------------------------------------ configuration and spec

def test_configuration_reads_every_key_and_refuses_what_it_does_not_know():
    cfg = GokolixConfig.from_dicts(GOKOLIX["A"])
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.embedding_scale) == (96, 64, 1e-5, 3.0)
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 3, 3)
    a, r, l = cfg.layers[3].mixer, cfg.layers[1].mixer, cfg.layers[2].mixer
    assert (a.heads, a.kv_heads, a.dim, a.scale, a.bias_max, a.window, a.buckets) == (6, 2, 8, 0.9, 9.0, 5, 6)
    assert (r.width, r.blocks, r.conv) == (48, 3, 3)
    assert (l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank, l.scale, l.rot_base, l.window) == (2, 24, 8, 16, 40, 0.3, 500.0, 24)
    assert l.rot_scaling.factor == 4.0 and l.rot_scaling.original == 32
    assert cfg.layers[2].ff is None and cfg.layers[0].ff == 80
    assert GokolixConfig.from_dicts(cfg.to_config_json()) == cfg
    assert GokolixConfig.from_dicts(GOKOLIX["B"]).loop is None and GokolixConfig.from_dicts(GOKOLIX["B"]).layers[2].mixer.window is None
    for path, value in [(("layers", 0, "mixer", "rot"), {}), (("layers", 0, "mlp", "kind"), "moe"), (("layers", 0, "type"), "conv"),
                        (("layers", 0, "mixer", "vdim"), 8), (("layers", 1, "mixer", "blocks"), 5), (("loop", "stop"), 9),
                        (("loop", "times"), 0), (("sink",), True), (("layers", 2, "mixer", "rot", "dims"), 6),
                        (("layers", 3, "mixer", "kv_heads"), 4), (("layers", 0, "mixer", "mask", "size"), 0)]:
        raw = copy.deepcopy(GOKOLIX["A"])
        at = raw
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(UnsupportedModelError):
            GokolixConfig.from_dicts(raw)


def test_the_bias_tables_rows_come_from_the_checkpoint(folders):
    raw = json.loads((folders["A"] / "config.json").read_text())
    assert all("buckets" not in entry["mixer"] for entry in raw["layers"])
    assert GokolixConfig.from_dicts(raw).layers[0].mixer.buckets is None
    with pytest.raises(UnsupportedModelError):
        build_gokolix_spec(GokolixConfig.from_dicts(raw))
    arch, cfg, _ = read_model_dir(folders["A"])
    assert arch.name == "Gokolix" and [l.mixer.buckets for l in cfg.layers if l.type == "attention"] == [12, 6]


def test_a_repeated_stretch_is_listed_once_per_pass_with_caches_of_its_own(folders):
    spec = build_gokolix_spec(read_model_dir(folders["A"])[1])
    assert [(r.layer, r.before, r.pass_index) for r in spec.order] == [
        (0, (), 0), (1, ("reentry",), 0), (2, (), 0), (1, ("reentry",), 1), (2, (), 1), (1, ("reentry",), 2), (2, (), 2), (3, (), 0)]
    assert sorted(r.cache for r in spec.order) == list(range(8)) and all(r.writes_cache for r in spec.order)
    runner = runner_for(folders["A"], 8)
    assert sorted(runner.model.state_needs()) == [1, 3, 5]            # the recurrence's three runs
    assert runner.model.state_needs()[1].shape == (3 * 48,)
    assert len(runner.layer_groups) == 3 and sorted(len(g.entries) for g in runner.layer_groups) == [1, 1, 3]
    assert sorted((w is None, w) for w in runner.windows) == [(False, 5), (False, 8), (False, 24)]
    spec_b = build_gokolix_spec(read_model_dir(folders["B"])[1])
    assert not spec_b.stream_transforms and all(not r.before for r in spec_b.order)
    spec_c = build_gokolix_spec(read_model_dir(folders["C"])[1])
    assert [r.before for r in spec_c.order] == [("reentry",), (), ()]  # one pass is still entered through the transform


# ------------------------------------------------------------------ mechanisms, one at a time

@pytest.mark.parametrize("buckets,far", [(12, 20), (6, 9), (16, 40), (4, 6), (32, 100), (2, 3.5), (9, 17.5)])
def test_distance_table_against_the_plain_buckets(buckets, far):
    rel = torch.randn(buckets, 3)
    table = distance_table(rel, far)
    for n in list(range(table.shape[1])) + [table.shape[1] + 5, 10 * table.shape[1]]:
        row = plain.distance_bucket(n, buckets, far)
        assert torch.equal(table[:, min(n, table.shape[1] - 1)], rel[row]), n
    half = buckets // 2
    assert [plain.distance_bucket(n, buckets, far) for n in range(half)] == list(range(half))
    assert plain.distance_bucket(int(np.ceil(far)), buckets, far) == buckets - 1


@pytest.mark.parametrize("dims,base,scaling", [(8, 500.0, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}),
                                               (4, 10000.0, None), (16, 50.0, {"factor": 16.0, "original": 16, "fast": 4.0, "slow": 0.5})])
def test_rotation_table_against_the_plain_frequencies(dims, base, scaling):
    rot = YarnRotary(dims, dims, base, scaling)
    rot.bind({}, Runtime(torch.device("cpu"), torch.float32, None, Workspace(torch.device("cpu"))))
    rot.prepare(200)
    freq, gain = plain.yarn_frequencies(dims, base, scaling)
    ang = np.arange(200)[:, None] * freq[None, :]
    assert np.abs(rot.table[:, :, 0].numpy() - np.cos(ang) * gain).max() < 1e-6
    assert np.abs(rot.table[:, :, 1].numpy() - np.sin(ang) * gain).max() < 1e-6


ONE_LAYER = {
    "attention": attention(6, 2, 8, 0.9, 9, 6, window=5),
    "attention-no-window": attention(2, 2, 20, 0.5, 30, 10),
    "latent": latent(3, 12, 6, 10, 20, 0.4, 300.0, {"factor": 8.0, "original": 24, "fast": 6.0, "slow": 1.0}, window=11),
    "latent-no-scaling": latent(2, 8, 8, 8, 8, 0.6, 10000.0),
    "recurrence": recurrence(24, 2, 4),
}


@pytest.mark.parametrize("kind", list(ONE_LAYER))
@pytest.mark.parametrize("ff", [None, 24])
def test_each_mixer_alone(kind, ff, tmp_path):
    """A model of one layer: whatever differs from the plain model is that mixer's (or the block's)."""
    folder = write_gokolix(tmp_path, model(50, 32, 1e-5, 2.0, [layer(ONE_LAYER[kind], ff)]), seed=8)
    toks = np.random.default_rng(1).integers(0, 50, 45).tolist()
    want = plain.PlainGokolix(folder).logits(toks)
    assert close(whole(runner_for(folder, 4), toks), want)


def test_the_plain_mixers_agree_with_their_step_by_step_definitions():
    """The oracle's own recurrence and window against the definitions written out token by token."""
    rng = np.random.default_rng(5)
    m = {"width": 6, "blocks": 2, "conv": 3}
    w = {"y": rng.normal(size=(6, 4)), "y.b": rng.normal(size=6), "x": rng.normal(size=(6, 4)), "x.b": rng.normal(size=6),
         "conv": rng.normal(size=(6, 3)), "conv.b": rng.normal(size=6), "ra": rng.normal(size=(2, 3, 3)), "ra.b": rng.normal(size=(2, 3)),
         "ri": rng.normal(size=(2, 3, 3)), "ri.b": rng.normal(size=(2, 3)), "lam": rng.normal(size=6), "o": rng.normal(size=(4, 6))}
    h = rng.normal(size=(7, 4))
    got = plain.gated_recurrence(h, w, m)
    xs = [np.zeros(6), np.zeros(6)]
    state = np.zeros(6)
    for t in range(7):
        xs.append(w["x"] @ h[t] + w["x.b"])
        u = w["conv.b"] + w["conv"][:, 0] * xs[-3] + w["conv"][:, 1] * xs[-2] + w["conv"][:, 2] * xs[-1]
        r = np.concatenate([plain.sigmoid(w["ra"][b] @ u[3 * b: 3 * b + 3] + w["ra.b"][b]) for b in range(2)])
        g = np.concatenate([plain.sigmoid(w["ri"][b] @ u[3 * b: 3 * b + 3] + w["ri.b"][b]) for b in range(2)])
        a = np.exp(-8.0 * r * np.log1p(np.exp(w["lam"])))
        state = a * state + np.sqrt(1 - a * a) * g * u
        y = plain.gelu_tanh(w["y"] @ h[t] + w["y.b"])
        assert np.allclose(got[t], w["o"] @ (state * y), rtol=1e-10, atol=1e-12)
    p = plain.windowed_weights(rng.normal(size=(1, 6, 6)), 3, np.array([0.5]))
    assert np.all(p[0, 5, :3] == 0) and np.all(p[0, 5, 3:] > 0) and np.all(p[0, 1, 2:] == 0)
    assert 0 < p[0, 5].sum() < 1 and 0 < p[0, 0].sum() < 1          # the sink takes its share, also of the first token


# ------------------------------------------------------------------ whole models

LENGTHS = [70, 33, 97, 18, 64, 45, 1, 52, 2, 81, 29, 3]


@pytest.mark.parametrize("name", list(GOKOLIX))
def test_every_cutting_matches_the_plain_model_on_the_host(name, folders):
    rng = np.random.default_rng(4)
    reqs = [rng.integers(0, GOKOLIX[name]["vocab"], n).tolist() for n in LENGTHS]
    pm = plain.PlainGokolix(folders[name])
    truth = [pm.logits(t) for t in reqs]
    runner = runner_for(folders[name], 32)
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        assert traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL) < TOL
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=2)
    assert sum(len(r) for r in reqs) > 1.3 * peak
    small = runner_for(folders[name], peak // 16, slots=3)
    for t in small.pools.tensors:
        t.fill_(1e30)                                       # a page that is used again never holds zeros
    for s in small.states.values():
        s.fill_(1e30)                                       # nor does a state slot
    rp = TraceReplayer(small)
    assert traces.compare(rp.run_step, steps, expect, truth, TOL) < TOL
    assert all(rp.cache.num_free(g) == peak // 16 for g in range(rp.cache.num_groups))


def test_layers_follow_the_plain_model_one_by_one(folders):
    """The stream behind every run of a layer: a fault shows in the run that makes it."""
    toks = np.random.default_rng(9).integers(0, 96, 37).tolist()
    want = plain.PlainGokolix(folders["A"]).hidden(toks, every_layer=True)
    runner = runner_for(folders["A"], 8)
    seen = []
    for blk in runner.model.blocks:
        inner = blk.forward

        def forward(residual, *a, _inner=inner, **kw):
            out = _inner(residual, *a, **kw)
            seen.append((residual + out.float() if out is not None else residual).clone().numpy())
            return out

        blk.forward = forward
    runner.step([StepItem(key="a", tokens=toks, start=0, block_tables=[[0, 1, 2]] * 3, slot=0, want=[36])])
    assert len(seen) == len(want) == 8
    for i, (got, exp) in enumerate(zip(seen, want)):
        assert close(got, exp), f"run {i}"


def peaky(tensors):
    """Weights under which single keys carry the softmax and the sink matters: a fault at a window's
    edge, in the bias table's rows or in the sink then moves the logits by far more than rounding."""
    for name, t in tensors.items():
        if name.endswith(".sink"):
            t.copy_(torch.full_like(t, 2.0))
        if name.endswith(".rel"):
            t.mul_(4.0)


def test_a_wrong_window_sink_bucket_or_state_would_show(tmp_path):
    cfg = model(60, 32, 1e-5, 2.0, [layer(attention(2, 1, 16, 3.0, 12, 8, window=10), 24),
                                    layer(latent(2, 8, 4, 8, 12, 3.0, 100.0, window=9), None),
                                    layer(recurrence(16, 2, 3), 24)])
    folder = write_gokolix(tmp_path, cfg, seed=2, edit=peaky)
    toks = np.random.default_rng(3).integers(0, 60, 60).tolist()
    pm = plain.PlainGokolix(folder)
    truth = pm.logits(toks)
    got = whole(runner_for(folder, 4), toks)
    assert close(got, truth)

    def wrong(change) -> float:
        other = plain.PlainGokolix(folder)
        change(other)
        return float(np.abs(other.logits(toks) - truth).max() / np.abs(truth).max())

    def set_window(i, size):
        return lambda m: m.cfg["layers"][i]["mixer"]["mask"].update(size=size)

    def drop(name):
        return lambda m: m.w.__setitem__(name, m.w[name] * 0 - 60.0)

    for change in (set_window(0, 9), set_window(0, 11), set_window(1, 8), set_window(1, 10), drop("l0.mix.sink"), drop("l1.mix.sink"),
                   lambda m: m.w.__setitem__("l0.mix.rel", np.roll(m.w["l0.mix.rel"], 1, axis=0)),
                   lambda m: m.cfg["layers"][0]["mixer"].update(bias_max=7),
                   lambda m: m.cfg["layers"][2]["mixer"].update(conv=2) or m.w.__setitem__("l2.mix.conv", m.w["l2.mix.conv"][:, 1:])):
        assert wrong(change) > 100 * TOL


def test_first_tokens_and_long_decoding(folders):
    """Sequences of one, two and three tokens, and 150 tokens decoded one by one past every window."""
    pm = plain.PlainGokolix(folders["A"])
    runner = runner_for(folders["A"], 16)
    rng = np.random.default_rng(6)
    for n in (1, 2, 3):
        toks = rng.integers(0, 96, n).tolist()
        assert close(whole(runner, toks), pm.logits(toks))
    toks = rng.integers(0, 96, 170).tolist()
    truth = pm.logits(toks)
    steps, expect = traces.decode_tail([toks], tail=150)
    assert traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], TOL) < TOL


def test_greedy_generation_through_the_engine_and_scheduler(folders):
    """The package's entry point: prompts in portions of 16 under a budget, three requests at a time,
    few pages, state slots taken and given back; no prefix cache (a recurrence keeps state)."""
    from prefixserve_amd.engine.engine import Engine, EngineConfig
    from prefixserve_amd.generation import generate

    pm = plain.PlainGokolix(folders["B"])
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, 130, n).tolist() for n in (5, 23, 40, 9, 31)]
    eng = Engine(EngineConfig(model_path=str(folders["B"]), dtype="float32", device="cpu", max_num_seqs=3,
                              max_prefill_tokens=16, max_seq_len=128, num_blocks=14, use_graphs=False), ops=EmulatedOps())
    outs, _stats = generate(eng, prompts, 12, temperature=0.0, ignore_eos=True)
    for p, o in zip(prompts, outs):
        assert list(o.tokens) == pm.greedy(p, 12)
    assert all(o.cached_tokens == 0 for o in outs)
