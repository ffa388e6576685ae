"""Radivik on the GPU: its kernels one by one against plain formulas, and the engine against the
plain implementation (tests/plain/radivik_plain.py) in every way of cutting the work, in 32-bit
and in bfloat16, with pages that are used again, long decoding through captured graphs, keys far
back under a sharp softmax, generation through the package's entry point and the replay program."""

from __future__ import annotations

import copy
import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import traces
from plain import radivik_plain as plain
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner
from radivik_configs import RADIVIK, write_radivik

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def ops():
    from prefixserve_amd.kernels.ops import HipOps
    from prefixserve_amd.parts.base import Workspace

    return HipOps(torch.device(DEV), Workspace(torch.device(DEV)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_radivik(tmp_path_factory.mktemp(f"radivik-{name}"), name) for name in RADIVIK}


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(DEV)


def rel(got, want):
    got, want = torch.as_tensor(got).double().cpu(), torch.as_tensor(want).double().cpu()
    return float((got - want).abs().max() / want.abs().max())


# ------------------------------------------------------------------ kernels

@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,form", [(96, "none"), (192, "plain"), (1000, "slices"), (4104, "slices"), (4104, "plain"),
                                         (998, "slices"), (999, "plain"), (8192, "slices"), (8200, "slices"), (2048, "five")])
def test_norm_behind_the_sum(ops, act, hidden, form):
    t, eps, alpha = 5, 1e-5, 1.75
    res = rnd(t, hidden, seed=1)
    w = (1 + 0.1 * rnd(hidden, seed=3)).to(torch.bfloat16)
    delta = {"none": None, "plain": rnd(t, hidden, dtype=act, seed=2), "slices": rnd(3, t, hidden, seed=2),
             "five": rnd(5, t, hidden, seed=2)}[form]
    x = alpha * res.double()
    if delta is not None:
        x = x + (delta.double().sum(0) if delta.dim() == 3 else delta.double())
    want = plain.rms_norm(x.cpu().numpy(), w.double().cpu().numpy(), eps)
    out = None if act == torch.float32 else torch.empty(t, hidden, dtype=act, device=DEV)
    r = res.clone()
    ops.scaled_add_rmsnorm(r, delta, alpha, w, eps, out)
    assert rel(r, want) < 3e-6                                         # the stream itself, in 32-bit
    if out is not None:
        assert torch.equal(out, r.to(act))                             # and its copy, rounded once


def test_to_activation(ops):
    x = rnd(7, 100, seed=4)
    out = torch.empty(7, 100, dtype=torch.bfloat16, device=DEV)
    ops.to_activation(x, out)
    assert torch.equal(out, x.to(torch.bfloat16))


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d,norm_dim", [(6, 2, 48, 32), (4, 4, 32, 24), (8, 1, 16, 16), (5, 0, 80, 64), (2, 1, 256, 200), (3, 1, 32, 0)])
def test_rope_norm_kv_append(ops, act, hq, hkv, d, norm_dim):
    """Rotation, unit norm over the head's own dimensions and the page writes, against the plain
    formulas; the slots beyond ``norm_dim`` hold zeros as the mixer's layout leaves them."""
    t, blocks, eps = 37, 5, 1e-5
    qkv = rnd(t, (hq + 2 * hkv) * d, dtype=act, seed=5)
    heads = qkv.view(t, hq + 2 * hkv, d)
    if norm_dim:
        heads[:, : hq + hkv, norm_dim // 2: d // 2] = 0                # unused slots of each half
        heads[:, : hq + hkv, d // 2 + (norm_dim - norm_dim // 2):] = 0
    before = heads.double().cpu().numpy()
    positions = torch.randint(0, 90, (t,), dtype=torch.int32, device=DEV)
    table = torch.stack([torch.cos(rnd(90, d // 2, seed=6)), torch.sin(rnd(90, d // 2, seed=6))], dim=-1).contiguous()
    slots = torch.randperm(blocks * 16)[:t].to(torch.int32).to(DEV)
    kv = torch.full((blocks, 2, max(hkv, 1), 16 * d), 7.0, dtype=act, device=DEV) if hkv else None
    ops.rope_norm_kv_append(qkv, hq, hkv, d, positions, table, kv, slots, norm_dim, eps)
    cs = table[positions.long()].double().cpu().numpy()
    cos, sin = cs[..., 0][:, None, :], cs[..., 1][:, None, :]
    x = before[:, : hq + hkv]
    rot = np.concatenate([x[..., : d // 2] * cos - x[..., d // 2:] * sin, x[..., d // 2:] * cos + x[..., : d // 2] * sin], -1)
    if norm_dim:
        rot = rot / np.sqrt((rot ** 2).sum(-1, keepdims=True) / norm_dim + eps)
    tol = 2e-6 if act == torch.float32 else 5e-3
    got = qkv.view(t, hq + 2 * hkv, d)
    assert rel(got[:, : hq + hkv], rot) < tol
    if hkv:
        assert torch.equal(got[:, hq + hkv:].cpu(), torch.as_tensor(before[:, hq + hkv:]).to(act))   # values untouched
        page, off = (slots // 16).long(), (slots % 16).long()
        keys = kv[:, 0].view(blocks, hkv, 16, d)[page, :, off]
        vals = kv[:, 1].view(blocks, hkv, d, 16)[page, :, :, off]
        assert torch.equal(keys, got[:, hq: hq + hkv]) and torch.equal(vals, got[:, hq + hkv:])
        written = torch.zeros(blocks * 16, dtype=torch.bool)
        written[slots.long().cpu()] = True
        untouched = kv[:, 0].view(blocks, hkv, 16, d).permute(0, 2, 1, 3).reshape(blocks * 16, -1)[~written.to(DEV)]
        assert bool((untouched == 7.0).all())                          # nobody else's slot is written


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t,k,e,top", [(1, 96, 5, 2), (9, 64, 4, 4), (70, 128, 9, 1), (3, 200, 130, 8), (333, 256, 40, 6), (17, 100, 7, 3)])
def test_router_picks_the_largest_scores(ops, act, t, k, e, top):
    x = rnd(t, k, dtype=act, seed=7)
    w = rnd(e, k, seed=8, scale=0.3).to(torch.bfloat16).float()       # a router as checkpoints store it
    if e >= 4:
        w[3] = w[1]                                                    # equal scores: the lower index wins
    chosen = torch.empty(t, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(t, top, device=DEV)
    ops.moe_route(x, w, chosen, weight, w.to(act))                     # more than 16 tokens: product kernel + choice
    want_e, want_s = plain.route(x.double().cpu().numpy(), w.double().cpu().numpy(), top)
    s = plain.sigmoid(x.double().cpu().numpy() @ w.double().cpu().numpy().T)
    got_e = chosen.cpu().numpy()
    for i in range(t):
        for j in range(top):
            # the same expert, or one whose score is equal to within the 32-bit sum's rounding
            assert got_e[i, j] == want_e[i, j] or abs(s[i, got_e[i, j]] - want_s[i, j]) < 1e-6, (i, j)
        assert len(set(got_e[i].tolist())) == top
        if e >= 4 and 1 in got_e[i] and 3 in got_e[i]:
            assert list(got_e[i]).index(1) < list(got_e[i]).index(3)
    np.testing.assert_allclose(weight.cpu().numpy(), np.take_along_axis(s, got_e.astype(np.int64), -1), atol=2e-6)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t,k,f,e,top,limit", [(1, 96, 40, 5, 2, 0.7), (9, 64, 56, 4, 3, 6.0), (70, 128, 24, 9, 1, 0.3), (4, 100, 33, 3, 3, 1.0),
                                                  (300, 128, 72, 6, 2, 0.5), (40, 200, 64, 16, 4, 0.8), (2, 64, 16, 3, 2, 0.5), (130, 384, 200, 5, 5, 0.6)])
def test_experts_weight_their_input_and_clamp(ops, act, t, k, f, e, top, limit):
    x = rnd(t, k, dtype=act, seed=9)
    gate_up = rnd(e, 2 * f, k, dtype=act, seed=10, scale=0.15)
    down = rnd(e, k, f, dtype=act, seed=11, scale=0.15)
    gen = torch.Generator().manual_seed(12)
    chosen = torch.stack([torch.randperm(e, generator=gen)[:top] for _ in range(t)]).to(torch.int32).to(DEV)
    weight = (0.4 + 0.6 * torch.rand(t, top, generator=gen)).to(DEV)
    act_buf = torch.empty(t * top, f, dtype=act, device=DEV)
    out = torch.full((top, t, k), 3.0, device=DEV)
    ops.moe_experts(x, chosen, weight, gate_up, down, act_buf, out, 1.702, limit, 1.0)
    xs, gu, dn = x.double().cpu().numpy(), gate_up.double().cpu().numpy(), down.double().cpu().numpy()
    want = np.zeros((top, t, k))
    clamped = 0
    for i in range(t):
        for j in range(top):
            ex = int(chosen[i, j])
            h = float(weight[i, j]) * xs[i]
            want[j, i] = plain.expert(h, gu[ex, :f], gu[ex, f:], dn[ex], limit)
            clamped += int((np.abs(gu[ex, f:] @ h) > limit).sum() + ((gu[ex, :f] @ h) > limit).sum())
    assert clamped > 0 or limit > 5 or t < 4                           # the clamps are at work in this test
    assert rel(out, want) < (1e-5 if act == torch.float32 else 2e-2)


def test_kernels_refuse_what_they_do_not_take(ops):
    from prefixserve_amd.kernels.ops import KernelError

    x = rnd(2, 64)
    with pytest.raises(KernelError):
        ops.moe_route(x, rnd(4, 64).to(torch.bfloat16), torch.empty(2, 1, dtype=torch.int32, device=DEV), torch.empty(2, 1, device=DEV))
    with pytest.raises(KernelError):
        ops.moe_route(x, rnd(4, 64), torch.empty(2, 5, dtype=torch.int32, device=DEV), torch.empty(2, 5, device=DEV))
    with pytest.raises(KernelError):
        ops.rope_norm_kv_append(rnd(2, 4 * 32), 2, 1, 32, torch.zeros(2, dtype=torch.int32, device=DEV), None, None, None, 40, 1e-5)
    with pytest.raises(KernelError):
        ops.scaled_add_rmsnorm(rnd(2, 64), rnd(2, 32), 1.0, rnd(64), 1e-5, None)


# ------------------------------------------------------------------- engine

LENGTHS = [70, 33, 120, 97, 64, 18, 130, 45, 101, 77]


def runner_for(folder, dtype, pages, graphs=True, max_seq_len=None):
    return ModelRunner(folder, dtype=dtype, device=DEV, num_blocks=pages, max_seq_len=max_seq_len or min(pages * 16, 512),
                       max_num_seqs=8, use_graphs=graphs)


def bf16_bars(folder, truth, reqs):
    rough = plain.PlainRadivik(folder, bf16=True)
    rows = np.concatenate([np.abs(rough.logits(t) - w).max(-1) / np.abs(w).max(-1) for t, w in zip(reqs, truth)])
    return float(rows.mean()), float(rows.max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(RADIVIK))
def test_every_cutting_matches_the_plain_model(name, dtype, folders):
    rng = np.random.default_rng(1)
    reqs = [rng.integers(0, RADIVIK[name]["vocab"], n).tolist() for n in LENGTHS]
    model = plain.PlainRadivik(folders[name])
    truth = [model.logits(t) for t in reqs]
    mean_bar, row_bar = (0.0, 2e-5) if dtype == "float32" else bf16_bars(folders[name], truth, reqs)
    tol = 2e-5 if dtype == "float32" else 2.0 * row_bar
    runner = runner_for(folders[name], dtype, 64)
    errors, worst = [], {}
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        worst[build.__name__] = traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, tol, errors)
    steps, expect, peak = traces.mixed(reqs, seed=3)
    assert sum(len(r) for r in reqs) > 1.5 * peak
    small = runner_for(folders[name], dtype, peak // 16)
    for t in small.pools.tensors:
        t.fill_(1e30)                                                  # a page that is used again never holds zeros
    rp = TraceReplayer(small)
    worst["mixed"] = traces.compare(rp.run_step, steps, expect, truth, tol, errors)
    assert all(rp.cache.num_free(g) == peak // 16 for g in range(rp.cache.num_groups))
    print(name, dtype, {k: f"{v:.2e}" for k, v in worst.items()}, f"mean {np.mean(errors):.2e} (plain bf16 {mean_bar:.2e}, row {row_bar:.2e})")
    if dtype == "bfloat16":
        assert np.mean(errors) <= 1.25 * mean_bar


def test_cuttings_agree_with_each_other_in_32_bit(folders):
    """A position's logits do not depend on how its prompt was cut or on the batch, beyond rounding."""
    rng = np.random.default_rng(5)
    reqs = [rng.integers(0, 120, n).tolist() for n in (150, 99)]
    runner = runner_for(folders["P"], "float32", 64)
    rows = {}
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        rp, got = TraceReplayer(runner), {}
        for st, ex in zip(steps, expect):
            out = rp.run_step(st)
            got.update(zip(ex, out if out is not None else []))
        rows[build.__name__] = got
    n = 0
    for key, ref in rows["whole"].items():
        for other in ("decode_tail", "portions"):
            if key in rows[other]:
                assert rel(rows[other][key], ref) < 5e-6, (other, key)
                n += 1
    assert n > 250


SHARP = copy.deepcopy(RADIVIK["P"])
for _layer in SHARP["layers"]:
    _layer["mixer"]["scale"] = 1.6           # q.k of unit-norm heads reaches +-32: one key takes nearly all the weight


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_keys_under_a_sharp_softmax_and_long_decoding(dtype, tmp_path):
    """With a score scale this large a query's weight sits on one or two keys, wherever they are:
    hundreds of tokens back, in another page, just across a page border. A key that is lost,
    read from the wrong page or rotated by the wrong position changes the logits outright. The
    prompt is cut at and beside page borders; 150 tokens are then decoded one by one through
    captured graphs, beside a second request that starts later."""
    folder = write_radivik(tmp_path, "P", seed=8, config=SHARP)
    rng = np.random.default_rng(21)
    a, b = rng.integers(0, 120, 560).tolist(), rng.integers(0, 120, 230).tolist()
    model = plain.PlainRadivik(folder)
    truth = [model.logits(a), model.logits(b)]
    # Layer 0, head 0 from the plain formulas: how many of the last queries put most of their weight
    # on a key more than 200 tokens back.
    pos, q_pos = np.arange(len(a)), np.arange(400, 560)
    x = model.w["embed"][np.asarray(a)]
    m = SHARP["layers"][0]["mixer"]
    freq, gain = plain.yarn_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"]["scaling"])
    k, _ = model.keys_values(0, x, pos)
    q = plain.unit_rms(plain.rotate((x @ model.w["l0.mix.q"].T).reshape(len(a), 6, 32), pos, freq, gain), 1e-5)
    w = plain.attention_weights(q[:, 0], k[:, 0], 1.6)
    far = int(((w[q_pos].argmax(-1) < q_pos - 200) & (w[q_pos].max(-1) > 0.5)).sum())
    assert far >= 10                                                   # the test does look far back
    # scores near 50 carry their 32-bit rounding into the exponent: the 32-bit bar is the package's 1e-4 here
    tol = 1e-4 if dtype == "float32" else 2.0 * bf16_bars(folder, truth, [a, b])[1]
    runner = runner_for(folder, dtype, 52, max_seq_len=576)
    rp = TraceReplayer(runner)
    steps, expect, p = [], [], 0
    for c in (15, 2, 31, 16, 17, 95, 48, 2, 64, 120):                  # 410 tokens, cut at, before and behind page borders
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": a[p:p + c], "want": list(range(c))}], "end": []})
        expect.append([(0, q) for q in range(p, p + c)])
        p += c
    pb = 0
    for k in range(150):
        entries = [{"id": "a", "tokens": [a[p]], "want": [0]}]
        exp = [(0, p)]
        p += 1
        if k >= 20:
            c = 40 if k == 20 else 1
            entries.append({"id": "b", "tokens": b[pb:pb + c], "want": [c - 1]})
            exp.append((1, pb + c - 1))
            pb += c
        steps.append({"step": len(steps), "entries": entries, "end": []})
        expect.append(exp)
    worst = traces.compare(rp.run_step, steps, expect, truth, tol)
    if dtype == "bfloat16":
        assert any(k[0] in (1, 2) for k in runner._graphs)             # the decode steps ran as captured graphs
    print(dtype, f"worst {worst:.2e} (bar {tol:.2e}), {far} queries of head 0 look more than 200 tokens back")


def test_graph_replay_equals_eager_decoding(folders):
    rng = np.random.default_rng(9)
    reqs = [rng.integers(0, 200, n).tolist() for n in (90, 61, 40)]

    def decode(graphs):
        runner = runner_for(folders["R"], "bfloat16", 32, graphs=graphs, max_seq_len=256)
        rp, rows = TraceReplayer(runner), []
        for i, t in enumerate(reqs):
            rp.run_step({"step": 0, "entries": [{"id": f"r{i}", "tokens": t[:20], "want": []}], "end": []})
        for k in range(20):
            entries = [{"id": f"r{i}", "tokens": [reqs[i][20 + k]], "want": [0]} for i in range(3)]
            rows.append(rp.run_step({"step": k, "entries": entries, "end": []}))
            if k % 7 == 3:                                             # eager work between replays
                rp.run_step({"step": 100 + k, "entries": [{"id": "x", "tokens": list(range(5, 40)), "want": [34]}], "end": ["x"]})
        assert bool(runner._graphs) == graphs
        return np.stack(rows)

    eager, replayed = decode(False), decode(True)
    assert rel(replayed, eager) < 2e-2 and np.isfinite(replayed).all()
    model = plain.PlainRadivik(folders["R"])
    for i, t in enumerate(reqs):
        want = model.logits(t[:40])[20:40]
        assert rel(replayed[:, i], want) < 6e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(dtype, folders):
    from prefixserve_amd.engine.engine import Engine, EngineConfig
    from prefixserve_amd.generation import generate

    model = plain.PlainRadivik(folders["Q"])
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, 90, n).tolist() for n in (5, 23, 40, 9, 31, 64)]
    prompts.append(prompts[2][:33] + [7, 8])
    eng = Engine(EngineConfig(model_path=str(folders["Q"]), dtype=dtype, device=DEV, max_num_seqs=3,
                              max_prefill_tokens=16, max_seq_len=128, num_blocks=16))
    outs, _ = generate(eng, prompts, 14, temperature=0.0, ignore_eos=True, decode_steps=1 if dtype == "float32" else 4)
    agree = 0
    for p, o in zip(prompts, outs):
        assert len(o.tokens) == 14
        if dtype == "float32":
            assert list(o.tokens) == model.greedy(p, 14)
        else:
            # teacher-forced: given the engine's own tokens, the plain model's choice at every place
            # is the engine's, or its logit for the engine's token is within rounding of the best
            rows = model.logits(list(p) + list(o.tokens))[len(p) - 1:-1]
            for row, tok in zip(rows, o.tokens):
                assert row.max() - row[tok] < 0.15 * np.abs(row).max()
                agree += int(row.argmax() == tok)
    assert dtype == "float32" or agree > 0.85 * 14 * len(prompts)


def test_the_replay_program_on_a_radivik_folder(folders, tmp_path):
    rng = np.random.default_rng(15)
    reqs = [rng.integers(0, 120, n).tolist() for n in (40, 23)]
    model = plain.PlainRadivik(folders["P"])
    truth = [model.logits(t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, seed=4)
    env = dict(os.environ, HOME=str(tmp_path))
    # in bfloat16 a row may be as far off as twice the worst row of a plain bfloat16 run (an expert's
    # score that nearly ties with the next one's can fall the other way)
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 2.0 * bf16_bars(folders["P"], truth, reqs)[1])):
        out = tmp_path / f"out-{dtype}"
        proc = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(folders["P"]), "--dtype", dtype, "--out", str(out),
                               "--max-tokens", str(peak)], input="".join(json.dumps(s) + "\n" for s in steps), text=True,
                              capture_output=True, env=env, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        for s, exp in zip(steps, expect):
            if not exp:
                continue
            got = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(exp), -1)
            for row, (i, p) in zip(got, exp):
                assert rel(row, truth[i][p]) < tol, (dtype, s["step"], i, p)


def _random_radivik(rng) -> dict:
    """A configuration drawn at random: sizes that are no multiples of 8 or 16, head sizes in either
    order, rotations from none of the head to all of it, layers that read earlier layers, layers
    without a feed-forward, one to all experts per token."""
    width = int(rng.choice([40, 72, 100, 136, 192]))
    mixers = []
    for _ in range(int(rng.integers(1, 3))):
        kv_heads = int(rng.choice([1, 2, 3]))
        dim = int(rng.choice([8, 20, 32, 48, 72]))
        dims = int(rng.choice([0, 2, dim // 2 // 2 * 2, dim // 2 * 2]))
        scaling = None if rng.random() < 0.3 else {"factor": float(rng.choice([1.0, 2.0, 8.0, 40.0])), "original": int(rng.choice([16, 64, 512])),
                                                    "fast": float(rng.choice([4.0, 32.0])), "slow": float(rng.choice([0.25, 1.0, 2.0]))}
        rot = {"base": float(rng.choice([10.0, 10000.0, 1e6])), "dims": dims}
        if scaling is not None:
            rot["scaling"] = scaling
        mixers.append({"heads": kv_heads * int(rng.choice([1, 2, 4])), "kv_heads": kv_heads, "dim": dim,
                       "vdim": int(rng.choice([8, 12, 32, 40, 80])), "scale": float(rng.choice([0.1, 0.3, 0.7])), "rot": rot})
    layers, owners = [], {}
    for i in range(int(rng.integers(2, 6))):
        which = int(rng.integers(0, len(mixers)))
        m = dict(mixers[which])
        if which in owners and rng.random() < 0.5:
            m["kv_from"] = int(rng.choice(owners[which]))
        else:
            owners.setdefault(which, []).append(i)
        experts = int(rng.integers(1, 13))
        mlp = None if rng.random() < 0.2 else {"kind": "moe", "router": {"experts": experts, "top": int(rng.integers(1, min(experts, 4) + 1))},
                                               "expert": {"ff": int(rng.choice([8, 20, 36, 64])), "limit": float(rng.choice([0.3, 1.0, 4.0]))}}
        layers.append({"type": "attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Radivik", "vocab": int(rng.choice([50, 131, 300])), "width": width,
            "norm": {"eps": float(rng.choice([1e-6, 1e-5, 1e-3]))}, "postln_alpha": float(rng.choice([0.5, 1.0, 2.0, 4.0])), "layers": layers}


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_in_both_dtypes(seed, tmp_path):
    rng = np.random.default_rng(4000 + seed)
    cfg = _random_radivik(rng)
    folder = write_radivik(tmp_path, "", seed=seed, config=cfg)
    model = plain.PlainRadivik(folder)
    reqs = [rng.integers(0, cfg["vocab"], n).tolist() for n in (75, 40, 97, 18, 66)]
    truth = [model.logits(t) for t in reqs]
    mean_bar, row_bar = bf16_bars(folder, truth, reqs)
    for dtype in ("float32", "bfloat16"):
        tol = 2e-5 if dtype == "float32" else max(2.0 * row_bar, 0.05)
        runner = runner_for(folder, dtype, 32)
        errors = []
        for build in (traces.decode_tail, traces.portions):
            steps, expect = build(reqs)
            traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, tol, errors)
        steps, expect, peak = traces.mixed(reqs, seed=seed)
        small = runner_for(folder, dtype, peak // 16)
        for t in small.pools.tensors:
            t.fill_(1e30)
        traces.compare(TraceReplayer(small).run_step, steps, expect, truth, tol, errors)
        shape = [(l["mixer"]["heads"], l["mixer"]["kv_heads"], l["mixer"]["dim"], l["mixer"]["vdim"], l["mixer"]["rot"]["dims"],
                  l["mixer"].get("kv_from"), None if l["mlp"] is None else (l["mlp"]["router"]["experts"], l["mlp"]["router"]["top"],
                                                                         l["mlp"]["expert"]["ff"])) for l in cfg["layers"]]
        print(seed, dtype, cfg["width"], shape, f"worst {max(errors):.2e} mean {np.mean(errors):.2e} (plain bf16 {mean_bar:.2e}, row {row_bar:.2e})")
        if dtype == "bfloat16":
            assert np.mean(errors) <= 1.5 * mean_bar + 2e-3           # an expert score that nearly ties may fall the other way


def test_the_command_line_on_a_radivik_folder(tmp_path):
    """``random-model`` writes a Radivik folder from its config.json, ``generate`` runs it: the same
    commands as for any other architecture, chosen by the file."""
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(RADIVIK["R"]))
    proc = subprocess.run([sys.executable, "-m", "prefixserve_amd.cli", "random-model", "--config", str(cfg),
                           "--out", str(tmp_path / "m"), "--seed", "9"], capture_output=True, text=True, cwd=ROOT)
    assert proc.returncode == 0 and (tmp_path / "m" / "model.safetensors").exists(), proc.stderr
    # the default spread of 0.02 leaves near-ties; the comparison is on a folder with the tests' spread
    folder = write_radivik(tmp_path / "w", "R", seed=9)
    prompt = [5, 17, 3, 190, 41, 7, 7, 19, 0, 64, 11]
    want = plain.PlainRadivik(folder).greedy(prompt, 6)
    for model in (tmp_path / "m", folder):
        proc = subprocess.run(
            [sys.executable, "-m", "prefixserve_amd.cli", "generate", "--model", str(model), "--dtype", "float32",
             "--max-seq-len", "128", "--num-blocks", "16", "--max-running-requests", "2", "--chunked-prefill-size", "5",
             "--max-tokens", "6", "--ignore-eos", "--prompt-ids", ",".join(map(str, prompt))],
            capture_output=True, text=True, cwd=ROOT, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        out = json.loads(proc.stdout.strip().splitlines()[-1])
        assert len(out["outputs"][0]["tokens"]) == 6 and out["outputs"][0]["finish_reason"] == "length"
    assert out["outputs"][0]["tokens"] == want


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (4, 4, 128), (6, 2, 80)])
def test_softmax_weights_enter_the_second_product_unrounded(ops, hq, hkv, d):
    """With the same value row under every key, what a run of keys hands to the merge is that row
    times the sum of the weights as the product saw them, beside the sum of the weights in 32-bit: in
    float32, before any output is rounded. Their ratio is 1 to float32 rounding with ``exact_weights``
    and off by the bfloat16 step over the root of the number of keys without. (Two long contexts, so
    that the decode kernel cuts the keys into runs and writes partial results.)"""
    from prefixserve_amd.engine.batch import GroupMeta, StepItem, StepPacker

    blocks, old = 400, [3000, 2500]
    gen = torch.Generator().manual_seed(hq + d)
    vec = (torch.randn(hkv, d, generator=gen) + 3.0).to(torch.bfloat16).to(DEV)
    pk = StepPacker(torch.device(DEV), [GroupMeta(blocks, None)], 10, 100000, 8, ops.PREFILL_TILE_Q, skew_rule=ops.decode_is_skewed)
    kv = torch.zeros((blocks, 2, hkv, 16 * d), dtype=torch.bfloat16, device=DEV)
    perm = torch.randperm(blocks, generator=gen).tolist()
    items = []
    for i, o in enumerate(old):
        table = [perm.pop() for _ in range(-(-(o + 1) // 16))]
        pos = torch.arange(o + 1)
        pg = torch.tensor(table)[pos // 16].to(DEV)
        kv[:, 0].view(blocks, hkv, 16, d)[pg, :, (pos % 16).to(DEV), :] = rnd(o + 1, hkv, d, dtype=torch.bfloat16, seed=50 + i, scale=0.5)
        kv[:, 1].view(blocks, hkv, d, 16)[pg, :, :, (pos % 16).to(DEV)] = vec
        items.append(StepItem(i, [1], o, [table], slot=i))
    ctx = pk.pack(items)
    qkv = rnd(2, (hq + 2 * hkv) * d, dtype=torch.bfloat16, seed=77)
    want = vec.float().repeat_interleave(hq // hkv, 0)                                 # [hq, d]
    off = {}
    for exact in (False, True):
        out = torch.empty(2, hq * d, dtype=torch.bfloat16, device=DEV)
        ops.paged_attention(qkv, out, kv, ctx, 0, hq, hkv, d, 1.0 / d ** 0.5, None, exact_weights=exact)
        assert rel(out.view(2, hq, d), want[None].expand(2, hq, d)) < 4e-3         # the softmax weights sum to 1
        nsplit, _ = ops.decode_plan(2, ctx.max_kv_len, ctx.decode_skewed, hkv, 0)
        assert nsplit >= 2
        rows = 2 * hq * nsplit                                                      # (request, head, run)
        part_o = ops.ws._bufs["attn.part_o"][: rows * d].view(2, hq, nsplit, d)
        total = ops.ws._bufs["attn.part_ml"][: rows * 2].view(2, hq, nsplit, 2)[..., 1]
        used = total > 0.5                                                          # runs that held keys in this step
        assert int(used.sum()) >= 4 * hq
        ratio = (part_o / want[None, :, None, :]).mean(-1) / total.clamp_min(1e-30)
        off[exact] = float((ratio[used] - 1.0).abs().max())
    print(hq, hkv, d, off)
    assert off[True] < 3e-6 and off[False] > 10 * off[True]
