"""Plain, slow Radivik: the oracle the engine's Radivik tests are compared with.

Whole sequences, no cache, no paging, no batching; numpy only; one function per
mechanism. It shares no code with the product package (its file reader is the plain
Llama oracle's, which is test code too).

The design, in this file's notation. A layer keeps its norm behind the sum,
    x <- N1(a x + mix(x)),   x <- N2(a x + ff(x))        (the second only with a feed-forward)
with N(y) = w * y / sqrt(mean(y^2) + eps) and a = ``postln_alpha``. The mixer is causal
grouped-query attention whose queries and keys are rotated over their first ``rot.dims``
dimensions (rotate-half pairing inside those, YaRN-scaled frequencies, cos and sin scaled
by 0.1 ln(factor) + 1), then brought to unit root mean square per head, with a score scale
from the configuration and a value size of its own; a layer with ``kv_from: j`` brings no
keys and values and reads layer j's. The feed-forward is a mixture of experts with sigmoid
router scores, the ``top`` largest taken as they are, each weight multiplying its expert's
input; an expert is down(g' * sigmoid(1.702 g') * (u' + 1)) with g' = min(g, limit),
u' = clamp(u, -limit, limit).
"""

from __future__ import annotations

import json
import math
from pathlib import Path
from typing import Any

import numpy as np

from .llama_plain import read_safetensors, round_bf16  # noqa: F401  (test-side helpers)

# ------------------------------------------------------------------- formulas


def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    return unit_rms(x, eps) * weight


def yarn_frequencies(dims: int, base: float, scaling: dict[str, Any] | None) -> tuple[np.ndarray, float]:
    """(f_i for i < dims/2, the factor on cos and sin). Plain f_i = base^(-2i/dims). With
    scaling (factor s, original length L, fast, slow): the dimension at which a wave makes t
    turns over L is dim(t) = dims ln(L / (2 pi t)) / (2 ln base); between lo = floor(dim(fast))
    and hi = ceil(dim(slow)) (kept inside [0, dims - 1]) the share r_i of the slowed frequency
    f_i / s rises from 0 to 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    s, orig = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s * ramp + f * (1.0 - ramp), 0.1 * math.log(s) + 1.0


def rotate(x: np.ndarray, positions: np.ndarray, freq: np.ndarray, gain: float) -> np.ndarray:
    """x [n, heads, dim]; dimension i < len(freq) pairs with i + len(freq); the rest pass."""
    half = len(freq)
    ang = positions.astype(np.float64)[:, None] * freq[None, :]
    cos, sin = (np.cos(ang) * gain)[:, None, :], (np.sin(ang) * gain)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half: 2 * half]
    out[..., :half] = u * cos - v * sin
    out[..., half: 2 * half] = v * cos + u * sin
    return out


def attention_weights(q: np.ndarray, k: np.ndarray, scale: float) -> np.ndarray:
    """softmax over the keys at or before each query; q [n, dim], k [n, dim] -> [n, n]."""
    n = q.shape[0]
    s = (q @ k.T) * scale
    pos = np.arange(n)
    s = np.where(pos[None, :] > pos[:, None], -np.inf, s)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def attend(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float) -> np.ndarray:
    """q [n, H, dim], k [n, G, dim], v [n, G, vdim] -> [n, H, vdim]; head h reads h // (H/G)."""
    n, heads, _ = q.shape
    rep = heads // k.shape[1]
    out = np.empty((n, heads, v.shape[-1]), dtype=q.dtype)
    for h in range(heads):
        out[:, h, :] = attention_weights(q[:, h, :], k[:, h // rep, :], scale) @ v[:, h // rep, :]
    return out


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-z))


def _same(x: np.ndarray) -> np.ndarray:
    return x


def expert(h: np.ndarray, gate: np.ndarray, up: np.ndarray, down: np.ndarray, limit: float, r: Any = _same) -> np.ndarray:
    """``r`` rounds what a 16-bit engine would keep in 16 bits (a product's output, an activation)."""
    g = np.minimum(r(h @ gate.T), limit)
    u = np.clip(r(h @ up.T), -limit, limit)
    return r(g * sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def route(h: np.ndarray, router: np.ndarray, top: int) -> tuple[np.ndarray, np.ndarray]:
    """(chosen experts [n, top], their scores [n, top]): the largest sigmoid scores, as they are."""
    s = sigmoid(h @ router.T)
    chosen = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return chosen, np.take_along_axis(s, chosen, axis=-1)


def mixture(h: np.ndarray, router: np.ndarray, experts: list[tuple[np.ndarray, np.ndarray, np.ndarray]], top: int,
            limit: float, r: Any = _same) -> np.ndarray:
    chosen, score = route(h, router, top)
    out = np.zeros((h.shape[0], experts[0][2].shape[0]), dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t], score[t]):
            out[t] += expert(r(w * h[t]), *experts[int(e)], limit, r)
    return out


# ---------------------------------------------------------------------- model


class PlainRadivik:
    def __init__(self, model_dir: str | Path, dtype: Any = np.float64, bf16: bool = False) -> None:
        """``bf16``: the yardstick for a 16-bit engine. The outputs of products and the activations
        between them are rounded to bfloat16; what the design computes in 32-bit (angles, unit
        norms, scores and softmax, router, the sum and the norm behind it) is float32."""
        model_dir = Path(model_dir)
        self.r = (lambda x: round_bf16(x).astype(np.float32)) if bf16 else _same
        dtype = np.float32 if bf16 else dtype
        self.cfg = json.loads((model_dir / "config.json").read_text())
        self.w = {k: (v.astype(dtype) if v.dtype.kind == "f" else v)
                  for k, v in read_safetensors(model_dir / "model.safetensors").items()}
        self.eps = float(self.cfg["norm"]["eps"])
        self.alpha = float(self.cfg["postln_alpha"])
        self.dtype = dtype

    def keys_values(self, i: int, x: np.ndarray, pos: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
        m = self.cfg["layers"][i]["mixer"]
        n, p = x.shape[0], f"l{i}.mix."
        freq, gain = yarn_frequencies(int(m["rot"]["dims"]), float(m["rot"]["base"]), m["rot"].get("scaling"))
        r = self.r
        k = r(x @ self.w[p + "k"].T).reshape(n, int(m["kv_heads"]), int(m["dim"]))
        v = r(x @ self.w[p + "v"].T).reshape(n, int(m["kv_heads"]), int(m["vdim"]))
        return r(unit_rms(rotate(k, pos, freq, gain), self.eps).astype(self.dtype)), v

    def mixer(self, i: int, x: np.ndarray, pos: np.ndarray, kept: dict[int, Any]) -> np.ndarray:
        m = self.cfg["layers"][i]["mixer"]
        n, p = x.shape[0], f"l{i}.mix."
        freq, gain = yarn_frequencies(int(m["rot"]["dims"]), float(m["rot"]["base"]), m["rot"].get("scaling"))
        r = self.r
        x = r(x)
        q = r(x @ self.w[p + "q"].T).reshape(n, int(m["heads"]), int(m["dim"]))
        q = r(unit_rms(rotate(q, pos, freq, gain), self.eps).astype(self.dtype))
        if m.get("kv_from") is not None:
            k, v = kept[int(m["kv_from"])]
        else:
            k, v = kept[i] = self.keys_values(i, x, pos)
        return r(r(attend(q, k, v, float(m["scale"])).reshape(n, -1)) @ self.w[p + "o"].T)

    def feed_forward(self, i: int, x: np.ndarray) -> np.ndarray:
        f = self.cfg["layers"][i]["mlp"]
        p = f"l{i}.mlp."
        experts = [(self.w[f"{p}e{e}.gate"], self.w[f"{p}e{e}.up"], self.w[f"{p}e{e}.down"])
                   for e in range(int(f["router"]["experts"]))]
        return mixture(self.r(x), self.w[p + "router"], experts, int(f["router"]["top"]), float(f["expert"]["limit"]), self.r)

    def hidden(self, tokens: Any, every_layer: bool = False) -> Any:
        ids = np.asarray(tokens, dtype=np.int64)
        pos = np.arange(len(ids))
        x = self.w["embed"][ids]
        kept: dict[int, Any] = {}
        trail = []
        for i, layer in enumerate(self.cfg["layers"]):
            assert layer["type"] == "attention"
            x = rms_norm(self.alpha * x + self.mixer(i, x, pos, kept), self.w[f"l{i}.norm1"], self.eps)
            if layer.get("mlp") is not None:
                x = rms_norm(self.alpha * x + self.feed_forward(i, x), self.w[f"l{i}.norm2"], self.eps)
            trail.append(x)
        return np.stack(trail) if every_layer else x

    def logits(self, tokens: Any) -> np.ndarray:
        return self.r(rms_norm(self.hidden(tokens), self.w["final.norm"], self.eps)) @ self.w["head"].T

    def greedy(self, prompt: Any, steps: int) -> list[int]:
        ids = [int(t) for t in prompt]
        for _ in range(steps):
            ids.append(int(np.argmax(self.logits(ids)[-1])))
        return ids[len(prompt):]
