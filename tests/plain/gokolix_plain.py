"""A plain, slow Gokolix in numpy (float64), whole sequences at a time, one function per
mechanism. It shares no code with the package: it is what the engine is compared with.

Gokolix is a decoder whose layers are parallel blocks, x <- x + mixer(n(x)) + ff(n(x)) with one
norm n per layer whose weight is stored as its distance from one. A layer's mixer is one of:
grouped-query attention without rotation whose values are its un-normed keys, with biases,
a weighted norm per head, a learned bias per bucket of the distance, a sliding window and a
learned sink in the softmax; latent attention (keys and values made from one compressed
vector per token plus one rotated key part shared by the heads); a gated linear recurrence
behind a short convolution. A run of layers may be passed through several times with the same
weights; in front of every pass the stream is mixed with the token table's output again.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np


def load_tensors(folder: Path) -> dict[str, np.ndarray]:
    """Every tensor of model.safetensors as float64 (integer tables stay integers), read from the
    file's own layout: 8 bytes of header length, a JSON header, then the data."""
    raw = (Path(folder) / "model.safetensors").read_bytes()
    n = int.from_bytes(raw[:8], "little")
    head = json.loads(raw[8:8 + n])
    out = {}
    for name, meta in head.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        buf = raw[8 + n + a: 8 + n + b]
        if meta["dtype"] == "BF16":
            bits = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            arr = bits.view(np.float32).astype(np.float64)
        elif meta["dtype"] == "F32":
            arr = np.frombuffer(buf, dtype="<f4").astype(np.float64)
        elif meta["dtype"] == "I32":
            arr = np.frombuffer(buf, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {meta['dtype']}")
        out[name] = arr.reshape(meta["shape"])
    return out


# ------------------------------------------------------------------ small pieces

def rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def offset_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """The layers' norm: the weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def weighted_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return rms(x, eps) * w


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z: np.ndarray) -> np.ndarray:
    return np.logaddexp(0.0, z)


def distance_bucket(n: int, buckets: int, far: float) -> int:
    """The row of the bias table for a key n tokens back: one row per distance in the first half
    of the table, then rows whose reach grows geometrically up to ``far``; beyond, the last row."""
    half = buckets // 2
    if n < half:
        return n
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (buckets - half))))


def yarn_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[np.ndarray, float]:
    """(frequency of every pair, the factor on cosine and sine)."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    s, length = float(scaling["factor"]), float(scaling["original"])

    def place(turns: float) -> float:
        return dims * math.log(length / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(place(float(scaling["fast"]))), 0)
    hi = min(math.ceil(place(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s * ramp + f * (1.0 - ramp), 0.1 * math.log(s) + 1.0


def rotate_pairs(x: np.ndarray, pos: np.ndarray, freq: np.ndarray, gain: float) -> np.ndarray:
    """x [T, ..., dims]: neighbours (2i, 2i + 1) turned by pos x freq[i]; cosine and sine times gain."""
    shape = (len(pos),) + (1,) * (x.ndim - 2) + (len(freq),)
    ang = (pos[:, None].astype(np.float64) * freq[None, :]).reshape(shape)
    c, s = np.cos(ang) * gain, np.sin(ang) * gain
    u, v = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


def windowed_weights(scores: np.ndarray, window: int | None, sink: np.ndarray | None) -> np.ndarray:
    """scores [H, T, T] -> softmax weights over the keys a query sees (itself and the window - 1
    tokens before it); ``sink`` [H] adds exp(sink) to every denominator and nothing else."""
    h, t, _ = scores.shape
    i, j = np.arange(t)[:, None], np.arange(t)[None, :]
    seen = j <= i
    if window is not None:
        seen &= (i - j) < window
    s = np.where(seen[None], scores, -np.inf)
    m = s.max(-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink[:, None, None])
    e = np.exp(s - m)
    den = e.sum(-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink[:, None, None] - m)
    return e / den


# ------------------------------------------------------------------ mixers, whole sequences

def biased_attention(h: np.ndarray, w: dict, m: dict, eps: float) -> np.ndarray:
    t = h.shape[0]
    heads, kvh, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w["q"].T + w["q.b"]).reshape(t, heads, d)
    k = (h @ w["k"].T + w["k.b"]).reshape(t, kvh, d)
    v = k                                                # the values are the keys as projected
    q = weighted_norm(q, w["q.norm"], eps)
    k = weighted_norm(k, w["k.norm"], eps)
    rep = heads // kvh
    buckets = w["rel"].shape[0]
    by_distance = np.array([distance_bucket(n, buckets, m["bias_max"]) for n in range(t)])
    rows = by_distance[np.clip(np.arange(t)[:, None] - np.arange(t)[None, :], 0, None)]     # [query, key]; keys ahead are masked
    scores = np.empty((heads, t, t))
    for a in range(heads):
        scores[a] = q[:, a] @ k[:, a // rep].T * m["scale"] + w["rel"][rows, a]
    p = windowed_weights(scores, (m.get("mask") or {}).get("size"), w.get("sink"))
    out = np.stack([p[a] @ v[:, a // rep] for a in range(heads)], axis=1)        # [T, H, vdim]
    return out.reshape(t, -1) @ w["o"].T


def latent_attention(h: np.ndarray, pos: np.ndarray, w: dict, m: dict, eps: float) -> np.ndarray:
    t = h.shape[0]
    heads, d, r, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["q"].T).reshape(t, heads, d + r)
    down = h @ w["dkv"].T
    c = weighted_norm(down[:, :rank], w["dkv.norm"], eps)
    freq, gain = yarn_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    shared = rotate_pairs(down[:, rank:], pos, freq, gain)                       # [T, r]
    q_turn = rotate_pairs(q[..., d:], pos, freq, gain)                           # [T, H, r]
    k_flat = (c @ w["uk"].T).reshape(t, heads, d)
    v = (c @ w["uv"].T).reshape(t, heads, vd)
    scores = np.empty((heads, t, t))
    for a in range(heads):
        scores[a] = (q[:, a, :d] @ k_flat[:, a].T + q_turn[:, a] @ shared.T) * m["scale"]
    p = windowed_weights(scores, (m.get("mask") or {}).get("size"), w.get("sink"))
    out = np.stack([p[a] @ v[:, a] for a in range(heads)], axis=1)
    return out.reshape(t, -1) @ w["o"].T


def gated_recurrence(h: np.ndarray, w: dict, m: dict) -> np.ndarray:
    t = h.shape[0]
    width, blocks, taps = m["width"], m["blocks"], m["conv"]
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    x = h @ w["x"].T + w["x.b"]
    padded = np.concatenate([np.zeros((taps - 1, width)), x], axis=0)
    u = w["conv.b"] + sum(padded[j: j + t] * w["conv"][:, j] for j in range(taps))   # the last column is the current token's
    ub = u.reshape(t, blocks, width // blocks)
    r = sigmoid(np.einsum("tbi,boi->tbo", ub, w["ra"]) + w["ra.b"]).reshape(t, width)
    g = sigmoid(np.einsum("tbi,boi->tbo", ub, w["ri"]) + w["ri.b"]).reshape(t, width)
    a = np.exp(-8.0 * r * softplus(w["lam"]))
    inflow = np.sqrt(1.0 - a * a) * g * u
    state = np.zeros(width)
    out = np.empty((t, width))
    for s in range(t):
        state = a[s] * state + inflow[s]
        out[s] = state
    return (out * y) @ w["o"].T


def gated_feed_forward(h: np.ndarray, w: dict) -> np.ndarray:
    return (np.maximum(h @ w["gate"].T, 0.0) * (h @ w["up"].T)) @ w["down"].T


# ------------------------------------------------------------------ the model

class PlainGokolix:
    def __init__(self, folder: str | Path) -> None:
        folder = Path(folder)
        self.cfg = json.loads((folder / "config.json").read_text())
        self.w = load_tensors(folder)
        self.eps = float(self.cfg["norm"]["eps"])

    def part(self, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def layer(self, i: int, x: np.ndarray, pos: np.ndarray) -> np.ndarray:
        entry = self.cfg["layers"][i]
        h = offset_norm(x, self.w[f"l{i}.norm1"], self.eps)
        w, m = self.part(f"l{i}.mix."), entry["mixer"]
        if entry["type"] == "attention":
            mixed = biased_attention(h, w, m, self.eps)
        elif entry["type"] == "latent_attention":
            mixed = latent_attention(h, pos, w, m, self.eps)
        elif entry["type"] == "rglru":
            mixed = gated_recurrence(h, w, m)
        else:
            raise ValueError(entry["type"])
        if entry.get("mlp") is not None:
            mixed = mixed + gated_feed_forward(h, self.part(f"l{i}.mlp."))
        return x + mixed

    def runs(self) -> list[tuple[int, int | None]]:
        """(layer, number of the pass it opens or None) in the order the layers run."""
        n, loop = len(self.cfg["layers"]), self.cfg.get("loop")
        if not loop:
            return [(i, None) for i in range(n)]
        a, b, times = loop["start"], loop["stop"], loop["times"]
        out = [(i, None) for i in range(a)]
        for p in range(times):
            out += [(i, p if i == a else None) for i in range(a, b)]
        return out + [(i, None) for i in range(b, n)]

    def hidden(self, tokens, every_layer: bool = False):
        toks = np.asarray(tokens)
        pos = np.arange(len(toks))
        x0 = self.w["embed"][toks] * float(self.cfg["embedding"]["scale"])
        x, seen = x0, []
        for i, opens in self.runs():
            if opens is not None:
                x = np.concatenate([x, x0], axis=-1) @ self.w["loop.in"].T + self.w["loop.step"][opens]
            x = self.layer(i, x, pos)
            seen.append(x)
        return seen if every_layer else x

    def logits(self, tokens) -> np.ndarray:
        x = offset_norm(self.hidden(tokens), self.w["final.norm"], self.eps)
        return x @ self.w["embed"].T

    def greedy(self, prompt, n: int) -> list[int]:
        toks, out = list(prompt), []
        for _ in range(n):
            nxt = int(np.argmax(self.logits(toks)[-1]))
            out.append(nxt)
            toks.append(nxt)
        return out
