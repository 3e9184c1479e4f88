"""Plain, slow restatement of the Lobidra design on the CPU (test infrastructure only; shares no code with the product path
under nano_vllm_amd/). One function per mechanism, float64 throughout, loops over tokens wherever the design has a
recurrence, a convolution over time or a mask.

The design: a decoder whose layers are listed one by one. Every sublayer is normed on both sides,
x += nb(mixer(na(x))), x += nb'(ff(na'(x))), with RMS norms whose weights are stored as offsets from one. Mixers:
`attention` (short causal convolutions on the query / key projections, keys before rotation double as values, rotation of the
leading dimensions in interleaved pairs with band-wise scaled frequencies, a softmax whose denominator holds an extra one, a
sigmoid gate per head) and `parallel` (position-free attention with a query temperature that grows with the logarithm of the
position and a learned per-head sink in the denominator, beside a matrix-memory recurrence with exponential gates that are
kept in range by a running maximum). Feed-forwards: a GELU layer, or gated experts picked by a table over token ids plus a
shared expert. A layer may run with the weights of an earlier one.
"""
from __future__ import annotations

import math

import numpy as np


def f64(t) -> np.ndarray:
    import torch
    if isinstance(t, torch.Tensor):
        return t.to(torch.float64).numpy() if t.is_floating_point() else t.numpy().astype(np.int64)
    return np.asarray(t)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def offset_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """RMS norm whose weight is stored as its distance from one."""
    return rms(x, eps) * (1.0 + w)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * sigmoid(z)


def short_conv(u: np.ndarray, w: np.ndarray) -> np.ndarray:
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token."""
    T, taps = u.shape[0], w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                y[t] += w[:, j] * u[src]
    return y


def banded_frequencies(rot: dict) -> np.ndarray:
    """Frequencies base^(-2i/dims) of the rotated pairs; with `scaling`, pairs whose wavelength exceeds original/low are slowed by
    `factor`, those shorter than original/high stay, and the band between blends the two linearly in original/wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = f.copy()
    for i, fi in enumerate(f):
        wl = 2.0 * math.pi / fi
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[i] = fi / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_pairs(x: np.ndarray, pos: np.ndarray, freq: np.ndarray) -> np.ndarray:
    """x [T, heads, d]: entries (2i, 2i+1), i < len(freq), turn by pos * freq[i]; the rest pass."""
    out = x.copy()
    for i, fi in enumerate(freq):
        a = pos.astype(np.float64) * fi
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def sink_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, sink: np.ndarray) -> np.ndarray:
    """Causal attention, q [T, H, d], k [T, G, d], v [T, G, dv]; the denominator of head a also holds exp(sink[a]) (no value)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for a in range(H):
            g = a // (H // G)
            s = (k[:t + 1, g] @ q[t, a]) * scale
            m = max(s.max(), sink[a])
            e = np.exp(s - m)
            out[t, a] = (e @ v[:t + 1, g]) / (e.sum() + math.exp(sink[a] - m))
    return out


def conv_attention(h: np.ndarray, w: dict, m: dict) -> np.ndarray:
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = short_conv(h @ w["q"].T, w["q.conv"]).reshape(T, H, d)
    k = short_conv(h @ w["k"].T, w["k.conv"]).reshape(T, G, d)
    v = k                                              # the keys as they leave the convolution are the values
    pos = np.arange(T)
    rot = m.get("rot")
    if rot:
        freq = banded_frequencies(rot)
        q, k = rotate_pairs(q, pos, freq), rotate_pairs(k, pos, freq)
    o = sink_attention(q, k, v, float(m["scale"]), np.zeros(H))
    o = o * sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, -1) @ w["o"].T


def tempered_attention(h: np.ndarray, w: dict, m: dict) -> np.ndarray:
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).reshape(T, H, d)
    k = (h @ w["k"].T).reshape(T, G, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    qt = m.get("q_temp")
    if qt:
        p = np.arange(T)
        q = q * (1.0 + float(qt["coef"]) * np.log(np.floor((p + 1) / int(qt["every"])) + 1.0))[:, None, None]
    o = sink_attention(q, k, v, float(m["scale"]), w["sink"])
    return (o.reshape(T, -1) * sigmoid(h @ w["g"].T)) @ w["o"].T


def matrix_memory(h: np.ndarray, w: dict, m: dict, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, d, dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    q = (h @ w["q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).reshape(T, H, d)
    v = (h @ w["v"].T).reshape(T, H, dv)
    gi = cap * np.tanh((h @ w["i"].T + w["i.b"]) / cap)
    zf = cap * np.tanh((h @ w["f"].T + w["f.b"]) / cap)
    gf = -np.logaddexp(0.0, -zf)                       # log sigmoid
    out = np.zeros((T, H, dv))
    for a in range(H):
        S, n, mx = np.zeros((d, dv)), np.zeros(d), 0.0
        for t in range(T):
            mn = max(gf[t, a] + mx, gi[t, a])
            keep, take = math.exp(gf[t, a] + mx - mn), math.exp(gi[t, a] - mn)
            S = keep * S + take * np.outer(k[t, a], v[t, a])
            n = keep * n + take * k[t, a]
            mx = mn
            out[t, a] = (S.T @ q[t, a]) / (max(abs(n @ q[t, a]), math.exp(-mx)) + 1e-6)
    o = rms(out, eps).reshape(T, -1) * w["norm"] * sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def _sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def side_by_side(h: np.ndarray, w: dict, m: dict, eps: float) -> np.ndarray:
    return float(m["left_scale"]) * tempered_attention(h, _sub(w, "left."), m["left"]) + \
        float(m["right_scale"]) * matrix_memory(h, _sub(w, "right."), m["right"], eps)


def gated_unit(h: np.ndarray, w: dict) -> np.ndarray:
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def table_experts(h: np.ndarray, tokens: np.ndarray, w: dict, mlp: dict) -> np.ndarray:
    top = int(mlp["router"]["top"])
    out = np.zeros_like(h)
    table = w["table"].astype(np.int64)
    for t in range(h.shape[0]):
        for e in table[tokens[t]]:
            out[t] += gated_unit(h[t:t + 1], _sub(w, f"e{int(e)}."))[0] / top
    if mlp.get("shared"):
        out = out + gated_unit(h, _sub(w, "shared."))
    return out


def feed_forward(h: np.ndarray, tokens: np.ndarray, w: dict, mlp: dict) -> np.ndarray:
    if mlp["kind"] == "dense":
        return gelu_tanh(h @ w["up"].T) @ w["down"].T
    return table_experts(h, tokens, w, mlp)


def forward(raw: dict, tensors: dict, tokens, trace: list | None = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence; `trace` receives the residual rows after every layer."""
    eps = float(raw["norm"]["eps"])
    tokens = np.asarray(tokens)
    x = tensors["embed"][tokens] * float(raw["embedding"]["scale"])
    for i, layer in enumerate(raw["layers"]):
        w = _sub(tensors, f"l{int(layer.get('weights_of', i))}.")
        h = offset_norm(x, w["norm1"], eps)
        if layer["type"] == "attention":
            y = conv_attention(h, _sub(w, "mix."), layer["mixer"])
        else:
            assert layer["type"] == "parallel"
            y = side_by_side(h, _sub(w, "mix."), layer["mixer"], eps)
        x = x + offset_norm(y, w["norm1b"], eps)
        if layer.get("mlp") is not None:
            y = feed_forward(offset_norm(x, w["norm2"], eps), tokens, _sub(w, "mlp."), layer["mlp"])
            x = x + offset_norm(y, w["norm2b"], eps)
        if trace is not None:
            trace.append(x.copy())
    return offset_norm(x, tensors["final.norm"], eps) @ tensors["head"].T


class Model:
    """A checkpoint (configuration + tensors) read into float64."""

    def __init__(self, cfg: dict, tensors: dict):
        self.cfg, self.tensors = cfg, {k: f64(v) for k, v in tensors.items()}

    @classmethod
    def load(cls, path: str) -> "Model":
        import json
        import os

        from safetensors.torch import load_file
        with open(os.path.join(path, "config.json")) as fh:
            cfg = json.load(fh)
        return cls(cfg, load_file(os.path.join(path, "model.safetensors")))

    def run(self, tokens, trace: list | None = None) -> np.ndarray:
        return forward(self.cfg, self.tensors, tokens, trace)
