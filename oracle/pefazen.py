"""Plain float64 model of the Pefazen family: token loops and explicit sums, one function per mechanism, no code shared
with the package's product path. Tests hold the engine's kernels against it.

Notation: x [n, W] residual rows of ONE sequence at positions 0 .. n-1; every function sees whole sequences (no cache, no
portions): whatever the engine does with pages, slots and batches has to agree with this.
"""
from __future__ import annotations

import math

import numpy as np


def f64(t) -> np.ndarray:
    """A tensor (torch, any float type) or array as float64 numpy."""
    if hasattr(t, "detach"):
        t = t.detach().to("cpu").double().numpy()
    return np.asarray(t, dtype=np.float64)


def layer_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """Centered norm without bias: (x - mean) / sqrt(var + eps) * w, var = mean of squared deviations."""
    out = np.empty_like(x)
    for t in range(x.shape[0]):
        mu = x[t].sum() / x.shape[1]
        dev = x[t] - mu
        var = (dev * dev).sum() / x.shape[1]
        out[t] = dev / math.sqrt(var + eps) * w
    return out


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    out = np.empty_like(x)
    for t in range(x.shape[0]):
        out[t] = x[t] / math.sqrt((x[t] * x[t]).sum() / x.shape[1] + eps) * w
    return out


def rotary_table(rot: dict) -> tuple[np.ndarray, float]:
    """(frequency of every pair, magnitude factor on cos and sin). With `scaling` the frequencies of slow pairs are divided by
    `factor`, blended over the pairs between the two wavelength marks, and the magnitude becomes 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    freq = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return freq, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def pair_at(turns: float) -> float:                  # the (fractional) pair that makes `turns` turns over `orig` positions
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_at(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_at(float(sc["slow"]))), dims - 1)
    out = np.empty_like(freq)
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = freq[i] / factor * ramp + freq[i] * (1.0 - ramp)
    return out, 0.1 * math.log(factor) + 1.0


def rotate(v: np.ndarray, pos: int, freq: np.ndarray, mag: float, halves: bool) -> np.ndarray:
    """Turn the leading 2 * len(freq) entries of v by pos * freq; pairs are (2i, 2i+1), or (i, i + dims/2) with `halves`."""
    out = v.copy()
    half = len(freq)
    for i in range(half):
        a, b = (i, i + half) if halves else (2 * i, 2 * i + 1)
        c, s = math.cos(pos * freq[i]) * mag, math.sin(pos * freq[i]) * mag
        out[a] = v[a] * c - v[b] * s
        out[b] = v[b] * c + v[a] * s
    return out


def latent_kv(h: np.ndarray, w: dict, m: dict, eps: float, halves: bool) -> tuple[np.ndarray, np.ndarray]:
    """What a latent-attention layer keeps per token: the normed latent [n, kv_rank] and the rotated shared key part [n, rot_dim]."""
    r = int(m["kv_rank"])
    freq, mag = rotary_table(m["rot"])
    down = h @ f64(w["dkv"]).T
    lat = rms_norm(down[:, :r], f64(w["dkv.norm"]), eps)
    kr = np.stack([rotate(down[t, r:], t, freq, mag, halves) for t in range(h.shape[0])])
    return lat, kr


def latent_attention(h: np.ndarray, w: dict, m: dict, eps: float, halves: bool, window: int, gated: bool,
                     kv: tuple[np.ndarray, np.ndarray]) -> np.ndarray:
    """Attention with keys and values up-projected from a per-token latent; `kv` = (latent, rotated key part) of this layer
    or of the layer it borrows from. window > 0: a query sees itself and the window - 1 positions before it."""
    n = h.shape[0]
    H, d, dr, dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    freq, mag = rotary_table(m["rot"])
    lat, kr = kv
    cq = rms_norm(h @ f64(w["dq"]).T, f64(w["dq.norm"]), eps)
    q = (cq @ f64(w["uq"]).T).reshape(n, H, d + dr)
    ku = (lat @ f64(w["uk"]).T).reshape(n, H, d)
    vu = (lat @ f64(w["uv"]).T).reshape(n, H, dv)
    gate = h @ f64(w["g"]).T if gated else None
    out = np.zeros((n, H, dv))
    for t in range(n):
        first = max(t - window + 1, 0) if window > 0 else 0
        for a in range(H):
            qr = rotate(q[t, a, d:], t, freq, mag, halves)
            keys = slice(first, t + 1)                          # the visible positions
            sc = (ku[keys, a] @ q[t, a, :d] + kr[keys] @ qr) * float(m["scale"])
            p = np.exp(sc - sc.max())
            o = (p / p.sum()) @ vu[keys, a]
            if gated:
                o = o / (1.0 + math.exp(-gate[t, a]))
            out[t, a] = o
    return out.reshape(n, H * dv) @ f64(w["o"]).T


def route(z: np.ndarray, correction: np.ndarray, top: int) -> tuple[np.ndarray, np.ndarray]:
    """Sigmoid scores; the `top` largest of score + correction are chosen (lower index on a tie); weights = the plain scores."""
    n = z.shape[0]
    ids, wts = np.zeros((n, top), dtype=np.int64), np.zeros((n, top))
    for t in range(n):
        s = 1.0 / (1.0 + np.exp(-z[t]))
        c = s + correction
        order = sorted(range(len(c)), key=lambda e: (-c[e], e))[:top]
        ids[t], wts[t] = order, s[order]
    return ids, wts


def routed_experts(h: np.ndarray, w: dict, mlp: dict) -> np.ndarray:
    """Mixture of experts W_down relu(W_up h)^2; weights are not renormalised."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    ids, wts = route(h @ f64(w["router"]).T, f64(w["correction"]), top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(ids[t, k])
            assert 0 <= e < E
            a = np.maximum(f64(w[f"e{e}.up"]) @ h[t], 0.0)
            out[t] += wts[t, k] * (f64(w[f"e{e}.down"]) @ (a * a))
    return out


def _sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(raw: dict, tensors: dict, tokens, trace: list | None = None) -> np.ndarray:
    """Logits [n, vocab] of one sequence; `trace` receives the residual rows after every layer."""
    eps, mult = float(raw["norm"]["eps"]), float(raw["residual_mult"])
    x = f64(tensors["embed"])[np.asarray(tokens)]
    kept: dict[int, tuple] = {}
    for i, layer in enumerate(raw["layers"]):
        w, m = _sub(tensors, f"l{i}."), layer["mixer"]
        second = layer["type"] == "latent_attention_2"
        assert second or layer["type"] == "latent_attention"
        h = layer_norm(x, f64(w["norm1"]), eps)
        mix = _sub(w, "mix.")
        src = m.get("kv_from")
        kv = kept[int(src)] if src is not None else latent_kv(h, mix, m, eps, second)
        kept[i] = kv
        window = 0 if second else int(m["mask"]["size"])
        x = x + mult * latent_attention(h, mix, m, eps, second, window, not second, kv)
        if layer.get("mlp") is not None:
            x = x + mult * routed_experts(layer_norm(x, f64(w["norm2"]), eps), _sub(w, "mlp."), layer["mlp"])
        if trace is not None:
            trace.append(x.copy())
    z = layer_norm(x, f64(tensors["final.norm"]), eps) @ f64(tensors["head"]).T * float(raw.get("logit_scale", 1.0))
    cap = float(raw.get("logit_softcap") or 0.0)
    return cap * np.tanh(z / cap) if cap > 0 else z


class Model:
    """A checkpoint directory read into float64 (config.json + model.safetensors)."""

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
