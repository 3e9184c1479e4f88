"""Sequence mixers and feed-forwards beyond full attention, as layers any model of the package can compose:

  WindowAttention     paged softmax attention with a local mask (a sliding window, or blocks of positions, or none), any
                      query / value head size, optional per-head q/k RMS norm, optional rotation of the leading dimensions
                      in interleaved pairs, optional sigmoid output gate
  AttentionMixer      fused biased q | k | v projection -> WindowAttention -> out projection
  ConvAttentionMixer  attention whose query and key projections pass a short stateful causal convolution, whose keys (before
                      rotation) are also its values, with a constant or learned sink in the softmax and a gate per head
  GatedMemoryCore     matrix memory with exponential input / forget gates held in range by a running maximum (mLSTM style),
                      per-head RMS norm, sigmoid gate; consumes column ranges of its owner's fused projection
  AttentionMemoryMixer  position-free attention (query temperature, learned sinks, gated) beside a GatedMemoryCore on the same
                      input: ONE fused in-projection, two out-projections; the caller adds the two with the design's scales
  LatentAttentionMixer  attention whose keys and values are up-projections of a cached low-rank latent plus one rotated key part
                      shared by the heads; runs in the latent space on WindowAttention's kernels (one kv head), with a query
                      latent, either rotary pairing, optional frequency scaling, window or causal mask, optional per-head
                      sigmoid gate, and optionally the cache of an earlier layer instead of its own
  LightningMixer      linear attention as a decaying outer-product recurrence (per-head constant decay), SiLU on q / k / v,
                      RMS norm over the heads together, sigmoid gate
  SSDMixer            state-space-duality (Mamba-2 style) mixer: stateful causal convolution + SiLU, the recurrence in
                      32-bit, gate-then-group-norm
  RGLRUMixer          recurrent block with a real-gated linear recurrent unit (block-diagonal gates)
  ParallelMixer       two mixers on the same input; the caller averages their RMS-normed outputs
  XIELUFeedForward    up -> xIELU -> down
  ClampedGLU          [gate | up] -> min(g, limit) sigmoid(alpha g) (clamp(u) + 1) -> down
  GeluFeedForward     up -> GELU (tanh form) -> down
  RoutedExperts       mixture of experts (gated SiLU units, or ungated squared-ReLU units): softmax or sigmoid router with a
                      choice-only correction, choice limited to the best groups of experts, weights renormalised or not,
                      pass-through experts, optional shared expert with a sigmoid gate per token; or, instead of a router, a
                      table from token ids to experts with equal weights

Every constant a design may change is a constructor argument. Matrix products are the vendor library's (F.linear /
baddbmm); everything else is a kernel of libnvl_seq.so (ops_seq). Layers read the step's packed-portion description from
the attention-metadata context (`portions`, `slot_mapping`, `block_tables`); the runner injects the per-layer cache and
state tensors named by `kv_shapes()` / `state_shapes()`.

Weights live in fused tensors (one in-projection per mixer); `named_loaders()` maps a checkpoint's tensor names to
functions that copy into them.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops_seq
from .attn_meta import get_context


def _param(*shape, dtype=None):
    return nn.Parameter(torch.zeros(*shape, dtype=dtype), requires_grad=False)


def _copy_into(dst: torch.Tensor):
    def load(t: torch.Tensor):
        assert tuple(t.shape) == tuple(dst.shape), (tuple(t.shape), tuple(dst.shape))
        dst.copy_(t.to(dst.dtype))
    return load


class WindowAttention(nn.Module):
    """Consumes q | k | v | gate column ranges of the owner's fused projection output."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, eps: float,
                 qk_norm: bool = True, block_size: int = 256, chunk: int = 0, rot_dims: int = 0, rot_base: float = 10000.0,
                 rot_freqs: list | None = None, sink: str | None = None, q_temp: tuple | None = None, gate_per_head: bool = False):
        """window > 0: the last `window` positions are visible; chunk > 0: the positions of the query's own block of `chunk`
        (counted from the start of the sequence); neither: all earlier positions. rot_dims > 0: entries (2i, 2i+1),
        i < rot_dims / 2, of every query and key head turn by position * rot_base^(-2i / rot_dims), or by position * rot_freqs[i]
        when the caller brings its own table of rot_dims / 2 frequencies. sink: "zero" puts one more score of 0 (no value) into every
        softmax denominator, "learned" a score per head (parameter `sink`, 32-bit). q_temp (coef, every): the query at position p
        is multiplied by 1 + coef ln(floor((p + 1) / every) + 1). gate_per_head: the gate has one entry per head."""
        super().__init__()
        assert sink in (None, "zero", "learned") and (rot_freqs is None or len(rot_freqs) == rot_dims // 2)
        self.gate_per_head, self.q_temp = bool(gate_per_head), (float(q_temp[0]), int(q_temp[1])) if q_temp else None
        if sink == "learned":
            self.sink = _param(heads, dtype=torch.float32)
        else:
            self.register_buffer("sink", torch.zeros(heads, dtype=torch.float32) if sink else None, persistent=False)
        assert heads % kv_heads == 0 and dim <= 256 and vdim <= 256 and not (window > 0 and chunk > 0)
        assert rot_dims % 2 == 0 and 0 <= rot_dims <= dim
        self.H, self.G, self.d, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.window, self.eps, self.block_size = float(scale), int(window), eps, block_size
        self.chunk = int(chunk)
        # frequencies in double precision on the host, rounded once; angles are position * frequency in 32-bit
        freqs = rot_freqs if rot_freqs is not None else [float(rot_base) ** (-2.0 * i / rot_dims) for i in range(rot_dims // 2)]
        self.register_buffer("rot_freq", torch.tensor(freqs, dtype=torch.float32) if rot_dims else None, persistent=False)
        self.q_norm = _param(dim) if qk_norm else None
        self.k_norm = _param(dim) if qk_norm else None
        self.k_cache = self.v_cache = None            # [pages * block_size, G, d] / [..., G, dv] (values page-transposed), from the runner

    @property
    def widths(self) -> tuple[int, int, int, int]:
        """Columns of q, k, v and the gate in the fused projection."""
        return self.H * self.d, self.G * self.d, self.G * self.dv, self.H * self.dv

    def kv_shapes(self) -> tuple[tuple, tuple]:
        """Per-token shapes of this layer's K and V pages."""
        return (self.G, self.d), (self.G, self.dv)

    def forward(self, q, k, v, gate, positions: torch.Tensor | None = None) -> torch.Tensor:
        ctx = get_context()
        ops_seq.knorm_kvstore(k, v, self.k_norm, self.eps, self.G, self.d, self.dv, self.block_size, ctx.slot_mapping, self.k_cache,
                              self.v_cache, positions, self.rot_freq)
        out = torch.empty(q.shape[0], self.H * self.dv, dtype=q.dtype, device=q.device)
        ops_seq.window_attn(q, self.q_norm, self.eps, gate, self.k_cache, self.v_cache, ctx.block_tables, self.block_size,
                            ctx.portions, self.H, self.G, self.d, self.dv, self.scale, self.window, out, self.chunk, self.rot_freq,
                            gate_per_head=self.gate_per_head, sink=self.sink, q_temp=self.q_temp)
        return out


class AttentionMixer(nn.Module):
    """q | k | v in ONE biased projection, attention (WindowAttention: mask, rotation), out projection."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float, block_size: int,
                 window: int = 0, chunk: int = 0, rot_dims: int = 0, rot_base: float = 10000.0, qk_norm: bool = False):
        super().__init__()
        self.attn = WindowAttention(heads, kv_heads, dim, vdim, scale, window, eps, qk_norm=qk_norm, block_size=block_size,
                                    chunk=chunk, rot_dims=rot_dims, rot_base=rot_base)
        self.cols = self.attn.widths[:3]
        total = sum(self.cols)
        self.in_w, self.in_b = _param(total, width), _param(total)
        self.o_w = _param(width, heads * vdim)

    def named_loaders(self) -> dict:
        q, k, v = self.cols
        return {"q": _copy_into(self.in_w[:q]), "q.b": _copy_into(self.in_b[:q]), "k": _copy_into(self.in_w[q:q + k]),
                "k.b": _copy_into(self.in_b[q:q + k]), "v": _copy_into(self.in_w[q + k:]), "v.b": _copy_into(self.in_b[q + k:]),
                "o": _copy_into(self.o_w)}

    def forward(self, xh: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        proj = F.linear(xh, self.in_w, self.in_b)
        q, k, v = self.cols
        return F.linear(self.attn(proj[:, :q], proj[:, q:q + k], proj[:, q + k:], None, positions), self.o_w)


def rotary_frequencies(dims: int, base: float, scaling: dict | None = None) -> tuple[list[float], float]:
    """Frequencies of the dims / 2 rotated pairs, base^(-2i/dims), in double precision, and the factor on cos and sin (1).
    With `scaling` = {factor, original, fast, slow} (YaRN): pairs that turn fewer than `slow` times over `original` positions have
    their frequency divided by `factor`, pairs that turn more than `fast` times keep it, the pairs between the two marks
    (rounded outwards to whole pairs) blend linearly, and cos and sin are multiplied by 0.1 ln(factor) + 1."""
    import math
    freq = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freq, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def mark(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
    lo, hi = max(math.floor(mark(float(scaling["fast"]))), 0), min(math.ceil(mark(float(scaling["slow"]))), dims - 1)
    span = max(hi - lo, 0.001)
    ramps = [min(max((i - lo) / span, 0.0), 1.0) for i in range(dims // 2)]
    return [f / factor * r + f * (1.0 - r) for f, r in zip(freq, ramps)], 0.1 * math.log(factor) + 1.0


def banded_rotary_frequencies(dims: int, base: float, scaling: dict | None = None) -> list[float]:
    """Frequencies base^(-2i/dims) of the dims / 2 rotated pairs, in double precision. With `scaling` = {factor, low, high,
    original} the pairs are treated by wavelength l = 2 pi / f: shorter than original / high they stay, longer than original / low
    they are divided by `factor`, and between the two marks s = (original / l - low) / (high - low) blends (1 - s) f / factor + s f."""
    import math
    freq = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return freq
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = []
    for f in freq:
        wavelength = 2.0 * math.pi / f
        if wavelength < original / high:
            out.append(f)
        elif wavelength > original / low:
            out.append(f / factor)
        else:
            s_ = (original / wavelength - low) / (high - low)
            out.append((1.0 - s_) * f / factor + s_ * f)
    return out


class ConvAttentionMixer(nn.Module):
    """q = conv(W_q h), k = conv(W_k h): a causal convolution of `taps` taps over time on every channel, right after the projection
    (no bias, no activation; the last taps - 1 projected rows of a sequence are its state). The keys as they leave the convolution
    are also the values (so vdim == dim and there is no W_v); q and k are then rotated (WindowAttention: rot_dims, rot_freqs).
    Softmax with a sink (`sink`), head a's output times sigmoid(W_g h)_a, out projection. ONE fused in-projection [q | k | g]."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, taps: int, scale: float, eps: float, block_size: int,
                 window: int = 0, rot_dims: int = 0, rot_base: float = 10000.0, rot_freqs: list | None = None, sink: str | None = "zero"):
        super().__init__()
        assert taps >= 1
        self.attn = WindowAttention(heads, kv_heads, dim, dim, scale, window, eps, qk_norm=False, block_size=block_size, rot_dims=rot_dims,
                                    rot_base=rot_base, rot_freqs=rot_freqs, sink=sink, gate_per_head=True)
        self.q_cols, self.k_cols, self.taps = heads * dim, kv_heads * dim, int(taps)
        self.channels = self.q_cols + self.k_cols
        self.in_w = _param(self.channels + heads, width)
        self.conv_w = _param(self.channels, taps)
        self.o_w = _param(width, heads * dim)
        self.conv_state = None

    def state_shapes(self) -> dict:
        return {"conv_state": (self.taps - 1, self.channels)}

    def named_loaders(self) -> dict:
        q, c = self.q_cols, self.channels
        return {"q": _copy_into(self.in_w[:q]), "k": _copy_into(self.in_w[q:c]), "g": _copy_into(self.in_w[c:]),
                "q.conv": _copy_into(self.conv_w[:q]), "k.conv": _copy_into(self.conv_w[q:]), "o": _copy_into(self.o_w)}

    def forward(self, xh: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        por = get_context().portions
        q, c = self.q_cols, self.channels
        proj = F.linear(xh, self.in_w)
        qk = torch.empty(xh.shape[0], c, dtype=xh.dtype, device=xh.device)
        ops_seq.causal_conv(proj[:, :c], self.conv_w, None, 0, por, self.conv_state, qk)
        k = qk[:, q:]
        return F.linear(self.attn(qk[:, :q], k, k, proj[:, c:], positions), self.o_w)


class GatedMemoryCore(nn.Module):
    """Matrix memory with exponential gates, per head: from the gate pre-activations zi = W_i h + b_i, zf = W_f h + b_f,
    i = cap tanh(zi / cap), f = logsigmoid(cap tanh(zf / cap)); a running maximum m' = max(f + m, i) (m = 0 before the first token)
    keeps exp(f + m - m') and exp(i - m') in range: S <- exp(f + m - m') S + exp(i - m') k v^T, n likewise with k alone,
    o = S^T q / (max(|n . q|, exp(-m')) + 1e-6) with q = W_q h / sqrt(dim). Every head's o is divided by its root mean square, then
    times `norm`, times sigmoid(W_g h). State (S with n as one more row, and m) and everything from the gates on are 32-bit.
    Consumes the columns [v | k | q | g | zi | zf] of its owner's fused projection, starting at col0."""

    def __init__(self, heads: int, dim: int, vdim: int, cap: float, eps: float):
        super().__init__()
        self.H, self.d, self.dv, self.cap, self.eps = heads, dim, vdim, float(cap), eps
        self.cols = (heads * vdim, heads * dim, heads * dim, heads * vdim, heads, heads)          # v | k | q | g | zi | zf
        self.i_b, self.f_b = _param(heads), _param(heads)
        self.norm = _param(heads * vdim)
        self.rec_state = self.max_state = None

    @property
    def in_width(self) -> int:
        return sum(self.cols)

    def state_shapes(self) -> dict:
        return {"rec_state": (self.H, self.dv + 1, self.d), "max_state": (self.H,)}

    def forward(self, proj: torch.Tensor, col0: int) -> torch.Tensor:
        por = get_context().portions
        n = proj.shape[0]
        v, k, q, g, _, _ = self.cols
        y = torch.empty(n, v, dtype=torch.float32, device=proj.device)
        den = torch.empty(n, self.H, dtype=torch.float32, device=proj.device)
        ops_seq.gated_memory_scan(proj, col0, col0 + v, col0 + v + k, col0 + v + k + q + g, col0 + v + k + q + g + self.H, self.i_b,
                                  self.f_b, self.cap, self.d ** -0.5, self.H, self.d, self.dv, por, self.rec_state, self.max_state, y, den)
        out = torch.empty(n, v, dtype=proj.dtype, device=proj.device)
        ops_seq.gated_group_norm(y, proj[:, col0 + v + k + q:col0 + v + k + q + g], self.norm, self.H, self.eps, out, norm_first=True, den=den)
        return out


class AttentionMemoryMixer(nn.Module):
    """Two mixers on the same input. Left: attention without any rotation, whose queries are multiplied by a temperature that
    grows with the logarithm of the position (WindowAttention: q_temp), a learned sink per head in the softmax denominator, the
    concatenated heads times sigmoid(W_g h), out projection. Right: GatedMemoryCore, out projection. ONE fused in-projection
    [q | k | v | g | right's columns]. Returns both outputs; the caller combines them (each has its own scale)."""

    def __init__(self, width: int, left: dict, right: dict, eps: float, block_size: int):
        super().__init__()
        qt = left.get("q_temp")
        self.attn = WindowAttention(left["heads"], left.get("kv_heads", left["heads"]), left["dim"], left.get("vdim", left["dim"]),
                                    left["scale"], 0, eps, qk_norm=False, block_size=block_size, sink="learned",
                                    q_temp=(qt["coef"], qt["every"]) if qt else None)
        self.mem = GatedMemoryCore(right["heads"], right["dim"], right.get("vdim", right["dim"]), right["gate_cap"], eps)
        self.cols = list(self.attn.widths) + [self.mem.in_width]
        self.in_w = _param(sum(self.cols), width)
        self.left_o = _param(width, self.attn.H * self.attn.dv)
        self.right_o = _param(width, self.mem.H * self.mem.dv)

    def named_loaders(self) -> dict:
        q, k, v, g, _ = self.cols
        o = [0, q, q + k, q + k + v, q + k + v + g]
        out = {"left.q": _copy_into(self.in_w[o[0]:o[1]]), "left.k": _copy_into(self.in_w[o[1]:o[2]]),
               "left.v": _copy_into(self.in_w[o[2]:o[3]]), "left.g": _copy_into(self.in_w[o[3]:o[4]]),
               "left.sink": _copy_into(self.attn.sink), "left.o": _copy_into(self.left_o), "right.o": _copy_into(self.right_o),
               "right.norm": _copy_into(self.mem.norm), "right.i.b": _copy_into(self.mem.i_b), "right.f.b": _copy_into(self.mem.f_b)}
        at = o[4]
        for name, cols in zip(("v", "k", "q", "g", "i", "f"), self.mem.cols):
            out["right." + name] = _copy_into(self.in_w[at:at + cols])
            at += cols
        return out

    def forward(self, xh: torch.Tensor, positions: torch.Tensor | None = None):
        proj = F.linear(xh, self.in_w)
        q, k, v, g, _ = self.cols
        att = self.attn(proj[:, :q], proj[:, q:q + k], proj[:, q + k:q + k + v], proj[:, q + k + v:q + k + v + g])
        return F.linear(att, self.left_o), F.linear(self.mem(proj, q + k + v + g), self.right_o)


class LatentAttentionMixer(nn.Module):
    """Attention over a cached latent. Per token the layer keeps c = rms(W_dkv h)[:kv_rank] * w (the latent) and ONE rotated key
    part of rot_dim entries (the last rows of W_dkv, not normed); head a's key is [W_uk,a c | rotated part], its value W_uv,a c.
    Queries come from a latent too: q = W_uq (rms(W_dq h) * w), per head [dim unrotated | rot_dim rotated].

    The attention runs in the latent space, which is the same sum reordered: the query of head a becomes
    [W_uk,a^T q_a | rotated q part] (kv_rank + rot_dim entries), the cached row [c | rotated key part] is the key of ALL heads and
    c itself the value; W_uv,a is applied to the attention output. That is WindowAttention's paged kernel with one kv head.

    ONE fused in-projection [dq | dkv | gate]; two batched products per head (W_uk^T on the query, W_uv on the output).
    window > 0: the last `window` positions, else causal. rot_dims (<= rot_dim) leading entries of the rotated parts turn; the pair
    of i is (2i, 2i+1), or (i, i + rot_dims / 2) with rot_halves. gated: head a's output times sigmoid(W_g h)_a.
    source: an earlier layer's mixer whose cache this layer reads instead of keeping one (it then has no W_dkv)."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float, eps: float,
                 block_size: int, window: int = 0, rot_dims: int | None = None, rot_base: float = 10000.0, rot_halves: bool = False,
                 rot_scaling: dict | None = None, gated: bool = False, source: "LatentAttentionMixer | None" = None):
        super().__init__()
        rot_dims = rot_dim if rot_dims is None else int(rot_dims)
        assert rot_dims % 2 == 0 and 0 <= rot_dims <= rot_dim
        # (rows of up to 256 entries run on the matrix cores in bf16, longer ones on the scalar kernel)
        assert kv_rank + rot_dim <= 1024, f"latent row of {kv_rank} + {rot_dim} entries: the attention kernels take up to 1024"
        self.H, self.d, self.dr, self.dv, self.qr, self.r = heads, dim, rot_dim, vdim, q_rank, kv_rank
        self.scale, self.eps, self.window, self.gated, self.block_size = float(scale), eps, int(window), bool(gated), block_size
        self._source = (source,) if source is not None else ()          # (a tuple: not a submodule of this layer)
        if source is not None:
            assert source.r == kv_rank and source.dr == rot_dim and not source._source, "the borrowed cache has other sizes, or is borrowed itself"
        freq, self.rot_mag = rotary_frequencies(rot_dims, rot_base, rot_scaling) if rot_dims else ([], 1.0)
        self.rot_halves = bool(rot_halves)
        self.register_buffer("rot_freq", torch.tensor(freq, dtype=torch.float32) if rot_dims else None, persistent=False)
        self.kv_col = q_rank if source is None else -1
        self.g_col = q_rank + (kv_rank + rot_dim if source is None else 0)
        self.in_w = _param(self.g_col + (heads if gated else 0), width)
        self.q_norm, self.uq = _param(q_rank), _param(heads * (dim + rot_dim), q_rank)
        self.kv_norm = _param(kv_rank) if source is None else None
        self.uk, self.uv = _param(heads, dim, kv_rank), _param(heads, vdim, kv_rank)
        self.o_w = _param(width, heads * vdim)
        self.k_cache = self.v_cache = None            # [pages * block_size, 1, kv_rank + rot_dim] / [.., 1, kv_rank], from the runner

    def kv_shapes(self):
        """Per-token shapes of this layer's pages: the row [latent | rotated key part] and the latent again as the value (the
        kernels read values page-transposed). None: the layer reads another layer's pages."""
        return None if self._source else ((1, self.r + self.dr), (1, self.r))

    def named_loaders(self) -> dict:
        out = {"dq": _copy_into(self.in_w[:self.qr]), "dq.norm": _copy_into(self.q_norm), "uq": _copy_into(self.uq),
               "uk": _copy_into(self.uk.view(self.H * self.d, self.r)), "uv": _copy_into(self.uv.view(self.H * self.dv, self.r)),
               "o": _copy_into(self.o_w)}
        if not self._source:
            out.update({"dkv": _copy_into(self.in_w[self.qr:self.g_col]), "dkv.norm": _copy_into(self.kv_norm)})
        if self.gated:
            out["g"] = _copy_into(self.in_w[self.g_col:])
        return out

    def forward(self, xh: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        n, H, d, dr, dv, r = xh.shape[0], self.H, self.d, self.dr, self.dv, self.r
        owner = self._source[0] if self._source else self
        rot = ops_seq.Rotation(self.rot_freq, self.rot_halves, self.rot_mag) if self.rot_freq is not None else None
        proj = F.linear(xh, self.in_w)
        cq = torch.empty(n, self.qr, dtype=xh.dtype, device=xh.device)
        ops_seq.latent_prep(proj, 0, self.qr, self.q_norm, cq, self.eps, self.kv_col, r, dr, self.kv_norm, positions, rot,
                            owner.block_size, ctx.slot_mapping, owner.k_cache, owner.v_cache)
        q = F.linear(cq, self.uq).view(n, H, d + dr)
        qf = torch.empty(n, H, r + dr, dtype=xh.dtype, device=xh.device)
        torch.bmm(q[:, :, :d].transpose(0, 1), self.uk, out=qf[:, :, :r].transpose(0, 1))          # W_uk^T q per head
        ops_seq.rotate_heads(q[:, :, d:], qf[:, :, r:], positions, rot)
        lat = torch.empty(n, H * r, dtype=xh.dtype, device=xh.device)
        ops_seq.window_attn(qf.view(n, H * (r + dr)), None, self.eps, proj[:, self.g_col:] if self.gated else None, owner.k_cache,
                            owner.v_cache, ctx.block_tables, owner.block_size, ctx.portions, H, 1, r + dr, r, self.scale, self.window,
                            lat, gate_per_head=True)
        out = torch.empty(n, H, dv, dtype=xh.dtype, device=xh.device)
        torch.bmm(lat.view(n, H, r).transpose(0, 1), self.uv.transpose(1, 2), out=out.transpose(0, 1))   # W_uv on the latent output
        return F.linear(out.view(n, H * dv), self.o_w)


class LightningMixer(nn.Module):
    """Linear attention in its recurrent form: q, k, v = SiLU of the projections; per head S <- decay_h S + k v^T, o = S^T q
    (state and products in 32-bit); the heads together are RMS-normed (weight `norm`), multiplied by sigmoid(W_g h) and
    projected. ONE in-projection [v | k | q | g]; SiLU is applied inside the scan as it stages its operands."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, eps: float):
        super().__init__()
        assert len(decay) == heads
        self.H, self.d, self.dv, self.eps = heads, dim, vdim, eps
        self.cols = (heads * vdim, heads * dim, heads * dim, heads * vdim)          # v | k | q | g
        self.in_w = _param(sum(self.cols), width)
        self.register_buffer("decay", torch.tensor([float(a) for a in decay], dtype=torch.float32), persistent=False)
        self.norm = _param(heads * vdim)
        self.o_w = _param(width, heads * vdim)
        self.rec_state = None

    def state_shapes(self) -> dict:
        return {"rec_state": (self.H, self.dv, self.d)}

    def named_loaders(self) -> dict:
        v, k, q, g = self.cols
        return {"v": _copy_into(self.in_w[:v]), "k": _copy_into(self.in_w[v:v + k]), "q": _copy_into(self.in_w[v + k:v + k + q]),
                "g": _copy_into(self.in_w[v + k + q:]), "norm": _copy_into(self.norm), "o": _copy_into(self.o_w)}

    def forward(self, xh: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        por = get_context().portions
        n = xh.shape[0]
        v, k, q, g = self.cols
        proj = F.linear(xh, self.in_w)
        y = torch.empty(n, v, dtype=torch.float32, device=xh.device)
        ops_seq.decay_scan(proj, 0, v, v + k, self.decay, self.H, self.d, self.dv, por, self.rec_state, y)
        out = torch.empty(n, v, dtype=xh.dtype, device=xh.device)
        ops_seq.gated_group_norm(y, proj[:, v + k + q:], self.norm, 1, self.eps, out, norm_first=True)
        return F.linear(out, self.o_w)


class SSDMixer(nn.Module):
    """Consumes z | x B C | dt column ranges of the owner's fused projection output; returns the normed gated y."""

    def __init__(self, heads: int, vdim: int, state: int, groups: int, conv: int, norm_groups: int, eps: float):
        super().__init__()
        assert heads % groups == 0 and (heads * vdim) % norm_groups == 0
        self.heads, self.P, self.N, self.groups, self.taps, self.norm_groups, self.eps = heads, vdim, state, groups, conv, norm_groups, eps
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        self.conv_w, self.conv_b = _param(self.channels, conv), _param(self.channels)
        self.dt_bias, self.A_log, self.D = _param(heads), _param(heads), _param(heads)
        self.norm = _param(self.inner)
        self.conv_state = self.rec_state = None

    @property
    def in_width(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.N + self.heads

    def state_shapes(self) -> dict:
        return {"conv_state": (self.taps - 1, self.channels), "rec_state": (self.heads, self.P, self.N)}

    def forward(self, proj: torch.Tensor, col0: int) -> torch.Tensor:
        """`proj`: the fused projection output; this mixer's columns start at col0."""
        por = get_context().portions
        n = proj.shape[0]
        z = proj[:, col0:col0 + self.inner]
        xbc_in = proj[:, col0 + self.inner:col0 + self.inner + self.channels]
        xbc = torch.empty(n, self.channels, dtype=torch.float32, device=proj.device)
        ops_seq.causal_conv(xbc_in, self.conv_w, self.conv_b, 1, por, self.conv_state, xbc)
        y = torch.empty(n, self.inner, dtype=torch.float32, device=proj.device)
        ops_seq.ssd_scan(xbc, proj, col0 + self.inner + self.channels, self.dt_bias, self.A_log, self.D, self.heads, self.P, self.N,
                         self.groups, por, self.rec_state, y)
        out = torch.empty(n, self.inner, dtype=proj.dtype, device=proj.device)
        ops_seq.gated_group_norm(y, z, self.norm, self.norm_groups, self.eps, out)
        return out


class ParallelMixer(nn.Module):
    """Windowed attention and a state-space mixer side by side on the same input: ONE fused in-projection
    [q | k | v | gate | z | x B C | dt], two out-projections. Returns both branch outputs; the residual kernel
    norms each with `left_out` / `right_out`, halves their sum and norms the result."""

    def __init__(self, width: int, left: dict, right: dict, eps: float, block_size: int, dtype):
        super().__init__()
        self.attn = WindowAttention(left["heads"], left["kv_heads"], left["dim"], left["vdim"], left["scale"],
                                    left["mask"]["size"], eps, qk_norm=True, block_size=block_size)
        self.ssd = SSDMixer(right["heads"], right["vdim"], right["state"], right["groups"], right["conv"], right["norm_groups"], eps)
        self.cols = list(self.attn.widths) + [self.ssd.in_width]
        total = sum(self.cols)
        self.in_w, self.in_b = _param(total, width), _param(total)
        hdv = self.attn.H * self.attn.dv
        self.left_o, self.left_o_b = _param(width, hdv), _param(width)
        self.right_o = _param(width, self.ssd.inner)
        self.left_out, self.right_out = _param(width), _param(width)

    def named_loaders(self) -> dict:
        a, s = self.attn, self.ssd
        q, k, v, g, _ = self.cols
        o = [0, q, q + k, q + k + v, q + k + v + g]
        return {
            "left.q": _copy_into(self.in_w[o[0]:o[1]]), "left.q.b": _copy_into(self.in_b[o[0]:o[1]]),
            "left.k": _copy_into(self.in_w[o[1]:o[2]]), "left.k.b": _copy_into(self.in_b[o[1]:o[2]]),
            "left.v": _copy_into(self.in_w[o[2]:o[3]]), "left.v.b": _copy_into(self.in_b[o[2]:o[3]]),
            "left.g": _copy_into(self.in_w[o[3]:o[4]]), "right.in": _copy_into(self.in_w[o[4]:]),
            "left.q.norm": _copy_into(a.q_norm), "left.k.norm": _copy_into(a.k_norm),
            "left.o": _copy_into(self.left_o), "left.o.b": _copy_into(self.left_o_b),
            "right.conv": _copy_into(s.conv_w), "right.conv.b": _copy_into(s.conv_b), "right.dt_bias": _copy_into(s.dt_bias),
            "right.A_log": _copy_into(s.A_log), "right.D": _copy_into(s.D), "right.norm": _copy_into(s.norm),
            "right.o": _copy_into(self.right_o), "left.out": _copy_into(self.left_out), "right.out": _copy_into(self.right_out),
        }

    def forward(self, xh: torch.Tensor):
        proj = F.linear(xh, self.in_w, self.in_b)
        q, k, v, g, _ = self.cols
        att = self.attn(proj[:, :q], proj[:, q:q + k], proj[:, q + k:q + k + v], proj[:, q + k + v:q + k + v + g])
        left = F.linear(att, self.left_o, self.left_o_b)
        right = F.linear(self.ssd(proj, q + k + v + g), self.right_o)
        return left, right


class RGLRUMixer(nn.Module):
    """y = gelu_tanh(W_y h + b), u = conv(W_x h + b); per block of channels r = sigmoid(R u_b + b_r), i = sigmoid(I u_b + b_i);
    a = exp(-c r softplus(lam)); S <- a S + sqrt(1 - a^2) i u; out = W_o (S * y). The gates' matrices are kept in 32-bit
    and applied to the 32-bit convolution output."""

    def __init__(self, width: int, channels: int, blocks: int, conv: int, dtype, c: float = 8.0):
        super().__init__()
        assert channels % blocks == 0
        self.C, self.blocks, self.taps, self.c = channels, blocks, conv, float(c)
        bw = channels // blocks
        self.in_w, self.in_b = _param(2 * channels, width), _param(2 * channels)            # [y | x]
        self.conv_w, self.conv_b = _param(channels, conv), _param(channels)
        self.gate_w = _param(blocks, bw, 2 * bw, dtype=torch.float32)                       # per block [in, r-out | i-out]
        self.gate_b = _param(blocks, 1, 2 * bw, dtype=torch.float32)
        self.lam = _param(channels)
        self.o_w = _param(width, channels)
        self.conv_state = self.rec_state = None

    def state_shapes(self) -> dict:
        return {"conv_state": (self.taps - 1, self.C), "rec_state": (self.C,)}

    def named_loaders(self) -> dict:
        C, bw = self.C, self.C // self.blocks

        def gate(lo):
            def load(t):                                   # [blocks, out, in] -> [blocks, in, out]
                self.gate_w[:, :, lo:lo + bw].copy_(t.to(torch.float32).transpose(1, 2))
            return load

        def gate_bias(lo):
            def load(t):
                self.gate_b[:, 0, lo:lo + bw].copy_(t.to(torch.float32))
            return load
        return {
            "y": _copy_into(self.in_w[:C]), "y.b": _copy_into(self.in_b[:C]), "x": _copy_into(self.in_w[C:]),
            "x.b": _copy_into(self.in_b[C:]), "conv": _copy_into(self.conv_w), "conv.b": _copy_into(self.conv_b),
            "ra": gate(0), "ra.b": gate_bias(0), "ri": gate(bw), "ri.b": gate_bias(bw), "lam": _copy_into(self.lam),
            "o": _copy_into(self.o_w),
        }

    def forward(self, xh: torch.Tensor) -> torch.Tensor:
        por = get_context().portions
        n, C, bw = xh.shape[0], self.C, self.C // self.blocks
        proj = F.linear(xh, self.in_w, self.in_b)
        u = torch.empty(n, C, dtype=torch.float32, device=xh.device)
        ops_seq.causal_conv(proj[:, C:], self.conv_w, self.conv_b, 0, por, self.conv_state, u)
        gates = torch.baddbmm(self.gate_b, u.view(n, self.blocks, bw).transpose(0, 1), self.gate_w)     # [blocks, n, 2 bw] fp32
        s = torch.empty(n, C, dtype=xh.dtype, device=xh.device)
        ops_seq.rglru_scan(gates, u, proj[:, :C], self.lam, self.c, self.blocks, por, self.rec_state, s)
        return F.linear(s, self.o_w)


class XIELUFeedForward(nn.Module):

    def __init__(self, width: int, ff: int, beta: float = 0.5):
        super().__init__()
        self.up, self.down, self.act, self.beta = _param(ff, width), _param(width, ff), _param(2), beta

    def named_loaders(self) -> dict:
        return {"up": _copy_into(self.up), "down": _copy_into(self.down), "act": _copy_into(self.act)}

    def forward(self, xh: torch.Tensor) -> torch.Tensor:
        return F.linear(ops_seq.xielu(F.linear(xh, self.up), self.act, self.beta), self.down)


class GeluFeedForward(nn.Module):
    """W_down gelu(W_up h), GELU in its tanh form."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.ff, self.up, self.down = ff, _param(ff, width), _param(width, ff)

    def named_loaders(self) -> dict:
        return {"up": _copy_into(self.up), "down": _copy_into(self.down)}

    def forward(self, xh: torch.Tensor) -> torch.Tensor:
        z = F.linear(xh, self.up)
        act = torch.empty_like(z)
        ops_seq.glu_act(z, self.ff, act, kind=2)
        return F.linear(act, self.down)


class ClampedGLU(nn.Module):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(alpha g) (u + 1))."""

    def __init__(self, width: int, ff: int, limit: float, alpha: float = 1.702):
        super().__init__()
        self.ff, self.limit, self.alpha = ff, float(limit), float(alpha)
        self.gu, self.down = _param(2 * ff, width), _param(width, ff)

    def named_loaders(self) -> dict:
        return {"gate": _copy_into(self.gu[:self.ff]), "up": _copy_into(self.gu[self.ff:]), "down": _copy_into(self.down)}

    def forward(self, xh: torch.Tensor) -> torch.Tensor:
        gu = F.linear(xh, self.gu)
        act = torch.empty(xh.shape[0], self.ff, dtype=xh.dtype, device=xh.device)
        ops_seq.glu_act(gu, self.ff, act, kind=1, limit=self.limit, alpha=self.alpha)
        return F.linear(act, self.down)


class RoutedExperts(nn.Module):
    """Mixture of `experts` gated feed-forwards W_down (silu(W_gate h) * W_up h), `top` per token.

    Router (32-bit): s = softmax(W_r h) over experts + `identity` pass-through entries (the last ones; their output is h);
    choice scores s + correction; entries form `group_count` equal groups of neighbours of which the `group_keep` best (by
    their largest choice score) may be chosen from; weights s[chosen] / sum * `scale`. A shared expert of the same form
    (`shared_ff`) runs for every token, times sigmoid(w_sg . h). The router's matrix carries w_sg as its last row."""

    def __init__(self, width: int, experts: int, ff: int, top: int, scale: float = 1.0, identity: int = 0, group_count: int = 1,
                 group_keep: int = 1, shared_ff: int = 0, gated: bool = True, sigmoid: bool = False, renorm: bool = True,
                 table_vocab: int = 0, shared_gate: bool = True):
        """gated False: an expert is W_down max(W_up h, 0)^2 (checkpoint names e<i>.up / e<i>.down). sigmoid: scores are each
        entry's own sigmoid instead of a softmax over the entries. renorm False: the chosen scores are the weights as they are.
        table_vocab > 0: there is no router; row `token id` of `table` [table_vocab, top] (integers) names the token's experts,
        each with the weight 1 / top, and forward() takes the token ids. shared_gate False: the shared expert is added as it is."""
        super().__init__()
        self.table_vocab, self.shared_gate = int(table_vocab), bool(shared_gate) and not table_vocab
        self.gated, self.sigmoid, self.renorm = bool(gated), bool(sigmoid), bool(renorm)
        self.E, self.ident, self.ff, self.top, self.scale = experts, identity, ff, top, float(scale)
        self.count, self.keep, self.shared_ff = group_count, group_keep, shared_ff
        total = experts + identity
        assert total % group_count == 0 and 1 <= group_keep <= group_count and top <= group_keep * (total // group_count)
        if table_vocab:
            assert identity == 0 and group_count == 1
            self.table = _param(table_vocab, top, dtype=torch.int32)
        else:
            self.router = _param(total + (1 if shared_ff and self.shared_gate else 0), width, dtype=torch.float32)
            self.correction = _param(total, dtype=torch.float32)
        self.w_gu, self.w_down = _param(experts, (2 if gated else 1) * ff, width), _param(experts, width, ff)
        if shared_ff:
            self.s_gu, self.s_down = _param(2 * shared_ff, width), _param(width, shared_ff)

    def named_loaders(self) -> dict:
        total, ff = self.E + self.ident, self.ff
        out = {"table": _copy_into(self.table)} if self.table_vocab else \
            {"router": _copy_into(self.router[:total]), "correction": _copy_into(self.correction)}
        for e in range(self.E):
            if self.gated:
                out[f"e{e}.gate"] = _copy_into(self.w_gu[e, :ff])
                out[f"e{e}.up"] = _copy_into(self.w_gu[e, ff:])
            else:
                out[f"e{e}.up"] = _copy_into(self.w_gu[e])
            out[f"e{e}.down"] = _copy_into(self.w_down[e])
        if self.shared_ff:
            sf = self.shared_ff
            out.update({"shared.gate": _copy_into(self.s_gu[:sf]), "shared.up": _copy_into(self.s_gu[sf:]),
                        "shared.down": _copy_into(self.s_down)})
            if self.shared_gate:
                out["shared.sg"] = _copy_into(self.router[total:])
        return out

    def forward(self, xh: torch.Tensor, tokens: torch.Tensor | None = None) -> torch.Tensor:
        n, width = xh.shape
        total = self.E + self.ident
        if self.table_vocab:
            z = None
            ids, wts = ops_seq.moe_table_route(tokens, self.table, 1.0 / self.top)
        else:
            z = F.linear(xh.float(), self.router)                                 # 32-bit, [n, total (+ 1: the shared gate)]
            ids, wts = ops_seq.moe_route(z, total, self.correction, self.top, self.count, self.keep, self.scale, self.sigmoid, self.renorm)
        per_expert = n * self.top // self.E                 # rows an expert gets on average: the tile height follows it
        plan = ops_seq.moe_plan(ids, self.E, 128 if per_expert >= 256 else (64 if per_expert >= 64 else 16))
        act = torch.empty(plan.cap, self.ff, dtype=xh.dtype, device=xh.device)
        ops_seq.moe_gemm(xh, self.w_gu, plan, self.gated, act, relu2=not self.gated)
        rows = torch.empty(plan.cap, width, dtype=xh.dtype, device=xh.device)
        ops_seq.moe_gemm(act, self.w_down, plan, False, rows)
        shared = gate = None
        if self.shared_ff:
            sact = torch.empty(n, self.shared_ff, dtype=xh.dtype, device=xh.device)
            ops_seq.glu_act(F.linear(xh, self.s_gu), self.shared_ff, sact, kind=0)
            shared, gate = F.linear(sact, self.s_down), (z[:, total:] if self.shared_gate else None)
        out = torch.empty(n, width, dtype=xh.dtype, device=xh.device)
        ops_seq.moe_combine(rows, plan, wts, xh, shared, gate, out)
        return out


def tie_parameters(dst: nn.Module, src: nn.Module) -> None:
    """Make every parameter of `dst` the SAME tensor as in `src` (two modules of one construction): a layer that runs
    several times per step with the same weights but caches and state of its own per run."""
    for name, _ in list(dst.named_parameters()):
        d, s_ = dst, src
        parts = name.split(".")
        for part in parts[:-1]:
            d, s_ = getattr(d, part), getattr(s_, part)
        setattr(d, parts[-1], getattr(s_, parts[-1]))
