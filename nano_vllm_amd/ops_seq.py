"""ctypes binding of libnvl_seq.so (C ABI in include/nvl_seq.h): the kernels of layers that carry per-sequence state,
of windowed paged attention with any head size and of norms on a 32-bit residual stream.

As in ops.py, PyTorch owns memory and the stream and every function hands raw device pointers to a hand-written gfx950
kernel; there is no fallback. Activation / weight tensors are bfloat16 or float32 (`_code`), state and the residual
stream are float32. The library is built on first use when it is missing (a fresh checkout), by hipcc, in-tree.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

import torch

from . import build as _build

ABI_VERSION = 5
_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float

SIGNATURES = {
    "nvs_abi_version": (c_int, []),
    "nvs_last_error": (c_char_p, []),
    "nvs_embed_sinusoid": (c_int, [_P, _I, _P, _P, _L, _I, _F, _F, _P, _P, _P]),
    "nvs_norm_residual": (c_int, [_P, _P, _P, _P, _P, _I, _L, _I, _F, _P, _P, _P]),
    "nvs_scalar_norm_rows": (c_int, [_P, _P, _L, _I, _P, _I, _F, _P, _P]),
    "nvs_xielu": (c_int, [_P, _P, _F, _I, _L, _P, _P]),
    "nvs_causal_conv": (c_int, [_P, _L, _I, _P, _P, _I, _I, _I, _P, _P, _P, _P, _I, _L, _P, _P, _I, _P]),
    "nvs_sandwich_norm": (c_int, [_P, _P, _F, _P, _F, _P, _P, _L, _P, _F, _I, _I, _F, _P, _P]),
    "nvs_gated_memory_scan_workspace": (c_int64, [_I, _I, _I, _I, _L]),
    "nvs_gated_memory_scan": (c_int, [_P, _L, _L, _L, _L, _L, _L, _I, _P, _P, _F, _F, _I, _I, _I, _P, _P, _P, _I, _L, _L, _P, _P, _P, _P, _P,
                                      _L, _P]),
    "nvs_moe_table_route": (c_int, [_P, _P, _L, _I, _F, _P, _P, _P]),
    "nvs_rglru_scan_workspace": (c_int64, [_I, _I, _L]),
    "nvs_rglru_scan": (c_int, [_P, _P, _P, _L, _I, _P, _F, _I, _I, _P, _P, _P, _I, _L, _L, _P, _P, _P, _L, _P]),
    "nvs_ssd_scan_workspace": (c_int64, [_I, _I, _I, _I, _L]),
    "nvs_ssd_scan": (c_int, [_P, _P, _L, _L, _I, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _I, _L, _L, _P, _P, _P, _L, _P]),
    "nvs_decay_scan": (c_int, [_P, _L, _L, _L, _L, _I, _P, _I, _I, _I, _P, _P, _P, _I, _L, _L, _P, _P, _P, _L, _P]),
    "nvs_gated_group_norm": (c_int, [_P, _P, _L, _I, _P, _I, _I, _F, _I, _L, _P, _P, _P]),
    "nvs_knorm_kvstore": (c_int, [_P, _P, _L, _I, _P, _F, _I, _I, _I, _I, _P, _P, _P, _I, _L, _P, _P, _P]),
    "nvs_window_attn_force_scalar": (None, [_I]),
    "nvs_window_attn": (c_int, [_P, _L, _P, _F, _P, _L, _I, _I, _P, _P, _P, _L, _I, _P, _P, _P, _I, _L, _I, _I, _I, _I, _F, _I,
                                _I, _P, _I, _P, _F, _I, _P, _P]),
    "nvs_add_group_norm": (c_int, [_P, _P, _F, _P, _P, _L, _P, _I, _I, _I, _F, _I, _P, _P]),
    "nvs_scale_softcap": (c_int, [_P, _I, _F, _F, _L, _P, _P]),
    "nvs_latent_prep": (c_int, [_P, _L, _I, _I, _I, _P, _P, _I, _I, _I, _P, _P, _P, _I, _I, _F, _F, _I, _P, _P, _P, _L, _P]),
    "nvs_rotate_heads": (c_int, [_P, _L, _I, _P, _L, _I, _I, _I, _I, _P, _P, _I, _I, _F, _L, _P]),
    "nvs_glu_act": (c_int, [_P, _L, _I, _I, _I, _F, _F, _L, _P, _P]),
    "nvs_moe_route": (c_int, [_P, _L, _P, _L, _I, _I, _I, _I, _F, _I, _I, _P, _P, _P]),
    "nvs_moe_rows": (c_int64, [_L, _I, _I]),
    "nvs_moe_plan": (c_int, [_P, _L, _I, _I, _I, _P, _P, _P, _P]),
    "nvs_moe_gemm": (c_int, [_P, _L, _P, _I, _I, _I, _I, _P, _P, _L, _I, _P, _L, _P]),
    "nvs_moe_force_plain": (None, [_I]),
    "nvs_moe_combine": (c_int, [_P, _L, _P, _P, _I, _P, _L, _P, _P, _L, _I, _L, _I, _P, _P]),
}

_lib = None


class NvsError(RuntimeError):
    pass


def load_library() -> ctypes.CDLL:
    """Load libnvl_seq.so, building it first when the checkout has none (or an older one than its sources)."""
    global _lib
    if _lib is not None:
        return _lib
    path = _build.build_seq()
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    if lib.nvs_abi_version() != ABI_VERSION:
        raise NvsError(f"libnvl_seq.so ABI version {lib.nvs_abi_version()} != binding version {ABI_VERSION}; rebuild")
    if os.environ.get("NVL_ATTN_SCALAR") == "1":      # A/B switch: bf16 windowed attention on the scalar kernel too
        lib.nvs_window_attn_force_scalar(1)
    elif os.environ.get("NVL_ATTN_NO_LDS") == "1":    # ... or on the matrix cores without the LDS-shared K / V tiles
        lib.nvs_window_attn_force_scalar(2)
    elif os.environ.get("NVL_ATTN_UNPACKED") == "1":  # ... or never with heads in the query tiles of single-token steps
        lib.nvs_window_attn_force_scalar(3)
    _lib = lib
    return lib


def _check(rc: int) -> None:
    if rc != 0:
        raise NvsError(f"nvs error {rc}: {_lib.nvs_last_error().decode()}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _code(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 0
    if t.dtype == torch.float32:
        return 1
    raise NvsError(f"unsupported activation dtype {t.dtype} (bfloat16 or float32)")


def _ptr(t: torch.Tensor | None) -> int | None:
    if t is None:
        return None
    if not t.is_cuda:
        raise NvsError("device (HIP) tensors only; the hot path has no CPU fallback")
    return t.data_ptr()


def _same(code_of: torch.Tensor, *others: torch.Tensor | None) -> int:
    for o in others:
        if o is not None and o.dtype != code_of.dtype:
            raise NvsError(f"dtype mismatch: {o.dtype} beside {code_of.dtype}")
    return _code(code_of)


class Portions:
    """Device-side description of a step's packed portions (see include/nvl_seq.h): cu_q [nseq + 1], ctx0 [nseq],
    slot [nseq], tseq [n], all int32."""
    __slots__ = ("cu_q", "ctx0", "slot", "tseq", "nseq", "n", "max_q")

    def __init__(self, cu_q, ctx0, slot, tseq, nseq: int, n: int, max_q: int = 0):
        self.cu_q, self.ctx0, self.slot, self.tseq, self.nseq, self.n = cu_q, ctx0, slot, tseq, nseq, n
        self.max_q = max_q or n                        # the longest portion (a host-side bound; n when unknown)
        for t in (cu_q, ctx0, slot, tseq):
            assert t.dtype == torch.int32 and t.is_cuda and t.is_contiguous()
        assert cu_q.numel() >= nseq + 1 and ctx0.numel() >= nseq and slot.numel() >= nseq and tseq.numel() >= n


def embed_sinusoid(table, ids, pos, scale: float, base: float, x: torch.Tensor, xh: torch.Tensor | None):
    lib = load_library()
    n, width = ids.numel(), table.shape[1]
    assert x.dtype == torch.float32 and x.shape == (n, width) and x.is_contiguous() and table.is_contiguous()
    assert ids.dtype == torch.int64 and pos.dtype == torch.int64 and pos.numel() == n
    assert xh is None or (xh.shape == x.shape and xh.is_contiguous())
    _check(lib.nvs_embed_sinusoid(_ptr(table), _same(table, xh), _ptr(ids), _ptr(pos), n, width, scale, base, _ptr(x),
                                  _ptr(xh), _stream()))


def norm_residual(x: torch.Tensor, m: torch.Tensor, g: torch.Tensor, eps: float, xh: torch.Tensor | None,
                  m2: torch.Tensor | None = None, w1: torch.Tensor | None = None, w2: torch.Tensor | None = None):
    """x += g * rms(m), or with a second branch x += g * rms((rms(m) w1 + rms(m2) w2) / 2)."""
    lib = load_library()
    n, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and m.shape == x.shape and m.is_contiguous()
    assert m2 is None or (m2.shape == x.shape and m2.is_contiguous() and w1.numel() == width and w2.numel() == width)
    assert xh is None or (xh.shape == x.shape and xh.is_contiguous())
    _check(lib.nvs_norm_residual(_ptr(m), _ptr(m2), _ptr(w1), _ptr(w2), _ptr(g), _same(m, m2, w1, w2, g, xh), n, width, eps,
                                 _ptr(x), _ptr(xh), _stream()))


def scalar_norm_rows(x: torch.Tensor, rows: torch.Tensor | None, nrows: int, g: torch.Tensor, eps: float, out: torch.Tensor):
    lib = load_library()
    assert x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous() and out.shape == (nrows, x.shape[1])
    assert rows is None or (rows.dtype == torch.int32 and rows.numel() >= nrows)
    assert rows is not None or nrows <= x.shape[0]
    _check(lib.nvs_scalar_norm_rows(_ptr(x), _ptr(rows), nrows, x.shape[1], _ptr(g), _same(out, g), eps, _ptr(out), _stream()))


def xielu(z: torch.Tensor, pq: torch.Tensor, beta: float = 0.5) -> torch.Tensor:
    """In place."""
    lib = load_library()
    assert z.is_contiguous() and pq.numel() == 2
    _check(lib.nvs_xielu(_ptr(z), _ptr(pq), beta, _same(z, pq), z.numel(), _ptr(z), _stream()))
    return z


def causal_conv(inp: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None, act: int, por: Portions, state: torch.Tensor,
                out: torch.Tensor):
    """inp: [n, channels] view (unit column stride) of a projection output; state [nslots, taps - 1, channels] fp32; out 32-bit or
    of inp's type."""
    lib = load_library()
    channels, taps = w.shape
    assert inp.shape == (por.n, channels) and inp.stride(1) == 1 and w.is_contiguous()
    assert state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (taps - 1, channels)
    assert out.dtype in (torch.float32, inp.dtype) and out.is_contiguous() and out.shape == (por.n, channels)
    _check(lib.nvs_causal_conv(_ptr(inp), inp.stride(0), _same(inp, w, b), _ptr(w), _ptr(b), channels, taps, act, _ptr(por.cu_q),
                               _ptr(por.ctx0), _ptr(por.slot), _ptr(por.tseq), por.nseq, por.n, _ptr(state), _ptr(out), _code(out), _stream()))


def rglru_scan(gates: torch.Tensor, u: torch.Tensor, ypre: torch.Tensor, lam: torch.Tensor, c: float, blocks: int, por: Portions,
               S: torch.Tensor, out: torch.Tensor):
    lib = load_library()
    n, channels = u.shape
    bw = channels // blocks
    assert n == por.n and gates.dtype == torch.float32 and gates.is_contiguous() and gates.shape == (blocks, n, 2 * bw)
    assert u.dtype == torch.float32 and u.is_contiguous() and ypre.shape == (n, channels) and ypre.stride(1) == 1
    assert S.dtype == torch.float32 and S.is_contiguous() and S.shape[1] == channels and lam.numel() == channels
    assert out.shape == (n, channels) and out.is_contiguous()
    need = 0 if torch.cuda.is_current_stream_capturing() else lib.nvs_rglru_scan_workspace(channels, por.nseq, por.max_q)
    ws = torch.empty(need, dtype=torch.float32, device=u.device) if need else None
    _check(lib.nvs_rglru_scan(_ptr(gates), _ptr(u), _ptr(ypre), ypre.stride(0), _same(ypre, lam, out), _ptr(lam), c, channels,
                              blocks, _ptr(por.cu_q), _ptr(por.ctx0), _ptr(por.slot), por.nseq, n, por.max_q, _ptr(S), _ptr(out), _ptr(ws), need,
                              _stream()))


def ssd_scan(xbc: torch.Tensor, proj: torch.Tensor, dt_col: int, dt_bias, A_log, D, heads: int, P: int, N: int, G: int,
             por: Portions, S: torch.Tensor, y: torch.Tensor):
    lib = load_library()
    n = por.n
    inner = heads * P
    assert xbc.dtype == torch.float32 and xbc.is_contiguous() and xbc.shape == (n, inner + 2 * G * N)
    assert proj.shape[0] == n and proj.stride(1) == 1 and dt_col + heads <= proj.shape[1]
    assert S.dtype == torch.float32 and S.is_contiguous() and tuple(S.shape[1:]) == (heads, P, N)
    assert y.dtype == torch.float32 and y.is_contiguous() and y.shape == (n, inner)
    assert dt_bias.numel() == heads and A_log.numel() == heads and D.numel() == heads
    need = 0 if torch.cuda.is_current_stream_capturing() else lib.nvs_ssd_scan_workspace(heads, P, N, por.nseq, por.max_q)
    ws = torch.empty(need, dtype=torch.float32, device=xbc.device) if need else None
    _check(lib.nvs_ssd_scan(_ptr(xbc), _ptr(proj), proj.stride(0), dt_col, _same(proj, dt_bias, A_log, D), _ptr(dt_bias),
                            _ptr(A_log), _ptr(D), heads, P, N, G, _ptr(por.cu_q), _ptr(por.ctx0), _ptr(por.slot), por.nseq, n,
                            por.max_q, _ptr(S), _ptr(y), _ptr(ws), need, _stream()))


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, w: torch.Tensor, groups: int, eps: float, out: torch.Tensor,
                     norm_first: bool = False, den: torch.Tensor | None = None):
    """out = group_rms(y * silu(z)) * w, or with norm_first group_rms(y) * w * sigmoid(z); den [n, groups] (32-bit, norm_first only):
    group g of row t is divided by den[t, g] before anything else."""
    lib = load_library()
    n, inner = y.shape
    assert y.dtype == torch.float32 and y.is_contiguous() and z.shape == (n, inner) and z.stride(1) == 1
    assert w.numel() == inner and out.shape == (n, inner) and out.is_contiguous()
    assert den is None or (norm_first and den.dtype == torch.float32 and den.shape == (n, groups) and den.is_contiguous())
    _check(lib.nvs_gated_group_norm(_ptr(y), _ptr(z), z.stride(0), _same(z, w, out), _ptr(w), inner, groups, eps, int(norm_first), n,
                                    _ptr(den), _ptr(out), _stream()))


def _rotation(rot_freq: torch.Tensor | None) -> int:
    if rot_freq is None:
        return 0
    assert rot_freq.dtype == torch.float32 and rot_freq.is_contiguous() and rot_freq.is_cuda
    return 2 * rot_freq.numel()


def knorm_kvstore(k: torch.Tensor, v: torch.Tensor, knorm: torch.Tensor | None, eps: float, G: int, d: int, dv: int,
                  block_size: int, slots: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  pos: torch.Tensor | None = None, rot_freq: torch.Tensor | None = None):
    """k [n, G*d], v [n, G*dv]: column ranges of ONE projection output (same row stride). v_cache has the shape
    [pages * block_size, G, dv] but is laid out [page][G][dv][block_size] (see include/nvl_seq.h)."""
    assert k_cache.shape[0] % block_size == 0
    lib = load_library()
    n = k.shape[0]
    assert k.shape == (n, G * d) and v.shape == (n, G * dv) and k.stride(1) == 1 and v.stride(1) == 1 and k.stride(0) == v.stride(0)
    assert slots.dtype == torch.int32 and slots.numel() >= n
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert tuple(k_cache.shape[1:]) == (G, d) and tuple(v_cache.shape[1:]) == (G, dv)
    assert rot_freq is None or (pos is not None and pos.dtype == torch.int64 and pos.numel() >= n and pos.is_contiguous())
    _check(lib.nvs_knorm_kvstore(_ptr(k), _ptr(v), k.stride(0), _same(k, v, knorm, k_cache, v_cache), _ptr(knorm), eps, G, d, dv,
                                 block_size, _ptr(slots), _ptr(pos) if rot_freq is not None else None, _ptr(rot_freq),
                                 _rotation(rot_freq), n, _ptr(k_cache), _ptr(v_cache), _stream()))


def window_attn(q: torch.Tensor, qnorm: torch.Tensor | None, eps: float, gate: torch.Tensor | None, k_cache, v_cache,
                block_tables: torch.Tensor, block_size: int, por: Portions, H: int, G: int, d: int, dv: int, scale: float,
                window: int, out: torch.Tensor, chunk: int = 0, rot_freq: torch.Tensor | None = None, gate_per_head: bool = False,
                sink: torch.Tensor | None = None, q_temp: tuple[float, int] | None = None):
    """window > 0: the last `window` positions; chunk > 0: the query's own block of `chunk` positions; neither: causal.
    rot_freq [r / 2] (32-bit): the first r entries of every query head turn in interleaved pairs by position * rot_freq.
    gate [n, H * dv], or [n, H] with gate_per_head: out *= sigmoid(gate). sink [H] (32-bit): head h's softmax denominator also holds
    exp(sink[h]). q_temp (coef, every): the query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)."""
    lib = load_library()
    n = por.n
    assert q.shape == (n, H * d) and q.stride(1) == 1 and out.shape == (n, H * dv) and out.is_contiguous()
    assert gate is None or (gate.shape == (n, H if gate_per_head else H * dv) and gate.stride(1) == 1)
    assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1 and block_tables.shape[0] >= por.nseq
    assert tuple(k_cache.shape[1:]) == (G, d) and tuple(v_cache.shape[1:]) == (G, dv)
    assert sink is None or (sink.dtype == torch.float32 and sink.numel() == H and sink.is_contiguous() and sink.is_cuda)
    qt_coef, qt_every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 0)
    _check(lib.nvs_window_attn(_ptr(q), q.stride(0), _ptr(qnorm), eps, _ptr(gate), gate.stride(0) if gate is not None else 0,
                               int(gate_per_head), _same(q, qnorm, gate, k_cache, v_cache, out), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
                               block_tables.stride(0), block_size, _ptr(por.cu_q), _ptr(por.ctx0), _ptr(por.tseq), por.nseq, n, H,
                               G, d, dv, scale, window, chunk, _ptr(rot_freq), _rotation(rot_freq), _ptr(sink), qt_coef, qt_every, _ptr(out),
                               _stream()))


def add_group_norm(x: torch.Tensor, w: torch.Tensor | None, groups: int, eps: float, out: torch.Tensor | None,
                   a: torch.Tensor | None = None, b: torch.Tensor | None = None, a_mult: float = 1.0, center: bool = False):
    """x += a_mult * a + b (in place; a in the activation type, b 32-bit, both optional), then out = group_rms(x) * w (out None:
    adds only); center: every group's mean is taken off first (layer norm without bias)."""
    lib = load_library()
    n, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert a is None or (a.shape == x.shape and a.is_contiguous())
    assert b is None or (b.shape == x.shape and b.is_contiguous() and b.dtype == torch.float32)
    assert out is None or (out.shape == x.shape and out.is_contiguous() and w is not None and w.numel() == width)
    ref = out if out is not None else a
    assert ref is not None, "nothing to do"
    _check(lib.nvs_add_group_norm(_ptr(x), _ptr(a), a_mult, _ptr(b), None, n, _ptr(w) if out is not None else None, _same(ref, a, w, out),
                                  width, groups, eps, int(center), _ptr(out), _stream()))


def group_norm_rows(x: torch.Tensor, rows: torch.Tensor | None, nrows: int, w: torch.Tensor, groups: int, eps: float, out: torch.Tensor,
                    center: bool = False):
    """out[r] = group_rms(x[rows[r]]) * w (rows None: row r); center: as add_group_norm."""
    lib = load_library()
    assert x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous() and out.shape == (nrows, x.shape[1])
    assert rows is None or (rows.dtype == torch.int32 and rows.numel() >= nrows)
    assert rows is not None or nrows <= x.shape[0]
    _check(lib.nvs_add_group_norm(_ptr(x), None, 1.0, None, _ptr(rows), nrows, _ptr(w), _same(out, w), x.shape[1], groups, eps, int(center),
                                  _ptr(out), _stream()))


def sandwich_norm(x: torch.Tensor, a: torch.Tensor | None, wa: torch.Tensor | None, w: torch.Tensor | None, eps: float,
                  out: torch.Tensor | None, a2: torch.Tensor | None = None, a_mult: float = 1.0, a2_mult: float = 1.0, w_off: float = 1.0):
    """x += rms(a_mult * a + a2_mult * a2) * (w_off + wa) (in place; a None: no add), then out = rms(x) * (w_off + w) (out None: no
    second norm)."""
    lib = load_library()
    n, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert a is None or (a.shape == x.shape and a.is_contiguous() and wa is not None and wa.numel() == width)
    assert a2 is None or (a is not None and a2.shape == x.shape and a2.is_contiguous())
    assert out is None or (out.shape == x.shape and out.is_contiguous() and w is not None and w.numel() == width)
    ref = out if out is not None else a
    assert ref is not None, "nothing to do"
    _check(lib.nvs_sandwich_norm(_ptr(x), _ptr(a), a_mult, _ptr(a2), a2_mult, _ptr(wa) if a is not None else None, None, n,
                                 _ptr(w) if out is not None else None, w_off, _same(ref, a, a2, wa if a is not None else None,
                                                                                   w if out is not None else None, out), width, eps, _ptr(out), _stream()))


def offset_norm_rows(x: torch.Tensor, rows: torch.Tensor | None, nrows: int, w: torch.Tensor, eps: float, out: torch.Tensor, w_off: float = 1.0):
    """out[r] = rms(x[rows[r]]) * (w_off + w) (rows None: row r)."""
    lib = load_library()
    assert x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous() and out.shape == (nrows, x.shape[1])
    assert rows is None or (rows.dtype == torch.int32 and rows.numel() >= nrows)
    assert rows is not None or nrows <= x.shape[0]
    _check(lib.nvs_sandwich_norm(_ptr(x), None, 1.0, None, 1.0, None, _ptr(rows), nrows, _ptr(w), w_off, _same(out, w), x.shape[1], eps,
                                 _ptr(out), _stream()))


def gated_memory_scan(proj: torch.Tensor, v_col: int, k_col: int, q_col: int, i_col: int, f_col: int, i_bias: torch.Tensor,
                      f_bias: torch.Tensor, cap: float, q_scale: float, heads: int, dk: int, dv: int, por: Portions, S: torch.Tensor,
                      M: torch.Tensor, y: torch.Tensor, den: torch.Tensor):
    """The matrix memory with exponential gates (see include/nvl_seq.h): S [nslots, heads, dv + 1, dk] and M [nslots, heads] are the
    state; y [n, heads * dv] receives the numerators, den [n, heads] the divisors."""
    lib = load_library()
    n = por.n
    assert proj.shape[0] == n and proj.stride(1) == 1 and i_bias.numel() == heads and f_bias.numel() == heads
    assert S.dtype == torch.float32 and S.is_contiguous() and tuple(S.shape[1:]) == (heads, dv + 1, dk)
    assert M.dtype == torch.float32 and M.is_contiguous() and tuple(M.shape[1:]) == (heads,) and M.shape[0] == S.shape[0]
    assert y.dtype == torch.float32 and y.is_contiguous() and y.shape == (n, heads * dv)
    assert den.dtype == torch.float32 and den.is_contiguous() and den.shape == (n, heads)
    need = 0 if torch.cuda.is_current_stream_capturing() else lib.nvs_gated_memory_scan_workspace(heads, dk, dv, por.nseq, por.max_q)
    ws = torch.empty(need, dtype=torch.float32, device=proj.device) if need else None
    _check(lib.nvs_gated_memory_scan(_ptr(proj), proj.stride(0), v_col, k_col, q_col, i_col, f_col, _same(proj, i_bias, f_bias), _ptr(i_bias),
                                     _ptr(f_bias), cap, q_scale, heads, dk, dv, _ptr(por.cu_q), _ptr(por.ctx0), _ptr(por.slot), por.nseq, n,
                                     por.max_q, _ptr(S), _ptr(M), _ptr(y), _ptr(den), _ptr(ws), need, _stream()))


def scale_softcap(logits: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
    """32-bit cap * tanh(logits * scale / cap) (cap <= 0: logits * scale)."""
    lib = load_library()
    assert logits.is_contiguous()
    out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    _check(lib.nvs_scale_softcap(_ptr(logits), _code(logits), scale, cap, logits.numel(), _ptr(out), _stream()))
    return out


class Rotation:
    """How the leading `dims` entries of a vector turn with the position: 32-bit frequencies of the pairs (device), the pairing
    ((2i, 2i+1), or (i, i + dims / 2) with `halves`) and a factor on cos and sin."""
    __slots__ = ("freq", "dims", "halves", "mag")

    def __init__(self, freq: torch.Tensor, halves: bool = False, mag: float = 1.0):
        assert freq.dtype == torch.float32 and freq.is_contiguous()
        self.freq, self.dims, self.halves, self.mag = freq, 2 * freq.numel(), bool(halves), float(mag)


def latent_prep(proj: torch.Tensor, q_col: int, q_rank: int, q_norm: torch.Tensor, cq: torch.Tensor, eps: float, kv_col: int = -1,
                kv_rank: int = 0, rot_dim: int = 0, kv_norm: torch.Tensor | None = None, pos: torch.Tensor | None = None,
                rot: Rotation | None = None, block_size: int = 0, slots: torch.Tensor | None = None, k_cache: torch.Tensor | None = None,
                v_cache: torch.Tensor | None = None):
    """Norms of the query latent (-> cq [n, q_rank]) and, with kv_col >= 0, of the key/value latent, the rotation of the shared key
    part and the store of both into the paged cache: k_cache [slots, 1, kv_rank + rot_dim], v_cache [slots, 1, kv_rank] (the
    latent again, page-transposed like every value cache)."""
    lib = load_library()
    n = proj.shape[0]
    assert proj.stride(1) == 1 and cq.shape == (n, q_rank) and cq.is_contiguous() and q_norm.numel() == q_rank
    if kv_col >= 0:
        assert kv_norm.numel() == kv_rank and slots.dtype == torch.int32 and slots.numel() >= n
        assert pos.dtype == torch.int64 and pos.numel() >= n and pos.is_contiguous()
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape[0] % block_size == 0
        assert tuple(k_cache.shape[1:]) == (1, kv_rank + rot_dim) and tuple(v_cache.shape[1:]) == (1, kv_rank)
        assert rot is None or (rot.freq.is_cuda and rot.dims <= rot_dim)
    _check(lib.nvs_latent_prep(_ptr(proj), proj.stride(0), _same(proj, q_norm, cq, kv_norm, k_cache, v_cache), q_col, q_rank, _ptr(q_norm),
                               _ptr(cq), kv_col, kv_rank, rot_dim, _ptr(kv_norm), _ptr(pos), _ptr(rot.freq) if rot else None,
                               rot.dims if rot else 0, int(rot.halves) if rot else 0, rot.mag if rot else 1.0, eps, block_size, _ptr(slots),
                               _ptr(k_cache), _ptr(v_cache), n, _stream()))


def rotate_heads(inp: torch.Tensor, out: torch.Tensor, pos: torch.Tensor, rot: Rotation | None):
    """inp, out [n, H, width] views (unit stride along the last axis): out = inp with the leading rot.dims entries of every head rotated."""
    lib = load_library()
    n, H, width = inp.shape
    assert out.shape == inp.shape and inp.stride(2) == 1 and out.stride(2) == 1 and pos.dtype == torch.int64 and pos.numel() >= n
    assert rot is None or rot.dims <= width
    _check(lib.nvs_rotate_heads(_ptr(inp), inp.stride(0), inp.stride(1), _ptr(out), out.stride(0), out.stride(1), _same(inp, out), H, width,
                                _ptr(pos), _ptr(rot.freq) if rot else None, rot.dims if rot else 0, int(rot.halves) if rot else 0,
                                rot.mag if rot else 1.0, n, _stream()))


def decay_scan(proj: torch.Tensor, v_col: int, k_col: int, q_col: int, decay: torch.Tensor, heads: int, dk: int, dv: int,
               por: Portions, S: torch.Tensor, y: torch.Tensor):
    """Per head S = decay S + k v^T, y = S^T q on SiLU of the named columns of proj; S [nslots, heads, dv, dk], y [n, heads * dv]."""
    lib = load_library()
    n = por.n
    assert proj.shape[0] == n and proj.stride(1) == 1
    assert decay.dtype == torch.float32 and decay.numel() == heads and decay.is_contiguous()
    assert S.dtype == torch.float32 and S.is_contiguous() and tuple(S.shape[1:]) == (heads, dv, dk)
    assert y.dtype == torch.float32 and y.is_contiguous() and y.shape == (n, heads * dv)
    need = 0 if torch.cuda.is_current_stream_capturing() else lib.nvs_ssd_scan_workspace(heads, dv, dk, por.nseq, por.max_q)
    ws = torch.empty(need, dtype=torch.float32, device=proj.device) if need else None
    _check(lib.nvs_decay_scan(_ptr(proj), proj.stride(0), v_col, k_col, q_col, _code(proj), _ptr(decay), heads, dk, dv, _ptr(por.cu_q),
                              _ptr(por.ctx0), _ptr(por.slot), por.nseq, n, por.max_q, _ptr(S), _ptr(y), _ptr(ws), need, _stream()))


def glu_act(gu: torch.Tensor, ff: int, out: torch.Tensor, kind: int = 0, limit: float = 0.0, alpha: float = 1.0):
    """gu [n, 2 ff] = [gate | up] -> out [n, ff]. kind 0: silu(g) u; kind 1: min(g, limit) sigmoid(alpha g) (clamp(u) + 1);
    kind 2: gu [n, ff], no gate: the tanh form of GELU."""
    lib = load_library()
    n = gu.shape[0]
    assert gu.shape[1] == (1 if kind == 2 else 2) * ff and gu.stride(1) == 1 and out.shape == (n, ff) and out.is_contiguous()
    _check(lib.nvs_glu_act(_ptr(gu), gu.stride(0), _same(gu, out), ff, kind, limit, alpha, n, _ptr(out), _stream()))


def moe_route(z: torch.Tensor, total: int, correction: torch.Tensor | None, top: int, count: int, keep: int, scale: float,
              sigmoid: bool = False, renorm: bool = True):
    """z [n, >= total] 32-bit router logits -> (ids [n, top] int32, weights [n, top] 32-bit). Scores are a softmax over the entries,
    or with `sigmoid` every entry's own sigmoid; weights are the chosen scores, divided by their sum with `renorm`, times scale."""
    lib = load_library()
    n = z.shape[0]
    assert z.dtype == torch.float32 and z.stride(1) == 1 and z.shape[1] >= total
    assert correction is None or (correction.dtype == torch.float32 and correction.numel() == total and correction.is_contiguous())
    ids = torch.empty(n, top, dtype=torch.int32, device=z.device)
    wts = torch.empty(n, top, dtype=torch.float32, device=z.device)
    _check(lib.nvs_moe_route(_ptr(z), z.stride(0), _ptr(correction), n, total, top, count, keep, scale, int(sigmoid), int(renorm), _ptr(ids),
                             _ptr(wts), _stream()))
    return ids, wts


def moe_table_route(tokens: torch.Tensor, table: torch.Tensor, weight: float):
    """tokens [n] int64, table [vocab, top] int32 -> (ids [n, top] = table[tokens], weights [n, top] = weight)."""
    lib = load_library()
    n, top = tokens.numel(), table.shape[1]
    assert tokens.dtype == torch.int64 and tokens.is_contiguous() and table.dtype == torch.int32 and table.is_contiguous()
    ids = torch.empty(n, top, dtype=torch.int32, device=tokens.device)
    wts = torch.empty(n, top, dtype=torch.float32, device=tokens.device)
    _check(lib.nvs_moe_table_route(_ptr(tokens), _ptr(table), n, top, weight, _ptr(ids), _ptr(wts), _stream()))
    return ids, wts


class MoePlan:
    __slots__ = ("tile_expert", "row_token", "pair_row", "cap", "tm")


def moe_plan(ids: torch.Tensor, experts: int, tm: int) -> MoePlan:
    """Pairs (token, choice) sorted by expert into tiles of tm rows (ids >= experts get no row)."""
    lib = load_library()
    n, top = ids.shape
    assert ids.dtype == torch.int32 and ids.is_contiguous()
    p = MoePlan()
    p.tm, p.cap = tm, lib.nvs_moe_rows(n * top, experts, tm)
    p.tile_expert = torch.empty(p.cap // tm, dtype=torch.int32, device=ids.device)
    p.row_token = torch.empty(p.cap, dtype=torch.int32, device=ids.device)
    p.pair_row = torch.empty(n, top, dtype=torch.int32, device=ids.device)
    _check(lib.nvs_moe_plan(_ptr(ids), n, top, experts, tm, _ptr(p.tile_expert), _ptr(p.row_token), _ptr(p.pair_row), _stream()))
    return p


def moe_gemm(x: torch.Tensor, w: torch.Tensor, plan: MoePlan, glu: bool, out: torch.Tensor, relu2: bool = False):
    """glu: w [experts, 2 nout, K], rows gathered by token, out = silu(gate) * up; relu2: w [experts, nout, K], rows gathered by
    token, out = max(w x, 0)^2; neither: w [experts, nout, K], x holds the planned rows."""
    lib = load_library()
    assert not (glu and relu2)
    nout, K = (w.shape[1] // 2 if glu else w.shape[1]), w.shape[2]
    assert w.is_contiguous() and x.stride(1) == 1 and x.shape[1] == K and out.shape == (plan.cap, nout) and out.stride(1) == 1
    assert glu or relu2 or x.shape[0] == plan.cap
    _check(lib.nvs_moe_gemm(_ptr(x), x.stride(0), _ptr(w), _same(x, w, out), 1 if glu else (2 if relu2 else 0), nout, K, _ptr(plan.tile_expert), _ptr(plan.row_token),
                            plan.cap, plan.tm, _ptr(out), out.stride(0), _stream()))


def moe_combine(rows: torch.Tensor, plan: MoePlan, wts: torch.Tensor, h: torch.Tensor, shared: torch.Tensor | None,
                shared_gate: torch.Tensor | None, out: torch.Tensor):
    """out[t] = sum_k wts[t, k] * (row of the pair, or h[t] for a pass-through choice) + sigmoid(shared_gate[t]) * shared[t]."""
    lib = load_library()
    n, width = h.shape
    top = wts.shape[1]
    assert rows.stride(1) == 1 and rows.shape[1] == width and h.stride(1) == 1 and out.shape == (n, width) and out.is_contiguous()
    assert wts.dtype == torch.float32 and wts.is_contiguous() and plan.pair_row.shape == (n, top)
    assert shared is None or (shared.shape == (n, width) and shared.is_contiguous())
    assert shared_gate is None or (shared is not None and shared_gate.dtype == torch.float32 and shared_gate.shape[0] == n)
    _check(lib.nvs_moe_combine(_ptr(rows), rows.stride(0), _ptr(plan.pair_row), _ptr(wts), top, _ptr(h), h.stride(0), _ptr(shared),
                               _ptr(shared_gate), shared_gate.stride(0) if shared_gate is not None else 0, _same(rows, h, shared, out), n,
                               width, _ptr(out), _stream()))
