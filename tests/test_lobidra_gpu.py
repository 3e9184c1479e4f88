"""Lobidra on the GPU against the plain float64 restatement (oracle/lobidra.py): every mechanism alone at the kernel or layer
boundary, then the engine — whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, reused pages
and slots, far keys, sinks, long decoding, greedy generation through LLM.generate(). Configurations and weights are made here;
float32 serving is compared tightly, bfloat16 serving within rounding. Experts are chosen by a table over token ids, so no
choice depends on rounding."""
import json
import math
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import lobidra as plain  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EPS = 1e-5


def dev(t, dtype=None):
    return t.to("cuda", dtype=dtype or t.dtype).contiguous()


def portions(lens, ctx0, slots, max_q=0):
    from nano_vllm_amd.ops_seq import Portions
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tseq = np.repeat(np.arange(len(lens)), lens).astype(np.int32)
    i32 = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device="cuda")
    return Portions(i32(cu), i32(ctx0), i32(slots), i32(tseq), len(lens), int(cu[-1]), max_q)


def close(got, want, tol, what=""):
    got = got.double().cpu().numpy() if hasattr(got, "cpu") else np.asarray(got, dtype=np.float64)
    want = want.double().cpu().numpy() if hasattr(want, "cpu") else np.asarray(want, dtype=np.float64)
    err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-9)
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


def bf(t):
    return t.to(torch.bfloat16)


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("W", [48, 352, 70, 1536, 1])
def test_norms_on_both_sides_of_a_sublayer(dtype, tol, W):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(W)
    n = 7
    x0 = torch.randn(n, W, generator=g) * torch.linspace(0.01, 30, W)
    a, a2 = (3 * torch.randn(n, W, generator=g)).to(dtype), torch.randn(n, W, generator=g).to(dtype)
    wa, w = (0.3 * torch.randn(W, generator=g)).to(dtype), (0.3 * torch.randn(W, generator=g)).to(dtype)
    x, out = dev(x0), torch.empty(n, W, device="cuda", dtype=dtype)
    ops_seq.sandwich_norm(x, None, None, dev(w), EPS, out)
    close(x, x0, 0, "nothing to add")
    close(out, plain.offset_norm(plain.f64(x0), plain.f64(w), EPS), tol, "input norm alone")
    ops_seq.sandwich_norm(x, dev(a), dev(wa), dev(w), EPS, out)
    s = plain.f64(x0) + plain.offset_norm(plain.f64(a), plain.f64(wa), EPS)
    close(x, s, 3e-7, "normed output added")
    close(out, plain.offset_norm(s, plain.f64(w), EPS), tol, "norm after the add")
    ops_seq.sandwich_norm(x, dev(a), dev(wa), None, EPS, None, a2=dev(a2), a_mult=0.6, a2_mult=-1.3)
    s = s + plain.offset_norm(0.6 * plain.f64(a) - 1.3 * plain.f64(a2), plain.f64(wa), EPS)
    close(x, s, 3e-7, "two branches with a scale each")
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device="cuda")
    sel = torch.empty(3, W, device="cuda", dtype=dtype)
    ops_seq.offset_norm_rows(x, rows, 3, dev(w), EPS, sel)
    close(sel, plain.offset_norm(s[[6, 0, 3]], plain.f64(w), EPS), tol, "selected rows")
    ops_seq.sandwich_norm(x, dev(a), dev(wa), None, EPS, None, w_off=0.0)
    close(x, s + plain.rms(plain.f64(a), EPS) * plain.f64(wa), 3e-7, "a weight that is not stored as an offset")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 2.0 ** -8)])
def test_gelu_feed_forward_activation(dtype, tol):
    from nano_vllm_amd import ops_seq
    z = torch.linspace(-9, 9, 33 * 21).view(33, 21).to(dtype)
    wide = torch.cat([z, 7 + 0 * z], dim=1)                                          # a row stride beyond the columns read
    out = torch.empty(33, 21, device="cuda", dtype=dtype)
    ops_seq.glu_act(dev(wide)[:, :21], 21, out, kind=2)
    close(out, plain.gelu_tanh(plain.f64(z)), tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("taps,C", [(3, 40), (1, 7), (4, 300), (8, 64)])
def test_short_convolution_continues_from_its_state(dtype, tol, taps, C):
    """Portions of 1, 2 and more tokens (shorter than the taps too), two sequences interleaved, slots that held other values; the
    output in the activation type, as the attention mixer takes it."""
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(taps * 100 + C)
    T = 40
    u = {s: bf(torch.randn(T, C + 5, generator=g)) for s in "ab"}
    w = bf(torch.randn(C, taps, generator=g))
    want = {s: plain.short_conv(plain.f64(u[s][:, :C]), plain.f64(w)) for s in "ab"}
    state = torch.full((3, max(taps - 1, 0), C), 5.0, device="cuda")
    at, got = {"a": 0, "b": 0}, {"a": [], "b": []}
    for step in ([("a", 1)], [("a", 2), ("b", 1)], [("b", 2), ("a", 1)], [("a", 20), ("b", 1)], [("b", 36), ("a", 16)]):
        rows = torch.cat([u[s][at[s]:at[s] + c] for s, c in step])
        out = torch.empty(rows.shape[0], C, device="cuda", dtype=dtype)
        ops_seq.causal_conv(dev(rows, dtype)[:, :C], dev(w, dtype), None, 0, portions([c for _, c in step], [at[s] for s, _ in step],
                                                                                       [2 if s == "a" else 0 for s, _ in step]), state, out)
        o = 0
        for s, c in step:
            got[s].append(out[o:o + c].float().cpu())
            o, at[s] = o + c, at[s] + c
    assert at == {"a": T, "b": T}
    for s in "ab":
        close(torch.cat(got[s]), want[s], tol, s)


def test_banded_frequencies_follow_the_wavelength():
    from nano_vllm_amd.mixers import banded_rotary_frequencies
    for rot in ROTS:
        if rot:
            close(torch.tensor(banded_rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling")), dtype=torch.float64),
                  plain.banded_frequencies(rot), 1e-13)
    sc = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    f = banded_rotary_frequencies(16, 10000.0, sc)
    f0 = banded_rotary_frequencies(16, 10000.0, None)
    kinds = set()
    for a, b in zip(f, f0):
        wl = 2 * math.pi / b
        kinds.add("kept" if wl < 16 else ("slowed" if wl > 64 else "blend"))
        assert (a == b) if wl < 16 else (a == b / 8 if wl > 64 else b / 8 < a < b)
    assert kinds == {"kept", "slowed", "blend"}


ROTS = [None, {"dims": 8, "base": 100.0}, {"dims": 16, "base": 10000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}},
        {"dims": 24, "base": 500000.0, "scaling": {"factor": 3.0, "low": 2.0, "high": 16.0, "original": 512}}]


def with_context(mix, h, dtype, block, cuts, path="auto", slot=1):
    """The product's mixer on h, cut into portions `cuts` (one sequence, dirty pages in scrambled order, a dirty state slot)."""
    from nano_vllm_amd import ops_seq
    from nano_vllm_amd.attn_meta import reset_context, set_context
    T = h.shape[0]
    pages = -(-T // block)
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(T))[:pages].to(torch.int32)
    for m in mix.modules():
        if hasattr(m, "kv_shapes"):
            ks, vs = m.kv_shapes()
            m.block_size = block
            m.k_cache = torch.full(((pages + 3) * block, *ks), 7.0, device="cuda", dtype=dtype)
            m.v_cache = torch.full(((pages + 3) * block, *vs), -7.0, device="cuda", dtype=dtype)
        if hasattr(m, "state_shapes"):
            for name, shape in m.state_shapes().items():
                setattr(m, name, torch.full((3, *shape), 3.0, device="cuda"))
    ops_seq.load_library().nvs_window_attn_force_scalar({"auto": 0, "scalar": 1, "nolds": 2, "unpacked": 3}[path])
    outs, at = [], 0
    try:
        with torch.inference_mode():
            for c in cuts:
                pos = torch.arange(at, at + c)
                slots = (order[pos // block].long() * block + pos % block).to(torch.int32)
                set_context(True, slot_mapping=dev(slots), block_tables=dev(order.view(1, -1)), portions=portions([c], [at], [slot]))
                out = mix(dev(h[at:at + c], dtype), dev(pos))
                outs.append(out if isinstance(out, tuple) else (out,))
                at += c
    finally:
        reset_context()
        ops_seq.load_library().nvs_window_attn_force_scalar(0)
    assert at == T
    return [torch.cat([o[i].float().cpu() for o in outs]) for i in range(len(outs[0]))]


def build(cls, w, dtype, *args, **kw):
    with torch.inference_mode():
        prev = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            mix = cls(*args, **kw).to("cuda")
        finally:
            torch.set_default_dtype(prev)
        loaders = mix.named_loaders()
        assert set(loaders) == set(w), sorted(set(loaders) ^ set(w))
        for k, fn in loaders.items():
            fn(w[k].to("cuda"))
    return mix


def conv_attention_case(H, G, d, taps, rot, T, seed, W=40):
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "conv": taps, "scale": d ** -0.5}
    if rot:
        m["rot"] = rot
    w = {"q": 2 * rnd(H * d, W) / W ** 0.5, "k": 2 * rnd(G * d, W) / W ** 0.5, "g": 2 * rnd(H, W) / W ** 0.5, "o": rnd(W, H * d) / (H * d) ** 0.5,
         "q.conv": rnd(H * d, taps) / taps ** 0.5, "k.conv": rnd(G * d, taps) / taps ** 0.5}
    return m, {k: bf(v) for k, v in w.items()}, bf(rnd(T, W))


def build_conv_attention(m, w, dtype, block, W=40):
    from nano_vllm_amd.mixers import ConvAttentionMixer, banded_rotary_frequencies
    rot = m.get("rot")
    return build(ConvAttentionMixer, w, dtype, W, m["heads"], m["kv_heads"], m["dim"], m["conv"], m["scale"], EPS, block,
                 rot_dims=rot["dims"] if rot else 0,
                 rot_freqs=banded_rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling")) if rot else None, sink="zero")


@pytest.mark.parametrize("dtype,path,tol", [(torch.float32, "auto", 3e-5), (torch.bfloat16, "auto", 3e-2), (torch.bfloat16, "nolds", 3e-2),
                                            (torch.bfloat16, "scalar", 3e-2), (torch.bfloat16, "unpacked", 3e-2)])
@pytest.mark.parametrize("H,G,d,taps,rot,block", [(4, 2, 16, 3, ROTS[1], 16), (6, 3, 24, 4, ROTS[3], 32), (8, 1, 16, 2, ROTS[2], 64),
                                                  (1, 1, 40, 1, ROTS[0], 16), (20, 2, 8, 3, ROTS[1], 16), (3, 3, 20, 5, ROTS[2], 48),
                                                  (2, 1, 128, 3, ROTS[3], 64)])
def test_conv_attention_against_the_plain_loop(H, G, d, taps, rot, block, dtype, path, tol):
    """One prompt portion, then short portions and single tokens (shorter than the convolution's taps); heads that are no multiple
    of 8 entries wide, one head, 8 and 10 query heads per kv head (single tokens then run with heads packed into the query tiles)."""
    T = 150
    m, w, h = conv_attention_case(H, G, d, taps, rot, T, seed=H * 100 + d)
    want = plain.conv_attention(plain.f64(h), {k: plain.f64(v) for k, v in w.items()}, m)
    for cuts in ([T], [97, 2, 1, 1, 30, 1, 1, 1, 16]):
        close(with_context(build_conv_attention(m, w, dtype, block), h, dtype, block, cuts, path)[0], want, tol, f"cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype,path", [(torch.float32, "auto"), (torch.bfloat16, "auto"), (torch.bfloat16, "nolds"), (torch.bfloat16, "unpacked")])
def test_the_zero_sink_takes_its_share_when_every_score_is_low(dtype, path):
    """Keys that point away from every query: all scores are far below zero, so nearly all of the softmax's mass goes to the sink
    and the output is close to nothing — without the sink the weights would still add up to one. Then scores far above zero: the
    sink's share vanishes."""
    T, H, G, d, W = 70, 8, 1, 16, 16
    m, w, h = conv_attention_case(H, G, d, 1, None, T, seed=5, W=W)
    eye = torch.zeros(d, W)
    eye[:, :d] = torch.eye(d)
    h = bf(2 * torch.ones(T, W) + 0.1 * torch.randn(T, W, generator=torch.Generator().manual_seed(1)))
    for sign in (-1.0, 1.0):
        w["q"], w["k"] = bf(torch.cat([eye] * H)), bf(sign * eye)
        w["q.conv"], w["k.conv"] = bf(torch.ones(H * d, 1)), bf(torch.ones(G * d, 1))
        w["g"] = bf(torch.full((H, W), 0.5))
        w["o"] = bf(torch.cat([torch.eye(W)[:, :d]] * H, dim=1))
        want = plain.conv_attention(plain.f64(h), {k: plain.f64(v) for k, v in w.items()}, m)
        for cuts in ([T], [60] + [1] * 10):
            got = with_context(build_conv_attention(m, w, dtype, 16, W=W), h, dtype, 16, cuts, path)[0]
            close(got, want, 3e-5 if dtype == torch.float32 else 3e-2, f"sign {sign}")
        if sign < 0:
            assert np.abs(want).max() < 0.2                           # (a softmax without the sink would give about 16 here)
        else:
            assert np.abs(want).max() > 4


def memory_case(H, d, dv, cap, T, seed, W=40, i_bias=0.0, f_bias=2.0, gate=2.0):
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}
    w = {"q": 2 * rnd(H * d, W) / W ** 0.5, "k": 2 * rnd(H * d, W) / W ** 0.5, "v": rnd(H * dv, W) / W ** 0.5, "g": rnd(H * dv, W) / W ** 0.5,
         "o": rnd(W, H * dv) / (H * dv) ** 0.5, "norm": 1 + 0.2 * rnd(H * dv), "i": gate * rnd(H, W) / W ** 0.5, "i.b": i_bias + rnd(H),
         "f": gate * rnd(H, W) / W ** 0.5, "f.b": f_bias + rnd(H)}
    return m, {k: bf(v) for k, v in w.items()}, bf(rnd(T, W))


def left_case(H, G, d, dv, q_temp, T, seed, W=40):
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    w = {"q": 2 * rnd(H * d, W) / W ** 0.5, "k": 2 * rnd(G * d, W) / W ** 0.5, "v": rnd(G * dv, W) / W ** 0.5, "g": rnd(H * dv, W) / W ** 0.5,
         "o": rnd(W, H * dv) / (H * dv) ** 0.5, "sink": 2 * rnd(H)}
    return m, {k: bf(v) for k, v in w.items()}


def build_parallel(left, wl, right, wr, dtype, block, W=40):
    from nano_vllm_amd.mixers import AttentionMemoryMixer
    w = {"left." + k: v for k, v in wl.items()}
    w.update({"right." + k: v for k, v in wr.items()})
    return build(AttentionMemoryMixer, w, dtype, W, left, right, EPS, block)


@pytest.mark.parametrize("dtype,path,tol", [(torch.float32, "auto", 3e-5), (torch.bfloat16, "auto", 3e-2), (torch.bfloat16, "scalar", 3e-2),
                                            (torch.bfloat16, "unpacked", 3e-2)])
@pytest.mark.parametrize("left,right,block", [((4, 2, 24, 40, (0.3, 16)), (2, 16, 24, 8.0), 16), ((8, 1, 16, 8, (1.0, 1)), (3, 40, 16, 15.0), 32),
                                              ((2, 2, 8, 8, None), (1, 128, 128, 12.0), 64), ((5, 5, 20, 12, (0.5, 7)), (5, 8, 9, 3.0), 16),
                                              ((1, 1, 64, 64, (0.1, 64)), (2, 64, 20, 30.0), 48)])
def test_attention_beside_the_matrix_memory_against_the_plain_loops(left, right, block, dtype, path, tol):
    """Both halves of the parallel mixer on one fused projection: learned sinks, a temperature that changes every few positions (also
    every position), memory heads whose sizes are no multiples of 16 or of the rows a thread holds, one head, portions of one and
    two tokens through a dirty slot."""
    T = 150
    ml, wl = left_case(*left, T, seed=left[0] * 10 + left[2])
    mr, wr, h = memory_case(*right, T, seed=right[0] * 10 + right[1])
    hh = plain.f64(h)
    want_l = plain.tempered_attention(hh, {k: plain.f64(v) for k, v in wl.items()}, ml)
    want_r = plain.matrix_memory(hh, {k: plain.f64(v) for k, v in wr.items()}, mr, EPS)
    for cuts in ([T], [97, 2, 1, 1, 30, 1, 1, 1, 16], [1] * 20 + [130]):
        got_l, got_r = with_context(build_parallel(ml, wl, mr, wr, dtype, block), h, dtype, block, cuts, path)
        close(got_l, want_l, tol, f"attention, cuts {cuts[:3]}")
        # (bf16: the gates' pre-activations are rounded before they are exponentiated, and the state carries that on)
        close(got_r, want_r, tol if dtype == torch.float32 else 2 * tol, f"memory, cuts {cuts[:3]}")


@pytest.mark.parametrize("i_bias,f_bias,gate", [(9.0, 6.0, 1.0), (-9.0, -6.0, 1.0), (0.0, 0.0, 40.0)])
def test_matrix_memory_gates_at_their_extremes_over_a_long_sequence(i_bias, f_bias, gate):
    """Input gates whose exponentials would overflow without the running maximum, forget gates that keep everything or nearly nothing,
    pre-activations far into the cap's tanh; 700 tokens in one portion and in portions that end inside the kernel's token rounds."""
    T = 700
    mr, wr, h = memory_case(2, 16, 24, 10.0, T, seed=3, i_bias=i_bias, f_bias=f_bias, gate=gate)
    ml, wl = left_case(1, 1, 8, 8, None, T, seed=4)
    want = plain.matrix_memory(plain.f64(h), {k: plain.f64(v) for k, v in wr.items()}, mr, EPS)
    for cuts in ([T], [333, 1, 17, 349]):
        close(with_context(build_parallel(ml, wl, mr, wr, torch.float32, 64), h, torch.float32, 64, cuts)[1], want, 1e-4, f"cuts {cuts[:2]}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_is_found_and_the_temperature_sharpens_it(dtype):
    """One early key is made to stand out for the last queries (a large shared component), 900 positions back and across many
    pages; the temperature (every 64 positions) multiplies its lead. The output must be that key's value, as in the plain model."""
    T, W, d = 960, 32, 16
    ml, wl = left_case(2, 1, d, d, (0.5, 64), T, seed=9, W=W)
    mr, wr, _ = memory_case(1, 8, 8, 10.0, T, seed=9, W=W)
    h = 0.3 * torch.randn(T, W, generator=torch.Generator().manual_seed(10))
    h[:, :2] = 0.0
    h[37, 1] = 2.0                                                    # the far key's mark ...
    h[-30:, 0] = 2.0                                                  # ... and the mark of the queries that look for it
    h = bf(h)
    u, c = torch.ones(d) / d ** 0.5, 6.0 ** 0.5                       # both marks map to the same direction: 6 more score before the temperature
    q, k = wl["q"].float(), wl["k"].float()
    q[:, :2], k[:, :2] = 0.0, 0.0
    q[:, 0], k[:, 1] = torch.cat([u, u]) * c, u * c
    wl["q"], wl["k"] = bf(q), bf(k)
    hh = plain.f64(h)
    want = plain.tempered_attention(hh, {k: plain.f64(v) for k, v in wl.items()}, ml)
    cold = plain.tempered_attention(hh, {k: plain.f64(v) for k, v in wl.items()}, {k: v for k, v in ml.items() if k != "q_temp"})
    assert np.abs(want[-30:] - cold[-30:]).max() > 0.05 * np.abs(want).max(), "the case does not show the temperature"
    for cuts in ([T], [930] + [1] * 30, [100, 2, 500, 330, 2] + [1] * 26):
        got = with_context(build_parallel(ml, wl, mr, wr, dtype, 64, W=W), h, dtype, 64, cuts)[0]
        close(got, want, 3e-5 if dtype == torch.float32 else 3e-2, f"cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("experts,top,ff,shared,n,plain_kernel", [(6, 2, 32, 48, 50, 0), (4, 1, 24, 0, 7, 0), (5, 5, 16, 8, 300, 0), (9, 3, 40, 16, 1500, 0),
                                                                   (6, 2, 32, 48, 50, 1)])
def test_experts_chosen_by_a_table_over_token_ids(dtype, tol, experts, top, ff, shared, n, plain_kernel):
    from nano_vllm_amd import ops_seq
    from nano_vllm_amd.mixers import RoutedExperts
    W, V = 64, 37
    g = torch.Generator().manual_seed(experts * 10 + top)
    rnd = lambda *s: torch.randn(*s, generator=g)
    w = {"table": torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(V)]).to(torch.int32)}
    for e in range(experts):
        w.update({f"e{e}.gate": bf(2 * rnd(ff, W) / W ** 0.5), f"e{e}.up": bf(2 * rnd(ff, W) / W ** 0.5), f"e{e}.down": bf(rnd(W, ff) / ff ** 0.5)})
    if shared:
        w.update({"shared.gate": bf(rnd(shared, W) / W ** 0.5), "shared.up": bf(rnd(shared, W) / W ** 0.5), "shared.down": bf(rnd(W, shared) / shared ** 0.5)})
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}, "shared": {"ff": shared} if shared else None}
    h, toks = bf(rnd(n, W)), torch.randint(0, V, (n,), generator=g)
    want = plain.table_experts(plain.f64(h), toks.numpy(), {k: plain.f64(v) for k, v in w.items()}, mlp)
    mix = build(RoutedExperts, w, dtype, W, experts, ff, top, shared_ff=shared, table_vocab=V, shared_gate=False)
    ops_seq.load_library().nvs_moe_force_plain(plain_kernel)
    try:
        with torch.inference_mode():
            got = mix(dev(h, dtype), dev(toks))
    finally:
        ops_seq.load_library().nvs_moe_force_plain(0)
    close(got, want, tol)


# ---------------------------------------------------------------------------------------------- the engine
def small_config(variant: int) -> dict:
    def att(H, G, d, taps, rot, weights_of=None, mlp=None):
        m = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "conv": taps, "scale": 1.3 * d ** -0.5}
        if rot:
            m["rot"] = rot
        out = {"type": "attention", "mixer": m, "mlp": mlp}
        if weights_of is not None:
            out["weights_of"] = weights_of
        return out

    def par(left, right, scales, weights_of=None, mlp=None):
        H, G, d, dv, qt = left
        a = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5}
        if qt:
            a["q_temp"] = {"coef": qt[0], "every": qt[1]}
        b = {"heads": right[0], "dim": right[1], "vdim": right[2], "gate_cap": right[3]}
        out = {"type": "parallel", "mixer": {"left": a, "right": b, "left_scale": scales[0], "right_scale": scales[1]}, "mlp": mlp}
        if weights_of is not None:
            out["weights_of"] = weights_of
        return out
    dense = lambda ff: {"kind": "dense", "ff": ff}
    moe = lambda e, top, ff, shared: {"kind": "moe", "router": {"experts": e, "top": top}, "expert": {"ff": ff},
                                      **({"shared": {"ff": shared}} if shared else {})}
    if variant == 0:
        a0, p1 = att(4, 2, 16, 4, ROTS[2], mlp=dense(160)), par((4, 1, 24, 40, (0.3, 16)), (2, 16, 24, 8.0), (0.7, 1.1), mlp=moe(6, 2, 32, 48))
        layers = [a0, p1, dict(a0, weights_of=0), dict(p1, weights_of=1)]
        return {"architecture": "Lobidra", "vocab": 200, "width": 96, "layers": layers, "norm": {"eps": 1e-5}, "embedding": {"scale": 9.0}}
    if variant == 1:
        layers = [par((2, 2, 8, 8, None), (3, 40, 16, 15.0), (1.0, 0.5)), att(1, 1, 32, 2, None, mlp=moe(4, 1, 24, 0)),
                  att(8, 1, 16, 1, ROTS[1], mlp=dense(72))]
        return {"architecture": "Lobidra", "vocab": 150, "width": 128, "layers": layers, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}}
    a0 = att(6, 3, 24, 3, ROTS[3], mlp=moe(5, 3, 16, 40))
    layers = [a0, dict(a0, weights_of=0), dict(a0, weights_of=0), par((3, 3, 16, 16, (1.0, 5)), (1, 24, 40, 6.0), (1.0, 1.0), mlp=dense(64))]
    return {"architecture": "Lobidra", "vocab": 96, "width": 64, "layers": layers, "norm": {"eps": 1e-3}, "embedding": {"scale": 3.0}}


@pytest.fixture(scope="module")
def checkpoints():
    from nano_vllm_amd.lobidra import write_synthetic_checkpoint
    root = tempfile.mkdtemp(prefix="lbd_")
    return [write_synthetic_checkpoint(os.path.join(root, f"m{v}"), small_config(v), seed=41 + v) for v in range(3)]


def engine(path, dtype="float32", pages=40, page=16, live=4, **kw):
    from nano_vllm_amd import LLM
    kw.setdefault("enforce_eager", True)
    kw.setdefault("max_num_batched_tokens", 1024)
    kw.setdefault("max_model_len", 640)
    return LLM(path, dtype=dtype, kvcache_block_size=page, num_kvcache_blocks=pages, max_num_seqs=live, **kw)


def rel(got, want, scale):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / scale)


TOL = {"float32": 5e-5, "bfloat16": 4e-2}


def test_checkpoint_names_and_loaders_agree_and_a_layer_with_borrowed_weights_has_its_own_cache(checkpoints):
    from nano_vllm_amd.lobidra import tensor_shapes
    llm = engine(checkpoints[0])
    try:
        model = llm.model_runner.model
        assert set(model.named_loaders()) == set(tensor_shapes(small_config(0)))
        assert not any(n.startswith(("l2.", "l3.")) for n in model.named_loaders())
        a, b = model.layers[0], model.layers[2]
        assert b.mixer.in_w is a.mixer.in_w and b.norm1b is a.norm1b and b.mlp.up is a.mlp.up
        assert b.mixer.attn.k_cache is not a.mixer.attn.k_cache and b.mixer.conv_state is not a.mixer.conv_state
        p, q = model.layers[1], model.layers[3]
        assert q.mixer.attn.sink is p.mixer.attn.sink and q.mixer.mem.rec_state is not p.mixer.mem.rec_state
        assert q.mixer.mem.max_state.shape == (5, 2) and p.mixer.mem.rec_state.shape == (5, 2, 25, 16)
    finally:
        llm.exit()


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_decoding_agree_with_the_plain_model(checkpoints, variant, dtype):
    path = checkpoints[variant]
    ref = plain.Model.load(path)
    toks = torch.randint(0, ref.cfg["vocab"], (150,), generator=torch.Generator().manual_seed(variant)).tolist()
    layers = []
    want = ref.run(toks, layers)
    scale = float(want.std())
    llm = engine(path, dtype)
    try:
        model = llm.model_runner.model
        model.layer_trace = []
        whole = llm.replay_step([{"id": "w", "tokens": toks, "want": list(range(150))}], ["w"])
        seen, model.layer_trace = model.layer_trace, None
        assert len(seen) == len(ref.cfg["layers"])
        if dtype == "float32":                                       # layer by layer, in 32-bit
            for i, x in enumerate(seen):
                close(x, layers[i], 2e-5, f"residual after layer {i}")
        assert rel(whole, want, scale) <= TOL[dtype]
        # portions of changing size, down to two tokens and single tokens, cut inside pages and token rounds
        for name, cuts in (("a", [2, 3, 2, 40, 1, 1, 17, 2, 64, 18]), ("b", [149, 1]), ("c", [1] * 60 + [90]), ("d", [2] * 75)):
            at, rows = 0, []
            for c in cuts:
                rows.append(llm.replay_step([{"id": name, "tokens": toks[at:at + c], "want": list(range(c))}],
                                            [name] if at + c == 150 else []))
                at += c
            assert at == 150 and rel(np.concatenate(rows), want, scale) <= TOL[dtype], name
            if dtype == "float32":
                assert rel(np.concatenate(rows), whole, scale) <= 2e-5, "portions against the whole prompt"
        assert llm.scheduler.block_manager.num_free == 40 and llm.scheduler.state_slots.num_free == 4
    finally:
        llm.exit()


def test_unequal_requests_in_one_batch_equal_each_alone_with_pages_and_slots_reused(checkpoints):
    """Five requests through four slots and a pool that cannot hold them all at once: prompts in portions beside single tokens
    of others, requests that sit out steps, ends that free pages and slots for the next request."""
    path = checkpoints[0]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(4)
    lens = {"p": 130, "q": 61, "r": 3, "s": 97, "t": 200}
    toks = {k: torch.randint(0, ref.cfg["vocab"], (n,), generator=g).tolist() for k, n in lens.items()}
    want = {k: ref.run(v) for k, v in toks.items()}
    scale = float(want["p"].std())
    llm = engine(path, "float32", pages=28)                          # 448 token places for 491 tokens
    try:
        plan = [[("p", 50), ("q", 2)], [("p", 1), ("q", 30), ("r", 3)], [("p", 1), ("s", 64)], [("q", 29), ("p", 2), ("s", 1)],
                [("p", 76), ("s", 32)], [("t", 128)], [("t", 2)], [("t", 1)], [("t", 69)]]
        at = {k: 0 for k in lens}
        got = {k: [] for k in lens}
        used_slots = {}
        for step in plan:
            entries, end = [], []
            for k, c in step:
                entries.append({"id": k, "tokens": toks[k][at[k]:at[k] + c], "want": list(range(c))})
                at[k] += c
                if at[k] == lens[k]:
                    end.append(k)
            out = llm.replay_step(entries, end)
            o = 0
            for k, c in step:
                got[k].append(out[o:o + c])
                o += c
            for k, _ in step:
                if k in llm._replay:
                    used_slots[k] = llm._replay[k].state_slot
        assert at == lens
        for k in lens:
            assert rel(np.concatenate(got[k]), want[k], scale) <= 5e-5, k
        assert used_slots["s"] == 2 and used_slots["t"] == 0, "freed slots are handed out again, lowest first"
        assert llm.scheduler.block_manager.num_free == 28 and llm.scheduler.state_slots.num_free == 4
    finally:
        llm.exit()


@pytest.mark.parametrize("variant", [0, 1])
def test_a_long_portion_scanned_in_segments_beside_a_short_one(checkpoints, variant):
    """600 tokens in one step: the matrix memory cuts such a portion into segments that are scanned twice; the request beside it
    has one segment. The decoded tokens after it continue from the state the segmented pass left."""
    path = checkpoints[variant]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(21)
    long, short = (torch.randint(0, ref.cfg["vocab"], (n,), generator=g).tolist() for n in (604, 9))
    wl, ws = ref.run(long), ref.run(short)
    scale = float(wl.std())
    llm = engine(path, "float32", pages=42)
    try:
        out = llm.replay_step([{"id": "l", "tokens": long[:600], "want": [0, 300, 511, 512, 599]}, {"id": "s", "tokens": short[:5], "want": [4]}])
        assert rel(out[:5], wl[[0, 300, 511, 512, 599]], scale) <= 5e-5 and rel(out[5:], ws[[4]], scale) <= 5e-5
        for i in range(4):
            out = llm.replay_step([{"id": "s", "tokens": [short[5 + i]], "want": [0]}, {"id": "l", "tokens": [long[600 + i]], "want": [0]}])
            assert rel(out[:1], ws[[5 + i]], scale) <= 5e-5 and rel(out[1:], wl[[600 + i]], scale) <= 5e-5, i
    finally:
        llm.exit()


def test_long_decoding_across_many_pages(checkpoints):
    path = checkpoints[2]
    ref = plain.Model.load(path)
    toks = torch.randint(0, ref.cfg["vocab"], (330,), generator=torch.Generator().manual_seed(8)).tolist()
    want = ref.run(toks)
    llm = engine(path, "float32", pages=24)
    try:
        rows = [llm.replay_step([{"id": 0, "tokens": toks[:10], "want": list(range(10))}])]
        rows += [llm.replay_step([{"id": 0, "tokens": [t], "want": [0]}]) for t in toks[10:]]
        assert rel(np.concatenate(rows), want, float(want.std())) <= 5e-5
    finally:
        llm.exit()


@pytest.mark.parametrize("eager", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_generate_matches_the_plain_model(checkpoints, dtype, eager):
    """LLM.generate() with token-id prompts: scheduler, chunked prefill, block manager, slots, sampler; eagerly and with decode
    steps replayed from captured graphs. Where the plain model's two best logits are a close call the comparison stops."""
    from nano_vllm_amd import SamplingParams
    path = checkpoints[0]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, ref.cfg["vocab"], (n,), generator=g).tolist() for n in (5, 70, 31)]
    llm = engine(path, dtype, pages=30, enforce_eager=eager, max_num_batched_tokens=48)      # prompts are prefilled in chunks
    try:
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True), use_tqdm=False)
        assert eager or llm.model_runner.sgraphs, "decode steps were meant to replay graphs"
        assert llm.scheduler.block_manager.num_free == 30 and llm.scheduler.state_slots.num_free == 4
    finally:
        llm.exit()
    margin = 0.05 if dtype == "float32" else 0.15      # (the sampler reads bf16 logits in both)
    checked = 0
    for prompt, o in zip(prompts, outs):
        gen = o["token_ids"]
        assert len(gen) == 24
        logits = ref.run(prompt + gen[:-1])[len(prompt) - 1:]
        for t, row in zip(gen, logits):
            best = np.sort(row)[-2:]
            if float(best[1] - best[0]) > margin * float(row.std()):
                assert t == int(row.argmax())
                checked += 1
    assert checked >= 30


def test_preemption_recomputes_and_a_sampled_run_repeats_itself(checkpoints):
    from nano_vllm_amd import SamplingParams
    path = checkpoints[1]
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 150, (n,), generator=g).tolist() for n in (30, 31, 29, 17)]
    greedy = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    outs = []
    for pages in (40, 11):
        llm = engine(path, "float32", pages=pages, max_num_batched_tokens=256, max_model_len=128)
        try:
            outs.append([o["token_ids"] for o in llm.generate(prompts, greedy, use_tqdm=False)])
        finally:
            llm.exit()
    assert outs[0] == outs[1]
    warm = []
    for _ in range(2):
        llm = engine(path, "bfloat16", pages=40, max_num_batched_tokens=256, max_model_len=128)
        try:
            warm.append([o["token_ids"] for o in llm.generate(prompts, SamplingParams(temperature=0.8, max_tokens=16, ignore_eos=True),
                                                               use_tqdm=False)])
        finally:
            llm.exit()
    assert warm[0] == warm[1] and warm[0] != [o[:16] for o in outs[0]]


def test_the_schedule_replayer_as_a_program(checkpoints, tmp_path):
    path = checkpoints[2]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(12)
    a, b = (torch.randint(0, ref.cfg["vocab"], (n,), generator=g).tolist() for n in (90, 41))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:64], "want": [0, 63]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[64:66], "want": []}, {"id": "b", "tokens": b[:40], "want": [39]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[40:], "want": [0]}, {"id": "a", "tokens": a[66:], "want": [23]}], "end": ["a", "b"]}]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                          timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = ref.run(a), ref.run(b)
    scale = float(wa.std())
    got = [np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, ref.cfg["vocab"]) for i in range(3)]
    assert rel(got[0], wa[[0, 63]], scale) <= 5e-5 and rel(got[1], wb[[39]], scale) <= 5e-5
    assert rel(got[2], np.stack([wb[40], wa[89]]), scale) <= 5e-5
