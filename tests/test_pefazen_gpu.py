"""Pefazen on the GPU against the plain float64 restatement (oracle/pefazen.py): every mechanism alone at the kernel or layer
boundary, then the engine — whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, reused
pages and slots, window edges, far keys, long decoding, greedy generation through LLM.generate(). Configurations and
weights are made here; float32 serving is compared tightly, bfloat16 serving within rounding.

Routing is a discrete choice: in bfloat16 serving the router sees a rounded input and a near-tie may fall the other way
than in the oracle. The mechanism tests leave out tokens whose choice is a close call, and the bfloat16 ENGINE tests use
corrections that decide the choice by themselves (the weights still vary from token to token)."""
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

from oracle import pefazen as plain  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


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


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("W", [48, 352, 70, 1536, 1])
def test_centered_norm_with_the_scaled_add_before_it(dtype, tol, W):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(W)
    n, eps, m = 7, 1e-3, 0.37
    x0 = torch.randn(n, W, generator=g) * torch.linspace(0.01, 30, W) + 11.0        # a mean far from zero
    a = torch.randn(n, W, generator=g).to(dtype)
    w = (1 + 0.3 * torch.randn(W, generator=g)).to(dtype)
    x, out = dev(x0), torch.empty(n, W, device="cuda", dtype=dtype)
    ops_seq.add_group_norm(x, dev(w), 1, eps, out, center=True)
    close(x, x0, 0, "nothing to add")
    close(out, plain.layer_norm(plain.f64(x0), plain.f64(w), eps), tol, "norm alone")
    ops_seq.add_group_norm(x, dev(w), 1, eps, out, a=dev(a), a_mult=m, center=True)
    s = plain.f64(x0) + m * plain.f64(a)
    close(x, s, 3e-7, "residual sum")
    close(out, plain.layer_norm(s, plain.f64(w), eps), tol, "norm after the add")
    ops_seq.add_group_norm(x, None, 1, eps, None, a=dev(a), a_mult=-2.0)
    close(x, s - 2.0 * plain.f64(a), 3e-7, "add alone")
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device="cuda")
    sel = torch.empty(3, W, device="cuda", dtype=dtype)
    ops_seq.group_norm_rows(x, rows, 3, dev(w), 1, eps, sel, center=True)
    close(sel, plain.layer_norm((s - 2.0 * plain.f64(a))[[6, 0, 3]], plain.f64(w), eps), tol, "selected rows")


def test_logit_scale_and_cap():
    from nano_vllm_amd import ops_seq
    z = torch.linspace(-90, 90, 77 * 13).view(77, 13)
    for dtype in (torch.float32, torch.bfloat16):
        zz = z.to(dtype)
        close(ops_seq.scale_softcap(dev(zz), 0.4, 12.0), 12.0 * np.tanh(plain.f64(zz) * 0.4 / 12.0), 2e-6, "capped")
        close(ops_seq.scale_softcap(dev(zz), 3.0, 0.0), plain.f64(zz) * 3.0, 1e-7, "no cap")


ROTS = [{"dims": 16, "base": 30000.0}, {"dims": 8, "base": 100.0},
        {"dims": 32, "base": 200000.0, "scaling": {"factor": 3.0, "original": 256, "fast": 24.0, "slow": 2.0}},
        {"dims": 12, "base": 3000.0, "scaling": {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 0.5}}]


@pytest.mark.parametrize("rot", ROTS)
@pytest.mark.parametrize("halves", [False, True])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2.0 ** -8)])
def test_rotation_of_query_heads_both_pairings_scaled_frequencies_far_positions(rot, halves, dtype, tol):
    """Positions up to 5000: the angle is a 32-bit product, so the result may differ from float64 by the rounding of the angle
    (1e-7 of it); entries behind the rotated ones pass unchanged."""
    from nano_vllm_amd import ops_seq
    from nano_vllm_amd.mixers import rotary_frequencies
    H, extra, lead = 3, 6, 10
    width = rot["dims"] + extra
    g = torch.Generator().manual_seed(rot["dims"])
    pos = torch.tensor([0, 1, 2, 63, 64, 511, 512, 1999, 5000])
    src = torch.randn(len(pos), H, lead + width, generator=g).to(dtype)
    freq, mag = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    rfreq, rmag = plain.rotary_table(rot)
    close(torch.tensor(freq, dtype=torch.float64), rfreq, 1e-12, "frequencies")
    assert abs(mag - rmag) < 1e-12 and (mag > 1.0) == ("scaling" in rot)
    out = torch.full((len(pos), H, width + 5), 9.0, device="cuda", dtype=dtype)
    ops_seq.rotate_heads(dev(src)[:, :, lead:], out[:, :, :width], dev(pos), ops_seq.Rotation(dev(torch.tensor(freq, dtype=torch.float32)), halves, mag))
    want = np.stack([np.stack([plain.rotate(plain.f64(src[t, h, lead:]), int(pos[t]), rfreq, rmag, halves) for h in range(H)]) for t in range(len(pos))])
    close(out[:, :, :width], want, max(tol, 2e-3 if dtype == torch.float32 else tol), "rotated heads")       # (angle rounding at position 5000)
    close(out[:4, :, :width], want[:4], tol, "near positions")
    assert float((out[:, :, width:] - 9.0).abs().max()) == 0.0


def latent_case(H, d, dr, dv, qr, r, window, second, rot, T, seed, W=40, borrowed=False):
    """Mixer configuration, float64-exact bf16 weights and inputs."""
    g = torch.Generator().manual_seed(seed)
    m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": r, "scale": (d + dr) ** -0.5, "rot": rot}
    if window:
        m["mask"] = {"size": window}
    rnd = lambda *s: torch.randn(*s, generator=g)
    w = {"dq": rnd(qr, W) / W ** 0.5, "dq.norm": 1 + 0.2 * rnd(qr), "uq": 2 * rnd(H * (d + dr), qr) / qr ** 0.5,
         "dkv": rnd(r + dr, W) / W ** 0.5, "dkv.norm": 1 + 0.2 * rnd(r), "uk": 2 * rnd(H * d, r) / r ** 0.5, "uv": rnd(H * dv, r) / r ** 0.5,
         "o": rnd(W, H * dv) / (H * dv) ** 0.5}
    if not second:
        w["g"] = 2 * rnd(H, W) / W ** 0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    return m, w, rnd(T, W).to(torch.bfloat16)


def build_mixer(m, w, second, dtype, block, source=None, W=40, eps=1e-5):
    from nano_vllm_amd.mixers import LatentAttentionMixer
    rot = m["rot"]
    with torch.inference_mode():
        prev = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            mix = LatentAttentionMixer(W, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"], m["scale"], eps, block,
                                       window=m["mask"]["size"] if m.get("mask") else 0, rot_dims=rot["dims"], rot_base=rot["base"],
                                       rot_halves=second, rot_scaling=rot.get("scaling"), gated=not second, source=source).to("cuda")
        finally:
            torch.set_default_dtype(prev)
        loaders = mix.named_loaders()
        assert set(loaders) == set(w) - ({"dkv", "dkv.norm"} if source is not None else set())
        for k, fn in loaders.items():
            fn(w[k].to("cuda"))
    return mix


def run_mixer(m, w, h, second, dtype, block, cuts, path="auto", lend_to=None):
    """The product's mixer on h, cut into portions `cuts` (one sequence; dirty pages in scrambled order). `lend_to` = (m2, w2, second2):
    a second mixer that reads the first one's pages; its output is returned instead."""
    from nano_vllm_amd import ops_seq
    from nano_vllm_amd.attn_meta import reset_context, set_context
    T = h.shape[0]
    pages = -(-T // block)
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(T))[:pages].to(torch.int32)
    mix = build_mixer(m, w, second, dtype, block, W=h.shape[1])
    mix.block_size = block
    mix.k_cache = torch.full(((pages + 3) * block, 1, m["kv_rank"] + m["rot_dim"]), 7.0, device="cuda", dtype=dtype)
    mix.v_cache = torch.full(((pages + 3) * block, 1, m["kv_rank"]), -7.0, device="cuda", dtype=dtype)
    other = build_mixer(lend_to[0], lend_to[1], lend_to[2], dtype, block, source=mix, W=h.shape[1]) if lend_to else None
    assert other is None or other.kv_shapes() is None
    ops_seq.load_library().nvs_window_attn_force_scalar({"auto": 0, "scalar": 1, "nolds": 2, "unpacked": 3}[path])
    outs, at = [], 0
    try:
        with torch.inference_mode():
            for c in cuts:
                pos = torch.arange(at, at + c)
                slots = (order[pos // block].long() * block + pos % block).to(torch.int32)
                set_context(True, slot_mapping=dev(slots), block_tables=dev(order.view(1, -1)), portions=portions([c], [at], [0]))
                out = mix(dev(h[at:at + c], dtype), dev(pos))
                if other is not None:
                    out = other(dev(h[at:at + c], dtype), dev(pos))
                outs.append(out.float().cpu())
                at += c
    finally:
        reset_context()
        ops_seq.load_library().nvs_window_attn_force_scalar(0)
    assert at == T
    return torch.cat(outs)


def plain_mixer(m, w, h, second, kv=None):
    hh = plain.f64(h)
    own = plain.latent_kv(hh, w, m, 1e-5, second) if kv is None else kv
    return plain.latent_attention(hh, w, m, 1e-5, second, m["mask"]["size"] if m.get("mask") else 0, not second, own)


@pytest.mark.parametrize("dtype,path,tol", [(torch.float32, "auto", 3e-5), (torch.bfloat16, "auto", 3e-2), (torch.bfloat16, "nolds", 3e-2),
                                            (torch.bfloat16, "scalar", 3e-2), (torch.bfloat16, "unpacked", 3e-2)])
@pytest.mark.parametrize("H,d,dr,dv,qr,r,window,second,rot,block", [
    (8, 16, 8, 16, 24, 40, 23, False, ROTS[1], 16), (20, 8, 16, 24, 32, 176, 0, True, dict(ROTS[3], dims=16), 32), (70, 8, 8, 8, 16, 24, 50, False, ROTS[1], 64),
    (5, 24, 16, 40, 36, 48, 37, False, ROTS[0], 16), (4, 16, 32, 16, 24, 64, 0, True, ROTS[2], 64), (1, 8, 8, 8, 8, 16, 5, False, ROTS[1], 32),
    (3, 20, 12, 28, 50, 30, 0, True, ROTS[3], 16), (2, 64, 16, 64, 96, 200, 64, False, ROTS[0], 64), (2, 16, 16, 24, 20, 272, 70, False, ROTS[0], 16)])
def test_latent_attention_against_the_plain_loop(H, d, dr, dv, qr, r, window, second, rot, block, dtype, path, tol):
    """One prompt portion, then short portions and single tokens; windows that do not line up with pages or query tiles, latent
    rows that are not multiples of 8 or 16 and one longer than the matrix-core kernels take, one head, both pairings; with 8 heads
    and more the single tokens run with heads packed into the query tiles (20: a partial tile; 70: two workgroups per token)."""
    T = 150
    m, w, h = latent_case(H, d, dr, dv, qr, r, window, second, rot, T, seed=H * 100 + r)
    want = plain_mixer(m, w, h, second)
    for cuts in ([T], [97, 2, 1, 1, 30, 1, 1, 1, 16]):
        close(run_mixer(m, w, h, second, dtype, block, cuts, path), want, tol, f"cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("second_owner,second_reader", [(False, False), (True, False), (False, True)])
def test_a_layer_that_reads_another_layers_pages(second_owner, second_reader, dtype, tol):
    """The reader has other heads, head sizes, query rank, window and weights; only the latent sizes and the rotation are shared.
    Its keys must come from the owner's pages (the owner's down projection and norm), not from weights of its own."""
    T, r, dr = 120, 40, 16
    rot = dict(ROTS[2], dims=16) if second_owner else ROTS[0]
    m1, w1, h = latent_case(3, 16, dr, 24, 28, r, 0 if second_owner else 50, second_owner, rot, T, seed=1)
    m2, w2, _ = latent_case(5, 8, dr, 12, 20, r, 0 if second_reader else 21, second_reader, rot, T, seed=2)
    kv = plain.latent_kv(plain.f64(h), w1, m1, 1e-5, second_owner)
    want = plain_mixer(m2, w2, h, second_reader, kv=kv)
    w2r = {k: v for k, v in w2.items() if k not in ("dkv", "dkv.norm")}
    for cuts in ([T], [60, 2, 1, 1, 40, 16]):
        close(run_mixer(m1, w1, h, second_owner, dtype, 16, cuts, lend_to=(m2, w2r, second_reader)), want, tol, f"cuts {cuts[:3]}")
    assert np.abs(want - plain_mixer(m2, w2, h, second_reader)).max() > 0.05, "the case must tell the two caches apart"


def standout_case(window, T, marks, H=3, d=8, dr=8, dv=6, qr=8, r=16, W=24):
    """Every query asks for entry 0 of the unrotated key; only the marked positions have a key there, and a value of their own.
    All other tokens have a zero latent: zero keys (score 0) and zero values."""
    m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": r, "scale": 1.0, "rot": ROTS[1]}
    if window:
        m["mask"] = {"size": window}
    z = torch.zeros
    w = {"dq": z(qr, W), "dq.norm": torch.ones(qr), "uq": z(H * (d + dr), qr), "dkv": z(r + dr, W), "dkv.norm": torch.ones(r),
         "uk": z(H * d, r), "uv": z(H * dv, r), "o": torch.eye(W)[:, :H * dv], "g": z(H, W)}
    w["dq"][0, W - 1] = 1.0                       # the last input column is 1 for every token: the query latent is e_0 * sqrt(qr)
    w["uq"][0::d + dr, 0] = 4.0                   # -> entry 0 of every head's unrotated query
    h = z(T, W)
    h[:, W - 1] = 1.0
    assert len(marks) <= min(r, W - 1)
    for c, j in enumerate(marks):                 # mark c enters through input column c into latent entry c (normed: sqrt(r))
        h[j, c] = 1.0
        w["dkv"][c, c] = 1.0
        w["uk"][0::d, c] = 2.0                    # key entry 0 of every head
        w["uv"][:, c] = (10.0 + c) / 4.0          # a value that names the mark
    return m, {k: v.to(torch.bfloat16) for k, v in w.items()}, h.to(torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,block", [(100, 64), (50, 16), (64, 64), (33, 32), (1, 16)])
def test_a_standout_key_just_inside_and_just_outside_the_window(window, block, dtype):
    """A marked key's score is 4 * sqrt(8) * 2 * 4 = 90 above everybody else's: a query that still sees it returns (half of)
    its value, the query one position further returns zero — in a prompt and decoded one by one, at page borders, for the
    first tokens of the sequence."""
    T = 2 * window + 70
    marks = [0, 1, 15, 16, 63, 64, window + 20]
    m, w, h = standout_case(window, T, marks)
    want = plain_mixer(m, w, h, False)
    for j in marks:                                                              # the oracle itself shows every edge
        last = j + window - 1                                                    # the last query that sees mark j
        assert abs(want[last]).max() > 2.0 and abs(want[last] - want[last + 1]).max() > 0.1
    for cuts in ([T], [window - 1] + [1] * (T - window + 1), [2, window + 13, 2, window - 1, 2] + [1] * (T - 2 * window - 18)):
        if min(cuts) < 1:
            continue
        got = run_mixer(m, w, h, False, dtype, block, cuts)
        close(got, want, 1e-5 if dtype == torch.float32 else 1e-2, f"cuts {cuts[:5]}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_without_a_window(dtype):
    T = 900
    m, w, h = standout_case(0, T, [3, 64, 449])
    m["rot"] = dict(ROTS[3], dims=8)
    del w["g"]                                        # the causal mixer has no gate: outputs are whole values
    g = torch.Generator().manual_seed(3)
    w["dkv"][16:] = (0.3 * torch.randn(8, 24, generator=g)).to(torch.bfloat16)          # rotated key parts of ordinary size everywhere
    w["uq"] = w["uq"] + (0.05 * torch.randn(w["uq"].shape, generator=g)).to(torch.bfloat16)
    want = plain_mixer(m, w, h, True)
    assert abs(want[899]).max() > 3.0
    for cuts in ([T], [700] + [1] * 200, [2] * 450):
        close(run_mixer(m, w, h, True, dtype, 64, cuts), want, 2e-5 if dtype == torch.float32 else 1e-2, f"cuts {cuts[:3]}")


def margins(z, corr, top):
    """Per token: gap between the last chosen and the first rejected choice score (float64)."""
    s = 1.0 / (1.0 + np.exp(-z)) + corr
    srt = -np.sort(-s, axis=1)
    return srt[:, top - 1] - (srt[:, top] if s.shape[1] > top else -np.inf)


@pytest.mark.parametrize("total,top", [(12, 2), (16, 4), (7, 1), (64, 6), (130, 8), (4, 4), (3, 2)])
def test_sigmoid_router_choice_by_corrected_score_weights_without_it(total, top):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(total)
    n = 200
    z = 2.5 * torch.randn(n, total, generator=g)
    z[0] = -30.0                                      # scores ~ 1e-13: a negative correction makes choice scores negative
    corr = 0.4 * torch.randn(total, generator=g)
    ids, wts = ops_seq.moe_route(dev(z), total, dev(corr), top, 1, 1, 1.0, sigmoid=True, renorm=False)
    wid, wwt = plain.route(plain.f64(z), plain.f64(corr), top)
    sure = margins(plain.f64(z), plain.f64(corr), top) > 1e-5
    sure[0] = False
    assert sure.sum() > n // 2
    assert (ids.cpu().numpy()[sure] == wid[sure]).all()
    close(wts.cpu()[torch.tensor(sure)], wwt[sure], 2e-6, "weights are the plain sigmoids, not renormalised")
    assert float(wts.sum(1).max()) > 1.2 or top == 1
    ids2, wts2 = ops_seq.moe_route(dev(z), total, dev(corr), top, 1, 1, 1.0, sigmoid=True, renorm=True)
    assert (ids2 == ids).all()
    close(wts2.cpu()[torch.tensor(sure)].sum(1), np.ones(int(sure.sum())), 1e-5, "renormalised weights")


def moe_case(W, E, ff, top, seed):
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    w = {"router": 3 * rnd(E, W) / W ** 0.5, "correction": 0.2 * rnd(E)}
    for e in range(E):
        w[f"e{e}.up"], w[f"e{e}.down"] = rnd(ff, W) / W ** 0.5, rnd(W, ff) / ff ** 0.5
    return {"router": {"experts": E, "top": top}, "expert": {"ff": ff}, "kind": "moe"}, {k: v.to(torch.bfloat16) for k, v in w.items()}


@pytest.mark.parametrize("dtype,plain_kernel,tol", [(torch.float32, False, 2e-5), (torch.bfloat16, False, 2e-2), (torch.bfloat16, True, 2e-2)])
@pytest.mark.parametrize("W,E,ff,top,n", [(352, 7, 88, 3, 50), (40, 5, 24, 2, 33), (64, 12, 64, 2, 600), (128, 3, 40, 3, 5), (96, 9, 20, 1, 1),
                                          (256, 4, 128, 2, 1500)])
def test_ungated_squared_relu_experts_with_sigmoid_weights(W, E, ff, top, n, dtype, plain_kernel, tol):
    """All three grouped-product kernels (tile heights 16, 64, 128) and the plain one; sizes off the matrix-core step; every
    expert chosen and only one."""
    from nano_vllm_amd import ops_seq
    from nano_vllm_amd.mixers import RoutedExperts
    mlp, w = moe_case(W, E, ff, top, seed=W + E)
    g = torch.Generator().manual_seed(n)
    h = torch.randn(n, W, generator=g).to(torch.bfloat16)
    z = plain.f64(h) @ plain.f64(w["router"]).T
    sure = margins(z, plain.f64(w["correction"]), top) > (1e-5 if dtype == torch.float32 else 0.05)
    assert sure.sum() >= max(1, n // 3) or n == 1
    with torch.inference_mode():
        prev = torch.get_default_dtype()
        torch.set_default_dtype(dtype)
        try:
            mod = RoutedExperts(W, E, ff, top, gated=False, sigmoid=True, renorm=False).to("cuda")
        finally:
            torch.set_default_dtype(prev)
        loaders = mod.named_loaders()
        assert set(loaders) == set(w)
        for k, fn in loaders.items():
            fn(w[k].to("cuda"))
        ops_seq.load_library().nvs_moe_force_plain(int(plain_kernel))
        try:
            got = mod(dev(h, dtype)).float().cpu().numpy()
        finally:
            ops_seq.load_library().nvs_moe_force_plain(0)
    want = plain.routed_experts(plain.f64(h), w, mlp)
    if sure.any():
        close(got[sure], want[sure], tol, "experts")


# ---------------------------------------------------------------------------------------------- the engine
def small_config(variant: int = 0) -> dict:
    """Three models that differ in every size. 0: both mixers, a borrowed cache, a layer without feed-forward; 1: one head / one
    expert chosen / every expert chosen, a window shorter than a page, a type-2 layer lending to a type-1 layer; 2: wider, no cap."""
    yarn = {"factor": 4.0, "original": 128, "fast": 16.0, "slow": 2.0}

    def la(H, d, dr, dv, qr, r, size, base=20000.0, kv_from=None):
        m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": r, "scale": (d + dr) ** -0.5 * 1.5,
             "rot": {"base": base, "dims": dr}, "mask": {"size": size}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "latent_attention", "mixer": m}

    def la2(H, d, dr, dv, qr, r, base=100000.0, scaling=yarn):
        return {"type": "latent_attention_2", "mixer": {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": r,
                                                        "scale": (d + dr) ** -0.5 * 1.3, "rot": {"base": base, "dims": dr, "scaling": scaling}}}

    def moe(E, top, ff):
        return {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff}}

    if variant == 0:
        layers = [dict(la2(3, 24, 16, 40, 36, 48), mlp=moe(6, 2, 40)), dict(la(5, 16, 8, 24, 28, 56, 37), mlp=None),
                  dict(la(2, 32, 8, 16, 44, 56, 90, kv_from=1), mlp=moe(9, 3, 24)), dict(la2(4, 8, 24, 8, 20, 72), mlp=moe(4, 1, 56))]
        return {"architecture": "Pefazen", "vocab": 211, "width": 88, "layers": layers, "norm": {"eps": 1e-4}, "residual_mult": 0.45,
                "logit_scale": 0.5, "logit_softcap": 8.0}
    if variant == 1:
        layers = [dict(la2(1, 16, 16, 16, 16, 32, scaling={"factor": 1.5, "original": 32, "fast": 8.0, "slow": 1.0}), mlp=moe(3, 3, 16)),
                  dict(la(1, 8, 16, 8, 12, 32, 11, kv_from=0), mlp=moe(5, 1, 8)), dict(la(2, 12, 4, 20, 16, 20, 64), mlp=moe(2, 1, 32))]
        return {"architecture": "Pefazen", "vocab": 97, "width": 48, "layers": layers, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
                "logit_scale": 1.0, "logit_softcap": 30.0}
    layers = [dict(la(4, 40, 32, 24, 64, 104, 130), mlp=moe(16, 4, 48)), dict(la2(10, 16, 8, 40, 56, 144), mlp=moe(8, 2, 96)),
              dict(la(4, 24, 32, 16, 48, 104, 17, kv_from=0), mlp=moe(16, 2, 32))]
    return {"architecture": "Pefazen", "vocab": 384, "width": 256, "layers": layers, "norm": {"eps": 1e-5}, "residual_mult": 0.25,
            "logit_scale": 2.0}


def decisive(tensors: dict) -> dict:
    """Corrections spaced wider than any sigmoid: the choice no longer depends on the token (the weights still do)."""
    out = dict(tensors)
    for name, t in tensors.items():
        if name.endswith(".correction"):
            perm = torch.randperm(t.numel(), generator=torch.Generator().manual_seed(t.numel()))
            out[name] = (perm.float() * 2.0 - t.numel()).to(t.dtype)
    return out


@pytest.fixture(scope="module")
def checkpoints():
    from nano_vllm_amd.pefazen import random_tensors, write_synthetic_checkpoint
    root = tempfile.mkdtemp(prefix="pfz_")
    free = [write_synthetic_checkpoint(os.path.join(root, f"m{v}"), small_config(v), seed=31 + v) for v in range(3)]
    fixed = [write_synthetic_checkpoint(os.path.join(root, f"d{v}"), small_config(v), tensors=decisive(random_tensors(small_config(v), 31 + v)))
             for v in range(3)]
    return {"float32": free, "bfloat16": fixed}


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


def test_checkpoint_names_and_loaders_agree_and_the_borrowing_layer_owns_no_pages(checkpoints):
    from nano_vllm_amd.pefazen import tensor_shapes
    llm = engine(checkpoints["float32"][0])
    try:
        model = llm.model_runner.model
        assert set(model.named_loaders()) == set(tensor_shapes(small_config(0)))
        own = [l.mixer.kv_shapes() is not None for l in model.layers]
        assert own == [True, True, False, True]
        assert model.layers[2].mixer.k_cache is None and model.layers[1].mixer.k_cache.shape == (40 * 16, 1, 64)
        assert not any(n.endswith("norm2") for n in model.layers[1].named_loaders())
    finally:
        llm.exit()


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_decoding_agree_with_the_plain_model(checkpoints, variant, dtype):
    path = checkpoints[dtype][variant]
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
        # portions of changing size, down to two tokens and single tokens, cut inside pages and windows
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
    of others, requests that sit out steps, ends that free pages for the next request."""
    path = checkpoints["float32"][0]
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


def test_long_decoding_across_many_windows_and_pages(checkpoints):
    path = checkpoints["float32"][1]
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
    path = checkpoints[dtype][2]
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
    path = checkpoints["float32"][0]
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 200, (n,), generator=g).tolist() for n in (30, 31, 29, 17)]
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
    path = checkpoints["float32"][1]
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
