"""Host side of stateful model families, no GPU: state slots, page tables that grow by portions, the caller-fixed step of
the scheduler, the prefix cache switch, the model registry and the Foduzen configuration / checkpoint naming."""
import json
import os
import types

import pytest
import torch

from nano_vllm_amd.engine.kv_blocks import BlockManager
from nano_vllm_amd.engine.sched import Scheduler
from nano_vllm_amd.engine.seq import Sequence, SequenceStatus
from nano_vllm_amd.engine.state_slots import StateSlotManager


def fdz_raw():
    par = {"type": "parallel", "mlp": {"kind": "dense", "ff": 24},
           "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 16, "scale": 0.3, "mask": {"size": 5}},
                     "right": {"heads": 2, "vdim": 8, "state": 4, "groups": 1, "conv": 3, "norm_groups": 2}}}
    rec = {"type": "rglru", "mlp": None, "mixer": {"width": 24, "blocks": 3, "conv": 2}}
    return {"architecture": "Foduzen", "embedding": {"scale": 2.0}, "layers": [rec, par], "norm": {"eps": 1e-5}, "vocab": 31, "width": 16}


def sched_config(stateful=True, blocks=8, block_size=16, seqs=2, budget=64):
    from nano_vllm_amd.foduzen import FoduzenConfig
    hf = FoduzenConfig(fdz_raw()) if stateful else None
    return types.SimpleNamespace(max_num_seqs=seqs, max_num_batched_tokens=budget, eos=-1, kvcache_block_size=block_size,
                                 num_kvcache_blocks=blocks, hf_config=hf)


def test_state_slots_lowest_first_and_reused():
    m = StateSlotManager(3)
    a, b, c = Sequence([1]), Sequence([2]), Sequence([3])
    assert [m.allocate(s) for s in (a, b, c)] == [0, 1, 2] and not m.can_allocate()
    m.release(b)
    assert b.state_slot == -1 and m.num_free == 1
    d = Sequence([4])
    assert m.allocate(d) == 1
    m.release(a), m.release(c), m.release(d)
    m.release(d)                                   # releasing twice is harmless
    assert m.num_free == 3
    with pytest.raises(AssertionError):
        m.allocate(a), m.allocate(a)


def test_block_manager_without_prefix_cache_never_shares_and_extends_by_portions():
    Sequence.block_size = 4
    bm = BlockManager(6, 4, prefix_cache=False)
    a, b = Sequence([7] * 9), Sequence([7] * 9)                    # identical prompts
    assert bm.can_allocate(a) == 0
    bm.allocate(a, 0)
    a.num_scheduled_tokens = 9
    bm.hash_blocks(a)
    assert bm.can_allocate(b) == 0 and not bm.hash_to_block_id      # nothing to find
    bm.allocate(b, 0)
    assert not set(a.block_table) & set(b.block_table) and bm.num_free == 0
    bm.deallocate(a)
    c = Sequence([1, 2])
    assert bm.blocks_to_extend(c, 2) == 1 and bm.can_extend(c, 2)
    bm.extend(c, 2)
    gen = c.table_gen
    assert len(c.block_table) == 1 and gen > 0
    for t in range(3, 11):
        c.append_token(t)
    assert bm.blocks_to_extend(c, 10) == 2
    bm.extend(c, 10)
    assert len(c.block_table) == 3 and c.table_gen == gen and bm.num_free == 0
    assert not bm.can_extend(c, 13)
    Sequence.block_size = 256


def test_caller_fixed_steps_admit_grow_and_retire():
    Sequence.block_size = 16
    s = Scheduler(sched_config(blocks=4, seqs=2))
    assert s.stateful and not s.block_manager.prefix_cache
    a, b = Sequence(list(range(20))), Sequence([5])
    batch = s.schedule_portions([(a, 3), (b, 1)])
    assert batch == [a, b] and (a.state_slot, b.state_slot) == (0, 1) and len(a.block_table) == 1
    assert a.num_scheduled_tokens == 3 and a.status is SequenceStatus.RUNNING
    s.finish_portions(batch)
    assert a.num_cached_tokens == 3 and b.num_cached_tokens == 1
    batch = s.schedule_portions([(a, 17)])                          # b sits this step out
    assert len(a.block_table) == 2
    s.finish_portions(batch)
    c = Sequence([1] * 40)
    with pytest.raises(RuntimeError, match="state slot"):
        s.schedule_portions([(c, 1)])
    s.retire(b)
    assert b.state_slot == -1 and not b.block_table
    with pytest.raises(RuntimeError, match="KV pool"):
        s.schedule_portions([(c, 40)])                              # 3 pages needed, 2 free
    s.retire(a)
    s.retire(c)
    assert s.block_manager.num_free == 4 and s.state_slots.num_free == 2 and s.is_finished()
    Sequence.block_size = 256


def test_scheduler_of_a_stateful_model_ties_slots_to_pages():
    """generate()'s own scheduling: a slot with the pages at admission, both back at the end or on preemption."""
    Sequence.block_size = 16
    s = Scheduler(sched_config(blocks=3, seqs=2, budget=64))
    from nano_vllm_amd.api import SamplingParams
    seqs = [Sequence([1] * 15, SamplingParams(temperature=0, max_tokens=30, ignore_eos=True)) for _ in range(3)]
    for q in seqs:
        s.add(q)
    batch, prefill = s.schedule()
    assert prefill and batch == seqs[:2] and [q.state_slot for q in seqs] == [0, 1, -1]      # max_num_seqs
    s.postprocess(batch, [9, 9], True)
    steps = preempted = 0
    orig = s.preempt
    s.preempt = lambda q: (orig(q), globals().__setitem__("_p", q))[0]
    while not s.is_finished() and steps < 400:
        batch, prefill = s.schedule()
        for q in list(s.waiting):
            assert q.state_slot == -1 and not q.block_table
        for q in batch:
            assert q.state_slot >= 0 and q.block_table
        s.postprocess(batch, [9] * len(batch), prefill)
        steps += 1
    assert s.is_finished() and s.state_slots.num_free == 2 and s.block_manager.num_free == 3
    assert all(q.num_completion_tokens == 30 for q in seqs)
    Sequence.block_size = 256


def test_registry_reads_both_config_layouts(tmp_path):
    from nano_vllm_amd.registry import REGISTRY, architecture_of, resolve, spec_of
    (tmp_path / "config.json").write_text(json.dumps(fdz_raw()))
    spec, cfg = resolve(str(tmp_path))
    assert spec.stateful and spec.block_multiple == 16 and "float32" in spec.dtypes
    assert cfg.vocab_size == 31 and cfg.hidden_size == 16 and cfg.num_hidden_layers == 2 and spec_of(cfg) is spec
    assert architecture_of({"architectures": ["Qwen3ForCausalLM"]}) == "Qwen3ForCausalLM"
    assert not REGISTRY["Qwen3ForCausalLM"].stateful and REGISTRY["Qwen3ForCausalLM"].block_multiple == 256
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Nothing"}))
    with pytest.raises(ValueError, match="unsupported"):
        resolve(str(tmp_path))
    bad = fdz_raw()
    bad["layers"][0]["type"] = "lstm"
    (tmp_path / "config.json").write_text(json.dumps(bad))
    with pytest.raises(ValueError, match="mixer type"):
        resolve(str(tmp_path))


def test_config_checks_follow_the_family(tmp_path):
    from nano_vllm_amd.api import Config
    (tmp_path / "config.json").write_text(json.dumps(fdz_raw()))
    c = Config(str(tmp_path), kvcache_block_size=48, dtype="fp32")
    assert c.dtype == "float32" and c.hf_config.architecture == "Foduzen"
    with pytest.raises(AssertionError):
        Config(str(tmp_path), kvcache_block_size=40)
    with pytest.raises(AssertionError):
        Config(str(tmp_path), tensor_parallel_size=2)


def test_checkpoint_names_and_the_models_loaders_agree():
    """Every tensor the synthetic checkpoint writes has a loader in the model and the other way round, shapes included."""
    from nano_vllm_amd.foduzen import FoduzenConfig, FoduzenForCausalLM, random_tensors, tensor_shapes
    raw = fdz_raw()
    model = FoduzenForCausalLM(FoduzenConfig(raw), torch.float32, block_size=16)
    loaders = model.named_loaders()
    shapes = tensor_shapes(raw)
    assert set(loaders) == set(shapes)
    tensors = random_tensors(raw, seed=3)
    with torch.no_grad():
        for name, t in tensors.items():
            assert tuple(t.shape) == tuple(shapes[name]) and t.dtype == torch.bfloat16
            loaders[name](t)
    mix = model.layers[1].mix
    q = mix.attn.widths[0]
    assert torch.equal(mix.in_w[:q], tensors["l1.mix.left.q"].float())
    assert torch.equal(mix.in_b[q + sum(mix.attn.widths[1:]):], torch.zeros(mix.ssd.in_width))      # no bias on that part
    rec = model.layers[0].mix
    assert torch.equal(rec.gate_w[1, :, :8], tensors["l0.mix.ra"][1].float().T)
    assert model.layers[0].mlp is None and model.layers[0].norm2 is None
    with pytest.raises(AssertionError):
        loaders["embed"](torch.zeros(3, 3))


# ---- Nokipel: configuration, layer runs, shared weights, checkpoint names (no GPU) -----------------------------------
def nkp_raw():
    light = {"type": "lightning", "mixer": {"heads": 2, "dim": 8, "vdim": 12, "decay": [0.5, 0.99]}, "mlp": {"kind": "dense", "ff": 20, "limit": 2.0}}
    attn = {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 6, "scale": 0.3, "mask": {"size": 5},
                                           "rot": {"dims": 4, "base": 100.0}},
            "mlp": {"kind": "moe", "expert": {"ff": 10}, "shared": {"ff": 14},
                    "router": {"experts": 3, "identity": 1, "top": 2, "scale": 1.5, "groups": {"count": 2, "keep": 1}}}}
    bare = {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 6, "vdim": 6, "scale": 0.4}, "mlp": None}
    return {"architecture": "Nokipel", "embedding": {"scale": 2.0}, "layers": [light, attn, bare, light], "loop": {"start": 1, "stop": 3, "times": 3},
            "norm": {"eps": 1e-5, "groups": 2}, "vocab": 29, "width": 16}


def test_nokipel_registry_config_and_order_of_layer_runs(tmp_path):
    from nano_vllm_amd.registry import REGISTRY, resolve
    (tmp_path / "config.json").write_text(json.dumps(nkp_raw()))
    spec, cfg = resolve(str(tmp_path))
    assert spec is REGISTRY["Nokipel"] and spec.stateful and set(spec.dtypes) == {"bfloat16", "float32"}
    assert cfg.vocab_size == 29 and cfg.hidden_size == 16 and cfg.norm_groups == 2
    assert cfg.runs() == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (3, 0)]
    raw = nkp_raw()
    del raw["loop"]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    assert resolve(str(tmp_path))[1].runs() == [(0, 0), (1, 0), (2, 0), (3, 0)]
    for key, bad, msg in (("type", "lstm", "mixer type"), ("mlp", {"kind": "conv"}, "feed-forward kind")):
        raw = nkp_raw()
        raw["layers"][0][key] = bad
        (tmp_path / "config.json").write_text(json.dumps(raw))
        with pytest.raises(ValueError, match=msg):
            resolve(str(tmp_path))
    raw = nkp_raw()
    raw["loop"]["stop"] = 9
    (tmp_path / "config.json").write_text(json.dumps(raw))
    with pytest.raises(ValueError, match="loop"):
        resolve(str(tmp_path))


def test_nokipel_checkpoint_names_loaders_and_weights_shared_between_runs():
    """Every tensor the synthetic checkpoint writes has a loader in the model and the other way round; a layer inside the
    repeated span has one mixer per run, all on the SAME weight tensors, each with cache / state attributes of its own."""
    from nano_vllm_amd.nokipel import NokipelConfig, NokipelForCausalLM, random_tensors, tensor_shapes
    raw = nkp_raw()
    model = NokipelForCausalLM(NokipelConfig(raw), torch.float32, block_size=16)
    loaders = model.named_loaders()
    shapes = tensor_shapes(raw)
    assert set(loaders) == set(shapes)
    tensors = random_tensors(raw, seed=3)
    with torch.no_grad():
        for name, t in tensors.items():
            assert tuple(t.shape) == tuple(shapes[name]) and t.dtype == torch.bfloat16
            loaders[name](t)
    assert [len(layer.mixers) for layer in model.layers] == [1, 3, 3, 1]
    a = model.layers[1].mixers
    assert a[0].in_w is a[1].in_w is a[2].in_w and a[0].o_w is a[2].o_w and a[0].attn is not a[2].attn
    q, k, v = a[0].cols
    assert (q, k, v) == (32, 16, 12) and torch.equal(a[2].in_w[q:q + k], tensors["l1.mix.k"].float())
    assert torch.equal(a[1].in_b[q + k:], tensors["l1.mix.v.b"].float())
    assert a[0].attn.chunk == 5 and a[0].attn.window == 0 and a[0].attn.rot_freq.tolist() == [1.0, pytest.approx(0.1)]
    assert model.layers[2].mixers[0].attn.chunk == 0 and model.layers[2].mixers[0].attn.rot_freq is None and model.layers[2].mlp is None
    kv_layers = [m for m in model.modules() if hasattr(m, "kv_shapes")]
    st_layers = [m for m in model.modules() if hasattr(m, "state_shapes")]
    assert len(kv_layers) == 6 and len(st_layers) == 2 and st_layers[0].state_shapes() == {"rec_state": (2, 12, 8)}
    n_params = sum(p.numel() for p in model.parameters())                     # shared tensors count once
    assert n_params == sum(int(torch.tensor(s).prod()) for s in shapes.values())
    lig = model.layers[0].mixers[0]
    v, k, q, g = lig.cols
    assert torch.equal(lig.in_w[v + k:v + k + q], tensors["l0.mix.q"].float()) and lig.decay.tolist() == [0.5, pytest.approx(0.99)]
    moe = model.layers[1].mlp
    assert moe.router.dtype == torch.float32 and moe.router.shape == (5, 16) and torch.equal(moe.router[4:], tensors["l1.mlp.shared.sg"].float())
    assert torch.equal(moe.w_gu[2, 10:], tensors["l1.mlp.e2.up"].float()) and moe.correction.dtype == torch.float32
    with pytest.raises(AssertionError):
        loaders["embed"](torch.zeros(3, 3))


# ---- Pefazen: configuration, borrowed caches, scaled rotation table, checkpoint names (no GPU) ----------------------------
def pfz_raw():
    def mixer(H, d, dr, dv, qr, r, **kw):
        return dict({"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": r, "scale": 0.2}, **kw)
    moe = {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 3, "top": 2}}
    a = {"type": "latent_attention", "mixer": mixer(2, 6, 4, 8, 5, 12, mask={"size": 7}, rot={"dims": 4, "base": 100.0}), "mlp": moe}
    b = {"type": "latent_attention_2", "mlp": None,
         "mixer": mixer(3, 4, 8, 6, 7, 10, rot={"dims": 8, "base": 10000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}})}
    c = {"type": "latent_attention", "mixer": mixer(4, 2, 4, 2, 3, 12, mask={"size": 3}, rot={"dims": 4, "base": 100.0}, kv_from=0), "mlp": moe}
    return {"architecture": "Pefazen", "layers": [a, b, c], "norm": {"eps": 1e-5}, "vocab": 29, "width": 16, "residual_mult": 0.5,
            "logit_scale": 0.125, "logit_softcap": 20.0}


def test_pefazen_registry_and_config_checks(tmp_path):
    from nano_vllm_amd.registry import REGISTRY, resolve
    (tmp_path / "config.json").write_text(json.dumps(pfz_raw()))
    spec, cfg = resolve(str(tmp_path))
    assert spec is REGISTRY["Pefazen"] and spec.stateful and set(spec.dtypes) == {"bfloat16", "float32"}
    assert (cfg.vocab_size, cfg.hidden_size, cfg.residual_mult, cfg.logit_scale, cfg.logit_softcap) == (29, 16, 0.5, 0.125, 20.0)
    cases = [(lambda r: r["layers"][0].update(type="lstm"), "mixer type"), (lambda r: r["layers"][0].update(mlp={"kind": "dense"}), "feed-forward kind"),
             (lambda r: r["layers"][2]["mixer"].update(kv_from=2), "kv_from"), (lambda r: r["layers"][1]["mixer"].update(kv_from=2), "kv_from"),
             (lambda r: r["layers"][2]["mixer"].update(kv_rank=14), "latent sizes")]
    for change, msg in cases:
        raw = pfz_raw()
        change(raw)
        (tmp_path / "config.json").write_text(json.dumps(raw))
        with pytest.raises(ValueError, match=msg):
            resolve(str(tmp_path))


def test_pefazen_checkpoint_names_loaders_and_the_borrowed_cache():
    """Every tensor the synthetic checkpoint writes has a loader in the model and the other way round; the layer that reads
    another layer's cache has no down projection for keys and values and asks the engine for no pages."""
    from nano_vllm_amd.pefazen import PefazenConfig, PefazenForCausalLM, random_tensors, tensor_shapes
    raw = pfz_raw()
    model = PefazenForCausalLM(PefazenConfig(raw), torch.float32, block_size=16)
    loaders, shapes = model.named_loaders(), tensor_shapes(raw)
    assert set(loaders) == set(shapes) and "l2.mix.dkv" not in shapes and "l1.mix.g" not in shapes and "l1.norm2" not in shapes
    tensors = random_tensors(raw, seed=3)
    with torch.no_grad():
        for name, t in tensors.items():
            assert tuple(t.shape) == tuple(shapes[name]) and t.dtype == torch.bfloat16
            loaders[name](t)
    a, b, c = (layer.mixer for layer in model.layers)
    assert a.kv_shapes() == ((1, 16), (1, 12)) and b.kv_shapes() == ((1, 18), (1, 10)) and c.kv_shapes() is None
    assert c._source[0] is a and len(list(c.parameters())) == len(list(a.parameters())) - 1
    assert sum(p.numel() for p in model.parameters()) == sum(int(torch.tensor(s).prod()) for s in shapes.values())
    # fused in-projection: [query latent | key/value latent + rotated key part | gate]
    assert a.in_w.shape == (5 + 16 + 2, 16) and b.in_w.shape == (7 + 18, 16) and c.in_w.shape == (3 + 4, 16)
    assert torch.equal(a.in_w[5:21], tensors["l0.mix.dkv"].float()) and torch.equal(c.in_w[3:], tensors["l2.mix.g"].float())
    assert torch.equal(a.uk.view(12, 12), tensors["l0.mix.uk"].float()) and torch.equal(b.uv[2], tensors["l1.mix.uv"].float()[12:18])
    assert (a.window, b.window, c.window) == (7, 0, 3) and (a.gated, b.gated) == (True, False) and (a.rot_halves, b.rot_halves) == (False, True)
    assert a.rot_mag == 1.0 and a.rot_freq.tolist() == [1.0, pytest.approx(0.1)]
    moe = model.layers[0].mlp
    assert (moe.gated, moe.sigmoid, moe.renorm) == (False, True, False) and moe.w_gu.shape == (3, 10, 16) and model.layers[1].mlp is None


def test_scaled_rotation_table_blends_between_the_two_marks():
    """factor 4 over 64 original positions: pairs turning more than 8 times keep their frequency, pairs turning less than once
    have it divided by 4, the pairs between blend linearly in the pair index; cos and sin grow by 0.1 ln 4 + 1."""
    import math
    from nano_vllm_amd.mixers import rotary_frequencies
    base, dims = 10000.0, 8
    freq, mag = rotary_frequencies(dims, base, {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0})
    plain = [base ** (-2 * i / dims) for i in range(dims // 2)]
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    lo = math.floor(dims * math.log(64 / (2 * math.pi * 8.0)) / (2 * math.log(base)))        # 0
    hi = math.ceil(dims * math.log(64 / (2 * math.pi * 1.0)) / (2 * math.log(base)))         # 2
    assert (lo, hi) == (0, 2)
    assert freq[0] == pytest.approx(plain[0]) and freq[1] == pytest.approx(plain[1] * (0.5 / 4 + 0.5))
    assert freq[2] == pytest.approx(plain[2] / 4) and freq[3] == pytest.approx(plain[3] / 4)
    assert rotary_frequencies(dims, base) == (plain, 1.0)


def test_attention_in_the_latent_space_is_the_same_sum_reordered():
    """What the product computes per head — scores of [W_uk^T q | rotated q part] against the cached row [c | rotated key part],
    softmax, the weighted sum of the latents, then W_uv — equals the plain model's attention over up-projected keys and values
    (float64, numpy; a window shorter than the sequence, gate included)."""
    import numpy as np
    from oracle import pefazen as plain
    rng = np.random.default_rng(0)
    n, W, H, d, dr, dv, qr, r, window = 23, 20, 3, 6, 4, 5, 7, 9, 8
    m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": r, "scale": 0.4, "rot": {"dims": dr, "base": 50.0}, "mask": {"size": window}}
    w = {"dq": rng.normal(size=(qr, W)), "dq.norm": rng.normal(size=qr), "uq": rng.normal(size=(H * (d + dr), qr)), "dkv": rng.normal(size=(r + dr, W)),
         "dkv.norm": rng.normal(size=r), "uk": rng.normal(size=(H * d, r)), "uv": rng.normal(size=(H * dv, r)), "o": np.eye(H * dv), "g": rng.normal(size=(H, W))}
    h = rng.normal(size=(n, W))
    lat, kr = plain.latent_kv(h, w, m, 1e-5, False)
    want = plain.latent_attention(h, w, m, 1e-5, False, window, True, (lat, kr))
    freq, mag = plain.rotary_table(m["rot"])
    q = (plain.rms_norm(h @ w["dq"].T, w["dq.norm"], 1e-5) @ w["uq"].T).reshape(n, H, d + dr)
    rows = np.concatenate([lat, kr], 1)                                     # the cache: one row per token for all heads
    got = np.zeros((n, H, dv))
    for t in range(n):
        keys = slice(max(t - window + 1, 0), t + 1)
        for a in range(H):
            qa = np.concatenate([w["uk"].reshape(H, d, r)[a].T @ q[t, a, :d], plain.rotate(q[t, a, d:], t, freq, mag, False)])
            sc = rows[keys] @ qa * m["scale"]
            p = np.exp(sc - sc.max())
            got[t, a] = w["uv"].reshape(H, dv, r)[a] @ ((p / p.sum()) @ lat[keys]) / (1.0 + np.exp(-(h[t] @ w["g"][a])))
    assert np.abs(got.reshape(n, H * dv) - want).max() < 1e-12


# ---- Lobidra --------------------------------------------------------------------------------------------------------------
def lbd_raw():
    att = {"type": "attention", "mlp": {"kind": "dense", "ff": 20},
           "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 6, "conv": 3, "scale": 0.4,
                     "rot": {"dims": 4, "base": 100.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}}}
    par = {"type": "parallel", "mlp": {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 3, "top": 2}, "shared": {"ff": 12}},
           "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 8, "scale": 0.5, "q_temp": {"coef": 0.25, "every": 8}},
                     "right": {"heads": 3, "dim": 4, "vdim": 2, "gate_cap": 9.0}, "left_scale": 0.5, "right_scale": 2.0}}
    return {"architecture": "Lobidra", "layers": [att, par, dict(att, weights_of=0), dict(par, weights_of=1, mlp=par["mlp"])],
            "norm": {"eps": 1e-5}, "vocab": 29, "width": 16, "embedding": {"scale": 4.0}}


def test_lobidra_registry_and_config_checks(tmp_path):
    from nano_vllm_amd.registry import REGISTRY, resolve
    (tmp_path / "config.json").write_text(json.dumps(lbd_raw()))
    spec, cfg = resolve(str(tmp_path))
    assert spec is REGISTRY["Lobidra"] and spec.stateful and set(spec.dtypes) == {"bfloat16", "float32"}
    assert (cfg.vocab_size, cfg.hidden_size, cfg.embedding_scale, cfg.eps) == (29, 16, 4.0, 1e-5)
    assert [cfg.owner(i) for i in range(4)] == [0, 1, 0, 1]
    cases = [(lambda r: r["layers"][0].update(type="lstm"), "mixer type"), (lambda r: r["layers"][0].update(mlp={"kind": "glu"}), "feed-forward kind"),
             (lambda r: r["layers"][2].update(weights_of=3), "weights_of"), (lambda r: r["layers"][3].update(weights_of=2), "weights_of"),
             (lambda r: r["layers"][2].update(weights_of=1), "another type"), (lambda r: r["layers"][0]["mixer"].update(vdim=8), "vdim")]
    for change, msg in cases:
        raw = json.loads(json.dumps(lbd_raw()))
        change(raw)
        (tmp_path / "config.json").write_text(json.dumps(raw))
        with pytest.raises(ValueError, match=msg):
            resolve(str(tmp_path))


def test_lobidra_checkpoint_names_loaders_and_weights_shared_between_layers():
    """Every tensor the synthetic checkpoint writes has a loader in the model and the other way round; a layer that runs with another
    layer's weights has no tensors and holds the very same parameter objects."""
    from nano_vllm_amd.lobidra import LobidraConfig, LobidraForCausalLM, random_tensors, tensor_shapes
    raw = lbd_raw()
    model = LobidraForCausalLM(LobidraConfig(raw), torch.float32, block_size=16)
    loaders, shapes = model.named_loaders(), tensor_shapes(raw)
    assert set(loaders) == set(shapes) and not any(n.startswith(("l2.", "l3.")) for n in shapes)
    assert "l0.mix.v" not in shapes and "l0.mix.q.conv" in shapes and "l1.mlp.router" not in shapes and shapes["l1.mlp.table"] == (29, 2)
    tensors = random_tensors(raw, seed=3)
    with torch.no_grad():
        for name, t in tensors.items():
            assert tuple(t.shape) == tuple(shapes[name]) and t.dtype == (torch.int32 if name.endswith(".table") else torch.bfloat16)
            loaders[name](t)
    assert all(len(set(row)) == 2 and max(row) < 3 for row in tensors["l1.mlp.table"].tolist())
    a, p, a2, p2 = model.layers
    assert a2.mixer.in_w is a.mixer.in_w and a2.norm1b is a.norm1b and p2.mlp.w_gu is p.mlp.w_gu and p2.mixer.attn.sink is p.mixer.attn.sink
    assert sum(p_.numel() for p_ in set(model.parameters())) == sum(int(torch.tensor(s).prod()) for s in shapes.values())
    # fused in-projections: [q | k | gate per head] and [q | k | v | g || v | k | q | g | zi | zf]
    assert a.mixer.in_w.shape == (24 + 12 + 4, 16) and a.mixer.conv_w.shape == (36, 3) and a.mixer.state_shapes() == {"conv_state": (2, 36)}
    assert torch.equal(a.mixer.in_w[24:36], tensors["l0.mix.k"].float()) and torch.equal(a.mixer.conv_w[24:], tensors["l0.mix.k.conv"].float())
    assert a.mixer.attn.kv_shapes() == ((2, 6), (2, 6)) and a.mixer.attn.sink.tolist() == [0.0] * 4 and a.mixer.attn.gate_per_head
    assert p.mixer.in_w.shape == (8 + 4 + 8 + 16 + 6 + 12 + 12 + 6 + 3 + 3, 16) and p.mixer.attn.q_temp == (0.25, 8)
    assert torch.equal(p.mixer.in_w[36 + 6 + 12:36 + 6 + 24], tensors["l1.mix.right.q"].float())
    assert torch.equal(p.mixer.in_w[-3:], tensors["l1.mix.right.f"].float()) and torch.equal(p.mixer.attn.sink, tensors["l1.mix.left.sink"].float())
    assert p.mixer.mem.state_shapes() == {"rec_state": (3, 3, 4), "max_state": (3,)} and p.scales == (0.5, 2.0) and a.scales == (1.0, 1.0)
    assert p.mlp.table_vocab == 29 and not p.mlp.shared_gate and not hasattr(p.mlp, "router") and a.mlp.up.shape == (20, 16)
    # the rotation's table: wavelengths 2 pi and 20 pi against marks at 8 and 16 positions: the first pair stays, the second is slowed
    assert a.mixer.attn.rot_freq.tolist() == [1.0, pytest.approx(0.05)]
