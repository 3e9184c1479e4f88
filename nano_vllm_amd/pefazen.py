"""Pefazen: a pre-norm decoder-only family whose layers are listed one by one in config.json. Every layer is

    x += m * mixer(ln1(x));  x += m * ff(ln2(x))          ln: layer norm with a weight and no bias, m = `residual_mult`

on a 32-bit residual stream. Both mixers are latent attention (mixers.LatentAttentionMixer): queries through a normed latent,
keys and values up-projected from a cached normed latent, one rotated key part shared by the heads.

    latent_attention      pairs (2i, 2i+1) rotate, sliding window of `mask.size` positions, per-head sigmoid output gate;
                          with `kv_from: j` the layer reads layer j's cached latents and rotated key parts and has no down
                          projection of its own
    latent_attention_2    pairs (i, i + dims/2) rotate, frequencies scaled by `rot.scaling` (YaRN; cos and sin carry its
                          magnitude factor), causal, no gate

The feed-forward is a mixture of ungated experts W_down max(W_up h, 0)^2 with a sigmoid router: choice by score + correction,
weights = the chosen scores as they are. A layer may have no feed-forward (`mlp: null`).

    x = embed[token];   logits = cap * tanh(head ln(x) * logit_scale / cap)

Per-step dataflow on the MI355X (bf16 serving; with dtype float32 every tensor below is 32-bit):

    embed kernel -> x (fp32)
    per sublayer:   add + norm kernel (x += m * the previous sublayer's output, h = ln(x) in bf16)
    mixer:          [dq | dkv | gate] GEMM -> latent kernel (both RMS norms, key rotation, paged store) -> q GEMM ->
                    per-head W_uk^T q (batched GEMM) + query rotation kernel -> paged attention in the latent space (mask and
                    gate fused) -> per-head W_uv (batched GEMM) -> out GEMM
    feed-forward:   router GEMM (fp32) -> route kernel -> plan kernel -> grouped up product (squared ReLU fused) -> grouped
                    down product -> combine kernel
    logits:         norm of the wanted rows -> head GEMM -> scale + cap kernel (fp32)

All sizes, the layer order and the design's free constants come from config.json; 0.1 in the magnitude factor of scaled
rotations is fixed by the design.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops_seq
from .attn_meta import get_context
from .mixers import LatentAttentionMixer, RoutedExperts, _copy_into, _param

MIXERS = ("latent_attention", "latent_attention_2")


class PefazenConfig:
    """config.json of the family, with the few attribute names the engine reads from any configuration."""

    def __init__(self, raw: dict):
        self.raw = raw
        self.architecture = raw["architecture"]
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers = list(raw["layers"])
        self.num_hidden_layers = len(self.layers)
        self.eps = float(raw["norm"]["eps"])
        self.residual_mult = float(raw.get("residual_mult", 1.0))
        self.logit_scale = float(raw.get("logit_scale", 1.0))
        self.logit_softcap = float(raw.get("logit_softcap") or 0.0)
        self.max_position_embeddings = 1 << 24          # positions are exact integers in a 32-bit float up to here
        self.eos_token_id = raw.get("eos_token_id", -1)
        for i, layer in enumerate(self.layers):
            if layer["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"].get("kind") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {layer['mlp'].get('kind')!r}")
            src = layer["mixer"].get("kv_from")
            if src is not None:
                if not (0 <= int(src) < i) or self.layers[int(src)]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from {src} is not an earlier layer with a cache of its own")
                a, b = layer["mixer"], self.layers[int(src)]["mixer"]
                if (a["kv_rank"], a["rot_dim"]) != (b["kv_rank"], b["rot_dim"]):
                    raise ValueError(f"layer {i}: its latent sizes differ from those of layer {src}, whose cache it reads")


def _mixer(width: int, spec: dict, eps: float, block_size: int, source) -> LatentAttentionMixer:
    m, second = spec["mixer"], spec["type"] == "latent_attention_2"
    rot = m["rot"]
    return LatentAttentionMixer(width, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["q_rank"]),
                                int(m["kv_rank"]), float(m["scale"]), eps, block_size,
                                window=0 if second else int(m["mask"]["size"]), rot_dims=int(rot["dims"]), rot_base=float(rot["base"]),
                                rot_halves=second, rot_scaling=rot.get("scaling") if second else None, gated=not second, source=source)


def _feed_forward(width: int, mlp: dict | None):
    if mlp is None:
        return None
    r = mlp["router"]
    return RoutedExperts(width, int(r["experts"]), int(mlp["expert"]["ff"]), int(r["top"]), gated=False, sigmoid=True, renorm=False)


class PefazenLayer(nn.Module):

    def __init__(self, width: int, spec: dict, eps: float, block_size: int, source):
        super().__init__()
        self.mixer = _mixer(width, spec, eps, block_size, source)
        self.mlp = _feed_forward(width, spec.get("mlp"))
        self.norm1 = _param(width)
        self.norm2 = _param(width) if self.mlp is not None else None

    def named_loaders(self) -> dict:
        out = {"mix." + k: v for k, v in self.mixer.named_loaders().items()}
        out["norm1"] = _copy_into(self.norm1)
        if self.mlp is not None:
            out.update({"mlp." + k: v for k, v in self.mlp.named_loaders().items()})
            out["norm2"] = _copy_into(self.norm2)
        return out


class PefazenForCausalLM(nn.Module):
    stateful = True

    def __init__(self, config: PefazenConfig, dtype=None, block_size: int | None = None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.block_size = block_size or getattr(config, "kvcache_block_size", 256)
        self.embed = _param(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList()
        for spec in config.layers:
            src = spec["mixer"].get("kv_from")
            self.layers.append(PefazenLayer(config.hidden_size, spec, config.eps, self.block_size,
                                            self.layers[int(src)].mixer if src is not None else None))
        self.final_norm = _param(config.hidden_size)
        self.head = _param(config.vocab_size, config.hidden_size)
        self.geo = dict(vocab=config.vocab_size, hidden=config.hidden_size, layers=len(config.layers), tie=False)

    def named_loaders(self) -> dict:
        out = {"embed": _copy_into(self.embed), "head": _copy_into(self.head), "final.norm": _copy_into(self.final_norm)}
        for i, layer in enumerate(self.layers):
            out.update({f"l{i}.{k}": v for k, v in layer.named_loaders().items()})
        return out

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the 32-bit residual stream after the last layer, [n, width]. Every sublayer's output is added to the
        stream, times m, by the kernel that norms the stream for the NEXT sublayer (`pending` below)."""
        n, cfg = input_ids.numel(), self.config
        dev, m = input_ids.device, cfg.residual_mult
        x = torch.empty(n, cfg.hidden_size, dtype=torch.float32, device=dev)
        ops_seq.embed_sinusoid(self.embed, input_ids, positions, 1.0, 0.0, x, None)
        trace = getattr(self, "layer_trace", None)          # tests: the residual stream after every layer
        pending = None
        for layer in self.layers:
            h = torch.empty(n, cfg.hidden_size, dtype=self.dtype, device=dev)
            ops_seq.add_group_norm(x, layer.norm1, 1, cfg.eps, h, a=pending, a_mult=m, center=True)
            pending = layer.mixer(h, positions)
            if layer.mlp is not None:
                h = torch.empty(n, cfg.hidden_size, dtype=self.dtype, device=dev)
                ops_seq.add_group_norm(x, layer.norm2, 1, cfg.eps, h, a=pending, a_mult=m, center=True)
                pending = layer.mlp(h)
            if trace is not None:
                ops_seq.add_group_norm(x, None, 1, cfg.eps, None, a=pending, a_mult=m)
                pending = None
                trace.append(x.clone())
        if pending is not None:
            ops_seq.add_group_norm(x, None, 1, cfg.eps, None, a=pending, a_mult=m)
        return x

    def compute_logits(self, x: torch.Tensor, rows: torch.Tensor | None = None, nrows: int | None = None) -> torch.Tensor:
        """32-bit logits of the residual rows `rows` (int32 device indices; default: each portion's last token)."""
        cfg = self.config
        if rows is None:
            ctx = get_context()
            nrows = ctx.portions.nseq
            rows = (ctx.portions.cu_q[1:nrows + 1] - 1).to(torch.int32)
        if nrows == 0:
            return torch.empty(0, cfg.vocab_size, dtype=torch.float32, device=x.device)
        normed = torch.empty(nrows, x.shape[1], dtype=self.dtype, device=x.device)
        ops_seq.group_norm_rows(x, rows, nrows, self.final_norm, 1, cfg.eps, normed, center=True)
        return ops_seq.scale_softcap(F.linear(normed, self.head), cfg.logit_scale, cfg.logit_softcap)


# ---- synthetic checkpoints (tests, benchmarks, dummy weights) -----------------------------------------------------------
def tensor_shapes(raw: dict) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a configuration (the parsed config.json)."""
    W, V = raw["width"], raw["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, d, dr, dv, qr, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
        out.update({p + "norm1": (W,), p + "mix.dq": (qr, W), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (d + dr), qr),
                    p + "mix.uk": (H * d, r), p + "mix.uv": (H * dv, r), p + "mix.o": (W, H * dv)})
        if m.get("kv_from") is None:
            out.update({p + "mix.dkv": (r + dr, W), p + "mix.dkv.norm": (r,)})
        if layer["type"] == "latent_attention":
            out[p + "mix.g"] = (H, W)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = (W,)
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        for e in range(E):
            out.update({p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
        out.update({p + "mlp.router": (E, W), p + "mlp.correction": (E,)})
    return out


def random_tensors(raw: dict, seed: int = 0) -> dict[str, torch.Tensor]:
    """Seeded random bf16 weights in ranges that keep every mechanism alive: matrices scaled by their fan-in (the up-projections
    of keys and queries a little larger, so that the softmax is not flat), norm weights around one, router rows large enough
    that choices differ from token to token, corrections that reorder choices."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=gen, dtype=torch.float32, device="cpu")
        if leaf in ("norm", "norm1", "norm2"):
            t = 1.0 + 0.1 * r
        elif leaf == "correction":
            t = 0.1 * r
        elif name == "embed":
            t = r
        elif leaf in ("router", "uq", "uk", "g"):
            t = 2.0 * r / (shape[-1] ** 0.5)
        else:
            t = r / (shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def write_synthetic_checkpoint(path: str, raw: dict, seed: int = 0, tensors: dict | None = None) -> str:
    """config.json + model.safetensors of a random model of the family (no tokenizer: requests are token ids)."""
    import json
    import os
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(raw, fh, indent=1)
    tensors = tensors if tensors is not None else random_tensors(raw, seed)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def _init_random(self, seed: int = 0) -> None:
    loaders = self.named_loaders()
    dev = self.embed.device
    for name, t in random_tensors(self.config.raw, seed).items():
        loaders[name](t.to(dev))


PefazenForCausalLM.init_random = _init_random
