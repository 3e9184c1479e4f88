"""Lobidra: a decoder-only family whose layers are listed one by one in config.json. Every sublayer is normed on BOTH sides,

    x += nb1(mixer(na1(x)));  x += nb2(ff(na2(x)))        n(v) = v / sqrt(mean(v^2) + eps) * (1 + w): weights stored around zero

on a 32-bit residual stream. Mixers: `attention` (mixers.ConvAttentionMixer: short causal convolutions on the query / key
projections, keys before rotation are the values, band-wise scaled rotary frequencies, one more score of zero in every softmax
denominator, a gate per head) and `parallel` (mixers.AttentionMemoryMixer: position-free attention with a query temperature and
learned sinks beside a matrix memory with exponential gates; the two outputs are added with a scale each). Feed-forwards:
`dense` (GELU), `moe` (gated experts chosen by a table over token ids, equal weights, plus an ungated-by-anything shared expert),
or none. A layer with `weights_of: j` runs with layer j's weights (mixer, feed-forward, norms) and pages / state of its own.

    x = embed[token] * scale;   logits = head n(x)

Per-step dataflow on the MI355X (bf16 serving; with dtype float32 every tensor below is 32-bit):

    embed kernel -> x (fp32)
    per sublayer:     sandwich norm kernel (x += nb(previous sublayer's output); h = na(x) in bf16) — one launch per sublayer
    attention:        [q|k|g] GEMM -> causal convolution (state: last taps - 1 rows) -> key rotation + paged K/V store (V = the
                      unrotated keys) -> attention (query rotation, sink, per-head gate fused) -> out GEMM
    parallel:         ONE [q|k|v|g | v|k|q|g|zi|zf] GEMM -> K/V store -> attention (temperature, sinks, gate fused) -> out GEMM;
                      gated memory scan (fp32 state) -> per-head norm + gate kernel -> out GEMM; the sandwich kernel adds both
    dense ff:         up GEMM -> GELU kernel -> down GEMM
    moe ff:           table route kernel -> plan kernel -> grouped [gate|up] product (SiLU GLU fused) -> grouped down product ->
                      combine kernel (weights, shared expert)

All sizes, the layer order and the design's free constants come from config.json; the 1e-6 in the memory's divisor, the
memory's running maximum starting at 0 and the GELU's constants are fixed by the design.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops_seq
from .attn_meta import get_context
from .mixers import (AttentionMemoryMixer, ConvAttentionMixer, GeluFeedForward, RoutedExperts, _copy_into, _param,
                     banded_rotary_frequencies, tie_parameters)


class LobidraConfig:
    """config.json of the family, with the few attribute names the engine reads from any configuration."""

    def __init__(self, raw: dict):
        self.raw = raw
        self.architecture = raw["architecture"]
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers = list(raw["layers"])
        self.num_hidden_layers = len(self.layers)
        self.eps = float(raw["norm"]["eps"])
        self.embedding_scale = float(raw["embedding"]["scale"])
        self.max_position_embeddings = 1 << 24          # positions are exact integers in a 32-bit float up to here
        self.eos_token_id = raw.get("eos_token_id", -1)
        for i, layer in enumerate(self.layers):
            if layer["type"] not in ("attention", "parallel"):
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            src = layer.get("weights_of")
            if src is not None:
                src = int(src)
                if not (0 <= src < i) or self.layers[src].get("weights_of") is not None:
                    raise ValueError(f"layer {i}: weights_of {src} must name an earlier layer that has weights of its own")
                if self.layers[src]["type"] != layer["type"]:
                    raise ValueError(f"layer {i}: weights_of {src} names a layer of another type")
            if layer["type"] == "attention":
                m = layer["mixer"]
                if int(m.get("vdim", m["dim"])) != int(m["dim"]):
                    raise ValueError(f"layer {i}: the keys are the values, so vdim {m.get('vdim')} must equal dim {m['dim']}")

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs with."""
        src = self.layers[i].get("weights_of")
        return i if src is None else int(src)


def _mixer(width: int, spec: dict, eps: float, block_size: int):
    m = spec["mixer"]
    if spec["type"] == "attention":
        rot = m.get("rot")
        return ConvAttentionMixer(width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], int(m.get("conv", 1)), m["scale"], eps,
                                  block_size, rot_dims=int(rot["dims"]) if rot else 0,
                                  rot_freqs=banded_rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling")) if rot else None,
                                  sink="zero")
    return AttentionMemoryMixer(width, m["left"], m["right"], eps, block_size)


def _feed_forward(width: int, vocab: int, mlp: dict | None):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return GeluFeedForward(width, mlp["ff"])
    r, shared = mlp["router"], mlp.get("shared")
    return RoutedExperts(width, r["experts"], mlp["expert"]["ff"], r["top"], shared_ff=shared["ff"] if shared else 0, table_vocab=vocab,
                         shared_gate=False)


class LobidraLayer(nn.Module):
    """One layer: its mixer, feed-forward and four norms. A layer that runs with another's weights is built alike and has all its
    parameters tied to that layer's tensors (mixers.tie_parameters): what stays its own is the cache / state the runner injects."""

    def __init__(self, width: int, vocab: int, spec: dict, eps: float, block_size: int):
        super().__init__()
        self.mixer = _mixer(width, spec, eps, block_size)
        self.parallel = spec["type"] == "parallel"
        self.scales = (float(spec["mixer"]["left_scale"]), float(spec["mixer"]["right_scale"])) if self.parallel else (1.0, 1.0)
        self.mlp = _feed_forward(width, vocab, spec.get("mlp"))
        self.routed = isinstance(self.mlp, RoutedExperts)
        self.norm1, self.norm1b = _param(width), _param(width)
        self.norm2 = _param(width) if self.mlp is not None else None
        self.norm2b = _param(width) if self.mlp is not None else None

    def named_loaders(self) -> dict:
        out = {"mix." + k: v for k, v in self.mixer.named_loaders().items()}
        out.update({"norm1": _copy_into(self.norm1), "norm1b": _copy_into(self.norm1b)})
        if self.mlp is not None:
            out.update({"mlp." + k: v for k, v in self.mlp.named_loaders().items()})
            out.update({"norm2": _copy_into(self.norm2), "norm2b": _copy_into(self.norm2b)})
        return out


class LobidraForCausalLM(nn.Module):
    stateful = True

    def __init__(self, config: LobidraConfig, dtype=None, block_size: int | None = None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.block_size = block_size or getattr(config, "kvcache_block_size", 256)
        self.embed = _param(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList()
        for i, spec in enumerate(config.layers):
            src = config.owner(i)
            layer = LobidraLayer(config.hidden_size, config.vocab_size, config.layers[src], config.eps, self.block_size)
            if src != i:
                tie_parameters(layer, self.layers[src])
            self.layers.append(layer)
        self.final_norm = _param(config.hidden_size)
        self.head = _param(config.vocab_size, config.hidden_size)
        self.geo = dict(vocab=config.vocab_size, hidden=config.hidden_size, layers=len(config.layers), tie=False)

    def named_loaders(self) -> dict:
        out = {"embed": _copy_into(self.embed), "head": _copy_into(self.head), "final.norm": _copy_into(self.final_norm)}
        for i, layer in enumerate(self.layers):
            if self.config.owner(i) == i:
                out.update({f"l{i}.{k}": v for k, v in layer.named_loaders().items()})
        return out

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the 32-bit residual stream after the last layer, [n, width]. A sublayer's output is normed and added to the
        stream by the kernel that norms the stream for the NEXT sublayer (`pending` below: output(s), scales, the norm's weight)."""
        n, cfg = input_ids.numel(), self.config
        dev = input_ids.device
        x = torch.empty(n, cfg.hidden_size, dtype=torch.float32, device=dev)
        ops_seq.embed_sinusoid(self.embed, input_ids, positions, cfg.embedding_scale, 0.0, x, None)
        trace = getattr(self, "layer_trace", None)          # tests: the residual stream after every layer
        pending = None                                      # (a, a2, a_mult, a2_mult, weight of the norm on the output)

        def sandwich(w_next):
            h = torch.empty(n, cfg.hidden_size, dtype=self.dtype, device=dev) if w_next is not None else None
            if pending is None:
                ops_seq.sandwich_norm(x, None, None, w_next, cfg.eps, h)
            else:
                a, a2, m1, m2, wb = pending
                ops_seq.sandwich_norm(x, a, wb, w_next, cfg.eps, h, a2=a2, a_mult=m1, a2_mult=m2)
            return h

        for layer in self.layers:
            h = sandwich(layer.norm1)
            if layer.parallel:
                left, right = layer.mixer(h, positions)
                pending = (left, right, layer.scales[0], layer.scales[1], layer.norm1b)
            else:
                pending = (layer.mixer(h, positions), None, 1.0, 1.0, layer.norm1b)
            if layer.mlp is not None:
                h = sandwich(layer.norm2)
                y = layer.mlp(h, input_ids) if layer.routed else layer.mlp(h)
                pending = (y, None, 1.0, 1.0, layer.norm2b)
            if trace is not None:
                sandwich(None)
                pending = None
                trace.append(x.clone())
        if pending is not None:
            sandwich(None)
        return x

    def compute_logits(self, x: torch.Tensor, rows: torch.Tensor | None = None, nrows: int | None = None) -> torch.Tensor:
        """Logits of the residual rows `rows` (int32 device indices; default: each portion's last token)."""
        if rows is None:
            ctx = get_context()
            nrows = ctx.portions.nseq
            rows = (ctx.portions.cu_q[1:nrows + 1] - 1).to(torch.int32)
        if nrows == 0:
            return torch.empty(0, self.config.vocab_size, dtype=self.dtype, device=x.device)
        normed = torch.empty(nrows, x.shape[1], dtype=self.dtype, device=x.device)
        ops_seq.offset_norm_rows(x, rows, nrows, self.final_norm, self.config.eps, normed)
        return F.linear(normed, self.head)


# ---- synthetic checkpoints (tests, benchmarks, dummy weights) -----------------------------------------------------------
def tensor_shapes(raw: dict) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a configuration (the parsed config.json). Integer tensors: names ending in `.table`."""
    W, V = raw["width"], raw["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(raw["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        out.update({p + "norm1": (W,), p + "norm1b": (W,)})
        if layer["type"] == "attention":
            H, d = m["heads"], m["dim"]
            G, taps = m.get("kv_heads", H), m.get("conv", 1)
            out.update({p + "mix.q": (H * d, W), p + "mix.k": (G * d, W), p + "mix.q.conv": (H * d, taps), p + "mix.k.conv": (G * d, taps),
                        p + "mix.g": (H, W), p + "mix.o": (W, H * d)})
        else:
            a, b = m["left"], m["right"]
            H, d = a["heads"], a["dim"]
            G, dv = a.get("kv_heads", H), a.get("vdim", d)
            out.update({p + "mix.left.q": (H * d, W), p + "mix.left.k": (G * d, W), p + "mix.left.v": (G * dv, W), p + "mix.left.sink": (H,),
                        p + "mix.left.g": (H * dv, W), p + "mix.left.o": (W, H * dv)})
            H, d = b["heads"], b["dim"]
            dv = b.get("vdim", d)
            out.update({p + "mix.right.q": (H * d, W), p + "mix.right.k": (H * d, W), p + "mix.right.v": (H * dv, W),
                        p + "mix.right.g": (H * dv, W), p + "mix.right.o": (W, H * dv), p + "mix.right.norm": (H * dv,),
                        p + "mix.right.i": (H, W), p + "mix.right.i.b": (H,), p + "mix.right.f": (H, W), p + "mix.right.f.b": (H,)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out.update({p + "norm2": (W,), p + "norm2b": (W,)})
        if mlp["kind"] == "dense":
            out.update({p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            r, ff = mlp["router"], mlp["expert"]["ff"]
            for e in range(r["experts"]):
                out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
            out[p + "mlp.table"] = (V, r["top"])
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf)})
    return out


def random_tensors(raw: dict, seed: int = 0) -> dict[str, torch.Tensor]:
    """Seeded random bf16 weights (tables: int32 rows of distinct experts) in ranges that keep every mechanism alive: matrices
    scaled by their fan-in, norm offsets around zero, sinks and gate biases of order one, convolution taps of order one."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        leaf = name.split(".")[-1]
        if leaf == "table":
            layer = raw["layers"][int(name.split(".")[0][1:])]
            experts = layer["mlp"]["router"]["experts"]
            order = torch.rand(shape[0], experts, generator=gen, dtype=torch.float32, device="cpu").argsort(dim=1)
            out[name] = order[:, :shape[1]].to(torch.int32)             # a row: the first `top` of a random order of the experts
            continue
        r = torch.randn(shape, generator=gen, dtype=torch.float32, device="cpu")
        if name.endswith("right.norm"):
            t = 1.0 + 0.1 * r
        elif leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b"):
            t = 0.1 * r
        elif leaf == "sink":
            t = r
        elif leaf == "b":
            t = r + (2.0 if name.endswith("f.b") else 0.0)
        elif leaf == "conv":
            t = r / (shape[-1] ** 0.5)
        elif name == "embed":
            t = r / (raw["embedding"]["scale"] or 1.0)
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


LobidraForCausalLM.init_random = _init_random
