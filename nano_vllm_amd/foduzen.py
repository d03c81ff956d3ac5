"""Foduzen: a decoder-only family whose layers are listed one by one in config.json — recurrent blocks (real-gated linear
recurrent unit) and parallel blocks (sliding-window attention beside a state-space-duality mixer), each followed by an
xIELU feed-forward, on a 32-bit residual stream with the norm on every sublayer's OUTPUT:

    x = embed[token] * scale + sinusoid(position)
    x += g1 * rms(mixer(x));  x += g2 * rms(ff(x))          (g1, g2: one number each; sublayers read x itself)
    logits = head (g * rms(x))

Per-step dataflow on the MI355X (bf16 serving; with dtype float32 every tensor below is 32-bit):

    embed+sinusoid kernel -> x (fp32) and xh (bf16 copy for the next GEMM)
    recurrent block:  [y|x] GEMM -> stateful conv kernel (fp32 out) -> block-diagonal gate GEMM (fp32) -> scan kernel
                      (gates, decay, state update, GELU branch, product: one launch) -> out GEMM
    parallel block:   [q|k|v|gate|z|xBC|dt] GEMM -> key norm + paged K/V store -> windowed attention (q norm and sigmoid
                      gate fused) -> out GEMM;  stateful conv+SiLU -> SSD scan -> gate + group norm -> out GEMM
    residual kernel:  both branch norms, their mean, the scalar norm and the add in one launch (also emits xh)
    feed-forward:     up GEMM -> xIELU kernel (in place) -> down GEMM -> residual kernel

All sizes, the layer order and the design's free constants come from config.json; the sinusoid base (10000), the
recurrence's decay constant (8) and xIELU's linear coefficient (1/2) are fixed by the design and are defaults of the layers.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops_seq
from .attn_meta import get_context
from .mixers import ParallelMixer, RGLRUMixer, XIELUFeedForward, _copy_into, _param


class FoduzenConfig:
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
            if layer["type"] not in ("rglru", "parallel"):
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"].get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {layer['mlp'].get('kind')!r}")


class FoduzenLayer(nn.Module):

    def __init__(self, width: int, spec: dict, eps: float, block_size: int, dtype):
        super().__init__()
        self.kind, self.eps = spec["type"], eps
        m = spec["mixer"]
        if self.kind == "rglru":
            self.mix = RGLRUMixer(width, m["width"], m["blocks"], m["conv"], dtype)
        else:
            self.mix = ParallelMixer(width, m["left"], m["right"], eps, block_size, dtype)
        self.mlp = XIELUFeedForward(width, spec["mlp"]["ff"]) if spec.get("mlp") is not None else None
        self.norm1 = _param(1)
        self.norm2 = _param(1) if self.mlp is not None else None

    def named_loaders(self) -> dict:
        out = {"mix." + k: v for k, v in self.mix.named_loaders().items()}
        out["norm1"] = _copy_into(self.norm1.view(()))
        if self.mlp is not None:
            out.update({"mlp." + k: v for k, v in self.mlp.named_loaders().items()})
            out["norm2"] = _copy_into(self.norm2.view(()))
        return out

    def forward(self, x: torch.Tensor, xh: torch.Tensor, xh_out: torch.Tensor | None):
        """x: the 32-bit residual (updated in place); xh: x in the activation type (x itself in 32-bit serving)."""
        if self.kind == "rglru":
            ops_seq.norm_residual(x, self.mix(xh), self.norm1, self.eps, xh_out)
        else:
            left, right = self.mix(xh)
            ops_seq.norm_residual(x, left, self.norm1, self.eps, xh_out, m2=right, w1=self.mix.left_out, w2=self.mix.right_out)
        if self.mlp is not None:
            xin = xh_out if xh_out is not None else x
            ops_seq.norm_residual(x, self.mlp(xin), self.norm2, self.eps, xh_out)


class FoduzenForCausalLM(nn.Module):
    stateful = True

    def __init__(self, config: FoduzenConfig, dtype=None, block_size: int | None = None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.block_size = block_size or getattr(config, "kvcache_block_size", 256)
        self.embed = _param(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([FoduzenLayer(config.hidden_size, spec, config.eps, self.block_size, self.dtype)
                                     for spec in config.layers])
        self.final_norm = _param(1)
        self.head = _param(config.vocab_size, config.hidden_size)
        self.geo = dict(vocab=config.vocab_size, hidden=config.hidden_size, layers=len(config.layers), tie=False)

    def named_loaders(self) -> dict:
        out = {"embed": _copy_into(self.embed), "head": _copy_into(self.head), "final.norm": _copy_into(self.final_norm.view(()))}
        for i, layer in enumerate(self.layers):
            out.update({f"l{i}.{k}": v for k, v in layer.named_loaders().items()})
        return out

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Returns the 32-bit residual stream after the last layer, [n, width]."""
        n, cfg = input_ids.numel(), self.config
        x = torch.empty(n, cfg.hidden_size, dtype=torch.float32, device=input_ids.device)
        xh = None if self.dtype == torch.float32 else torch.empty(n, cfg.hidden_size, dtype=self.dtype, device=input_ids.device)
        ops_seq.embed_sinusoid(self.embed, input_ids, positions, cfg.embedding_scale, 10000.0, x, xh)
        trace = getattr(self, "layer_trace", None)          # tests: the residual stream after every layer
        for layer in self.layers:
            layer(x, xh if xh is not None else x, xh)
            if trace is not None:
                trace.append(x.clone())
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
        ops_seq.scalar_norm_rows(x, rows, nrows, self.final_norm, self.config.eps, normed)
        return F.linear(normed, self.head)


# ---- synthetic checkpoints (tests, benchmarks, dummy weights) -----------------------------------------------------------
def tensor_shapes(raw: dict) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a configuration (the parsed config.json)."""
    W, V = raw["width"], raw["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": ()}
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = ()
        if layer["type"] == "rglru":
            C, nb = m["width"], m["blocks"]
            bw = C // nb
            out.update({p + "mix.y": (C, W), p + "mix.y.b": (C,), p + "mix.x": (C, W), p + "mix.x.b": (C,),
                        p + "mix.conv": (C, m["conv"]), p + "mix.conv.b": (C,), p + "mix.ra": (nb, bw, bw), p + "mix.ra.b": (nb, bw),
                        p + "mix.ri": (nb, bw, bw), p + "mix.ri.b": (nb, bw), p + "mix.lam": (C,), p + "mix.o": (W, C)})
        else:
            le, ri = m["left"], m["right"]
            H, G, d, dv = le["heads"], le["kv_heads"], le["dim"], le["vdim"]
            inner, gn = ri["heads"] * ri["vdim"], ri["groups"] * ri["state"]
            out.update({p + "mix.left.q": (H * d, W), p + "mix.left.q.b": (H * d,), p + "mix.left.k": (G * d, W),
                        p + "mix.left.k.b": (G * d,), p + "mix.left.v": (G * dv, W), p + "mix.left.v.b": (G * dv,),
                        p + "mix.left.q.norm": (d,), p + "mix.left.k.norm": (d,), p + "mix.left.g": (H * dv, W),
                        p + "mix.left.o": (W, H * dv), p + "mix.left.o.b": (W,),
                        p + "mix.right.in": (2 * inner + 2 * gn + ri["heads"], W), p + "mix.right.conv": (inner + 2 * gn, ri["conv"]),
                        p + "mix.right.conv.b": (inner + 2 * gn,), p + "mix.right.dt_bias": (ri["heads"],),
                        p + "mix.right.A_log": (ri["heads"],), p + "mix.right.D": (ri["heads"],), p + "mix.right.norm": (inner,),
                        p + "mix.right.o": (W, inner), p + "mix.left.out": (W,), p + "mix.right.out": (W,)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff), p + "mlp.act": (2,)})
    return out


def random_tensors(raw: dict, seed: int = 0) -> dict[str, torch.Tensor]:
    """Seeded random bf16 weights in ranges that keep every mechanism alive: decays spread between fast and slow, step
    sizes around 0.1, matrices scaled by their fan-in."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=gen, dtype=torch.float32, device="cpu")
        if name.endswith(".lam"):
            t = -5.0 + 3.0 * torch.rand(shape, generator=gen, device="cpu")                  # a between ~0.6 and ~0.99 at r = 1/2
        elif leaf == "A_log":
            t = -2.0 + 2.5 * torch.rand(shape, generator=gen, device="cpu")
        elif leaf == "dt_bias":
            t = -3.5 + 2.5 * torch.rand(shape, generator=gen, device="cpu")
        elif leaf == "D" or leaf in ("norm", "out", "norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.1 * r
        elif leaf == "act":
            t = 0.5 * r
        elif leaf == "b" or len(shape) == 1:
            t = 0.1 * r
        elif name == "embed":
            t = 0.05 * r
        elif leaf in ("conv",):
            t = 0.5 * r
        else:
            t = r / (shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def write_synthetic_checkpoint(path: str, raw: dict, seed: int = 0) -> str:
    """config.json + model.safetensors of a random model of the family (no tokenizer: requests are token ids)."""
    import json
    import os
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(raw, fh, indent=1)
    save_file({k: v.contiguous() for k, v in random_tensors(raw, seed).items()}, os.path.join(path, "model.safetensors"))
    return path


def _init_random(self, seed: int = 0) -> None:
    loaders = self.named_loaders()
    dev = self.embed.device
    for name, t in random_tensors(self.config.raw, seed).items():
        loaders[name](t.to(dev))


FoduzenForCausalLM.init_random = _init_random
