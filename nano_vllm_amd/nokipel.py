"""Nokipel: a pre-norm decoder-only family whose layers are listed one by one in config.json. Every layer is

    x += mixer(gn1(x));  x += ff(gn2(x))          gn: RMS norm in `norm.groups` equal parts of the row, then a weight

on a 32-bit residual stream. Mixers: `attention` (softmax attention inside blocks of positions, grouped kv heads, biased
projections, rotation of the leading dimensions of each head in interleaved pairs) and `lightning` (linear attention as a
decaying outer-product recurrence, gated). Feed-forwards: `dense` (clamped gated unit), `moe` (routed experts with grouped
top-k choice, pass-through experts and a gated shared expert), or none. `loop` names a span of layers that runs several times
with the same weights; every run has its own K/V pages or recurrent state, and the embedding output is added to the stream
again before every run of the span but the first.

    x = embed[token] * scale;   logits = head gn(x)

Per-step dataflow on the MI355X (bf16 serving; with dtype float32 every tensor below is 32-bit):

    embed kernel -> x (fp32)
    per sublayer:     add + group norm kernel (x += the previous sublayer's output [+ the embedding], h = gn(x) in bf16)
    attention:        [q|k|v] GEMM (bias) -> key rotation + paged K/V store -> block-masked attention (query rotation fused) -> out GEMM
    lightning:        [v|k|q|g] GEMM -> decay scan (SiLU fused, fp32 state) -> norm + sigmoid gate kernel -> out GEMM
    dense ff:         [gate|up] GEMM -> clamped GLU kernel -> down GEMM
    moe ff:           router GEMM (fp32) -> route kernel -> plan kernel -> grouped [gate|up] product (SiLU GLU fused) ->
                      grouped down product -> combine kernel (weights, pass-through experts, gated shared expert)

All sizes, the layer order and the design's free constants come from config.json; the slope of the dense unit's sigmoid
(1.702) and the router's 1e-20 are fixed by the design.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops_seq
from .attn_meta import get_context
from .mixers import AttentionMixer, ClampedGLU, LightningMixer, RoutedExperts, _copy_into, _param, tie_parameters


class NokipelConfig:
    """config.json of the family, with the few attribute names the engine reads from any configuration."""

    def __init__(self, raw: dict):
        self.raw = raw
        self.architecture = raw["architecture"]
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers = list(raw["layers"])
        self.num_hidden_layers = len(self.layers)
        self.eps = float(raw["norm"]["eps"])
        self.norm_groups = int(raw["norm"].get("groups", 1))
        self.embedding_scale = float(raw["embedding"]["scale"])
        self.max_position_embeddings = 1 << 24          # positions are exact integers in a 32-bit float up to here
        self.eos_token_id = raw.get("eos_token_id", -1)
        loop = raw.get("loop") or {"start": 0, "stop": 0, "times": 1}
        self.loop_start, self.loop_stop, self.loop_times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        n = len(self.layers)
        if not (0 <= self.loop_start <= self.loop_stop <= n and self.loop_times >= 1):
            raise ValueError(f"loop {loop} does not fit {n} layers")
        if self.hidden_size % self.norm_groups:
            raise ValueError(f"width {self.hidden_size} is not a multiple of norm.groups {self.norm_groups}")
        for i, layer in enumerate(self.layers):
            if layer["type"] not in ("attention", "lightning"):
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"].get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {layer['mlp'].get('kind')!r}")

    def runs(self) -> list[tuple[int, int]]:
        """(layer, pass) in execution order."""
        out = [(i, 0) for i in range(self.loop_start)]
        for k in range(self.loop_times):
            out += [(i, k) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, 0) for i in range(self.loop_stop, len(self.layers))]


def _mixer(width: int, spec: dict, eps: float, block_size: int):
    m = spec["mixer"]
    if spec["type"] == "attention":
        rot, mask = m.get("rot"), m.get("mask")
        return AttentionMixer(width, m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"]), m["scale"], eps,
                              block_size, chunk=int(mask["size"]) if mask else 0, rot_dims=int(rot["dims"]) if rot else 0,
                              rot_base=float(rot["base"]) if rot else 10000.0)
    decay = m["decay"]
    if isinstance(decay, (int, float)):                # one number: every head decays alike
        decay = [decay] * m["heads"]
    return LightningMixer(width, m["heads"], m["dim"], m.get("vdim", m["dim"]), decay, eps)


def _feed_forward(width: int, mlp: dict | None):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return ClampedGLU(width, mlp["ff"], mlp["limit"])
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    shared = mlp.get("shared")
    return RoutedExperts(width, r["experts"], mlp["expert"]["ff"], r["top"], r.get("scale", 1.0), r.get("identity", 0),
                         groups["count"], groups["keep"], shared["ff"] if shared else 0)


class NokipelLayer(nn.Module):
    """One layer's weights; `passes` mixers share them and differ in the cache / state the runner gives each."""

    def __init__(self, width: int, spec: dict, eps: float, block_size: int, passes: int):
        super().__init__()
        self.mixers = nn.ModuleList([_mixer(width, spec, eps, block_size) for _ in range(passes)])
        for other in self.mixers[1:]:
            tie_parameters(other, self.mixers[0])
        self.mlp = _feed_forward(width, spec.get("mlp"))
        self.norm1 = _param(width)
        self.norm2 = _param(width) if self.mlp is not None else None

    def named_loaders(self) -> dict:
        out = {"mix." + k: v for k, v in self.mixers[0].named_loaders().items()}
        out["norm1"] = _copy_into(self.norm1)
        if self.mlp is not None:
            out.update({"mlp." + k: v for k, v in self.mlp.named_loaders().items()})
            out["norm2"] = _copy_into(self.norm2)
        return out


class NokipelForCausalLM(nn.Module):
    stateful = True

    def __init__(self, config: NokipelConfig, dtype=None, block_size: int | None = None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.block_size = block_size or getattr(config, "kvcache_block_size", 256)
        self.embed = _param(config.vocab_size, config.hidden_size)
        in_loop = range(config.loop_start, config.loop_stop)
        self.layers = nn.ModuleList([NokipelLayer(config.hidden_size, spec, config.eps, self.block_size,
                                                  config.loop_times if i in in_loop else 1)
                                     for i, spec in enumerate(config.layers)])
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
        stream by the kernel that norms the stream for the NEXT sublayer (`pending` below)."""
        n, cfg = input_ids.numel(), self.config
        dev = input_ids.device
        x = torch.empty(n, cfg.hidden_size, dtype=torch.float32, device=dev)
        ops_seq.embed_sinusoid(self.embed, input_ids, positions, cfg.embedding_scale, 0.0, x, None)
        again = cfg.loop_times > 1 and cfg.loop_stop > cfg.loop_start
        e0 = x.clone() if again else None
        trace = getattr(self, "layer_trace", None)          # tests: the residual stream after every layer run
        pending = None
        for i, k in cfg.runs():
            layer = self.layers[i]
            h = torch.empty(n, cfg.hidden_size, dtype=self.dtype, device=dev)
            ops_seq.add_group_norm(x, layer.norm1, cfg.norm_groups, cfg.eps, h, a=pending,
                                   b=e0 if (k > 0 and i == cfg.loop_start) else None)
            pending = layer.mixers[k](h, positions)
            if layer.mlp is not None:
                h = torch.empty(n, cfg.hidden_size, dtype=self.dtype, device=dev)
                ops_seq.add_group_norm(x, layer.norm2, cfg.norm_groups, cfg.eps, h, a=pending)
                pending = layer.mlp(h)
            if trace is not None:
                ops_seq.add_group_norm(x, None, cfg.norm_groups, cfg.eps, None, a=pending)
                pending = None
                trace.append(x.clone())
        if pending is not None:
            ops_seq.add_group_norm(x, None, cfg.norm_groups, cfg.eps, None, a=pending)
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
        ops_seq.group_norm_rows(x, rows, nrows, self.final_norm, self.config.norm_groups, self.config.eps, normed)
        return F.linear(normed, self.head)


# ---- synthetic checkpoints (tests, benchmarks, dummy weights) -----------------------------------------------------------
def tensor_shapes(raw: dict) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a configuration (the parsed config.json)."""
    W, V = raw["width"], raw["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        H, d = m["heads"], m["dim"]
        dv = m.get("vdim", d)
        if layer["type"] == "attention":
            G = m.get("kv_heads", H)
            out.update({p + "mix.q": (H * d, W), p + "mix.q.b": (H * d,), p + "mix.k": (G * d, W), p + "mix.k.b": (G * d,),
                        p + "mix.v": (G * dv, W), p + "mix.v.b": (G * dv,), p + "mix.o": (W, H * dv)})
        else:
            out.update({p + "mix.q": (H * d, W), p + "mix.k": (H * d, W), p + "mix.v": (H * dv, W), p + "mix.g": (H * dv, W),
                        p + "mix.o": (W, H * dv), p + "mix.norm": (H * dv,)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = (W,)
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            out.update({p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
        else:
            r, ff = mlp["router"], mlp["expert"]["ff"]
            total = r["experts"] + r.get("identity", 0)
            for e in range(r["experts"]):
                out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
            out.update({p + "mlp.router": (total, W), p + "mlp.correction": (total,)})
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf),
                            p + "mlp.shared.sg": (1, W)})
    return out


def random_tensors(raw: dict, seed: int = 0) -> dict[str, torch.Tensor]:
    """Seeded random bf16 weights in ranges that keep every mechanism alive: matrices scaled by their fan-in, norm weights
    around one, router rows large enough that choices differ from token to token, corrections that reorder choices."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        leaf = name.split(".")[-1]
        r = torch.randn(shape, generator=gen, dtype=torch.float32, device="cpu")
        if leaf in ("norm", "norm1", "norm2"):
            t = 1.0 + 0.1 * r
        elif leaf == "correction":
            t = 0.05 * r
        elif leaf == "b":
            t = 0.1 * r
        elif name == "embed":
            t = r / (raw["embedding"]["scale"] or 1.0)
        elif leaf == "router":
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


NokipelForCausalLM.init_random = _init_random
