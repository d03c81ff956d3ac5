"""Plain, slow restatement of the Nokipel design on the CPU (test infrastructure only; shares no code with the product
path under nano_vllm_amd/). One function per mechanism, token loops where the design has a recurrence or a mask,
float64 throughout. `Model.run(tokens, state)` continues a sequence from `state`, so the same functions serve as the
oracle for whole prompts, portions and single decoded tokens.

The design: a pre-norm decoder. Every layer is x += mixer(gn(x)); x += ff(gn(x)) with gn a group-wise RMS norm; mixers are
softmax attention restricted to the query's own block of positions (grouped kv heads, biased projections, rotation of the
leading dimensions of every head in interleaved pairs) or a decaying outer-product recurrence ("lightning" linear
attention, gated); feed-forwards are a clamped gated unit, or a routed mixture with grouped top-k choice, a choice-only
correction, pass-through experts and a gated shared expert. A span of layers may run several times with the same weights
(and separate caches), the embedding being added again before every repeat.

Notation: T tokens of a portion, W model width, eps the norm's epsilon.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Each of `groups` equal consecutive parts of a row divided by its own root mean square; then the weight."""
    T, W = x.shape
    return rms(x.view(T, groups, W // groups), eps).reshape(T, W) * w


def rotate(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, d]: entries (2i, 2i+1), i < dims/2, turn by the angle p * base^(-2i/dims); the rest pass."""
    out = x.clone()
    for i in range(dims // 2):
        a = positions.to(F64) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def block_attention(h, p, cfg, st):
    """Softmax attention in which position i sees j <= i of its own block of `mask.size` positions (blocks counted from
    the start of the sequence; no mask entry: every j <= i). st holds the keys and values so far."""
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = (h @ p["q"].T + p["q.b"]).view(T, H, d)
    k = (h @ p["k"].T + p["k.b"]).view(T, G, d)
    v = (h @ p["v"].T + p["v.b"]).view(T, G, dv)
    n0 = st["k"].shape[0]
    pos = torch.arange(n0, n0 + T)
    if cfg.get("rot"):
        q = rotate(q, pos, cfg["rot"]["dims"], cfg["rot"]["base"])
        k = rotate(k, pos, cfg["rot"]["dims"], cfg["rot"]["base"])
    st["k"] = torch.cat([st["k"], k], 0)
    st["v"] = torch.cat([st["v"], v], 0)
    K, V = st["k"], st["v"]
    size = cfg["mask"]["size"] if cfg.get("mask") else None
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        i = n0 + t
        lo = (i // size) * size if size else 0
        for hh in range(H):
            g = hh // (H // G)
            s = (K[lo:i + 1, g] @ q[t, hh]) * cfg["scale"]
            out[t, hh] = torch.softmax(s, 0) @ V[lo:i + 1, g]
    return out.reshape(T, H * dv) @ p["o"].T


def lightning(h, p, cfg, eps, st):
    """Per head S <- decay S + k v^T, o = S^T q on SiLU-activated projections; the heads together are RMS-normed,
    gated by a sigmoid and projected."""
    H, d, dv = cfg["heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = silu(h @ p["q"].T).view(T, H, d)
    k = silu(h @ p["k"].T).view(T, H, d)
    v = silu(h @ p["v"].T).view(T, H, dv)
    S = st["S"]
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        for hh in range(H):
            S[hh] = cfg["decay"][hh] * S[hh] + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S[hh].T @ q[t, hh]
    y = rms(o.reshape(T, H * dv), eps) * p["norm"]
    return (y * sigmoid(h @ p["g"].T)) @ p["o"].T


def clamped_glu(h, p, limit: float):
    g = torch.clamp(h @ p["gate"].T, max=limit)
    u = torch.clamp(h @ p["up"].T, min=-limit, max=limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ p["down"].T


def expert(h, p):
    return (silu(h @ p["gate"].T) * (h @ p["up"].T)) @ p["down"].T


def route(z: torch.Tensor, correction: torch.Tensor, top: int, count: int, keep: int, scale: float):
    """z: router logits of one token. Returns (chosen indices, weights)."""
    s = torch.softmax(z, 0)
    c = s + correction
    n = z.shape[0]
    per = n // count
    best = torch.stack([c[g * per:(g + 1) * per].max() for g in range(count)])
    kept = torch.topk(best, keep).indices.tolist()
    masked = torch.full_like(c, -math.inf)
    for g in kept:
        masked[g * per:(g + 1) * per] = c[g * per:(g + 1) * per]
    idx = torch.topk(masked, top).indices
    w = s[idx] / (s[idx].sum() + 1e-20) * scale
    return idx.tolist(), w


def mixture(h, p, cfg):
    r = cfg["router"]
    E, ident = r["experts"], r.get("identity", 0)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ p["router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        idx, w = route(z[t], p["correction"], r["top"], groups["count"], groups["keep"], r["scale"])
        for e, we in zip(idx, w):
            if e >= E:
                assert e < E + ident
                out[t] += we * h[t]
            else:
                out[t] += we * expert(h[t:t + 1], {k[len(f"e{e}."):]: v for k, v in p.items() if k.startswith(f"e{e}.")})[0]
    if cfg.get("shared"):
        sp = {k[len("shared."):]: v for k, v in p.items() if k.startswith("shared.")}
        out = out + expert(h, sp) * sigmoid(h @ sp["sg"].T)
    return out


class Model:
    """Weights as float64 tensors by name; config as the parsed config.json."""

    def __init__(self, config: dict, tensors: dict):
        self.cfg = config
        self.w = {k: v.to(F64) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]
        self.groups = config["norm"].get("groups", 1)
        n = len(config["layers"])
        loop = config.get("loop") or {"start": 0, "stop": 0, "times": 1}
        self.runs = [(i, 0) for i in range(loop["start"])]                      # (layer, pass)
        for k in range(loop["times"]):
            self.runs += [(i, k) for i in range(loop["start"], loop["stop"])]
        self.runs += [(i, 0) for i in range(loop["stop"], n)]
        self.loop = loop

    @classmethod
    def load(cls, path: str) -> "Model":
        from safetensors.torch import load_file
        with open(os.path.join(path, "config.json")) as fh:
            cfg = json.load(fh)
        return cls(cfg, load_file(os.path.join(path, "model.safetensors")))

    def sub(self, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def new_state(self) -> dict:
        st = {"pos": 0, "runs": []}
        for i, _ in self.runs:
            layer = self.cfg["layers"][i]
            m = layer["mixer"]
            if layer["type"] == "attention":
                st["runs"].append({"k": torch.zeros(0, m["kv_heads"], m["dim"], dtype=F64),
                                   "v": torch.zeros(0, m["kv_heads"], m["vdim"], dtype=F64)})
            else:
                st["runs"].append({"S": torch.zeros(m["heads"], m["dim"], m["vdim"], dtype=F64)})
        return st

    def run(self, tokens, state: dict | None = None, trace_layers: bool = False):
        """Logits [T, vocab] of the portion `tokens`, continuing `state` (updated in place)."""
        st = state if state is not None else self.new_state()
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        st["pos"] += len(tokens)
        e0 = self.w["embed"][tokens] * self.cfg["embedding"]["scale"]
        x = e0.clone()
        seen = []
        for r, (i, k) in enumerate(self.runs):
            layer = self.cfg["layers"][i]
            if k > 0 and i == self.loop["start"]:
                x = x + e0
            h = group_norm(x, self.w[f"l{i}.norm1"], self.groups, self.eps)
            p = self.sub(f"l{i}.mix.")
            if layer["type"] == "attention":
                x = x + block_attention(h, p, layer["mixer"], st["runs"][r])
            elif layer["type"] == "lightning":
                x = x + lightning(h, p, layer["mixer"], self.eps, st["runs"][r])
            else:
                raise ValueError(layer["type"])
            if layer.get("mlp") is not None:
                h = group_norm(x, self.w[f"l{i}.norm2"], self.groups, self.eps)
                p = self.sub(f"l{i}.mlp.")
                if layer["mlp"]["kind"] == "dense":
                    x = x + clamped_glu(h, p, layer["mlp"]["limit"])
                elif layer["mlp"]["kind"] == "moe":
                    x = x + mixture(h, p, layer["mlp"])
                else:
                    raise ValueError(layer["mlp"]["kind"])
            seen.append(x.clone())
        logits = group_norm(x, self.w["final.norm"], self.groups, self.eps) @ self.w["head"].T
        return (logits, torch.stack(seen)) if trace_layers else logits
