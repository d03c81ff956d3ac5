"""Plain, slow restatement of the Foduzen design on the CPU (test infrastructure only; shares no code with the
product path under nano_vllm_amd/). One function per mechanism, token loops where the design has a recurrence,
float64 throughout. `Model.run(tokens, state)` continues a sequence from `state`, so the same functions serve as
the oracle for whole prompts, portions and single decoded tokens.

Notation: T tokens of a portion, W model width, eps the layer's epsilon.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def xielu(z, p, q):
    """Quadratic above zero, saturating below, linear coefficient 1/2 on both sides:
    a = softplus(p), b = 1/2 + softplus(q);  f(z) = a z^2 + z/2 (z > 0),  b (e^z - 1 - z) + z/2 (z <= 0)."""
    ap, aq = softplus(p), 0.5 + softplus(q)
    zn = torch.clamp(z, max=0.0)
    return torch.where(z > 0, ap * z * z + 0.5 * z, aq * (torch.exp(zn) - 1.0 - zn) + 0.5 * z)


def embed(table, tokens, positions, scale):
    """table[token] * scale + sinusoid: entry 2i = sin(p * 10000^(-2i/W)), entry 2i+1 = cos of the same angle."""
    x = table[tokens] * scale
    W = table.shape[1]
    i = torch.arange((W + 1) // 2, dtype=F64)
    ang = positions.to(F64)[:, None] * torch.pow(torch.tensor(10000.0, dtype=F64), -2.0 * i / W)[None, :]
    pe = torch.zeros(len(tokens), W, dtype=F64)
    pe[:, 0::2] = torch.sin(ang)[:, : (W + 1) // 2]
    pe[:, 1::2] = torch.cos(ang)[:, : W // 2]
    return x + pe


def causal_conv(x, w, b, tail):
    """Per-channel causal convolution. x [T, C]; w [C, taps] (last column multiplies the current token); `tail` holds
    the taps - 1 inputs before x (zeros at the start of a sequence). Returns (y [T, C], new tail)."""
    taps = w.shape[1]
    full = torch.cat([tail, x], 0)                       # [taps - 1 + T, C]
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(taps):
            y[t] += w[:, j] * full[t + j]
        y[t] += b
    return y, full[full.shape[0] - (taps - 1):].clone()


def rglru(u, y, p, blocks, state):
    """Real-gated linear recurrent unit over u [T, C] with output branch y; state S [C]."""
    T, C = u.shape
    bw = C // blocks
    out = torch.zeros_like(u)
    sp = softplus(p["lam"])
    S = state
    for t in range(T):
        ub = u[t].view(blocks, bw)
        r = sigmoid(torch.einsum("boi,bi->bo", p["ra"], ub) + p["ra.b"]).reshape(C)
        i = sigmoid(torch.einsum("boi,bi->bo", p["ri"], ub) + p["ri.b"]).reshape(C)
        log_a = -8.0 * r * sp
        a = torch.exp(log_a)
        S = a * S + torch.sqrt(1.0 - a * a) * i * u[t]
        out[t] = S * y[t]
    return out, S


def rglru_mixer(h, p, cfg, st):
    y = gelu_tanh(h @ p["y"].T + p["y.b"])
    u, st["conv"] = causal_conv(h @ p["x"].T + p["x.b"], p["conv"], p["conv.b"], st["conv"])
    s, st["S"] = rglru(u, y, p, cfg["blocks"], st["S"])
    return s @ p["o"].T


def window_attention(h, p, cfg, eps, st):
    """Sliding-window softmax attention with per-head q/k RMS norm, no rotation, sigmoid output gate."""
    H, G, d, dv, win = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"], cfg["mask"]["size"]
    T = h.shape[0]
    q = (h @ p["q"].T + p["q.b"]).view(T, H, d)
    k = (h @ p["k"].T + p["k.b"]).view(T, G, d)
    v = (h @ p["v"].T + p["v.b"]).view(T, G, dv)
    q = rms(q, eps) * p["q.norm"]
    k = rms(k, eps) * p["k.norm"]
    st["k"] = torch.cat([st["k"], k], 0)
    st["v"] = torch.cat([st["v"], v], 0)
    K, V = st["k"], st["v"]
    n0 = K.shape[0] - T                                  # position of the portion's first token
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        i = n0 + t
        lo = max(0, i - win + 1)
        for hh in range(H):
            g = hh // (H // G)
            s = (K[lo:i + 1, g] @ q[t, hh]) * cfg["scale"]
            w = torch.softmax(s, 0)
            out[t, hh] = w @ V[lo:i + 1, g]
    gate = sigmoid(h @ p["g"].T)
    return (out.reshape(T, H * dv) * gate) @ p["o"].T + p["o.b"]


def ssd_mixer(h, p, cfg, eps, st):
    """State-space-duality mixer in its recurrent form. State S [heads, N, vdim]."""
    Hn, P, N, G = cfg["heads"], cfg["vdim"], cfg["state"], cfg["groups"]
    inner = Hn * P
    T = h.shape[0]
    zxbcdt = h @ p["in"].T
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc, st["conv"] = causal_conv(xbc, p["conv"], p["conv.b"], st["conv"])
    xbc = silu(xbc)
    x = xbc[:, :inner].view(T, Hn, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + p["dt_bias"])
    A = -torch.exp(p["A_log"])
    S = st["S"]
    y = torch.zeros(T, Hn, P, dtype=F64)
    for t in range(T):
        for hh in range(Hn):
            g = hh // (Hn // G)
            S[hh] = torch.exp(A[hh] * dt[t, hh]) * S[hh] + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S[hh].T @ C[t, g] + p["D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    ng = cfg["norm_groups"]
    y = (rms(y.view(T, ng, inner // ng), eps)).reshape(T, inner) * p["norm"]
    return y @ p["o"].T


def parallel_mixer(h, p, cfg, eps, st):
    left = window_attention(h, {k[5:]: v for k, v in p.items() if k.startswith("left.")}, cfg["left"], eps, st["left"])
    right = ssd_mixer(h, {k[6:]: v for k, v in p.items() if k.startswith("right.")}, cfg["right"], eps, st["right"])
    return 0.5 * (rms(left, eps) * p["left.out"] + rms(right, eps) * p["right.out"])


def dense_ff(h, p):
    return xielu(h @ p["up"].T, p["act"][0], p["act"][1]) @ p["down"].T


class Model:
    """Weights as float64 tensors by name; config as the parsed config.json."""

    def __init__(self, config: dict, tensors: dict):
        self.cfg = config
        self.w = {k: v.to(F64) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]

    @classmethod
    def load(cls, path: str) -> "Model":
        from safetensors.torch import load_file
        with open(os.path.join(path, "config.json")) as fh:
            cfg = json.load(fh)
        return cls(cfg, load_file(os.path.join(path, "model.safetensors")))

    def sub(self, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def new_state(self) -> dict:
        st = {"pos": 0, "layers": []}
        for layer in self.cfg["layers"]:
            m = layer["mixer"]
            if layer["type"] == "rglru":
                st["layers"].append({"conv": torch.zeros(m["conv"] - 1, m["width"], dtype=F64),
                                     "S": torch.zeros(m["width"], dtype=F64)})
            else:
                le, ri = m["left"], m["right"]
                ch = ri["heads"] * ri["vdim"] + 2 * ri["groups"] * ri["state"]
                st["layers"].append({
                    "left": {"k": torch.zeros(0, le["kv_heads"], le["dim"], dtype=F64),
                             "v": torch.zeros(0, le["kv_heads"], le["vdim"], dtype=F64)},
                    "right": {"conv": torch.zeros(ri["conv"] - 1, ch, dtype=F64),
                              "S": torch.zeros(ri["heads"], ri["state"], ri["vdim"], dtype=F64)}})
        return st

    def run(self, tokens, state: dict | None = None, trace_layers: bool = False):
        """Logits [T, vocab] of the portion `tokens`, continuing `state` (updated in place)."""
        st = state if state is not None else self.new_state()
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        pos = torch.arange(st["pos"], st["pos"] + len(tokens))
        st["pos"] += len(tokens)
        x = embed(self.w["embed"], tokens, pos, self.cfg["embedding"]["scale"])
        seen = []
        for i, layer in enumerate(self.cfg["layers"]):
            p = self.sub(f"l{i}.mix.")
            if layer["type"] == "rglru":
                m = rglru_mixer(x, p, layer["mixer"], st["layers"][i])
            elif layer["type"] == "parallel":
                m = parallel_mixer(x, p, layer["mixer"], self.eps, st["layers"][i])
            else:
                raise ValueError(layer["type"])
            x = x + rms(m, self.eps) * self.w[f"l{i}.norm1"]
            if layer["mlp"] is not None:
                assert layer["mlp"]["kind"] == "dense"
                x = x + rms(dense_ff(x, self.sub(f"l{i}.mlp.")), self.eps) * self.w[f"l{i}.norm2"]
            seen.append(x.clone())
        logits = (rms(x, self.eps) * self.w["final.norm"]) @ self.w["head"].T
        return (logits, torch.stack(seen)) if trace_layers else logits
