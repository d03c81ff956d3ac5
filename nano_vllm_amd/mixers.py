"""Sequence mixers and feed-forwards beyond full attention, as layers any model of the package can compose:

  WindowAttention     paged softmax attention with a sliding window, any query / value head size, optional per-head
                      q/k RMS norm, optional sigmoid output gate, no rotation (positions do not enter the scores)
  SSDMixer            state-space-duality (Mamba-2 style) mixer: stateful causal convolution + SiLU, the recurrence in
                      32-bit, gate-then-group-norm
  RGLRUMixer          recurrent block with a real-gated linear recurrent unit (block-diagonal gates)
  ParallelMixer       two mixers on the same input; the caller averages their RMS-normed outputs
  XIELUFeedForward    up -> xIELU -> down

Every constant a design may change is a constructor argument. Matrix products are the vendor library's (F.linear /
baddbmm); everything else is a kernel of libnvl_seq.so (ops_seq). Layers read the step's packed-portion description from
the attention-metadata context (`portions`, `slot_mapping`, `block_tables`); the runner injects the per-layer cache and
state tensors named by `kv_shapes()` / `state_shapes()`.

Weights live in fused tensors (one in-projection per mixer); `named_loaders()` maps a checkpoint's tensor names to
functions that copy into them.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops_seq
from .attn_meta import get_context


def _param(*shape, dtype=None):
    return nn.Parameter(torch.zeros(*shape, dtype=dtype), requires_grad=False)


def _copy_into(dst: torch.Tensor):
    def load(t: torch.Tensor):
        assert tuple(t.shape) == tuple(dst.shape), (tuple(t.shape), tuple(dst.shape))
        dst.copy_(t.to(dst.dtype))
    return load


class WindowAttention(nn.Module):
    """Consumes q | k | v | gate column ranges of the owner's fused projection output."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, eps: float,
                 qk_norm: bool = True, block_size: int = 256):
        super().__init__()
        assert heads % kv_heads == 0 and dim <= 256 and vdim <= 256
        self.H, self.G, self.d, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.window, self.eps, self.block_size = float(scale), int(window), eps, block_size
        self.q_norm = _param(dim) if qk_norm else None
        self.k_norm = _param(dim) if qk_norm else None
        self.k_cache = self.v_cache = None            # [pages * block_size, G, d] / [..., G, dv] (values page-transposed), from the runner

    @property
    def widths(self) -> tuple[int, int, int, int]:
        """Columns of q, k, v and the gate in the fused projection."""
        return self.H * self.d, self.G * self.d, self.G * self.dv, self.H * self.dv

    def kv_shapes(self) -> tuple[tuple, tuple]:
        """Per-token shapes of this layer's K and V pages."""
        return (self.G, self.d), (self.G, self.dv)

    def forward(self, q, k, v, gate) -> torch.Tensor:
        ctx = get_context()
        ops_seq.knorm_kvstore(k, v, self.k_norm, self.eps, self.G, self.d, self.dv, self.block_size, ctx.slot_mapping, self.k_cache,
                              self.v_cache)
        out = torch.empty(q.shape[0], self.H * self.dv, dtype=q.dtype, device=q.device)
        ops_seq.window_attn(q, self.q_norm, self.eps, gate, self.k_cache, self.v_cache, ctx.block_tables, self.block_size,
                            ctx.portions, self.H, self.G, self.d, self.dv, self.scale, self.window, out)
        return out


class SSDMixer(nn.Module):
    """Consumes z | x B C | dt column ranges of the owner's fused projection output; returns the normed gated y."""

    def __init__(self, heads: int, vdim: int, state: int, groups: int, conv: int, norm_groups: int, eps: float):
        super().__init__()
        assert heads % groups == 0 and (heads * vdim) % norm_groups == 0
        self.heads, self.P, self.N, self.groups, self.taps, self.norm_groups, self.eps = heads, vdim, state, groups, conv, norm_groups, eps
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        self.conv_w, self.conv_b = _param(self.channels, conv), _param(self.channels)
        self.dt_bias, self.A_log, self.D = _param(heads), _param(heads), _param(heads)
        self.norm = _param(self.inner)
        self.conv_state = self.rec_state = None

    @property
    def in_width(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.N + self.heads

    def state_shapes(self) -> dict:
        return {"conv_state": (self.taps - 1, self.channels), "rec_state": (self.heads, self.P, self.N)}

    def forward(self, proj: torch.Tensor, col0: int) -> torch.Tensor:
        """`proj`: the fused projection output; this mixer's columns start at col0."""
        por = get_context().portions
        n = proj.shape[0]
        z = proj[:, col0:col0 + self.inner]
        xbc_in = proj[:, col0 + self.inner:col0 + self.inner + self.channels]
        xbc = torch.empty(n, self.channels, dtype=torch.float32, device=proj.device)
        ops_seq.causal_conv(xbc_in, self.conv_w, self.conv_b, 1, por, self.conv_state, xbc)
        y = torch.empty(n, self.inner, dtype=torch.float32, device=proj.device)
        ops_seq.ssd_scan(xbc, proj, col0 + self.inner + self.channels, self.dt_bias, self.A_log, self.D, self.heads, self.P, self.N,
                         self.groups, por, self.rec_state, y)
        out = torch.empty(n, self.inner, dtype=proj.dtype, device=proj.device)
        ops_seq.gated_group_norm(y, z, self.norm, self.norm_groups, self.eps, out)
        return out


class ParallelMixer(nn.Module):
    """Windowed attention and a state-space mixer side by side on the same input: ONE fused in-projection
    [q | k | v | gate | z | x B C | dt], two out-projections. Returns both branch outputs; the residual kernel
    norms each with `left_out` / `right_out`, halves their sum and norms the result."""

    def __init__(self, width: int, left: dict, right: dict, eps: float, block_size: int, dtype):
        super().__init__()
        self.attn = WindowAttention(left["heads"], left["kv_heads"], left["dim"], left["vdim"], left["scale"],
                                    left["mask"]["size"], eps, qk_norm=True, block_size=block_size)
        self.ssd = SSDMixer(right["heads"], right["vdim"], right["state"], right["groups"], right["conv"], right["norm_groups"], eps)
        self.cols = list(self.attn.widths) + [self.ssd.in_width]
        total = sum(self.cols)
        self.in_w, self.in_b = _param(total, width), _param(total)
        hdv = self.attn.H * self.attn.dv
        self.left_o, self.left_o_b = _param(width, hdv), _param(width)
        self.right_o = _param(width, self.ssd.inner)
        self.left_out, self.right_out = _param(width), _param(width)

    def named_loaders(self) -> dict:
        a, s = self.attn, self.ssd
        q, k, v, g, _ = self.cols
        o = [0, q, q + k, q + k + v, q + k + v + g]
        return {
            "left.q": _copy_into(self.in_w[o[0]:o[1]]), "left.q.b": _copy_into(self.in_b[o[0]:o[1]]),
            "left.k": _copy_into(self.in_w[o[1]:o[2]]), "left.k.b": _copy_into(self.in_b[o[1]:o[2]]),
            "left.v": _copy_into(self.in_w[o[2]:o[3]]), "left.v.b": _copy_into(self.in_b[o[2]:o[3]]),
            "left.g": _copy_into(self.in_w[o[3]:o[4]]), "right.in": _copy_into(self.in_w[o[4]:]),
            "left.q.norm": _copy_into(a.q_norm), "left.k.norm": _copy_into(a.k_norm),
            "left.o": _copy_into(self.left_o), "left.o.b": _copy_into(self.left_o_b),
            "right.conv": _copy_into(s.conv_w), "right.conv.b": _copy_into(s.conv_b), "right.dt_bias": _copy_into(s.dt_bias),
            "right.A_log": _copy_into(s.A_log), "right.D": _copy_into(s.D), "right.norm": _copy_into(s.norm),
            "right.o": _copy_into(self.right_o), "left.out": _copy_into(self.left_out), "right.out": _copy_into(self.right_out),
        }

    def forward(self, xh: torch.Tensor):
        proj = F.linear(xh, self.in_w, self.in_b)
        q, k, v, g, _ = self.cols
        att = self.attn(proj[:, :q], proj[:, q:q + k], proj[:, q + k:q + k + v], proj[:, q + k + v:q + k + v + g])
        left = F.linear(att, self.left_o, self.left_o_b)
        right = F.linear(self.ssd(proj, q + k + v + g), self.right_o)
        return left, right


class RGLRUMixer(nn.Module):
    """y = gelu_tanh(W_y h + b), u = conv(W_x h + b); per block of channels r = sigmoid(R u_b + b_r), i = sigmoid(I u_b + b_i);
    a = exp(-c r softplus(lam)); S <- a S + sqrt(1 - a^2) i u; out = W_o (S * y). The gates' matrices are kept in 32-bit
    and applied to the 32-bit convolution output."""

    def __init__(self, width: int, channels: int, blocks: int, conv: int, dtype, c: float = 8.0):
        super().__init__()
        assert channels % blocks == 0
        self.C, self.blocks, self.taps, self.c = channels, blocks, conv, float(c)
        bw = channels // blocks
        self.in_w, self.in_b = _param(2 * channels, width), _param(2 * channels)            # [y | x]
        self.conv_w, self.conv_b = _param(channels, conv), _param(channels)
        self.gate_w = _param(blocks, bw, 2 * bw, dtype=torch.float32)                       # per block [in, r-out | i-out]
        self.gate_b = _param(blocks, 1, 2 * bw, dtype=torch.float32)
        self.lam = _param(channels)
        self.o_w = _param(width, channels)
        self.conv_state = self.rec_state = None

    def state_shapes(self) -> dict:
        return {"conv_state": (self.taps - 1, self.C), "rec_state": (self.C,)}

    def named_loaders(self) -> dict:
        C, bw = self.C, self.C // self.blocks

        def gate(lo):
            def load(t):                                   # [blocks, out, in] -> [blocks, in, out]
                self.gate_w[:, :, lo:lo + bw].copy_(t.to(torch.float32).transpose(1, 2))
            return load

        def gate_bias(lo):
            def load(t):
                self.gate_b[:, 0, lo:lo + bw].copy_(t.to(torch.float32))
            return load
        return {
            "y": _copy_into(self.in_w[:C]), "y.b": _copy_into(self.in_b[:C]), "x": _copy_into(self.in_w[C:]),
            "x.b": _copy_into(self.in_b[C:]), "conv": _copy_into(self.conv_w), "conv.b": _copy_into(self.conv_b),
            "ra": gate(0), "ra.b": gate_bias(0), "ri": gate(bw), "ri.b": gate_bias(bw), "lam": _copy_into(self.lam),
            "o": _copy_into(self.o_w),
        }

    def forward(self, xh: torch.Tensor) -> torch.Tensor:
        por = get_context().portions
        n, C, bw = xh.shape[0], self.C, self.C // self.blocks
        proj = F.linear(xh, self.in_w, self.in_b)
        u = torch.empty(n, C, dtype=torch.float32, device=xh.device)
        ops_seq.causal_conv(proj[:, C:], self.conv_w, self.conv_b, 0, por, self.conv_state, u)
        gates = torch.baddbmm(self.gate_b, u.view(n, self.blocks, bw).transpose(0, 1), self.gate_w)     # [blocks, n, 2 bw] fp32
        s = torch.empty(n, C, dtype=xh.dtype, device=xh.device)
        ops_seq.rglru_scan(gates, u, proj[:, :C], self.lam, self.c, self.blocks, por, self.rec_state, s)
        return F.linear(s, self.o_w)


class XIELUFeedForward(nn.Module):

    def __init__(self, width: int, ff: int, beta: float = 0.5):
        super().__init__()
        self.up, self.down, self.act, self.beta = _param(ff, width), _param(width, ff), _param(2), beta

    def named_loaders(self) -> dict:
        return {"up": _copy_into(self.up), "down": _copy_into(self.down), "act": _copy_into(self.act)}

    def forward(self, xh: torch.Tensor) -> torch.Tensor:
        return F.linear(ops_seq.xielu(F.linear(xh, self.up), self.act, self.beta), self.down)
