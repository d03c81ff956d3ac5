"""Nokipel on the GPU against the plain CPU restatement (oracle/nokipel.py): every mechanism alone at the kernel boundary,
then the engine — whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, reused pages and
state slots, block edges, far keys, long decoding, greedy generation through LLM.generate(). Configurations and weights
are made here; float32 serving is compared tightly, bfloat16 serving within rounding.

Routing is a discrete choice: in bfloat16 serving the router sees a rounded input, and a near-tie may fall the other way
than in the float64 oracle, after which the two runs are different models. The mechanism tests therefore leave out tokens
whose choice is a close call, and the bfloat16 ENGINE tests use corrections that decide the choice by themselves (the
weights still vary from token to token); float32 engine tests route freely."""
import json
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import nokipel as plain  # noqa: E402

F64 = torch.float64
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
    got, want = got.double().cpu(), want.double().cpu()
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-9)
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2.0 ** -8)])
@pytest.mark.parametrize("W,groups", [(48, 1), (352, 4), (70, 5), (1536, 2), (96, 8)])
def test_group_norm_with_the_adds_before_it(dtype, tol, W, groups):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(W)
    n, eps = 7, 1e-3
    x0 = torch.randn(n, W, generator=g) * torch.linspace(0.01, 30, W)          # parts of very different size
    a, b = torch.randn(n, W, generator=g).to(dtype), torch.randn(n, W, generator=g)
    w = (1 + 0.3 * torch.randn(W, generator=g)).to(dtype)
    x, out = dev(x0), torch.empty(n, W, device="cuda", dtype=dtype)
    ops_seq.add_group_norm(x, dev(w), groups, eps, out)
    close(x, x0, 0, "nothing to add")
    close(out, plain.group_norm(x0.double(), w.double(), groups, eps), tol, "norm alone")
    ops_seq.add_group_norm(x, dev(w), groups, eps, out, a=dev(a), b=dev(b))
    s = x0.double() + a.double() + b.double()
    close(x, s, 3e-7, "residual sum")
    close(out, plain.group_norm(s, w.double(), groups, eps), tol, "norm after both adds")
    ops_seq.add_group_norm(x, None, groups, eps, None, a=dev(a))
    close(x, s + a.double(), 3e-7, "add alone")
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device="cuda")
    sel = torch.empty(3, W, device="cuda", dtype=dtype)
    ops_seq.group_norm_rows(x, rows, 3, dev(w), groups, eps, sel)
    close(sel, plain.group_norm((s + a.double())[[6, 0, 3]], w.double(), groups, eps), tol, "selected rows")


def test_embedding_scaled_without_a_sinusoid():
    from nano_vllm_amd import ops_seq
    table = torch.randn(30, 52).to(torch.bfloat16)
    ids, pos = torch.randint(0, 30, (11,)), torch.arange(100, 111)
    x = torch.empty(11, 52, device="cuda")
    ops_seq.embed_sinusoid(dev(table), dev(ids), dev(pos), 3.25, 0.0, x, None)
    close(x, table.double()[ids] * 3.25, 1e-7)


def test_clamped_and_plain_gated_units():
    from nano_vllm_amd import ops_seq
    ff = 37
    gu = torch.cat([torch.linspace(-9, 9, 2 * ff * 5).view(5, 2 * ff), torch.randn(6, 2 * ff) * 4])
    for limit in (1.25, 7.0, 0.25):
        out = torch.empty(11, ff, device="cuda")
        ops_seq.glu_act(dev(gu), ff, out, kind=1, limit=limit, alpha=1.702)
        g, u = gu[:, :ff].double().clamp(max=limit), gu[:, ff:].double().clamp(-limit, limit)
        close(out, g * plain.sigmoid(1.702 * g) * (u + 1), 2e-6, f"limit {limit}")
    out = torch.empty(11, ff, device="cuda")
    ops_seq.glu_act(dev(gu), ff, out, kind=0)
    close(out, plain.silu(gu[:, :ff].double()) * gu[:, ff:].double(), 2e-6, "silu unit")


def attention_case(H, G, d, dv, size, rot, T, seed, scale=None):
    g = torch.Generator().manual_seed(seed)
    W = 24
    cfg = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale or d ** -0.5}
    if size:
        cfg["mask"] = {"size": size}
    if rot:
        cfg["rot"] = {"dims": rot, "base": 5000.0}
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    p = {"q": r(H * d, W) / W ** 0.5, "q.b": 0.3 * r(H * d), "k": r(G * d, W) / W ** 0.5, "k.b": 0.3 * r(G * d), "v": r(G * dv, W),
         "v.b": r(G * dv), "o": torch.eye(H * dv, dtype=F64)}
    return cfg, p, r(T, W)


def run_attention(cfg, p, h, dtype, block, cuts, path="auto"):
    """The product's kernels on the projections of h, cut into portions `cuts` (one sequence, pages in scrambled order)."""
    from nano_vllm_amd import ops_seq
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = (h @ p["q"].T + p["q.b"]).to(dtype)
    kv = torch.cat([h @ p["k"].T + p["k.b"], h @ p["v"].T + p["v.b"]], 1).to(dtype)
    pages = -(-T // block)
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(T))[:pages].to(torch.int32)
    kc = torch.full(((pages + 3) * block, G, d), 7.0, device="cuda", dtype=dtype)          # dirty pages
    vc = torch.full(((pages + 3) * block, G, dv), -7.0, device="cuda", dtype=dtype)
    rot = cfg.get("rot")
    freq = None
    if rot:
        freq = dev(torch.tensor([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)], dtype=torch.float32))
    ops_seq.load_library().nvs_window_attn_force_scalar({"auto": 0, "scalar": 1, "nolds": 2}[path])
    outs, at = [], 0
    try:
        for c in cuts:
            pos = torch.arange(at, at + c)
            slots = (order[pos // block].long() * block + pos % block).to(torch.int32)
            qd, kvd = dev(q[at:at + c]), dev(kv[at:at + c])
            ops_seq.knorm_kvstore(kvd[:, :G * d], kvd[:, G * d:], None, 0.0, G, d, dv, block, dev(slots), kc, vc, dev(pos), freq)
            out = torch.empty(c, H * dv, device="cuda", dtype=dtype)
            ops_seq.window_attn(qd, None, 0.0, None, kc, vc, dev(order.view(1, -1)), block, portions([c], [at], [0]), H, G, d, dv,
                                cfg["scale"], 0, out, cfg["mask"]["size"] if cfg.get("mask") else 0, freq)
            outs.append(out.cpu())
            at += c
    finally:
        ops_seq.load_library().nvs_window_attn_force_scalar(0)
    assert at == T
    return torch.cat(outs)


def plain_attention(cfg, p, h):
    G, d, dv = cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    return plain.block_attention(h, p, cfg, {"k": torch.zeros(0, G, d, dtype=F64), "v": torch.zeros(0, G, dv, dtype=F64)})


@pytest.mark.parametrize("dtype,path,tol", [(torch.float32, "auto", 2e-5), (torch.bfloat16, "auto", 2e-2), (torch.bfloat16, "nolds", 2e-2),
                                            (torch.bfloat16, "scalar", 2e-2)])
@pytest.mark.parametrize("H,G,d,dv,size,rot,block", [(12, 3, 64, 48, 50, 24, 64), (4, 4, 32, 48, 37, 32, 16), (6, 3, 40, 24, 0, 8, 32),
                                                     (2, 1, 128, 128, 64, 0, 64), (3, 1, 20, 36, 5, 20, 16)])
def test_block_masked_rotary_attention_against_the_plain_loop(H, G, d, dv, size, rot, block, dtype, path, tol):
    """One prompt portion, then short portions and single tokens: rotation of the leading dimensions only, grouped kv heads,
    blocks of positions that do not line up with pages or query tiles, head sizes that are not multiples of 8 or 16."""
    T = 150
    cfg, p, h = attention_case(H, G, d, dv, size, rot, T, seed=H * 100 + d)
    want = plain_attention(cfg, p, h)
    for cuts in ([T], [97, 2, 1, 1, 30, 1, 1, 1, 16]):
        close(run_attention(cfg, p, h, dtype, block, cuts, path), want, tol, f"cuts {cuts[:3]}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("size,block", [(100, 64), (50, 16), (64, 64), (33, 32)])
def test_a_standout_key_just_inside_and_just_outside_a_block_of_positions(size, block, dtype):
    """The last key of a block and the first of the next carry a value nobody else has, and every query looks for exactly
    these keys: queries of the same block must return the value, the queries across the edge must not — in a prompt and
    decoded one by one, also at page borders and for the first tokens of the sequence."""
    H, G, d, dv, T = 4, 2, 32, 16, 3 * size + 7
    cfg, p, h = attention_case(H, G, d, dv, size, 0, T, seed=size, scale=1.0)
    for name in ("q", "k", "v"):
        p[name] = torch.zeros_like(p[name])
    p["q.b"] = torch.zeros(H * d, dtype=F64)
    p["q.b"][0::d] = 8.0                                # every query asks for entry 0 of its key head
    marks = [0, size - 1, size, 2 * size - 1, 2 * size]
    p["k.b"], p["v.b"] = torch.zeros(G * d, dtype=F64), torch.zeros(G * dv, dtype=F64)
    want_rows = []
    for i in range(T):
        lo = (i // size) * size
        want_rows.append([j for j in marks if lo <= j <= i])
    # a marked position's key and value enter through an input column of its own; all other tokens have zero keys and values
    h = torch.zeros(T, 24, dtype=F64)
    for c, j in enumerate(marks):
        h[j, c] = 1.0
        p["k"][0::d, c] = 4.0
        p["v"][:, c] = 100.0 + j
    want = plain_attention(cfg, p, h)
    for i in (size - 1, size, size + 1, 2 * size - 1, 2 * size, 0, 1):            # the oracle itself shows the edge
        if want_rows[i]:
            assert want[i].max() > 99.0
        else:
            assert want[i].abs().max() < 1e-9
    for cuts in ([T], [size - 1] + [1] * (T - size + 1), [2, size - 3, 2, size - 1, 2] + [1] * (T - 2 * size - 2)):
        got = run_attention(cfg, p, h, dtype, block, cuts)
        close(got, want, 1e-5 if dtype == torch.float32 else 1e-2, f"cuts {cuts[:5]}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_without_a_mask(dtype):
    H, G, d, dv, T = 2, 1, 64, 32, 900
    cfg, p, h = attention_case(H, G, d, dv, 0, 16, T, seed=5, scale=0.25)
    # every query carries 0.7 u on top of its own small part; the key of token 3 alone carries 0.7 u (through an input column that
    # is zero elsewhere), and a value of its own: score 0.49 |u|^2 scale = 7.8 above hundreds of keys near zero
    h = h * 0.2
    h[:, 0] = 0.0
    h[3, 0] = 1.0
    u = torch.ones(d, dtype=F64)
    u[:16] = 0.0                                             # (outside the rotated dimensions: the distance does not matter)
    p["q.b"] = 0.7 * u.repeat(H)
    p["q"][:, 0], p["k"][:, 0], p["v"][:, 0] = 0.0, 0.7 * u.repeat(G) * (d / (d - 16)) , 9.0
    want = plain_attention(cfg, p, h)
    far = plain_attention(cfg, p, torch.cat([h[:3], h[4:]]))
    assert (want[-1] - far[-1]).abs().max() > 1.0, "the far key decides the last rows"
    got = run_attention(cfg, p, h, dtype, 64, [T - 4, 1, 1, 2])
    close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


def lightning_case(H, dk, dv, T, seed, decay=None):
    g = torch.Generator().manual_seed(seed)
    W = 20
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    cfg = {"heads": H, "dim": dk, "vdim": dv, "decay": decay or [0.5 + 0.499 * i / max(H - 1, 1) for i in range(H)]}
    p = {"q": r(H * dk, W) * 0.3, "k": r(H * dk, W) * 0.3, "v": r(H * dv, W) * 0.3, "g": r(H * dv, W) * 0.3, "norm": 1 + 0.2 * r(H * dv),
         "o": torch.eye(H * dv, dtype=F64)}
    return cfg, p, r(T, W)


def run_lightning(cfg, p, seqs, dtype, plan, eps):
    """seqs: list of inputs h; plan: steps of (sequence, tokens) pairs, every sequence in a state slot that held other data."""
    from nano_vllm_amd import ops_seq
    H, dk, dv = cfg["heads"], cfg["dim"], cfg["vdim"]
    w = dev(torch.cat([p["v"], p["k"], p["q"], p["g"]]).to(dtype))
    decay = dev(torch.tensor(cfg["decay"], dtype=torch.float32))
    S = torch.full((len(seqs) + 2, H, dv, dk), 55.0, device="cuda")
    slots = [len(seqs) + 1 - i for i in range(len(seqs))]
    at = [0] * len(seqs)
    got = [[] for _ in seqs]
    for step in plan:
        lens = [c for _, c in step]
        x = torch.cat([seqs[i][at[i]:at[i] + c] for i, c in step]).to(dtype)
        proj = torch.nn.functional.linear(dev(x), w)
        por = portions(lens, [at[i] for i, _ in step], [slots[i] for i, _ in step], max(lens))
        y = torch.empty(sum(lens), H * dv, device="cuda")
        ops_seq.decay_scan(proj, 0, H * dv, H * dv + H * dk, decay, H, dk, dv, por, S, y)
        out = torch.empty(sum(lens), H * dv, device="cuda", dtype=dtype)
        ops_seq.gated_group_norm(y, proj[:, H * dv + 2 * H * dk:], dev(p["norm"].to(dtype)), 1, eps, out, norm_first=True)
        o = 0
        for i, c in step:
            got[i].append(out[o:o + c].cpu())
            o += c
            at[i] += c
    return [torch.cat(g) for g in got]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,dk,dv", [(4, 64, 64), (3, 24, 40), (2, 128, 32), (5, 16, 16), (1, 36, 100)])
def test_decaying_recurrence_with_gate_and_norm_in_portions_and_dirty_slots(H, dk, dv, dtype, tol):
    eps = 1e-5
    cfg, p, _ = lightning_case(H, dk, dv, 1, seed=dk)
    g = torch.Generator().manual_seed(H)
    seqs = [torch.randn(n, 20, generator=g, dtype=F64) for n in (70, 33)]
    if dtype == torch.bfloat16:
        seqs = [s.to(dtype).double() for s in seqs]
        p = {k: v.to(dtype).double() for k, v in p.items()}
    want = [plain.lightning(s, p, cfg, eps, {"S": torch.zeros(H, dk, dv, dtype=F64)}) for s in seqs]
    plan = [[(0, 17), (1, 2)], [(1, 1), (0, 1)], [(0, 2), (1, 29)], [(0, 50), (1, 1)]]
    got = run_lightning(cfg, p, seqs, dtype, plan, eps)
    for a, b in zip(got, want):
        close(a, b, tol)


def test_decaying_recurrence_long_portion_in_segments_equals_the_token_loop():
    """A long portion of few heads is scanned in segments; a decay of exactly one and a fast one ride along."""
    H, dk, dv, T, eps = 3, 32, 48, 1300, 1e-5
    cfg, p, _ = lightning_case(H, dk, dv, 1, seed=9, decay=[1.0, 0.999, 0.3])
    g = torch.Generator().manual_seed(2)
    seqs = [torch.randn(T, 20, generator=g, dtype=F64), torch.randn(5, 20, generator=g, dtype=F64)]
    want = [plain.lightning(s, p, cfg, eps, {"S": torch.zeros(H, dk, dv, dtype=F64)}) for s in seqs]
    got = run_lightning(cfg, p, seqs, torch.float32, [[(0, 40), (1, 2)], [(0, 1200), (1, 3)], [(0, 60)]], eps)
    for a, b in zip(got, want):
        close(a, b, 3e-5)


def margins(z, corr, top, count, keep):
    """Per token: how close the choice is to falling the other way (the smallest gap between a winner and a loser, among
    groups and among entries)."""
    out = []
    for t in range(z.shape[0]):
        s = torch.softmax(z[t], 0)
        c = s + corr
        per = c.shape[0] // count
        best = torch.stack([c[g * per:(g + 1) * per].max() for g in range(count)]).sort(descending=True).values
        m = float(best[keep - 1] - best[keep]) if keep < count else 1.0
        kept = torch.topk(torch.stack([c[g * per:(g + 1) * per].max() for g in range(count)]), keep).indices.tolist()
        cand = torch.cat([c[g * per:(g + 1) * per] for g in kept]).sort(descending=True).values
        if top < cand.shape[0]:
            m = min(m, float(cand[top - 1] - cand[top]))
        out.append(m)
    return torch.tensor(out)


@pytest.mark.parametrize("total,top,count,keep", [(12, 3, 2, 1), (16, 4, 4, 2), (7, 2, 1, 1), (64, 6, 8, 3), (130, 8, 10, 4), (4, 4, 2, 2), (6, 1, 3, 1)])
def test_router_choice_groups_correction_and_weights(total, top, count, keep):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(total)
    n = 200
    z = torch.randn(n, total + 3, generator=g) * 2.0                 # (columns beyond `total` are not the router's)
    corr = torch.randn(total, generator=g) * 0.2 - 0.5                # choice scores are mostly NEGATIVE: a dropped group must not win as 0
    ids, wts = ops_seq.moe_route(dev(z), total, dev(corr), top, count, keep, 2.5)
    ok = margins(z[:, :total].double(), corr.double(), top, count, keep) > 1e-5
    assert ok.sum() > n * 0.9
    for t in range(n):
        if not ok[t]:
            continue
        idx, w = plain.route(z[t, :total].double(), corr.double(), top, count, keep, 2.5)
        assert sorted(ids[t].tolist()) == sorted(idx), t
        got = dict(zip(ids[t].tolist(), wts[t].tolist()))
        for e, we in zip(idx, w.tolist()):
            assert abs(got[e] - we) <= 3e-6 * 2.5, (t, e)
    ids2, wts2 = ops_seq.moe_route(dev(z), total, None, top, 1, 1, 1.0)          # no correction, no groups: plain top-k of softmax
    s = torch.softmax(z[:, :total].double(), -1)
    tk = torch.topk(s, top, -1)
    assert (torch.sort(ids2.cpu().long(), -1).values == torch.sort(tk.indices, -1).values).float().mean() > 0.99
    close(wts2.sum(-1), torch.ones(n), 1e-5)


def moe_case(W, E, ident, ff, top, count, keep, sff, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).double()
    cfg = {"expert": {"ff": ff}, "router": {"experts": E, "identity": ident, "top": top, "scale": 1.7, "groups": {"count": count, "keep": keep}}}
    p = {"router": r(E + ident, W) * 2 / W ** 0.5, "correction": r(E + ident) * 0.05}
    for e in range(E):
        p.update({f"e{e}.gate": r(ff, W) / W ** 0.5, f"e{e}.up": r(ff, W) / W ** 0.5, f"e{e}.down": r(W, ff) / ff ** 0.5})
    if sff:
        cfg["shared"] = {"ff": sff}
        p.update({"shared.gate": r(sff, W) / W ** 0.5, "shared.up": r(sff, W) / W ** 0.5, "shared.down": r(W, sff) / sff ** 0.5,
                  "shared.sg": r(1, W) / W ** 0.5})
    return cfg, p


@pytest.mark.parametrize("dtype,plain_kernel,tol", [(torch.float32, False, 2e-5), (torch.bfloat16, False, 2e-2), (torch.bfloat16, True, 2e-2)])
@pytest.mark.parametrize("W,E,ident,ff,top,count,keep,sff,n", [(352, 7, 1, 88, 3, 2, 1, 104, 50), (40, 5, 1, 24, 2, 3, 2, 0, 33),
                                                                (72, 4, 0, 200, 4, 1, 1, 17, 9), (64, 6, 2, 48, 2, 1, 1, 40, 700),
                                                                (50, 3, 3, 10, 3, 2, 2, 8, 21), (72, 3, 1, 40, 2, 1, 1, 0, 600),
                                                                (256, 2, 0, 160, 1, 1, 1, 0, 1100)])
def test_routed_experts_pass_through_and_shared_expert(W, E, ident, ff, top, count, keep, sff, n, dtype, plain_kernel, tol):
    """Sizes whose inner dimensions are not multiples of the matrix-core step (or of 8: the plain kernel), few and many rows per
    expert (all three tile sizes), experts nobody chooses, pass-through experts, no shared expert."""
    from nano_vllm_amd import ops_seq
    from nano_vllm_amd.mixers import RoutedExperts
    cfg, p = moe_case(W, E, ident, ff, top, count, keep, sff, seed=W + n)
    h = torch.randn(n, W, generator=torch.Generator().manual_seed(n)).to(torch.bfloat16).double()
    want = plain.mixture(h, p, cfg)
    z = h @ p["router"].T
    ok = margins(z, p["correction"], top, count, keep) > 1e-4
    torch.set_default_device("cuda")
    try:
        mod = RoutedExperts(W, E, ff, top, 1.7, ident, count, keep, sff).to(dtype)
        mod.router.data, mod.correction.data = mod.router.data.float(), mod.correction.data.float()
    finally:
        torch.set_default_device("cpu")
    loaders = mod.named_loaders()
    assert set(loaders) == set(p)
    for k, v in p.items():
        loaders[k](dev(v.float()))
    ops_seq.load_library().nvs_moe_force_plain(int(plain_kernel))
    try:
        got = mod(dev(h.to(dtype)))
    finally:
        ops_seq.load_library().nvs_moe_force_plain(0)
    assert ok.sum() >= n * 0.6
    close(got.cpu()[ok], want[ok], tol)


# ---------------------------------------------------------------------------------------------- the engine
def small_config(variant: int = 0) -> dict:
    """Three models: sizes that differ from each other in every respect, a repeated span (three times; twice; none), layers
    without a feed-forward, routers with and without groups / pass-through / shared experts, attention with and without
    blocks and rotation, kv heads equal to and fewer than the query heads."""
    def light(H, dk, dv, fast=0.6):
        return {"type": "lightning", "mixer": {"heads": H, "dim": dk, "vdim": dv, "decay": [fast + (0.999 - fast) * i / max(H - 1, 1) for i in range(H)]}}

    def attn(H, G, d, dv, size, rot):
        m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5}
        if size:
            m["mask"] = {"size": size}
        if rot:
            m["rot"] = {"dims": rot, "base": 10000.0 * rot}
        return {"type": "attention", "mixer": m}

    dense = lambda ff, limit: {"kind": "dense", "ff": ff, "limit": limit}

    def moe(E, ident, ff, top, count, keep, sff, scale):
        m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "identity": ident, "top": top, "scale": scale}}
        if count:
            m["router"]["groups"] = {"count": count, "keep": keep}
        if sff:
            m["shared"] = {"ff": sff}
        return m

    if variant == 0:
        layers = [dict(light(4, 32, 48), mlp=dense(144, 1.25)), dict(attn(6, 2, 32, 48, 40, 16), mlp=moe(6, 2, 56, 3, 2, 1, 40, 2.5)),
                  dict(light(2, 64, 16, 0.9), mlp=moe(5, 0, 24, 2, 0, 0, 0, 1.0)), dict(attn(2, 1, 80, 16, 7, 80), mlp=None),
                  dict(light(3, 16, 32), mlp=dense(80, 0.7))]
        loop, width, groups = {"start": 1, "stop": 4, "times": 3}, 112, 4
    elif variant == 1:
        layers = [dict(attn(4, 4, 24, 24, 0, 0), mlp=dense(100, 3.0)), dict(light(5, 24, 40), mlp=None),
                  dict(attn(8, 2, 16, 32, 64, 8), mlp=moe(9, 3, 32, 4, 4, 2, 16, 1.5))]
        loop, width, groups = None, 64, 1
    else:
        layers = [dict(light(2, 40, 40), mlp=moe(4, 0, 72, 1, 2, 1, 72, 3.0)), dict(attn(3, 1, 64, 64, 33, 32), mlp=dense(200, 1.0))]
        loop, width, groups = {"start": 0, "stop": 2, "times": 2}, 96, 3
    cfg = {"architecture": "Nokipel", "embedding": {"scale": 3.0 + variant}, "layers": layers,
           "norm": {"eps": 1e-6 * (1 + variant), "groups": groups}, "vocab": 211 + variant, "width": width}
    if loop:
        cfg["loop"] = loop
    return cfg


def decisive(raw: dict, tensors: dict) -> dict:
    """Corrections spaced wider than any softmax value: the choice no longer depends on the token (the weights still do)."""
    out = dict(tensors)
    for name, t in tensors.items():
        if name.endswith(".correction"):
            perm = torch.randperm(t.numel(), generator=torch.Generator().manual_seed(t.numel()))
            out[name] = (perm.float() * 2.0 - t.numel()).to(t.dtype)
    return out


@pytest.fixture(scope="module")
def checkpoints():
    from nano_vllm_amd.nokipel import random_tensors, write_synthetic_checkpoint
    root = tempfile.mkdtemp(prefix="nkp_")
    free = [write_synthetic_checkpoint(os.path.join(root, f"m{v}"), small_config(v), seed=21 + v) for v in range(3)]
    fixed = [write_synthetic_checkpoint(os.path.join(root, f"d{v}"), small_config(v), tensors=decisive(small_config(v), random_tensors(small_config(v), 21 + v)))
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


TOL = {"float32": 5e-5, "bfloat16": 4e-2}      # bf16: logits themselves are bf16 (2^-9 of their size), on top of the layers


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_decoding_agree_with_the_plain_model(checkpoints, variant, dtype):
    path = checkpoints[dtype][variant]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(variant)
    toks = torch.randint(0, ref.cfg["vocab"], (150,), generator=g).tolist()
    want, layers = ref.run(toks, trace_layers=True)
    want = want.numpy()
    scale = float(want.std())
    llm = engine(path, dtype)
    try:
        model = llm.model_runner.model
        model.layer_trace = []
        whole = llm.replay_step([{"id": "w", "tokens": toks, "want": list(range(150))}], ["w"])
        seen, model.layer_trace = model.layer_trace, None
        assert len(seen) == len(ref.runs)
        if dtype == "float32":                                       # layer run by layer run, in 32-bit
            for i, x in enumerate(seen):
                close(x, layers[i], 2e-5, f"residual after layer run {i}")
        assert rel(whole, want, scale) <= TOL[dtype]
        # portions of changing size, down to two tokens and single tokens, cut inside pages and blocks of positions
        for name, cuts in (("a", [2, 3, 2, 40, 1, 1, 17, 2, 64, 18]), ("b", [149, 1]), ("c", [1] * 60 + [90])):
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
    """Five requests through four state slots and a pool that cannot hold them all at once: prompts in portions beside
    single tokens of others, requests that sit out steps, ends that free pages for the next request."""
    path = checkpoints["float32"][0]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(4)
    lens = {"p": 130, "q": 61, "r": 3, "s": 97, "t": 200}
    toks = {k: torch.randint(0, ref.cfg["vocab"], (n,), generator=g).tolist() for k, n in lens.items()}
    want = {k: ref.run(v).numpy() for k, v in toks.items()}
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


def test_long_decoding_across_many_blocks_of_positions_and_pages(checkpoints):
    path = checkpoints["float32"][1]
    ref = plain.Model.load(path)
    toks = torch.randint(0, ref.cfg["vocab"], (330,), generator=torch.Generator().manual_seed(8)).tolist()
    want = ref.run(toks).numpy()
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
    """LLM.generate() with token-id prompts: scheduler, chunked prefill, block manager, state slots, sampler; eagerly and
    with decode steps replayed from captured graphs. Where the plain model's two best logits are a close call the
    comparison stops (a different token is then a different, equally valid continuation)."""
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
            top = torch.topk(row, 2)
            if float(top.values[0] - top.values[1]) > margin * float(row.std()):
                assert t == int(top.indices[0])
                checked += 1
    assert checked >= 30


def test_sampled_generation_is_reproducible_and_preemption_recomputes_pages_and_state(checkpoints):
    """A pool so small that running sequences are preempted: a preempted sequence loses its pages AND its state slot (every
    run of a repeated layer included) and is recomputed from its first token; greedy results must not change, and a sampled
    run repeats itself."""
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
    wa, wb = ref.run(a).numpy(), ref.run(b).numpy()
    scale = float(wa.std())
    got = [np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, ref.cfg["vocab"]) for i in range(3)]
    assert rel(got[0], wa[[0, 63]], scale) <= 5e-5 and rel(got[1], wb[[39]], scale) <= 5e-5
    assert rel(got[2], np.stack([wb[40], wa[89]]), scale) <= 5e-5
