"""Foduzen on the GPU against the plain CPU restatement (oracle/foduzen.py): every mechanism alone at the kernel boundary,
then the engine — whole prompts, portions down to two tokens, token-by-token decoding, unequal batches, reused pages and
state slots, window edges, far keys, long decoding, greedy generation through LLM.generate(). Configurations and weights
are made here; float32 serving is compared tightly, bfloat16 serving within rounding."""
import json
import os
import tempfile

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import foduzen as plain  # noqa: E402

F64 = torch.float64


def dev(t, dtype=None):
    return t.to("cuda", dtype=dtype or t.dtype).contiguous()


def portions(lens, ctx0, slots):
    from nano_vllm_amd.ops_seq import Portions
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tseq = np.repeat(np.arange(len(lens)), lens).astype(np.int32)
    i32 = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device="cuda")
    return Portions(i32(cu), i32(ctx0), i32(slots), i32(tseq), len(lens), int(cu[-1]))


def close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-9)
    assert err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_sinusoid(dtype):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(1)
    V, W, n = 50, 70, 33                       # a width that is not a multiple of the wavefront
    table = torch.randn(V, W, generator=g).to(dtype)
    ids = torch.randint(0, V, (n,), generator=g)
    pos = torch.cat([torch.arange(0, 20), torch.tensor([511, 512, 1000, 4095, 4096, 9999, 20000, 3, 2, 1, 0, 77, 78])])
    x = torch.empty(n, W, device="cuda")
    xh = torch.empty(n, W, device="cuda", dtype=dtype)
    ops_seq.embed_sinusoid(dev(table), dev(ids), dev(pos), 7.5, 10000.0, x, xh)
    want = plain.embed(table.to(F64), ids, pos, 7.5)
    # the angle is a 32-bit product: at position p its rounding alone moves sin / cos by up to p * 2^-24
    assert (x.double().cpu() - want).abs().max().item() <= 2e-5 + 20000 * 2.0 ** -21
    close(x[:20], want[:20], 2e-6, "first positions")
    close(xh, x, 2.0 ** -8 if dtype == torch.bfloat16 else 0, "activation copy")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1e-5)])
@pytest.mark.parametrize("W", [48, 256, 1536])
def test_output_norm_with_residual_one_and_two_branches(dtype, tol, W):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(W)
    n, eps = 9, 1e-3
    x0 = torch.randn(n, W, generator=g)
    m, m2 = (torch.randn(n, W, generator=g) * 3).to(dtype), (torch.randn(n, W, generator=g) * 0.01).to(dtype)
    w1, w2 = (1 + 0.3 * torch.randn(W, generator=g)).to(dtype), (1 + 0.3 * torch.randn(W, generator=g)).to(dtype)
    gs = torch.tensor([1.7]).to(dtype)
    x = dev(x0)
    xh = torch.empty(n, W, device="cuda", dtype=dtype)
    ops_seq.norm_residual(x, dev(m), dev(gs), eps, xh)
    close(x, x0.double() + plain.rms(m.double(), eps) * gs.double(), tol, "one branch")
    x = dev(x0)
    ops_seq.norm_residual(x, dev(m), dev(gs), eps, xh, m2=dev(m2), w1=dev(w1), w2=dev(w2))
    mean = 0.5 * (plain.rms(m.double(), eps) * w1.double() + plain.rms(m2.double(), eps) * w2.double())
    close(x, x0.double() + plain.rms(mean, eps) * gs.double(), tol, "two branches")
    close(xh, x, 2.0 ** -8 if dtype == torch.bfloat16 else 0, "activation copy")
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device="cuda")
    out = torch.empty(3, W, device="cuda", dtype=dtype)
    ops_seq.scalar_norm_rows(x, rows, 3, dev(gs), eps, out)
    close(out, plain.rms(x.double().cpu()[[8, 0, 3]], eps) * gs.double(), 2.0 ** -8 if dtype == torch.bfloat16 else tol, "row norm")


def test_xielu_both_sides_and_large_arguments():
    from nano_vllm_amd import ops_seq
    z = torch.cat([torch.linspace(-30, 30, 601), torch.tensor([0.0, -0.0, 1e-6, -1e-6])])
    for p, q in ((0.3, -0.8), (-2.0, 1.5)):
        pq = torch.tensor([p, q])
        got = ops_seq.xielu(dev(z.clone()), dev(pq))
        close(got, plain.xielu(z.double(), pq[0].double(), pq[1].double()), 2e-6, f"xielu p={p} q={q}")


@pytest.mark.parametrize("taps,act", [(2, 0), (3, 1), (4, 1), (1, 0)])
def test_causal_convolution_carries_its_tail_across_portions_and_slots(taps, act):
    """Two sequences in interleaved portions (lengths around taps - 1, down to one token), in slots that held other
    data before: the outputs must equal one pass over each whole sequence."""
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(taps)
    C, stride = 37, 50
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    seqs = [torch.randn(23, C, generator=g), torch.randn(17, C, generator=g)]
    want = []
    for s in seqs:
        y, _ = plain.causal_conv(s.double(), w.double(), b.double(), torch.zeros(taps - 1, C, dtype=F64))
        want.append(plain.silu(y) if act else y)
    state = torch.full((5, max(taps - 1, 0), C), 123.0, device="cuda")           # dirty slots
    cuts = [[1, 1, 2, 5, 1, 13], [3, 1, 1, 12]]
    at = [0, 0]
    got = [[], []]
    for step in range(6):
        live = [i for i in (0, 1) if step < len(cuts[i])]
        lens = [cuts[i][step] for i in live]
        buf = torch.zeros(sum(lens), stride)
        o = 0
        for i, L in zip(live, lens):
            buf[o:o + L, 5:5 + C] = seqs[i][at[i]:at[i] + L]
            o += L
        por = portions(lens, [at[i] for i in live], [4 if i == 0 else 2 for i in live])
        out = torch.empty(sum(lens), C, device="cuda")
        ops_seq.causal_conv(dev(buf)[:, 5:5 + C], dev(w), dev(b), act, por, state, out)
        o = 0
        for i, L in zip(live, lens):
            got[i].append(out[o:o + L].cpu())
            o += L
            at[i] += L
    for i in (0, 1):
        close(torch.cat(got[i]), want[i], 3e-6, f"sequence {i}")


def test_gated_recurrence_against_the_token_loop_with_slow_decay():
    """Decays close to one (the state remembers hundreds of tokens) and a portion split in the middle."""
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(5)
    C, blocks, T = 96, 3, 300
    bw = C // blocks
    p = {"ra": torch.randn(blocks, bw, bw, generator=g) * 0.2, "ra.b": torch.randn(blocks, bw, generator=g),
         "ri": torch.randn(blocks, bw, bw, generator=g) * 0.2, "ri.b": torch.randn(blocks, bw, generator=g),
         "lam": -7.0 + 5 * torch.rand(C, generator=g)}
    u, ypre = torch.randn(T, C, generator=g), torch.randn(T, C, generator=g)
    want, S = plain.rglru(u.double(), plain.gelu_tanh(ypre.double()), {k: v.double() for k, v in p.items()}, blocks,
                          torch.zeros(C, dtype=F64))
    ub = u.double().view(T, blocks, bw)
    gr = torch.einsum("boi,tbi->bto", p["ra"].double(), ub) + p["ra.b"].double()[:, None]
    gi = torch.einsum("boi,tbi->bto", p["ri"].double(), ub) + p["ri.b"].double()[:, None]
    state = torch.full((3, C), -9.0, device="cuda")
    outs = []
    for lo, hi in ((0, 131), (131, 133), (133, 300)):
        gates = dev(torch.cat([gr[:, lo:hi], gi[:, lo:hi]], -1).float())
        out = torch.empty(hi - lo, C, device="cuda")
        ops_seq.rglru_scan(gates, dev(u[lo:hi]), dev(ypre[lo:hi]), dev(p["lam"]), 8.0, blocks, portions([hi - lo], [lo], [1]), state, out)
        outs.append(out)
    close(torch.cat(outs), want, 2e-5, "outputs")
    close(state[1], S, 2e-5, "final state")
    assert (state[0] == -9).all() and (state[2] == -9).all()


@pytest.mark.parametrize("heads,P,N,G", [(4, 48, 48, 2), (3, 64, 128, 1), (2, 16, 8, 2), (6, 32, 20, 3)])
def test_state_space_recurrence_against_the_token_loop(heads, P, N, G):
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(heads * P)
    T, inner = 90, heads * P
    xbc = torch.randn(T, inner + 2 * G * N, generator=g)
    proj = torch.randn(T, 11 + heads, generator=g)
    dt_bias, A_log, D = torch.randn(heads, generator=g) - 2, torch.randn(heads, generator=g) - 1, torch.randn(heads, generator=g)
    x = xbc[:, :inner].double().view(T, heads, P)
    B = xbc[:, inner:inner + G * N].double().view(T, G, N)
    Cm = xbc[:, inner + G * N:].double().view(T, G, N)
    dt = plain.softplus(proj[:, 11:].double() + dt_bias.double())
    S = torch.zeros(heads, N, P, dtype=F64)
    want = torch.zeros(T, heads, P, dtype=F64)
    for t in range(T):
        for h in range(heads):
            gg = h // (heads // G)
            S[h] = torch.exp(-torch.exp(A_log[h].double()) * dt[t, h]) * S[h] + dt[t, h] * torch.outer(B[t, gg], x[t, h])
            want[t, h] = S[h].T @ Cm[t, gg] + D[h].double() * x[t, h]
    state = torch.full((2, heads, P, N), 5.0, device="cuda")
    outs = []
    for lo, hi in ((0, 1), (1, 3), (3, 50), (50, 90)):
        y = torch.empty(hi - lo, inner, device="cuda")
        ops_seq.ssd_scan(dev(xbc[lo:hi]), dev(proj[lo:hi]), 11, dev(dt_bias), dev(A_log), dev(D), heads, P, N, G,
                         portions([hi - lo], [lo], [1]), state, y)
        outs.append(y)
    close(torch.cat(outs).view(T, heads, P), want, 2e-5, "outputs")
    close(state[1].transpose(1, 2), S, 2e-5, "final state")      # kept [heads, P, N]


def test_gate_then_group_norm():
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(3)
    n, inner, groups, eps = 7, 120, 3, 1e-4
    y, z, w = torch.randn(n, inner, generator=g), torch.randn(n, inner + 9, generator=g), torch.randn(inner, generator=g)
    out = torch.empty(n, inner, device="cuda")
    ops_seq.gated_group_norm(dev(y), dev(z)[:, 4:4 + inner], dev(w), groups, eps, out)
    v = y.double() * plain.silu(z[:, 4:4 + inner].double())
    want = plain.rms(v.view(n, groups, inner // groups), eps).reshape(n, inner) * w.double()
    close(out, want, 3e-6)


def _attend(q, k, v, H, G, d, dv, scale, window, block, lens, order, qn=None, kn=None, gate=None, eps=1e-5, dtype=torch.float32):
    """Run key store + attention for sequences given whole (one portion each), pages handed out in `order`."""
    from nano_vllm_amd import ops_seq
    nseq = len(lens)
    nblk = [-(-L // block) for L in lens]
    pages = list(order)
    tables = [[pages.pop(0) for _ in range(b)] for b in nblk]
    bt = torch.full((nseq, max(nblk)), -1, dtype=torch.int32)
    slots = []
    for s, L in enumerate(lens):
        bt[s, :nblk[s]] = torch.tensor(tables[s], dtype=torch.int32)
        slots += [tables[s][j // block] * block + j % block for j in range(L)]
    total = (max(order) + 1) * block
    kc = torch.full((total, G, d), 77.0, device="cuda", dtype=dtype)
    vc = torch.full((total, G, dv), 77.0, device="cuda", dtype=dtype)
    kv = dev(torch.cat([k, v], 1).to(dtype))
    ops_seq.knorm_kvstore(kv[:, :G * d], kv[:, G * d:], None if kn is None else dev(kn.to(dtype)), eps, G, d, dv, block,
                          torch.tensor(slots, dtype=torch.int32, device="cuda"), kc, vc)
    out = torch.empty(sum(lens), H * dv, device="cuda", dtype=dtype)
    ops_seq.window_attn(dev(q.to(dtype)), None if qn is None else dev(qn.to(dtype)), eps, None if gate is None else dev(gate.to(dtype)),
                        kc, vc, dev(bt), block, portions(lens, [0] * nseq, list(range(nseq))), H, G, d, dv, scale, window, out)
    return out


def _plain_attention(q, k, v, H, G, d, dv, scale, window, qn=None, kn=None, gate=None, eps=1e-5):
    T = q.shape[0]
    q, k, v = q.double().view(T, H, d), k.double().view(T, G, d), v.double().view(T, G, dv)
    if qn is not None:
        q, k = plain.rms(q, eps) * qn.double(), plain.rms(k, eps) * kn.double()
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = max(0, i - window + 1) if window > 0 else 0
        for h in range(H):
            gg = h // (H // G)
            w = torch.softmax((k[lo:i + 1, gg] @ q[i, h]) * scale, 0)
            out[i, h] = w @ v[lo:i + 1, gg]
    out = out.reshape(T, H * dv)
    return out * plain.sigmoid(gate.double()) if gate is not None else out


@pytest.mark.parametrize("H,G,d,dv,window,block", [(4, 2, 32, 48, 20, 16), (3, 3, 64, 128, 64, 64), (8, 1, 16, 16, 1, 16),
                                                   (2, 2, 80, 200, 0, 32), (6, 2, 128, 64, 33, 48)])
@pytest.mark.parametrize("dtype,path", [(torch.float32, "scalar"), (torch.bfloat16, "matrix"), (torch.bfloat16, "matrix_own_loads"),
                                        (torch.bfloat16, "scalar")])
def test_windowed_attention_against_the_plain_loop(H, G, d, dv, window, block, dtype, path):
    """float32 takes the one-query-per-wavefront kernel; bfloat16 the matrix-core kernel with K / V tiles shared through LDS,
    the one in which every wavefront loads its own operands (tiles too large for LDS) when forced, or the scalar one when
    forced — the path head sizes outside the matrix-core kernels' reach take."""
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(H * d)
    lens = [70, 5, 129]
    T = sum(lens)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(dtype).float()
    q, k, v = rnd(T, H * d), rnd(T, G * d), rnd(T, G * dv)
    qn, kn, gate = (1 + 0.2 * rnd(d)).to(dtype).float(), (1 + 0.2 * rnd(d)).to(dtype).float(), rnd(T, H * dv)
    order = torch.randperm(sum(-(-L // block) for L in lens) + 3, generator=g).tolist()      # scattered pages
    ops_seq.load_library().nvs_window_attn_force_scalar({"scalar": 1, "matrix": 0, "matrix_own_loads": 2}[path])
    try:
        got = _attend(q, k, v, H, G, d, dv, 0.4, window, block, lens, order, qn, kn, gate, dtype=dtype)
    finally:
        ops_seq.load_library().nvs_window_attn_force_scalar(0)
    o = 0
    for L in lens:
        want = _plain_attention(q[o:o + L], k[o:o + L], v[o:o + L], H, G, d, dv, 0.4, window, qn, kn, gate[o:o + L])
        close(got[o:o + L], want, 1e-5 if dtype == torch.float32 else 2e-2, f"sequence of {L}")
        o += L


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,block", [(96, 64), (50, 16), (64, 64), (65, 32)])
def test_a_standout_key_just_inside_and_just_outside_the_window(window, block, dtype):
    """One key carries a score far above the rest and a value nobody else has: the query `window - 1` tokens later must
    return that value, the next query must not see it at all — at page borders as elsewhere."""
    H = G = 1
    d = dv = 16
    T = 3 * window + 7
    g = torch.Generator().manual_seed(window)
    for hot in (0, 5, block - 1, block, window + 3):
        q, k, v = 0.01 * torch.randn(T, d, generator=g), 0.01 * torch.randn(T, d, generator=g), torch.zeros(T, dv)
        k[hot, 0] = 30.0
        q[:, 0] = 30.0
        v[hot, 3] = 1.0
        got = _attend(q, k, v, H, G, d, dv, 1.0, window, block, [T], list(range(-(-T // block))), dtype=dtype)[:, 3].float().cpu()
        last = hot + window - 1
        assert got[hot:last + 1].min() > 0.99, (hot, "inside the window")
        assert got[last + 1:].abs().max() == 0 and (hot == 0 or got[:hot].abs().max() == 0), (hot, "outside the window")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_without_a_window(dtype):
    H, G, d, dv, T = 2, 1, 32, 32, 900
    g = torch.Generator().manual_seed(9)
    q, k, v = 0.01 * torch.randn(T, H * d, generator=g), 0.01 * torch.randn(T, d, generator=g), torch.zeros(T, dv)
    k[2, 1], v[2, 0] = 25.0, 1.0
    q[:, 1], q[:, d + 1] = 25.0, 25.0
    got = _attend(q, k, v, H, G, d, dv, 1.0, 0, 64, [T], list(range(15))[::-1], dtype=dtype).float().cpu()
    assert got[2:, 0].min() > 0.99 and got[2:, dv].min() > 0.999 and got[:2].abs().max() == 0


# ---------------------------------------------------------------------------------------------- the engine
def small_config(variant: int = 0) -> dict:
    """Configurations unlike each other: head counts that do not divide evenly into the wavefront, kv groups, one and several
    norm groups, convolutions of 2 to 4 taps, a window shorter than a page and one longer, a layer without feed-forward."""
    par_a = {"type": "parallel", "mlp": {"kind": "dense", "ff": 144},
             "mixer": {"left": {"heads": 6, "kv_heads": 2, "dim": 32, "vdim": 48, "scale": 0.2, "mask": {"size": 40}},
                       "right": {"heads": 4, "vdim": 24, "state": 20, "groups": 1, "conv": 4, "norm_groups": 1}}}
    par_b = {"type": "parallel", "mlp": None,
             "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 80, "vdim": 16, "scale": 0.11, "mask": {"size": 7}},
                       "right": {"heads": 6, "vdim": 16, "state": 40, "groups": 3, "conv": 2, "norm_groups": 4}}}
    rec_a = {"type": "rglru", "mlp": {"kind": "dense", "ff": 80}, "mixer": {"width": 160, "blocks": 5, "conv": 2}}
    rec_b = {"type": "rglru", "mlp": {"kind": "dense", "ff": 200}, "mixer": {"width": 96, "blocks": 1, "conv": 4}}
    layers = [[rec_a, par_a, par_b, rec_b], [par_b, par_a], [rec_b, rec_a, rec_a]][variant]
    return {"architecture": "Foduzen", "embedding": {"scale": 5.0}, "layers": layers, "norm": {"eps": 1e-6 * (1 + variant)},
            "vocab": 211 + variant, "width": [112, 64, 96][variant]}


@pytest.fixture(scope="module")
def checkpoints():
    from nano_vllm_amd.foduzen import write_synthetic_checkpoint
    root = tempfile.mkdtemp(prefix="fdz_")
    return [write_synthetic_checkpoint(os.path.join(root, f"m{v}"), small_config(v), seed=11 + v) for v in range(3)]


def engine(path, dtype="float32", pages=40, page=16, live=4, **kw):
    from nano_vllm_amd import LLM
    return LLM(path, dtype=dtype, kvcache_block_size=page, num_kvcache_blocks=pages, max_num_seqs=live,
               max_num_batched_tokens=1024, max_model_len=640, enforce_eager=True, **kw)


def rel(got, want, scale):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / scale)


TOL = {"float32": 5e-5, "bfloat16": 4e-2}      # bf16: logits themselves are bf16 (2^-9 of their size), on top of the layers


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_decoding_agree_with_the_plain_model(checkpoints, variant, dtype):
    path = checkpoints[variant]
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
        if dtype == "float32":                                       # layer by layer, in 32-bit
            for i, x in enumerate(seen):
                close(x, layers[i], 2e-5, f"residual after layer {i}")
        assert rel(whole, want, scale) <= TOL[dtype]
        # portions of changing size, down to two tokens and single tokens, cut inside pages and windows
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
    path = checkpoints[0]
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


def test_long_decoding_past_every_window_and_many_pages(checkpoints):
    path = checkpoints[1]
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
    """LLM.generate(): the scheduler admits, chunks (a token budget smaller than the longest prompt) and decodes; every
    generated token must be the plain model's argmax wherever its margin exceeds the serving precision. `eager=False`:
    decode-only steps replay captured graphs (three batch buckets here, padded rows included), with eager prefill steps
    between the replays."""
    from nano_vllm_amd import LLM, SamplingParams
    path = checkpoints[0]
    ref = plain.Model.load(path)
    g = torch.Generator().manual_seed(21)
    prompts = [torch.randint(0, ref.cfg["vocab"], (n,), generator=g).tolist() for n in (5, 70, 33, 1, 64, 18)]
    llm = LLM(path, dtype=dtype, kvcache_block_size=16, num_kvcache_blocks=30, max_num_seqs=4, max_num_batched_tokens=48,
              max_model_len=256, enforce_eager=eager)
    try:
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True), use_tqdm=False)
        assert eager or llm.model_runner.sgraphs, "decode steps were meant to replay graphs"
        assert llm.scheduler.block_manager.num_free == 30 and llm.scheduler.state_slots.num_free == 4
    finally:
        llm.exit()
    margin = 0.05 if dtype == "float32" else 0.15      # (the sampler reads bf16 logits in both)
    checked = 0
    for prompt, o in zip(prompts, outs):
        gen = o["token_ids"]
        assert len(gen) == 12
        logits = ref.run(prompt + gen[:-1])[len(prompt) - 1:]
        for t, row in zip(gen, logits):
            top = torch.topk(row, 2)
            if float(top.values[0] - top.values[1]) > margin * float(row.std()):
                assert t == int(top.indices[0])
                checked += 1
    assert checked >= 30


def test_sampled_generation_is_reproducible_and_preemption_recomputes_state(checkpoints):
    """A pool so small that running sequences are preempted: a preempted sequence loses pages AND state slot and is
    recomputed from its first token; greedy results must not change."""
    from nano_vllm_amd import LLM, SamplingParams
    path = checkpoints[2]
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 200, (n,), generator=g).tolist() for n in (30, 31, 29, 17)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    outs = []
    for pages in (40, 11):
        llm = LLM(path, dtype="float32", kvcache_block_size=16, num_kvcache_blocks=pages, max_num_seqs=4,
                  max_num_batched_tokens=256, max_model_len=128, enforce_eager=True)
        try:
            outs.append([o["token_ids"] for o in llm.generate(prompts, sp, use_tqdm=False)])
        finally:
            llm.exit()
    assert outs[0] == outs[1]


def test_the_schedule_replayer_as_a_program(checkpoints, tmp_path):
    """bin/trace_run as a user starts it: JSON lines in, `done <step>` lines and little-endian float32 files out, pages of
    64 tokens and four state slots reused as requests end, exit code 0 at the end of its input."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    path = checkpoints[0]
    ref = plain.Model.load(path)
    V = ref.cfg["vocab"]
    g = torch.Generator().manual_seed(31)
    toks = {k: torch.randint(0, V, (n,), generator=g).tolist() for k, n in (("a", 130), ("b", 70), ("c", 9), ("d", 64), ("e", 100))}
    want = {k: ref.run(v).numpy() for k, v in toks.items()}
    steps = [[("a", 100, [0, 99]), ("b", 2, [1])], [("a", 1, [0]), ("b", 60, [3, 59]), ("c", 9, [8])], [("b", 8, [7]), ("a", 29, [28]), ("d", 64, [63])],
             [("e", 64, [0, 63])], [], [("e", 2, [0, 1])], [("e", 34, [33])]]
    out = tmp_path / "out"
    p = subprocess.Popen([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(out),
                          "--max-tokens", "384"], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd=root)
    at = {k: 0 for k in toks}
    scale = float(want["a"].std())
    for n, step in enumerate(steps):
        entries, rows, end = [], [], []
        for k, c, w in step:
            entries.append({"id": k, "tokens": toks[k][at[k]:at[k] + c], "want": w})
            rows += [(k, at[k] + i) for i in w]
            at[k] += c
            if at[k] == len(toks[k]):
                end.append(k)
        p.stdin.write(json.dumps({"step": n, "entries": entries, "end": end}) + "\n")
        p.stdin.flush()
        while True:
            line = p.stdout.readline()
            assert line, "the program ended early"
            if line.strip() == f"done {n}":
                break
        f = out / f"{n}.f32"
        if rows:
            got = np.fromfile(f, dtype="<f4").reshape(len(rows), V)
            exp = np.stack([want[k][i] for k, i in rows])
            assert rel(got, exp, scale) <= 5e-5, n
        else:
            assert not f.exists()
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    assert at == {k: len(v) for k, v in toks.items()}


def test_state_space_recurrence_cut_into_segments_equals_the_token_loop():
    """A long portion with few heads is scanned in segments (local states, then combined): it must equal the token loop,
    start from the state an earlier portion left, leave the right state behind, and not disturb a short portion beside it."""
    from nano_vllm_amd import ops_seq
    heads, P, N, G = 2, 16, 24, 1
    inner = heads * P
    g = torch.Generator().manual_seed(77)
    lens = [40, 700, 3]                                     # first call: 40 tokens of sequence A; second: 700 more of A beside 3 of B
    TA, TB_ = 740, 3
    def inputs(T):
        return (torch.randn(T, inner + 2 * G * N, generator=g), torch.randn(T, heads, generator=g))
    (xa, pa), (xb, pb) = inputs(TA), inputs(TB_)
    dt_bias, A_log, D = torch.randn(heads, generator=g) - 3, torch.randn(heads, generator=g) - 2, torch.randn(heads, generator=g)

    def loop(xbc, proj):
        T = xbc.shape[0]
        x, B, C = xbc[:, :inner].double().view(T, heads, P), xbc[:, inner:inner + N].double(), xbc[:, inner + N:].double()
        dt = plain.softplus(proj.double() + dt_bias.double())
        S = torch.zeros(heads, N, P, dtype=F64)
        y = torch.zeros(T, heads, P, dtype=F64)
        for t in range(T):
            for h in range(heads):
                S[h] = torch.exp(-torch.exp(A_log[h].double()) * dt[t, h]) * S[h] + dt[t, h] * torch.outer(B[t], x[t, h])
                y[t, h] = S[h].T @ C[t] + D[h].double() * x[t, h]
        return y.reshape(T, inner), S
    (ya, Sa), (yb, Sb) = loop(xa, pa), loop(xb, pb)
    state = torch.full((3, heads, P, N), 9.0, device="cuda")
    y0 = torch.empty(40, inner, device="cuda")
    ops_seq.ssd_scan(dev(xa[:40]), dev(pa[:40]), 0, dev(dt_bias), dev(A_log), dev(D), heads, P, N, G, portions([40], [0], [2]), state, y0)
    por = portions([700, 3], [40, 0], [2, 0])
    por.max_q = 700
    assert ops_seq.load_library().nvs_ssd_scan_workspace(heads, P, N, 2, 700) > 0, "this shape was meant to be segmented"
    y1 = torch.empty(703, inner, device="cuda")
    ops_seq.ssd_scan(dev(torch.cat([xa[40:], xb])), dev(torch.cat([pa[40:], pb])), 0, dev(dt_bias), dev(A_log), dev(D), heads, P, N, G,
                     por, state, y1)
    close(torch.cat([y0, y1[:700]]), ya, 3e-5, "long sequence")
    close(y1[700:], yb, 3e-5, "short neighbour")
    close(state[2].transpose(1, 2), Sa, 3e-5, "state of the long sequence")
    close(state[0].transpose(1, 2), Sb, 3e-5, "state of the short one")
    assert (state[1] == 9).all()


def test_gated_recurrence_cut_into_segments_equals_the_token_loop():
    """A long portion of a narrow layer is scanned in segments; beside it a short portion of another sequence that continues
    from a stored state."""
    from nano_vllm_amd import ops_seq
    g = torch.Generator().manual_seed(6)
    C, blocks, T, T2 = 40, 2, 1500, 3
    bw = C // blocks
    p = {"ra": torch.randn(blocks, bw, bw, generator=g) * 0.2, "ra.b": torch.randn(blocks, bw, generator=g),
         "ri": torch.randn(blocks, bw, bw, generator=g) * 0.2, "ri.b": torch.randn(blocks, bw, generator=g),
         "lam": -8.0 + 6 * torch.rand(C, generator=g)}
    pd = {k: v.double() for k, v in p.items()}
    u, ypre = torch.randn(T + T2, C, generator=g), torch.randn(T + T2, C, generator=g)
    s2 = torch.randn(C, generator=g)                                      # what the second sequence's slot holds
    want1, S1 = plain.rglru(u[:T].double(), plain.gelu_tanh(ypre[:T].double()), pd, blocks, torch.zeros(C, dtype=F64))
    want2, S2 = plain.rglru(u[T:].double(), plain.gelu_tanh(ypre[T:].double()), pd, blocks, s2.double())
    ub = u.double().view(T + T2, blocks, bw)
    gr = torch.einsum("boi,tbi->bto", pd["ra"], ub) + pd["ra.b"][:, None]
    gi = torch.einsum("boi,tbi->bto", pd["ri"], ub) + pd["ri.b"][:, None]
    state = torch.full((3, C), -9.0, device="cuda")
    state[0] = dev(s2)
    por = portions([T, T2], [0, 17], [2, 0])
    por.max_q = T
    assert ops_seq.load_library().nvs_rglru_scan_workspace(C, 2, T) > 0, "this shape was meant to be segmented"
    out = torch.empty(T + T2, C, device="cuda")
    ops_seq.rglru_scan(dev(torch.cat([gr, gi], -1).float()), dev(u), dev(ypre), dev(p["lam"]), 8.0, blocks, por, state, out)
    close(out[:T], want1, 3e-5, "long sequence")
    close(out[T:], want2, 3e-5, "short neighbour")
    close(state[2], S1, 3e-5, "state of the long sequence")
    close(state[0], S2, 3e-5, "state of the short one")
    assert (state[1] == -9).all()
