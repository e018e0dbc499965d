"""Each HIP kernel alone against a plain float32/float64 PyTorch reference of the same
operation, at sizes other than the engine's test models (odd widths, head sizes in steps of
16, head counts and groups that are no power of two)."""
import math

import numpy as np
import pytest
import torch

from helpers import rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
# relative error allowed for one operation: float32 arithmetic vs one bf16 rounding of the result
OP_TOL = {torch.float32: 2e-6, torch.bfloat16: 6e-3}


def ops_for(dtype):
    from minivllm_amd.kernels.ops import get_ops
    return get_ops(dtype)


def dev(t):
    return t.to("cuda")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
def test_embedding(dtype, wdtype):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(0)
    V, h, n = 301, 72, 19
    table = torch.randn(V, h, generator=g).to(wdtype)
    ids = torch.randint(0, V, (n,), generator=g, dtype=torch.int32)
    resid = torch.full((n, h), 7.0, device="cuda")
    ops.embedding(dev(ids), dev(table), resid, scale=1.5)
    want = table.float()[ids.long()] * 1.5
    assert rel_err(resid.cpu().numpy(), want.numpy()) <= 1e-7


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [72, 1000, 2049])
def test_add_rmsnorm(dtype, h):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(1)
    n, eps = 7, 1e-5
    resid = torch.randn(n, h, generator=g)
    delta = torch.randn(n, h, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(h, generator=g)).to(dtype)
    r_dev, out = dev(resid).clone(), torch.empty(n, h, dtype=dtype, device="cuda")
    ops.add_rmsnorm(r_dev, dev(delta), dev(w), eps, out)
    s = resid.double() + delta.double()
    want = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    assert rel_err(r_dev.cpu().numpy(), s.float().numpy()) <= 1e-7
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[dtype]
    # rows: only the chosen rows, the residual untouched, a negative row gives zeros
    rows = torch.tensor([5, -1, 0], dtype=torch.int32)
    r2, out2 = dev(resid).clone(), torch.empty(3, h, dtype=dtype, device="cuda")
    ops.add_rmsnorm(r2, dev(delta), dev(w), eps, out2, rows=dev(rows))
    assert torch.equal(r2.cpu(), resid)
    assert rel_err(out2[0].float().cpu().numpy(), want[5].numpy()) <= OP_TOL[dtype]
    assert rel_err(out2[2].float().cpu().numpy(), want[0].numpy()) <= OP_TOL[dtype]
    assert float(out2[1].float().abs().max()) == 0.0
    # unit offset: the weight is 1 + w
    out3 = torch.empty(n, h, dtype=dtype, device="cuda")
    ops.add_rmsnorm(dev(resid).clone(), None, dev(w), eps, out3, unit_offset=True)
    r = resid.double()
    want3 = r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps) * (1 + w.double())
    assert rel_err(out3.float().cpu().numpy(), want3.numpy()) <= OP_TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_strided(dtype):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(9, 200, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(48, generator=g)).float()       # a weight kept in float32
    xd = dev(x)
    view = xd[:, 16:64]
    out = torch.empty(9, 48, dtype=dtype, device="cuda")
    ops.rmsnorm(view, dev(w), 1e-6, out)
    v = x[:, 16:64].double()
    want = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-6) * w.double()
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[dtype]


def test_rope_table():
    ops = ops_for(torch.float32)
    rot, theta, max_pos = 48, 50000.0, 700
    inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float) / rot))
    table = ops.rope_table(dev(inv), max_pos).cpu()
    ang = torch.arange(max_pos, dtype=torch.float)[:, None] * inv[None, :]      # float32 product, as the kernel
    want = torch.cat([ang.double().cos(), ang.double().sin()], dim=-1)
    assert table.shape == (max_pos, rot)
    assert float((table.double() - want).abs().max()) <= 3e-7


def paged_cache(num_pages, Hkv, ps, D, dtype):
    k = torch.zeros(num_pages, Hkv, ps, D, dtype=dtype, device="cuda")
    v = torch.zeros(num_pages, Hkv, D, ps, dtype=dtype, device="cuda")
    return k, v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,D,rot,inter", [(6, 3, 48, 48, False), (5, 5, 16, 8, True), (8, 2, 128, 128, False)])
def test_qk_norm_rope_store(dtype, H, Hkv, D, rot, inter):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(3)
    ps, n = 4, 11
    eps = 1e-5
    # two sequences: tokens 0..6 of seq 0 at positions 3..9, tokens 7..10 of seq 1 at positions 0..3
    positions = torch.tensor(list(range(3, 10)) + list(range(0, 4)), dtype=torch.int32)
    token_seq = torch.tensor([0] * 7 + [1] * 4, dtype=torch.int32)
    token_seq[5] = -1                                   # a padding row: nothing may be written for it
    bt = torch.tensor([[5, 2, 7], [1, -1, -1]], dtype=torch.int32)
    width = (H + 2 * Hkv) * D
    qkv = torch.randn(n, width, generator=g).to(dtype)
    qw = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    kw = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    inv = 1.0 / (10000.0 ** (torch.arange(0, rot, 2, dtype=torch.float) / rot))
    table = ops.rope_table(dev(inv), 64)
    kp, vp = paged_cache(9, Hkv, ps, D, dtype)
    kp.fill_(9.0); vp.fill_(9.0)
    qkv_dev = dev(qkv).clone()
    ops.qk_norm_rope_store(qkv_dev, H, Hkv, D, dev(positions), dev(token_seq), dev(qw), dev(kw), eps, table, inter,
                           kp, vp, dev(bt), ps)

    def norm_rope(x, w):           # x [n, heads, D] float64
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.double()
        ang = positions.double()[:, None] * inv.double()[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        y = x.clone()
        half = rot // 2
        if inter:
            a, b = x[..., 0:rot:2], x[..., 1:rot:2]
            y[..., 0:rot:2] = a * c - b * s
            y[..., 1:rot:2] = b * c + a * s
        else:
            a, b = x[..., :half], x[..., half:rot]
            y[..., :half] = a * c - b * s
            y[..., half:rot] = b * c + a * s
        return y

    q = qkv[:, :H * D].double().view(n, H, D)
    k = qkv[:, H * D:(H + Hkv) * D].double().view(n, Hkv, D)
    v = qkv[:, (H + Hkv) * D:].double().view(n, Hkv, D)
    q_want, k_want = norm_rope(q, qw), norm_rope(k, kw)
    got_q = qkv_dev[:, :H * D].float().cpu().view(n, H, D)
    tol = max(OP_TOL[dtype], 3e-6)      # the table's angles are float32
    live = [i for i in range(n) if token_seq[i] >= 0]
    assert rel_err(got_q[live].numpy(), q_want[live].numpy()) <= tol
    assert torch.equal(got_q[5], qkv[5, :H * D].float().view(H, D))          # padding row untouched
    kc, vc = kp.float().cpu(), vp.float().cpu()
    written = set()
    for i in live:
        page = int(bt[token_seq[i], positions[i] // ps]); slot = int(positions[i] % ps)
        written.add((page, slot))
        assert rel_err(kc[page, :, slot, :].numpy(), k_want[i].numpy()) <= tol
        assert rel_err(vc[page, :, :, slot].numpy(), v[i].to(dtype).double().numpy()) <= 1e-7
    for page in range(9):
        for slot in range(ps):
            if (page, slot) not in written:
                assert float((kc[page, :, slot, :] - 9.0).abs().max()) == 0.0
                assert float((vc[page, :, :, slot] - 9.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,D,ps", [(4, 2, 128, 16), (3, 3, 48, 8)])
def test_qk_norm_rope_store_many_tokens(dtype, H, Hkv, D, ps):
    """Enough tokens for the separate value pass: three sequences (one starting mid-page, one
    padding row), pages in scrambled order, untouched slots must stay untouched."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(33)
    spans = [(0, 50), (21, 40), (5, 7)]                       # (start position, tokens)
    positions, token_seq = [], []
    for s_, (start, cnt) in enumerate(spans):
        positions += list(range(start, start + cnt)); token_seq += [s_] * cnt
    n = len(positions)
    token_seq[60] = -1
    pages_per = [-(-(start + cnt) // ps) for start, cnt in spans]
    num_pages = sum(pages_per) + 2
    perm = torch.randperm(num_pages, generator=g).tolist()
    bt = torch.full((3, max(pages_per)), -1, dtype=torch.int32)
    cur = 0
    for s_, n_p in enumerate(pages_per):
        bt[s_, :n_p] = torch.tensor(perm[cur:cur + n_p], dtype=torch.int32); cur += n_p
    positions = torch.tensor(positions, dtype=torch.int32); token_seq = torch.tensor(token_seq, dtype=torch.int32)
    qkv = torch.randn(n, (H + 2 * Hkv) * D, generator=g).to(dtype)
    kp, vp = paged_cache(num_pages, Hkv, ps, D, dtype)
    kp.fill_(9.0); vp.fill_(9.0)
    qd = dev(qkv).clone()
    ops.qk_norm_rope_store(qd, H, Hkv, D, dev(positions), dev(token_seq), None, None, 1e-6, None, False, kp, vp, dev(bt), ps)
    kc, vc = kp.float().cpu(), vp.float().cpu()
    k = qkv[:, H * D:(H + Hkv) * D].float().view(n, Hkv, D)
    v = qkv[:, (H + Hkv) * D:].float().view(n, Hkv, D)
    written = set()
    for i in range(n):
        if token_seq[i] < 0:
            continue
        page = int(bt[token_seq[i], positions[i] // ps]); slot = int(positions[i] % ps)
        written.add((page, slot))
        assert torch.equal(kc[page, :, slot, :], k[i]) and torch.equal(vc[page, :, :, slot], v[i]), i
    for page in range(num_pages):
        for slot in range(ps):
            if (page, slot) not in written:
                assert float((kc[page, :, slot, :] - 9.0).abs().max()) == 0.0
                assert float((vc[page, :, :, slot] - 9.0).abs().max()) == 0.0
    assert torch.equal(qd.cpu(), qkv)                         # no norm, no rotation: q is unchanged


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(dtype):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(4)
    n, I = 5, 173
    gu = (3 * torch.randn(n, 2 * I, generator=g)).to(dtype)
    out = torch.empty(n, I, dtype=dtype, device="cuda")
    ops.swiglu(dev(gu), out)
    want = torch.nn.functional.silu(gu[:, :I].double()) * gu[:, I:].double()
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 70, 96), (33, 129, 200), (130, 64, 1000)])
def test_gemm_exact(dtype, wdtype, M, N, K):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(5)
    a = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(wdtype)
    b = torch.randn(N, generator=g).to(wdtype)
    want = a.double() @ w.double().T + b.double()
    for out_dtype in {dtype, torch.float32}:
        out = torch.empty(M, N, dtype=out_dtype, device="cuda")
        ops.gemm(dev(a), dev(w), out, dev(b), exact=True)
        tol = 3e-6 if out_dtype == torch.float32 else OP_TOL[dtype]
        assert rel_err(out.float().cpu().numpy(), want.numpy()) <= tol
    # a row's result does not depend on the rows around it
    out_all = torch.empty(M, N, dtype=torch.float32, device="cuda")
    out_one = torch.empty(1, N, dtype=torch.float32, device="cuda")
    ops.gemm(dev(a), dev(w), out_all, exact=True)
    ops.gemm(dev(a[M - 1:M]), dev(w), out_one, exact=True)
    assert torch.equal(out_all[M - 1:M], out_one)


def reference_attention(q, k_all, v_all, positions, token_seq, H, Hkv, scale, window):
    """q [n, H, D] float64; k_all/v_all: per sequence [ctx, Hkv, D]."""
    n, _, D = q.shape
    out = torch.zeros(n, H, D, dtype=torch.float64)
    for i in range(n):
        s = int(token_seq[i])
        if s < 0:
            continue
        p = int(positions[i])
        lo = 0 if window is None else max(0, p - window)
        for h in range(H):
            kh = h // (H // Hkv)
            keys = k_all[s][lo:p + 1, kh]
            vals = v_all[s][lo:p + 1, kh]
            sc = torch.softmax((keys @ q[i, h]) * scale, dim=0)
            out[i, h] = sc @ vals
    return out


def fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype):
    kp, vp = paged_cache(num_pages, Hkv, ps, D, dtype)
    kc, vc = torch.full(kp.shape, float("nan")), torch.full(vp.shape, float("nan"))
    for s, table in enumerate(tables):
        for pos in range(k_all[s].shape[0]):
            page, slot = table[pos // ps], pos % ps
            if page < 0:
                continue
            kc[page, :, slot, :] = k_all[s][pos]
            vc[page, :, :, slot] = v_all[s][pos]
    kp.copy_(kc.to(dtype)); vp.copy_(vc.to(dtype))
    return kp, vp


def make_plan(q_lens, ctx_lens, max_context_len=None, decode_only=None):
    from minivllm_amd.engine.step import AttentionPlan
    from minivllm_amd.parts import Workspace
    cu = torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32, device="cuda")
    if decode_only is None:
        decode_only = all(q == 1 for q in q_lens)
    return AttentionPlan(decode_only=decode_only, max_q_len=max(q_lens),
                         max_context_len=max_context_len or max(ctx_lens), n_seqs=len(q_lens), q_lens=list(q_lens),
                         cu_seqlens=cu, workspace=Workspace(torch.device("cuda:0")))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("with_plan", [False, True])
@pytest.mark.parametrize("H,Hkv,D,ps,window", [(6, 3, 48, 4, None), (4, 1, 16, 8, 9), (8, 2, 128, 16, None),
                                                (5, 5, 80, 3, 130), (16, 8, 128, 16, 40), (4, 4, 64, 32, None),
                                                (14, 2, 64, 16, 25), (32, 1, 128, 16, None)])
def test_attention_general(dtype, with_plan, H, Hkv, D, ps, window):
    """Mixed step: a long portion, a short one and single decoded tokens, over pages in
    scrambled order; unused pages hold NaN. With a plan the bfloat16 path takes the MFMA kernel
    where the sizes allow it."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(6)
    ctx_lens = [150, 37, 1, 290]            # context after the step
    q_lens = [150, 5, 1, 1]                 # whole prompt, portion, first token, decoded token
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 5
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    if window is not None:                  # pages wholly behind the window of the first query are gone
        for s, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
            first_needed = max(0, (c - ql) - window) // ps
            for i in range(first_needed):
                tables[s][i] = -1
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    width = max(pages_per)
    bt = torch.full((len(tables), width), -1, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    positions, token_seq = [], []
    for s, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
        positions += list(range(c - ql, c)); token_seq += [s] * ql
    n = len(positions)
    positions = torch.tensor(positions, dtype=torch.int32)
    token_seq = torch.tensor(token_seq, dtype=torch.int32)
    # sharpen: one far key gets a large score for the last query of sequence 3
    q = torch.randn(n, H, D, generator=g)
    q[-1] = 6.0 * k_all[3][2 if window is None else 290 - 1 - window].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)
    q = q.to(dtype)
    scale = 1.0 / math.sqrt(D)
    # queries live in a wider row, as in the packed qkv buffer
    qrow = torch.zeros(n, H * D + 24, dtype=dtype)
    qrow[:, :H * D] = q.view(n, H * D)
    qd = dev(qrow)
    out = torch.empty(n, H * D, dtype=dtype, device="cuda")
    plan = make_plan(q_lens, ctx_lens) if with_plan else None
    ops.attention(qd[:, :H * D], out, kp, vp, dev(bt), ps, dev(positions), dev(token_seq), H, Hkv, D, scale, window,
                  plan=plan)
    want = reference_attention(q.double(), k_all, v_all, positions, token_seq, H, Hkv, scale, window)
    # the MFMA kernel rounds the probabilities to bfloat16 before the second product
    tol = max(OP_TOL[dtype], 5e-6) * (2 if with_plan else 1)
    assert rel_err(out.float().cpu().view(n, H, D).numpy(), want.numpy()) <= tol


@pytest.mark.parametrize("nt,kw", [(1, 1), (1, 2), (2, 1), (2, 2)])
@pytest.mark.parametrize("H,Hkv,D,ps,window", [(4, 2, 128, 16, None), (8, 2, 64, 32, 150), (16, 2, 128, 64, 70)])
def test_attention_prompt_variants(nt, kw, H, Hkv, D, ps, window):
    """Every variant of the MFMA prompt kernel (16 or 32 columns a wave, four or eight waves a
    workgroup) on the same step, whatever the launch rule would choose for it: portions that end
    inside a unit and inside a block of keys, walks of one, two, three and many rounds (the stages
    are used again from the third pair of blocks on), a window with pages given back, and slots
    beyond a sequence's end that hold NaN."""
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(67)
    ctx_lens = [19, 61, 100, 333, 517]
    q_lens = [19, 40, 7, 333, 130]
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    if window is not None:
        for s, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
            for i in range(max(0, (c - ql) - window) // ps):
                tables[s][i] = -1
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    bt = torch.full((len(tables), max(pages_per) + 2), -1, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    positions, token_seq = [], []
    for s, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
        positions += list(range(c - ql, c)); token_seq += [s] * ql
    n = len(positions)
    positions = torch.tensor(positions, dtype=torch.int32)
    token_seq = torch.tensor(token_seq, dtype=torch.int32)
    q = torch.randn(n, H, D, generator=g)
    starts = np.cumsum([0] + q_lens)
    for s in range(len(q_lens)):          # the last query of every sequence looks at a far key (or the window's edge)
        far = 0 if window is None else max(0, ctx_lens[s] - 1 - window)
        q[starts[s + 1] - 1] = 6.0 * k_all[s][far].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)
    q = q.to(dtype)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((n, H * D), float("nan"), dtype=dtype, device="cuda")
    plan = make_plan(q_lens, ctx_lens)
    plan.prefill_variant = (nt, kw)
    ledger, ops.ledger = ops.ledger, []
    try:
        ops.attention(dev(q.view(n, H * D)), out, kp, vp, dev(bt), ps, dev(positions), dev(token_seq), H, Hkv, D, scale,
                      window, plan=plan)
        seen = [line[0] for line in ops.ledger]
    finally:
        ops.ledger = ledger
    assert seen == ["mv_attention_prefill"], seen
    want = reference_attention(q.double(), k_all, v_all, positions, token_seq, H, Hkv, scale, window)
    assert rel_err(out.float().cpu().view(n, H, D).numpy(), want.numpy()) <= 2 * OP_TOL[dtype]


@pytest.mark.parametrize("H,Hkv,D,ps,window", [(4, 2, 128, 16, None), (8, 2, 64, 32, 300), (8, 1, 128, 16, None)])
@pytest.mark.parametrize("ctx_lens,q_lens", [([1203, 1170, 1050], [1203, 70, 1]), ([5003, 6100, 2050], [5003, 650, 1])])
def test_attention_prompts_with_long_contexts(H, Hkv, D, ps, window, ctx_lens, q_lens):
    """Prompt portions over thousands of keys (the MFMA kernel then walks the keys with two wave
    groups per workgroup and merges them): a whole long prompt, a late portion of another, and a
    single token, with a far key (or the one at the window's edge) made to stand out."""
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(61)
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 5
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    if window is not None:
        for s, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
            for i in range(max(0, (c - ql) - window) // ps):
                tables[s][i] = -1
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    bt = torch.full((len(tables), max(pages_per)), -1, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    positions, token_seq = [], []
    for s, (c, ql) in enumerate(zip(ctx_lens, q_lens)):
        positions += list(range(c - ql, c)); token_seq += [s] * ql
    n = len(positions)
    positions = torch.tensor(positions, dtype=torch.int32)
    token_seq = torch.tensor(token_seq, dtype=torch.int32)
    q = torch.randn(n, H, D, generator=g)
    for row, s in ((q_lens[0] - 1, 0), (q_lens[0] + q_lens[1] - 1, 1), (n - 1, 2)):      # the last query of every sequence
        far = 3 if window is None else ctx_lens[s] - 1 - window
        q[row] = 6.0 * k_all[s][far].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)
    q = q.to(dtype)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((n, H * D), float("nan"), dtype=dtype, device="cuda")
    plan = make_plan(q_lens, ctx_lens)
    assert plan.max_context_len >= 1024
    ops.attention(dev(q.view(n, H * D)), out, kp, vp, dev(bt), ps, dev(positions), dev(token_seq), H, Hkv, D, scale,
                  window, plan=plan)
    # the reference for a sample of the rows: a spread of each sequence, every row around the seam between
    # the first two, and the last ones
    first = q_lens[0]
    rows = sorted(set(list(range(0, first, max(37, first // 40))) + list(range(first - 23, first + 40)) +
                      list(range(first + 40, n, 31)) + list(range(n - 5, n))))
    want = reference_attention(q[rows].double(), k_all, v_all, positions[rows], token_seq[rows], H, Hkv, scale, window)
    got = out.float().cpu().view(n, H, D)
    assert not torch.isnan(got).any()
    assert rel_err(got[rows].numpy(), want.numpy()) <= 2 * OP_TOL[dtype]


@pytest.mark.parametrize("H,Hkv,D,ps,window", [(16, 8, 128, 16, None), (8, 1, 128, 32, None), (6, 2, 64, 16, 50),
                                                (16, 1, 64, 16, None)])
@pytest.mark.parametrize("max_context", [None, 4096, 40000])
@pytest.mark.parametrize("splits", [None, 1, 3, 16, 64])
def test_attention_decode_kernel(H, Hkv, D, ps, window, max_context, splits):
    """Decode steps on the MFMA kernel: one token per sequence at very different context lengths, a
    padding sequence in the middle; the keys split over as many workgroups as the launch rule
    chooses (None), over one, a few and many (more than some sequences have blocks of keys: those
    splits end at once and the others add the partial results up among themselves), planned for the
    longest context, for a longer one, and (forced splits, no max_context) for a shorter one than
    the sequences really have: the page ids beyond the plan are then looked up as the keys go."""
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(16)
    ctx_lens = [1, 17, 300, 1200, 33, 64]
    if max_context == 40000 and Hkv == 1:
        ctx_lens[2] = 18000                         # more pages than the kernel keeps ids of at once
    q_lens = [1, 1, 1, 0, 1, 1]                     # sequence 3 is padding: no token
    live = [s for s, ql in enumerate(q_lens) if ql]
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    if window is not None:
        for s, c in enumerate(ctx_lens):
            for i in range(max(0, (c - 1) - window) // ps):
                tables[s][i] = -1
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    bt = torch.full((len(tables), max(pages_per)), -1, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    positions = torch.tensor([ctx_lens[s] - 1 for s in live], dtype=torch.int32)
    token_seq = torch.tensor(live, dtype=torch.int32)
    n = len(live)
    q = torch.randn(n, H, D, generator=g)
    far = 5 if window is None else ctx_lens[2] - 1 - window  # a far key, or the one at the window's edge
    q[2] = 6.0 * k_all[2][far].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)
    q = q.to(dtype)
    scale = 1.0 / math.sqrt(D)
    out = torch.empty(n, H * D, dtype=dtype, device="cuda")
    plan = make_plan(q_lens, ctx_lens, max_context_len=max_context if max_context else (200 if splits else None),
                     decode_only=True)
    plan.decode_splits = splits
    ops.attention(dev(q.view(n, H * D)), out, kp, vp, dev(bt), ps, dev(positions), dev(token_seq), H, Hkv, D, scale,
                  window, plan=plan)
    want = reference_attention(q.double(), k_all, v_all, positions, token_seq, H, Hkv, scale, window)
    assert rel_err(out.float().cpu().view(n, H, D).numpy(), want.numpy()) <= 2 * OP_TOL[dtype]


@pytest.mark.parametrize("H,Hkv,D", [(16, 8, 128), (8, 8, 64)])
@pytest.mark.parametrize("fused", [False, True])
def test_attention_decode_with_more_workgroups_than_compute_units(H, Hkv, D, fused):
    """Forty sequences of eight kv heads: more workgroups than the chip has compute units, for
    which the kernel is built with half the registers so that two workgroups share a unit. Both
    forms: finished queries against a finished cache, and raw rows whose key and value the kernel
    writes itself."""
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(44)
    ps, n = 16, 40
    assert n * Hkv > 256
    ctx_lens = [int(c) for c in torch.randint(1, 400, (n,), generator=g)]
    ctx_lens[3], ctx_lens[17] = 1, 16
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    bt = torch.full((n, max(pages_per)), -1, dtype=torch.int32)
    for s_, t in enumerate(tables):
        bt[s_, :len(t)] = torch.tensor(t, dtype=torch.int32)
    positions = torch.tensor([c - 1 for c in ctx_lens], dtype=torch.int32)
    token_seq = torch.arange(n, dtype=torch.int32)
    q = torch.randn(n, H, D, generator=g)
    for s_ in range(n):
        if ctx_lens[s_] > 40:           # a far key stands out
            q[s_] = 6.0 * k_all[s_][3].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)
    q = q.to(dtype)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((n, H * D), float("nan"), dtype=dtype, device="cuda")
    plan = make_plan([1] * n, ctx_lens, decode_only=True)
    if fused:
        raw = torch.cat([q.view(n, -1)] + [torch.stack([x[c - 1] for x, c in zip(kv, ctx_lens)]).to(dtype).view(n, -1)
                                           for kv in (k_all, v_all)], dim=1)
        for s_, c in enumerate(ctx_lens):        # the new slots are not written yet
            kp[tables[s_][(c - 1) // ps], :, (c - 1) % ps, :] = float("nan")
            vp[tables[s_][(c - 1) // ps], :, :, (c - 1) % ps] = float("nan")
        assert ops.attention_decode_fused(dev(raw), out, kp, vp, dev(bt), ps, dev(positions), dev(token_seq), H, Hkv, D,
                                          scale, None, plan, None, None, 1e-6, None, False, True)
    else:
        ops.attention(dev(q.view(n, H * D)), out, kp, vp, dev(bt), ps, dev(positions), dev(token_seq), H, Hkv, D, scale,
                      None, plan=plan)
    want = reference_attention(q.double(), k_all, v_all, positions, token_seq, H, Hkv, scale, None)
    assert rel_err(out.float().cpu().view(n, H, D).numpy(), want.numpy()) <= 2 * OP_TOL[dtype]
    if fused:
        for s_, c in enumerate(ctx_lens):
            page, slot = tables[s_][(c - 1) // ps], (c - 1) % ps
            assert torch.equal(kp[page, :, slot, :].float().cpu().double(), k_all[s_][c - 1])
            assert torch.equal(vp[page, :, :, slot].float().cpu().double(), v_all[s_][c - 1])


@pytest.mark.parametrize("splits", [4, 10, 37])
def test_attention_decode_splits_agree_over_many_launches(splits):
    """The workgroups that share a sequence's keys hand their partial results to whichever of them
    finishes last, through memory and a counter, with no second launch in between. Three hundred
    launches in a row (other launches in between, so that the caches hold other data) give the very
    same bits each time and agree with the reference, and every counter is back at zero: a workgroup
    that read a row before it had arrived, or a counter left standing, would show here."""
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(77)
    H, Hkv, D, ps = 16, 8, 128, 16
    ctx_lens = [1160, 900, 1200, 77, 1024, 1153, 640, 1199]
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    bt = torch.full((len(tables), max(pages_per)), -1, dtype=torch.int32)
    for s_, t in enumerate(tables):
        bt[s_, :len(t)] = torch.tensor(t, dtype=torch.int32)
    n = len(ctx_lens)
    positions = torch.tensor([c - 1 for c in ctx_lens], dtype=torch.int32)
    token_seq = torch.arange(n, dtype=torch.int32)
    q = torch.randn(n, H, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    plan = make_plan([1] * n, ctx_lens, max_context_len=2048, decode_only=True)
    plan.decode_splits = splits
    qd, btd, posd, seqd = dev(q.view(n, H * D)), dev(bt), dev(positions), dev(token_seq)
    outs = [torch.full((n, H * D), float("nan"), dtype=dtype, device="cuda") for _ in range(300)]
    churn = torch.randn(1 << 22, device="cuda")
    for it, out in enumerate(outs):
        ops.attention(qd, out, kp, vp, btd, ps, posd, seqd, H, Hkv, D, scale, None, plan=plan)
        if it % 7 == 0:
            churn.mul_(1.0001)
    torch.cuda.synchronize()
    want = reference_attention(q.double(), k_all, v_all, positions, token_seq, H, Hkv, scale, None)
    assert rel_err(outs[0].float().cpu().view(n, H, D).numpy(), want.numpy()) <= 2 * OP_TOL[dtype]
    first = outs[0].view(torch.int16)
    differing = [i for i, o in enumerate(outs) if not torch.equal(o.view(torch.int16), first)]
    assert differing == []
    assert int(ops._attn_counters.abs().sum()) == 0


def test_attention_decode_one_workgroup_over_more_pages_than_it_stages():
    """One workgroup walks 18,000 keys (1,125 pages of 16): more page ids than it keeps in LDS, the
    rest are read from the block table as it goes."""
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(31)
    H, Hkv, D, ps, ctx = 4, 1, 64, 16, 18000
    k_all = [torch.randn(ctx, Hkv, D, generator=g).to(dtype).double()]
    v_all = [torch.randn(ctx, Hkv, D, generator=g).to(dtype).double()]
    pages = -(-ctx // ps)
    table = torch.randperm(pages + 2, generator=g).tolist()[:pages]
    kp, vp = fill_pages(k_all, v_all, [table], ps, Hkv, D, pages + 2, dtype)
    bt = dev(torch.tensor([table], dtype=torch.int32))
    q = torch.randn(1, H, D, generator=g)
    q[0] = 6.0 * k_all[0][17000].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)   # a key far into the walk
    q = q.to(dtype)
    qd = dev(q.view(1, H * D))
    out = torch.full((1, H * D), float("nan"), dtype=dtype, device="cuda")
    pos = dev(torch.tensor([ctx - 1], dtype=torch.int32))
    cu = dev(torch.tensor([0, 1], dtype=torch.int32))
    seq0 = dev(torch.zeros(1, dtype=torch.int32))
    ops.lib.call("mv_attention_decode", qd.data_ptr(), H * D, out.data_ptr(), H * D, kp.data_ptr(), vp.data_ptr(),
                 bt.data_ptr(), pages, ps, pos.data_ptr(), cu.data_ptr(), 1, H, Hkv, D, D ** -0.5, -1, 0, 0, 1, 0, 4,
                 seq0.data_ptr(), ops._stream())
    torch.cuda.synchronize()
    want = reference_attention(q.double(), k_all, v_all, torch.tensor([ctx - 1]), torch.tensor([0]), H, Hkv, D ** -0.5, None)
    assert rel_err(out.float().cpu().view(1, H, D).numpy(), want.numpy()) <= 2 * OP_TOL[dtype]


@pytest.mark.parametrize("H,Hkv,D,ps,window", [(16, 8, 128, 16, None), (8, 1, 128, 32, None), (6, 2, 64, 16, 50),
                                                (16, 1, 64, 64, None)])
@pytest.mark.parametrize("with_norm,with_rope,store", [(True, True, True), (False, True, True), (True, False, True),
                                                       (True, True, False)])
@pytest.mark.parametrize("max_context", [None, 40000])
@pytest.mark.parametrize("splits", [None, 1, 5, 64])
@pytest.mark.parametrize("gathered", [False, True])
def test_attention_decode_fused_kernel(H, Hkv, D, ps, window, with_norm, with_rope, store, max_context, splits, gathered):
    """A decode step from the raw [q | k | v] rows: per-head norm, rotation, cache write and attention
    in one kernel. The slot of the new position holds NaN before (unless the cache is another
    layer's and already complete), the finished key and value afterwards. ``gathered``: the rotation
    angles come as rows gathered for the step's tokens (the padding row's are NaN), not from the table."""
    if gathered and not with_rope:
        pytest.skip("no rotation, no rows")
    ops = ops_for(torch.bfloat16)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(21)
    ctx_lens = [1, 17, 300, 1200, 33, 64, 16]
    q_lens = [1, 1, 1, 0, 1, 1, 1]                  # sequence 3 is padding: no token
    live = [s for s, ql in enumerate(q_lens) if ql]
    n = len(live)
    eps = 1e-5
    qw = (1 + 0.2 * torch.randn(D, generator=g)).to(dtype) if with_norm else None
    kw = (1 + 0.2 * torch.randn(D, generator=g)).to(dtype) if with_norm else None
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2, dtype=torch.float32) / D)))
    table = ops.rope_table(dev(inv_freq), 1300) if with_rope else None

    def finish(x, w, pos):                      # x [heads, D] raw (bf16 values), float64 math
        x = x.double()
        if w is not None:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.double()
        if with_rope:
            ang = pos * inv_freq.double()
            c, sn = torch.cos(ang), torch.sin(ang)
            a, b = x[:, :D // 2], x[:, D // 2:]
            x = torch.cat([a * c - b * sn, b * c + a * sn], dim=-1)
        return x.to(dtype).double()

    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype).double() for c in ctx_lens]
    raw = torch.randn(n, (H + 2 * Hkv) * D, generator=g).to(dtype)
    far = 5 if window is None else 300 - 1 - window
    raw[2, :H * D] = (6.0 * k_all[2][far].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)).reshape(-1).to(dtype)
    q_fin = torch.zeros(n, H, D, dtype=torch.float64)
    for t, s in enumerate(live):
        pos = ctx_lens[s] - 1
        q_fin[t] = finish(raw[t, :H * D].view(H, D), qw, pos)
        if store:
            k_all[s][pos] = finish(raw[t, H * D:(H + Hkv) * D].view(Hkv, D), kw, pos)
            v_all[s][pos] = raw[t, (H + Hkv) * D:].view(Hkv, D).double()
    pages_per = [-(-c // ps) for c in ctx_lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, cur = [], 0
    for n_p in pages_per:
        tables.append(perm[cur:cur + n_p]); cur += n_p
    if window is not None:
        for s, c in enumerate(ctx_lens):
            for i in range(max(0, (c - 1) - window) // ps):
                tables[s][i] = -1
    kp, vp = fill_pages(k_all, v_all, tables, ps, Hkv, D, num_pages, dtype)
    want_k, want_v = kp.clone(), vp.clone()
    if store:                                        # the new slots are not written yet
        for s in live:
            pos = ctx_lens[s] - 1
            kp[tables[s][pos // ps], :, pos % ps, :] = float("nan")
            vp[tables[s][pos // ps], :, :, pos % ps] = float("nan")
    bt = torch.full((len(tables), max(pages_per)), -1, dtype=torch.int32)
    for s, t in enumerate(tables):
        bt[s, :len(t)] = torch.tensor(t, dtype=torch.int32)
    positions = torch.tensor([ctx_lens[s] - 1 for s in live], dtype=torch.int32)
    token_seq = torch.tensor(live, dtype=torch.int32)
    scale = 1.0 / math.sqrt(D)
    # as in the engine's padded decode steps: one row per sequence of the plan, padding at the end
    # (a sequence without a token, a row that belongs to no sequence)
    out = torch.full((n + 1, H * D), float("nan"), dtype=dtype, device="cuda")
    plan = make_plan([1] * n + [0], [ctx_lens[s] for s in live],
                     max_context_len=max_context if max_context else (200 if splits == 5 else None), decode_only=True)
    plan.decode_splits = splits
    rows = raw if store else raw[:, :H * D].contiguous()
    qkv = dev(torch.cat([rows, torch.full((1, rows.shape[1]), float("nan"), dtype=dtype)]))
    bt_rows = torch.cat([bt[live], torch.full((1, bt.shape[1]), -1, dtype=torch.int32)]).contiguous()
    rope_rows = None
    if gathered:
        rope_rows = torch.full((n + 1, D), float("nan"), dtype=torch.float32, device="cuda")
        ops.gather_rows(dev(positions), table, rope_rows[:n])
        assert torch.equal(rope_rows[:n].cpu(), table.cpu()[positions.long()])
    took = ops.attention_decode_fused(qkv, out, kp, vp, dev(bt_rows), ps,
                                      dev(torch.cat([positions, torch.zeros(1, dtype=torch.int32)])),
                                      dev(torch.tensor(list(range(n)) + [-1], dtype=torch.int32)), H, Hkv, D, scale,
                                      window, plan, dev(qw) if with_norm else None, dev(kw) if with_norm else None,
                                      eps, table, False, store, rope_rows=rope_rows)
    assert took
    out = out[:n]
    seqs = torch.arange(n, dtype=torch.int32)
    want = reference_attention(q_fin, [k_all[s] for s in live], [v_all[s] for s in live], positions, seqs, H, Hkv,
                               scale, window)
    assert rel_err(out.float().cpu().view(n, H, D).numpy(), want.numpy()) <= 2 * OP_TOL[dtype]
    # the cache: the new slots hold the finished key and the value, everything else is untouched
    def same(a, b):
        a, b = a.float().cpu(), b.float().cpu()
        return bool(torch.all((a == b) | (torch.isnan(a) & torch.isnan(b))))
    if store:
        for s in live:
            pos = ctx_lens[s] - 1
            page, slot = tables[s][pos // ps], pos % ps
            got_k = kp[page, :, slot, :].float().cpu().double()
            assert rel_err(got_k.numpy(), k_all[s][pos].numpy()) <= OP_TOL[dtype]
            assert torch.equal(vp[page, :, :, slot].float().cpu().double(), v_all[s][pos])
            want_k[page, :, slot, :] = kp[page, :, slot, :]
    assert same(kp, want_k) and same(vp, want_v)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 70, 96), (8, 1024, 1024), (17, 4100, 64), (64, 333, 3072), (33, 2048, 512),
                                    (5, 151936 // 8, 1024), (5, 5120, 256), (16, 6144, 128), (3, 330, 64),
                                    # weights of 16 MB and more: the loads of whole lines, up to 8 rows and 9 to 16
                                    (8, 4100, 2112), (2, 4099, 2112), (7, 4096, 12288)])
def test_gemm_weight_streaming(out_dtype, M, N, K):
    """The weight-streaming product, also at sizes where a workgroup takes a number of output
    columns that is no multiple of a tile (5120 and 6144 columns: 20 and 24 each; 330: 8, the last
    workgroup two)."""
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(17)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    want = a.double() @ w.double().T
    out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    ops.gemm(dev(a), dev(w), out)
    tol = 3e-6 if out_dtype == torch.float32 else OP_TOL[torch.bfloat16]
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= tol
    ops.gemm(dev(a), dev(w), out, dev(b))
    assert rel_err(out.float().cpu().numpy(), (want + b.double()).numpy()) <= tol
    # rows in a wider buffer, and a row's result does not depend on the rows around it
    wide = torch.zeros(M, K + 40, dtype=torch.bfloat16)
    wide[:, :K] = a
    out_w = torch.empty(M, N, dtype=torch.float32, device="cuda")
    ops.gemm(dev(wide)[:, :K], dev(w), out_w)
    out_one = torch.empty(1, N, dtype=torch.float32, device="cuda")
    ops.gemm(dev(a[M - 1:M]), dev(w), out_one)
    assert torch.equal(out_w[M - 1:M], out_one)
    assert rel_err(out_w.cpu().numpy(), want.numpy()) <= 3e-6


@pytest.mark.parametrize("M,N,K", [(12, 5000, 2048), (16, 8200, 1024), (9, 4099, 2112)])
def test_gemm_weight_streaming_whole_lines_for_9_to_16_rows(M, N, K):
    """Weights of 16 MB and more at 9 to 16 rows go to the tiled product; the weight-streaming kernel's
    variant for them (whole-line loads of the weights, two MFMAs a load) serves the fused norm and
    callers of the entry point. Here with the tiled product switched off: right, and a row's bits are
    those of the same row alone (the variant for up to 8 rows)."""
    from minivllm_amd.kernels.ops import Ops
    ops = Ops(torch.bfloat16)
    ops.use_tiled_gemm = False
    g = torch.Generator().manual_seed(18)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    want = a.double() @ w.double().T + b.double()
    ops.ledger = []
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ops.gemm(dev(a), dev(w), out, dev(b))
    assert [l[0] for l in ops.ledger] == ["mv_gemm_skinny"]
    assert rel_err(out.cpu().numpy(), want.numpy()) <= 3e-6
    one = torch.empty(1, N, dtype=torch.float32, device="cuda")
    ops.gemm(dev(a[M - 1:M]), dev(w), one, dev(b))
    assert torch.equal(out[M - 1:M], one)


@pytest.mark.parametrize("M,N,K,swiglu,out_dtype", [
    (17, 3100, 4096, False, torch.bfloat16), (32, 4096, 3072, False, torch.bfloat16),
    (30, 6144, 2048, False, torch.float32), (31, 6144, 2048, True, torch.bfloat16),
    (25, 2 * 1571, 4096, True, torch.bfloat16), (20, 151936 // 4, 1024, False, torch.float32),
    (9, 3100, 4096, False, torch.bfloat16), (1, 5120, 25600, False, torch.bfloat16),
    (3, 2 * 12032, 5120, True, torch.bfloat16)])
def test_gemm_for_a_few_dozen_rows_against_large_weights(M, N, K, swiglu, out_dtype):
    """The kernel that shares the activation rows through LDS and splits K over workgroups (partial
    sums added in a fixed order): it serves what the tiled product does not take (gated pairs of a few
    dozen megabytes below 32 rows, the largest weights below 8 rows, K no multiple of 64), and here,
    with the tiled product switched off, everything it used to."""
    from minivllm_amd.kernels.ops import Ops
    ops = Ops(torch.bfloat16)
    ops.use_tiled_gemm = False        # (the tiled product has taken most of these shapes over: see test_which_product_...)
    g = torch.Generator().manual_seed(19)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    full = a.double() @ w.double().T
    ops._mid_work = None
    if swiglu:
        I = N // 2
        want = torch.nn.functional.silu(full[:, :I]) * full[:, I:]
        out = torch.full((M, I), float("nan"), dtype=out_dtype, device="cuda")
        assert ops.gemm_swiglu(dev(a), dev(w), out)
        again = torch.full((1, I), float("nan"), dtype=out_dtype, device="cuda")
    else:
        b = torch.randn(N, generator=g).to(torch.bfloat16)
        want = full + b.double()
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
        ops.gemm(dev(a), dev(w), out, dev(b))
    assert ops._mid_work is not None, "the shape was left to another kernel"
    tol = 3e-6 if out_dtype == torch.float32 else OP_TOL[torch.bfloat16]
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= tol
    # rows in a wider buffer; a row's result does not depend on the rows around it
    wide = torch.zeros(M, K + 40, dtype=torch.bfloat16)
    wide[:, :K] = a
    half = M // 2 + 1
    if not swiglu:
        out_w = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
        ops.gemm(dev(wide)[:, :K], dev(w), out_w, dev(b))
        assert torch.equal(out_w, out)
        if ops.wants_mid(half, N, K):    # fewer rows may go to the weight-streaming kernel, which sums in another order
            out_h = torch.full((half, N), float("nan"), dtype=out_dtype, device="cuda")
            ops.gemm(dev(a[M - half:]), dev(w), out_h, dev(b))
            assert torch.equal(out_h, out[M - half:])


@pytest.mark.parametrize("M,N,K", [(65, 1024, 2048), (200, 333, 1024), (256, 4096, 1024), (130, 1024, 3072)])
def test_gemm_weight_streaming_many_rows(M, N, K):
    """Inside captured graphs the library's product is not used: the weight-streaming kernel deals
    more than 64 rows out to groups of workgroups, also in the gated form."""
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(23)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    want = a.double() @ w.double().T + b.double()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    library = ops.use_library_gemm
    ops.use_library_gemm = False
    try:
        ops.gemm(dev(a), dev(w), out, dev(b))
        assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[torch.bfloat16]
        if N % 2 == 0:
            I = N // 2
            full = a.double() @ w.double().T
            gated = torch.nn.functional.silu(full[:, :I]) * full[:, I:]
            act = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device="cuda")
            assert ops.gemm_swiglu(dev(a), dev(w), act)
            assert rel_err(act.float().cpu().numpy(), gated.numpy()) <= OP_TOL[torch.bfloat16]
    finally:
        ops.use_library_gemm = library


@pytest.mark.parametrize("M,N,K,with_bias,out_dtype", [
    (97, 1024, 2048, True, torch.bfloat16), (300, 4096, 4096, False, torch.bfloat16), (200, 336, 1024, False, torch.bfloat16),
    (2048, 6144, 1024, False, torch.bfloat16), (300, 4096, 12288, True, torch.bfloat16),
    (2048, 51200, 5120, False, torch.bfloat16), (128, 151936, 1024, False, torch.float32),
    (1, 151936, 1024, False, torch.float32), (8, 151936, 1024, False, torch.float32), (40, 151936, 1024, True, torch.float32),
    (100, 1001, 96, True, torch.float32), (400, 50021, 4096, False, torch.float32)])
def test_gemm_through_the_library(M, N, K, with_bias, out_dtype):
    """More than 64 rows outside graphs, and any number of rows into float32 against a very large
    weight (the logits): the library's product, called directly. The largest bf16 shape is one for
    which the library's first choice wants more workspace than a small one would hold."""
    ops = ops_for(torch.bfloat16)
    assert ops.lib.has("mv_gemm_lt")
    g = torch.Generator(device="cuda").manual_seed(29)
    a = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g, device="cuda").to(torch.bfloat16) if with_bias else None
    out = torch.full((M, N + 8), float("nan"), dtype=out_dtype, device="cuda")[:, :N]   # rows in a wider buffer
    calls = []
    real = ops._library_product
    ops._library_product = lambda *args: (calls.append(1), real(*args))[1]
    try:
        ops.gemm(a, w, out, b)
    finally:
        del ops._library_product
    assert calls, "the shape was left to another kernel"
    cols = torch.arange(0, N, max(1, N // 512), device="cuda")
    want = a.double() @ w[cols].double().T
    if with_bias:
        want = want + b[cols].double()
    tol = OP_TOL[torch.bfloat16] if out_dtype == torch.bfloat16 else 3e-6
    assert rel_err(out[:, cols].float().cpu().numpy(), want.cpu().numpy()) <= tol
    assert bool(torch.isfinite(out.float()).all())


TILE_SHAPES = {"auto": 0, "128x128": 40401, "128x128 deep": 140401, "64x128": 20401, "128x64": 40201, "64x64": 20201,
               "64x64 K/3": 20203, "128x128 K/2": 40402, "64x128 K/4": 20404}


@pytest.mark.parametrize("M,N,K,gated,out_dtype,with_bias", [
    (65, 4096, 1024, False, torch.bfloat16, True), (200, 333, 1024, False, torch.float32, True),
    (130, 2 * 1571, 4096, True, torch.bfloat16, False), (33, 1024, 3072, False, torch.bfloat16, False),
    (256, 6144, 1024, True, torch.bfloat16, False), (1000, 520, 192, False, torch.bfloat16, True),
    (40, 2 * 96, 64, True, torch.float32, False), (513, 136, 512, False, torch.float32, False)])
@pytest.mark.parametrize("shape", list(TILE_SHAPES))
def test_gemm_tiled(M, N, K, gated, out_dtype, with_bias, shape):
    """The tiled product for many rows at every tile it has (rows and columns that are no multiple
    of a tile, a K of one to 64 chunks, split or not), plain and as a gated pair with the activation
    in its epilogue, against float64; rows in a wider buffer give the same bits."""
    if gated and shape == "128x64":
        pytest.skip("a gated pair has no 128 x 64 tile")
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(31)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = ((2 if gated else 1) * torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    full = a.double() @ w.double().T
    if gated:
        want = torch.nn.functional.silu(full[:, :N // 2]) * full[:, N // 2:]
    else:
        want = full + b.double() if with_bias else full
    n_out = N // 2 if gated else N
    out = torch.full((M, n_out), float("nan"), dtype=out_dtype, device="cuda")
    assert ops.gemm_tile(dev(a), dev(w), out, dev(b) if with_bias else None, gated, TILE_SHAPES[shape])
    tol = 3e-6 if out_dtype == torch.float32 else OP_TOL[torch.bfloat16]
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= tol
    wide = torch.zeros(M, K + 40, dtype=torch.bfloat16)
    wide[:, :K] = a
    out_w = torch.full((M, n_out + 12), float("nan"), dtype=out_dtype, device="cuda")[:, :n_out]
    assert ops.gemm_tile(dev(wide)[:, :K], dev(w), out_w, dev(b) if with_bias else None, gated, TILE_SHAPES[shape])
    assert torch.equal(out_w, out)


@pytest.mark.parametrize("M,N,K,gated,with_bias", [(64, 4096, 1024, False, True), (96, 6144, 1024, True, False),
                                                   (40, 4100, 512, False, False), (33, 2 * 1571, 1024, True, False)])
# (each of these weights has at least 4 MB: smaller ones stay with the weight-streaming kernel)
def test_gemm_tiled_behind_a_folded_norm(M, N, K, gated, with_bias):
    """Rows that the product in front left weighted but not divided by their root mean square: the
    tiled product divides its output rows (before the bias, before the gate)."""
    from minivllm_amd.kernels.ops import WeightedRows
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(37)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = ((2 if gated else 1) * torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    P, eps = 7, 1e-5
    partial = torch.rand(M, P, generator=g) * K / P * 1.7
    rinv = torch.rsqrt(partial.double().sum(1, keepdim=True) / K + eps)
    full = (a.double() @ w.double().T) * rinv
    want = torch.nn.functional.silu(full[:, :N // 2]) * full[:, N // 2:] if gated else (full + b.double() if with_bias else full)

    class Fold:
        norm = None
    fold = Fold()
    fold.weighted, fold.partial, fold.eps, fold.normed = dev(a), dev(partial.float().contiguous()), eps, None
    rows = WeightedRows(ops, fold, P)
    n_out = N // 2 if gated else N
    out = torch.full((M, n_out), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.ledger = []
    try:
        if gated:
            assert ops.gemm_swiglu(rows, dev(w), out)
        else:
            ops.gemm(rows, dev(w), out, dev(b) if with_bias else None)
        assert [line[0] for line in ops.ledger] == ["mv_gemm_tile"], ops.ledger
    finally:
        ops.ledger = None
    assert rows.used
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[torch.bfloat16]


@pytest.mark.parametrize("M,N,K,gated,kernel", [
    (64, 4096, 1024, False, "mv_gemm_tile"), (300, 4096, 1024, False, "mv_gemm_tile"), (600, 4096, 1024, False, "mv_gemm_lt"),
    (32, 4096, 1024, False, "mv_gemm_skinny"), (100, 1024, 2048, False, "mv_gemm_lt"), (64, 4096, 4096, False, "mv_gemm_tile"),
    (200, 4096, 12288, False, "mv_gemm_tile"), (32, 4096, 4096, False, "mv_gemm_tile"), (40, 6144, 1024, True, "mv_gemm_tile"),
    (9, 4096, 4096, False, "mv_gemm_tile"), (8, 4096, 4096, False, "mv_gemm_skinny"), (8, 4096, 12288, False, "mv_gemm_tile"),
    (7, 4096, 12288, False, "mv_gemm_skinny"), (4, 5120, 25600, False, "mv_gemm_tile"), (12, 24576, 4096, True, "mv_gemm_tile"),
    (8, 24576, 4096, True, "mv_gemm_skinny_swiglu"), (20, 6144, 2048, True, "mv_gemm_mid"),
    (1024, 6144, 1024, True, "mv_gemm_tile"), (24, 6144, 1024, True, "mv_gemm_skinny_swiglu"),
    (40, 1024, 256, True, "mv_gemm_skinny_swiglu"),
    (100, 24576, 4096, True, "mv_gemm_tile"), (200, 24576, 4096, True, None)])
def test_which_product_takes_which_rows(M, N, K, gated, kernel):
    """Between the weight-streaming kernels (few rows) and the library (many), the tiled product."""
    ops = ops_for(torch.bfloat16)
    a = torch.randn(M, K, device="cuda").to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda") / math.sqrt(K)).to(torch.bfloat16)
    out = torch.empty(M, N // 2 if gated else N, dtype=torch.bfloat16, device="cuda")
    ops.ledger = []
    try:
        if gated:
            assert ops.gemm_swiglu(a, w, out) == (kernel is not None)
        else:
            ops.gemm(a, w, out)
        seen = [line[0] for line in ops.ledger]
    finally:
        ops.ledger = None
    assert seen == ([kernel] if kernel else []), seen


@pytest.mark.parametrize("M,I,K", [(1, 48, 64), (8, 3072, 1024), (40, 100, 96), (64, 560, 256),
                                   (6, 4104, 2048), (13, 4100, 2048)])     # (16 MB and more: loads of whole lines)
def test_gemm_swiglu_fused(M, I, K):
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(18)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (2 * torch.randn(2 * I, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    out = torch.full((M, I), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ops.gemm_swiglu(dev(a), dev(w), out)
    gu = a.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_beyond_two_to_the_31_elements(dtype):
    """A pool whose key and value tensors each hold more than 2^31 elements (what a small model gets
    when the device's memory is left to the cache): requests whose pages lie at the far end, among
    them the very last page, are written and read like any other. Three steps through every
    cache-writing and attention kernel: a prompt alone; a whole prompt beside a decoded token; both
    requests decoding (in bfloat16 also from the raw rows, by the kernel that writes the cache itself)."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(71)
    H, Hkv, D, ps = 16, 8, 128, 16
    page_elems = Hkv * ps * D
    num_pages = (1 << 31) // page_elems + 1500
    assert num_pages * page_elems > (1 << 31) + 1000 * page_elems
    kp = torch.empty(num_pages, Hkv, ps, D, dtype=dtype, device="cuda")
    vp = torch.empty(num_pages, Hkv, D, ps, dtype=dtype, device="cuda")
    ctx = [203, 302]                                        # lengths at the end
    pages_per = [-(-c // ps) for c in ctx]
    # pages from the top of the pool, the last one included, in scrambled order, and one low page each
    top = (num_pages - 2 - torch.randperm(1400, generator=g)[:sum(pages_per)]).tolist()
    top[3] = num_pages - 1
    tables = [top[:pages_per[0]], top[pages_per[0]:]]
    tables[0][5], tables[1][7] = 4, 11
    assert len(set(tables[0] + tables[1])) == sum(pages_per)
    for t in tables:                                        # what the kernels must not rely on
        idx = torch.tensor(t, device="cuda")
        kp[idx] = float("nan"); vp[idx] = float("nan")
    bt = torch.full((2, max(pages_per)), -1, dtype=torch.int32)
    for s_, t in enumerate(tables):
        bt[s_, :len(t)] = torch.tensor(t, dtype=torch.int32)
    bt = dev(bt)
    k_all = [torch.randn(c, Hkv, D, generator=g).to(dtype) for c in ctx]
    v_all = [torch.randn(c, Hkv, D, generator=g).to(dtype) for c in ctx]
    scale = 1.0 / math.sqrt(D)
    tol = 2 * max(OP_TOL[dtype], 5e-6)

    def run_step(spans, fused=False):
        """spans: (sequence, first position, tokens). Writes the tokens' keys and values, runs
        attention for them and compares with the reference over the sequences' whole prefixes."""
        positions, token_seq, rows_k, rows_v = [], [], [], []
        for s_, start, cnt in spans:
            positions += list(range(start, start + cnt)); token_seq += [s_] * cnt
            rows_k.append(k_all[s_][start:start + cnt]); rows_v.append(v_all[s_][start:start + cnt])
        n = len(positions)
        q = torch.randn(n, H, D, generator=g)
        for i in range(n):          # a key of the sequence's first page stands out for its last query
            if i + 1 == n or token_seq[i + 1] != token_seq[i]:
                q[i] = 6.0 * k_all[token_seq[i]][2].float().repeat_interleave(H // Hkv, dim=0) / math.sqrt(D)
        q = q.to(dtype)
        qkv = dev(torch.cat([q.view(n, -1), torch.cat(rows_k).view(n, -1), torch.cat(rows_v).view(n, -1)], dim=1))
        pos_t = torch.tensor(positions, dtype=torch.int32); seq_t = torch.tensor(token_seq, dtype=torch.int32)
        out = torch.full((n, H * D), float("nan"), dtype=dtype, device="cuda")
        q_lens = [cnt for _, _, cnt in spans]
        plan = make_plan(q_lens, [start + cnt for _, start, cnt in spans])
        plan_seq = dev(torch.tensor(sum(([i] * c for i, c in enumerate(q_lens)), []), dtype=torch.int32))
        step_bt = bt[[s_ for s_, _, _ in spans]].contiguous()
        if fused:
            assert ops.attention_decode_fused(qkv, out, kp, vp, step_bt, ps, dev(pos_t), plan_seq, H, Hkv, D, scale,
                                              None, plan, None, None, 1e-6, None, False, True)
        else:
            ops.qk_norm_rope_store(qkv, H, Hkv, D, dev(pos_t), plan_seq, None, None, 1e-6, None, False, kp, vp,
                                   step_bt, ps)
            ops.attention(qkv[:, :H * D], out, kp, vp, step_bt, ps, dev(pos_t), plan_seq, H, Hkv, D, scale, None,
                          plan=plan)
        torch.cuda.synchronize()
        want = reference_attention(q.double(), [k.double() for k in k_all], [v.double() for v in v_all], pos_t, seq_t,
                                   H, Hkv, scale, None)
        got = out.float().cpu().view(n, H, D)
        assert not torch.isnan(got).any()
        assert rel_err(got.numpy(), want.numpy()) <= tol

    run_step([(1, 0, 300)])                                 # a prompt alone (values go tile by tile)
    run_step([(0, 0, 201), (1, 300, 1)])                    # a whole prompt beside a decoded token
    run_step([(0, 201, 1), (1, 301, 1)])                    # both decode
    if dtype == torch.bfloat16:
        run_step([(0, 202, 1)], fused=True)                 # from the raw rows, one request
    # the pages hold exactly what was written, the last page of the pool included
    for s_, c in enumerate(ctx):
        upto = c if (dtype == torch.bfloat16 or s_ == 1) else c - 1
        for pos in (0, 1, 50, 3 * ps + 1, upto - 1):
            page, slot = tables[s_][pos // ps], pos % ps
            assert torch.equal(kp[page, :, slot, :].cpu(), k_all[s_][pos]), (s_, pos)
            assert torch.equal(vp[page, :, :, slot].cpu(), v_all[s_][pos]), (s_, pos)
    del kp, vp
    torch.cuda.empty_cache()


def test_attention_reduces_to_library_softmax():
    """One head, no window, whole sequence: equals torch's scaled_dot_product_attention."""
    ops = ops_for(torch.float32)
    g = torch.Generator().manual_seed(7)
    n, D, ps = 45, 32, 16
    q, k, v = (torch.randn(n, 1, D, generator=g) for _ in range(3))
    kp, vp = fill_pages([k.double()], [v.double()], [[2, 0, 1]], ps, 1, D, 3, torch.float32)
    bt = torch.tensor([[2, 0, 1]], dtype=torch.int32)
    pos = torch.arange(n, dtype=torch.int32)
    out = torch.empty(n, D, device="cuda")
    ops.attention(dev(q.view(n, D)), out, kp, vp, dev(bt), ps, dev(pos), dev(torch.zeros(n, dtype=torch.int32)),
                  1, 1, D, D ** -0.5, None)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None].double(), k.transpose(0, 1)[None].double(), v.transpose(0, 1)[None].double(),
        is_causal=True)[0, 0]
    assert rel_err(out.cpu().numpy(), want.numpy()) <= 3e-6


def test_sampling_greedy_and_draws():
    from plain import qwen3_plain as plain
    ops = ops_for(torch.float32)
    g = torch.Generator().manual_seed(8)
    M, V = 6, 1531
    logits = (2.5 * torch.randn(M, V, generator=g)).float()
    logits[1, 7] = logits[1, 900] = logits[1].max() + 1          # a tie: the lowest id wins
    out = torch.empty(M, dtype=torch.int32, device="cuda")
    ops.sample(dev(logits), out)
    want = [int(torch.argmax(logits[i])) for i in range(M)]
    want[1] = 7
    assert out.cpu().tolist() == want
    temps = torch.tensor([0.0, 0.7, 1.0, 1.3, 0.9, 2.0])
    top_k = torch.tensor([0, 0, 40, 0, 12, 3], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 1.0, 0.8, 0.6, 0.95])
    for counter in range(4):
        rng = torch.tensor([[1234 + i, counter] for i in range(M)], dtype=torch.int64)
        ops.sample(dev(logits), out, dev(temps), dev(top_k), dev(top_p), dev(rng))
        got = out.cpu().tolist()
        for i in range(M):
            tok, score = plain.sample_token(logits[i].numpy(), float(temps[i]), int(top_k[i]), float(top_p[i]),
                                            seed=1234 + i, counter=counter)
            # the same token, or one whose perturbed score ties within float rounding
            assert np.isfinite(score[got[i]]), f"row {i}: token {got[i]} is outside the kept set"
            assert score[got[i]] >= score[tok] - 1e-4 * max(1.0, abs(float(score[tok]))), (i, got[i], tok)


@pytest.mark.parametrize("V,pad", [(50021, 0), (50021, 3), (151936, 0)])
def test_sampling_large_vocabulary_two_passes(V, pad):
    """With a large vocabulary the rows that need no threshold are shared by many workgroups (two
    launches); every row gets the token the one-launch path gives it."""
    ops = ops_for(torch.float32)
    g = torch.Generator().manual_seed(81)
    M = 7
    wide = (2.0 * torch.randn(M, V + pad, generator=g)).float()
    logits = wide[:, :V]
    logits[0, 11] = logits[0, V - 5] = logits[0].max() + 1       # a tie across chunks: the lowest id wins
    temps = torch.tensor([0.0, 0.0, 0.9, 1.2, 0.8, 1.0, 0.0])
    top_k = torch.tensor([0, 5, 0, 0, 50, 0, 0], dtype=torch.int32)
    top_p = torch.tensor([1.0, 0.5, 1.0, 1.0, 1.0, 0.9, 1.0])
    rng = torch.tensor([[77 + i, 3] for i in range(M)], dtype=torch.int64)
    x = dev(wide)[:, :V]
    two = torch.empty(M, dtype=torch.int32, device="cuda")
    one = torch.empty(M, dtype=torch.int32, device="cuda")
    d_temps, d_k, d_p, d_rng = dev(temps), dev(top_k), dev(top_p), dev(rng)
    ops.sample(x, two, d_temps, d_k, d_p, d_rng)
    assert ops._sample_work is not None
    ops.lib.call("mv_sample", x.data_ptr(), x.stride(0), M, V, d_temps.data_ptr(), d_k.data_ptr(), d_p.data_ptr(),
                 d_rng.data_ptr(), one.data_ptr(), 0, 1, ops._stream())
    torch.cuda.synchronize()
    assert two.cpu().tolist() == one.cpu().tolist()
    assert two[0].item() == 11 and two[1].item() == int(torch.argmax(logits[1])) \
        and two[6].item() == int(torch.argmax(logits[6]))
    ops.sample(x, two)                                            # all rows greedy
    assert two.cpu().tolist() == [11] + [int(torch.argmax(logits[i])) for i in range(1, M)]


def test_sampling_frequencies():
    """Draws follow softmax(logits / T) on a small vocabulary."""
    ops = ops_for(torch.float32)
    V, T, draws = 11, 0.8, 4000
    logits = torch.linspace(-2, 2, V)[None].repeat(draws, 1).contiguous()
    out = torch.empty(draws, dtype=torch.int32, device="cuda")
    temps = torch.full((draws,), T)
    rng = torch.tensor([[99, c] for c in range(draws)], dtype=torch.int64)
    ops.sample(dev(logits), out, dev(temps), None, None, dev(rng))
    freq = np.bincount(out.cpu().numpy(), minlength=V) / draws
    p = torch.softmax(logits[0].double() / T, dim=0).numpy()
    assert np.abs(freq - p).max() < 4 * np.sqrt(p.max() / draws)


@pytest.mark.parametrize("M,N,K,swiglu", [(1, 4096, 1024, False), (8, 1000, 1024, False), (16, 96, 64, False),
                                          (8, 3072, 1024, True), (3, 200, 128, True), (5, 333, 2048, False),
                                          # (16 MB and more: loads of whole lines)
                                          (7, 6144, 2048, False), (8, 8200, 1536, False), (4, 2 * 4112, 2048, True)])
@pytest.mark.parametrize("with_delta", [True, False])
def test_gemm_with_fused_add_and_norm(M, N, K, swiglu, with_delta):
    """Residual add + RMSNorm + product (or gated pair) as one kernel, through the deferred-norm
    interface of the parts."""
    from minivllm_amd.parts import NORMS, HiddenStream, RMSNormSpec, Runtime, Workspace
    from minivllm_amd.parts.base import PendingNorm
    ops = ops_for(torch.bfloat16)
    rt = Runtime(device=torch.device("cuda:0"), dtype=torch.bfloat16, ops=ops,
                 workspace=Workspace(torch.device("cuda:0")), max_positions=16)
    g = torch.Generator().manual_seed(44)
    spec = RMSNormSpec(size=K, eps=1e-5)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16)
    norm = NORMS.get(spec.kind)(spec, {"weight": dev(nw)}, rt)
    resid = torch.randn(M, K, generator=g)
    delta = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn((2 * N if swiglu else N), K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    bias = None if swiglu else torch.randn(N, generator=g).to(torch.bfloat16)
    assert ops.can_fuse_norm(M, K)
    stream = HiddenStream(dev(resid).clone(), torch.full((M, K), float("nan"), device="cuda"))
    if with_delta:
        stream.delta = dev(delta)
    first = stream.resid
    pending = norm.pending(stream, None)
    assert isinstance(pending, PendingNorm)
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    if swiglu:
        assert ops.gemm_swiglu(pending, dev(w), out)
    else:
        ops.gemm(pending, dev(w), out, dev(bias))
    x = resid.double() + (delta.double() if with_delta else 0)
    a = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * nw.double()).to(torch.bfloat16).double()
    if swiglu:
        gu = a @ w.double().T
        want = torch.nn.functional.silu(gu[:, :N]) * gu[:, N:]
    else:
        want = a @ w.double().T + bias.double()
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[torch.bfloat16]
    # the stream moved on as if the norm had run: the sum sits in the other buffer, nothing pending
    assert stream.delta is None
    if with_delta:
        assert stream.resid is not first and stream.spare is first
        assert rel_err(stream.resid.cpu().numpy(), x.float().numpy()) <= 1e-7
        assert torch.equal(first.cpu(), resid)                   # the old sum was only read
    else:
        assert stream.resid is first


@pytest.mark.parametrize("M,N,K,N2,swiglu", [(64, 1024, 2048, 4096, False), (17, 1024, 3072, 3072, True),
                                             (40, 224, 96, 333, False), (33, 96, 64, 56, True),
                                             (8, 4096, 4096, 6144, False), (20, 992, 1024, 100, False),
                                             (80, 1024, 2048, 4096, False), (96, 1024, 3072, 3072, True)])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("consumer", ["product", "rows"])
def test_residual_add_and_norm_folded_into_the_products_around_them(M, N, K, N2, swiglu, with_bias, consumer):
    """A step of more rows than the fused add + norm + product kernel takes: the product in front of
    the norm adds its output to the residual and leaves the rows weighted with partial sums of
    squares (``gemm(..., fold=...)``), the product behind it divides its output rows by the root mean
    square (``gemm(WeightedRows, ...)``) — or, for a consumer that cannot, the rows are normalised by
    a kernel of their own. Against the stand-alone add and norm between two plain products."""
    from minivllm_amd.kernels.ops import WeightedRows
    from minivllm_amd.parts import NORMS, HiddenStream, RMSNormSpec, Runtime, Workspace
    ops = ops_for(torch.bfloat16)
    rt = Runtime(device=torch.device("cuda:0"), dtype=torch.bfloat16, ops=ops,
                 workspace=Workspace(torch.device("cuda:0")), max_positions=16)
    g = torch.Generator().manual_seed(45)
    eps = 1e-5
    spec = RMSNormSpec(size=N, eps=eps)
    nw = (1 + 0.1 * torch.randn(N, generator=g)).to(torch.bfloat16)
    norm = NORMS.get(spec.kind)(spec, {"weight": dev(nw)}, rt)
    resid = 3.0 * torch.randn(M, N, generator=g)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    b1 = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    w2 = (torch.randn((2 * N2 if swiglu else N2), N, generator=g) / math.sqrt(N)).to(torch.bfloat16)
    b2 = torch.randn(N2, generator=g).to(torch.bfloat16) if (with_bias and not swiglu) else None
    assert not ops.can_fuse_norm(M, N) and ops.can_fold_norm(M, N, (w2.shape[0], N, swiglu))
    assert not ops.can_fold_norm(97, N, (w2.shape[0], N, swiglu)) and not ops.can_fold_norm(80, 4096, (6144, 4096, False))
    stream = HiddenStream(dev(resid).clone(), torch.full((M, N), float("nan"), device="cuda"))
    assert norm.fold(stream, None) is None                      # nobody said what comes behind the norm
    assert norm.fold(stream, None, (200 * 1000, N, False)) is None or N * 200 * 1000 < 96 * 1000 * 1000   # the library's
    fold = norm.fold(stream, None, (w2.shape[0], N, swiglu))
    assert fold is not None
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    rows = ops.gemm(dev(a), dev(w1), y, dev(b1) if b1 is not None else None, defer_sum=True, fold=fold)
    assert isinstance(rows, WeightedRows) and torch.isnan(y.float()).all()      # the delta was never written
    stream.weighted = rows
    # the reference: plain product, rounded; add; norm; plain product
    delta = (a.double() @ w1.double().T + (b1.double() if b1 is not None else 0)).to(torch.bfloat16).double()
    x = resid.double() + delta
    assert rel_err(stream.resid.cpu().numpy(), x.float().numpy()) <= 2e-3       # a delta may round the other way
    normed = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * nw.double())
    out = torch.full((M, N2), float("nan"), dtype=torch.bfloat16, device="cuda")
    if consumer == "rows":
        h = norm.forward(stream, None)              # whoever wants a tensor gets the normalised rows
        assert rel_err(h.float().cpu().numpy(), normed.numpy()) <= OP_TOL[torch.bfloat16]
        assert stream.weighted is None
        return
    h = norm.pending(stream, None)
    assert h is rows and stream.weighted is None
    if swiglu:
        assert ops.gemm_swiglu(h, dev(w2), out)
        gu = normed.to(torch.bfloat16).double() @ w2.double().T
        want = torch.nn.functional.silu(gu[:, :N2]) * gu[:, N2:]
    else:
        ops.gemm(h, dev(w2), out, dev(b2) if b2 is not None else None)
        want = normed.to(torch.bfloat16).double() @ w2.double().T + (b2.double() if b2 is not None else 0)
    assert rows.used
    assert rel_err(out.float().cpu().numpy(), want.numpy()) <= OP_TOL[torch.bfloat16]


def test_norm_is_not_deferred_for_many_rows():
    from minivllm_amd.parts import NORMS, HiddenStream, RMSNormSpec, Runtime, Workspace
    ops = ops_for(torch.bfloat16)
    rt = Runtime(device=torch.device("cuda:0"), dtype=torch.bfloat16, ops=ops,
                 workspace=Workspace(torch.device("cuda:0")), max_positions=16)
    spec = RMSNormSpec(size=128, eps=1e-5)
    norm = NORMS.get(spec.kind)(spec, {"weight": torch.ones(128, device="cuda")}, rt)
    stream = HiddenStream(torch.randn(17, 128, device="cuda"), torch.empty(17, 128, device="cuda"))
    assert isinstance(norm.pending(stream, None), torch.Tensor)
    assert not ops_for(torch.float32).can_fuse_norm(4, 128)


@pytest.mark.parametrize("M,N,K,with_bias,with_rows", [(12, 4096, 4096, False, False), (33, 3080, 4096, True, False),
                                                      (64, 2048, 8192, False, True), (2, 5120, 25600, False, False)])
def test_partial_sums_of_a_product_go_straight_into_the_norm(M, N, K, with_bias, with_rows):
    """A product whose K was split leaves its partial sums to the residual add + norm that follows
    (``defer_sum``): the new residual and the normalised rows are bit for bit those of the path that
    adds the sums up in a kernel of its own first; asking for the tensor instead gives the same
    product; and the next product of the kind adds an unused one up before it takes the work area."""
    from minivllm_amd.kernels.ops import SplitSum
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(29)
    a = dev(torch.randn(M, K, generator=g).to(torch.bfloat16))
    w = dev((torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16))
    b = dev(torch.randn(N, generator=g).to(torch.bfloat16)) if with_bias else None
    nw = dev((1 + 0.1 * torch.randn(N, generator=g)).to(torch.bfloat16))
    resid0 = dev(torch.randn(M, N, generator=g))
    rows = dev(torch.tensor([M - 1, 0], dtype=torch.int32)) if with_rows else None
    n_out = 2 if with_rows else M

    plain = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    assert ops.gemm(a, w, plain, b) is None
    resid_a, out_a = resid0.clone(), torch.full((n_out, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(resid_a, plain, nw, 1e-6, out_a, rows=rows)

    target = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    split = ops.gemm(a, w, target, b, defer_sum=True)
    assert isinstance(split, SplitSum), "the shape was left to another kernel"
    resid_b, out_b = resid0.clone(), torch.full((n_out, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.add_rmsnorm(resid_b, split, nw, 1e-6, out_b, rows=rows)
    assert torch.equal(out_a, out_b) and torch.equal(resid_a, resid_b)
    assert split.done != with_rows          # with rows the delta stays pending in the stream
    if with_rows:
        assert torch.isnan(target.float()).all()
        assert torch.equal(split.materialize(), plain)

    # an unused one is added up when the next product needs the work area
    first = ops.gemm(a, w, target, b, defer_sum=True)
    other = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    second = ops.gemm(a, w, other, b, defer_sum=True)
    assert first.done and torch.equal(target, plain)
    assert torch.equal(second.materialize(), plain) and second.done and ops._split_pending is None


def test_kernels_that_load_straight_into_lds_repeat_their_results():
    """The K-splitting product, the tiled product and the prompt attention bring operands into LDS with
    loads whose completion they wait for by count. A wait that came too early would show as results
    that differ from call to call; here many calls in a row give the same bits."""
    ops = ops_for(torch.bfloat16)
    g = torch.Generator().manual_seed(31)
    for M, N, K, gated in ((64, 4096, 4096, False), (200, 4096, 1024, False), (96, 6144, 1024, True), (256, 4096, 12288, False),
                           (1024, 6144, 1024, True)):
        a = dev(torch.randn(M, K, generator=g).to(torch.bfloat16))
        w = dev((torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16))
        first = torch.empty(M, N // 2 if gated else N, dtype=torch.bfloat16, device="cuda")
        assert ops.wants_tile(M, N, K, gated) and ops.gemm_tile(a, w, first, None, gated)
        for _ in range(30):
            again = torch.empty_like(first)
            assert ops.gemm_tile(a, w, again, None, gated)
            assert torch.equal(first, again)
    ops.use_tiled_gemm = False
    try:
        for M, N, K in ((32, 4096, 4096), (9, 3100, 8192), (30, 12288, 2048)):
            a = dev(torch.randn(M, K, generator=g).to(torch.bfloat16))
            w = dev((torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16))
            ops._mid_work = None
            first = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
            ops.gemm(a, w, first)
            assert ops._mid_work is not None
            for _ in range(30):
                again = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
                ops.gemm(a, w, again)
                assert torch.equal(first, again)
    finally:
        ops.use_tiled_gemm = True
    # prompt attention: one long portion over scrambled pages, both walks of the keys
    H, Hkv, D, ps = 16, 8, 128, 16
    for T in (700, 2048):
        k_all = [torch.randn(T, Hkv, D, generator=g)]
        v_all = [torch.randn(T, Hkv, D, generator=g)]
        pages = -(-T // ps)
        order = torch.randperm(pages + 3, generator=g)[:pages].tolist()
        kp, vp = fill_pages(k_all, v_all, [order], ps, Hkv, D, pages + 3, torch.bfloat16)
        bt = dev(torch.tensor([order], dtype=torch.int32))
        q = dev(torch.randn(T, H * D, generator=g).to(torch.bfloat16))
        pos = dev(torch.arange(T, dtype=torch.int32))
        tseq = dev(torch.zeros(T, dtype=torch.int32))
        plan = make_plan([T], [T])
        first = torch.empty(T, H * D, dtype=torch.bfloat16, device="cuda")
        ops.attention(q, first, kp, vp, bt, ps, pos, tseq, H, Hkv, D, D ** -0.5, None, plan=plan)
        for _ in range(20):
            again = torch.empty(T, H * D, dtype=torch.bfloat16, device="cuda")
            ops.attention(q, again, kp, vp, bt, ps, pos, tseq, H, Hkv, D, D ** -0.5, None, plan=plan)
            assert torch.equal(first, again)
