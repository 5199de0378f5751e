"""Every kernel of ops.seqmix against the fp32 PyTorch reference of the same op (ops.reference), in bf16 and in true
fp32, at sizes that are not multiples of the tiles and at sizes that take the vectorised / MFMA paths."""

import pytest
import torch

from k8s_llm_scheduler_amd.ops import reference as ref
from k8s_llm_scheduler_amd.ops import seqmix as sm

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)]
T = 37


def close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    if a.numel() == 0:
        assert a.shape == b.shape
        return
    assert (a - b).abs().max().item() <= tol * max(b.abs().max().item(), 1e-6)


def batch():
    """Four sequences (one empty, one resumed mid-sequence, one starting at 0) over T tokens."""
    cu = torch.tensor([0, 9, 10, 10, T], dtype=torch.int32)
    pos = torch.cat([torch.arange(0, 9), torch.tensor([5]), torch.arange(3, 30)]).int()
    slots = torch.tensor([2, 0, 1, 3], dtype=torch.int32)
    tok_seq = torch.searchsorted(cu[1:].contiguous(), torch.arange(T, dtype=torch.int32), right=True).int()
    return cu, pos, slots, tok_seq


@pytest.mark.parametrize("dt,tol", DTYPES)
def test_stream_ops(dt, tol):
    torch.manual_seed(0)
    W = 200
    ids = torch.randint(0, 50, (T,), dtype=torch.int32)
    table = torch.randn(50, W).to(dt)
    close(sm.embed_rows(ids.to(DEV), table.to(DEV)), sm.embed_rows(ids, table), 0)
    x, br, rv, w = torch.randn(T, W), torch.randn(T, W).to(dt), torch.randn(W).to(dt), (torch.randn(W) * 0.1).to(dt)
    xg, xc = x.to(DEV).clone(), x.clone()
    og = sm.resnorm(xg, w.to(DEV), 1e-6, branch=br.to(DEV), mult=0.3, rowvec=rv.to(DEV), offset=1.0, out_dtype=dt)
    oc = sm.resnorm(xc, w, 1e-6, branch=br, mult=0.3, rowvec=rv, offset=1.0, out_dtype=dt)
    close(og, oc, tol)
    close(xg, xc, 1e-6)
    assert sm.resnorm(xg, None, 1e-6, branch=br.to(DEV), mult=2.0, out_dtype=dt) is None
    sm.resnorm(xc, None, 1e-6, branch=br, mult=2.0, out_dtype=dt)
    close(xg, xc, 1e-6)
    for kind in (sm.ACT_GELU_TANH, sm.ACT_SWISH_CLAMP, sm.ACT_TANH, sm.ACT_SILU):
        a = torch.randn(T, 140).to(dt) * 2
        close(sm.act(a.to(DEV), kind, 1.0, 1.702), sm.act(a, kind, 1.0, 1.702), tol)
    a = torch.randn(T, 140).to(dt) * 3
    close(sm.act(a.to(DEV), sm.ACT_SWISH_CLAMP, 0.0, 1.702), sm.act(a, sm.ACT_SWISH_CLAMP, 0.0, 1.702), tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("M,N,K", [(37, 200, 96), (1, 16, 256), (130, 70, 16), (64, 64, 64), (5, 640, 255), (3, 7, 5),
                                   (200, 136, 72), (65, 129, 1032), (1100, 2056, 40), (2048, 1024, 64)])
def test_gemm_shapes(dt, tol, M, N, K):
    torch.manual_seed(1)
    a, w = torch.randn(M, K).to(dt), (torch.randn(N, K) / K ** 0.5).to(dt)
    for out in (dt, torch.float32):
        close(sm.gemm(a.to(DEV), w.to(DEV), out), sm.gemm(a, w, out), tol)
    if dt == torch.float32:      # true fp32: far below any reduced-precision matrix mode
        exact = a.double() @ w.double().T
        assert (sm.gemm(a.to(DEV), w.to(DEV)).cpu().double() - exact).abs().max() < 1e-5 * max(1.0, K ** 0.5)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,Dn,R,C", [(6, 40, 24, 72), (3, 7, 5, 9)])
def test_gemm_batched_strided(dt, tol, H, Dn, R, C):
    torch.manual_seed(2)
    q, uk = torch.randn(T, H * (Dn + R)).to(dt), (torch.randn(H, C, Dn) / Dn ** 0.5).to(dt)

    def run(q, uk):
        out = torch.empty(T, H, C, dtype=dt, device=q.device)
        sm.gemm(q.view(T, H, Dn + R)[:, :, :Dn].permute(1, 0, 2), uk, out=out.permute(1, 0, 2))
        return out

    close(run(q.to(DEV), uk.to(DEV)), run(q, uk), tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
def test_token_shift_and_save(dt, tol):
    torch.manual_seed(3)
    W = 200
    cu, pos, slots, tok_seq = batch()
    h, mu, st = torch.randn(T, W).to(dt), torch.rand(5, W).to(dt), torch.randn(4, W).to(dt)
    d = lambda *ts: (t.to(DEV) for t in ts)
    close(sm.token_shift(*d(h, mu, st, cu, tok_seq, slots, pos)), sm.token_shift(h, mu, st, cu, tok_seq, slots, pos), tol)
    sg, sc = st.to(DEV).clone(), st.clone()
    sm.shift_save(sg, *d(h, cu, slots, pos))
    sm.shift_save(sc, h, cu, slots, pos)
    close(sg, sc, 0)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,D", [(3, 48), (2, 32), (2, 80), (5, 20), (1, 128)])
def test_wkv_scan(dt, tol, H, D):
    torch.manual_seed(4)
    cu, pos, slots, _ = batch()
    HD = H * D
    r, k, v, g = (torch.randn(T, HD).to(dt) for _ in range(4))
    z, w0 = torch.randn(T, HD), (torch.rand(HD) * 3 - 2).to(dt)
    u, lnw = (torch.randn(HD) * 0.5).to(dt), (1 + 0.1 * torch.randn(HD)).to(dt)
    S = torch.randn(4, H, D, D)
    Sg, Sc = S.to(DEV).clone(), S.clone()
    og = sm.wkv_scan(*(t.to(DEV) for t in (r, k, v, g, z, w0, u, lnw)), Sg, cu.to(DEV), slots.to(DEV), pos.to(DEV), H, D, 1e-6)
    oc = sm.wkv_scan(r, k, v, g, z, w0, u, lnw, Sc, cu, slots, pos, H, D, 1e-6)
    close(og, oc, tol * 3)
    close(Sg, Sc, 1e-4)
    assert torch.equal(Sg[1].cpu(), S[1])        # the empty sequence's slot is untouched
    for chunk in (4, 5, 16, 64):                  # the three-pass form over chunks: the same outputs and end states
        Sk = S.to(DEV).clone()
        ok = sm.wkv_scan(*(t.to(DEV) for t in (r, k, v, g, z, w0, u, lnw)), Sk, cu.to(DEV), slots.to(DEV), pos.to(DEV), H, D,
                         1e-6, chunk=chunk)
        close(ok, oc, tol * 3)
        close(Sk, Sc, 1e-4)
        assert torch.equal(Sk[1].cpu(), S[1])


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,Dn,R,C,dims,win", [(6, 40, 24, 72, 24, 7), (3, 16, 8, 130, 4, 0), (10, 32, 32, 64, 32, 100),
                                               (2, 64, 64, 512, 64, 20), (20, 16, 8, 48, 8, 0), (16, 8, 24, 96, 24, 13),
                                               (5, 32, 40, 272, 40, 33)])
def test_latent_attention(dt, tol, H, Dn, R, C, dims, win):
    torch.manual_seed(5)
    cu, pos, slots, tok_seq = batch()
    bs, per = 16, 2
    L = C + R
    cache = torch.randn(4 * per * bs, L).to(dt)
    bt = torch.randperm(4 * per).view(4, per).int()         # disjoint blocks per sequence
    slot_map = torch.tensor([int(bt[tok_seq[t], pos[t] // bs]) * bs + int(pos[t]) % bs for t in range(T)],
                            dtype=torch.int32)
    slot_map[9] = -1                                          # a row whose cache write is dropped
    dkv, nw = torch.randn(T, L).to(dt), (1 + 0.1 * torch.randn(C)).to(dt)
    q = torch.randn(T, H * (Dn + R)).to(dt)
    cs = ref.rope_table(dims, 64, 10000.0)
    cg, qg, cc, qc = cache.to(DEV).clone(), q.to(DEV).clone(), cache.clone(), q.clone()
    sm.latent_kv_write(cg, dkv.to(DEV), nw.to(DEV), qg, cs.to(DEV), pos.to(DEV), slot_map.to(DEV), C, R, H, Dn, dims, 1e-6)
    sm.latent_kv_write(cc, dkv, nw, qc, cs, pos, slot_map, C, R, H, Dn, dims, 1e-6)
    close(cg, cc, tol)
    close(qg, qc, tol)
    qabs = torch.randn(T, H, C).to(dt) * 0.3
    oc = sm.latent_attention(qabs, qc, cc, bt, tok_seq, pos, C, R, H, Dn, win, 0.2, bs)
    for kw in ({}, {"cu_q": cu.to(DEV), "max_qlen": 27}):      # per token, and four tokens of a sequence per workgroup
        og = sm.latent_attention(qabs.to(DEV), qc.to(DEV), cc.to(DEV), bt.to(DEV), tok_seq.to(DEV), pos.to(DEV), C, R, H,
                                 Dn, win, 0.2, bs, **kw)
        close(og, oc, tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("E,top,F,W", [(16, 2, 24, 200), (70, 3, 24, 40), (4, 4, 7, 33), (8, 2, 64, 128)])
def test_moe(dt, tol, E, top, F, W):
    torch.manual_seed(6)
    lg = torch.randn(T, E + 1) * 2
    ig, wg = sm.moe_route(lg.to(DEV), E, top, 2.5)
    ic, wc = sm.moe_route(lg, E, top, 2.5)
    assert torch.equal(ig.cpu(), ic)
    close(wg, wc, 1e-5)
    stg, pg, sgg, tg = sm.moe_align(ig, E)
    stc, pc, sgc, tc = sm.moe_align(ic, E)
    assert torch.equal(sgg.cpu(), sgc)
    for e in range(E):                                       # the same tokens under every expert, in any order
        a, b = int(sgc[e]), int(sgc[e + 1])
        assert sorted(stg.cpu()[a:b].tolist()) == sorted(stc[a:b].tolist())
    assert torch.equal(stg.cpu()[pg.cpu().long()], torch.arange(T).repeat_interleave(top).int())
    live = tg.cpu()[tg.cpu()[:, 0] >= 0]
    assert int(live[:, 2].sum()) == T * top
    hh, wgu, wd = torch.randn(T, W).to(dt), (torch.randn(E, 2 * F, W) / W ** 0.5).to(dt), (torch.randn(E, W, F) / F ** 0.5).to(dt)
    sh = torch.randn(T, W).to(dt)

    def run(hh, wgu, wd, sh, st_, p_, seg_, t_, w_, lg_):
        gu = sm.gemm(hh, wgu, a_rows=st_, tiles=t_, rows=T * top, seg=seg_)
        D = sm.gemm(sm.act(gu, sm.ACT_SWISH_CLAMP, 1.0, 1.702), wd, tiles=t_, rows=T * top, seg=seg_)
        return sm.moe_combine(D, p_, w_, sh, lg_, E), sm.moe_combine(D, p_, w_, None, lg_, -1)

    for a, b in zip(run(hh.to(DEV), wgu.to(DEV), wd.to(DEV), sh.to(DEV), stg, pg, sgg, tg, wg, lg.to(DEV)),
                    run(hh, wgu, wd, sh, stc, pc, sgc, tc, wc, lg)):
        close(a, b, tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,win", [(4, 0), (20, 0), (6, 40), (3, 64), (3, 65), (16, 1)])
def test_latent_attention_long_contexts(dt, tol, H, win):
    """Few tokens over long contexts: several 32-key steps, key splits and their merge, window starts that are not
    multiples of the step, an idle row."""
    torch.manual_seed(7)
    C, R, Dn, bs, nb = 96, 32, 24, 16, 20
    pos = torch.tensor([299, 300, 31, 32, 33, -1, 64, 130], dtype=torch.int32)
    tok_seq = torch.tensor([0, 0, 1, 1, 1, 2, 3, 3], dtype=torch.int32)
    Tn = pos.numel()
    bt = torch.randperm(4 * nb).view(4, nb).int()
    cache = torch.randn(4 * nb * bs, C + R).to(dt)
    q = torch.randn(Tn, H * (Dn + R)).to(dt)
    qabs = (torch.randn(Tn, H, C) * 0.3).to(dt)
    for max_keys in (0, 512):
        og = sm.latent_attention(qabs.to(DEV), q.to(DEV), cache.to(DEV), bt.to(DEV), tok_seq.to(DEV), pos.to(DEV), C, R, H,
                                 Dn, win, 0.15, bs, max_keys)
        oc = sm.latent_attention(qabs, q, cache, bt, tok_seq, pos, C, R, H, Dn, win, 0.15, bs)
        live = pos >= 0
        close(og.cpu()[live], oc[live], tol)
        assert torch.equal(og.cpu()[~live].float(), torch.zeros(1, H, C))
    assert sm.latent_splits(Tn, H, 512) > 1 and sm.latent_splits(4096, H, 512) == 1


def test_grouped_gemm_many_rows():
    """Enough row tiles for the wide (64 x 128) form of the MFMA GEMM, grouped by expert with gathered rows."""
    torch.manual_seed(8)
    Tn, top, E, N, K = 1500, 2, 4, 1032, 64
    idx = torch.randint(0, E, (Tn, top), dtype=torch.int32)
    st, pos, seg, tiles = sm.moe_align(idx.to(DEV), E)
    stc, posc, segc, tilesc = sm.moe_align(idx, E)
    h, w = torch.randn(Tn, K).to(torch.bfloat16), (torch.randn(E, N, K) / K ** 0.5).to(torch.bfloat16)
    got = sm.gemm(h.to(DEV), w.to(DEV), a_rows=st, tiles=tiles, rows=Tn * top).cpu().float()
    want = sm.gemm(h, w, a_rows=stc, tiles=tilesc, rows=Tn * top, seg=segc).float()
    # rows of an expert may come in another order: compare per (token, choice) pair
    close(got[pos.cpu().long()], want[posc.long()], 2e-2)


# ----------------------------------------------------------------------------- grouped norm, row-scaled gelu, sigmoid router
@pytest.mark.parametrize("dt,tol", DTYPES)
def test_grouped_norm_scaled_embedding_and_row_factors(dt, tol):
    torch.manual_seed(20)
    W = 240
    ids = torch.randint(0, 50, (T,), dtype=torch.int32)
    table = torch.randn(50, W).to(dt)
    close(sm.embed_rows(ids.to(DEV), table.to(DEV), 3.7), sm.embed_rows(ids, table, 3.7), 1e-6)
    for groups in (2, 5, 8, 240):
        x, br, rv, w = torch.randn(T, W), torch.randn(T, W).to(dt), torch.randn(W).to(dt), torch.randn(W).to(dt)
        xg, xc = x.to(DEV).clone(), x.clone()
        og = sm.resnorm(xg, w.to(DEV), 1e-6, branch=br.to(DEV), rowvec=rv.to(DEV), out_dtype=dt, groups=groups)
        oc = sm.resnorm(xc, w, 1e-6, branch=br, rowvec=rv, out_dtype=dt, groups=groups)
        close(og, oc, tol)
        close(xg, xc, 1e-6)
    a = (torch.randn(T, 70) * 2).to(dt)
    close(sm.act(a.to(DEV), sm.ACT_GELU_ERF), sm.act(a, sm.ACT_GELU_ERF), tol)
    sc, perm = torch.rand(T) * 2, torch.randperm(T).int()
    close(sm.act(a.to(DEV), sm.ACT_GELU_ERF, row_scale=sc.to(DEV), row_map=perm.to(DEV)),
          sm.act(a, sm.ACT_GELU_ERF, row_scale=sc, row_map=perm), tol)
    close(sm.act(a.to(DEV), sm.ACT_SILU, row_scale=sc.to(DEV)), sm.act(a, sm.ACT_SILU, row_scale=sc), tol)


@pytest.mark.parametrize("E,top", [(8, 2), (70, 4), (5, 5), (3, 1)])
def test_sigmoid_router_and_plain_combine(E, top):
    torch.manual_seed(21)
    logits = torch.randn(T, E + 1) * 2
    ig, wg = sm.moe_route(logits.to(DEV), E, top, 1.0, score="sigmoid")
    ic, wc = sm.moe_route(logits, E, top, 1.0, score="sigmoid")
    assert torch.equal(ig.cpu(), ic)
    close(wg, wc, 1e-6)
    assert torch.allclose(wc, torch.sigmoid(logits[:, :E]).gather(1, ic.long()))
    D = torch.randn(T * top, 24)
    pos = torch.randperm(T * top).int()
    shared = torch.randn(T, 24)
    close(sm.moe_combine(D.to(DEV), pos.to(DEV), None, shared.to(DEV), None, -1, top=top),
          sm.moe_combine(D, pos, None, shared, None, -1, top=top), 1e-6)
    close(sm.moe_combine(D.to(DEV), pos.to(DEV), None, None, None, -1, top=top),
          sm.moe_combine(D, pos, None, None, None, -1, top=top), 1e-6)


# ----------------------------------------------------------------------------- windowed attention with pooled blocks
def window_case(H, G, D, V, window, P, dims, dt, bs=16, seed=0, chunk=0, softcap=0.0, sinks=False, per_head=False,
                half=False, qk_norm=False, unit=True):
    """Three sequences over shuffled pages: a prompt from 0, a portion that resumes at position 70 and a single token at
    position 130; their earlier tokens are written to the caches first (in two batches, so pooled blocks straddle
    them).  ``chunk`` / ``softcap`` / ``sinks`` / ``per_head`` / ``half`` / ``qk_norm`` / ``unit``: the chunked mask,
    capped scores, learned sinks, one gate number per head, the half rotation layout, whole-projection norms, unit
    heads."""
    torch.manual_seed(seed)
    nblk = 40
    lens = [(0, 90), (70, 55), (130, 1)]
    perm = torch.randperm(nblk).int()
    bt = torch.zeros(3, 12, dtype=torch.int32)
    for s in range(3):
        bt[s] = perm[12 * s:12 * s + 12]
    ncol = H * D + G * D + G * V + H * V
    cs = ref.rope_table(dims, 256, 1000.0, {"type": "linear", "factor": 2.0}) if dims else None

    def rows(n):
        return (torch.randn(n, ncol) * 0.7).to(dt)

    def meta(spans):
        cu, pos, tok_seq, slots = [0], [], [], []
        for s, (a, n) in spans:
            cu.append(cu[-1] + n)
            pos += range(a, a + n)
            tok_seq += [s] * n
            slots += [int(bt[s, p // bs]) * bs + p % bs for p in range(a, a + n)]
        i32 = lambda v: torch.tensor(v, dtype=torch.int32)
        return i32(cu), i32(pos), i32(tok_seq), i32(slots)

    qb, kb, vb = (torch.randn(n).to(dt) * 0.3 for n in (H * D, G * D, G * V))
    qnw, knw = ((1.0 + 0.3 * torch.randn(n)).to(dt) if qk_norm else None for n in (H * D, G * D))
    sv = torch.randn(H) * 2.0 if sinks else None
    e = nblk * sm.pool_entries_per_page(bs, P) if P else 1
    caches = {}
    for dev in ("cpu", DEV):
        kc, vc = torch.zeros(nblk * bs, G, D, dtype=dt, device=dev), torch.zeros(nblk * bs, G, V, dtype=dt, device=dev)
        kp, vp = torch.zeros(e, G, D, device=dev), torch.zeros(e, G, V, device=dev)
        caches[dev] = (kc, vc, kp, vp)
    batches = [meta([(1, (0, 41)), (2, (0, 77))]), meta([(1, (41, 29)), (2, (77, 53))]),
               meta([(s, l) for s, l in enumerate(lens)])]
    outs = {}
    for dev in ("cpu", DEV):
        kc, vc, kp, vp = caches[dev]
        mv = lambda t: None if t is None else t.to(dev)
        torch.manual_seed(seed + 1)
        for cu, pos, tok_seq, slots in batches:
            x = rows(pos.shape[0]).to(dev)
            vfirst = (torch.randn(pos.shape[0], G * V)).to(dev)
            sm.window_kv_write(kc, vc, x, H * D, H * D + G * D, mv(qb), mv(kb), mv(vb), mv(cs), pos.to(dev), slots.to(dev),
                               H, G, D, V, dims, 1e-6, unit, vfirst_in=vfirst, lam=0.3, half_layout=half, qnw=mv(qnw),
                               knw=mv(knw))
            sm.window_pool(kp, vp, kc, vc, bt.to(dev), tok_seq.to(dev), pos.to(dev), P, bs)
        goff = H * D + G * D + G * V
        gate = x[:, goff:goff + H] if per_head else x[:, goff:]
        outs[dev] = (x, sm.window_attention(x, gate, kc, vc, kp if P else None, vp if P else None, bt.to(dev),
                                            tok_seq.to(dev), pos.to(dev), H, window, P, 0.35, True, bs, cu.to(dev),
                                            max(n for _, n in lens), chunk=chunk, softcap=softcap, sinks=mv(sv),
                                            gate_per_head=per_head))
    return outs, caches


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,G,D,V,window,P,dims", [
    (4, 2, 24, 20, 33, 5, 8),        # odd sizes: the plain kernel in both types
    (6, 2, 16, 16, 20, 16, 16),      # three query heads per key head: no matrix-core tiling
    (12, 3, 64, 64, 40, 10, 24),     # matrix cores in bf16: four query heads per key head
    (4, 4, 128, 128, 64, 7, 64),     # one query head per key head, 128-wide heads
    (16, 1, 32, 48, 17, 3, 0),       # sixteen query heads on one key head, no rotation
    (8, 4, 72, 80, 0, 0, 8),         # no window
    (2, 1, 40, 32, 25, 0, 4),        # a window without pooled blocks
])
def test_window_attention_ops(dt, tol, H, G, D, V, window, P, dims):
    outs, caches = window_case(H, G, D, V, window, P, dims, dt)
    for a, b in zip(caches[DEV], caches["cpu"]):
        close(a, b, tol)
    close(outs[DEV][0][:, :H * D], outs["cpu"][0][:, :H * D], tol)       # prepared queries
    close(outs[DEV][1], outs["cpu"][1], tol * 2)


def test_window_attention_matrix_cores_match_plain_kernel():
    """The same caches through both kernels in bf16 (the plain one is also the fp32 path)."""
    outs, _ = window_case(12, 3, 64, 64, 40, 10, 24, torch.bfloat16, seed=3)
    old = sm.WINDOW_MFMA
    try:
        sm.WINDOW_MFMA = False
        plain, _ = window_case(12, 3, 64, 64, 40, 10, 24, torch.bfloat16, seed=3)
    finally:
        sm.WINDOW_MFMA = old
    close(outs[DEV][1], plain[DEV][1], 2e-2)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,G,D,V,chunk,dims,kw", [
    (4, 2, 24, 20, 33, 8, dict(softcap=1.5, per_head=True, half=True, unit=False)),       # plain kernel, odd sizes
    (12, 3, 64, 64, 40, 24, dict(sinks=True, half=True, qk_norm=True, unit=False)),       # matrix cores in bf16
    (8, 2, 32, 48, 16, 32, dict(softcap=0.8, sinks=True, per_head=True, half=True)),      # chunk = page, full rotation
    (4, 4, 128, 128, 1, 64, dict(half=True, qk_norm=True)),                                # chunks of one token
    (6, 2, 16, 16, 1000, 0, dict(per_head=True, sinks=True)),                              # one chunk holds everything
])
def test_chunked_attention_variants(dt, tol, H, G, D, V, chunk, dims, kw):
    """The chunked mask, capped scores, learned sinks, per-head gates, the half rotation layout and whole-projection
    norms against the reference op, over shuffled pages."""
    outs, caches = window_case(H, G, D, V, 0, 0, dims, dt, chunk=chunk, **kw)
    for a, b in zip(caches[DEV][:2], caches["cpu"][:2]):
        close(a, b, tol)
    close(outs[DEV][0][:, :H * D], outs["cpu"][0][:, :H * D], tol)
    close(outs[DEV][1], outs["cpu"][1], tol * 2)


@pytest.mark.parametrize("dt,tol", DTYPES)
def test_queries_only_preparation(dt, tol):
    """A layer that attends another layer's cache prepares its queries and writes no keys or values."""
    torch.manual_seed(5)
    H, D, dims = 3, 20, 12
    x = torch.randn(T, H * D + 5).to(dt)
    pos = torch.arange(T, dtype=torch.int32)
    pos[4] = -1
    cs = ref.rope_table(dims, 64, 500.0)
    qnw = (1.0 + 0.2 * torch.randn(H * D)).to(dt)
    xc, xg = x.clone(), x.to(DEV).clone()
    slots = torch.arange(T, dtype=torch.int32)
    sm.window_kv_write(None, None, xc, 0, 0, None, None, None, cs, pos, slots, H, 0, D, D, dims, 1e-5, False,
                       half_layout=True, qnw=qnw)
    sm.window_kv_write(None, None, xg, 0, 0, None, None, None, cs.to(DEV), pos.to(DEV), slots.to(DEV), H, 0, D, D, dims,
                       1e-5, False, half_layout=True, qnw=qnw.to(DEV))
    close(xg, xc, tol)
    assert torch.equal(xc[4], x[4]) and torch.equal(xg[4].cpu(), x[4])


@pytest.mark.parametrize("dt,tol", DTYPES)
def test_parallel_block_ops(dt, tol):
    """Two branches in one residual add, the joined norms of two mixers, the relu gate and the soft cap."""
    torch.manual_seed(6)
    W = 200
    x, b1, b2, w = torch.randn(T, W), torch.randn(T, W).to(dt), torch.randn(T, W).to(dt), torch.randn(W).to(dt)
    xg, xc = x.to(DEV).clone(), x.clone()
    og = sm.resnorm(xg, w.to(DEV), 1e-5, branch=b1.to(DEV), branch2=b2.to(DEV), out_dtype=dt)
    oc = sm.resnorm(xc, w, 1e-5, branch=b1, branch2=b2, out_dtype=dt)
    close(og, oc, tol)
    close(xg, xc, 1e-6)
    wa, wb = torch.randn(W).to(dt), torch.randn(W).to(dt)
    for out in (dt, torch.float32):
        close(sm.norm_mix(b1.to(DEV), wa.to(DEV), b2.to(DEV), wb.to(DEV), 1e-5, 0.5, 0.25, out),
              sm.norm_mix(b1, wa, b2, wb, 1e-5, 0.5, 0.25, out), tol)
    close(sm.norm_mix(b1.to(DEV), wa.to(DEV), None, None, 1e-5, 2.0), sm.norm_mix(b1, wa, None, None, 1e-5, 2.0), tol)
    a = torch.randn(T, 140).to(dt) * 2
    close(sm.act(a.to(DEV), sm.ACT_RELU), sm.act(a, sm.ACT_RELU), tol)
    z = torch.randn(T, 77) * 20
    close(sm.act(z.to(DEV), sm.ACT_SOFTCAP, limit=12.0), sm.act(z, sm.ACT_SOFTCAP, limit=12.0), 2e-6)


# ----------------------------------------------------------------------------- short convolutions, delta rule, RG-LRU
def _dev(v):
    return v.to(DEV) if isinstance(v, torch.Tensor) else v


@pytest.mark.parametrize("taps,C,unit", [(4, 70, None), (3, 2 * 2 * 24 + 3 * 40, (2 * 2 * 24, 24, 2 * 24, 24 ** -0.5)),
                                         (1, 33, None), (2, 300, (256, 128, 128, 0.3)), (7, 64, (64, 64, 0, 1.0))])
def test_short_conv(taps, C, unit):
    """Convolutions over the batch of `batch()` (an empty sequence, one resumed mid-sequence), twice, so that the second
    call reads the inputs the first one saved -- also for portions shorter than the taps."""
    torch.manual_seed(40)
    cu, pos, slots, tok_seq = batch()
    w, ib, ob = torch.randn(C, taps), torch.randn(C), torch.randn(C)
    kw = dict(in_bias=ib, out_bias=ob, act=sm.CONV_SILU if unit else sm.CONV_NONE)
    if unit:
        kw.update(unit_cols=unit[0], unit_dim=unit[1], scale_cols=unit[2], scale=unit[3])
    state = torch.randn(4, max(taps - 1, 0), C)
    sc, sg = state.clone(), state.to(DEV).clone()
    x = torch.randn(T, C + 9)[:, 4:4 + C]                 # a view with a row stride
    for step in range(2):
        oc = sm.short_conv(x, w, sc, cu, tok_seq, slots, pos, **kw)
        og = sm.short_conv(x.to(DEV), w.to(DEV), sg, cu.to(DEV), tok_seq.to(DEV), slots.to(DEV), pos.to(DEV),
                           **{k: _dev(v) for k, v in kw.items()})
        close(og, oc, 2e-5)
        close(sg, sc, 1e-6)
        # next: every sequence goes on by one or two tokens (shorter than the taps)
        cu = torch.tensor([0, 2, 3, 3, 4], dtype=torch.int32)
        pos = torch.tensor([9, 10, 6, 30], dtype=torch.int32)
        tok_seq = torch.tensor([0, 0, 1, 3], dtype=torch.int32)
        x = torch.randn(4, C)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,G,D,V", [(3, 3, 20, 28), (4, 2, 64, 128), (2, 1, 100, 5), (2, 2, 128, 256), (1, 1, 256, 64),
                                     (6, 2, 160, 192), (8, 2, 16, 16)])
def test_delta_scan(dt, tol, H, G, D, V):
    torch.manual_seed(41)
    cu, pos, slots, _ = batch()
    q = torch.nn.functional.normalize(torch.randn(T, G, D), dim=-1) * D ** -0.5
    k = torch.nn.functional.normalize(torch.randn(T, G, D), dim=-1)
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), torch.randn(T, H * V)], 1).contiguous()
    cols = {"b": 2, "a": 2 + H + 1, "g": 2 + 2 * H + 3}
    proj = torch.randn(T, cols["g"] + H * V + 2) * 1.5
    neg_a, dtb, normw = -torch.exp(torch.randn(H) * 0.5), torch.randn(H), 1.0 + 0.2 * torch.randn(V)
    state = torch.randn(4, H, D * V) * 0.5
    sc, sg = state.clone(), state.to(DEV).clone()
    oc = sm.delta_scan(qkv, proj, cols, neg_a, dtb, normw, sc, cu, slots, pos, H, G, D, V, 1e-6, dt)
    og = sm.delta_scan(qkv.to(DEV), proj.to(DEV), cols, neg_a.to(DEV), dtb.to(DEV), normw.to(DEV), sg, cu.to(DEV),
                       slots.to(DEV), pos.to(DEV), H, G, D, V, 1e-6, dt)
    close(og, oc, tol)
    close(sg, sc, 1e-4)
    assert torch.equal(sg[1].cpu(), state[1])            # the empty sequence's slot
    for chunk in (4, 7, 16, 64):                         # three passes over chunks: same outputs, same final states
        s2 = state.to(DEV).clone()
        o2 = sm.delta_scan(qkv.to(DEV), proj.to(DEV), cols, neg_a.to(DEV), dtb.to(DEV), normw.to(DEV), s2, cu.to(DEV),
                           slots.to(DEV), pos.to(DEV), H, G, D, V, 1e-6, dt, chunk=chunk)
        close(o2, oc, tol)
        close(s2, sc, 1e-4)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("C,blocks,n", [(70, 2, 37), (64, 1, 37), (300, 10, 37), (130, 5, 700)])
def test_rglru_scan(dt, tol, C, blocks, n):
    """Short portions (one pass) and a long one (time slices joined exactly), with final states."""
    torch.manual_seed(42)
    if n == T:
        cu, pos, slots, _ = batch()
    else:
        cu = torch.tensor([0, n - 40, n - 39, n], dtype=torch.int32)
        pos = torch.cat([torch.arange(0, n - 40), torch.tensor([17]), torch.arange(5, 44)]).int()
        slots = torch.tensor([2, 0, 3], dtype=torch.int32)
    u, gates = torch.randn(n, C), torch.randn(n, blocks, 2 * C // blocks) * 2
    gb, rate = torch.randn(blocks, 2 * C // blocks), -8.0 * torch.nn.functional.softplus(torch.randn(C))
    proj, yb = torch.randn(n, C + 7) * 1.5, torch.randn(C)
    state = torch.randn(4, C)
    sc, sg = state.clone(), state.to(DEV).clone()
    mq = int((cu[1:] - cu[:-1]).max())
    oc = sm.rglru_scan(u, gates, gb, rate, proj, 3, yb, sc, cu, slots, pos, blocks, dt, mq)
    og = sm.rglru_scan(u.to(DEV), gates.to(DEV), gb.to(DEV), rate.to(DEV), proj.to(DEV), 3, yb.to(DEV), sg, cu.to(DEV),
                       slots.to(DEV), pos.to(DEV), blocks, dt, mq)
    close(og, oc, tol)
    close(sg, sc, 2e-5)


# ----------------------------------------------------------------------------- gated matrix-state recurrences
@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("kind,H,D,V", [(sm.SCAN_HGRN2, 3, 20, 28), (sm.SCAN_HGRN2, 2, 64, 128), (sm.SCAN_HGRN2, 1, 100, 5),
                                        (sm.SCAN_MLSTM, 3, 20, 28), (sm.SCAN_MLSTM, 2, 128, 64), (sm.SCAN_MLSTM, 5, 7, 70),
                                        (sm.SCAN_HGRN2, 2, 128, 256), (sm.SCAN_MLSTM, 1, 256, 64), (sm.SCAN_MLSTM, 2, 160, 192),
                                        (sm.SCAN_HGRN2, 1, 200, 136)])
def test_gated_scan(dt, tol, kind, H, D, V):
    torch.manual_seed(30)
    cu, pos, slots, _ = batch()
    if kind == sm.SCAN_HGRN2:
        parts = (("q", H * D), ("f", H * D), ("v", H * V))
    else:
        parts = (("q", H * D), ("k", H * D), ("v", H * V), ("i", H), ("f", H), ("g", H * V))
    cols, at = {}, 3                                   # parts need not start the row
    for key, n in parts:
        cols[key] = at
        at += n + 1
    proj = torch.randn(T, at) * 1.5
    nf = H * D if kind == sm.SCAN_HGRN2 else H
    fb, ib = torch.randn(nf).to(dt), torch.randn(H).to(dt)
    lower = torch.rand(H * D).to(dt)
    normw = torch.randn(V if kind == sm.SCAN_HGRN2 else H * V).to(dt)
    state = torch.randn(4, H, sm.gated_scan_record(kind, D, V)) * 0.5
    kw = dict(fbias=fb, ibias=ib if kind == sm.SCAN_MLSTM else None, lower=lower if kind == sm.SCAN_HGRN2 else None,
              cap=6.0)
    sc, sg = state.clone(), state.to(DEV).clone()
    oc = sm.gated_scan(proj, kind, cols, normw, sc, cu, slots, pos, H, D, V, 1e-6, dt, **kw)
    og = sm.gated_scan(proj.to(DEV), kind, cols, normw.to(DEV), sg, cu.to(DEV), slots.to(DEV), pos.to(DEV), H, D, V,
                       1e-6, dt, **{k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()})
    close(og, oc, tol)
    close(sg, sc, 1e-4)
    assert torch.equal(sg[3].cpu(), state[3]) is False and torch.equal(sg[1].cpu(), state[1])    # the empty sequence's slot
    for chunk in (4, 7, 16, 64):                       # three passes over chunks: same outputs, same final states
        s2 = state.to(DEV).clone()
        o2 = sm.gated_scan(proj.to(DEV), kind, cols, normw.to(DEV), s2, cu.to(DEV), slots.to(DEV), pos.to(DEV), H, D, V,
                           1e-6, dt, chunk=chunk, **{k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()})
        close(o2, oc, tol)
        close(s2, sc, 1e-4)


# ----------------------------------------------------------------------------- norms after the sum, gates, grouped norms
@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("W", [200, 64, 5000])
def test_postnorm_and_gates(dt, tol, W):
    torch.manual_seed(50)
    x, b1, b2 = torch.randn(T, W) * 2, torch.randn(T, W).to(dt), torch.randn(T, W).to(dt)
    for kw in (dict(), dict(branch2=b2, c1=1.2, c2=-0.4)):
        xg, xc = x.to(DEV).clone(), x.clone()
        og = sm.postnorm(xg, b1.to(DEV), 2.0, 0.8, 1e-6, out_dtype=dt, **{k: _dev(v) for k, v in kw.items()})
        oc = sm.postnorm(xc, b1, 2.0, 0.8, 1e-6, out_dtype=dt, **kw)
        close(og, oc, tol)
        close(xg, xc, 1e-5)
    xg, xc = x.to(DEV).clone(), x.clone()
    assert sm.postnorm(xg, None, 1.5, 1.1, 1e-6) is None and sm.postnorm(xc, None, 1.5, 1.1, 1e-6) is None
    close(xg, xc, 1e-5)
    close(sm.postnorm(xg, None, 1.0, 0.5, 1e-6, out_dtype=dt), sm.postnorm(xc, None, 1.0, 0.5, 1e-6, out_dtype=dt), tol)
    # gates on column slices of wider tensors; an fp32 input gated into the activation type
    F = min(W, 300)
    wide, y = (torch.randn(T, F + 24) * 2).to(dt), torch.randn(T, F + 8)
    for kind in (sm.GATE_SIGMOID, sm.GATE_SILU):
        for yy in (y[:, 8:], y[:, :F].to(dt)):
            close(sm.gate_mul(yy.to(DEV), wide.to(DEV)[:, 16:16 + F], kind), sm.gate_mul(yy, wide[:, 16:16 + F], kind), tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("W,groups", [(192, 1), (192, 4), (70, 7), (96, 96), (640, 2)])
def test_norm_of_a_slice_in_groups(dt, tol, W, groups):
    torch.manual_seed(51)
    wide = torch.randn(T, W + 40)
    w = 1 + 0.2 * torch.randn(W)
    for a, ww in ((wide[:, 24:24 + W], w), (wide.to(dt)[:, 24:24 + W], w.to(dt))):
        og = sm.norm_mix(a.to(DEV), ww.to(DEV), None, None, 1e-5, ca=0.7, out_dtype=dt, groups=groups)
        close(og, sm.norm_mix(a, ww, None, None, 1e-5, ca=0.7, out_dtype=dt, groups=groups), tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("taps,C", [(3, 70), (1, 64), (8, 300)])
def test_short_conv_with_residual(dt, tol, taps, C):
    """x + conv(x) in the activation type, twice, so that the second call reads the inputs the first one saved."""
    torch.manual_seed(52)
    cu, pos, slots, tok_seq = batch()
    w = torch.randn(C, taps)
    state = torch.randn(4, max(taps - 1, 0), C)
    sc, sg = state.clone(), state.to(DEV).clone()
    x = torch.randn(T, C)
    for step in range(2):
        oc = sm.short_conv(x, w, sc, cu, tok_seq, slots, pos, residual=True, out_dtype=dt)
        og = sm.short_conv(x.to(DEV), w.to(DEV), sg, cu.to(DEV), tok_seq.to(DEV), slots.to(DEV), pos.to(DEV),
                           residual=True, out_dtype=dt)
        assert og.dtype == dt
        close(og, oc, tol)
        close(sg, sc, 1e-6)
        cu = torch.tensor([0, 2, 3, 3, 4], dtype=torch.int32)
        pos = torch.tensor([9, 10, 6, 30], dtype=torch.int32)
        tok_seq = torch.tensor([0, 0, 1, 3], dtype=torch.int32)
        x = torch.randn(4, C)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,Dn,R,C,dims", [(6, 40, 24, 72, 24), (3, 16, 8, 130, 4), (20, 16, 8, 48, 8), (16, 32, 16, 64, 16),
                                           (1, 2, 2, 1, 2), (4, 16, 64, 256, 64), (18, 16, 64, 128, 32), (4, 24, 32, 128, 32),
                                           (5, 16, 32, 64, 32), (16, 64, 64, 512, 64)])
def test_latent_attention_interleaved_pairs_and_sinks(dt, tol, H, Dn, R, C, dims):
    """The latent row as a slice of a wider projection, the rotation of the pairs (2i, 2i + 1), and a learned term per
    head in the softmax's denominator: per token, four tokens per workgroup, and few tokens with key splits."""
    torch.manual_seed(53)
    cu, pos, slots, tok_seq = batch()
    bs, per = 16, 2
    L = C + R
    cache = torch.randn(4 * per * bs, L).to(dt)
    bt = torch.randperm(4 * per).view(4, per).int()
    slot_map = torch.tensor([int(bt[tok_seq[t], pos[t] // bs]) * bs + int(pos[t]) % bs for t in range(T)],
                            dtype=torch.int32)
    wide, nw = torch.randn(T, L + 48).to(dt), (1 + 0.1 * torch.randn(C)).to(dt)
    q = torch.randn(T, H * (Dn + R)).to(dt)
    cs = ref.rope_table(dims, 64, 10000.0)
    cg, qg, cc, qc = cache.to(DEV).clone(), q.to(DEV).clone(), cache.clone(), q.clone()
    sm.latent_kv_write(cg, wide.to(DEV)[:, 32:32 + L], nw.to(DEV), qg, cs.to(DEV), pos.to(DEV), slot_map.to(DEV), C, R, H,
                       Dn, dims, 1e-6, interleaved=True)
    sm.latent_kv_write(cc, wide[:, 32:32 + L], nw, qc, cs, pos, slot_map, C, R, H, Dn, dims, 1e-6, interleaved=True)
    close(cg, cc, tol)
    close(qg, qc, tol)
    half = q.clone()
    sm.latent_kv_write(cache.clone(), wide[:, 32:32 + L], nw, half, cs, pos, slot_map, C, R, H, Dn, dims, 1e-6)
    assert dims == 2 or not torch.allclose(half.float(), qc.float(), atol=1e-2)   # the pair layout matters
    qabs = torch.randn(T, H, C).to(dt) * 0.3
    sinks = torch.randn(H) * 2
    sinks[0] = 9.0                                                            # above every score
    oc = sm.latent_attention(qabs, qc, cc, bt, tok_seq, pos, C, R, H, Dn, 0, 0.2, bs, sinks=sinks)
    assert not torch.allclose(oc.float(), sm.latent_attention(qabs, qc, cc, bt, tok_seq, pos, C, R, H, Dn, 0, 0.2, bs).float(),
                              atol=1e-2)
    for kw in ({}, {"cu_q": cu.to(DEV), "max_qlen": 27}):
        og = sm.latent_attention(qabs.to(DEV), qc.to(DEV), cc.to(DEV), bt.to(DEV), tok_seq.to(DEV), pos.to(DEV), C, R, H,
                                 Dn, 0, 0.2, bs, sinks=sinks.to(DEV), **kw)
        close(og, oc, tol)
    few = torch.tensor([3, 20, 30], dtype=torch.long)                         # few tokens: key splits and their merge
    og = sm.latent_attention(qabs[few].to(DEV), qc[few].to(DEV), cc.to(DEV), bt.to(DEV), tok_seq[few].to(DEV),
                             pos[few].to(DEV), C, R, H, Dn, 0, 0.2, bs, 64, sinks=sinks.to(DEV))
    close(og, oc[few], tol)


@pytest.mark.parametrize("dt,tol", DTYPES)
@pytest.mark.parametrize("H,G,D,V", [(8, 4, 32, 128), (3, 1, 20, 12), (6, 3, 80, 72), (16, 4, 128, 64)])
def test_per_head_normed_queries_and_keys(dt, tol, H, G, D, V):
    torch.manual_seed(54)
    cu, pos, slots, tok_seq = batch()
    bs = 16
    n = 8 * bs
    koff, voff = H * D + 16, H * D + 16 + G * D
    proj = torch.randn(T, voff + G * V + 5).to(dt)
    slot_map = torch.randperm(n)[:T].int()
    qw, kw_ = (1 + 0.3 * torch.randn(D)).to(dt), (1 + 0.3 * torch.randn(D)).to(dt)
    out = {}
    for dev in ("cpu", DEV):
        kc, vc = torch.zeros(n, G, D, dtype=dt, device=dev), torch.zeros(n, G, V, dtype=dt, device=dev)
        p = proj.to(dev).clone()
        sm.window_kv_write(kc, vc, p, koff, voff, None, None, None, None, pos.to(dev), slot_map.to(dev), H, G, D, V, 0,
                           1e-6, False, head_qnw=qw.to(dev), head_knw=kw_.to(dev))
        out[dev] = (kc, vc, p)
    for a, b in zip(out[DEV], out["cpu"]):
        close(a, b, tol)
    q = out["cpu"][2][:, :H * D].float().view(T, H, D)
    ratio = q.pow(2).mean(-1).sqrt() / (qw.float().pow(2).mean().sqrt())
    assert (ratio - 1).abs().max() < 0.35                                     # every head normed by itself


# ----------------------------------------------------------------------------- state-space recurrence
@pytest.mark.parametrize("H,G,N,V", [(4, 2, 16, 24), (8, 4, 40, 56), (3, 1, 100, 5), (2, 2, 128, 64), (6, 3, 64, 128),
                                     (1, 1, 256, 200), (5, 5, 7, 70)])
def test_ssd_scan(H, G, N, V):
    torch.manual_seed(55)
    cu, pos, slots, _ = batch()
    inner = H * V
    cols = {"v": 2, "k": 2 + inner + 1, "q": 2 + inner + 1 + G * N + 3, "g": 1, "f": 1 + inner + 5}
    xbc = torch.randn(T, cols["q"] + G * N + 2)
    aux = torch.randn(T, cols["f"] + H + 3) * 1.5
    hp = torch.stack([-torch.exp(torch.randn(H) * 0.7 - 1.0), torch.randn(H), torch.randn(H)]).contiguous()
    state = torch.randn(4, H, N * V) * 0.5
    sc, sg = state.clone(), state.to(DEV).clone()
    args = lambda d, s: (xbc.to(d), sm.SCAN_SSD, cols, None, s, cu.to(d), slots.to(d), pos.to(d), H, N, V, 1e-6,
                         torch.float32)
    kw = lambda d: dict(aux=aux.to(d), head_params=hp.to(d), groups=G)
    oc = sm.gated_scan(*args("cpu", sc), **kw("cpu"))
    og = sm.gated_scan(*args(DEV, sg), **kw(DEV))
    assert og.dtype == torch.float32
    close(og, oc, 2e-5)
    close(sg, sc, 1e-4)
    assert torch.equal(sg[1].cpu(), state[1])                                  # the empty sequence's slot
    for chunk in (4, 7, 16, 64):                       # three passes over chunks: same outputs, same final states
        s2 = state.to(DEV).clone()
        o2 = sm.gated_scan(*args(DEV, s2), chunk=chunk, **kw(DEV))
        close(o2, oc, 2e-5)
        close(s2, sc, 1e-4)


@pytest.mark.parametrize("width", [64, 5000, 9000])
def test_latent_attention_prompt_with_long_block_tables(width):
    """Block tables of many entries per sequence: staged in LDS beside the key tile while they fit, read from memory
    when they do not; the same rows either way."""
    torch.manual_seed(56)
    dt, tol = torch.bfloat16, 2e-2
    cu, pos, slots, tok_seq = batch()
    H, Dn, R, C, bs, per = 4, 16, 64, 512, 16, 2
    cache = torch.randn(4 * per * bs, C + R).to(dt)
    bt = torch.zeros(4, width, dtype=torch.int32)
    bt[:, :per] = torch.randperm(4 * per).view(4, per).int()
    q = torch.randn(T, H * (Dn + R)).to(dt)
    qabs = (torch.randn(T, H, C) * 0.3).to(dt)
    oc = sm.latent_attention(qabs, q, cache, bt[:, :per].contiguous(), tok_seq, pos, C, R, H, Dn, 0, 0.2, bs)
    og = sm.latent_attention(qabs.to(DEV), q.to(DEV), cache.to(DEV), bt.to(DEV), tok_seq.to(DEV), pos.to(DEV), C, R, H, Dn,
                             0, 0.2, bs, cu_q=cu.to(DEV), max_qlen=27)
    close(og, oc, tol)
