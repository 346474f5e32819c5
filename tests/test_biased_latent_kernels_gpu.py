"""HIP kernels behind the Tarunex mixers and feed-forward against the PyTorch rendering of the
same ops (CPU tensors), in fp32 and bf16: the residual pass with two normed outputs, rotation
of channel stretches, the unrotated attention input pass, score cap / distance penalty / head
gates in both window attention kernels, latent attention without a sink and with a rotated
key part in the cached row, the router with a bias and a softmax over the chosen logits, and
the silu epilogue of the grouped expert product."""
import pytest
import torch

from p2p_llm_chat_go_amd.ops import seqmix as sm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-4, atol=2e-5)


def _d(*ts):
    return [None if t is None else t.to(DEV) for t in ts]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wide", [200, 4100])   # rows kept in registers / rows read twice
def test_embed_scale_add_norm2(dt, wide):
    g = torch.Generator().manual_seed(0)
    V, W, R = 50, wide, 23
    emb = torch.randn(V, W, generator=g).to(dt)
    ids = torch.randint(0, V, (R,), generator=g, dtype=torch.int32)
    x1 = sm.embed_rows(emb, ids, torch.empty(R, W), scale=3.5)
    x2 = sm.embed_rows(emb.to(DEV), ids.to(DEV), torch.empty(R, W, device=DEV), scale=3.5)
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-6, atol=1e-6)
    a, b = (torch.randn(R, W + 8, generator=g).to(dt)[:, 8:] for _ in range(2))
    rows, vec = torch.randn(R, W, generator=g), torch.randn(W, generator=g)
    one, two, per = torch.tensor([1.25]), torch.tensor([0.75]), 1 + 0.1 * torch.randn(W, generator=g)
    top = 3
    ry, rw = torch.randn(R * top + 2, W, generator=g).to(dt), torch.rand(R, top, generator=g)
    cases = [dict(a=a), dict(a=a, b=b), dict(rows=rows, vec=vec), dict(a=a, b=b, rows=rows, vec=vec), dict(vec=vec), {},
             dict(a=a, routed=(ry, rw)), dict(routed=(ry, rw), rows=rows)]
    for kw in cases:
        for w1, w2 in ((None, None), (one, None), (one, two), (per, two), (per, per)):
            outs = []
            for dev in ("cpu", DEV):
                x = x1.clone().to(dev)
                h1 = torch.zeros(R, W, dtype=dt, device=dev) if w1 is not None else None
                h2 = torch.zeros(R, W, dtype=dt, device=dev) if w2 is not None else None
                args = {k: tuple(t.to(dev) for t in v) if isinstance(v, tuple) else v.to(dev) for k, v in kw.items()}
                sm.add_norm2(x, eps=1e-5, w1=None if w1 is None else w1.to(dev), out1=h1,
                             w2=None if w2 is None else w2.to(dev), out2=h2, **args)
                outs.append((x.cpu(), h1, h2))
            torch.testing.assert_close(outs[1][0], outs[0][0], rtol=1e-5, atol=1e-5)
            for k in (1, 2):
                if outs[0][k] is not None:
                    torch.testing.assert_close(outs[1][k].cpu().float(), outs[0][k].float(), **_tol(dt))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_rope_rows_qtemp_gate_softcap(dt):
    g = torch.Generator().manual_seed(1)
    R, H, hs, nrot = 19, 5, 22, 3
    src = torch.randn(R, H * hs + 4, generator=g).to(dt)
    pos = torch.randint(0, 3000, (R,), generator=g, dtype=torch.int32)
    inv = sm.rope_inv_freq(700.0, 2 * nrot, "cpu")
    # heads of a row, rotated stretch at channel 10 of each head, into a [H, R, n] buffer's tail
    q1, q2 = torch.zeros(H, R, 30, dtype=dt), torch.zeros(H, R, 30, dtype=dt, device=DEV)
    sm.rope_rows(src[:, 10:], H, hs, inv, pos, q1[0, :, 24:], q1.stride(0))
    sm.rope_rows(src.to(DEV)[:, 10:], H, hs, inv.to(DEV), pos.to(DEV), q2[0, :, 24:], q2.stride(0))
    torch.testing.assert_close(q2.cpu().float(), q1.float(), **_tol(dt))
    assert float(q1[:, :, :24].abs().max()) == 0.0 and float(q2[:, :, :24].abs().max()) == 0.0
    # one shared stretch scattered into pool rows
    rows = torch.randperm(40, generator=g)[:R].to(torch.int32)
    p1, p2 = torch.zeros(40, 16, dtype=dt), torch.zeros(40, 16, dtype=dt, device=DEV)
    sm.rope_rows(src[:, 3:3 + 2 * nrot], 1, 0, inv, pos, p1[:, 10:], 0, out_rows=rows)
    sm.rope_rows(src.to(DEV)[:, 3:3 + 2 * nrot], 1, 0, inv.to(DEV), pos.to(DEV), p2[:, 10:], 0,
                 out_rows=rows.to(DEV))
    torch.testing.assert_close(p2.cpu().float(), p1.float(), **_tol(dt))
    # query temperature + key/value store
    nq, nkv = 35, 27
    proj = torch.randn(R, nq + nkv + 6, generator=g).to(dt)
    pos2 = torch.tensor([0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 14, 15, 16, 63, 64, 1000, 4095], dtype=torch.int32)
    for coef, every in ((0.7, 4), (0.0, 1), (2.0, 1), (0.25, 32)):
        qa, qb = torch.empty(R, nq, dtype=dt), torch.empty(R, nq, dtype=dt, device=DEV)
        pa, pb = torch.zeros(40, nkv, dtype=dt), torch.zeros(40, nkv, dtype=dt, device=DEV)
        sm.qtemp_kv_store(proj, nq, nkv, coef, every, pos2, rows, pa, qa)
        sm.qtemp_kv_store(proj.to(DEV), nq, nkv, coef, every, pos2.to(DEV), rows.to(DEV), pb, qb)
        torch.testing.assert_close(qb.cpu().float(), qa.float(), **_tol(dt))
        torch.testing.assert_close(pb.cpu().float(), pa.float(), rtol=0, atol=0)
    # both latents normed, the key part rotated (two of its channels pass unchanged), in one pass
    nq, nc, nr = 37, 70, 2 * nrot + 2
    proj = torch.randn(R, nq + nc + nr + 3, generator=g).to(dt)
    qw, cw = 1 + 0.1 * torch.randn(nq, generator=g), 1 + 0.1 * torch.randn(nc, generator=g)
    ca, cb = torch.empty(R, nq, dtype=dt), torch.empty(R, nq, dtype=dt, device=DEV)
    pa, pb = torch.zeros(40, nc + nr, dtype=dt), torch.zeros(40, nc + nr, dtype=dt, device=DEV)
    sm.latent_prep(proj, nq, nc, nr, qw, cw, inv, pos, rows, pa, 1e-5, ca)
    sm.latent_prep(proj.to(DEV), nq, nc, nr, *_d(qw, cw, inv, pos, rows), pb, 1e-5, cb)
    torch.testing.assert_close(cb.cpu().float(), ca.float(), **_tol(dt))
    torch.testing.assert_close(pb.cpu().float(), pa.float(), **_tol(dt))
    ref = sm.rmsnorm(proj[:, nq:nq + nc], cw, 1e-5, torch.empty(R, nc, dtype=dt))
    torch.testing.assert_close(pa[rows.long(), :nc].float(), ref.float(), **_tol(dt))
    kr = sm.rope_rows(proj[:, nq + nc:], 1, 0, inv, pos, torch.zeros(R, nr, dtype=dt), 0)
    torch.testing.assert_close(pa[rows.long(), nc:nc + 2 * nrot].float(), kr[:, :2 * nrot].float(), **_tol(dt))
    assert (pa[rows.long(), nc + 2 * nrot:] == proj[:, nq + nc + 2 * nrot:nq + nc + nr]).all()
    # one gate per head
    Vd = 20
    o, gt = torch.randn(H, R, Vd, generator=g).to(dt), torch.randn(R, H + 3, generator=g).to(dt)
    a = sm.sigmoid_gate(o, gt, torch.empty(R, H * Vd, dtype=dt), H, Vd, per_head=True)
    b = sm.sigmoid_gate(o.to(DEV), gt.to(DEV), torch.empty(R, H * Vd, dtype=dt, device=DEV), H, Vd, per_head=True)
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    # scaled and capped logits
    y = (torch.randn(R, 333, generator=g) * 40).to(dt)
    for cap, scale in ((25.0, 0.25), (0.0, 0.5), (30.0, 1.0)):
        a = sm.softcap(y, cap, torch.empty(R, 333), scale=scale)
        b = sm.softcap(y.to(DEV), cap, torch.empty(R, 333, device=DEV), scale=scale)
        torch.testing.assert_close(b.cpu(), a, rtol=1e-5, atol=1e-5)


def _step(lens, starts, bt):
    ent, r0 = [], 0
    for i, (n, s) in enumerate(zip(lens, starts)):
        ent.append((r0, n, s, i))
        r0 += n
    row_ent = torch.tensor([i for i, e in enumerate(ent) for _ in range(e[1])], dtype=torch.int32)
    pos = torch.tensor([s + i for n, s in zip(lens, starts) for i in range(n)], dtype=torch.int32)
    return ent, row_ent, pos, r0


ATTN_SHAPES = [
    # H, G, D, V
    (6, 2, 24, 40),      # three heads per key/value head
    (4, 4, 16, 8),       # one head per key/value head
    (16, 2, 80, 112),    # eight heads per key/value head
    (34, 2, 8, 16),      # more heads per key/value head than a wavefront's pairs
    (3, 1, 7, 5),        # sizes off the matrix cores' grid
]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V", ATTN_SHAPES)
@pytest.mark.parametrize("extras", ["all", "cap", "penalty", "gate"])
def test_window_attention_extras(dt, H, G, D, V, extras):
    g = torch.Generator().manual_seed(2)
    lens, starts = [70, 9, 1], [0, 150, 131]
    bt = torch.tensor([[3, 5, 0], [7, 2, 9], [1, 4, 8]], dtype=torch.int32)
    ent, row_ent, pos, R = _step(lens, starts, bt)
    pool = torch.randn(12 * PAGE, G * (D + V), generator=g).to(dt)
    q = torch.randn(R, H * D, generator=g).to(dt)
    sink = torch.zeros(H)
    cap = 1.5 if extras in ("all", "cap") else 0.0
    dist = (torch.rand(H, generator=g) * 2, torch.rand(H, generator=g) * 0.5) if extras in ("all", "penalty") else None
    gate = torch.randn(R, H + 5, generator=g).to(dt)[:, 2:] if extras in ("all", "gate") else None
    o1 = torch.empty(R, H * V, dtype=dt)
    sm.window_attn(q, pool, bt, row_ent, pos, sink, 0.5, 1 << 30, o1, PAGE, H, G, D, V, softcap=cap, dist=dist,
                   gate=gate)
    plain = torch.empty(R, H * V, dtype=dt)
    sm.window_attn(q, pool, bt, row_ent, pos, sink, 0.5, 1 << 30, plain, PAGE, H, G, D, V)
    assert (plain.float() - o1.float()).abs().max() > 1e-2      # the extras are at work
    q2, pool2 = q.to(DEV), pool.to(DEV)
    dist2 = None if dist is None else tuple(_d(*dist))
    gate2 = None if gate is None else gate.to(DEV)
    for mfma in ([False, True] if dt == torch.bfloat16 else [False]):
        for max_keys in (None, 300):    # whole windows / windows cut into runs
            units = None
            if mfma:
                if not sm.window_mfma_ok(q2, pool2, D, V):
                    assert D % 8 or V % 8
                    continue
                units = sm.make_units(ent, sm.window_rows_per_wave(H // G)).to(DEV)
            o2 = torch.empty(R, H * V, dtype=dt, device=DEV)
            sm.window_attn(q2, pool2, *_d(bt, row_ent, pos, sink), 0.5, 1 << 30, o2, PAGE, H, G, D, V,
                           units=units, max_keys=max_keys, softcap=cap, dist=dist2, gate=gate2)
            torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,rank,win", [(6, 120, 1 << 30), (3, 40, 7), (16, 512, 1 << 30), (20, 64, 64), (1, 8, 3),
                                        (4, 100, 1 << 30)])
def test_latent_attn_without_sink(dt, H, rank, win):
    g = torch.Generator().manual_seed(4)
    cache = torch.randn(12 * PAGE, rank, generator=g).to(dt)
    bt = torch.tensor([[3, 7, 1, 9], [2, 5, 0, 0], [4, 6, 0, 0]], dtype=torch.int32)
    lens, starts = [40, 1, 3], [100, 70, 0]       # the last portion holds a sequence's first tokens
    ent, row_ent, pos, R = _step(lens, starts, bt)
    qa = (torch.randn(R, H, rank, generator=g) * 0.3).to(dt).transpose(0, 1)
    a = sm.latent_attn(qa, cache, bt, row_ent, pos, None, 0.2, win, torch.empty(H, R, rank, dtype=dt), PAGE)
    b = sm.latent_attn(qa.to(DEV), cache.to(DEV), *_d(bt, row_ent, pos), None, 0.2, win,
                       torch.empty(H, R, rank, dtype=dt, device=DEV), PAGE)
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    # the first token of a sequence attends to itself alone: its latent comes back
    r_first = 41
    first = cache[int(bt[2, 0]) * PAGE].float()
    torch.testing.assert_close(a[:, r_first].float(), first.expand(H, rank), **_tol(dt))
    if dt == torch.bfloat16 and rank % 8 == 0:
        qc = qa.contiguous().to(DEV)
        assert sm.latent_mfma_ok(qc, cache.to(DEV))
        units = sm.make_units(ent, sm.latent_rows_per_wave(H)).to(DEV)
        for max_keys in (None, 140):
            c = sm.latent_attn(qc, cache.to(DEV), *_d(bt, row_ent, pos), None, 0.2, win,
                               torch.empty(H, R, rank, dtype=dt, device=DEV), PAGE, units=units, max_keys=max_keys)
            torch.testing.assert_close(c.cpu().float(), a.float(), **_tol(dt))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,top,W,Fd", [(10, 4, 72, 48), (8, 2, 64, 64), (6, 6, 50, 33), (70, 5, 96, 32), (2, 1, 40, 16)])
@pytest.mark.parametrize("R", [45, 300])     # few slots per expert / the large prompt tile
def test_router_bias_and_silu_experts(dt, E, top, W, Fd, R):
    g = torch.Generator().manual_seed(5)
    h = torch.randn(R, W, generator=g).to(dt)
    wr = torch.randn(E, W, generator=g) * 0.5
    bias = torch.randn(E, generator=g) * 2
    bias[E // 2] += 40.0
    res = []
    for dev in ("cpu", DEV):
        ids = torch.empty(R, top, dtype=torch.int32, device=dev)
        wts = torch.empty(R, top, device=dev)
        cnt = torch.empty(E, dtype=torch.int32, device=dev)
        rows = torch.full((E, R * top), -1, dtype=torch.int32, device=dev)
        sm.group_route(h.to(dev), wr.to(dev), top, 1, 1, ids, wts, cnt, rows, score="top_softmax",
                       bias=bias.to(dev))
        res.append((ids.cpu(), wts.cpu(), cnt.cpu(), rows.cpu()))
    (i1, w1, c1, r1), (i2, w2, c2, r2) = res
    z = h.float() @ wr.t() + bias
    val, idx = z.topk(top, -1)
    torch.testing.assert_close(w1, torch.softmax(val, -1), rtol=1e-5, atol=1e-6)   # the rendering itself
    assert (i1 == idx.to(torch.int32)).all()
    same = (i1 == i2).all(-1)
    assert same.float().mean() > 0.98            # a tie within rounding may fall the other way
    torch.testing.assert_close(w2[same], w1[same], rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(w2.sum(-1), torch.ones(R), rtol=1e-5, atol=1e-5)
    assert int(c2.sum()) == R * top and int(c2[E // 2]) > R // 2
    got = sorted(s_ for e in range(E) for s_ in r2[e, :int(c2[e])].tolist())
    assert got == list(range(R * top))
    if Fd % 16:
        return
    wg = (torch.randn(E, 2 * Fd, W, generator=g) / W ** 0.5).to(dt)
    wi = sm.interleave_gate_up(wg[:, :Fd], wg[:, Fd:])
    gu = sm.expert_gemm(h, top, wg, c2, r2, torch.zeros(R * top, 2 * Fd, dtype=dt), R * top)
    a0 = sm.glu_act(gu, torch.empty(R * top, Fd, dtype=dt), "silu")
    a1 = sm.expert_gemm(h, top, wi, c2, r2, torch.zeros(R * top, Fd, dtype=dt), R * top, silu_glu=True)
    a2 = sm.expert_gemm(h.to(DEV), top, wi.to(DEV), c2.to(DEV), r2.to(DEV),
                        torch.zeros(R * top, Fd, dtype=dt, device=DEV), R * top, silu_glu=True)
    torch.testing.assert_close(a1.float(), a0.float(), **_tol(dt))
    torch.testing.assert_close(a2.cpu().float(), a1.float(), **_tol(dt))
