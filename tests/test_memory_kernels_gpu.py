"""HIP kernels of the matrix-memory scan, the per-head normed / rotate-half attention inputs,
the sink-free attention, the softmax router with identity experts and the pointwise steps of
ops.seqmix against the PyTorch rendering of the same ops (CPU tensors), in fp32 and bf16, at
sizes that are not multiples of the kernels' tiles, with several entries per step and state
carried over a second step."""
import pytest
import torch

from p2p_llm_chat_go_amd.ops import seqmix as sm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def _ents(lens, starts, slots):
    ent, r0 = [], 0
    for n, s, sl in zip(lens, starts, slots):
        ent.append((r0, n, s, sl))
        r0 += n
    row_ent = [i for i, e in enumerate(ent) for _ in range(e[1])]
    return ent, torch.tensor(ent, dtype=torch.int32), torch.tensor(row_ent, dtype=torch.int32), r0


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-4, atol=2e-5)


def _d(*ts):
    return [t.to(DEV) for t in ts]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,V", [(3, 20, 12), (4, 56, 24), (2, 40, 72), (1, 130, 200), (6, 8, 15), (1, 1, 1),
                                   (2, 32, 32), (1, 256, 256)])
@pytest.mark.parametrize("lens", [[37, 1, 5], [200, 3, 131]], ids=["short", "chunked"])
@pytest.mark.parametrize("cap", [20.0, 0.7])
def test_mlstm_scan(dt, H, D, V, lens, cap):
    g = torch.Generator().manual_seed(3)
    nq, nv = H * D, H * V
    bi, bf = torch.randn(H, generator=g), torch.randn(H, generator=g) + 2.0
    normw = 1 + 0.1 * torch.randn(nv, generator=g)
    S1 = torch.randn(5, H, D, V + 1, generator=g)
    m1 = torch.randn(5, H, generator=g)
    S2, m2 = S1.to(DEV), m1.to(DEV)
    for starts in ([0, 7, 0], [lens[0], 8, lens[2]]):      # second step continues the first one's slots
        ent, ent_t, _re, R = _ents(lens, starts, [2, 0, 3])
        proj = torch.randn(R, 2 * nq + 2 * nv + 2 * H + 3, generator=g).to(dt)
        proj[:, 2 * nq + 2 * nv:2 * nq + 2 * nv + 2 * H] *= 3.0     # gates well spread
        o1, o2 = torch.empty(R, nv, dtype=dt), torch.empty(R, nv, dtype=dt, device=DEV)
        sm.mlstm_scan(proj, bi, bf, cap, normw, S1, m1, ent_t, ent, o1, H, D, V, 1e-5, out_scale=1.3)
        sm.mlstm_scan(proj.to(DEV), *_d(bi, bf), cap, normw.to(DEV), S2, m2, ent_t.to(DEV), ent, o2,
                      H, D, V, 1e-5, out_scale=1.3)
        tol = _tol(dt)
        tol["atol"] *= max(1, D // 64)     # sums over the key index in another order
        torch.testing.assert_close(o2.cpu().float(), o1.float(), **tol)
        torch.testing.assert_close(S2.cpu(), S1, rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(m2.cpu(), m1, rtol=1e-5, atol=1e-5)


ATTN_SHAPES = [
    # H, G, D, V, rotated channels
    (6, 2, 24, 40, 16),      # three heads per key/value head, part of the head rotated
    (4, 4, 16, 8, 16),       # one head per key/value head, everything rotated
    (5, 1, 40, 72, 0),       # no rotation
    (16, 2, 80, 112, 80),    # eight heads per key/value head
    (3, 1, 7, 5, 4),         # odd sizes
    (40, 1, 8, 112, 8),      # a group whose heads x values exceed one block of the fp32 kernel
]


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,rot", ATTN_SHAPES)
def test_head_norm_half_rotation_plain_softmax(dt, H, G, D, V, rot):
    g = torch.Generator().manual_seed(2)
    lens, starts = [70, 9, 1], [0, 150, 131]
    ent, ent_t, row_ent, R = _ents(lens, starts, [0, 1, 2])
    pos = torch.tensor([s + i for n, s in zip(lens, starts) for i in range(n)], dtype=torch.int32)
    bt = torch.tensor([[3, 5, 0], [7, 2, 9], [1, 4, 8]], dtype=torch.int32)
    rows = torch.tensor([int(bt[e, p // PAGE]) * PAGE + p % PAGE
                         for e, (n, s) in enumerate(zip(lens, starts)) for p in range(s, s + n)],
                        dtype=torch.int32)
    pool = torch.randn(12 * PAGE, G * (D + V), generator=g).to(dt)
    nq, nk, nv = H * D, G * D, G * V
    proj = torch.randn(R, nq + nk + nv + 5, generator=g).to(dt)
    qw, kw = 1 + 0.1 * torch.randn(D, generator=g), 1 + 0.1 * torch.randn(D, generator=g)
    inv = sm.rope_inv_freq(3000.0, rot, "cpu", {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 40})
    q1, q2 = torch.empty(R, nq, dtype=dt), torch.empty(R, nq, dtype=dt, device=DEV)
    pool2 = pool.to(DEV)
    kw_ = dict(per_head=True, half=True)
    sm.qk_norm_rope_store(proj, H, G, D, V, qw, kw, inv, pos, rows, pool, 1e-5, q1, **kw_)
    sm.qk_norm_rope_store(proj.to(DEV), H, G, D, V, *_d(qw, kw, inv, pos, rows), pool2, 1e-5, q2, **kw_)
    torch.testing.assert_close(q2.cpu().float(), q1.float(), **_tol(dt))
    torch.testing.assert_close(pool2.cpu().float(), pool.float(), **_tol(dt))
    # queries alone (a layer that reads another layer's keys and values): the pool stays as it is
    q3 = torch.empty(R, nq, dtype=dt, device=DEV)
    before = pool2.clone()
    sm.qk_norm_rope_store(proj.to(DEV)[:, :nq], H, G, D, V, qw.to(DEV), None, inv.to(DEV), pos.to(DEV),
                          rows.to(DEV), None, 1e-5, q3, **kw_)
    torch.testing.assert_close(q3.cpu().float(), q1.float(), **_tol(dt))
    assert torch.equal(pool2, before)
    pool2.copy_(pool)
    q2.copy_(q1)
    win = 1 << 30
    o1 = torch.empty(R, H * V + 8, dtype=dt)[:, 8:]
    sm.window_attn(q1, pool, bt, row_ent, pos, None, 0.3, win, o1, PAGE, H, G, D, V)
    for mfma in ([False, True] if dt == torch.bfloat16 else [False]):
        for max_keys in (None, 300):    # whole prefixes / prefixes cut into runs
            o2 = torch.empty(R, H * V + 8, dtype=dt, device=DEV)[:, 8:]
            units = None
            if mfma:
                if not sm.window_mfma_ok(q2, pool2, D, V):
                    assert D % 8 or V % 8
                    continue
                units = sm.make_units(ent, sm.window_rows_per_wave(H // G)).to(DEV)
            sm.window_attn(q2, pool2, *_d(bt, row_ent, pos), None, 0.3, win, o2, PAGE, H, G, D, V,
                           units=units, max_keys=max_keys)
            torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [200, 8200])
def test_pointwise_and_residual(dt, W):
    g = torch.Generator().manual_seed(1)
    R, Fd = 9, 70
    gu = (torch.randn(R, 2 * Fd + 3, generator=g) * 2).to(dt)
    a = sm.glu_act(gu, torch.empty(R, Fd, dtype=dt), "gelu_tanh")
    b = sm.glu_act(gu.to(DEV), torch.empty(R, Fd, dtype=dt, device=DEV), "gelu_tanh")
    torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    ref = torch.nn.functional.gelu(gu[:, :Fd].float(), approximate="tanh") * gu[:, Fd:2 * Fd].float()
    torch.testing.assert_close(a.float(), ref.to(dt).float(), **_tol(dt))
    for gate in (True, False):
        gt = gu[:, Fd:Fd + 1] if gate else None
        a = sm.relu2_gate(gu, gt, torch.empty(R, Fd, dtype=dt))
        gd = gu.to(DEV)
        b = sm.relu2_gate(gd, gd[:, Fd:Fd + 1] if gate else None, torch.empty(R, Fd, dtype=dt, device=DEV))
        torch.testing.assert_close(b.cpu().float(), a.float(), **_tol(dt))
    big = torch.randn(R, 2 * W + 3, generator=g).to(dt)     # the addends as column views
    w = torch.randn(W, generator=g)
    x1, h1 = torch.randn(R, W, generator=g), torch.empty(R, W, dtype=dt)
    x2, h2 = x1.to(DEV), torch.empty(R, W, dtype=dt, device=DEV)
    bigd = big.to(DEV)
    sm.add_norm(x1, big[:, :W], big[:, W + 3:], 1e-5, next_w=w, next_out=h1)
    sm.add_norm(x2, bigd[:, :W], bigd[:, W + 3:], 1e-5, next_w=w.to(DEV), next_out=h2)
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(h2.cpu().float(), h1.float(), **_tol(dt))
    sm.add_norm(x1, big[:, :W])
    sm.add_norm(x2, bigd[:, :W])
    torch.testing.assert_close(x2.cpu(), x1, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E,ident,groups,keep,top,W,Fd", [(10, 2, 3, 2, 3, 72, 40), (8, 0, 1, 1, 2, 64, 64),
                                                           (1, 5, 6, 2, 2, 50, 33), (63, 7, 7, 3, 5, 96, 24),
                                                           (0, 4, 2, 1, 2, 40, 48)])
@pytest.mark.parametrize("R", [45, 300])     # few slots per expert / the large prompt tile
def test_softmax_router_identity_experts(dt, E, ident, groups, keep, top, W, Fd, R):
    g = torch.Generator().manual_seed(5)
    EA = E + ident
    h = torch.randn(R, W, generator=g).to(dt)
    wr = torch.randn(EA, W, generator=g) * 0.5
    corr = torch.randn(EA, generator=g) * 0.1 - 2.0          # every choice score is negative
    res = []
    for dev in ("cpu", DEV):
        ids = torch.empty(R, top, dtype=torch.int32, device=dev)
        wts = torch.empty(R, top, device=dev)
        cnt = torch.empty(EA, dtype=torch.int32, device=dev)
        rows = torch.full((EA, R * top), -1, dtype=torch.int32, device=dev)
        sm.group_route(h.to(dev), wr.to(dev), top, groups, keep, ids, wts, cnt, rows, score="softmax",
                       corr=corr.to(dev), group_score="max")
        res.append((ids.cpu(), wts.cpu(), cnt.cpu(), rows.cpu()))
    (i1, w1, c1, r1), (i2, w2, c2, r2) = res
    same = (i1 == i2).all(-1)
    assert (~same).float().mean() < 0.02         # the same choice, except where two scores tie within rounding
    torch.testing.assert_close(w2[same], w1[same], rtol=1e-5, atol=1e-7)
    assert int(c2.sum()) == R * top
    got = sorted(s_ for e in range(EA) for s_ in r2[e, :int(c2[e])].tolist())
    assert got == list(range(R * top))           # every slot in exactly one expert's list
    if E == 0:
        return
    # grouped products through the device's own slot lists: ungated squared-relu experts,
    # slots of identity experts are left out of the products and filled in by the weighted sum
    wu = (torch.randn(E, Fd, W, generator=g) / W ** 0.5).to(dt)
    wd = (torch.randn(E, W, Fd, generator=g) / Fd ** 0.5).to(dt)
    a1 = torch.zeros(R * top, Fd, dtype=dt)
    a2 = torch.zeros(R * top, Fd, dtype=dt, device=DEV)
    sm.expert_gemm(h, top, wu, c2, r2, a1, R * top, relu2=True)
    sm.expert_gemm(h.to(DEV), top, wu.to(DEV), c2.to(DEV), r2.to(DEV), a2, R * top, relu2=True)
    torch.testing.assert_close(a2.cpu().float(), a1.float(), **_tol(dt))
    y1 = torch.full((R * top, W), 7.0, dtype=dt)
    y2 = torch.full((R * top, W), 7.0, dtype=dt, device=DEV)
    sm.expert_gemm(a1, 1, wd, c2, r2, y1, R * top)
    sm.expert_gemm(a1.to(DEV), 1, wd.to(DEV), c2.to(DEV), r2.to(DEV), y2, R * top)
    torch.testing.assert_close(y2.cpu().float(), y1.float(), **_tol(dt))
    o1 = sm.expert_combine(y1, w2, torch.empty(R, W, dtype=dt), ids=i2, n_real=E, x=h)
    o2 = sm.expert_combine(y1.to(DEV), w2.to(DEV), torch.empty(R, W, dtype=dt, device=DEV), ids=i2.to(DEV),
                           n_real=E, x=h.to(DEV))
    torch.testing.assert_close(o2.cpu().float(), o1.float(), **_tol(dt))
    # by hand for one row
    r = 3
    want = sum(float(w2[r, k]) * (h[r].float() if int(i2[r, k]) >= E else y1[r * top + k].float())
               for k in range(top))
    torch.testing.assert_close(o1[r].float(), want.to(dt).float(), **_tol(dt))
