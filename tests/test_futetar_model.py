"""The Futetar hybrid model on the engine against the plain oracle (tests/futetar_oracle.py).

Every test builds its own small configuration and random checkpoint, runs the oracle once
over whole sequences in float64, and drives the engine's step function / generate / server
in float32 (and bfloat16 with a loose bound).  The CPU variants exercise the model, cache,
batching and scheduling code with the ops' PyTorch rendering; the ``gpu`` variants run the
same cases on the HIP kernels.
"""
import copy
import math

import pytest
import torch

import futetar_oracle as O
from p2p_llm_chat_go_amd.engine.hybrid import HybridEngine
from p2p_llm_chat_go_amd.models import hybrid as Hy
from p2p_llm_chat_go_amd.ops import PAGE

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]

DENSE = {"kind": "dense", "ff": 72}
MOE = {"kind": "moe", "expert": {"ff": 24}, "shared": {"ff": 40},
       "router": {"experts": 7, "identity": 2, "top": 3, "groups": {"count": 3, "keep": 2}}}
ML = {"type": "mlstm", "mixer": {"heads": 3, "dim": 12, "vdim": 20, "gate_cap": 6.0}, "mlp": None}
ROT = {"base": 300.0, "dims": 10, "scaling": {"factor": 3.0, "low": 1.0, "high": 6.0, "original": 60}}
AT = {"type": "attention", "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "rot": ROT, "scale": 0.4},
      "mlp": None}


def layer(base, mlp=None, **mixer):
    L = copy.deepcopy(base)
    L["mlp"] = copy.deepcopy(mlp)
    L["mixer"].update(copy.deepcopy(mixer))
    return L


def make(layers, width=48, vocab=97, seed=0, eps=1e-5):
    c = {"architecture": "Futetar", "width": width, "vocab": vocab, "norm": {"eps": eps},
         "layers": copy.deepcopy(layers)}
    cfg = Hy.HybridConfig.from_dict(c)
    sd = Hy.random_state_dict(cfg, seed)
    return c, cfg, sd


def engine(cfg, sd, dev, dtype=torch.float32, pages=24, slots=4, **kw):
    return HybridEngine(cfg, Hy.HybridWeights(cfg, sd, dev, dtype), dev, kv_pages=pages,
                        num_slots=slots, max_batch=slots, **kw)


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, ref, tol=2e-4, over=0.0):
    """Difference of logits rows, mean removed, RMS over the vocabulary, relative to the
    RMS of the reference logits.  over: share of rows that may exceed the bound (bf16 rounding
    can move a router's choice between two experts with nearly equal scores)."""
    got, ref = got.detach().cpu().double(), ref.double()
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    scale = (ref - ref.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    err = d.pow(2).mean(-1).sqrt() / scale
    bad = (err >= tol).double().mean().item()
    assert bad <= over, "relative logits error %.3g, %.3g of the rows over %g" % (err.max().item(), bad, tol)


def run_whole(eng, key, t):
    out = eng.step([(key, t, list(range(len(t))))])
    eng.release(key)
    return out


def run_cuts(eng, key, t, cuts):
    at, outs = 0, []
    for n in cuts:
        n = min(n, len(t) - at)
        if n <= 0:
            break
        outs.append(eng.step([(key, t[at:at + n], list(range(n)))]))
        at += n
    if at < len(t):
        outs.append(eng.step([(key, t[at:], list(range(len(t) - at)))]))
    eng.release(key)
    return torch.cat(outs)


# ------------------------------------------------------------------ each mechanism alone
NO_EXTRAS = {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 5, "top": 2}}
ALONE = {
    "mlstm": [ML],
    "attention": [AT],
    "attention_borrowed_kv": [AT, layer(AT, kv_from=0)],
    "dense_ff": [layer(ML, DENSE)],
    "moe_ff": [layer(ML, MOE)],
    "moe_plain": [layer(AT, NO_EXTRAS)],          # no groups, no identity experts, no shared expert
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(ALONE))
def test_single_mechanism(dev, name):
    c, cfg, sd = make(ALONE[name], seed=3)
    t = toks(70, cfg.vocab, 1)
    ref = O.forward(c, sd, t)
    close(run_whole(engine(cfg, sd, dev), "a", t), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_layers_match_oracle(dev):
    c, cfg, sd = make([layer(AT, MOE), layer(ML, DENSE), layer(AT, DENSE, kv_from=0), layer(ML, MOE), AT,
                       layer(AT, MOE, kv_from=4)], seed=4)
    t = toks(40, cfg.vocab, 2)
    ref, lay = O.forward(c, sd, t, return_layers=True)
    eng = engine(cfg, sd, dev)
    got = []
    out = eng.step([("a", t, list(range(len(t))))], return_layers=got)
    assert len(got) == len(lay)
    for i, x in enumerate(got):
        torch.testing.assert_close(x.cpu().double(), lay[i], rtol=1e-4, atol=1e-4, msg="layer %d" % i)
    close(out, ref)


def test_oracle_pieces():
    """The oracle's own building blocks on cases that can be worked out by hand."""
    # routing: 2 groups of 3, ranked by their best choice score; weights are the plain scores
    z = torch.tensor([2.0, 1.9, 1.8, 2.05, -9.0, -9.0], dtype=torch.float64)
    s = torch.softmax(z, 0)
    zero = torch.zeros(6, dtype=torch.float64)
    r = {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 1}}
    got = O.route(z, zero, r)
    assert [e for e, _ in got] == [3, 4]      # the group of the single best expert wins as a whole
    assert abs(float(got[0][1]) - float(s[3])) < 1e-15
    # a correction moves the choice and leaves the weights alone; choice scores may be negative
    corr = torch.tensor([-5.0, -5.0, -5.0, -6.0, -6.0, -6.0], dtype=torch.float64)
    got = O.route(z, corr, r)
    assert [e for e, _ in got] == [0, 1] and abs(float(got[1][1]) - float(s[1])) < 1e-15
    assert [e for e, _ in O.route(z, zero, dict(r, groups={"count": 2, "keep": 2}))] == [3, 0]
    # rotation: base 1 -> angle = position; channel 0 pairs with channel dims/2
    x = torch.zeros(3, 1, 6, dtype=torch.float64)
    x[:, 0, 0] = 1.0
    x[:, 0, 4] = 5.0
    y = O.rotate_half(x, {"base": 1.0, "dims": 4})
    torch.testing.assert_close(y[2, 0, [0, 2]], torch.tensor([math.cos(2.0), math.sin(2.0)], dtype=torch.float64))
    assert float(y[2, 0, 4]) == 5.0 and float(y[2, 0, 1]) == 0.0
    # stretched wavelengths: all three cases occur in the shared test rotation
    f0 = [ROT["base"] ** (-2.0 * i / ROT["dims"]) for i in range(ROT["dims"] // 2)]
    f1 = O.scaled_freqs(ROT)
    kinds = {"kept" if a == b else "slowed" if abs(b - a / 3.0) < 1e-15 else "between" for a, b in zip(f0, f1)}
    assert kinds == {"kept", "slowed", "between"}
    # matrix memory, one head, one channel: two steps by hand (m starts at 0, not at -inf)
    t = {"q": torch.tensor([[1.0]]), "k": torch.tensor([[1.0]]), "v": torch.tensor([[2.0]]),
         "g": torch.tensor([[0.0]]), "o": torch.tensor([[1.0]]), "norm": torch.tensor([1.0]),
         "i": torch.tensor([[0.0]]), "i.b": torch.tensor([-3.0]), "f": torch.tensor([[0.0]]),
         "f.b": torch.tensor([0.0])}
    t = {k: v.double() for k, v in t.items()}
    h = torch.tensor([[1.0], [1.0]], dtype=torch.float64)
    out = O.mlstm(h, t, "", {"heads": 1, "dim": 1, "vdim": 1, "gate_cap": 100.0}, 0.0)
    # o is a single channel: after the head norm it is its sign; times sigmoid(0)
    torch.testing.assert_close(out, torch.tensor([[0.5], [0.5]], dtype=torch.float64))
    i_, f_ = 100.0 * math.tanh(-0.03), math.log(0.5)
    m1 = max(f_ + 0.0, i_)
    assert m1 == f_                            # with m_0 = -inf it would be i_
    assert abs(float(O.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


# ------------------------------------------------------------------ other sizes
VARIANTS = {
    # one head, one kv head, one expert chosen, one group, one identity expert, nothing rotated
    "ones": [layer(ML, {"kind": "moe", "expert": {"ff": 16}, "shared": {"ff": 8},
                        "router": {"experts": 3, "identity": 1, "top": 1, "groups": {"count": 1, "keep": 1}}},
                   heads=1, dim=24, vdim=8, gate_cap=1.0),
             {"type": "attention", "mixer": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 1.0},
              "mlp": None}],
    # sizes that are not multiples of 8 or 16, partial rotation without stretching, every group kept,
    # only identity experts beside one real one
    "odd": [layer(AT, {"kind": "moe", "expert": {"ff": 10},
                       "router": {"experts": 1, "identity": 5, "top": 4, "groups": {"count": 3, "keep": 3}}},
                  heads=5, kv_heads=5, dim=6, vdim=10, rot={"base": 40000.0, "dims": 2}, scale=0.05),
            layer(ML, {"kind": "dense", "ff": 50}, heads=5, dim=6, vdim=4, gate_cap=30.0),
            layer(AT, None, heads=5, kv_heads=5, dim=6, vdim=10, rot={"base": 40000.0, "dims": 2}, scale=0.05,
                  kv_from=0)],
    # wide states, value size above key size, full rotation
    "wide": [layer(ML, None, heads=1, dim=72, vdim=80),
             layer(AT, DENSE, heads=4, kv_heads=1, dim=40, vdim=72,
                   rot={"base": 1000.0, "dims": 40, "scaling": {"factor": 2.0, "low": 2.0, "high": 3.0, "original": 50}},
                   scale=0.5),
             layer(ML, MOE, heads=2, dim=40, vdim=72, gate_cap=2.5)],
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes(dev, name):
    c, cfg, sd = make(VARIANTS[name], width=40 if name != "wide" else 100, vocab=61, seed=5, eps=1e-3)
    t = toks(75, cfg.vocab, 3)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    # first part as a prompt, the rest in portions of 1, 2 and 5 tokens
    close(run_cuts(eng, "a", t, [40, 1, 2, 5, 1, 1, 2, 23]), ref)


# ------------------------------------------------------------------ prefill vs decode, portions
@pytest.mark.parametrize("dev", DEVICES)
def test_prefill_decode_and_portions(dev):
    c, cfg, sd = make([layer(AT, MOE), layer(ML, DENSE), layer(AT, None, kv_from=0), ML], seed=6)
    n = 2 * PAGE + 21                      # crosses two page borders and the scans' chunks
    t = toks(n, cfg.vocab, 4)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "w", t), ref)
    # token by token from the first token on
    close(run_cuts(eng, "d", t, [1] * n), ref)
    # portions of changing size, down to two tokens and one, cut inside pages and chunks
    for sizes in ([2] * 20 + [63, 1, 1, 2, 40, 3], [5, 59, 1, 64, 7, 2, 3, 8], [129, 2, 1, 17]):
        close(run_cuts(eng, "p", t, sizes), ref)


# ------------------------------------------------------------------ batches, reuse of pages and slots
@pytest.mark.parametrize("dev", DEVICES)
def test_mixed_batches_and_reuse(dev):
    c, cfg, sd = make([layer(ML, MOE), layer(AT, DENSE), layer(AT, MOE, kv_from=1)], seed=7)
    lens = [150, 9, 70, 1, 33, 130, 64, 65]
    reqs = {i: toks(n, cfg.vocab, 10 + i) for i, n in enumerate(lens)}
    refs = {i: O.forward(c, sd, t) for i, t in reqs.items()}
    # a pool that holds three of the long requests at most: pages and slots must come back
    eng = engine(cfg, sd, dev, pages=8, slots=3)
    got = {i: [] for i in reqs}
    at = {i: 0 for i in reqs}
    waiting, live, step = sorted(reqs), [], 0
    sizes = [7, 1, 30, 2, 1, 64, 3, 1, 1, 19]
    while waiting or live:
        while waiting and len(live) < 3:
            need = sum(-(-len(reqs[i]) // PAGE) for i in live) + -(-len(reqs[waiting[0]]) // PAGE)
            if need > 7:
                break
            live.append(waiting.pop(0))
        entries = []
        for j, i in enumerate(live):
            if (step + j) % 4 == 3 and len(live) > 1:
                continue                      # a request may sit a step out
            n = min(sizes[(step + 3 * j) % len(sizes)], len(reqs[i]) - at[i])
            entries.append((i, reqs[i][at[i]:at[i] + n], list(range(n))))
            at[i] += n
        out = eng.step(entries)
        o = 0
        for i, tk, w in entries:
            got[i].append(out[o:o + len(w)])
            o += len(w)
        for i in [i for i in live if at[i] == len(reqs[i])]:
            eng.release(i)
            live.remove(i)
        step += 1
    assert eng.cache.live == 0 and eng.cache.allocator.free_pages == 7 and eng.cache.slots.free_slots == 3
    for i in reqs:
        close(torch.cat(got[i]), refs[i])


@pytest.mark.parametrize("dev", DEVICES)
def test_first_tokens_in_a_used_slot(dev):
    """A sequence that starts in a slot and pages another one left behind sees none of it:
    zero memory and normaliser, a running maximum of 0, no keys before position 0.  The input
    gate's bias is far below zero, so the running maximum of the first tokens comes from its
    start value."""
    c, cfg, sd = make([ML, AT, layer(ML, MOE), layer(AT, None, kv_from=1)], seed=8)
    for i in (0, 2):
        sd["l%d.mix.i.b" % i] = torch.full_like(sd["l%d.mix.i.b" % i], -4.0)
    eng = engine(cfg, sd, dev, pages=3, slots=1)
    a, b = toks(100, cfg.vocab, 20), toks(7, cfg.vocab, 21)
    eng.step([("a", a, [])])
    eng.release("a")
    ref = O.forward(c, sd, b)
    outs = [eng.step([("b", [b[0]], [0])]), eng.step([("b", b[1:3], [0, 1])]), eng.step([("b", b[3:], [0, 1, 2, 3])])]
    close(torch.cat(outs), ref)


# ------------------------------------------------------------------ far tokens, long decoding
@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("which", ["remember", "saturated_gates"])
def test_memory_far_tokens_and_long_decoding(dev, which):
    c, cfg, sd = make([ML, layer(ML, DENSE)], seed=9)
    for i in (0, 1):
        p = "l%d.mix." % i
        if which == "remember":            # forget gates near 1: the memory keeps the first tokens
            sd[p + "f.b"] = torch.full_like(sd[p + "f.b"], 5.0)
        else:                              # pre-activations far beyond the cap, both signs
            sd[p + "i"] = sd[p + "i"] * 40
            sd[p + "f"] = sd[p + "f"] * 40
    n = 3 * PAGE + 10
    t = toks(n, cfg.vocab, 30)
    ref = O.forward(c, sd, t)
    if which == "remember":
        t2 = list(t)
        t2[2] = (t[2] + 1) % cfg.vocab
        ref2 = O.forward(c, sd, t2)
        assert (ref[-1] - ref2[-1]).abs().max() > 1e-3     # token 2 still matters 200 tokens on
    else:
        t2, ref2 = t, ref
        flat = dict(c, layers=[layer(L, L["mlp"], gate_cap=1e4) for L in c["layers"]])
        assert (O.forward(flat, sd, t) - ref).abs().max() > 1e-2   # the cap is at work
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "w", t), ref)
    close(run_cuts(eng, "a", t, [20] + [1] * (n - 20)), ref)          # 180+ decoded tokens
    close(run_cuts(eng, "b", t2, [20] + [1] * (n - 20))[-1:], ref2[-1:])


@pytest.mark.parametrize("dev", DEVICES)
def test_scan_chunk_edges(dev):
    """Long portions of a memory layer run as chunks of 64 tokens side by side once a portion
    has 128 tokens: lengths just below, at and above these edges, alone and continued, with a
    memory that keeps its first tokens."""
    c, cfg, sd = make([layer(ML, None, heads=2, dim=16, vdim=16), layer(ML, DENSE)], seed=19)
    for i in (0, 1):
        sd["l%d.mix.f.b" % i] = torch.full_like(sd["l%d.mix.f.b" % i], 4.0)
    t = toks(4 * PAGE + 2, cfg.vocab, 31)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    for cuts in ([127, 1, 128, 2], [128, 129], [129, 127, 2], [63, 65, 130], [191, 67], [192, 66], [193, 1, 64]):
        close(run_cuts(eng, "a", t, cuts), ref)
    # two long portions and a decoded token of other requests in one step
    a, b = t[:200], t[:150]
    eng.step([("x", a[:10], []), ("y", b[:149], [])])
    out = eng.step([("x", a[10:], [189]), ("y", b[149:], [0]), ("z", t[:130], [129])])
    close(out, torch.stack([ref[199], ref[149], ref[129]]))


# ------------------------------------------------------------------ far keys, page borders, causal edge
def spike_model(hot, qtok, beta=25.0, seed=11, borrowed=False):
    """Attention alone whose query projection is rebuilt so that every query points along the
    unrotated part of the key of token ``hot``: where ``hot`` is visible it takes nearly all
    the softmax weight, however far back it is."""
    mx = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "rot": {"base": 100.0, "dims": 4}, "scale": 1.0}
    first = {"type": "attention", "mixer": mx, "mlp": None}
    layers = [first, layer(first, kv_from=0)] if borrowed else [first]
    c, cfg, sd = make(layers, width=32, vocab=50, seed=seed)
    f = lambda k: sd[k].double()
    eps = c["norm"]["eps"]
    H, G, D = mx["heads"], mx["kv_heads"], mx["dim"]
    sd["l0.mix.k.norm"] = torch.ones_like(sd["l0.mix.k.norm"])
    last = "l%d.mix." % (len(layers) - 1)
    sd[last + "q.norm"] = torch.ones_like(sd[last + "q.norm"])
    if borrowed:   # the first layer adds nothing, so the second sees the same input
        sd["l0.mix.o"] = torch.zeros_like(sd["l0.mix.o"])
        sd["l1.norm1"] = sd["l0.norm1"].clone()
    u = O.norm_one_plus(f("embed"), f("l0.norm1"), eps)
    k = O.rms((f("l0.mix.k") @ u[hot]).view(G, D), eps).clone()
    rot = [0, 1, 2, 3]                       # pairs (0, 2) and (1, 3)
    k[:, rot] = 0.0
    target = k.repeat_interleave(H // G, 0).reshape(-1)                  # [H * D]
    xq = u[qtok]
    sd[last + "q"] = (target[:, None] * xq[None, :] / (xq @ xq)).to(torch.bfloat16)
    qn = O.rms(target.view(H, D), eps)
    c["layers"][-1]["mixer"]["scale"] = beta / float((qn[0] * k[0]).sum())
    if borrowed:
        c["layers"][0]["mixer"]["scale"] = c["layers"][-1]["mixer"]["scale"]
    cfg = Hy.HybridConfig.from_dict(c)
    return c, cfg, sd


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("borrowed", [False, True])
@pytest.mark.parametrize("n,where", [(3 * PAGE + 9, 0), (3 * PAGE + 9, PAGE - 1), (3 * PAGE + 9, PAGE),
                                     (2 * PAGE + 1, 2 * PAGE - 1), (2 * PAGE + 1, 2 * PAGE), (40, 3)])
def test_far_keys_and_page_borders(dev, n, where, borrowed):
    """One key among hundreds takes the weight: at the sequence's start, on both sides of page
    borders, as the newest key; in a prompt and when decoding; in a layer with keys of its own
    and in one that reads another layer's."""
    hot, qtok = 7, 11
    c, cfg, sd = spike_model(hot, qtok, borrowed=borrowed)
    g = torch.Generator().manual_seed(n * 1000 + where)
    t = torch.randint(0, cfg.vocab, (n,), generator=g).tolist()
    t = [x if x not in (hot, qtok) else 8 for x in t]
    t[-1] = qtok
    base = O.forward(c, sd, t)
    tt = list(t)
    tt[where] = hot
    ref = O.forward(c, sd, tt)
    assert (ref[-1] - base[-1]).abs().max() > 0.05, "the hot key does not show in the oracle"
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "w", tt), ref)
    k = min(5, n - 1)
    close(run_cuts(eng, "d", tt, [n - k] + [1] * k), ref)
    # the hot key decoded alone, the query in a portion of two
    close(run_cuts(eng, "e", tt, [max(1, where), 1] + [2] * n), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_causal_edge(dev):
    """The query sees its own key and not the next one: a hot key at the query's place shows,
    one place later it does not (in the oracle and in the engine)."""
    hot, qtok = 7, 11
    c, cfg, sd = spike_model(hot, qtok)
    # make the query token's own key the hot one by querying from the hot token itself
    c2, cfg2, sd2 = spike_model(hot, hot, seed=11)
    n = PAGE + 4
    t = [x if x != hot else 8 for x in toks(n, cfg2.vocab, 70)]
    t[PAGE] = hot
    ref = O.forward(c2, sd2, t)
    t2 = list(t)
    t2[PAGE + 1] = hot
    ref2 = O.forward(c2, sd2, t2)
    torch.testing.assert_close(ref2[PAGE], ref[PAGE], rtol=1e-12, atol=1e-12)   # the future is not seen
    eng = engine(cfg2, sd2, dev)
    close(run_whole(eng, "a", t2), ref2)
    close(run_cuts(eng, "b", t2, [PAGE, 1, 1, 2]), ref2)
    close(run_cuts(eng, "c", t2, [PAGE - 1, 2, 2]), ref2)


@pytest.mark.parametrize("dev", DEVICES)
def test_rotation_depends_on_distance_only(dev):
    """With every wavelength kept (no stretching at work) the same tokens behind a prefix whose
    keys get no weight give the same attention: here the check is simply that the engine follows
    the oracle at positions where stretched and unstretched wavelengths differ widely."""
    mx = dict(AT["mixer"], rot={"base": 50.0, "dims": 16,
                                "scaling": {"factor": 16.0, "low": 1.0, "high": 2.0, "original": 24}})
    c, cfg, sd = make([{"type": "attention", "mixer": mx, "mlp": None}], seed=21)
    t = toks(2 * PAGE + 30, cfg.vocab, 22)
    ref = O.forward(c, sd, t)
    plain = copy.deepcopy(c)
    del plain["layers"][0]["mixer"]["rot"]["scaling"]
    assert (O.forward(plain, sd, t)[-1] - ref[-1]).abs().max() > 1e-3
    close(run_cuts(engine(cfg, sd, dev), "s", t, [PAGE + 3, 7, 1, 1, 2]), ref)


# ------------------------------------------------------------------ router
@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("case", ["negative_choice", "identity_wins", "correction_moves_choice"])
def test_router_cases(dev, case):
    moe = {"kind": "moe", "expert": {"ff": 24}, "shared": {"ff": 16},
           "router": {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}}}
    c, cfg, sd = make([layer(ML, moe)], seed=23)
    t = toks(60, cfg.vocab, 24)
    # corrections on a grid that survives the shifts below in bfloat16
    sd["l0.mlp.correction"] = (torch.round(sd["l0.mlp.correction"].float() * 64) / 64).to(torch.bfloat16)
    base = O.forward(c, sd, t)
    corr = sd["l0.mlp.correction"].float()
    if case == "negative_choice":        # every choice score below zero: struck-out groups must rank lower still
        corr = corr - 3.0
    elif case == "identity_wins":        # the last group (the identity experts) is always kept and chosen
        corr[-2:] += 2.0
    else:                                # one expert is pushed into every choice; its weight stays its score
        corr[1] += 2.0
    sd["l0.mlp.correction"] = corr.to(torch.bfloat16)
    ref = O.forward(c, sd, t)
    if case != "negative_choice":
        assert (ref - base).abs().max() > 1e-3
    else:
        torch.testing.assert_close(ref, base, rtol=1e-9, atol=1e-9)   # a common shift changes nothing
    close(run_cuts(engine(cfg, sd, dev), "a", t, [33, 1, 2, 24]), ref)


# ------------------------------------------------------------------ bf16 serving precision
@pytest.mark.parametrize("dev", DEVICES)
def test_bfloat16(dev):
    c, cfg, sd = make([layer(ML, DENSE, heads=4, dim=16, vdim=32),
                       layer(AT, DENSE, heads=8, kv_heads=2, dim=32, vdim=32,
                             rot=dict(ROT, dims=32)),
                       layer(AT, None, heads=8, kv_heads=2, dim=32, vdim=32, rot=dict(ROT, dims=32), kv_from=1),
                       layer(ML, MOE, heads=4, dim=16, vdim=32)], width=128, vocab=200, seed=13)
    t = toks(PAGE + 30, cfg.vocab, 50)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev, dtype=torch.bfloat16)
    # the experts sit in the last layer only: a choice that rounding moves between two experts
    # with nearly equal scores then changes that row alone, not the states after it
    close(run_whole(eng, "a", t), ref, tol=0.08, over=0.1)
    close(run_cuts(eng, "b", t, [50] + [1] * 44), ref, tol=0.08, over=0.1)


# ------------------------------------------------------------------ generation
def near_tie(c, sd, prompt, got, n):
    """Greedy tokens equal the oracle's, or differ only where its top two logits tie."""
    seq = list(prompt)
    for tkn in got[:n]:
        lg = O.forward(c, sd, seq)[-1]
        assert tkn == int(lg.argmax()) or float(lg.max() - lg[tkn]) < 1e-3 * float(lg.abs().max())
        seq.append(tkn)


@pytest.mark.parametrize("dev", DEVICES)
def test_generate_greedy(dev):
    c, cfg, sd = make([layer(ML, MOE), layer(AT, DENSE), layer(AT, None, kv_from=1)], seed=14)
    prompts = [toks(n, cfg.vocab, 60 + n) for n in (12, 70, 3)]
    eng = engine(cfg, sd, dev, max_prefill_tokens=32)      # prompts are cut into portions
    res = eng.generate(prompts, max_new_tokens=12, stop_on_eos=False)
    for p, r in zip(prompts, res):
        assert len(r.tokens) == 12 and r.prompt_eval_count == len(p)
        near_tie(c, sd, p, r.tokens, 12)
    assert eng.cache.live == 0 and eng.cache.slots.free_slots == 4


@pytest.mark.parametrize("dev", DEVICES)
def test_server_scheduler_greedy(dev):
    """Through the continuous-batching server: the native scheduler owns the pages, requests
    arrive while others decode, state slots are handed back and used again."""
    native = pytest.importorskip("p2p_llm_chat_go_amd.native")
    try:
        native.load()
    except Exception as e:  # noqa: BLE001
        pytest.skip("native runtime not built: %s" % e)
    from p2p_llm_chat_go_amd.engine.sampling import SamplingParams
    from p2p_llm_chat_go_amd.engine.server import EngineServer

    c, cfg, sd = make([layer(ML, DENSE), layer(AT, MOE), layer(AT, None, kv_from=1)], seed=15)
    eng = engine(cfg, sd, dev, pages=40, slots=2, max_prefill_tokens=48)
    srv = EngineServer(eng, max_batch=2, decode_chunk=4)
    try:
        prompts = [toks(n, cfg.vocab, 80 + n) for n in (20, 5, 66, 9, 31)]
        futs = [srv.submit(p, SamplingParams(max_tokens=10, stop_on_eos=False)) for p in prompts]
        for p, f in zip(prompts, futs):
            r = f.result(timeout=120)
            assert len(r["tokens"]) == 10
            near_tie(c, sd, p, r["tokens"], 10)
        assert eng.cache.slots.free_slots == 2
    finally:
        srv.close()


@pytest.mark.gpu
def test_decode_graph_matches_eager():
    """Greedy decoding through the captured step graph, replayed many times with eager steps
    of other requests in between, gives the tokens of the eager engine."""
    c, cfg, sd = make([layer(ML, MOE), layer(AT, DENSE), layer(AT, MOE, kv_from=1), ML], width=64, seed=16)
    prompts = [toks(n, cfg.vocab, 90 + n) for n in (70, 5, 33)]
    w = Hy.HybridWeights(cfg, sd, "cuda:0", torch.bfloat16)
    outs = []
    for graph in (True, False):
        eng = HybridEngine(cfg, w, "cuda:0", kv_pages=24, num_slots=4, max_batch=4, use_graph=graph)
        res = eng.generate(prompts, max_new_tokens=40, stop_on_eos=False)
        res2 = eng.generate(prompts[:2], max_new_tokens=70, stop_on_eos=False)
        outs.append([r.tokens for r in res + res2])
        assert bool(eng._graphs) == graph
    assert outs[0] == outs[1]
    for p, t in zip(prompts, outs[0]):
        assert len(t) == 40


def test_trace_runner_cli(tmp_path):
    """bin/trace_run on a saved checkpoint: steps on stdin, logits files and 'done' lines out,
    finished requests hand their pages and slot back (the pool is smaller than the sum)."""
    import json
    import os
    import subprocess

    import numpy as np
    from safetensors.torch import save_file

    c, cfg, sd = make([layer(ML, MOE), AT, layer(AT, DENSE, kv_from=1)], seed=17)
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(c))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model / "model.safetensors"))
    a, b, d = toks(90, cfg.vocab, 1), toks(40, cfg.vocab, 2), toks(100, cfg.vocab, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:50], "want": [0, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[50:88], "want": []},
                                {"id": "b", "tokens": b[:39], "want": [38]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[39:], "want": [0]},
                                {"id": "a", "tokens": a[88:], "want": [0, 1]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "d", "tokens": d, "want": [99]}], "end": ["d"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "192", "--device", "cpu"],
                       input="".join(json.dumps(x) + "\n" for x in steps), capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == ["done %d" % i for i in range(4)]
    ra, rb, rd = (O.forward(c, sd, t) for t in (a, b, d))
    got = {i: torch.from_numpy(np.fromfile(out / ("%d.f32" % i), dtype="<f4").reshape(-1, cfg.vocab))
           for i in (0, 1, 2, 3)}
    close(got[0], ra[[0, 49]])
    close(got[1], rb[[38]])
    close(got[2], torch.stack([rb[39], ra[88], ra[89]]))
    close(got[3], rd[[99]])


def test_preset_through_registry(tmp_path):
    """The preset and a saved checkpoint both reach the hybrid engine through the registry."""
    import json

    from safetensors.torch import save_file

    from p2p_llm_chat_go_amd.models import registry
    from p2p_llm_chat_go_amd.models.config import get_config

    cfg = get_config("tiny-futetar")
    assert cfg.design == "Futetar" and cfg.is_moe and not cfg.traits.positions
    sd = Hy.random_state_dict(cfg, 3)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    assert registry.is_hybrid_dir(str(tmp_path)) and registry.supports_dtype(str(tmp_path), torch.float32)
    cfg2, w = registry.load_checkpoint(str(tmp_path), "cpu", torch.float32)
    assert cfg2.layers == cfg.layers
    eng = registry.make_engine(cfg2, w, "cpu", kv_pages=6, num_slots=2, max_batch=2, dtype=torch.float32)
    p = toks(9, cfg.vocab, 5)
    r = eng.generate([p], max_new_tokens=4, stop_on_eos=False)[0]
    near_tie(cfg.to_dict(), sd, p, r.tokens, 4)


def test_config_roundtrip_and_errors():
    c, cfg, sd = make([layer(ML, MOE), layer(AT, DENSE), layer(AT, None, kv_from=1)])
    again = Hy.HybridConfig.from_dict(cfg.to_dict())
    assert again.layers == cfg.layers and again.design == "Futetar" and again.is_moe
    assert set(Hy.tensor_shapes(cfg)) == set(sd) and "pos" not in sd
    assert "l2.mix.k" not in sd and "l2.mix.k.norm" not in sd and "l2.mix.q.norm" in sd
    assert "l0.mlp.e6.up" in sd and "l0.mlp.e7.up" not in sd and sd["l0.mlp.router"].shape[0] == 9
    # the layer that lends its keys and values keeps the only pool; the borrower keeps nothing
    specs = Hy.HybridWeights(cfg, sd, "cpu", torch.float32).cache_specs()
    assert specs[1][0] == "paged" and specs[2] is None and specs[0][0] == "state"
    bad = dict(sd)
    bad["l0.mix.i.b"] = bad["l0.mix.i.b"][:2]
    with pytest.raises(ValueError):
        Hy.HybridWeights(cfg, bad, "cpu", torch.float32)
    for layers in ([layer(AT, None, kv_from=1), AT],                     # a later layer
                   [ML, layer(AT, None, kv_from=0)],                     # not an attention layer
                   [AT, layer(AT, None, kv_from=0), layer(AT, None, kv_from=1)],   # a borrower itself
                   [AT, layer(AT, None, kv_from=0, kv_heads=3)]):        # another shape
        c2, cfg2, sd2 = make(layers)
        with pytest.raises(ValueError):
            Hy.HybridWeights(cfg2, sd2, "cpu", torch.float32)
    with pytest.raises(ValueError):       # more experts chosen than the kept groups hold
        make([layer(ML, dict(MOE, router={"experts": 7, "identity": 2, "top": 4, "groups": {"count": 3, "keep": 1}}))])
    with pytest.raises(ValueError):       # experts + identity experts do not split into the groups
        make([layer(ML, dict(MOE, router={"experts": 7, "identity": 1, "top": 2, "groups": {"count": 3, "keep": 2}}))])
    eng = engine(cfg, sd, "cpu", pages=2, slots=1)
    eng.step([("a", [1, 2, 3], [2])])
    with pytest.raises(MemoryError):
        eng.step([("b", [1], [0])])          # no second state slot
    with pytest.raises(MemoryError):
        eng.step([("a", [1] * PAGE, [])])    # no second page
