"""The Tarunex hybrid model on the engine against the plain oracle (tests/tarunex_oracle.py).

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

import tarunex_oracle as O
from p2p_llm_chat_go_amd.engine.hybrid import HybridEngine
from p2p_llm_chat_go_amd.models import hybrid as Hy
from p2p_llm_chat_go_amd.ops import PAGE

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]

MOE = {"kind": "moe", "expert": {"ff": 24}, "shared": {"ff": 40}, "router": {"experts": 7, "top": 3}}
PLAIN = {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 5, "top": 2}}   # no shared expert
BA = {"type": "attention",
      "mixer": {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.3, "softcap": 8.0,
                "q_temp": {"coef": 0.4, "every": 5}},
      "mlp": None}
LA = {"type": "latent_attention",
      "mixer": {"heads": 3, "dim": 12, "rot_dim": 8, "vdim": 20, "kv_rank": 24, "q_rank": 28,
                "rot": {"base": 300.0, "dims": 8}, "scale": 0.25},
      "mlp": None}


def layer(base, mlp=None, **mixer):
    L = copy.deepcopy(base)
    L["mlp"] = copy.deepcopy(mlp)
    L["mixer"].update(copy.deepcopy(mixer))
    return L


def make(layers, width=48, vocab=97, seed=0, eps=1e-5, loop=None, embed_scale=3.0, logit_scale=0.5,
         logit_softcap=20.0):
    c = {"architecture": "Tarunex", "width": width, "vocab": vocab, "norm": {"eps": eps},
         "embedding": {"scale": embed_scale}, "logit_scale": logit_scale, "logit_softcap": logit_softcap,
         "layers": copy.deepcopy(layers)}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
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
    can move a router's choice between two experts with nearly equal logits)."""
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
ALONE = {
    "biased_attention": ([BA], None),
    "biased_attention_bare": ([layer(BA, None, softcap=0.0, q_temp=None)], None),
    "latent_attention": ([LA], None),
    "moe_shared": ([layer(BA, MOE)], None),
    "moe_plain": ([layer(LA, PLAIN)], None),
    "dense_ff": ([layer(LA, {"kind": "dense", "ff": 72})], None),
    "passes": ([BA, LA], (0, 2, 3)),
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(ALONE))
def test_single_mechanism(dev, name):
    layers, loop = ALONE[name]
    c, cfg, sd = make(layers, seed=3, loop=loop)
    t = toks(70, cfg.vocab, 1)
    ref = O.forward(c, sd, t)
    close(run_whole(engine(cfg, sd, dev), "a", t), ref)


@pytest.mark.parametrize("dev", DEVICES)
def test_layers_match_oracle(dev):
    c, cfg, sd = make([layer(LA, MOE), layer(BA, MOE), layer(LA, PLAIN), BA, layer(BA, MOE)], seed=4, loop=(1, 4, 2))
    t = toks(40, cfg.vocab, 2)
    lay = []
    ref = O.forward(c, sd, t, layers_out=lay)
    eng = engine(cfg, sd, dev)
    got = []
    out = eng.step([("a", t, list(range(len(t))))], return_layers=got)
    assert len(got) == len(lay) == 1 + 2 * 3 + 1
    for i, x in enumerate(got):
        torch.testing.assert_close(x.cpu().double(), lay[i], rtol=1e-4, atol=2e-4, msg="layer run %d" % i)
    close(out, ref)
    # the same rows when the residual pass is not split for the listing
    close(run_whole(eng, "b", t), ref)


def test_oracle_pieces():
    """The oracle's own building blocks on cases that can be worked out by hand."""
    # the temperature steps up when position + 1 reaches a multiple of `every`
    assert O.query_temperature(0, 0.5, 4) == 1.0 and O.query_temperature(2, 0.5, 4) == 1.0
    assert abs(O.query_temperature(3, 0.5, 4) - (1 + 0.5 * math.log(2))) < 1e-15
    assert abs(O.query_temperature(10, 0.5, 4) - (1 + 0.5 * math.log(3))) < 1e-15
    assert abs(O.query_temperature(11, 0.5, 4) - (1 + 0.5 * math.log(4))) < 1e-15
    # router: the largest logits (bias included) win; the weights are the softmax over them alone
    t = {"router": torch.eye(4, dtype=torch.float64), "router.b": torch.tensor([0.0, 0.0, 5.0, 0.0], dtype=torch.float64)}
    h = torch.tensor([[3.0, 1.0, -1.0, 2.0]], dtype=torch.float64)
    idx, w = O.router_choice(h, t, "", {"router": {"experts": 4, "top": 2}})
    assert idx.tolist() == [[2, 0]]
    torch.testing.assert_close(w, torch.softmax(torch.tensor([[4.0, 3.0]], dtype=torch.float64), -1))
    # rotation: base 1 -> angle = position; channel 0 pairs with channel 1
    x = torch.zeros(3, 6, dtype=torch.float64)
    x[:, 0] = 1.0
    x[:, 4] = 5.0
    y = O.rotate_pairs(x, [0, 1, 2], 4, 1.0)
    torch.testing.assert_close(y[2, [0, 1]], torch.tensor([math.cos(2.0), math.sin(2.0)], dtype=torch.float64))
    assert float(y[2, 4]) == 5.0 and float(y[2, 2]) == 0.0
    # attention, one head, one channel, by hand: two tokens, all projections 1
    one = lambda *s: torch.ones(*s, dtype=torch.float64)
    t = {"q": one(1, 1), "q.b": one(1) * 0, "k": one(1, 1), "k.b": one(1) * 0, "v": one(1, 1), "v.b": one(1),
         "r1": one(1) * 2.0, "r2": one(1) * 3.0, "g": one(1, 1) * 0, "o": one(1, 1)}
    h = torch.tensor([[1.0], [2.0]], dtype=torch.float64)
    out = O.attention(h, t, "", {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 1, "scale": 1.0}, 0.0)
    e00 = math.exp(1.0)
    e10, e11 = math.exp(2.0 - 2.0 * math.log(4.0)), math.exp(4.0)
    want0 = 0.5 * e00 * 2.0 / (1 + e00)                       # the 1 in the denominator is the sink
    want1 = 0.5 * (e10 * 2.0 + e11 * 3.0) / (1 + e10 + e11)
    torch.testing.assert_close(out[:, 0], torch.tensor([want0, want1], dtype=torch.float64))
    # layer runs: a stretch in the middle, three passes
    runs = O.layer_runs({"layers": [0] * 4, "loop": {"start": 1, "stop": 3, "times": 3}})
    assert [r[0] for r in runs] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [r[1] for r in runs if r[2]] == [0, 1, 2]


# ------------------------------------------------------------------ other sizes
VARIANTS = {
    # one head, one kv head, one expert chosen of two, one pass, temperature step of one position
    "ones": ([layer(BA, {"kind": "moe", "expert": {"ff": 16}, "shared": {"ff": 8}, "router": {"experts": 2, "top": 1}},
                    heads=1, kv_heads=1, dim=8, vdim=8, q_temp={"coef": 0.2, "every": 1}),
              layer(LA, None, heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=6, q_rank=3, rot={"base": 10.0, "dims": 2})],
             (0, 1, 1)),
    # sizes that are not multiples of 8 or 16, every expert chosen, as many kv heads as heads
    "odd": ([layer(BA, {"kind": "moe", "expert": {"ff": 10}, "router": {"experts": 3, "top": 3}},
                   heads=5, kv_heads=5, dim=6, vdim=10, scale=0.05, softcap=2.0),
             layer(LA, {"kind": "dense", "ff": 50}, heads=5, dim=6, rot_dim=6, vdim=4, kv_rank=13, q_rank=9,
                   rot={"base": 40000.0, "dims": 4}),      # the last pair of the key part is not rotated
             layer(BA, None, heads=3, kv_heads=1, dim=10, vdim=6, q_temp={"coef": 1.5, "every": 7})],
            (1, 3, 2)),
    # wide heads and latents, value size above key size, the stretch of passes at the end
    "wide": ([layer(BA, None, heads=4, kv_heads=1, dim=40, vdim=72, scale=0.5),
              layer(LA, MOE, heads=2, dim=72, rot_dim=40, vdim=80, kv_rank=88, q_rank=60,
                    rot={"base": 1000.0, "dims": 40}),
              layer(BA, MOE, heads=2, kv_heads=2, dim=72, vdim=40)],
             (2, 3, 3)),
}


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_sizes(dev, name):
    layers, loop = VARIANTS[name]
    c, cfg, sd = make(layers, width=40 if name != "wide" else 100, vocab=61, seed=5, eps=1e-3, loop=loop,
                      embed_scale=1.0 if name == "ones" else 2.5, logit_scale=1.0 if name == "ones" else 0.7,
                      logit_softcap=0.0 if name == "odd" else 9.0)
    t = toks(75, cfg.vocab, 3)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    # first part as a prompt, the rest in portions of 1, 2 and 5 tokens
    close(run_cuts(eng, "a", t, [40, 1, 2, 5, 1, 1, 2, 23]), ref)


# ------------------------------------------------------------------ prefill vs decode, portions
@pytest.mark.parametrize("dev", DEVICES)
def test_prefill_decode_and_portions(dev):
    c, cfg, sd = make([layer(BA, MOE), layer(LA, PLAIN), BA, layer(LA, MOE)], seed=6, loop=(0, 2, 2))
    n = 2 * PAGE + 21                      # crosses two page borders
    t = toks(n, cfg.vocab, 4)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "w", t), ref)
    # token by token from the first token on
    close(run_cuts(eng, "d", t, [1] * n), ref)
    # portions of changing size, down to two tokens and one, cut inside pages
    for sizes in ([2] * 20 + [63, 1, 1, 2, 40, 3], [5, 59, 1, 64, 7, 2, 3, 8], [129, 2, 1, 17]):
        close(run_cuts(eng, "p", t, sizes), ref)


# ------------------------------------------------------------------ batches, reuse of pages and slots
@pytest.mark.parametrize("dev", DEVICES)
def test_mixed_batches_and_reuse(dev):
    c, cfg, sd = make([layer(LA, MOE), layer(BA, PLAIN), layer(BA, MOE)], seed=7, loop=(1, 3, 2))
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
def test_first_tokens_in_used_pages(dev):
    """A sequence that starts in pages another one left behind sees none of it: there are no
    keys before position 0, in any pass of a repeated layer; the first token's softmax holds
    its own key and the sink only."""
    c, cfg, sd = make([BA, LA, layer(BA, MOE)], seed=8, loop=(0, 3, 2))
    eng = engine(cfg, sd, dev, pages=3, slots=1)
    a, b = toks(100, cfg.vocab, 20), toks(7, cfg.vocab, 21)
    eng.step([("a", a, [])])
    eng.release("a")
    ref = O.forward(c, sd, b)
    outs = [eng.step([("b", [b[0]], [0])]), eng.step([("b", b[1:3], [0, 1])]), eng.step([("b", b[3:], [0, 1, 2, 3])])]
    close(torch.cat(outs), ref)


# ------------------------------------------------------------------ far keys, page borders, causal edge
def spike_attention(hot, qtok, beta=30.0, seed=11, penalty=True):
    """Biased attention alone whose query projection is rebuilt so that every query of token
    ``qtok`` points along the key of token ``hot``: where ``hot`` is visible it takes nearly
    all the softmax weight, however far back it is (the score is far above the sink's 0 and
    above what the distance penalty takes off)."""
    mx = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 1.0, "softcap": 0.0}
    c, cfg, sd = make([{"type": "attention", "mixer": mx, "mlp": None}], width=32, vocab=50, seed=seed)
    f = lambda k: sd[k].double()
    eps = c["norm"]["eps"]
    H, G, D = mx["heads"], mx["kv_heads"], mx["dim"]
    for b in ("q.b", "k.b"):
        sd["l0.mix." + b] = torch.zeros_like(sd["l0.mix." + b])
    if not penalty:
        sd["l0.mix.r1"] = torch.zeros_like(sd["l0.mix.r1"])
    u = O.rms(f("embed") * c["embedding"]["scale"], eps) * f("l0.norm1")
    k = (f("l0.mix.k") @ u[hot]).view(G, D)
    target = k.repeat_interleave(H // G, 0).reshape(-1)                  # [H * D]
    xq = u[qtok]
    sd["l0.mix.q"] = (target[:, None] * xq[None, :] / (xq @ xq)).to(torch.bfloat16)
    c["layers"][0]["mixer"]["scale"] = beta / float((k[0] * k[0]).sum())
    cfg = Hy.HybridConfig.from_dict(c)
    return c, cfg, sd


def spike_latent(hot, qtok, beta=25.0, seed=12, part="plain"):
    """Latent attention alone, the same construction through the up-projected key
    (``part`` "plain") or through the rotated key part that the heads share ("rot": the score
    then turns with the distance, so the hot key stands out only from nearby)."""
    mx = {"heads": 2, "dim": 16, "rot_dim": 4, "vdim": 8, "kv_rank": 12, "q_rank": 32,
          "rot": {"base": 100.0, "dims": 4}, "scale": 1.0}
    c, cfg, sd = make([{"type": "latent_attention", "mixer": mx, "mlp": None}], width=32, vocab=50, seed=seed)
    f = lambda k: sd[k].double()
    eps = c["norm"]["eps"]
    H, D, Rd, r = mx["heads"], mx["dim"], mx["rot_dim"], mx["kv_rank"]
    u = O.rms(f("embed") * c["embedding"]["scale"], eps) * f("l0.norm1")
    dkv = f("l0.mix.dkv") @ u[hot]
    lat = O.rms(dkv[:r], eps) * f("l0.mix.dkv.norm")
    kp = (f("l0.mix.uk") @ lat).view(H, D)
    target = torch.zeros(H, D + Rd, dtype=torch.float64)
    if part == "plain":
        target[:, :D] = kp
        norm2 = float((kp[0] * kp[0]).sum())
    else:
        target[:, D:] = dkv[r:]
        norm2 = float((dkv[r:] * dkv[r:]).sum())
    # the query latent of qtok, as the engine and the oracle form it
    cq = O.rms(f("l0.mix.dq") @ u[qtok], eps) * f("l0.mix.dq.norm")
    sd["l0.mix.uq"] = (target.reshape(-1)[:, None] * cq[None, :] / (cq @ cq)).to(torch.bfloat16)
    c["layers"][0]["mixer"]["scale"] = beta / norm2
    cfg = Hy.HybridConfig.from_dict(c)
    return c, cfg, sd


@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("kind", ["attention", "latent"])
@pytest.mark.parametrize("n,where", [(3 * PAGE + 9, 0), (3 * PAGE + 9, PAGE - 1), (3 * PAGE + 9, PAGE),
                                     (2 * PAGE + 1, 2 * PAGE - 1), (2 * PAGE + 1, 2 * PAGE), (40, 3)])
def test_far_keys_and_page_borders(dev, n, where, kind):
    """One key among hundreds takes the weight: at the sequence's start, on both sides of page
    borders, as the newest key; in a prompt and when decoding."""
    hot, qtok = 7, 11
    c, cfg, sd = spike_attention(hot, qtok) if kind == "attention" else spike_latent(hot, qtok)
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
def test_rotated_key_part(dev):
    """The shared rotated key part alone carries the score: the engine follows the oracle
    where the score depends on the distance through the rotation, at both sides of a page
    border, decoded and in portions."""
    hot, qtok = 7, 11
    c, cfg, sd = spike_latent(hot, qtok, part="rot")
    n = PAGE + 6
    t = [x if x not in (hot, qtok) else 8 for x in toks(n, cfg.vocab, 33)]
    for where in (n - 1, n - 2, PAGE, PAGE - 1):
        tt = list(t)
        tt[where] = hot
        tt[-1] = qtok if where != n - 1 else hot
        c2, cfg2, sd2 = (c, cfg, sd) if where != n - 1 else spike_latent(hot, hot, part="rot")
        ref = O.forward(c2, sd2, tt)
        eng = engine(cfg2, sd2, dev)
        close(run_whole(eng, "w", tt), ref)
        close(run_cuts(eng, "d", tt, [PAGE - 3, 2, 1, 1, 2, 1, 1, 1]), ref)
    # turning the keys by another base changes the result: the rotation is at work
    other = copy.deepcopy(c)
    other["layers"][0]["mixer"]["rot"]["base"] = 3.0
    assert (O.forward(other, sd, tt) - O.forward(c, sd, tt)).abs().max() > 1e-3


@pytest.mark.parametrize("dev", DEVICES)
def test_causal_edge(dev):
    """The query sees its own key and not the next one: a hot key at the query's place shows,
    one place later it does not (in the oracle and in the engine)."""
    hot = 7
    for build in (spike_attention, spike_latent):
        c2, cfg2, sd2 = build(hot, hot)
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
def test_sink_and_distance_penalty(dev):
    """Scores far below zero: nearly all of the softmax weight goes to the sink and the head
    adds almost nothing; without the 1 in the denominator the result would be another.  A large
    penalty makes all but the newest keys vanish; at distance 0 it takes nothing off."""
    c, cfg, sd = make([layer(BA, None, scale=0.6, softcap=0.0, q_temp=None)], seed=31)
    sd["l0.mix.q.b"] = torch.zeros_like(sd["l0.mix.q.b"])
    sd["l0.mix.k.b"] = torch.zeros_like(sd["l0.mix.k.b"])
    sd["l0.mix.k"] = -sd["l0.mix.q"][: sd["l0.mix.k"].shape[0]].clone()    # q . k < 0 for head 0 of each group
    sd["l0.mix.r1"] = torch.full_like(sd["l0.mix.r1"], 6.0)
    sd["l0.mix.r2"] = torch.full_like(sd["l0.mix.r2"], 4.0)
    t = toks(PAGE + 20, cfg.vocab, 32)
    ref = O.forward(c, sd, t)
    # the same model with the penalty switched off gives other logits: the penalty is at work
    sd0 = dict(sd)
    sd0["l0.mix.r1"] = torch.zeros_like(sd["l0.mix.r1"])
    assert (O.forward(c, sd0, t) - ref).abs().max() > 1e-3
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "a", t), ref)
    close(run_cuts(eng, "b", t, [PAGE - 2, 1, 1, 1, 2, 5, 1]), ref)
    close(run_cuts(engine(cfg, sd0, dev), "c", t, [PAGE + 3, 1, 2]), O.forward(c, sd0, t))


@pytest.mark.parametrize("dev", DEVICES)
def test_temperature_steps_and_score_cap(dev):
    """A temperature that rises steeply every 4 positions and scores well into the flat part of
    the cap: positions on both sides of every step, in prompts, portions of two and decoded."""
    c, cfg, sd = make([layer(BA, None, scale=2.0, softcap=1.5, q_temp={"coef": 3.0, "every": 4})], seed=41)
    t = toks(PAGE + 11, cfg.vocab, 42)
    ref = O.forward(c, sd, t)
    flat = copy.deepcopy(c)
    flat["layers"][0]["mixer"]["q_temp"]["every"] = 5
    assert (O.forward(flat, sd, t)[3] - ref[3]).abs().max() > 1e-3      # position 3 is the first step
    assert (O.forward(flat, sd, t)[2] - ref[2]).abs().max() < 1e-9
    uncapped = copy.deepcopy(c)
    uncapped["layers"][0]["mixer"]["softcap"] = 0.0
    assert (O.forward(uncapped, sd, t) - ref).abs().max() > 1e-2
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "a", t), ref)
    close(run_cuts(eng, "b", t, [2, 1, 1, 2, 2, 3, 1, 1, 1, 1, 2, PAGE - 19, 1, 1, 1, 2]), ref)


# ------------------------------------------------------------------ passes
@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("loop", [None, (0, 3, 1), (0, 1, 3), (2, 3, 2), (0, 3, 2), (1, 2, 4)])
def test_passes(dev, loop):
    """Repeated stretches at the start, in the middle, at the end and over the whole stack: every
    pass keeps keys of its own, the embedding comes back before later passes, every pass has
    its step vector."""
    c, cfg, sd = make([layer(BA, PLAIN), layer(LA, None), layer(BA, MOE)], seed=51, loop=loop)
    t = toks(PAGE + 9, cfg.vocab, 52)
    ref = O.forward(c, sd, t)
    if loop and loop[2] > 1:
        sd2 = dict(sd)
        sd2["loop.step"] = sd["loop.step"].clone()
        sd2["loop.step"][-1] += 0.5
        assert (O.forward(c, sd2, t) - ref).abs().max() > 1e-3
        w = Hy.HybridWeights(cfg, sd, "cpu", torch.float32)
        assert len(w.cache_specs()) == 3 + (loop[1] - loop[0]) * (loop[2] - 1)
    eng = engine(cfg, sd, dev)
    close(run_whole(eng, "a", t), ref)
    close(run_cuts(eng, "b", t, [PAGE - 1, 1, 1, 2, 1, 1, 1, 1, 1]), ref)


# ------------------------------------------------------------------ router
@pytest.mark.parametrize("dev", DEVICES)
@pytest.mark.parametrize("case", ["bias_decides", "all_chosen", "one_of_many"])
def test_router_cases(dev, case):
    moe = {"kind": "moe", "expert": {"ff": 24}, "shared": {"ff": 16},
           "router": {"experts": 6, "top": 6 if case == "all_chosen" else 1 if case == "one_of_many" else 2}}
    c, cfg, sd = make([layer(BA, moe)], seed=23)
    t = toks(60, cfg.vocab, 24)
    base = O.forward(c, sd, t)
    if case == "bias_decides":           # two experts are pushed into every choice; their weights stay a softmax
        b = sd["l0.mlp.router.b"].float()
        b[1] += 20.0
        b[4] += 20.0
        sd["l0.mlp.router.b"] = b.to(torch.bfloat16)
        ref = O.forward(c, sd, t)
        assert (ref - base).abs().max() > 1e-3
        u = O.rms(sd["embed"].double()[torch.tensor(t)] * c["embedding"]["scale"], c["norm"]["eps"])
        idx, _ = O.router_choice(u * sd["l0.norm2"].double(), {k: v.double() for k, v in sd.items()}, "l0.mlp.",
                                 c["layers"][0]["mlp"])
        assert set(idx.reshape(-1).tolist()) == {1, 4}
    else:
        ref = base
    close(run_cuts(engine(cfg, sd, dev), "a", t, [33, 1, 2, 24]), ref)


# ------------------------------------------------------------------ bf16 serving precision
@pytest.mark.parametrize("dev", DEVICES)
def test_bfloat16(dev):
    c, cfg, sd = make([layer(BA, {"kind": "dense", "ff": 96}, heads=8, kv_heads=2, dim=32, vdim=32, scale=0.15),
                       layer(LA, {"kind": "dense", "ff": 96}, heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48,
                             q_rank=64, rot={"base": 1000.0, "dims": 16}, scale=0.1),
                       layer(BA, MOE, heads=4, kv_heads=4, dim=16, vdim=32, scale=0.2)],
                      width=128, vocab=200, seed=13, loop=(0, 2, 2), embed_scale=4.0)
    t = toks(PAGE + 30, cfg.vocab, 50)
    ref = O.forward(c, sd, t)
    eng = engine(cfg, sd, dev, dtype=torch.bfloat16)
    # the experts sit in the last layer only: a choice that rounding moves between two experts
    # with nearly equal logits then changes that row alone, not the keys after it
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
    c, cfg, sd = make([layer(BA, MOE), layer(LA, PLAIN), BA], seed=14, loop=(0, 2, 2))
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
    arrive while others decode, pages are handed back and used again."""
    native = pytest.importorskip("p2p_llm_chat_go_amd.native")
    try:
        native.load()
    except Exception as e:  # noqa: BLE001
        pytest.skip("native runtime not built: %s" % e)
    from p2p_llm_chat_go_amd.engine.sampling import SamplingParams
    from p2p_llm_chat_go_amd.engine.server import EngineServer

    c, cfg, sd = make([layer(LA, MOE), layer(BA, PLAIN), LA], seed=15, loop=(1, 3, 2))
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
    c, cfg, sd = make([layer(BA, MOE), layer(LA, PLAIN), layer(BA, MOE), LA], width=64, seed=16, loop=(1, 3, 2))
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

    c, cfg, sd = make([layer(BA, MOE), LA, layer(BA, PLAIN)], seed=17, loop=(0, 2, 2))
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

    cfg = get_config("tiny-tarunex")
    assert cfg.design == "Tarunex" and cfg.is_moe and not cfg.traits.positions and cfg.loop == (1, 3, 2)
    sd = Hy.random_state_dict(cfg, 3)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    assert registry.is_hybrid_dir(str(tmp_path)) and registry.supports_dtype(str(tmp_path), torch.float32)
    cfg2, w = registry.load_checkpoint(str(tmp_path), "cpu", torch.float32)
    assert cfg2.layers == cfg.layers and cfg2.loop == cfg.loop and cfg2.embed_scale == cfg.embed_scale
    eng = registry.make_engine(cfg2, w, "cpu", kv_pages=6, num_slots=2, max_batch=2, dtype=torch.float32)
    p = toks(9, cfg.vocab, 5)
    r = eng.generate([p], max_new_tokens=4, stop_on_eos=False)[0]
    near_tie(cfg.to_dict(), sd, p, r.tokens, 4)


def test_config_roundtrip_and_errors():
    c, cfg, sd = make([layer(BA, MOE), layer(LA, PLAIN), layer(BA, None)], loop=(0, 2, 2))
    again = Hy.HybridConfig.from_dict(cfg.to_dict())
    assert again.layers == cfg.layers and again.design == "Tarunex" and again.is_moe
    assert (again.loop, again.embed_scale, again.logit_scale, again.logit_softcap) == \
        (cfg.loop, cfg.embed_scale, cfg.logit_scale, cfg.logit_softcap)
    assert set(Hy.tensor_shapes(cfg)) == set(sd) and "pos" not in sd
    assert sd["l0.norm1"].shape == () and sd["final.norm"].shape == () and sd["loop.step"].shape == (2, cfg.width)
    assert "l2.norm2" not in sd and "l1.mlp.shared.gate" not in sd and "l0.mlp.shared.gate" in sd
    assert sd["l0.mix.g"].shape == (6, cfg.width) and sd["l1.mix.dkv"].shape == (24 + 8, cfg.width)
    # every run of a repeated layer keeps a pool of its own
    specs = Hy.HybridWeights(cfg, sd, "cpu", torch.float32).cache_specs()
    assert [s[1] for s in specs] == [2 * (16 + 24), 24 + 8, 2 * (16 + 24), 24 + 8, 2 * (16 + 24)]
    bad = dict(sd)
    bad["l0.mix.r1"] = bad["l0.mix.r1"][:2]
    with pytest.raises(ValueError):
        Hy.HybridWeights(cfg, bad, "cpu", torch.float32)
    with pytest.raises(KeyError):
        Hy.HybridWeights(cfg, {k: v for k, v in sd.items() if k != "loop.step"}, "cpu", torch.float32)
    for loop in ((2, 2, 2), (0, 4, 2), (1, 2, 0)):
        with pytest.raises(ValueError):
            make([BA, LA, BA], loop=loop)
    with pytest.raises(ValueError):       # more experts chosen than there are
        make([layer(BA, dict(MOE, router={"experts": 3, "top": 4}))])
    with pytest.raises(ValueError):       # heads that do not split over the key/value heads
        Hy.HybridWeights(*make([layer(BA, None, heads=5, kv_heads=2)])[1:], "cpu", torch.float32)
    eng = engine(cfg, sd, "cpu", pages=2, slots=1)
    eng.step([("a", [1, 2, 3], [2])])
    with pytest.raises(MemoryError):
        eng.step([("b", [1], [0])])          # no second state slot
    with pytest.raises(MemoryError):
        eng.step([("a", [1] * PAGE, [])])    # no second page
