"""Plain, slow PyTorch rendering of the Tarunex decoder, one function per mechanism.

Everything runs with explicit loops over tokens, heads and keys in one precision (float64 by
default), straight from the equations; it shares nothing with the engine's model, cache or
kernels.  A model is a ``config`` dict (the keys of a Tarunex ``config.json``) and a dict of
tensors named as in its checkpoint.

Layer:  x <- x + mixer(N(x) g1) + ff(N(x) g2), g1 and g2 one number each.
Stack:  layers [start, stop) run ``times`` passes in a row with the same weights; before pass
t > 0 the embedding output is added to x, before every pass the row t of ``loop.step``.
"""
from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------ rotation
def rotate_pairs(x, positions, dims, base):
    """x [T, ..., n]: channels (2i, 2i+1), i < dims/2, turned by position * base^(-2i/dims)."""
    out = x.clone()
    for s, p in enumerate(positions):
        for i in range(dims // 2):
            a = p * base ** (-2.0 * i / dims)
            c, sn = math.cos(a), math.sin(a)
            u, v = x[s, ..., 2 * i], x[s, ..., 2 * i + 1]
            out[s, ..., 2 * i] = u * c - v * sn
            out[s, ..., 2 * i + 1] = v * c + u * sn
    return out


# ------------------------------------------------------------------ latent attention
def latent_attention(h, t, p, mx, eps):
    """Queries through a normed low-rank latent; keys and values as up-projections of a normed
    latent per token plus one rotated key part that all heads share; plain causal softmax;
    one sigmoid gate per head."""
    H, D, Rd, V, rank = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    T = h.shape[0]
    pos = list(range(T))
    cq = rms(h @ t[p + "dq"].T, eps) * t[p + "dq.norm"]
    q = (cq @ t[p + "uq"].T).view(T, H, D + Rd)
    q_plain = q[:, :, :D]
    q_rot = rotate_pairs(q[:, :, D:], pos, mx["rot"]["dims"], float(mx["rot"]["base"]))
    dkv = h @ t[p + "dkv"].T
    c = rms(dkv[:, :rank], eps) * t[p + "dkv.norm"]
    k_rot = rotate_pairs(dkv[:, rank:], pos, mx["rot"]["dims"], float(mx["rot"]["base"]))   # [T, Rd]
    k_plain = (c @ t[p + "uk"].T).view(T, H, D)
    v = (c @ t[p + "uv"].T).view(T, H, V)
    gate = torch.sigmoid(h @ t[p + "g"].T)                                                   # [T, H]
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for s in range(T):
        for hd in range(H):
            sc = (k_plain[:s + 1, hd] @ q_plain[s, hd] + k_rot[:s + 1] @ q_rot[s, hd]) * float(mx["scale"])
            w = torch.softmax(sc, 0)
            out[s, hd] = (w[:, None] * v[:s + 1, hd]).sum(0) * gate[s, hd]
    return out.reshape(T, H * V) @ t[p + "o"].T


# ------------------------------------------------------------------ attention
def query_temperature(position, coef, every):
    return 1.0 + coef * math.log(math.floor((position + 1) / every) + 1)


def attention(h, t, p, mx, eps):
    """Grouped-query attention with biased projections, no rotation: position-dependent query
    temperature, tanh-capped scores, a logarithmic distance penalty per head, a softmax whose
    denominator holds one more 1, one sigmoid gate per head."""
    H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    q = (h @ t[p + "q"].T + t[p + "q.b"]).view(T, H, D)
    k = (h @ t[p + "k"].T + t[p + "k.b"]).view(T, G, D)
    v = (h @ t[p + "v"].T + t[p + "v.b"]).view(T, G, V)
    qt = mx.get("q_temp")
    cap = float(mx.get("softcap") or 0.0)
    gate = torch.sigmoid(h @ t[p + "g"].T)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for s in range(T):
        temp = query_temperature(s, float(qt["coef"]), int(qt["every"])) if qt else 1.0
        for hd in range(H):
            g = hd // (H // G)
            sc = (k[:s + 1, g] @ (q[s, hd] * temp)) * float(mx["scale"])
            if cap:
                sc = cap * torch.tanh(sc / cap)
            dist = torch.arange(s, -1, -1, dtype=h.dtype)
            sc = sc - t[p + "r1"][hd] * torch.log(1.0 + t[p + "r2"][hd] * dist)
            e = torch.exp(sc)
            w = e / (1.0 + e.sum())
            out[s, hd] = (w[:, None] * v[:s + 1, g]).sum(0) * gate[s, hd]
    return out.reshape(T, H * V) @ t[p + "o"].T


MIXERS = {"latent_attention": latent_attention, "attention": attention}


# ------------------------------------------------------------------ feed-forward
def gated_unit(h, t, p):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def router_choice(h, t, p, mlp):
    """Per token: the ``top`` experts with the largest logits and the softmax over just those."""
    z = h @ t[p + "router"].T + t[p + "router.b"]
    val, idx = torch.topk(z, int(mlp["router"]["top"]), dim=-1)
    return idx, torch.softmax(val, -1)


def mixture(h, t, p, mlp):
    idx, w = router_choice(h, t, p, mlp)
    out = torch.zeros_like(h)
    for s in range(h.shape[0]):
        for e, we in zip(idx[s].tolist(), w[s]):
            out[s] += we * gated_unit(h[s:s + 1], t, p + "e%d." % e)[0]
    if mlp.get("shared"):
        out = out + gated_unit(h, t, p + "shared.")
    return out


def feed_forward(h, t, p, mlp):
    if mlp.get("kind", "moe") == "moe":
        return mixture(h, t, p, mlp)
    return gated_unit(h, t, p)


# ------------------------------------------------------------------ model
def layer_runs(config):
    """Layer indices in the order they run, with (pass number, first of its pass) for the
    layers of the repeated stretch and (None, False) for the others."""
    n = len(config["layers"])
    lp = config.get("loop")
    if not lp or int(lp["times"]) < 1:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    runs = [(i, None, False) for i in range(a)]
    for tt in range(times):
        runs += [(i, tt, i == a) for i in range(a, b)]
    return runs + [(i, None, False) for i in range(b, n)]


def forward(config, t, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of one sequence run from position 0."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in t.items()}
    eps = float(config["norm"]["eps"])
    x0 = t["embed"][torch.tensor(tokens)] * float(config["embedding"]["scale"])
    x = x0.clone()
    for i, tt, first in layer_runs(config):
        if first:
            if tt > 0:
                x = x + x0
            x = x + t["loop.step"][tt]
        L, p = config["layers"][i], "l%d." % i
        u = rms(x, eps)
        y = MIXERS[L["type"]](u * t[p + "norm1"], t, p + "mix.", L["mixer"], eps)
        if L.get("mlp"):
            y = y + feed_forward(u * t[p + "norm2"], t, p + "mlp.", L["mlp"])
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    z = (rms(x, eps) * t["final.norm"]) @ t["head"].T * float(config.get("logit_scale", 1.0))
    cap = float(config.get("logit_softcap") or 0.0)
    return cap * torch.tanh(z / cap) if cap else z
