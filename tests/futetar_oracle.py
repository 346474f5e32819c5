"""Plain, slow PyTorch rendering of the Futetar decoder, one function per mechanism.

Everything runs token by token (or with explicit loops over keys) in one precision (float64
by default), straight from the equations; it shares nothing with the engine's model, cache
or kernels.  A model is a ``config`` dict (the keys of a Futetar ``config.json``) and a dict
of tensors named as in its checkpoint.

Layer:  u = N(x) (1 + w);  x <- x + mixer(u) + ff(u)   (one norm feeds both sublayers).
"""
from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------ matrix memory (mLSTM)
def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


def mlstm(h, t, p, mx, eps):
    """Per head a dim x vdim memory C, a normaliser n and a running maximum m of the log
    gates; C, n and m start at zero."""
    H, D, V, cap = mx["heads"], mx["dim"], mx["vdim"], float(mx["gate_cap"])
    T = h.shape[0]
    q = (h @ t[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ t[p + "k"].T).view(T, H, D)
    v = (h @ t[p + "v"].T).view(T, H, V)
    ig = soft_cap(h @ t[p + "i"].T + t[p + "i.b"], cap)                       # log input gate
    fg = torch.nn.functional.logsigmoid(soft_cap(h @ t[p + "f"].T + t[p + "f.b"], cap))
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        C = torch.zeros(D, V, dtype=h.dtype)
        n = torch.zeros(D, dtype=h.dtype)
        m = 0.0
        for s in range(T):
            i_, f_ = float(ig[s, hd]), float(fg[s, hd])
            m_new = max(f_ + m, i_)
            a, b = math.exp(f_ + m - m_new), math.exp(i_ - m_new)
            C = a * C + b * torch.outer(k[s, hd], v[s, hd])
            n = a * n + b * k[s, hd]
            m = m_new
            den = max(abs(float(n @ q[s, hd])), math.exp(-m)) + 1e-6
            out[s, hd] = (C.T @ q[s, hd]) / den
    o = rms(out, eps).reshape(T, H * V) * t[p + "norm"]
    o = o * torch.sigmoid(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


# ------------------------------------------------------------------ attention
def scaled_freqs(rot):
    """f_i = base^(-2i/dims), long wavelengths slowed by ``factor``, a linear blend between."""
    dims, base = rot["dims"], float(rot["base"])
    sc = rot.get("scaling")
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            fac, lo, hi, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wl = 2.0 * math.pi / f
            if wl < orig / hi:
                pass
            elif wl > orig / lo:
                f = f / fac
            else:
                s = (orig / wl - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return out


def rotate_half(x, rot):
    """x [T, heads, dim]: channel i pairs with channel i + dims/2 among the first dims."""
    dims = rot["dims"]
    half = dims // 2
    fr = scaled_freqs(rot)
    out = x.clone()
    for s in range(x.shape[0]):
        for i in range(half):
            a = s * fr[i]
            c, sn = math.cos(a), math.sin(a)
            u, v = x[s, :, i], x[s, :, i + half]
            out[s, :, i] = u * c - v * sn
            out[s, :, i + half] = v * c + u * sn
    return out


def keys_values(h, t, p, mx, eps):
    """What a layer with projections of its own leaves for itself and for layers that borrow."""
    G, D, V = mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    k = rms((h @ t[p + "k"].T).view(T, G, D), eps) * t[p + "k.norm"]
    k = rotate_half(k, mx["rot"]) if mx.get("rot") else k
    return k, (h @ t[p + "v"].T).view(T, G, V)


def attention(h, t, p, mx, eps, kv):
    H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    T = h.shape[0]
    k, v = kv
    q = rms((h @ t[p + "q"].T).view(T, H, D), eps) * t[p + "q.norm"]
    q = rotate_half(q, mx["rot"]) if mx.get("rot") else q
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for s in range(T):
        for hd in range(H):
            g = hd // (H // G)
            sc = (k[:s + 1, g] @ q[s, hd]) * float(mx["scale"])
            w = torch.softmax(sc, 0)
            out[s, hd] = w @ v[:s + 1, g]
    return out.reshape(T, H * V) @ t[p + "o"].T


# ------------------------------------------------------------------ feed-forwards
def dense_ff(h, t, p, ml):
    return (gelu_tanh(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def relu2_expert(h, up, down):
    return (torch.relu(h @ up.T) ** 2) @ down.T


def route(z, corr, r):
    """z: router logits of one token (real experts first, identity experts last).  Returns
    [(expert, weight)]."""
    n, top = z.numel(), r["top"]
    s = torch.softmax(z, 0)
    c = s + corr
    g = r.get("groups") or {}
    count = int(g.get("count", 1))
    keep = int(g.get("keep", count))
    per = n // count
    best = sorted(range(count), key=lambda j: (-float(c[j * per:(j + 1) * per].max()), j))[:keep]
    ok = [e for e in range(n) if e // per in best]
    chosen = sorted(ok, key=lambda e: (-float(c[e]), e))[:top]
    return [(e, s[e]) for e in chosen]


def moe_ff(h, t, p, ml):
    """The router has ``experts`` + ``identity`` outputs; the last ``identity`` of them stand
    for experts that hand their input back."""
    r = ml["router"]
    n_real = int(r["experts"])
    out = torch.zeros_like(h)
    z = h @ t[p + "router"].T
    assert z.shape[1] == n_real + int(r.get("identity", 0))
    for s in range(h.shape[0]):
        for e, w in route(z[s], t[p + "correction"], r):
            if e >= n_real:
                out[s] += w * h[s]
            else:
                out[s] += w * relu2_expert(h[s], t[p + "e%d.up" % e], t[p + "e%d.down" % e])
    if ml.get("shared"):
        sh = relu2_expert(h, t[p + "shared.up"], t[p + "shared.down"])
        out = out + sh * torch.sigmoid(h @ t[p + "shared.sg"].T)
    return out


# ------------------------------------------------------------------ model
def forward(config, tensors, tokens, return_layers=False, dtype=torch.float64):
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(config["norm"]["eps"])
    x = t["embed"][torch.tensor(tokens)]
    kept, layers = {}, []
    for i, L in enumerate(config["layers"]):
        p = "l%d." % i
        u = norm_one_plus(x, t[p + "norm1"], eps)
        mx = L["mixer"]
        if L["type"] == "mlstm":
            m = mlstm(u, t, p + "mix.", mx, eps)
        elif L["type"] == "attention":
            if mx.get("kv_from") is None:
                kept[i] = keys_values(u, t, p + "mix.", mx, eps)
                kv = kept[i]
            else:
                kv = kept[int(mx["kv_from"])]
            m = attention(u, t, p + "mix.", mx, eps, kv)
        else:
            raise KeyError(L["type"])
        ml = L.get("mlp")
        if ml is None:
            f = 0.0
        elif ml.get("kind", "dense") == "dense":
            f = dense_ff(u, t, p + "mlp.", ml)
        else:
            f = moe_ff(u, t, p + "mlp.", ml)
        x = x + (m + f)
        layers.append(x.clone())
    logits = norm_one_plus(x, t["final.norm"], eps) @ t["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits
