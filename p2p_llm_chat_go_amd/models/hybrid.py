"""Hybrid decoders: a configurable stack of sequence mixers on an fp32 residual stream.

A model is a list of layers; each layer has one *mixer* (registered in ``MIXERS``) and
optionally a feed-forward (``FEEDFORWARDS``).  A design (``DESIGNS``) fixes how a sublayer f
is wrapped around the residual stream,

    "sandwich"    x <- x + scale * norm_b(f(norm_a(x)))      RMS norms, per-channel layer scale
    "gated_post"  x <- x + norm(f(x) * sigmoid(R x + b))     no norm on the way in; the norm
                                                             on the way out is taken in
                                                             equal parts of the vector
    "parallel"    x <- x + mixer(u) + ff(u),  u = norm(x)    one norm per layer feeds both
                                                             sublayers
    "parallel2"   x <- x + mixer(norm1(x)) + ff(norm2(x))    a norm per sublayer, each with
                                                             one weight for all channels; a
                                                             stretch of layers may run several
                                                             passes (``loop``)

and whether learned absolute positions are added to the token embedding.  Mixers:

  ``general_delta``     generalized delta rule: per head a D x D state with per-channel decay
                        and an in-context removal of the unit key direction;
  ``mamba2``            Mamba-2 selective state space (short causal convolution + scan);
  ``latent_attention``  attention over a cached low-rank latent per token (keys and values
                        are up-projections of it), causal sliding window, softmax with a
                        learned per-head sink, sigmoid output gate, no positional rotation;
  ``window_attention``  grouped-query attention over cached keys and values: RMS norm of the
                        whole query / key projection, rotary positions on adjacent channel pairs of the
                        first channels of each head, causal sliding window, softmax sink;
  ``gated_delta``       gated delta rule: short causal convolutions + silu on q, k, v, unit
                        keys, a per-channel decay and a write that corrects what the key reads;
  ``hgrn2``             gated linear attention: the write strength is 1 - forget gate;
  ``mlstm``             matrix memory of the xLSTM: exponential input gate, sigmoid forget gate,
                        both in the log domain under a running maximum, and a normaliser state;
  ``attention``         causal grouped-query attention with an ordinary softmax: RMS norm of
                        every query / key head (one weight shared by the heads), rotary
                        positions on channel pairs (i, i + dims/2) with optional stretching of
                        the long wavelengths; a layer may read an earlier layer's keys and
                        values (``kv_from``) instead of projecting its own;
  ``biased_attention``  causal grouped-query attention without rotation: biased projections, a
                        query temperature that grows with the logarithm of the position, capped
                        scores, a logarithmic distance penalty per head, a softmax sink with
                        score 0, one sigmoid gate per head;
  ``rope_latent_attention``  latent attention with low-rank queries and one rotated key part
                        that the heads share, cached beside the latent; plain causal softmax, one
                        sigmoid gate per head;
  ``parallel``          two mixers side by side on the same input, summed with fixed scales.

Feed-forwards: ``dense`` (silu-gated, or the clamped gated unit when the config gives a
limit), ``moe`` (sigmoid router, choice limited to the best groups of experts), ``moe_softmax``
and ``moe_top`` (biased router, softmax over the chosen logits, silu-gated experts, shared expert).
A design may give a config's ``type`` / ``kind`` names a meaning of its own (``Design.mixers``,
``Design.ff``).

"Regesun" stacks the first three mixers in the sandwich form with learned positions;
"Rotutar" stacks ``parallel`` (window attention beside the gated delta rule) and ``hgrn2``
layers in the gated post-norm form, without positions other than the rotation, and caps
its logits with a tanh.  "Futetar" stacks ``mlstm`` and ``attention`` layers in the parallel
form (norm weights stored around zero), with gelu-gated dense feed-forwards and mixtures of
squared-relu experts behind a softmax router.  "Tarunex" stacks ``biased_attention`` and
``rope_latent_attention`` layers (its config calls them "attention" and "latent_attention") in
the two-norm parallel form with ``moe_top`` feed-forwards, repeats a stretch of layers, scales
its embedding and scales and caps its logits.  A checkpoint is a ``config.json`` whose
``architecture`` names the design and one safetensors file (``load_dir``).

One ``forward`` serves every step: a flat list of token rows cut into entries (portions of
prompts and single decoded tokens side by side, ``StepBatch``); attention layers read and
write the paged latent pool, recurrent layers their sequence's state slot
(``engine.seq_cache``).  Matrix products are vendor GEMMs (``torch.nn.functional.linear``,
bf16 with fp32 accumulation or true fp32); everything between them runs on the kernels of
``ops.seqmix``.  Sums over the residual, norms, scores, softmax, decays, gates of the
recurrences and the states stay in fp32 in both precisions.
"""
from __future__ import annotations

import dataclasses
import json
import os

import torch
import torch.nn.functional as F

from ..ops import PAGE
from ..ops import seqmix as sm


# ---------------------------------------------------------------------------- config
@dataclasses.dataclass(frozen=True)
class LayerSpec:
    kind: str
    mixer: dict
    mlp: dict | None


@dataclasses.dataclass(frozen=True)
class Design:
    block: str                # how sublayers sit on the residual stream: "sandwich" | "gated_post" | "parallel"
    positions: str | None     # "learned": a position table is added to the embedding
    norm_offset: float = 0.0  # block and final norm weights are stored minus this (1: around zero)
    ff: tuple = ()            # (config kind, FEEDFORWARDS key) where the two differ
    mixers: tuple = ()        # (config type, MIXERS key) where the two differ
    scalar_norms: bool = False  # block and final norms have one weight for all channels

    def ff_key(self, kind: str) -> str:
        return dict(self.ff).get(kind, kind)

    def mixer_key(self, kind: str) -> str:
        return dict(self.mixers).get(kind, kind)


DESIGNS = {"Regesun": Design("sandwich", "learned"), "Rotutar": Design("gated_post", None),
           "Futetar": Design("parallel", None, norm_offset=1.0,
                             ff=(("dense", "dense_gelu"), ("moe", "moe_softmax"))),
           "Tarunex": Design("parallel2", None, scalar_norms=True, ff=(("moe", "moe_top"),),
                             mixers=(("latent_attention", "rope_latent_attention"),
                                     ("attention", "biased_attention")))}
NO_POS_LIMIT = 1 << 30


@dataclasses.dataclass(frozen=True)
class HybridConfig:
    name: str
    width: int
    vocab: int
    layers: tuple
    eps: float = 1e-5
    max_pos: int = 2048
    bos_id: int = 1
    eos_ids: tuple = ()
    is_moe: bool = False
    design: str = "Regesun"
    norm_groups: int = 1
    logit_softcap: float = 0.0
    logit_scale: float = 1.0
    embed_scale: float = 1.0
    loop: tuple | None = None   # (start, stop, times): layers start .. stop-1 run `times` passes

    @property
    def traits(self) -> Design:
        return DESIGNS[self.design]

    def runs(self) -> list:
        """The layers in the order they run: (layer, pass, first of its pass) per layer run; a
        layer outside the repeated stretch has pass None.  Every run has a cache of its own,
        addressed by its place in this list."""
        n = len(self.layers)
        if not self.loop:
            return [(i, None, False) for i in range(n)]
        a, b, times = self.loop
        runs = [(i, None, False) for i in range(a)]
        for t in range(times):
            runs += [(i, t, i == a) for i in range(a, b)]
        return runs + [(i, None, False) for i in range(b, n)]

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def hidden(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, c: dict, name: str | None = None) -> "HybridConfig":
        layers = tuple(LayerSpec(L["type"], dict(L["mixer"]), dict(L["mlp"]) if L.get("mlp") else None)
                       for L in c["layers"])
        design = str(c.get("architecture", "Regesun"))
        if design not in DESIGNS:
            raise KeyError("unknown design %r (known: %s)" % (design, ", ".join(sorted(DESIGNS))))
        for L in layers:
            if DESIGNS[design].mixer_key(L.kind) not in MIXERS:
                raise KeyError("unknown mixer %r (known: %s)" % (L.kind, ", ".join(sorted(MIXERS))))
            if L.mlp is not None and DESIGNS[design].ff_key(L.mlp.get("kind", "dense")) not in FEEDFORWARDS:
                raise KeyError("unknown feed-forward kind %r" % L.mlp.get("kind"))
        eos = c.get("eos_token_id", ())
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        width, groups = int(c["width"]), int(c["norm"].get("groups", 1))
        if groups < 1 or width % groups:
            raise ValueError("width %d does not split into %d norm groups" % (width, groups))
        max_pos = int(c["max_positions"]) if DESIGNS[design].positions else \
            int(c.get("max_positions", NO_POS_LIMIT))
        loop = None
        if c.get("loop"):
            loop = (int(c["loop"]["start"]), int(c["loop"]["stop"]), int(c["loop"]["times"]))
            if not 0 <= loop[0] < loop[1] <= len(layers) or loop[2] < 1:
                raise ValueError("loop over layers %d .. %d, %d times, of %d layers"
                                 % (loop[0], loop[1] - 1, loop[2], len(layers)))
            if DESIGNS[design].block != "parallel2":
                raise ValueError("design %s does not repeat layers" % design)
        return cls(name=name or design.lower(), width=width,
                   vocab=int(c["vocab"]), layers=layers, eps=float(c["norm"]["eps"]),
                   max_pos=max_pos, bos_id=int(c.get("bos_token_id", 1)),
                   eos_ids=eos, design=design, norm_groups=groups,
                   logit_softcap=float(c.get("logit_softcap") or 0.0),
                   logit_scale=float(c.get("logit_scale", 1.0)),
                   embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)), loop=loop,
                   is_moe=any(L.mlp is not None and L.mlp.get("kind") == "moe" for L in layers))

    def resolve(self, shapes: dict) -> "HybridConfig":
        """Fill the sizes that a config leaves to the checkpoint's tensor shapes (the ranks of
        low-rank projections).  shapes: tensor name -> shape."""
        layers = []
        for i, L in enumerate(self.layers):
            mx = MIXERS[self.traits.mixer_key(L.kind)].resolve_spec(dict(L.mixer), "l%d.mix." % i, shapes)
            layers.append(LayerSpec(L.kind, mx, L.mlp))
        return dataclasses.replace(self, layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": self.design, "width": self.width, "vocab": self.vocab,
             "norm": {"eps": self.eps, "groups": self.norm_groups},
             "layers": [{"type": L.kind, "mixer": L.mixer, "mlp": L.mlp} for L in self.layers]}
        if self.traits.positions or self.max_pos != NO_POS_LIMIT:
            d["max_positions"] = self.max_pos
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.logit_scale != 1.0:
            d["logit_scale"] = self.logit_scale
        if self.embed_scale != 1.0:
            d["embedding"] = {"scale": self.embed_scale}
        if self.loop:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return d


def _vec(t, dev):
    return t.to(dev).float().contiguous()


# ---------------------------------------------------------------------------- step batch
class StepBatch:
    """Device-side description of one step (see ``ops.seqmix`` for the conventions).

    entries: list of (slot, pages, start, tokens) -- a sequence's state slot, its page list,
    the position of its first token in this step and the tokens.  want: per entry the
    indices (within its tokens) whose logits are needed."""

    def __init__(self, entries: list, want: list, device, min_pages: int = 1):
        host, meta = self.build_host(entries, want, min_pages)
        self._adopt(host.to(device), meta)

    @staticmethod
    def build_host(entries: list, want: list, min_pages: int = 1):
        """All of the step's metadata as one int32 host tensor + how to cut it."""
        ids, pos, row_ent, rows, ent, outs = [], [], [], [], [], []
        maxp = max([min_pages] + [len(e[1]) for e in entries])
        bt = torch.zeros(len(entries), maxp, dtype=torch.int32)
        r0 = 0
        for i, (slot, pages, start, toks) in enumerate(entries):
            n = len(toks)
            if n < 1:
                raise ValueError("an entry needs at least one token")
            if (start + n + PAGE - 1) // PAGE > len(pages):
                raise ValueError("entry %d: %d pages do not hold %d tokens" % (i, len(pages), start + n))
            bt[i, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
            ids += list(toks)
            pos += range(start, start + n)
            row_ent += [i] * n
            rows += [pages[p // PAGE] * PAGE + p % PAGE for p in range(start, start + n)]
            ent.append((r0, n, start, slot))
            outs += [r0 + w for w in want[i]]
            r0 += n
        parts = [torch.tensor(x, dtype=torch.int32).reshape(-1)
                 for x in (ids, pos, row_ent, rows, ent, outs or [0])] + [bt.reshape(-1)]
        meta = {"R": r0, "E": len(entries), "ent_host": ent, "n_out": len(outs),
                "max_pos": max(pos), "maxp": maxp, "sizes": [p.numel() for p in parts]}
        return torch.cat(parts), meta

    def _adopt(self, flat, meta):
        """flat: the device copy of ``build_host``'s tensor (one host -> device copy)."""
        self.flat, self.meta = flat, meta
        self.R, self.E = meta["R"], meta["E"]
        self.ent_host, self.n_out, self.max_pos = meta["ent_host"], meta["n_out"], meta["max_pos"]
        # most keys any row of this step can see; a batch that is reloaded for a captured
        # graph reports the whole width of its block tables instead
        self.max_keys = meta["max_pos"] + 1
        cut, o = [], 0
        for n in meta["sizes"]:
            cut.append(flat[o:o + n])
            o += n
        self.ids, self.pos, self.row_ent, self.cache_rows = cut[0], cut[1], cut[2], cut[3]
        self.ent = cut[4].view(-1, 4)
        self.out_rows = cut[5][:self.n_out]
        self.block_tables = cut[6].view(meta["E"], meta["maxp"])
        self._units = {}

    def reload(self, entries: list, want: list):
        """Same shape of step (rows, entries, wanted rows, table width), new contents, written
        into the device tensors this batch already has (a captured graph reads them)."""
        host, meta = self.build_host(entries, want, self.meta["maxp"])
        if meta["sizes"] != self.meta["sizes"] or meta["maxp"] != self.meta["maxp"]:
            raise ValueError("a reloaded step must have the shape of the captured one")
        self.flat.copy_(host, non_blocking=True)
        self.ent_host, self.max_pos = meta["ent_host"], meta["max_pos"]
        self.meta = meta

    def units(self, rows_per_wave: int):
        """Row groups for the matrix-core attention kernel (``ops.seqmix.make_units``)."""
        u = self._units.get(rows_per_wave)
        if u is None:
            u = self._units[rows_per_wave] = sm.make_units(self.ent_host, rows_per_wave).to(
                self.ids.device)
        return u


# ---------------------------------------------------------------------------- mixers
class Mixer:
    """One sequence mixer: weights + forward on a step.  ``cache_spec`` tells the sequence
    cache what the layer keeps between steps."""
    kind = ""

    def __init__(self, spec: dict, width: int, eps: float):
        self.spec, self.width, self.eps = spec, width, eps

    @staticmethod
    def resolve_spec(spec: dict, prefix: str, shapes: dict) -> dict:
        """Sizes that the checkpoint's tensor shapes give rather than the config."""
        return spec

    def tensor_shapes(self) -> dict:
        raise NotImplementedError

    def load(self, get, dtype, dev):
        raise NotImplementedError

    def cache_spec(self):
        """("paged", width) | ("state", {name: shape}) | a list of those | None."""
        return None

    # A mixer either implements ``forward`` (it projects its input itself), or exposes the
    # rows that read the layer input as ``w_in`` and implements ``mix`` on their product, so
    # that whoever owns the input (a layer with a gate, a ``parallel`` mixer) can run every
    # projection of the same input as one matrix product.
    w_in = None
    b_in = None   # bias of the input product (activation type), or None
    wo = None
    n_mid = 0

    def mix(self, proj, b: "StepBatch", cache, layer: int, out, out_scale: float = 1.0):
        """proj [R, rows of w_in] -> out [R, n_mid] (the input of the output projection)."""
        raise NotImplementedError

    def forward_proj(self, proj, b: "StepBatch", cache, layer: int):
        mid = torch.empty(b.R, self.n_mid, device=proj.device, dtype=proj.dtype)
        return F.linear(self.mix(proj, b, cache, layer, mid), self.wo)

    def forward(self, h, b: "StepBatch", cache, layer: int):
        return self.forward_proj(F.linear(h, self.w_in, self.b_in), b, cache, layer)


class GeneralDelta(Mixer):
    kind = "general_delta"
    LOW_RANK = 32

    @staticmethod
    def resolve_spec(spec, prefix, shapes):
        if "decay_rank" not in spec and prefix + "w1" in shapes:
            spec["decay_rank"] = int(tuple(shapes[prefix + "w1"])[0])
        return spec

    def tensor_shapes(self):
        n, W = self.spec["heads"] * self.spec["dim"], self.width
        lr = int(self.spec.get("decay_rank", self.LOW_RANK))
        return {"r": (n, W), "k": (n, W), "v": (n, W), "g": (n, W), "a": (n, W), "a.b": (n,),
                "w1": (lr, W), "w2": (n, lr), "w0": (n,), "norm": (n,), "o": (W, n)}

    def load(self, get, dtype, dev):
        self.H, self.D = int(self.spec["heads"]), int(self.spec["dim"])
        self.n = self.H * self.D
        # one projection for everything that reads the layer input: r | k | v | g | a | w1
        self.w_in = torch.cat([get(k) for k in ("r", "k", "v", "g", "a", "w1")], 0).to(dev, dtype).contiguous()
        self.w2 = get("w2").to(dev, dtype).contiguous()
        self.w0, self.ab, self.normw = _vec(get("w0"), dev), _vec(get("a.b"), dev), _vec(get("norm"), dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("state", {"S": (self.H, self.D, self.D)})

    def forward(self, h, b, cache, layer):
        n = self.n
        proj = F.linear(h, self.w_in)
        low = proj[:, 5 * n:]
        sm.tanh_(low)
        lo = F.linear(low, self.w2)
        out = torch.empty(b.R, n, device=h.device, dtype=h.dtype)
        sm.gdelta_scan(proj[:, 0:n], proj[:, n:2 * n], proj[:, 2 * n:3 * n], proj[:, 3 * n:4 * n],
                       proj[:, 4 * n:5 * n], lo, self.w0, self.ab, self.normw,
                       cache.state[layer]["S"], b.ent, b.ent_host, out, self.H, self.D, self.eps)
        return F.linear(out, self.wo)


class Mamba2(Mixer):
    kind = "mamba2"

    def _dims(self):
        s = self.spec
        self.H, self.P, self.N, self.G = int(s["heads"]), int(s["vdim"]), int(s["state"]), int(s["groups"])
        self.K, self.ng = int(s["conv"]), int(s.get("norm_groups", 1))
        self.inner = self.H * self.P
        self.C = self.inner + 2 * self.G * self.N

    def tensor_shapes(self):
        self._dims()
        return {"in": (2 * self.inner + 2 * self.G * self.N + self.H, self.width),
                "conv": (self.C, self.K), "conv.b": (self.C,), "dt_bias": (self.H,),
                "A_log": (self.H,), "D": (self.H,), "norm": (self.inner,),
                "o": (self.width, self.inner)}

    def load(self, get, dtype, dev):
        self._dims()
        if self.H % self.G or self.inner % self.ng:
            raise ValueError("mamba2: heads %d / groups %d / norm groups %d do not divide"
                             % (self.H, self.G, self.ng))
        self.w_in = get("in").to(dev, dtype).contiguous()
        self.cw, self.cb = _vec(get("conv"), dev), _vec(get("conv.b"), dev)
        self.dt_bias, self.A_log, self.Dp = (_vec(get(k), dev) for k in ("dt_bias", "A_log", "D"))
        self.normw = _vec(get("norm"), dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("state", {"S": (self.H, self.N, self.P), "tail": (self.K - 1, self.C)})

    def forward(self, h, b, cache, layer):
        st = cache.state[layer]
        zx = F.linear(h, self.w_in)
        conv = torch.empty(b.R, self.C, device=h.device, dtype=torch.float32)
        sm.mamba_conv(zx, self.inner, self.cw, self.cb, st["tail"], b.ent, b.ent_host, b.row_ent, conv)
        y = torch.empty(b.R, self.inner, device=h.device, dtype=torch.float32)
        sm.mamba_scan(conv, zx, self.inner, self.inner + self.C, self.dt_bias, self.A_log, self.Dp,
                      st["S"], st["tail"], b.ent, b.ent_host, y, self.H, self.P, self.N, self.G)
        yn = torch.empty(b.R, self.inner, device=h.device, dtype=h.dtype)
        sm.rmsnorm(y, self.normw, self.eps, yn, parts=self.ng)
        return F.linear(yn, self.wo)


class LatentAttention(Mixer):
    kind = "latent_attention"

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V, self.rank = int(s["heads"]), int(s["dim"]), int(s["vdim"]), int(s["kv_rank"])
        self.win = int(s["mask"]["size"]) if s.get("mask") else 1 << 30
        self.scale = float(s["scale"]) if "scale" in s else self.D ** -0.5

    def tensor_shapes(self):
        self._dims()
        H, D, V, r, W = self.H, self.D, self.V, self.rank, self.width
        return {"q": (H * D, W), "dkv": (r, W), "dkv.norm": (r,), "uk": (H * D, r),
                "uv": (H * V, r), "sink": (H,), "g": (H * V, W), "o": (W, H * V)}

    def load(self, get, dtype, dev):
        self._dims()
        H, D, V, r = self.H, self.D, self.V, self.rank
        # one projection for everything that reads the layer input: q | latent | gate
        self.w_in = torch.cat([get("q"), get("dkv"), get("g")], 0).to(dev, dtype).contiguous()
        self.cnorm = _vec(get("dkv.norm"), dev)
        # keys and values are never formed: the query is carried into latent space with
        # W_uk (per head [D, rank]) and the attended latent leaves through W_uv^T
        self.uk = get("uk").to(dev, dtype).view(H, D, r).contiguous()
        self.uvt = get("uv").to(dev, dtype).view(H, V, r).transpose(1, 2).contiguous()
        self.sink = _vec(get("sink"), dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("paged", self.rank)

    def forward(self, h, b, cache, layer):
        H, D, V, r = self.H, self.D, self.V, self.rank
        pool = cache.paged[layer]
        proj = F.linear(h, self.w_in)
        sm.rmsnorm(proj[:, H * D:H * D + r], self.cnorm, self.eps, pool, out_rows=b.cache_rows)
        qa = torch.bmm(proj[:, :H * D].view(b.R, H, D).transpose(0, 1), self.uk)   # [H, R, rank]
        ol = torch.empty_like(qa)
        units = b.units(sm.latent_rows_per_wave(H)) if sm.latent_mfma_ok(qa, pool) else None
        sm.latent_attn(qa, pool, b.block_tables, b.row_ent, b.pos, self.sink, self.scale, self.win,
                       ol, PAGE, units=units, max_keys=b.max_keys)
        o = torch.bmm(ol, self.uvt)                                                # [H, R, V]
        gated = torch.empty(b.R, H * V, device=h.device, dtype=h.dtype)
        sm.sigmoid_gate(o, proj[:, H * D + r:], gated, H, V)
        return F.linear(gated, self.wo)


class WindowAttention(Mixer):
    """Grouped-query attention with cached keys and values (``ops.seqmix.window_attn``)."""
    kind = "window_attention"
    PER_HEAD = False   # query / key norm per head with one weight of D channels, or over the row
    HALF = False       # rotated pairs (i, i + dims/2) or (2i, 2i+1)
    SINK = True        # softmax denominator with a learned per-head sink

    def _dims(self):
        s = self.spec
        self.kv_from = int(s["kv_from"]) if s.get("kv_from") is not None else None
        self.H, self.D, self.V = int(s["heads"]), int(s["dim"]), int(s["vdim"])
        self.G = int(s.get("kv_heads", self.H))
        self.win = int(s["mask"]["size"]) if s.get("mask") else 1 << 30
        self.scale = float(s["scale"]) if "scale" in s else self.D ** -0.5
        rot = s.get("rot")
        self.rot_dims = int(rot["dims"]) if rot else 0
        self.rot_base = float(rot["base"]) if rot else 1.0
        self.rot_scaling = dict(rot["scaling"]) if rot and rot.get("scaling") else None
        if self.H % self.G or self.rot_dims % 2 or self.rot_dims > self.D:
            raise ValueError("window_attention: %d heads / %d kv heads / %d rotated of %d channels"
                             % (self.H, self.G, self.rot_dims, self.D))
        self.n_mid = self.H * self.V

    def tensor_shapes(self):
        self._dims()
        H, G, D, V, W = self.H, self.G, self.D, self.V, self.width
        d = {"q": (H * D, W), "q.norm": (D,) if self.PER_HEAD else (H * D,), "o": (W, H * V)}
        if self.kv_from is None:   # a layer that borrows keys and values has no tensors of them
            d.update({"k": (G * D, W), "v": (G * V, W), "k.norm": (D,) if self.PER_HEAD else (G * D,)})
        if self.SINK:
            d["sink"] = (H,)
        return d

    def load(self, get, dtype, dev):
        self._dims()
        own = self.kv_from is None
        names = ("q", "k", "v") if own else ("q",)
        self.w_in = torch.cat([get(k) for k in names], 0).to(dev, dtype).contiguous()
        self.qnorm = _vec(get("q.norm"), dev)
        self.knorm = _vec(get("k.norm"), dev) if own else None
        self.sink = _vec(get("sink"), dev) if self.SINK else None
        self.inv_freq = sm.rope_inv_freq(self.rot_base, self.rot_dims, dev, self.rot_scaling)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("paged", self.G * (self.D + self.V)) if self.kv_from is None else None

    def shares_cache_with(self, other) -> bool:
        """Whether this layer can read the keys and values that ``other`` leaves in its pool."""
        return (isinstance(other, WindowAttention) and other.kv_from is None
                and (other.G, other.D, other.V, other.PER_HEAD, other.HALF)
                == (self.G, self.D, self.V, self.PER_HEAD, self.HALF)
                and (other.rot_dims, other.rot_base, other.rot_scaling)
                == (self.rot_dims, self.rot_base, self.rot_scaling))

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        H, G, D, V = self.H, self.G, self.D, self.V
        own = self.kv_from is None
        pool = cache.paged[layer if own else self.kv_from]
        q = torch.empty(b.R, H * D, device=proj.device, dtype=proj.dtype)
        sm.qk_norm_rope_store(proj, H, G, D, V, self.qnorm, self.knorm, self.inv_freq, b.pos,
                              b.cache_rows, pool if own else None, self.eps, q,
                              per_head=self.PER_HEAD, half=self.HALF)
        units = b.units(sm.window_rows_per_wave(H // G)) if sm.window_mfma_ok(q, pool, D, V) else None
        sm.window_attn(q, pool, b.block_tables, b.row_ent, b.pos, self.sink, self.scale, self.win,
                       out, PAGE, H, G, D, V, units=units, max_keys=b.max_keys, out_scale=out_scale)
        return out


class Attention(WindowAttention):
    """Causal grouped-query attention with an ordinary softmax: per-head query / key norm,
    rotation of the pairs (i, i + dims/2) with optional stretching of long wavelengths
    (``rot.scaling``), no sink; ``mask`` (a window) stays optional.  ``kv_from: j`` reads layer
    j's keys and values as its cache holds them and projects only queries."""
    kind = "attention"
    PER_HEAD, HALF, SINK = True, True, False


class BiasedAttention(Mixer):
    """Causal grouped-query attention without rotation (``ops.seqmix.window_attn``): biased
    q / k / v projections; the query is multiplied by a temperature that grows with the
    logarithm of its position in steps of ``q_temp.every`` positions; scores are capped by
    ``softcap * tanh(. / softcap)`` and lose ``r1_h * ln(1 + r2_h * distance)`` per head; the
    softmax denominator holds one more 1 (a sink with score 0 and no value); every head leaves
    multiplied by one sigmoid gate.  ``mask`` (a window) stays optional."""
    kind = "biased_attention"

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V = int(s["heads"]), int(s["dim"]), int(s["vdim"])
        self.G = int(s.get("kv_heads", self.H))
        self.win = int(s["mask"]["size"]) if s.get("mask") else 1 << 30
        self.scale = float(s["scale"]) if "scale" in s else self.D ** -0.5
        self.cap = float(s.get("softcap") or 0.0)
        qt = s.get("q_temp") or {}
        self.qt_coef, self.qt_every = float(qt.get("coef", 0.0)), int(qt.get("every", 1))
        if self.H % self.G or self.qt_every < 1 or self.cap < 0:
            raise ValueError("biased_attention: %d heads / %d kv heads / temperature every %d / cap %g"
                             % (self.H, self.G, self.qt_every, self.cap))
        self.n_mid = self.H * self.V

    def tensor_shapes(self):
        self._dims()
        H, G, D, V, W = self.H, self.G, self.D, self.V, self.width
        return {"q": (H * D, W), "q.b": (H * D,), "k": (G * D, W), "k.b": (G * D,),
                "v": (G * V, W), "v.b": (G * V,), "r1": (H,), "r2": (H,), "g": (H, W),
                "o": (W, H * V)}

    def load(self, get, dtype, dev):
        self._dims()
        # one projection for everything that reads the layer input: q | k | v | head gates
        self.w_in = torch.cat([get(k) for k in ("q", "k", "v", "g")], 0).to(dev, dtype).contiguous()
        self.b_in = torch.cat([get("q.b"), get("k.b"), get("v.b"),
                               torch.zeros(self.H, dtype=get("q.b").dtype)]).to(dev, dtype).contiguous()
        self.r1, self.r2 = _vec(get("r1"), dev), _vec(get("r2"), dev)
        self.sink = torch.zeros(self.H, device=dev, dtype=torch.float32)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("paged", self.G * (self.D + self.V))

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        H, G, D, V = self.H, self.G, self.D, self.V
        pool = cache.paged[layer]
        nq, nkv = H * D, G * (D + V)
        q = torch.empty(b.R, nq, device=proj.device, dtype=proj.dtype)
        sm.qtemp_kv_store(proj, nq, nkv, self.qt_coef, self.qt_every, b.pos, b.cache_rows, pool, q)
        units = b.units(sm.window_rows_per_wave(H // G)) if sm.window_mfma_ok(q, pool, D, V) else None
        sm.window_attn(q, pool, b.block_tables, b.row_ent, b.pos, self.sink, self.scale, self.win,
                       out, PAGE, H, G, D, V, units=units, max_keys=b.max_keys, out_scale=out_scale,
                       softcap=self.cap, dist=(self.r1, self.r2), gate=proj[:, nq + nkv:])
        return out


class RopeLatentAttention(Mixer):
    """Latent attention with a rotated key part (``ops.seqmix.latent_attn``): queries come
    through a normed low-rank latent; every token caches its normed key/value latent c
    (``kv_rank`` numbers) and one rotated key part of ``rot_dim`` channels that all heads share.
    A head's score is q_plain . (W_uk c) + q_rot . k_rot; the first term is evaluated in latent
    space, (W_uk^T q_plain) . c, so keys and values are never formed: the cached row [c | k_rot]
    meets the query [W_uk^T q_plain | q_rot], and the attended latent leaves through W_uv.
    Rotation turns the pairs (2i, 2i+1).  Plain causal softmax (``mask`` optional), one sigmoid
    gate per head."""
    kind = "rope_latent_attention"

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V = int(s["heads"]), int(s["dim"]), int(s["vdim"])
        self.Rd, self.rank, self.qrank = int(s["rot_dim"]), int(s["kv_rank"]), int(s["q_rank"])
        self.win = int(s["mask"]["size"]) if s.get("mask") else 1 << 30
        self.scale = float(s["scale"]) if "scale" in s else (self.D + self.Rd) ** -0.5
        rot = s.get("rot") or {"dims": self.Rd, "base": 10000.0}
        self.rot_dims, self.rot_base = int(rot["dims"]), float(rot["base"])
        if self.rot_dims % 2 or self.rot_dims > self.Rd:
            raise ValueError("rope_latent_attention: %d rotated of %d channels" % (self.rot_dims, self.Rd))
        self.n_mid = self.H * self.V

    @staticmethod
    def resolve_spec(spec, prefix, shapes):
        if "q_rank" not in spec and prefix + "dq" in shapes:
            spec["q_rank"] = int(tuple(shapes[prefix + "dq"])[0])
        return spec

    def tensor_shapes(self):
        self._dims()
        H, D, V, Rd, r, qr, W = self.H, self.D, self.V, self.Rd, self.rank, self.qrank, self.width
        return {"dq": (qr, W), "dq.norm": (qr,), "uq": (H * (D + Rd), qr), "dkv": (r + Rd, W),
                "dkv.norm": (r,), "uk": (H * D, r), "uv": (H * V, r), "g": (H, W), "o": (W, H * V)}

    def load(self, get, dtype, dev):
        self._dims()
        H, D, V, r = self.H, self.D, self.V, self.rank
        # one projection for everything that reads the layer input: query latent | key/value
        # latent | rotated key part | head gates
        self.w_in = torch.cat([get("dq"), get("dkv"), get("g")], 0).to(dev, dtype).contiguous()
        self.qnorm, self.cnorm = _vec(get("dq.norm"), dev), _vec(get("dkv.norm"), dev)
        self.uq = get("uq").to(dev, dtype).contiguous()
        self.uk = get("uk").to(dev, dtype).view(H, D, r).contiguous()
        self.uvt = get("uv").to(dev, dtype).view(H, V, r).transpose(1, 2).contiguous()
        self.inv_freq = sm.rope_inv_freq(self.rot_base, self.rot_dims, dev)
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("paged", self.rank + self.Rd)

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        H, D, V, Rd, r, qr = self.H, self.D, self.V, self.Rd, self.rank, self.qrank
        R, dev, dt = b.R, proj.device, proj.dtype
        pool = cache.paged[layer]
        cq = torch.empty(R, qr, device=dev, dtype=dt)
        sm.latent_prep(proj, qr, r, Rd, self.qnorm, self.cnorm, self.inv_freq, b.pos, b.cache_rows,
                       pool, self.eps, cq)
        q = F.linear(cq, self.uq)                                                  # [R, H*(D+Rd)]
        nrot2 = self.rot_dims
        qa = torch.empty(H, R, r + Rd, device=dev, dtype=dt)
        q3 = q.view(R, H, D + Rd)
        torch.bmm(q3[:, :, :D].transpose(0, 1), self.uk, out=qa[:, :, :r])
        sm.rope_rows(q[:, D:], H, D + Rd, self.inv_freq, b.pos, qa[0, :, r:], qa.stride(0))
        if nrot2 < Rd:
            qa[:, :, r + nrot2:] = q3[:, :, D + nrot2:].transpose(0, 1)
        ol = torch.empty_like(qa)
        units = b.units(sm.latent_rows_per_wave(H)) if sm.latent_mfma_ok(qa, pool) else None
        sm.latent_attn(qa, pool, b.block_tables, b.row_ent, b.pos, None, self.scale, self.win, ol,
                       PAGE, units=units, max_keys=b.max_keys)
        o = torch.bmm(ol[:, :, :r], self.uvt)                                      # [H, R, V]
        sm.sigmoid_gate(o, proj[:, qr + r + Rd:], out, H, V, per_head=True)
        if out_scale != 1.0:
            out.mul_(out_scale)
        return out


class MLSTM(Mixer):
    """Matrix memory of the xLSTM (``ops.seqmix.mlstm_scan``): per head a D x V memory and a
    normaliser, written through an exponential input gate and decayed by a sigmoid forget gate
    whose pre-activations are capped by ``gate_cap * tanh(. / gate_cap)``; head norm, a weight
    per channel and a sigmoid output gate on the way out."""
    kind = "mlstm"

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V = int(s["heads"]), int(s["dim"]), int(s["vdim"])
        self.cap = float(s["gate_cap"])
        if self.cap <= 0:
            raise ValueError("mlstm: gate cap %g" % self.cap)
        self.n_mid = self.H * self.V

    def tensor_shapes(self):
        self._dims()
        H, D, V, W = self.H, self.D, self.V, self.width
        return {"q": (H * D, W), "k": (H * D, W), "v": (H * V, W), "g": (H * V, W), "o": (W, H * V),
                "norm": (H * V,), "i": (H, W), "i.b": (H,), "f": (H, W), "f.b": (H,)}

    def load(self, get, dtype, dev):
        self._dims()
        # one projection for everything that reads the layer input: q | k | v | gate | i | f
        self.w_in = torch.cat([get(k) for k in ("q", "k", "v", "g", "i", "f")], 0).to(dev, dtype).contiguous()
        self.bi, self.bf, self.normw = (_vec(get(k), dev) for k in ("i.b", "f.b", "norm"))
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        # column V of the memory holds the normaliser; m is the running maximum of the log gates
        return ("state", {"S": (self.H, self.D, self.V + 1), "m": (self.H,)})

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        st = cache.state[layer]
        sm.mlstm_scan(proj, self.bi, self.bf, self.cap, self.normw, st["S"], st["m"], b.ent,
                      b.ent_host, out, self.H, self.D, self.V, self.eps, out_scale=out_scale)
        return out


class GatedDelta(Mixer):
    """Gated delta rule behind short convolutions (``ops.seqmix.gated_delta_scan``)."""
    kind = "gated_delta"
    LOW_RANK = 16

    @staticmethod
    def resolve_spec(spec, prefix, shapes):
        for key, name in (("decay_rank", "a1"), ("gate_rank", "g1")):
            if key not in spec and prefix + name in shapes:
                spec[key] = int(tuple(shapes[prefix + name])[0])
        return spec

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V, self.K = int(s["heads"]), int(s["dim"]), int(s["vdim"]), int(s["conv"])
        self.G = int(s.get("kv_heads", self.H))
        self.ra = int(s.get("decay_rank", self.LOW_RANK))
        self.rg = int(s.get("gate_rank", self.LOW_RANK))
        if self.H % self.G or self.K < 1:
            raise ValueError("gated_delta: %d heads / %d kv heads / %d taps" % (self.H, self.G, self.K))
        self.C = 2 * self.G * self.D + self.H * self.V
        self.n_mid = self.H * self.V

    def tensor_shapes(self):
        self._dims()
        H, G, D, V, K, W = self.H, self.G, self.D, self.V, self.K, self.width
        return {"q": (G * D, W), "q.conv": (G * D, K), "k": (G * D, W), "k.conv": (G * D, K),
                "v": (H * V, W), "v.conv": (H * V, K), "b": (H, W), "A_log": (H,), "norm": (V,),
                "a1": (self.ra, W), "a2": (H * D, self.ra), "dt_bias": (H * D,),
                "g1": (self.rg, W), "g2": (H * V, self.rg), "o": (W, H * V)}

    def load(self, get, dtype, dev):
        self._dims()
        # one projection for everything that reads the layer input: q | k | v | beta | a1 | g1
        self.w_in = torch.cat([get(k) for k in ("q", "k", "v", "b", "a1", "g1")], 0).to(dev, dtype).contiguous()
        self.cw = torch.cat([_vec(get(k), dev) for k in ("q.conv", "k.conv", "v.conv")], 0).contiguous()
        self.cb = torch.zeros(self.C, device=dev, dtype=torch.float32)
        self.w_a2 = get("a2").to(dev, dtype).contiguous()
        self.w_g2 = get("g2").to(dev, dtype).contiguous()
        self.A_log, self.dt_bias, self.normw = (_vec(get(k), dev) for k in ("A_log", "dt_bias", "norm"))
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("state", {"S": (self.H, self.D, self.V), "tail": (self.K - 1, self.C)})

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        st, C, H = cache.state[layer], self.C, self.H
        conv = torch.empty(b.R, C, device=proj.device, dtype=torch.float32)
        sm.mamba_conv(proj, 0, self.cw, self.cb, st["tail"], b.ent, b.ent_host, b.row_ent, conv)
        sm.conv_tail_roll(proj, 0, st["tail"], b.ent, b.ent_host, C)
        araw = F.linear(proj[:, C + H:C + H + self.ra], self.w_a2)
        gate = F.linear(proj[:, C + H + self.ra:C + H + self.ra + self.rg], self.w_g2)
        sm.gated_delta_scan(conv, araw, proj[:, C:C + H], gate, self.A_log, self.dt_bias, self.normw,
                            st["S"], b.ent, b.ent_host, out, H, self.G, self.D, self.V, self.eps,
                            out_scale=out_scale)
        return out


class HGRN2(Mixer):
    """Gated linear attention with a lower-bounded forget gate (``ops.seqmix.hgrn2_scan``)."""
    kind = "hgrn2"

    def _dims(self):
        s = self.spec
        self.H, self.D, self.V = int(s["heads"]), int(s["dim"]), int(s["vdim"])
        self.n_mid = self.H * self.V

    def tensor_shapes(self):
        self._dims()
        n, W = self.H * self.D, self.width
        return {"q": (n, W), "f": (n, W), "f.b": (n,), "lower": (n,), "v": (self.H * self.V, W),
                "norm": (self.V,), "o": (W, self.H * self.V)}

    def load(self, get, dtype, dev):
        self._dims()
        self.w_in = torch.cat([get("q"), get("f"), get("v")], 0).to(dev, dtype).contiguous()
        self.fb, self.lower, self.normw = (_vec(get(k), dev) for k in ("f.b", "lower", "norm"))
        self.wo = get("o").to(dev, dtype).contiguous()

    def cache_spec(self):
        return ("state", {"S": (self.H, self.D, self.V)})

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        sm.hgrn2_scan(proj, self.lower, self.fb, self.normw, cache.state[layer]["S"], b.ent,
                      b.ent_host, out, self.H, self.D, self.V, self.eps, out_scale=out_scale)
        return out


class Parallel(Mixer):
    """Two mixers on the same input: ``left_scale * left + right_scale * right``.  Their input
    projections are one matrix product, and so are their output projections (each branch
    writes its scaled share of one buffer)."""
    kind = "parallel"
    BRANCHES = (("left", "window_attention"), ("right", "gated_delta"))

    def __init__(self, spec, width, eps):
        super().__init__(spec, width, eps)
        self.parts = [(name, MIXERS[spec[name].get("type", kind)](dict(spec[name]), width, eps),
                       float(spec.get(name + "_scale", 1.0))) for name, kind in self.BRANCHES]

    @staticmethod
    def resolve_spec(spec, prefix, shapes):
        for name, kind in Parallel.BRANCHES:
            sub = dict(spec[name])
            spec[name] = MIXERS[sub.get("type", kind)].resolve_spec(sub, prefix + name + ".", shapes)
        return spec

    def tensor_shapes(self):
        return {name + "." + k: s for name, m, _ in self.parts for k, s in m.tensor_shapes().items()}

    def load(self, get, dtype, dev):
        for name, m, _ in self.parts:
            m.load(lambda k, name=name: get(name + "." + k), dtype, dev)
        self.w_in = torch.cat([m.w_in for _, m, _ in self.parts], 0).contiguous()
        self.wo = torch.cat([m.wo for _, m, _ in self.parts], 1).contiguous()
        self.n_mid = sum(m.n_mid for _, m, _ in self.parts)

    def cache_spec(self):
        specs = []
        for _, m, _ in self.parts:
            s = m.cache_spec()
            specs += s if isinstance(s, list) else [s] if s else []
        return specs

    def mix(self, proj, b, cache, layer, out, out_scale=1.0):
        i0 = o0 = 0
        for _, m, scale in self.parts:
            n = m.w_in.shape[0]
            m.mix(proj[:, i0:i0 + n], b, cache, layer, out[:, o0:o0 + m.n_mid], out_scale * scale)
            i0, o0 = i0 + n, o0 + m.n_mid
        return out


MIXERS = {c.kind: c for c in (GeneralDelta, Mamba2, LatentAttention, WindowAttention, GatedDelta,
                              HGRN2, Parallel, Attention, MLSTM, BiasedAttention, RopeLatentAttention)}


class DenseFF:
    """Gated feed-forward W_down(act(W_gate h) * W_up h): silu-gated, or with a ``limit`` in its
    config the clamped unit of ``ops.seqmix.ff_act``.

    Every feed-forward offers two ways in: ``forward(h)``, or for a layer that runs the
    projections of its input and the output projections of its sublayers as one product each:
    ``w_in`` (rows that read the layer input, or None), ``fill(proj, h, mid)`` (writes the
    input of the output projection, [R, n_mid]; may return a part of the result that is added
    separately) and ``w_out`` [width, n_mid]."""
    ACT = "silu"

    def __init__(self, spec: dict, width: int):
        self.spec, self.width = spec, width
        self.F = self.n_mid = int(spec["ff"])
        self.limit = float(spec["limit"]) if spec.get("limit") is not None else None

    def tensor_shapes(self):
        return {"gate": (self.F, self.width), "up": (self.F, self.width), "down": (self.width, self.F)}

    def load(self, get, dtype, dev):
        self.w_gu = torch.cat([get("gate"), get("up")], 0).to(dev, dtype).contiguous()
        self.w_in = self.w_gu
        self.w_down = self.w_out = get("down").to(dev, dtype).contiguous()

    def fill(self, gu, h, mid):
        if self.limit is None:
            sm.glu_act(gu, mid, self.ACT)
        else:
            sm.ff_act(gu, mid, self.limit)
        return None

    def forward_proj(self, gu):
        """gu = [gate | up] projections of the input."""
        act = torch.empty(gu.shape[0], self.F, device=gu.device, dtype=gu.dtype)
        self.fill(gu, None, act)
        return F.linear(act, self.w_down)

    def forward(self, h):
        return self.forward_proj(F.linear(h, self.w_gu))


class MoEFF:
    """Mixture of clamped gated experts behind a sigmoid router whose choice is limited to
    the best groups of experts (``ops.seqmix.group_route``); the chosen experts' scores weight
    their outputs without rescaling.  The expert products run grouped over the routed rows
    (``ops.seqmix.expert_gemm``)."""
    w_in = w_out = None   # the router and the grouped products read the input themselves
    n_mid = 0

    def fill(self, proj, h, mid):
        return self.forward(h)

    def __init__(self, spec: dict, width: int):
        self.spec, self.width = spec, width
        r, e = spec["router"], spec["expert"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        g = r.get("groups") or {}
        self.groups, self.keep = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
        self.F, self.limit = int(e["ff"]), float(e["limit"])
        per = self.E // max(1, self.groups)
        if self.groups < 1 or self.E % self.groups or not 1 <= self.keep <= self.groups \
                or not 1 <= self.top <= self.keep * per:
            raise ValueError("moe: %d experts in %d groups, %d kept, %d chosen"
                             % (self.E, self.groups, self.keep, self.top))

    def tensor_shapes(self):
        d = {"router": (self.E, self.width)}
        for e in range(self.E):
            d.update({"e%d.gate" % e: (self.F, self.width), "e%d.up" % e: (self.F, self.width),
                      "e%d.down" % e: (self.width, self.F)})
        return d

    def load(self, get, dtype, dev):
        self.wr = get("router").to(dev).float().contiguous()
        gate = torch.stack([get("e%d.gate" % e) for e in range(self.E)])
        up = torch.stack([get("e%d.up" % e) for e in range(self.E)])
        # widths that are multiples of 16: gate and up rows interleaved, so that the first
        # product's epilogue applies the activation (otherwise gate | up and a pointwise pass)
        self.fused = self.F % 16 == 0
        w_gu = sm.interleave_gate_up(gate, up) if self.fused else torch.cat([gate, up], 1)
        self.w_gu = w_gu.to(dev, dtype).contiguous()
        self.w_down = torch.stack([get("e%d.down" % e) for e in range(self.E)]).to(dev, dtype).contiguous()

    def forward(self, h):
        R, top, dev = h.shape[0], self.top, h.device
        ids = torch.empty(R, top, device=dev, dtype=torch.int32)
        wts = torch.empty(R, top, device=dev, dtype=torch.float32)
        cnt = torch.empty(self.E, device=dev, dtype=torch.int32)
        rows = torch.empty(self.E, R * top, device=dev, dtype=torch.int32)
        sm.group_route(h, self.wr, top, self.groups, self.keep, ids, wts, cnt, rows)
        act = torch.empty(R * top, self.F, device=dev, dtype=h.dtype)
        if self.fused:
            sm.expert_gemm(h, top, self.w_gu, cnt, rows, act, R * top, act_limit=self.limit)
        else:
            gu = torch.empty(R * top, 2 * self.F, device=dev, dtype=h.dtype)
            sm.expert_gemm(h, top, self.w_gu, cnt, rows, gu, R * top)
            sm.ff_act(gu, act, self.limit)
        y = torch.empty(R * top, self.width, device=dev, dtype=h.dtype)
        sm.expert_gemm(act, 1, self.w_down, cnt, rows, y, R * top)
        out = torch.empty(R, self.width, device=dev, dtype=h.dtype)
        return sm.expert_combine(y, wts, out)


class GeluFF(DenseFF):
    """W_down(gelu(W_gate h) * W_up h) with the tanh form of gelu."""
    ACT = "gelu_tanh"


class SoftmaxMoEFF:
    """Mixture of ungated squared-relu experts, W_down relu(W_up h)^2, behind a softmax router
    (``ops.seqmix.group_route``): scores s = softmax over all router outputs; the choice is made
    on s + ``correction``, limited to the ``groups.keep`` groups of neighbouring experts whose
    best choice score is largest; the weights are the chosen s, not rescaled.  The last
    ``router.identity`` router outputs stand for experts without tensors that hand their input
    back.  An optional shared expert of the same form runs for every token, weighted by
    sigmoid(W_sg h); its products ride on the layer's input and output products."""

    def __init__(self, spec: dict, width: int):
        self.spec, self.width = spec, width
        r = spec["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])          # experts with tensors
        self.ident = int(r.get("identity", 0))
        self.EA = self.E + self.ident                                 # router outputs
        g = r.get("groups") or {}
        self.groups, self.keep = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
        self.F = int(spec["expert"]["ff"])
        self.Fs = self.n_mid = int(spec["shared"]["ff"]) if spec.get("shared") else 0
        per = self.EA // max(1, self.groups)
        if self.groups < 1 or self.EA % self.groups or not 1 <= self.keep <= self.groups \
                or not 1 <= self.top <= self.keep * per or self.E < 0 or self.ident < 0:
            raise ValueError("moe: %d + %d experts in %d groups, %d kept, %d chosen"
                             % (self.E, self.ident, self.groups, self.keep, self.top))

    def tensor_shapes(self):
        d = {"router": (self.EA, self.width), "correction": (self.EA,)}
        for e in range(self.E):
            d.update({"e%d.up" % e: (self.F, self.width), "e%d.down" % e: (self.width, self.F)})
        if self.Fs:
            d.update({"shared.up": (self.Fs, self.width), "shared.down": (self.width, self.Fs),
                      "shared.sg": (1, self.width)})
        return d

    def load(self, get, dtype, dev):
        self.wr = get("router").to(dev).float().contiguous()
        self.corr = _vec(get("correction"), dev)
        self.w_up = self.w_dn = None
        if self.E:
            self.w_up = torch.stack([get("e%d.up" % e) for e in range(self.E)]).to(dev, dtype).contiguous()
            self.w_dn = torch.stack([get("e%d.down" % e) for e in range(self.E)]).to(dev, dtype).contiguous()
        self.w_in = self.w_out = None
        if self.Fs:
            self.w_in = torch.cat([get("shared.up"), get("shared.sg")], 0).to(dev, dtype).contiguous()
            self.w_out = get("shared.down").to(dev, dtype).contiguous()

    def routed(self, h):
        R, top, dev = h.shape[0], self.top, h.device
        ids = torch.empty(R, top, device=dev, dtype=torch.int32)
        wts = torch.empty(R, top, device=dev, dtype=torch.float32)
        cnt = torch.empty(self.EA, device=dev, dtype=torch.int32)
        rows = torch.empty(self.EA, R * top, device=dev, dtype=torch.int32)
        sm.group_route(h, self.wr, top, self.groups, self.keep, ids, wts, cnt, rows,
                       score="softmax", corr=self.corr, group_score="max")
        y = torch.empty(R * top, self.width, device=dev, dtype=h.dtype)
        if self.E:
            act = torch.empty(R * top, self.F, device=dev, dtype=h.dtype)
            sm.expert_gemm(h, top, self.w_up, cnt, rows, act, R * top, relu2=True)
            sm.expert_gemm(act, 1, self.w_dn, cnt, rows, y, R * top)
        out = torch.empty(R, self.width, device=dev, dtype=h.dtype)
        return sm.expert_combine(y, wts, out, ids=ids if self.ident else None, n_real=self.E, x=h)

    def fill(self, proj, h, mid):
        if self.Fs:
            sm.relu2_gate(proj, proj[:, self.Fs:self.Fs + 1], mid)
        return self.routed(h)

    def forward(self, h):
        y = self.routed(h)
        if self.Fs:
            proj = F.linear(h, self.w_in)
            mid = torch.empty(h.shape[0], self.Fs, device=h.device, dtype=h.dtype)
            sm.relu2_gate(proj, proj[:, self.Fs:self.Fs + 1], mid)
            y = y + F.linear(mid, self.w_out)
        return y


class TopMoEFF:
    """Mixture of silu-gated experts, W_down (silu(W_gate h) * W_up h), behind a router with a
    bias: the ``top`` largest logits win and the weights are the softmax over the winners'
    logits only (``ops.seqmix.group_route``, "top_softmax").  An optional shared expert of the
    same form runs for every token; its products ride on the layer's input and output
    products."""

    def __init__(self, spec: dict, width: int):
        self.spec, self.width = spec, width
        r = spec["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        self.F = int(spec["expert"]["ff"])
        self.Fs = self.n_mid = int(spec["shared"]["ff"]) if spec.get("shared") else 0
        if not 1 <= self.top <= self.E:
            raise ValueError("moe: %d experts, %d chosen" % (self.E, self.top))

    def tensor_shapes(self):
        d = {"router": (self.E, self.width), "router.b": (self.E,)}
        for e in range(self.E):
            d.update({"e%d.gate" % e: (self.F, self.width), "e%d.up" % e: (self.F, self.width),
                      "e%d.down" % e: (self.width, self.F)})
        if self.Fs:
            d.update({"shared.gate": (self.Fs, self.width), "shared.up": (self.Fs, self.width),
                      "shared.down": (self.width, self.Fs)})
        return d

    def load(self, get, dtype, dev):
        self.wr, self.br = get("router").to(dev).float().contiguous(), _vec(get("router.b"), dev)
        gate = torch.stack([get("e%d.gate" % e) for e in range(self.E)])
        up = torch.stack([get("e%d.up" % e) for e in range(self.E)])
        # widths that are multiples of 16: gate and up rows interleaved, so that the first
        # product's epilogue applies the activation (otherwise gate | up and a pointwise pass)
        self.fused = self.F % 16 == 0
        w_gu = sm.interleave_gate_up(gate, up) if self.fused else torch.cat([gate, up], 1)
        self.w_gu = w_gu.to(dev, dtype).contiguous()
        self.w_down = torch.stack([get("e%d.down" % e) for e in range(self.E)]).to(dev, dtype).contiguous()
        self.w_in = self.w_out = None
        if self.Fs:
            self.w_in = torch.cat([get("shared.gate"), get("shared.up")], 0).to(dev, dtype).contiguous()
            self.w_out = get("shared.down").to(dev, dtype).contiguous()

    def routed(self, h, cnt=None):
        """(y [R * top, width], wts [R, top]): the chosen experts' outputs and their weights,
        to be summed by whoever adds them to the residual.  cnt: cleared int32 counts [E] (a
        model hands every layer a row of one buffer that it clears once per step)."""
        R, top, dev = h.shape[0], self.top, h.device
        ids = torch.empty(R, top, device=dev, dtype=torch.int32)
        wts = torch.empty(R, top, device=dev, dtype=torch.float32)
        cleared = cnt is not None
        if cnt is None:
            cnt = torch.empty(self.E, device=dev, dtype=torch.int32)
        rows = torch.empty(self.E, R * top, device=dev, dtype=torch.int32)
        sm.group_route(h, self.wr, top, 1, 1, ids, wts, cnt, rows, score="top_softmax", bias=self.br,
                       cleared=cleared)
        act = torch.empty(R * top, self.F, device=dev, dtype=h.dtype)
        if self.fused:
            sm.expert_gemm(h, top, self.w_gu, cnt, rows, act, R * top, silu_glu=True)
        else:
            gu = torch.empty(R * top, 2 * self.F, device=dev, dtype=h.dtype)
            sm.expert_gemm(h, top, self.w_gu, cnt, rows, gu, R * top)
            sm.glu_act(gu, act, "silu")
        y = torch.empty(R * top, self.width, device=dev, dtype=h.dtype)
        sm.expert_gemm(act, 1, self.w_down, cnt, rows, y, R * top)
        return y, wts

    def fill_routed(self, proj, h, mid, cnt=None):
        """``fill`` for a layer whose residual pass sums the routed experts itself."""
        if self.Fs:
            sm.glu_act(proj, mid, "silu")
        return self.routed(h, cnt)

    def fill(self, proj, h, mid):
        y, wts = self.fill_routed(proj, h, mid)
        return sm.expert_combine(y, wts, torch.empty(h.shape[0], self.width, device=h.device, dtype=h.dtype))

    def forward(self, h):
        y, wts = self.routed(h)
        y = sm.expert_combine(y, wts, torch.empty(h.shape[0], self.width, device=h.device, dtype=h.dtype))
        if self.Fs:
            mid = torch.empty(h.shape[0], self.Fs, device=h.device, dtype=h.dtype)
            sm.glu_act(F.linear(h, self.w_in), mid, "silu")
            y = y + F.linear(mid, self.w_out)
        return y


FEEDFORWARDS = {"dense": DenseFF, "moe": MoEFF, "dense_gelu": GeluFF, "moe_softmax": SoftmaxMoEFF,
                "moe_top": TopMoEFF}


# ---------------------------------------------------------------------------- weights
class HybridLayer:
    def __init__(self, spec: LayerSpec, cfg: HybridConfig):
        self.block = cfg.traits.block
        self.norm_offset = cfg.traits.norm_offset
        self.mixer = MIXERS[cfg.traits.mixer_key(spec.kind)](spec.mixer, cfg.width, cfg.eps)
        self.ff = FEEDFORWARDS[cfg.traits.ff_key(spec.mlp.get("kind", "dense"))](spec.mlp, cfg.width) \
            if spec.mlp is not None else None
        # parallel: the layer's input and output products (mixer and feed-forward together)
        self.w_in_all = self.w_out_all = None
        self.norm1 = self.norm1b = self.ls1 = self.norm2 = self.norm2b = self.ls2 = None
        # gated_post: the gates' projections ride on the sublayers' input products
        self.w_in1 = self.w_in2 = self.rg1b = self.rg2b = None

    def tensor_shapes(self, W):
        if self.block == "parallel2":
            d = {"norm1": ()}
            d.update({"mix." + k: s for k, s in self.mixer.tensor_shapes().items()})
            if self.ff is not None:
                d["norm2"] = ()
                d.update({"mlp." + k: s for k, s in self.ff.tensor_shapes().items()})
            return d
        if self.block == "parallel":
            d = {"norm1": (W,)}
            d.update({"mix." + k: s for k, s in self.mixer.tensor_shapes().items()})
            if self.ff is not None:
                d.update({"mlp." + k: s for k, s in self.ff.tensor_shapes().items()})
            return d
        gated = self.block == "gated_post"
        d = {"norm1": (W,), "rg1": (W, W), "rg1.b": (W,)} if gated else \
            {"norm1": (W,), "norm1b": (W,), "ls1": (W,)}
        d.update({"mix." + k: s for k, s in self.mixer.tensor_shapes().items()})
        if self.ff is not None:
            d.update({"norm2": (W,), "rg2": (W, W), "rg2.b": (W,)} if gated else
                     {"norm2": (W,), "norm2b": (W,), "ls2": (W,)})
            d.update({"mlp." + k: s for k, s in self.ff.tensor_shapes().items()})
        return d

    def load(self, sd, p, dtype, dev):
        self.mixer.load(lambda k: sd[p + "mix." + k], dtype, dev)
        if self.ff is not None:
            self.ff.load(lambda k: sd[p + "mlp." + k], dtype, dev)
        if self.block == "parallel2":
            # the mixer and the feed-forward read the same rows through norms of their own, so
            # each has its input product; their output products are one
            if self.mixer.w_in is None or self.mixer.wo is None:
                raise ValueError("mixer %r cannot share the layer's products" % self.mixer.kind)
            self.norm1 = (_vec(sd[p + "norm1"], dev).reshape(1) + self.norm_offset).contiguous()
            outs = [self.mixer.wo]
            if self.ff is not None:
                self.norm2 = (_vec(sd[p + "norm2"], dev).reshape(1) + self.norm_offset).contiguous()
                if self.ff.n_mid:
                    outs.append(self.ff.w_out)
            self.w_out_all = torch.cat(outs, 1).contiguous() if len(outs) > 1 else outs[0]
            return
        if self.block == "parallel":
            if self.mixer.w_in is None or self.mixer.wo is None:
                raise ValueError("mixer %r cannot share the layer's products" % self.mixer.kind)
            self.norm1 = (_vec(sd[p + "norm1"], dev) + self.norm_offset).contiguous()
            ins, outs = [self.mixer.w_in], [self.mixer.wo]
            if self.ff is not None and self.ff.w_in is not None:
                ins.append(self.ff.w_in)
            if self.ff is not None and self.ff.n_mid:
                outs.append(self.ff.w_out)
            self.w_in_all = torch.cat(ins, 0).contiguous() if len(ins) > 1 else ins[0]
            self.w_out_all = torch.cat(outs, 1).contiguous() if len(outs) > 1 else outs[0]
            return
        if self.block == "gated_post":
            if self.mixer.w_in is None:
                raise ValueError("mixer %r cannot share its input product with a gate" % self.mixer.kind)
            self.norm1, self.rg1b = _vec(sd[p + "norm1"], dev), _vec(sd[p + "rg1.b"], dev)
            self.w_in1 = torch.cat([self.mixer.w_in, sd[p + "rg1"].to(dev, dtype)], 0).contiguous()
            if self.ff is not None:
                self.norm2, self.rg2b = _vec(sd[p + "norm2"], dev), _vec(sd[p + "rg2.b"], dev)
                rg2 = sd[p + "rg2"].to(dev, dtype)
                self.w_in2 = rg2.contiguous() if self.ff.w_in is None else \
                    torch.cat([self.ff.w_in, rg2], 0).contiguous()
            return
        self.norm1, self.norm1b, self.ls1 = (_vec(sd[p + k], dev) for k in ("norm1", "norm1b", "ls1"))
        if self.ff is not None:
            self.norm2, self.norm2b, self.ls2 = (_vec(sd[p + k], dev) for k in ("norm2", "norm2b", "ls2"))


def tensor_shapes(cfg: HybridConfig) -> dict:
    """name -> shape of every tensor of a checkpoint of this config."""
    W = cfg.width
    d = {"embed": (cfg.vocab, W), "final.norm": () if cfg.traits.scalar_norms else (W,),
         "head": (cfg.vocab, W)}
    if cfg.traits.positions:
        d["pos"] = (cfg.max_pos, W)
    if cfg.loop:
        d["loop.step"] = (cfg.loop[2], W)
    for i, spec in enumerate(cfg.layers):
        d.update({"l%d.%s" % (i, k): s for k, s in HybridLayer(spec, cfg).tensor_shapes(W).items()})
    return d


class HybridWeights:
    """The weight store: matrices in the activation dtype ([out, in], as stored), vectors in
    fp32.  ``dtype`` is torch.bfloat16 (serving) or torch.float32 (exact)."""

    def __init__(self, cfg: HybridConfig, sd, device, dtype=torch.bfloat16):
        cfg = cfg.resolve({k: v.shape for k, v in sd.items()})
        self.cfg, self.dtype = cfg, dtype
        dev = self.device = torch.device(device)
        want = tensor_shapes(cfg)
        for k, s in want.items():
            if k not in sd:
                raise KeyError("checkpoint lacks tensor %r" % k)
            if tuple(sd[k].shape) != tuple(s):
                raise ValueError("tensor %r has shape %s, the config gives %s" % (k, tuple(sd[k].shape), s))
        self.embed = sd["embed"].to(dev, dtype).contiguous()
        self.pos = sd["pos"].to(dev, dtype).contiguous() if cfg.traits.positions else None
        self.final_norm = (_vec(sd["final.norm"], dev) + cfg.traits.norm_offset).expand(cfg.width).contiguous() \
            if cfg.traits.scalar_norms else (_vec(sd["final.norm"], dev) + cfg.traits.norm_offset).contiguous()
        self.head = sd["head"].to(dev, dtype).contiguous()
        self.loop_step = _vec(sd["loop.step"], dev) if cfg.loop else None
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            L = HybridLayer(spec, cfg)
            L.load(sd, "l%d." % i, dtype, dev)
            self.layers.append(L)
        check_shared_caches([L.mixer for L in self.layers])

    @classmethod
    def random(cls, cfg: HybridConfig, device="cuda", seed: int = 0, dtype=torch.bfloat16):
        return cls(cfg, random_state_dict(cfg, seed), device, dtype)

    def cache_specs(self) -> list:
        """What every layer run keeps between steps (a repeated layer once per pass)."""
        return [self.layers[i].mixer.cache_spec() for i, _t, _f in self.cfg.runs()]


def check_shared_caches(mixers: list):
    """A layer that reads another layer's keys and values names an earlier layer that keeps a
    pool of the same shape, filled the same way."""
    for i, m in enumerate(mixers):
        j = getattr(m, "kv_from", None)
        if j is None:
            continue
        if not 0 <= j < i or not m.shares_cache_with(mixers[j]):
            raise ValueError("layer %d cannot read the keys and values of layer %d" % (i, j))


def random_state_dict(cfg: HybridConfig, seed: int = 0) -> dict:
    """A random checkpoint (bf16 values): projections ~ N(0, 1/in), gains near 1, decay and
    step parameters in the ranges where the recurrences neither vanish nor blow up."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    shapes = tensor_shapes(cfg)
    for k, s in shapes.items():
        s = tuple(s) or (1,)   # a single number is drawn as one and stored without a shape
        leaf = k.split(".", 1)[1] if k.startswith("l") and "." in k else k
        if len(s) == 2 and not leaf.endswith("conv"):
            t = torch.randn(*s, generator=g) / (s[1] ** 0.5 if k not in ("embed", "pos") else 1.0)
        elif leaf.endswith("conv"):
            t = torch.randn(*s, generator=g) * 0.5
        elif leaf in ("norm1", "norm2", "norm1b", "norm2b") or k == "final.norm":
            t = (1.0 - cfg.traits.norm_offset) + 0.1 * torch.randn(*s, generator=g)
        elif leaf.endswith(".norm"):
            t = 1.0 + 0.1 * torch.randn(*s, generator=g)
        elif leaf.endswith("correction"):
            t = 0.05 * torch.randn(*s, generator=g)
        elif leaf.endswith("lower"):
            t = torch.rand(*s, generator=g) * 0.9
        elif leaf in ("ls1", "ls2"):
            t = 0.5 + 0.1 * torch.randn(*s, generator=g)
        elif leaf.endswith("A_log"):
            t = torch.rand(*s, generator=g) * 1.5 - 1.0
        elif leaf.endswith(("mix.r1", "mix.r2")):
            t = torch.rand(*s, generator=g) * (2.0 if leaf.endswith("r1") else 0.3)
        elif k == "loop.step":
            t = torch.randn(*s, generator=g) * 0.5
        elif leaf.endswith(("dt_bias", "mix.D")):
            t = torch.randn(*s, generator=g) * 0.5
        else:
            t = torch.randn(*s, generator=g) * 0.5
        sd[k] = t.to(torch.bfloat16).reshape(tuple(shapes[k]))
    return sd


def load_dir(path: str, device="cuda", dtype=torch.bfloat16):
    """(config, weights) of a checkpoint folder: ``config.json`` + ``model.safetensors``."""
    from safetensors.torch import load_file

    with open(os.path.join(path, "config.json")) as f:
        cfg = HybridConfig.from_dict(json.load(f), name=os.path.basename(os.path.normpath(path)))
    sd = load_file(os.path.join(path, "model.safetensors"))
    w = HybridWeights(cfg, sd, device, dtype)
    return w.cfg, w


# ---------------------------------------------------------------------------- model
class HybridModel:
    def __init__(self, weights: HybridWeights, cache):
        self.w, self.cfg, self.cache = weights, weights.cfg, cache
        self.device, self.dtype = weights.device, weights.dtype

    @torch.no_grad()
    def forward(self, b: StepBatch, layer_out=None):
        """Run one step; returns fp32 logits [n_out, vocab] of the wanted rows (None when no
        row is wanted).  layer_out: optional list that receives the residual stream after
        every layer (debugging / layer-by-layer checks)."""
        cfg, w = self.cfg, self.w
        if b.max_pos >= cfg.max_pos:
            raise ValueError("position %d exceeds the model's %d positions" % (b.max_pos, cfg.max_pos))
        if cfg.traits.block == "gated_post":
            return self._forward_gated_post(b, layer_out)
        if cfg.traits.block == "parallel":
            return self._forward_parallel(b, layer_out)
        if cfg.traits.block == "parallel2":
            return self._forward_parallel2(b, layer_out)
        x = torch.empty(b.R, cfg.width, device=self.device, dtype=torch.float32)
        sm.embed_pos(w.embed, w.pos, b.ids, b.pos, x)
        h = torch.empty(b.R, cfg.width, device=self.device, dtype=self.dtype)
        # every post-sublayer pass (norm, layer scale, residual add) also forms the next
        # sublayer's normed input from the updated rows
        sm.rmsnorm(x, w.layers[0].norm1, cfg.eps, h)
        for i, L in enumerate(w.layers):
            after = w.layers[i + 1].norm1 if i + 1 < len(w.layers) else None
            m = L.mixer.forward(h, b, self.cache, i)
            sm.norm_scale_add(x, m, L.norm1b, L.ls1, cfg.eps,
                              next_w=L.norm2 if L.ff is not None else after, next_out=h)
            if L.ff is not None:
                sm.norm_scale_add(x, L.ff.forward(h), L.norm2b, L.ls2, cfg.eps, next_w=after,
                                  next_out=h)
            if layer_out is not None:
                layer_out.append(x.clone())
        if b.n_out == 0:
            return None
        return self._logits(x, b)

    def _logits(self, x, b: StepBatch):
        cfg, w = self.cfg, self.w
        hn = torch.empty(b.n_out, cfg.width, device=self.device, dtype=self.dtype)
        sm.rmsnorm(x, w.final_norm, cfg.eps, hn, parts=cfg.norm_groups, in_rows=b.out_rows)
        y = F.linear(hn, w.head)
        if not cfg.logit_softcap and cfg.logit_scale == 1.0:
            return y.float()
        return sm.softcap(y, cfg.logit_softcap, torch.empty(y.shape, device=y.device, dtype=torch.float32),
                          scale=cfg.logit_scale)

    def _forward_parallel2(self, b: StepBatch, layer_out=None):
        """x <- x + mixer(N(x) g1) + ff(N(x) g2) over the layer runs of the config (a stretch of
        layers may run several passes; every run has its own cache).  One pass over the fp32
        rows adds what the previous layer produced (or, at the start of a pass, the embedding
        output and the pass's step vector) and writes both normed inputs of the next layer;
        the mixer and the shared expert write the inputs of their output projections side by
        side, one product sums the two in its fp32 accumulator, and the routed experts' sum is
        added in the same residual pass."""
        cfg, w = self.cfg, self.w
        R, W = b.R, cfg.width
        x = torch.empty(R, W, device=self.device, dtype=torch.float32)
        sm.embed_rows(w.embed, b.ids, x, None, scale=cfg.embed_scale)
        x0 = x.clone() if cfg.loop and cfg.loop[2] > 1 else None
        h1 = torch.empty(R, W, device=self.device, dtype=self.dtype)
        h2 = torch.empty(R, W, device=self.device, dtype=self.dtype)
        runs = cfg.runs()
        # the experts' slot counts of all layer runs, cleared by one fill
        moe = [hasattr(w.layers[i].ff, "fill_routed") for i, _t, _f in runs]
        cnts = torch.zeros(sum(moe), max([w.layers[i].ff.E for (i, _t, _f), m in zip(runs, moe) if m] or [1]),
                           device=self.device, dtype=torch.int32) if any(moe) else None
        y = extra = routed = None   # what the previous layer adds to x
        for k, (i, t, first) in enumerate(runs):
            L = w.layers[i]
            n2, o2 = (L.norm2, h2) if L.ff is not None else (None, None)
            if layer_out is not None and y is not None:   # the rows between two layers are asked for
                sm.add_norm2(x, y, extra, routed=routed)
                layer_out.append(x.clone())
                y = extra = routed = None
            sm.add_norm2(x, y, extra, rows=x0 if first and t > 0 else None,
                         vec=w.loop_step[t] if first else None, eps=cfg.eps,
                         w1=L.norm1, out1=h1, w2=n2, out2=o2, routed=routed)
            mm = L.mixer.n_mid
            mid = torch.empty(R, L.w_out_all.shape[1], device=self.device, dtype=self.dtype)
            L.mixer.mix(F.linear(h1, L.mixer.w_in, L.mixer.b_in), b, self.cache, k, mid[:, :mm])
            extra = routed = None
            if L.ff is not None:
                proj = F.linear(h2, L.ff.w_in) if L.ff.w_in is not None else None
                if moe[k]:
                    routed = L.ff.fill_routed(proj, h2, mid[:, mm:], cnts[sum(moe[:k]), :L.ff.E])
                else:
                    extra = L.ff.fill(proj, h2, mid[:, mm:])
            y = F.linear(mid, L.w_out_all)
        sm.add_norm2(x, y, extra, routed=routed)
        if layer_out is not None:
            layer_out.append(x.clone())
        if b.n_out == 0:
            return None
        return self._logits(x, b)

    def _forward_gated_post(self, b: StepBatch, layer_out=None):
        """x <- x + N(f(x) * sigmoid(R x + b)) per sublayer: the sublayer and its gate read the
        un-normalised residual rows (rounded to the activation type), so one matrix product
        serves both; the pass that adds the result also writes the next sublayer's input."""
        cfg, w = self.cfg, self.w
        x = torch.empty(b.R, cfg.width, device=self.device, dtype=torch.float32)
        # in float32 the sublayers read the residual stream itself
        h = x if self.dtype == torch.float32 else \
            torch.empty(b.R, cfg.width, device=self.device, dtype=self.dtype)
        nxt = None if h is x else h
        sm.embed_rows(w.embed, b.ids, x, nxt)
        parts, eps = cfg.norm_groups, cfg.eps
        for i, L in enumerate(w.layers):
            n = L.mixer.w_in.shape[0]
            proj = F.linear(h, L.w_in1)
            m = L.mixer.forward_proj(proj[:, :n], b, self.cache, i)
            sm.gate_norm_add(x, m, proj[:, n:], L.rg1b, L.norm1, parts, eps, next_out=nxt)
            if L.ff is not None:
                proj = F.linear(h, L.w_in2)
                if L.ff.w_in is None:
                    f, gate = L.ff.forward(h), proj
                else:
                    n = L.ff.w_in.shape[0]
                    f, gate = L.ff.forward_proj(proj[:, :n]), proj[:, n:]
                sm.gate_norm_add(x, f, gate, L.rg2b, L.norm2, parts, eps, next_out=nxt)
            if layer_out is not None:
                layer_out.append(x.clone())
        if b.n_out == 0:
            return None
        return self._logits(x, b)

    def _forward_parallel(self, b: StepBatch, layer_out=None):
        """x <- x + mixer(u) + ff(u) with u = norm(x): one product forms every projection of u
        (the mixer's and the feed-forward's), the sublayers write the inputs of their output
        projections side by side into one buffer, and one product with the joined output
        weights gives mixer(u) + ff(u) summed in its fp32 accumulator.  What a feed-forward
        computes apart from that (routed experts) is added in the same fp32 pass that updates
        the residual and forms the next layer's u."""
        cfg, w = self.cfg, self.w
        x = torch.empty(b.R, cfg.width, device=self.device, dtype=torch.float32)
        sm.embed_rows(w.embed, b.ids, x, None)
        h = torch.empty(b.R, cfg.width, device=self.device, dtype=self.dtype)
        sm.rmsnorm(x, w.layers[0].norm1, cfg.eps, h)
        for i, L in enumerate(w.layers):
            proj = F.linear(h, L.w_in_all)
            nm, mm = L.mixer.w_in.shape[0], L.mixer.n_mid
            mid = torch.empty(b.R, L.w_out_all.shape[1], device=self.device, dtype=self.dtype)
            L.mixer.mix(proj[:, :nm], b, self.cache, i, mid[:, :mm])
            extra = L.ff.fill(proj[:, nm:], h, mid[:, mm:]) if L.ff is not None else None
            y = F.linear(mid, L.w_out_all)
            nxt = w.layers[i + 1].norm1 if i + 1 < len(w.layers) else None
            sm.add_norm(x, y, extra, cfg.eps, next_w=nxt, next_out=h)
            if layer_out is not None:
                layer_out.append(x.clone())
        if b.n_out == 0:
            return None
        return self._logits(x, b)
