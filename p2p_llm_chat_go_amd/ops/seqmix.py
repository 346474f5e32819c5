"""Sequence-mixer ops: recurrent state layers (generalized delta rule, Mamba-2, gated delta
rule, HGRN2, the mLSTM's matrix memory), latent attention (optionally with a rotated key part
in the cached row and without a sink) and grouped-query attention with an optional sliding
window and softmax sink (query/key norm over the row or per head, rotary positions on adjacent
or half-split channel pairs and the cache write in one pass; or unrotated with a query
temperature, capped scores, a logarithmic distance penalty and a gate per head), a
group-limited expert router (sigmoid or softmax scores, optional score correction and bias,
softmax over the chosen logits) with grouped expert products and identity experts, learned
positions, and the norms, residual passes (one with two normed outputs and the routed experts'
weighted sum) and pointwise steps around them.

GPU tensors always run the gfx950 kernels of ``csrc/seqmix`` (``libp2p_seqmix.so``, built on
first use when missing); CPU tensors run the PyTorch rendering of the same math, which is
the plumbing / scheduling path of CPU tests, never a fallback for GPU tensors.

Conventions shared by every op:
  * activations (``x``-like matrices that feed or leave matrix products) are bf16 or fp32;
    vector parameters, recurrent state, the residual stream and every reduction are fp32;
  * a step is a flat list of R token rows cut into E *entries* (one per sequence portion):
    ``ent`` int32 [E, 4] = (first row, rows, first position, state slot); a portion whose
    first position is 0 starts from a zero state, others continue the slot's state;
  * ``row_ent`` int32 [R] names each row's entry, ``pos`` int32 [R] its position.
"""
from __future__ import annotations

import ctypes
import math
import os
import threading

import torch

from . import _lib

c_int, c_long, c_float, c_void_p = ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_void_p

_SIGS = {
    "p2p_sm_embed_pos": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                         c_void_p],
    "p2p_sm_rmsnorm": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p,
                       c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "p2p_sm_norm_scale_add": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int,
                              c_float, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "p2p_sm_gdelta_scan": [c_void_p] * 5 + [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                            c_int, c_float, c_int, c_void_p],
    "p2p_sm_gdelta_scan_chunked": [c_void_p] * 5 + [c_int, c_void_p, c_int, c_void_p, c_void_p,
                                                    c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                    c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                                    c_float, c_int, c_void_p],
    "p2p_sm_mamba_scan_chunked": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                  c_int, c_void_p],
    "p2p_sm_mamba_conv": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_mamba_scan": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                          c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_mamba_tail": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_void_p],
    "p2p_sm_latent_attn": [c_void_p, c_long, c_long, c_void_p, c_void_p, c_int, c_void_p,
                           c_void_p, c_void_p, c_float, c_int, c_void_p, c_long, c_long, c_int,
                           c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_latent_attn_mfma": [c_void_p, c_long, c_long, c_void_p, c_void_p, c_int, c_void_p,
                                c_void_p, c_void_p, c_int, c_void_p, c_float, c_int, c_void_p,
                                c_long, c_long, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    "p2p_sm_tanh": [c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_sigmoid_gate": [c_void_p, c_long, c_long, c_void_p, c_int, c_void_p, c_int, c_int,
                            c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_ff_act": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_float, c_int,
                      c_void_p],
    "p2p_sm_gate_norm_add": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                             c_int, c_int, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
    "p2p_sm_glu_act": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_relu2_gate": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int,
                          c_void_p],
    "p2p_sm_add_norm": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float,
                        c_void_p, c_void_p, c_int, c_int, c_void_p],
    "p2p_sm_add_norm2": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                         c_int, c_float, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                         c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "p2p_sm_latent_prep": [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                           c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int,
                           c_int, c_void_p],
    "p2p_sm_rope_rows": [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p,
                         c_void_p, c_long, c_long, c_int, c_int, c_void_p],
    "p2p_sm_qtemp_kv_store": [c_void_p, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "p2p_sm_mlstm_scan": [c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                          c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_float,
                          c_int, c_int, c_void_p],
    "p2p_sm_softcap": [c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_float, c_int, c_void_p],
    "p2p_sm_embed_rows": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float,
                          c_int, c_void_p],
    "p2p_sm_qk_norm_rope_store": [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                  c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_float,
                                  c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "p2p_sm_window_attn": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                           c_void_p, c_float, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_int, c_float, c_float, c_void_p, c_void_p, c_void_p, c_int,
                           c_int, c_void_p],
    "p2p_sm_window_attn_mfma": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                c_void_p, c_int, c_void_p, c_float, c_int, c_void_p, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_float,
                                c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    "p2p_sm_hgrn2_scan": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_void_p, c_int, c_int, c_int, c_int, c_float, c_float, c_int,
                          c_void_p],
    "p2p_sm_hgrn2_scan_chunked": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int,
                                  c_int, c_int, c_int, c_float, c_float, c_int, c_void_p],
    "p2p_sm_gated_delta_scan_chunked": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                        c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                        c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_int,
                                        c_void_p],
    "p2p_sm_gated_delta_scan": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_float,
                                c_int, c_void_p],
    "p2p_sm_group_route": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                           c_void_p, c_int, c_void_p],
    "p2p_sm_expert_gemm": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                           c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_int,
                           c_void_p],
    "p2p_sm_expert_combine": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                              c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
}

_lock = threading.Lock()
_so = None


def lib_path() -> str:
    from .. import _build

    return _build.SEQMIX_LIB


def lib():
    """Load (once) the sequence-mixer kernel library; build it first when it is missing.  A
    library that no build of the tree's sources produced is refused (build stamp)."""
    global _so
    if _so is not None:
        return _so
    with _lock:
        if _so is not None:
            return _so
        from .. import _build

        path = _build.SEQMIX_LIB
        if not os.path.exists(path):
            _build.build_seqmix(jobs=min(16, os.cpu_count() or 1))
        srcs, hdrs = _build.seqmix_sources()
        if srcs:
            import json

            try:
                with open(path + ".stamp") as f:
                    ok = json.load(f).get("sources_sha256") == _build.sources_digest(srcs + hdrs)
            except FileNotFoundError:
                ok = False
            if not ok and os.environ.get("P2P_ALLOW_STALE_LIB", "0") != "1":
                raise _lib.KernelError("%s was not built from the tree's csrc/seqmix -- rebuild "
                                       "with `python -m p2p_llm_chat_go_amd._build --only seqmix`"
                                       % path)
        L = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        for name, args in _SIGS.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = c_int
        _so = L
    return _so


def _st(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _f32(t) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError("activations are bfloat16 or float32, got %s" % t.dtype)


def _chk(err, name):
    if err != 0:
        raise _lib.KernelError("%s failed with hipError %d" % (name, err))


def _rows2d(t, name):
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError("%s must be a row-major 2-d view" % name)


def _vec(t, n, name):
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise ValueError("%s must be a contiguous float32 vector of %d" % (name, n))


def _rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


# ------------------------------------------------------------------ embedding / norms
def embed_pos(embed, pos_table, ids, pos, out):
    """out[r] = embed[ids[r]] (+ pos_table[pos[r]]) as fp32 rows."""
    R, W = out.shape
    if not out.is_cuda:
        v = embed[ids.long()].float()
        if pos_table is not None:
            v = v + pos_table[pos.long()].float()
        out.copy_(v)
        return out
    assert out.dtype == torch.float32 and out.is_contiguous() and embed.shape[1] == W
    assert ids.dtype == torch.int32 and pos.dtype == torch.int32 and ids.numel() >= R
    assert embed.is_contiguous() and (pos_table is None or (pos_table.is_contiguous()
                                                           and pos_table.dtype == embed.dtype))
    _chk(lib().p2p_sm_embed_pos(embed.data_ptr(), _lib.ptr(pos_table), ids.data_ptr(),
                                pos.data_ptr(), out.data_ptr(), R, W, _f32(embed), _st(out)),
         "embed_pos")
    return out


def embed_rows(embed, ids, out, h_out=None, scale: float = 1.0):
    """out[r] = embed[ids[r]] * scale as fp32 rows; h_out (activation type, optional): the same
    rows for a first sublayer that reads the residual stream as it is."""
    R, W = out.shape
    if not out.is_cuda:
        out.copy_(embed[ids[:R].long()].float() * scale)
        if h_out is not None:
            h_out[:R] = out.to(h_out.dtype)
        return out
    assert out.dtype == torch.float32 and out.is_contiguous() and embed.shape[1] == W
    assert ids.dtype == torch.int32 and ids.numel() >= R and embed.is_contiguous()
    ldh = 0
    if h_out is not None:
        _rows2d(h_out, "h_out")
        assert h_out.dtype == embed.dtype and h_out.shape[1] == W and h_out.shape[0] >= R
        ldh = h_out.stride(0)
    _chk(lib().p2p_sm_embed_rows(embed.data_ptr(), ids.data_ptr(), out.data_ptr(),
                                 _lib.ptr(h_out), ldh, R, W, scale, _f32(embed), _st(out)),
         "embed_rows")
    return out


def rmsnorm(x, w, eps, out, parts: int = 1, in_rows=None, out_rows=None):
    """out[o(r)] = x[i(r)] / sqrt(mean(x^2) + eps) * w, the mean taken over each of ``parts``
    equal parts of the row.  x: fp32 or activation type; out: activation type (or fp32).
    in_rows / out_rows: int32 row gathers / scatters (out row < 0: dropped)."""
    R = (in_rows if in_rows is not None else x).shape[0]
    n = x.shape[1]
    if not x.is_cuda:
        xs = x.float() if in_rows is None else x[in_rows.long()].float()
        v = _rms(xs.view(R, parts, n // parts), eps).reshape(R, n)
        if w is not None:
            v = v * w
        v = v.to(out.dtype)
        if out_rows is None:
            out[:R] = v
        else:
            keep = out_rows >= 0
            out[out_rows[keep].long()] = v[keep]
        return out
    _rows2d(x, "x")
    _rows2d(out, "out")
    if w is not None:
        _vec(w, n, "w")
    if n % parts:
        raise ValueError("row of %d does not split into %d parts" % (n, parts))
    assert out.shape[1] == n and (out_rows is not None or out.shape[0] >= R)
    _chk(lib().p2p_sm_rmsnorm(x.data_ptr(), x.stride(0), _f32(x), _lib.ptr(w), out.data_ptr(),
                              out.stride(0), _f32(out), _lib.ptr(in_rows), _lib.ptr(out_rows), R,
                              n, parts, eps, _st(x)), "rmsnorm")
    return out


def norm_scale_add(x, y, w, ls, eps, next_w=None, next_out=None):
    """x += y / sqrt(mean(y^2) + eps) * w * ls on the fp32 residual x (ls may be None).
    With next_w / next_out also the next sublayer's input in the same pass:
    next_out = x / sqrt(mean(x^2) + eps) * next_w from the updated rows."""
    R, n = x.shape
    if not x.is_cuda:
        v = _rms(y.float(), eps) * w
        if ls is not None:
            v = v * ls
        x += v
        if next_w is not None:
            next_out[:R] = (_rms(x, eps) * next_w).to(next_out.dtype)
        return x
    _rows2d(y, "y")
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == x.shape
    _vec(w, n, "w")
    if ls is not None:
        _vec(ls, n, "ls")
    ldh = 0
    if next_w is not None:
        _vec(next_w, n, "next_w")
        _rows2d(next_out, "next_out")
        assert next_out.dtype == y.dtype and next_out.shape[1] == n and next_out.shape[0] >= R
        ldh = next_out.stride(0)
    _chk(lib().p2p_sm_norm_scale_add(x.data_ptr(), y.data_ptr(), y.stride(0), w.data_ptr(),
                                     _lib.ptr(ls), R, n, eps, _lib.ptr(next_w),
                                     _lib.ptr(next_out if next_w is not None else None), ldh,
                                     _f32(y), _st(x)), "norm_scale_add")
    return x


def add_norm(x, a, b=None, eps: float = 0.0, next_w=None, next_out=None):
    """x += a (+ b) on the fp32 residual x, the addends summed first in fp32.  With next_w /
    next_out also the next layer's input in the same pass:
    next_out = x / sqrt(mean(x^2) + eps) * next_w from the updated rows."""
    R, n = x.shape
    if not x.is_cuda:
        y = a[:R].float()
        if b is not None:
            y = y + b[:R].float()
        x += y
        if next_w is not None:
            next_out[:R] = (_rms(x, eps) * next_w).to(next_out.dtype)
        return x
    _rows2d(a, "a")
    assert x.dtype == torch.float32 and x.is_contiguous() and a.shape[1] == n and a.shape[0] >= R
    ldb = 0
    if b is not None:
        _rows2d(b, "b")
        assert b.shape[1] == n and b.shape[0] >= R and b.dtype == a.dtype
        ldb = b.stride(0)
    ldh = 0
    if next_w is not None:
        _vec(next_w, n, "next_w")
        _rows2d(next_out, "next_out")
        assert next_out.dtype == a.dtype and next_out.shape[1] == n and next_out.shape[0] >= R
        ldh = next_out.stride(0)
    _chk(lib().p2p_sm_add_norm(x.data_ptr(), a.data_ptr(), a.stride(0), _lib.ptr(b), ldb, R, n, eps,
                               _lib.ptr(next_w), _lib.ptr(next_out if next_w is not None else None),
                               ldh, _f32(a), _st(x)), "add_norm")
    return x


def add_norm2(x, a=None, b=None, rows=None, vec=None, eps: float = 0.0, w1=None, out1=None,
              w2=None, out2=None, routed=None):
    """x += a + b + rows + vec + routed on the fp32 residual x (every addend optional; a, b
    activation typed [R, n], rows fp32 [R, n], vec fp32 [n]; routed = (y, wts): the weighted
    sum over a token's routed experts, sum_k wts[r, k] * y[r * top + k], y activation typed
    [R * top, n], wts fp32 [R, top]; they are summed in fp32 before they meet x), then up to two normed copies of the updated rows in the same pass,
    out_i = x / sqrt(mean(x^2) + eps) * w_i, each w_i fp32 with n numbers or a single one for
    all channels: the inputs of two sublayers that read the same rows through norms of
    their own."""
    R, n = x.shape
    if (w1 is None) != (out1 is None) or (w2 is None) != (out2 is None) or (w2 is not None and w1 is None):
        raise ValueError("add_norm2: a norm weight goes with its output, the first before the second")
    if not x.is_cuda:
        y = None
        for t in (a, b, rows):
            if t is not None:
                y = t[:R].float() if y is None else y + t[:R].float()
        if vec is not None:
            y = vec if y is None else y + vec
        if routed is not None:
            ry, rw = routed
            t = (ry[:R * rw.shape[1]].float().view(R, rw.shape[1], n) * rw[:R, :, None]).sum(1)
            y = t if y is None else y + t
        if y is not None:
            x += y
        for w, o in ((w1, out1), (w2, out2)):
            if w is not None:
                o[:R] = (_rms(x, eps) * w).to(o.dtype)
        return x
    assert x.dtype == torch.float32 and x.is_contiguous()
    lda = ldb = 0
    if a is not None:
        _rows2d(a, "a")
        assert a.shape[1] == n and a.shape[0] >= R
        lda = a.stride(0)
    if b is not None:
        _rows2d(b, "b")
        assert a is not None and b.shape[1] == n and b.shape[0] >= R and b.dtype == a.dtype
        ldb = b.stride(0)
    if rows is not None:
        assert rows.dtype == torch.float32 and rows.is_contiguous() and rows.shape == x.shape
    if vec is not None:
        _vec(vec, n, "vec")
    cy = cw = None
    ldcy = top = 0
    if routed is not None:
        cy, cw = routed
        top = cw.shape[1]
        _rows2d(cy, "routed y")
        assert cy.shape[1] == n and cy.shape[0] >= R * top and (a is None or cy.dtype == a.dtype)
        assert cw.dtype == torch.float32 and cw.is_contiguous() and cw.shape[0] >= R
        ldcy = cy.stride(0)
    ld1 = ld2 = 0
    for w, o, nm in ((w1, out1, "w1"), (w2, out2, "w2")):
        if w is not None:
            assert w.dtype == torch.float32 and w.is_contiguous() and w.numel() in (1, n), nm
            _rows2d(o, "out")
            assert o.shape[1] == n and o.shape[0] >= R and o.dtype == out1.dtype
            assert (a is None or o.dtype == a.dtype) and (cy is None or o.dtype == cy.dtype)
    if out1 is not None:
        ld1 = out1.stride(0)
    if out2 is not None:
        ld2 = out2.stride(0)
    act = a if a is not None else cy if cy is not None else out1
    _chk(lib().p2p_sm_add_norm2(x.data_ptr(), _lib.ptr(a), lda, _lib.ptr(b), ldb, _lib.ptr(rows),
                                _lib.ptr(vec), R, n, eps, _lib.ptr(w1),
                                1 if w1 is not None and w1.numel() > 1 else 0, _lib.ptr(out1), ld1,
                                _lib.ptr(w2), 1 if w2 is not None and w2.numel() > 1 else 0,
                                _lib.ptr(out2), ld2, _lib.ptr(cy), ldcy, _lib.ptr(cw), top,
                                _f32(act) if act is not None else 1, _st(x)),
         "add_norm2")
    return x


# ------------------------------------------------------------------ pointwise
def tanh_(x):
    if not x.is_cuda:
        x.copy_(torch.tanh(x.float()).to(x.dtype))
        return x
    _rows2d(x, "x")
    _chk(lib().p2p_sm_tanh(x.data_ptr(), x.stride(0), x.shape[1], x.shape[0], _f32(x), _st(x)),
         "tanh")
    return x


def sigmoid_gate(o, g, out, H: int, V: int, per_head: bool = False):
    """out[r, h*V + v] = o[h, r, v] * sigmoid(g[r, h*V + v]), or with ``per_head`` one gate for
    all channels of a head, sigmoid(g[r, h]); o is any [H, R, V] view whose last stride is 1."""
    R = g.shape[0]
    if not g.is_cuda:
        gg = torch.sigmoid(g.float())
        if per_head:
            gg = gg[:, :H].repeat_interleave(V, 1)
        out.copy_((o.float().permute(1, 0, 2).reshape(R, H * V) * gg).to(out.dtype))
        return out
    _rows2d(g, "g")
    _rows2d(out, "out")
    assert o.shape == (H, R, V) and o.stride(2) == 1 and o.dtype == g.dtype == out.dtype
    assert g.shape[1] >= (H if per_head else H * V)
    _chk(lib().p2p_sm_sigmoid_gate(o.data_ptr(), o.stride(0), o.stride(1), g.data_ptr(),
                                   g.stride(0), out.data_ptr(), out.stride(0), R, H, V,
                                   1 if per_head else 0, _f32(g), _st(g)), "sigmoid_gate")
    return out


def ff_act(gu, out, limit: float, alpha: float = 1.702):
    """[gate | up] -> min(gate, limit) * sigmoid(alpha * .) * (clamp(up, +-limit) + 1)."""
    R, F = out.shape
    if not gu.is_cuda:
        g = torch.clamp(gu[:, :F].float(), max=limit)
        u = torch.clamp(gu[:, F:].float(), -limit, limit)
        out.copy_((g * torch.sigmoid(alpha * g) * (u + 1)).to(out.dtype))
        return out
    _rows2d(gu, "gu")
    _rows2d(out, "out")
    assert gu.shape == (R, 2 * F) and gu.dtype == out.dtype
    _chk(lib().p2p_sm_ff_act(gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), R, F,
                             limit, alpha, _f32(gu), _st(gu)), "ff_act")
    return out


# ------------------------------------------------------------------ recurrences in chunks
# A portion of at least 2 * SCAN_CHUNK tokens is scanned in chunks of SCAN_CHUNK tokens that
# run side by side (local pass, chain over the chunks, output pass); shorter steps -- decode,
# small portions -- walk their tokens in one pass.  Both recurrences are linear in the state,
# so the chunked form computes the same sums in another order (fp32 throughout).
SCAN_CHUNK = int(os.environ.get("P2P_SCAN_CHUNK", "64"))


def scan_chunks(ent_host: list, chunk: int):
    """(chunks as entries [(row0, n, 1, chunk index)], per entry (first chunk, chunks, first
    position, slot)) as int32 tensors."""
    vent, cent = [], []
    for row0, n, start, slot in ent_host:
        c0 = len(vent)
        for r in range(row0, row0 + n, chunk):
            vent.append((r, min(chunk, row0 + n - r), 1, len(vent)))
        cent.append((c0, len(vent) - c0, start, slot))
    return torch.tensor(vent, dtype=torch.int32), torch.tensor(cent, dtype=torch.int32)


def _chunked(ent_host) -> bool:
    return SCAN_CHUNK > 0 and max(e[1] for e in ent_host) >= 2 * SCAN_CHUNK


# ------------------------------------------------------------------ generalized delta rule
GD_DECAY_SCALE = math.exp(-0.5)


def gdelta_scan(r, k, v, g, a, lo, w0, ab, normw, state, ent, ent_host, out, H: int, D: int,
                eps: float):
    """Generalized delta rule over the entries of a step, state carried in ``state`` slots.

    r, k, v, g, a: [R, H*D] views of one projection buffer (same row stride); lo [R, H*D] the
    decay logits before their bias w0; ab the removal-rate bias; normw the output weight.
    state fp32 [slots, H, D, D] (key index, value index).  ent_host: the entries as a list of
    (row0, n, start, slot) (the CPU path walks it; the kernel reads ``ent``)."""
    if not r.is_cuda:
        for row0, n, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            for t in range(row0, row0 + n):
                rr, kk, vv = (z[t].float().view(H, D) for z in (r, k, v))
                w = torch.exp(-GD_DECAY_SCALE * torch.sigmoid(lo[t].float() + w0)).view(H, D)
                aa = torch.sigmoid(a[t].float() + ab).view(H, D)
                u = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
                uS = torch.einsum("hk,hkv->hv", u, S)
                S = w[:, :, None] * S - (aa * u)[:, :, None] * uS[:, None, :] \
                    + kk[:, :, None] * vv[:, None, :]
                o = torch.einsum("hkv,hk->hv", S, rr)
                o = _rms(o, eps).reshape(H * D) * normw * torch.sigmoid(g[t].float())
                out[t] = o.to(out.dtype)
            state[slot] = S
        return out
    n = H * D
    for t_, nm in ((r, "r"), (k, "k"), (v, "v"), (g, "g"), (a, "a"), (lo, "lo"), (out, "out")):
        _rows2d(t_, nm)
        assert t_.shape[1] == n and t_.dtype == r.dtype, nm
    ld = r.stride(0)
    assert all(t_.stride(0) == ld for t_ in (k, v, g, a))
    for t_, nm in ((w0, "w0"), (ab, "ab"), (normw, "normw")):
        _vec(t_, n, nm)
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D)
    E = ent.shape[0]
    assert ent.dtype == torch.int32 and ent.is_contiguous() and ent.shape[1] == 4
    if D > 256:
        raise ValueError("gdelta_scan: head size %d > 256" % D)
    if _chunked(ent_host):
        vent, cent = (t_.to(r.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        tmp = torch.empty(3, vent.shape[0], H, D, D, device=r.device, dtype=torch.float32)
        _chk(lib().p2p_sm_gdelta_scan_chunked(
            r.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), a.data_ptr(), ld,
            lo.data_ptr(), lo.stride(0), w0.data_ptr(), ab.data_ptr(), normw.data_ptr(),
            state.data_ptr(), tmp.data_ptr(), vent.data_ptr(), vent.shape[0], cent.data_ptr(), E,
            out.data_ptr(), out.stride(0), H, D, eps, _f32(r), _st(r)), "gdelta_scan_chunked")
        return out
    _chk(lib().p2p_sm_gdelta_scan(r.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(),
                                  a.data_ptr(), ld, lo.data_ptr(), lo.stride(0), w0.data_ptr(),
                                  ab.data_ptr(), normw.data_ptr(), state.data_ptr(),
                                  ent.data_ptr(), E, out.data_ptr(), out.stride(0), H, D, eps,
                                  _f32(r), _st(r)), "gdelta_scan")
    return out


# ------------------------------------------------------------------ Mamba-2
def mamba_conv(zx, xoff: int, cw, cb, tail, ent, ent_host, row_ent, out):
    """Causal per-channel convolution + bias + silu over channels [xoff, xoff + C) of zx.
    cw fp32 [C, K] (column K-1 multiplies the newest input), tail fp32 [slots, K-1, C] the raw inputs
    before each slot's next token (read only here; ``mamba_scan`` rolls it)."""
    R, C = out.shape
    K = cw.shape[1]
    if not zx.is_cuda:
        for row0, n, start, slot in ent_host:
            raw = zx[row0:row0 + n, xoff:xoff + C].float()
            prev = tail[slot] if start > 0 else torch.zeros(K - 1, C)
            pad = torch.cat([prev, raw], 0)
            acc = cb.clone().expand(n, C).clone()
            for kk in range(K):
                acc += pad[kk:kk + n] * cw[:, kk]
            out[row0:row0 + n] = acc * torch.sigmoid(acc)
        return out
    _rows2d(zx, "zx")
    assert out.dtype == torch.float32 and out.is_contiguous()
    assert cw.dtype == torch.float32 and cw.is_contiguous() and cw.shape[0] == C
    _vec(cb, C, "cb")
    assert tail.dtype == torch.float32 and tail.is_contiguous() and tail.shape[1:] == (K - 1, C)
    assert xoff + C <= zx.shape[1] and row_ent.dtype == torch.int32
    _chk(lib().p2p_sm_mamba_conv(zx.data_ptr(), zx.stride(0), xoff, cw.data_ptr(), cb.data_ptr(),
                                 tail.data_ptr(), ent.data_ptr(), row_ent.data_ptr(),
                                 out.data_ptr(), R, C, K, _f32(zx), _st(zx)), "mamba_conv")
    return out


def conv_tail_roll(zx, xoff: int, tail, ent, ent_host, C: int):
    """After a step's convolutions: every entry's slot keeps the raw inputs (channels
    [xoff, xoff + C) of zx) of its last K-1 tokens, older ones shifted out.  tail fp32
    [slots, K-1, C]."""
    Km1 = tail.shape[1]
    if Km1 == 0:
        return tail
    if not zx.is_cuda:
        for row0, n, start, slot in ent_host:
            raw = zx[row0:row0 + n, xoff:xoff + C].float()
            prev = tail[slot] if start > 0 else torch.zeros(Km1, C)
            tail[slot] = torch.cat([prev, raw], 0)[-Km1:]
        return tail
    _rows2d(zx, "zx")
    assert tail.dtype == torch.float32 and tail.is_contiguous() and tail.shape[2] == C
    assert xoff + C <= zx.shape[1]
    _chk(lib().p2p_sm_mamba_tail(zx.data_ptr(), zx.stride(0), xoff, tail.data_ptr(),
                                 ent.data_ptr(), ent.shape[0], C, Km1 + 1, _f32(zx), _st(zx)),
         "conv_tail_roll")
    return tail


def mamba_scan(conv, zx, xoff: int, dtoff: int, dt_bias, A_log, Dp, state, tail, ent, ent_host,
               y, H: int, P: int, N: int, G: int):
    """Selective state-space scan.  conv fp32 [R, H*P + 2*G*N] = silu(conv(x | B | C)); zx the
    input projection (z at column 0, raw x|B|C at xoff, dt at dtoff).  state fp32
    [slots, H, N, P].  Writes y * silu(z) as fp32 [R, H*P] and rolls the convolution tail."""
    R, C = conv.shape
    inner = H * P
    Km1 = tail.shape[1]
    if not conv.is_cuda:
        hg = H // G
        A = -torch.exp(A_log)
        for row0, n, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            for t in range(row0, row0 + n):
                x = conv[t, :inner].view(H, P)
                B = conv[t, inner:inner + G * N].view(G, N).repeat_interleave(hg, 0)
                Cc = conv[t, inner + G * N:].view(G, N).repeat_interleave(hg, 0)
                dt = torch.nn.functional.softplus(zx[t, dtoff:dtoff + H].float() + dt_bias,
                                                  threshold=1e9)
                S = torch.exp(A * dt)[:, None, None] * S + (dt[:, None] * B)[:, :, None] * x[:, None, :]
                yy = torch.einsum("hnp,hn->hp", S, Cc) + Dp[:, None] * x
                z = zx[t, :inner].float()
                y[t] = yy.reshape(inner) * (z * torch.sigmoid(z))
            state[slot] = S
            if Km1:
                raw = zx[row0:row0 + n, xoff:xoff + C].float()
                prev = tail[slot] if start > 0 else torch.zeros(Km1, C)
                tail[slot] = torch.cat([prev, raw], 0)[-Km1:]
        return y
    _rows2d(zx, "zx")
    assert conv.dtype == torch.float32 and conv.is_contiguous() and C == inner + 2 * G * N
    assert y.dtype == torch.float32 and y.is_contiguous() and y.shape == (R, inner)
    for t_, nm in ((dt_bias, "dt_bias"), (A_log, "A_log"), (Dp, "D")):
        _vec(t_, H, nm)
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, N, P)
    assert tail.dtype == torch.float32 and tail.is_contiguous() and tail.shape[2] == C
    assert dtoff + H <= zx.shape[1] and xoff + C <= zx.shape[1] and H % G == 0
    if N > 256 or P > 256:
        raise ValueError("mamba_scan: state %d / value %d sizes above 256" % (N, P))
    E = ent.shape[0]
    if _chunked(ent_host):
        vent, cent = (t_.to(zx.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        NV = vent.shape[0]
        tmp = torch.empty(NV, H, N, P, device=zx.device, dtype=torch.float32)
        decay = torch.empty(NV, H, device=zx.device, dtype=torch.float32)
        _chk(lib().p2p_sm_mamba_scan_chunked(
            conv.data_ptr(), C, zx.data_ptr(), zx.stride(0), xoff, dtoff, dt_bias.data_ptr(),
            A_log.data_ptr(), Dp.data_ptr(), state.data_ptr(), tmp.data_ptr(), decay.data_ptr(),
            vent.data_ptr(), NV, cent.data_ptr(), E, y.data_ptr(), H, P, N, G, _f32(zx),
            _st(zx)), "mamba_scan_chunked")
    else:
        _chk(lib().p2p_sm_mamba_scan(conv.data_ptr(), C, zx.data_ptr(), zx.stride(0), xoff, dtoff,
                                     dt_bias.data_ptr(), A_log.data_ptr(), Dp.data_ptr(),
                                     state.data_ptr(), tail.data_ptr(), ent.data_ptr(), E,
                                     y.data_ptr(), H, P, N, G, Km1 + 1, _f32(zx), _st(zx)),
             "mamba_scan")
    _chk(lib().p2p_sm_mamba_tail(zx.data_ptr(), zx.stride(0), xoff, tail.data_ptr(),
                                 ent.data_ptr(), E, C, Km1 + 1, _f32(zx), _st(zx)), "mamba_tail")
    return y


# ------------------------------------------------------------------ latent attention
def latent_attn_ok(H: int, rank: int) -> bool:
    """One head's query, a tile of 4 keys and the accumulators must fit a block."""
    return rank <= 32 * 256 and (rank + 4 * (rank + 1) + 4 + 3) * 4 <= 64 * 1024


def latent_rows_per_wave(H: int) -> int:
    """Rows of one sequence portion that a wavefront of the matrix-core kernel takes: its 16
    (row, head) pairs are RW rows x HS head slots, HS the power of two >= min(H, 16)."""
    hs = 1
    while hs < H and hs < 16:
        hs *= 2
    return 16 // hs


def make_units(ent_host: list, rows_per_wave: int) -> torch.Tensor:
    """int32 [U, 2] (first row, rows): the entries' rows cut into groups of at most
    ``rows_per_wave`` consecutive rows; a group never spans two entries."""
    u = [(r, min(rows_per_wave, row0 + n - r)) for row0, n, _s, _sl in ent_host
         for r in range(row0, row0 + n, rows_per_wave)]
    return torch.tensor(u, dtype=torch.int32).view(-1, 2)


def latent_mfma_ok(qa, cache) -> bool:
    """The matrix-core kernel serves bf16 activations with a latent size that is a multiple
    of 8 up to 512 and 16-byte aligned rows; everything else (and float32) runs the fp32
    kernel.  P2P_LATENT_MFMA=0 switches it off."""
    rank = qa.shape[2]
    return (qa.is_cuda and qa.dtype == torch.bfloat16 and rank % 8 == 0 and 8 <= rank <= 512
            and qa.stride(0) % 8 == 0 and qa.stride(1) % 8 == 0 and qa.data_ptr() % 16 == 0
            and cache.data_ptr() % 16 == 0 and os.environ.get("P2P_LATENT_MFMA", "1") != "0")


LATENT_SPLIT_BLOCKS = 512   # split windows while a step has fewer blocks than this


def latent_attn(qa, cache, block_tables, row_ent, pos, sink, scale: float, win: int, out,
                page: int, units=None, max_keys=None):
    """Windowed attention over cached latents with a softmax sink.

    qa [H, R, rank] (any strides, last = 1): the queries already carried into latent space
    (W_uk^T q per head); cache [tokens, rank] one layer's latent pool, token t of a sequence
    at block_tables[e, t // page] * page + t % page.  out [H, R, rank] = sum_j p_j c_j with
    p = softmax over {sink_h} U {scale * qa . c_j : 0 <= pos - j < win}, the sink term having
    no value (sink None: an ordinary softmax over the visible keys).  A layer whose keys have a
    part outside the latent (a rotated part shared by the heads) appends it to the cached row and
    the matching query part to qa; the columns of out beyond the latent are then not used.
    units: ``make_units(entries, latent_rows_per_wave(H))`` on the device; with
    it, bf16 inputs run on the matrix cores (``latent_mfma_ok``).  max_keys: an upper bound of
    the keys any row sees (host side; lets a step of few rows split its windows)."""
    H, R, rank = qa.shape
    if not qa.is_cuda:
        bt = block_tables.long()
        for r in range(R):
            p = int(pos[r])
            lo = max(0, p - win + 1)
            j = torch.arange(lo, p + 1)
            tok = bt[int(row_ent[r])][j // page] * page + j % page
            c = cache[tok].float()                                  # [n, rank]
            s = (qa[:, r].float() @ c.T) * scale                    # [H, n]
            m = s.max(-1).values if sink is None else torch.maximum(s.max(-1).values, sink)
            e = torch.exp(s - m[:, None])
            den = e.sum(-1) if sink is None else e.sum(-1) + torch.exp(sink - m)
            out[:, r] = ((e / den[:, None]) @ c).to(out.dtype)
        return out
    assert qa.stride(2) == 1 and out.stride(2) == 1 and out.shape == qa.shape
    assert qa.dtype == cache.dtype == out.dtype
    assert cache.dim() == 2 and cache.is_contiguous() and cache.shape[1] == rank
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous()
    assert row_ent.dtype == torch.int32 and pos.dtype == torch.int32
    if sink is not None:
        _vec(sink, H, "sink")
    if units is not None and latent_mfma_ok(qa, cache):
        assert units.dtype == torch.int32 and units.is_contiguous() and units.shape[1] == 2
        # few row groups with long windows (decode): cut every window into runs of key tiles
        # so that the step fills the chip; the runs are merged by a second small kernel
        U = units.shape[0]
        hg = -(-H // (16 // latent_rows_per_wave(H)))
        splits = 1
        if max_keys is not None and U * hg < LATENT_SPLIT_BLOCKS:
            splits = max(1, min(-(-min(max_keys, win) // 64), LATENT_SPLIT_BLOCKS // (U * hg), 64))
        part = None
        if splits > 1:
            L = lib()
            L.p2p_sm_latent_attn_mfma_ws.restype = c_long
            n = L.p2p_sm_latent_attn_mfma_ws(U, H, rank, splits)
            part = torch.empty(n, device=qa.device, dtype=torch.float32)
        _chk(lib().p2p_sm_latent_attn_mfma(qa.data_ptr(), qa.stride(0), qa.stride(1),
                                           cache.data_ptr(), block_tables.data_ptr(),
                                           block_tables.shape[1], row_ent.data_ptr(),
                                           pos.data_ptr(), units.data_ptr(), units.shape[0],
                                           _lib.ptr(sink), scale, win, out.data_ptr(),
                                           out.stride(0), out.stride(1), H, rank, page, splits,
                                           _lib.ptr(part), _st(qa)),
             "latent_attn_mfma")
        return out
    if not latent_attn_ok(H, rank):
        raise ValueError("latent_attn: %d heads x latent %d exceed the kernel's tile" % (H, rank))
    _chk(lib().p2p_sm_latent_attn(qa.data_ptr(), qa.stride(0), qa.stride(1), cache.data_ptr(),
                                  block_tables.data_ptr(), block_tables.shape[1],
                                  row_ent.data_ptr(), pos.data_ptr(), _lib.ptr(sink), scale,
                                  win, out.data_ptr(), out.stride(0), out.stride(1), R, H, rank,
                                  page, _f32(qa), _st(qa)), "latent_attn")
    return out


# ------------------------------------------------------------------ post-norm gated residual
def gate_norm_add(x, y, g, gb, w, parts: int, eps: float, next_out=None):
    """x += N(y * sigmoid(g + gb)) * w on the fp32 residual x, N the RMS norm taken separately
    over ``parts`` equal parts of the row.  y, g: activation-typed [R, n] (g the gate's
    projection before its bias gb).  next_out (activation type): the updated rows, which the
    next sublayer takes as its input without a norm of its own."""
    R, n = x.shape
    if not x.is_cuda:
        v = y.float() * torch.sigmoid(g.float() + gb)
        x += _rms(v.view(R, parts, n // parts), eps).reshape(R, n) * w
        if next_out is not None:
            next_out[:R] = x.to(next_out.dtype)
        return x
    _rows2d(y, "y")
    _rows2d(g, "g")
    assert x.dtype == torch.float32 and x.is_contiguous() and y.shape == x.shape == g.shape
    assert y.dtype == g.dtype
    _vec(w, n, "w")
    _vec(gb, n, "gb")
    if parts < 1 or n % parts:
        raise ValueError("row of %d does not split into %d parts" % (n, parts))
    ldh = 0
    if next_out is not None:
        _rows2d(next_out, "next_out")
        assert next_out.shape[1] == n and next_out.shape[0] >= R
        ldh = next_out.stride(0)
    _chk(lib().p2p_sm_gate_norm_add(x.data_ptr(), y.data_ptr(), y.stride(0), g.data_ptr(),
                                    g.stride(0), gb.data_ptr(), w.data_ptr(), R, n, parts, eps,
                                    _lib.ptr(next_out), ldh,
                                    _f32(next_out) if next_out is not None else 0, _f32(y),
                                    _st(x)), "gate_norm_add")
    return x


GLU_ACTS = {"silu": 0, "gelu_tanh": 1}


def glu_act(gu, out, act: str = "silu"):
    """[gate | up] -> act(gate) * up; act: "silu", or "gelu_tanh" =
    0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""
    R, F = out.shape
    code = GLU_ACTS[act]
    if not gu.is_cuda:
        g = gu[:, :F].float()
        a = g * torch.sigmoid(g) if code == 0 else \
            0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
        out.copy_((a * gu[:, F:2 * F].float()).to(out.dtype))
        return out
    _rows2d(gu, "gu")
    _rows2d(out, "out")
    assert gu.shape[0] == R and gu.shape[1] >= 2 * F and gu.dtype == out.dtype
    _chk(lib().p2p_sm_glu_act(gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), R, F,
                              code, _f32(gu), _st(gu)), "glu_act")
    return out


def relu2_gate(u, g, out):
    """out[r, c] = relu(u[r, c])^2 * sigmoid(g[r]): an ungated squared-relu unit weighted by one
    gate per row (g: an [R, 1] view, or None for no gate)."""
    R, F = out.shape
    if not u.is_cuda:
        v = torch.relu(u[:R, :F].float()) ** 2
        if g is not None:
            v = v * torch.sigmoid(g[:R, :1].float())
        out.copy_(v.to(out.dtype))
        return out
    _rows2d(u, "u")
    _rows2d(out, "out")
    assert u.shape[0] == R and u.shape[1] >= F and u.dtype == out.dtype
    ldg = 0
    if g is not None:
        assert g.dim() == 2 and g.shape[0] == R and g.dtype == u.dtype
        ldg = g.stride(0)
    _chk(lib().p2p_sm_relu2_gate(u.data_ptr(), u.stride(0), _lib.ptr(g), ldg, out.data_ptr(),
                                 out.stride(0), R, F, _f32(u), _st(u)), "relu2_gate")
    return out


def softcap(y, cap: float, out, scale: float = 1.0):
    """out = cap * tanh(scale * y / cap) as fp32 (y: activation-typed or fp32 logits); cap 0:
    out = scale * y."""
    if not y.is_cuda:
        z = y.float() * scale
        out.copy_(cap * torch.tanh(z / cap) if cap else z)
        return out
    _rows2d(y, "y")
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape == y.shape
    _chk(lib().p2p_sm_softcap(y.data_ptr(), y.stride(0), out.data_ptr(), y.shape[0], y.shape[1],
                              cap, scale, _f32(y), _st(y)), "softcap")
    return out


# ------------------------------------------------------------------ windowed attention
def rope_inv_freq(base: float, dims: int, device, scaling: dict | None = None) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, evaluated in float64 and rounded to fp32.

    scaling = {factor, low, high, original} stretches the long wavelengths: with l = 2 pi / f,
    f stays where l < original / high, becomes f / factor where l > original / low, and in
    between is (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if scaling:
        fac, lo, hi = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        orig = float(scaling["original"])
        wl = 2.0 * math.pi / f
        s = (orig / wl - lo) / (hi - lo) if hi != lo else torch.zeros_like(f)
        mid = (1.0 - s) * f / fac + s * f
        f = torch.where(wl < orig / hi, f, torch.where(wl > orig / lo, f / fac, mid))
    return f.float().to(device)


def rope_rows(src, heads: int, src_hs: int, inv_freq, pos, dst, dst_hs: int, out_rows=None):
    """Rotary positions on a stretch of channels: for every row r and head h < heads the
    pairs (2i, 2i+1), i < len(inv_freq), of src[r, h*src_hs : ...] are turned by the angle
    pos[r] * inv_freq[i], (a, b) -> (a cos - b sin, b cos + a sin) in fp32, and written to
    dst[o(r), h*dst_hs : ...]; o(r) = out_rows[r] (a scatter, e.g. into a paged pool) or r.
    src and dst are 2-d views that start at the first rotated channel of head 0 (last stride
    1; a head may lie anywhere from there, also beyond the view's own width)."""
    R = src.shape[0]
    nrot = inv_freq.numel()
    if nrot == 0 or heads == 0:
        return dst
    if not src.is_cuda:
        ang = pos[:R].float()[:, None] * inv_freq[None, :]
        c, sn = torch.cos(ang), torch.sin(ang)
        ro = torch.arange(R) if out_rows is None else out_rows[:R].long()
        sv = torch.as_strided(src, (R, heads, 2 * nrot), (src.stride(0), src_hs, 1), src.storage_offset())
        dv = torch.as_strided(dst, (dst.shape[0], heads, 2 * nrot), (dst.stride(0), dst_hs, 1),
                              dst.storage_offset())
        a, b = sv[:, :, 0::2].float(), sv[:, :, 1::2].float()
        res = torch.stack([a * c[:, None] - b * sn[:, None], b * c[:, None] + a * sn[:, None]], -1)
        dv[ro] = res.reshape(R, heads, 2 * nrot).to(dst.dtype)
        return dst
    assert src.dim() == 2 and dst.dim() == 2 and src.stride(1) == 1 and dst.stride(1) == 1
    assert src.dtype == dst.dtype and pos.dtype == torch.int32
    assert inv_freq.dtype == torch.float32 and inv_freq.is_contiguous()
    assert out_rows is None or (out_rows.dtype == torch.int32 and out_rows.numel() >= R)
    assert pos.numel() >= R
    _chk(lib().p2p_sm_rope_rows(src.data_ptr(), src.stride(0), heads, src_hs, inv_freq.data_ptr(),
                                nrot, pos.data_ptr(), _lib.ptr(out_rows), dst.data_ptr(),
                                dst.stride(0), dst_hs, R, _f32(src), _st(src)), "rope_rows")
    return dst


def latent_prep(proj, nq: int, nc: int, nr: int, qw, cw, inv_freq, pos, cache_rows, pool, eps: float,
                cq_out):
    """Input pass of latent attention with low-rank queries.  proj = [query latent (nq) |
    key/value latent (nc) | key part (nr)] per row: both latents are RMS-normalised by
    themselves and weighted (qw [nq], cw [nc]); the pairs (2i, 2i+1), i < len(inv_freq), of the
    key part are turned by pos * inv_freq[i] (its other channels pass unchanged).  The query
    latent goes to cq_out [R, nq], the key/value latent and the key part to the rows
    ``cache_rows`` of the paged pool ([tokens, nc + nr]).  Norms, angles, rotation: fp32."""
    R = cq_out.shape[0]
    nrot = inv_freq.numel()
    if not proj.is_cuda:
        rows = cache_rows[:R].long()
        cq_out[:R] = (_rms(proj[:R, :nq].float(), eps) * qw).to(cq_out.dtype)
        pool[rows, :nc] = (_rms(proj[:R, nq:nq + nc].float(), eps) * cw).to(pool.dtype)
        k = proj[:R, nq + nc:nq + nc + nr].float().clone()
        ang = pos[:R].float()[:, None] * inv_freq[None, :]
        c, sn = torch.cos(ang), torch.sin(ang)
        a, b = k[:, 0:2 * nrot:2].clone(), k[:, 1:2 * nrot:2].clone()
        k[:, 0:2 * nrot:2] = a * c - b * sn
        k[:, 1:2 * nrot:2] = b * c + a * sn
        pool[rows, nc:] = k.to(pool.dtype)
        return cq_out
    _rows2d(proj, "proj")
    _rows2d(cq_out, "cq_out")
    assert proj.shape[1] >= nq + nc + nr and cq_out.shape[1] == nq and cq_out.dtype == proj.dtype
    assert pool.dim() == 2 and pool.is_contiguous() and pool.shape[1] == nc + nr and pool.dtype == proj.dtype
    _vec(qw, nq, "qw")
    _vec(cw, nc, "cw")
    assert inv_freq.dtype == torch.float32 and inv_freq.is_contiguous() and 2 * nrot <= nr
    assert pos.dtype == torch.int32 and cache_rows.dtype == torch.int32
    _chk(lib().p2p_sm_latent_prep(proj.data_ptr(), proj.stride(0), nq, nc, nr, qw.data_ptr(),
                                  cw.data_ptr(), inv_freq.data_ptr(), nrot, pos.data_ptr(),
                                  cache_rows.data_ptr(), pool.data_ptr(), eps, cq_out.data_ptr(),
                                  cq_out.stride(0), R, _f32(proj), _st(proj)), "latent_prep")
    return cq_out


def qtemp_kv_store(proj, nq: int, nkv: int, coef: float, every: int, pos, cache_rows, pool, q_out):
    """Prepares unrotated attention inputs from one projection buffer proj = [q (nq) | k and v
    (nkv)]: q goes to q_out multiplied by the query temperature of its position p,
    1 + coef * ln(floor((p + 1) / every) + 1) (fp32; coef 0: a plain copy), k | v go to the rows
    ``cache_rows`` of the paged pool ([tokens, nkv])."""
    R = q_out.shape[0]
    if every < 1:
        raise ValueError("query temperature step of %d positions" % every)
    if not proj.is_cuda:
        p = pos[:R].long()
        temp = 1.0 + coef * torch.log((torch.div(p + 1, every, rounding_mode="floor") + 1).float())
        q_out[:R] = (proj[:R, :nq].float() * temp[:, None]).to(q_out.dtype)
        pool[cache_rows[:R].long()] = proj[:R, nq:nq + nkv].to(pool.dtype)
        return q_out
    _rows2d(proj, "proj")
    _rows2d(q_out, "q_out")
    assert proj.shape[1] >= nq + nkv and q_out.shape[1] == nq and q_out.dtype == proj.dtype
    assert pool.dim() == 2 and pool.is_contiguous() and pool.shape[1] == nkv and pool.dtype == proj.dtype
    assert pos.dtype == torch.int32 and cache_rows.dtype == torch.int32
    _chk(lib().p2p_sm_qtemp_kv_store(proj.data_ptr(), proj.stride(0), nq, nkv, coef, every,
                                     pos.data_ptr(), cache_rows.data_ptr(), pool.data_ptr(),
                                     q_out.data_ptr(), q_out.stride(0), R, _f32(proj), _st(proj)),
         "qtemp_kv_store")
    return q_out


def qk_norm_rope_store(proj, H: int, G: int, D: int, V: int, qw, kw, inv_freq, pos, cache_rows,
                       pool, eps: float, q_out, per_head: bool = False, half: bool = False):
    """Prepares attention inputs from one projection buffer proj = [q (H*D) | k (G*D) | v (G*V)]:
    q and k are RMS-normalised and weighted -- one mean square per row (heads not separated)
    and weights qw [H*D] / kw [G*D], or with ``per_head`` one mean square per head and weights
    of D channels shared by the heads -- then nrot = len(inv_freq) channel pairs of every head,
    (2i, 2i+1) or with ``half`` (i, i + nrot), are rotated by pos * inv_freq[i].
    q goes to q_out [R, H*D]; k | v go to the paged pool rows ``cache_rows`` ([tokens,
    G*D + G*V]).  pool None: the layer reads another layer's keys and values, proj holds only
    q and only q is prepared.  Norm, angles and the rotation are fp32."""
    R = q_out.shape[0]
    nq, nk, nv = H * D, G * D, G * V
    nrot = inv_freq.numel()
    if not proj.is_cuda:
        ang = (pos[:R].float()[:, None] * inv_freq[None, :])
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        ia = torch.arange(nrot) if half else torch.arange(0, 2 * nrot, 2)
        ib = ia + nrot if half else ia + 1

        def prep(t, heads, w):
            if per_head:
                t = _rms(t.float().view(R, heads, D), eps) * w
            else:
                t = (_rms(t.float(), eps) * w).view(R, heads, D)
            t = t.clone()
            u, v = t[:, :, ia].clone(), t[:, :, ib].clone()
            t[:, :, ia] = u * c - v * s
            t[:, :, ib] = v * c + u * s
            return t.reshape(R, heads * D)

        q_out[:R] = prep(proj[:R, :nq], H, qw).to(q_out.dtype)
        if pool is not None:
            rows = cache_rows[:R].long()
            pool[rows, :nk] = prep(proj[:R, nq:nq + nk], G, kw).to(pool.dtype)
            pool[rows, nk:] = proj[:R, nq + nk:nq + nk + nv].to(pool.dtype)
        return q_out
    _rows2d(proj, "proj")
    _rows2d(q_out, "q_out")
    assert q_out.shape[1] == nq and q_out.dtype == proj.dtype
    _vec(qw, D if per_head else nq, "qw")
    if pool is not None:
        assert proj.shape[1] >= nq + nk + nv
        assert pool.dim() == 2 and pool.is_contiguous() and pool.shape[1] == nk + nv
        assert pool.dtype == proj.dtype and cache_rows.dtype == torch.int32
        _vec(kw, D if per_head else nk, "kw")
    else:
        assert proj.shape[1] >= nq
    assert inv_freq.dtype == torch.float32 and inv_freq.is_contiguous() and 2 * nrot <= D
    assert pos.dtype == torch.int32
    _chk(lib().p2p_sm_qk_norm_rope_store(proj.data_ptr(), proj.stride(0), H, G, D, V,
                                         qw.data_ptr(), _lib.ptr(kw if pool is not None else None),
                                         inv_freq.data_ptr(), nrot, pos.data_ptr(),
                                         cache_rows.data_ptr(), _lib.ptr(pool), eps,
                                         q_out.data_ptr(), q_out.stride(0), R,
                                         1 if per_head else 0, 1 if half else 0, _f32(proj),
                                         _st(proj)), "qk_norm_rope_store")
    return q_out


def window_rows_per_wave(HG: int) -> int:
    """Rows of one sequence portion that a wavefront of the matrix-core window attention takes:
    its 16 (row, head) pairs are RW rows x HS slots for the HG query heads of a key/value head."""
    return latent_rows_per_wave(HG)


def window_mfma_ok(q, pool, D: int, V: int) -> bool:
    """The matrix-core kernel serves bf16 with key / value sizes that are multiples of 8 up to
    256 and 16-byte aligned rows.  P2P_WINDOW_MFMA=0 switches it off."""
    return (q.is_cuda and q.dtype == torch.bfloat16 and D % 8 == 0 and V % 8 == 0
            and 8 <= D <= 256 and 8 <= V <= 256 and q.stride(0) % 8 == 0
            and q.data_ptr() % 16 == 0 and pool.data_ptr() % 16 == 0 and pool.shape[1] % 8 == 0
            and os.environ.get("P2P_WINDOW_MFMA", "1") != "0")


def window_attn(q, pool, block_tables, row_ent, pos, sink, scale: float, win: int, out, page: int,
                H: int, G: int, D: int, V: int, units=None, max_keys=None, out_scale: float = 1.0,
                softcap: float = 0.0, dist=None, gate=None):
    """Grouped-query attention over a paged key/value pool with a causal sliding window and a
    softmax sink.

    q [R, H*D] (rotated), pool [tokens, G*D + G*V] (token t of a sequence at
    block_tables[e, t // page] * page + t % page; keys first, then values), query head h reads
    key/value head h // (H/G).  out [R, H*V] = sum_j p_j v_j with
    p = softmax over {sink_h} U {scale * q . k_j : 0 <= pos - j < win}; the sink has no value
    (sink None: an ordinary softmax over the visible keys);
    the result is multiplied by out_scale before it is rounded.
    softcap c > 0: a score s becomes c * tanh(s / c).  dist = (r1, r2), fp32 [H] each: a key
    d = pos - j positions back loses r1_h * ln(1 + r2_h * d) of its score (after the cap).
    gate: a 2-d view [R, >= H] of the activation type; head h of row r leaves multiplied by
    sigmoid(gate[r, h]).  Scores, cap, penalty, softmax and gate are fp32.
    units: ``make_units(entries, window_rows_per_wave(H // G))`` on the device; with it bf16
    inputs run on the matrix cores (``window_mfma_ok``)."""
    R = q.shape[0]
    HG = H // G
    if not q.is_cuda:
        bt = block_tables.long()
        for r in range(R):
            p = int(pos[r])
            lo = max(0, p - win + 1)
            j = torch.arange(lo, p + 1)
            tok = bt[int(row_ent[r])][j // page] * page + j % page
            kv = pool[tok].float()
            k = kv[:, :G * D].view(-1, G, D).repeat_interleave(HG, 1)       # [n, H, D]
            v = kv[:, G * D:].view(-1, G, V).repeat_interleave(HG, 1)
            s = torch.einsum("hd,nhd->hn", q[r].float().view(H, D), k) * scale
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            if dist is not None:
                s = s - dist[0][:, None] * torch.log1p(dist[1][:, None] * (p - j).float()[None, :])
            m = s.max(-1).values if sink is None else torch.maximum(s.max(-1).values, sink)
            e = torch.exp(s - m[:, None])
            den = e.sum(-1) if sink is None else e.sum(-1) + torch.exp(sink - m)
            o = torch.einsum("hn,nhv->hv", e / den[:, None], v)
            if gate is not None:
                o = o * torch.sigmoid(gate[r, :H].float())[:, None]
            out[r] = (o.reshape(H * V) * out_scale).to(out.dtype)
        return out
    _rows2d(q, "q")
    _rows2d(out, "out")
    assert H % G == 0 and q.shape[1] == H * D and out.shape == (R, H * V)
    assert q.dtype == pool.dtype == out.dtype
    assert pool.dim() == 2 and pool.is_contiguous() and pool.shape[1] == G * (D + V)
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous()
    assert row_ent.dtype == torch.int32 and pos.dtype == torch.int32
    if sink is not None:
        _vec(sink, H, "sink")
    if win < 1:
        raise ValueError("window of %d keys" % win)
    r1 = r2 = None
    if dist is not None:
        r1, r2 = dist
        _vec(r1, H, "r1")
        _vec(r2, H, "r2")
    ldg = 0
    if gate is not None:
        _rows2d(gate, "gate")
        assert gate.shape[0] >= R and gate.shape[1] >= H and gate.dtype == q.dtype
        ldg = gate.stride(0)
    if units is not None and window_mfma_ok(q, pool, D, V):
        assert units.dtype == torch.int32 and units.is_contiguous() and units.shape[1] == 2
        U = units.shape[0]
        hs = 16 // window_rows_per_wave(HG)
        blocks = U * G * (-(-HG // hs))
        splits = 1
        if max_keys is not None and blocks < LATENT_SPLIT_BLOCKS:
            splits = max(1, min(-(-min(max_keys, win) // 64), LATENT_SPLIT_BLOCKS // blocks, 64))
        part = None
        if splits > 1:
            L = lib()
            L.p2p_sm_window_attn_mfma_ws.restype = c_long
            part = torch.empty(L.p2p_sm_window_attn_mfma_ws(U, H, G, V, splits), device=q.device,
                               dtype=torch.float32)
        _chk(lib().p2p_sm_window_attn_mfma(q.data_ptr(), q.stride(0), pool.data_ptr(),
                                           block_tables.data_ptr(), block_tables.shape[1],
                                           row_ent.data_ptr(), pos.data_ptr(), units.data_ptr(), U,
                                           _lib.ptr(sink), scale, win, out.data_ptr(),
                                           out.stride(0), H, G, D, V, page, splits, _lib.ptr(part),
                                           out_scale, softcap, _lib.ptr(r1), _lib.ptr(r2),
                                           _lib.ptr(gate), ldg, _st(q)), "window_attn_mfma")
        return out
    _chk(lib().p2p_sm_window_attn(q.data_ptr(), q.stride(0), pool.data_ptr(),
                                  block_tables.data_ptr(), block_tables.shape[1],
                                  row_ent.data_ptr(), pos.data_ptr(), _lib.ptr(sink), scale, win,
                                  out.data_ptr(), out.stride(0), R, H, G, D, V, page, out_scale,
                                  softcap, _lib.ptr(r1), _lib.ptr(r2), _lib.ptr(gate), ldg,
                                  _f32(q), _st(q)), "window_attn")
    return out


# ------------------------------------------------------------------ gated linear scans
# Per head a D x V fp32 state S (key channel i, value channel j), one step per token:
#   S <- diag(g) S;   u = v                      (plain write)
#                     u = beta * (v - S^T k)     (delta rule: the write corrects what k reads)
#   S <- S + k u^T;   o = S^T q                  (o is formed from the updated S)
# HGRN2 is the plain write with g = f and k = 1 - f; the gated delta rule has its own key.
def hgrn2_scan(proj, lower, fb, normw, state, ent, ent_host, out, H: int, D: int, V: int,
               eps: float, out_scale: float = 1.0):
    """proj = [q (H*D) | f (H*D) | v (H*V)] raw projections of the step's rows.  q = silu(q),
    f = lower + (1 - lower) * sigmoid(f + fb); S <- diag(f) S + (1 - f) v^T; o = S^T q; every
    head's o is RMS-normalised over V and weighted by normw [V].  state fp32 [slots, H, D, V];
    out [R, H*V] activation type."""
    n = H * D
    if not proj.is_cuda:
        for row0, cnt, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            for t in range(row0, row0 + cnt):
                qr = proj[t, :n].float()
                q = (qr * torch.sigmoid(qr)).view(H, D)
                f = (lower + (1 - lower) * torch.sigmoid(proj[t, n:2 * n].float() + fb)).view(H, D)
                v = proj[t, 2 * n:2 * n + H * V].float().view(H, V)
                S = f[:, :, None] * S + (1 - f)[:, :, None] * v[:, None, :]
                o = torch.einsum("hdv,hd->hv", S, q)
                out[t] = (_rms(o, eps) * normw * out_scale).reshape(H * V).to(out.dtype)
            state[slot] = S
        return out
    _rows2d(proj, "proj")
    _rows2d(out, "out")
    assert proj.shape[1] >= 2 * n + H * V and out.shape[1] == H * V and out.dtype == proj.dtype
    _vec(lower, n, "lower")
    _vec(fb, n, "fb")
    _vec(normw, V, "normw")
    _scan_state_ok(state, H, D, V, ent)
    if _chunked(ent_host):
        vent, cent = (t_.to(proj.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        NV = vent.shape[0]
        cs = torch.empty(NV, H, D, V, device=proj.device, dtype=torch.float32)
        cd = torch.empty(NV, H, D, device=proj.device, dtype=torch.float32)
        _chk(lib().p2p_sm_hgrn2_scan_chunked(
            proj.data_ptr(), proj.stride(0), lower.data_ptr(), fb.data_ptr(), normw.data_ptr(),
            state.data_ptr(), cs.data_ptr(), cd.data_ptr(), vent.data_ptr(), NV, cent.data_ptr(),
            ent.shape[0], out.data_ptr(), out.stride(0), H, D, V, eps, out_scale, _f32(proj),
            _st(proj)), "hgrn2_scan_chunked")
        return out
    _chk(lib().p2p_sm_hgrn2_scan(proj.data_ptr(), proj.stride(0), lower.data_ptr(), fb.data_ptr(),
                                 normw.data_ptr(), state.data_ptr(), ent.data_ptr(), ent.shape[0],
                                 out.data_ptr(), out.stride(0), H, D, V, eps, out_scale,
                                 _f32(proj), _st(proj)), "hgrn2_scan")
    return out


def _scan_state_ok(state, H, D, V, ent):
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, V)
    assert ent.dtype == torch.int32 and ent.is_contiguous() and ent.shape[1] == 4
    if D > 256 or V > 256:
        raise ValueError("gated scan: key %d / value %d sizes above 256" % (D, V))


def gated_delta_scan(conv, araw, braw, gate, A_log, dt_bias, normw, state, ent, ent_host, out,
                     H: int, G: int, D: int, V: int, eps: float, out_scale: float = 1.0):
    """Gated delta rule.  conv fp32 [R, 2*G*D + H*V] = silu(conv(q | k | v)); q and k become
    unit vectors per head (x / sqrt(|x|^2 + 1e-6)), q also times D^-1/2; head h reads q/k head
    h // (H/G).  araw [R, H*D]: decay logits, g = exp(-exp(A_log_h) * softplus(araw + dt_bias));
    braw [R, H]: beta = sigmoid(braw); gate [R, H*V]: the output gate's logits.  Every head's
    o is RMS-normalised over V, weighted by normw [V] and multiplied by sigmoid(gate).
    state fp32 [slots, H, D, V]; out [R, H*V] activation type."""
    R = out.shape[0]
    hg = H // G
    if not conv.is_cuda:
        nA = torch.exp(A_log)
        for row0, cnt, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            for t in range(row0, row0 + cnt):
                q = conv[t, :G * D].view(G, D)
                k = conv[t, G * D:2 * G * D].view(G, D)
                v = conv[t, 2 * G * D:].view(H, V)
                q = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5).repeat_interleave(hg, 0)
                k = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(hg, 0)
                dt = torch.nn.functional.softplus(araw[t].float() + dt_bias, threshold=1e9).view(H, D)
                g = torch.exp(-nA[:, None] * dt)
                beta = torch.sigmoid(braw[t].float())
                S = g[:, :, None] * S
                u = beta[:, None] * (v - torch.einsum("hdv,hd->hv", S, k))
                S = S + k[:, :, None] * u[:, None, :]
                o = torch.einsum("hdv,hd->hv", S, q)
                o = _rms(o, eps) * normw * torch.sigmoid(gate[t].float()).view(H, V)
                out[t] = (o.reshape(H * V) * out_scale).to(out.dtype)
            state[slot] = S
        return out
    assert conv.dtype == torch.float32 and conv.is_contiguous() and conv.shape[1] == 2 * G * D + H * V
    for t_, nm, n in ((araw, "araw", H * D), (braw, "braw", H), (gate, "gate", H * V), (out, "out", H * V)):
        _rows2d(t_, nm)
        assert t_.shape[1] == n and t_.dtype == out.dtype, nm
    _vec(A_log, H, "A_log")
    _vec(dt_bias, H * D, "dt_bias")
    _vec(normw, V, "normw")
    assert H % G == 0
    _scan_state_ok(state, H, D, V, ent)
    if _chunked(ent_host):
        vent, cent = (t_.to(conv.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        NV = vent.shape[0]
        cs = torch.empty(NV, H, D, V, device=conv.device, dtype=torch.float32)
        ct = torch.empty(NV, H, D, D, device=conv.device, dtype=torch.float32)
        _chk(lib().p2p_sm_gated_delta_scan_chunked(
            conv.data_ptr(), conv.stride(0), araw.data_ptr(), araw.stride(0), braw.data_ptr(),
            braw.stride(0), gate.data_ptr(), gate.stride(0), A_log.data_ptr(), dt_bias.data_ptr(),
            normw.data_ptr(), state.data_ptr(), cs.data_ptr(), ct.data_ptr(), vent.data_ptr(), NV,
            cent.data_ptr(), ent.shape[0], out.data_ptr(), out.stride(0), H, G, D, V, eps,
            out_scale, _f32(out), _st(out)), "gated_delta_scan_chunked")
        return out
    _chk(lib().p2p_sm_gated_delta_scan(conv.data_ptr(), conv.stride(0), araw.data_ptr(),
                                       araw.stride(0), braw.data_ptr(), braw.stride(0),
                                       gate.data_ptr(), gate.stride(0), A_log.data_ptr(),
                                       dt_bias.data_ptr(), normw.data_ptr(), state.data_ptr(),
                                       ent.data_ptr(), ent.shape[0], out.data_ptr(), out.stride(0),
                                       H, G, D, V, eps, out_scale, _f32(out), _st(out)),
         "gated_delta_scan")
    return out


def mlstm_scan(proj, bi, bf, cap: float, normw, state, mstate, ent, ent_host, out, H: int, D: int,
               V: int, eps: float, out_scale: float = 1.0):
    """Matrix memory of the mLSTM.  proj = [q (H*D) | k (H*D) | v (H*V) | gate (H*V) | zi (H) |
    zf (H)] raw projections of the step's rows.  Per head, with the capped log gates
    i = cap tanh((zi + bi) / cap), f = logsigmoid(cap tanh((zf + bf) / cap)) and the running
    maximum m <- max(f + m, i) (m = 0 before position 0):
        S <- exp(f + m' - m) S + exp(i - m) k v^T,   n likewise with k alone,
        o = S^T (q D^-1/2) / (max(|n . q D^-1/2|, exp(-m)) + 1e-6);
    every head's o is RMS-normalised over V, weighted by normw [H*V] and multiplied by
    sigmoid(gate).  state fp32 [slots, H, D, V + 1] (column V holds n), mstate fp32 [slots, H];
    out [R, H*V] activation type.  Gates, maximum, exponentials and state are fp32."""
    nq, nv = H * D, H * V
    if not proj.is_cuda:
        for row0, cnt, start, slot in ent_host:
            S = state[slot] if start > 0 else torch.zeros_like(state[slot])
            m = mstate[slot] if start > 0 else torch.zeros_like(mstate[slot])
            for t in range(row0, row0 + cnt):
                row = proj[t].float()
                q = row[:nq].view(H, D) * D ** -0.5
                k = row[nq:2 * nq].view(H, D)
                v1 = torch.cat([row[2 * nq:2 * nq + nv].view(H, V), torch.ones(H, 1)], 1)
                zi, zf = row[2 * nq + 2 * nv:2 * nq + 2 * nv + H], row[2 * nq + 2 * nv + H:2 * nq + 2 * nv + 2 * H]
                i = cap * torch.tanh((zi + bi) / cap)
                f = torch.nn.functional.logsigmoid(cap * torch.tanh((zf + bf) / cap))
                mn = torch.maximum(f + m, i)
                a, b = torch.exp(f + m - mn), torch.exp(i - mn)
                S = a[:, None, None] * S + (b[:, None] * k)[:, :, None] * v1[:, None, :]
                m = mn
                o = torch.einsum("hdv,hd->hv", S, q)
                den = torch.maximum(o[:, V].abs(), torch.exp(-m)) + 1e-6
                o = _rms(o[:, :V] / den[:, None], eps).reshape(nv) * normw
                o = o * torch.sigmoid(row[2 * nq + nv:2 * nq + 2 * nv]) * out_scale
                out[t] = o.to(out.dtype)
            state[slot] = S
            mstate[slot] = m
        return out
    _rows2d(proj, "proj")
    _rows2d(out, "out")
    assert proj.shape[1] >= 2 * nq + 2 * nv + 2 * H and out.shape[1] == nv and out.dtype == proj.dtype
    _vec(bi, H, "bi")
    _vec(bf, H, "bf")
    _vec(normw, nv, "normw")
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, V + 1)
    assert mstate.dtype == torch.float32 and mstate.is_contiguous() and mstate.shape[1:] == (H,)
    assert mstate.shape[0] == state.shape[0]
    assert ent.dtype == torch.int32 and ent.is_contiguous() and ent.shape[1] == 4
    if D > 256 or V > 256:
        raise ValueError("mlstm_scan: key %d / value %d sizes above 256" % (D, V))
    R = out.shape[0]
    coef = torch.empty(R, H, 3, device=proj.device, dtype=torch.float32)
    vent = cent = cs = cd = None
    NV = 0
    if _chunked(ent_host):
        vent, cent = (t_.to(proj.device) for t_ in scan_chunks(ent_host, SCAN_CHUNK))
        NV = vent.shape[0]
        cs = torch.empty(NV, H, D, V + 1, device=proj.device, dtype=torch.float32)
        cd = torch.empty(NV, H, D, device=proj.device, dtype=torch.float32)
    _chk(lib().p2p_sm_mlstm_scan(proj.data_ptr(), proj.stride(0), bi.data_ptr(), bf.data_ptr(), cap,
                                 normw.data_ptr(), state.data_ptr(), mstate.data_ptr(),
                                 coef.data_ptr(), ent.data_ptr(), ent.shape[0], _lib.ptr(cs),
                                 _lib.ptr(cd), _lib.ptr(vent), NV, _lib.ptr(cent), out.data_ptr(),
                                 out.stride(0), H, D, V, eps, out_scale,
                                 max(e[1] for e in ent_host), _f32(proj), _st(proj)),
         "mlstm_scan")
    return out


# ------------------------------------------------------------------ mixture of experts
ROUTE_SCORES = {"sigmoid": 0, "softmax": 1, "top_softmax": 2}


def group_route(h, wr, top: int, groups: int, keep: int, ids, wts, cnt, rows,
                score: str = "sigmoid", corr=None, group_score: str = "top2", bias=None,
                cleared: bool = False):
    """Router with group-limited choice.  z = h wr^T (+ bias, fp32 [E]) in fp32 (wr fp32
    [E, W]); the scores are s = sigmoid(z) or (``score`` "softmax") softmax(z) over all E, or
    (``score`` "top_softmax") s = z for the choice and the weights are the softmax over the
    chosen z only; the choice is made on
    c = s + corr (corr fp32 [E], optional).  The E experts are cut into ``groups`` contiguous
    blocks of equal size, a block is ranked by the sum of its two best c (``group_score``
    "top2") or by its best c ("max"), experts outside the ``keep`` best blocks are struck out;
    the ``top`` largest c among the rest win (ties: the lower index), their weights are their s.
    ids int32 / wts fp32 [R, top]; cnt int32 [E] and rows int32 [E, R*top] list per expert the
    slots (row * top + k) routed to it (cnt is cleared here, unless the caller says it has
    ``cleared`` it: a model clears the counts of all its layers with one fill per step)."""
    R = h.shape[0]
    E = wr.shape[0]
    per = E // groups
    if score not in ROUTE_SCORES or group_score not in ("top2", "max"):
        raise ValueError("group_route: score %r / group score %r" % (score, group_score))
    if not h.is_cuda:
        z = h[:R].float() @ wr.t()                                                # [R, E]
        if bias is not None:
            z = z + bias
        s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1) if score == "softmax" else z
        c = s if corr is None else s + corr
        gs = c.view(R, groups, per).topk(min(2, per) if group_score == "top2" else 1, dim=-1).values.sum(-1)
        best = gs.topk(keep, dim=-1).indices
        ok = torch.zeros(R, groups, dtype=torch.bool).scatter_(1, best, True)
        masked = torch.where(ok.repeat_interleave(per, 1), c, torch.full_like(c, -float("inf")))
        i = masked.topk(top, dim=-1).indices
        ids[:R] = i.to(torch.int32)
        wts[:R] = s.gather(1, i) if score != "top_softmax" else torch.softmax(s.gather(1, i), -1)
        cnt.zero_()   # (the rendering fills the lists from scratch either way)
        for slot, e in enumerate(i.reshape(-1).tolist()):
            rows[e, int(cnt[e])] = slot
            cnt[e] += 1
        return ids, wts
    _rows2d(h, "h")
    assert wr.dtype == torch.float32 and wr.is_contiguous() and wr.shape[1] == h.shape[1]
    assert E % groups == 0 and 1 <= keep <= groups and 1 <= top <= keep * per
    if E > 1024:
        raise ValueError("group_route: %d experts > 1024" % E)
    if corr is not None:
        _vec(corr, E, "corr")
    if bias is not None:
        _vec(bias, E, "bias")
    assert ids.dtype == torch.int32 and ids.is_contiguous() and ids.shape == (R, top)
    assert wts.dtype == torch.float32 and wts.is_contiguous() and wts.shape == (R, top)
    assert cnt.dtype == torch.int32 and cnt.numel() == E
    assert rows.dtype == torch.int32 and rows.is_contiguous() and rows.shape[0] == E \
        and rows.shape[1] >= R * top
    if not cleared:
        cnt.zero_()
    _chk(lib().p2p_sm_group_route(h.data_ptr(), h.stride(0), wr.data_ptr(), R, h.shape[1], E, top,
                                  groups, keep, ROUTE_SCORES[score], _lib.ptr(corr),
                                  1 if group_score == "max" else 0, ids.data_ptr(),
                                  wts.data_ptr(), cnt.data_ptr(), rows.data_ptr(), rows.stride(0),
                                  _lib.ptr(bias), _f32(h), _st(h)), "group_route")
    return ids, wts


def interleave_gate_up(gate, up):
    """[..., F, K] gate and up rows -> [..., 2F, K] as 16 gate rows, their 16 up rows, the next
    16 gate rows, ... (F a multiple of 16): the layout ``expert_gemm`` wants for its fused
    activation."""
    F, K = gate.shape[-2:]
    lead = gate.shape[:-2]
    g = gate.reshape(*lead, F // 16, 1, 16, K)
    u = up.reshape(*lead, F // 16, 1, 16, K)
    return torch.cat([g, u], dim=-3).reshape(*lead, 2 * F, K)


def expert_gemm(x, x_div: int, w, cnt, rows, out, total_slots: int, act_limit=None,
                act_alpha: float = 1.702, relu2: bool = False, silu_glu: bool = False):
    """Per expert e and each of its routed slots s = rows[e, i] (i < cnt[e]):
    out[s] = x[s // x_div] @ w[e]^T.  w [E, N, K] (activation type), x [*, K], out [slots, N].
    total_slots: the slots over all experts (every slot is in exactly one list; the grid is
    sized from it, so no launch depends on the counts).  Accumulation is fp32; a slot's
    result does not depend on the other slots.
    act_limit: w = ``interleave_gate_up(gate, up)`` and out [slots, N/2] receives
    min(g, L) * sigmoid(alpha * min(g, L)) * (clamp(u, -L, L) + 1) of the two products (fp32
    before the rounding) instead of the products themselves.
    silu_glu: w = ``interleave_gate_up(gate, up)`` and out [slots, N/2] receives g * sigmoid(g) * u.
    relu2: out receives relu(.)^2 of every product (an ungated unit; fp32 before the rounding).
    cnt may list more experts than w holds (experts without weights): their slots are left
    out."""
    E, N, K = w.shape
    fused = act_limit is not None or silu_glu
    if (act_limit is not None) + bool(relu2) + bool(silu_glu) > 1:
        raise ValueError("expert_gemm: one activation at a time")
    if not x.is_cuda:
        for e in range(E):
            sl = rows[e, :int(cnt[e])].long()
            if not sl.numel():
                continue
            y = torch.nn.functional.linear(x[sl // x_div].float(), w[e].float())
            if silu_glu:
                y = y.view(-1, N // 32, 2, 16)
                y = (y[:, :, 0] * torch.sigmoid(y[:, :, 0]) * y[:, :, 1]).reshape(-1, N // 2)
            elif fused:
                y = y.view(-1, N // 32, 2, 16)
                g = torch.clamp(y[:, :, 0], max=act_limit)
                u = torch.clamp(y[:, :, 1], -act_limit, act_limit)
                y = (g * torch.sigmoid(act_alpha * g) * (u + 1)).reshape(-1, N // 2)
            elif relu2:
                y = torch.relu(y) ** 2
            out[sl] = y.to(out.dtype)
        return out
    _rows2d(x, "x")
    _rows2d(out, "out")
    assert w.is_contiguous() and x.shape[1] == K and out.shape[1] == (N // 2 if fused else N)
    assert x.dtype == w.dtype == out.dtype and cnt.numel() >= E
    if fused and N % 32:
        raise ValueError("fused expert activation needs gate / up widths that are multiples of 16")
    _chk(lib().p2p_sm_expert_gemm(x.data_ptr(), x.stride(0), x_div, w.data_ptr(), cnt.data_ptr(),
                                  rows.data_ptr(), rows.stride(0), out.data_ptr(), out.stride(0),
                                  E, N, K, total_slots,
                                  3 if silu_glu else 1 if fused else 2 if relu2 else 0,
                                  float(act_limit) if act_limit is not None else 0.0, act_alpha,
                                  _f32(x), _st(x)),
         "expert_gemm")
    return out


def expert_combine(y, wts, out, ids=None, n_real: int = 0, x=None):
    """out[r] = sum_k wts[r, k] * y[r * top + k] (fp32 sum, activation-typed result).  With
    ids (int32 [R, top]) a slot whose expert index is >= n_real stands for an expert that hands
    its input back: its term is wts[r, k] * x[r]."""
    R, top = wts.shape
    if not y.is_cuda:
        t = y[:R * top].float().view(R, top, -1)
        if ids is not None:
            t = torch.where((ids[:R] >= n_real)[:, :, None], x[:R].float()[:, None, :], t)
        out[:R] = (t * wts[:, :, None]).sum(1).to(out.dtype)
        return out
    _rows2d(y, "y")
    _rows2d(out, "out")
    assert y.shape[0] >= R * top and out.shape[1] == y.shape[1] and y.dtype == out.dtype
    ldx = 0
    if ids is not None:
        _rows2d(x, "x")
        assert ids.dtype == torch.int32 and ids.is_contiguous() and ids.shape == (R, top)
        assert x.shape[1] == y.shape[1] and x.shape[0] >= R and x.dtype == y.dtype
        ldx = x.stride(0)
    _chk(lib().p2p_sm_expert_combine(y.data_ptr(), y.stride(0), wts.data_ptr(), out.data_ptr(),
                                     out.stride(0), R, top, y.shape[1], _lib.ptr(ids), n_real,
                                     _lib.ptr(x if ids is not None else None), ldx, _f32(y),
                                     _st(y)), "expert_combine")
    return out
