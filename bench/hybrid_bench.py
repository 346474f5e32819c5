"""Prefill and decode throughput of hybrid models (Regesun, Rotutar, Futetar, Tarunex) at layer sizes that
resemble real models, beside a dense Llama of the same width, depth and parameter count on
the same engine entry point (``generate``).  Random weights, random tokens.

    python bench.py --hybrid [--hybrid-design regesun|rotutar|futetar|tarunex|both] [--hybrid-sizes 1024,2048]
                    [--steps K] [--warmup W]

``--hybrid-design rotutar`` runs Rotutar beside Regesun (the closest model: same engine, same
width and depth) instead of the Llama; ``futetar`` runs Futetar beside Rotutar (gated scans,
grouped-query attention and routed experts in both); ``tarunex`` runs Tarunex beside Futetar
(parallel layers, grouped-query attention and routed experts with a shared expert in both; 16
layer runs each).

One JSON line per (size, model): prefill tokens/s of one long prompt (``prompt`` tokens),
decode tokens/s of ``batch`` sequences.  These lines are not the headline metric.
"""
from __future__ import annotations

import json
import time

import torch


def regesun_config(width: int):
    """A Regesun stack at a given width: blocks of delta / mamba / mamba / attention+ff."""
    from p2p_llm_chat_go_amd.models.hybrid import HybridConfig

    hd = 64
    gd = {"type": "general_delta", "mixer": {"heads": width // hd, "dim": hd}, "mlp": None}
    mb = {"type": "mamba2", "mixer": {"heads": 2 * width // hd, "vdim": hd, "state": 128,
                                      "groups": 8, "conv": 4, "norm_groups": 8}, "mlp": None}
    la = {"type": "latent_attention",
          "mixer": {"heads": width // 128, "dim": 128, "vdim": 128, "kv_rank": width // 4,
                    "mask": {"size": 1024}, "scale": 128 ** -0.5},
          "mlp": {"kind": "dense", "ff": 4 * width, "limit": 7.0}}
    return HybridConfig.from_dict(
        {"architecture": "Regesun", "width": width, "vocab": 32000, "max_positions": 8192,
         "norm": {"eps": 1e-5}, "layers": [gd, mb, mb, la] * 4}, name="regesun-w%d" % width)


def rotutar_config(width: int):
    """A Rotutar stack at a given width: blocks of hgrn2 / hgrn2+moe / hgrn2 / (window attention
    beside the gated delta rule)+dense ff, 128-wide heads."""
    from p2p_llm_chat_go_amd.models.hybrid import HybridConfig

    hd = 128
    nh = width // hd
    moe = {"kind": "moe", "expert": {"ff": width // 2, "limit": 7.0},
           "router": {"experts": 8, "top": 2, "groups": {"count": 4, "keep": 2}}}
    hg = {"type": "hgrn2", "mixer": {"heads": nh, "dim": hd, "vdim": hd}, "mlp": None}
    pa = {"type": "parallel",
          "mixer": {"left": {"heads": nh, "kv_heads": max(1, nh // 4), "dim": hd, "vdim": hd,
                             "mask": {"size": 1024}, "rot": {"base": 10000.0, "dims": 64},
                             "scale": hd ** -0.5},
                    "right": {"heads": nh, "kv_heads": max(1, nh // 2), "dim": hd, "vdim": hd,
                              "conv": 4},
                    "left_scale": 1.0, "right_scale": 1.0},
          "mlp": {"kind": "dense", "ff": 4 * width}}
    return HybridConfig.from_dict(
        {"architecture": "Rotutar", "width": width, "vocab": 32000,
         "norm": {"eps": 1e-5, "groups": 4}, "logit_softcap": 50.0,
         "layers": [hg, dict(hg, mlp=moe), hg, pa] * 4}, name="rotutar-w%d" % width)


def futetar_config(width: int):
    """A Futetar stack at a given width: blocks of mlstm+dense ff / attention+moe / mlstm+moe /
    attention on the block's first attention layer's keys and values + dense ff, 128-wide heads."""
    from p2p_llm_chat_go_amd.models.hybrid import HybridConfig

    hd = 128
    nh = width // hd
    moe = {"kind": "moe", "expert": {"ff": width // 2}, "shared": {"ff": width // 2},
           "router": {"experts": 8, "identity": 4, "top": 2, "groups": {"count": 4, "keep": 2}}}
    dense = {"kind": "dense", "ff": 4 * width}
    ml = {"heads": nh, "dim": hd, "vdim": hd, "gate_cap": 12.0}
    at = {"heads": nh, "kv_heads": max(1, nh // 4), "dim": hd, "vdim": hd, "scale": hd ** -0.5,
          "rot": {"base": 500000.0, "dims": hd,
                  "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    layers = []
    for b in range(4):
        layers += [{"type": "mlstm", "mixer": ml, "mlp": dense}, {"type": "attention", "mixer": at, "mlp": moe},
                   {"type": "mlstm", "mixer": ml, "mlp": moe},
                   {"type": "attention", "mixer": dict(at, kv_from=4 * b + 1), "mlp": dense}]
    return HybridConfig.from_dict(
        {"architecture": "Futetar", "width": width, "vocab": 32000, "norm": {"eps": 1e-6},
         "layers": layers}, name="futetar-w%d" % width)


def tarunex_config(width: int):
    """A Tarunex stack at a given width: 10 layers of which the middle 6 run two passes (16 layer
    runs), biased attention three times for every latent attention, every layer with routed
    experts and a shared expert, 128-wide heads."""
    from p2p_llm_chat_go_amd.models.hybrid import HybridConfig

    hd = 128
    nh = width // hd
    moe = {"kind": "moe", "expert": {"ff": width // 2}, "shared": {"ff": width // 2},
           "router": {"experts": 8, "top": 2}}
    ba = {"type": "attention",
          "mixer": {"heads": nh, "kv_heads": max(1, nh // 4), "dim": hd, "vdim": hd, "scale": hd ** -0.5,
                    "softcap": 50.0, "q_temp": {"coef": 0.1, "every": 512}}, "mlp": moe}
    la = {"type": "latent_attention",
          "mixer": {"heads": nh, "dim": hd, "rot_dim": 64, "vdim": hd, "kv_rank": 448, "q_rank": width // 2,
                    "rot": {"base": 10000.0, "dims": 64}, "scale": (hd + 64) ** -0.5}, "mlp": moe}
    layers = [ba, ba, ba, la, ba, ba, la, ba, ba, la]
    return HybridConfig.from_dict(
        {"architecture": "Tarunex", "width": width, "vocab": 32000, "norm": {"eps": 1e-5},
         "embedding": {"scale": width ** 0.5}, "logit_scale": 0.5, "logit_softcap": 50.0,
         "loop": {"start": 2, "stop": 8, "times": 2}, "layers": layers}, name="tarunex-w%d" % width)


def n_params(cfg) -> int:
    from p2p_llm_chat_go_amd.models.hybrid import tensor_shapes

    n = 0
    for s in tensor_shapes(cfg.resolve({})).values():
        k = 1
        for d in s:
            k *= d
        n += k
    return n


def llama_like(width: int, layers: int, params: int):
    """Dense Llama of the same width and depth whose ffn size makes the parameter count match."""
    from p2p_llm_chat_go_amd.models.config import ModelConfig

    nh = width // 128
    nkv = max(1, nh // 4)
    vocab = 32000
    attn = width * (nh + 2 * nkv) * 128 + nh * 128 * width
    per_layer = (params - 2 * vocab * width) / layers - attn
    ffn = max(256, int(per_layer / (3 * width)) // 256 * 256)
    return ModelConfig("llama-w%d" % width, hidden=width, n_layers=layers, n_heads=nh,
                       n_kv_heads=nkv, ffn=ffn, vocab=vocab, max_pos=8192, rope_theta=10000.0,
                       rope_llama3=None, bos_id=1, eos_ids=(2,))


def measure(eng, vocab, prompt, batch, ctx, new_tokens, steps, warmup, dev, phase="both"):
    g = torch.Generator().manual_seed(0)
    long_p = [torch.randint(3, vocab, (prompt,), generator=g).tolist()]
    many = [torch.randint(3, vocab, (ctx,), generator=g).tolist() for _ in range(batch)]
    out = {}
    for name, prompts, new in (("prefill", long_p, 2), ("decode", many, new_tokens)):
        if phase not in ("both", name):
            continue
        for _ in range(warmup):
            eng.generate(prompts, new, stop_on_eos=False)
        torch.cuda.synchronize(dev)
        pre = dec = 0.0
        for _ in range(steps):
            r = eng.generate(prompts, new, stop_on_eos=False)[0]
            pre += r.ttft_ns * 1e-9
            dec += r.eval_duration_ns * 1e-9
        torch.cuda.synchronize(dev)
        if name == "prefill":
            out["prefill_tok_s"] = round(steps * prompt / pre, 1)
            out["prefill_ms"] = round(1e3 * pre / steps, 3)
        else:
            out["decode_tok_s"] = round(steps * batch * (new - 1) / dec, 1)
            out["decode_ms_per_step"] = round(1e3 * dec / (steps * (new - 1)), 3)
    return out


def run(a):
    from p2p_llm_chat_go_amd.engine import Engine
    from p2p_llm_chat_go_amd.models import registry

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    prompt, batch, ctx, new = a.hybrid_prompt, a.hybrid_batch, a.hybrid_ctx, a.new_tokens
    pages = max(prompt // 64 + 4, batch * ((ctx + new) // 64 + 2)) + 8
    design = getattr(a, "hybrid_design", "regesun")
    for width in [int(w) for w in a.hybrid_sizes.split(",")]:
        hcfg = regesun_config(width)
        params = n_params(hcfg)
        lcfg = llama_like(width, hcfg.n_layers, params)
        todo = {"regesun": lambda: (hcfg, lcfg), "rotutar": lambda: (rotutar_config(width), hcfg),
                "futetar": lambda: (futetar_config(width), rotutar_config(width)),
                "tarunex": lambda: (tarunex_config(width), futetar_config(width)),
                "both": lambda: (rotutar_config(width), hcfg, lcfg)}[design]()
        for cfg in todo:
            if getattr(a, "hybrid_only", None) and a.hybrid_only not in cfg.name:
                continue
            hybrid = cfg is not lcfg
            if hybrid:
                params = n_params(cfg)
                eng = registry.make_engine(cfg, None, dev, kv_pages=pages, max_batch=batch,
                                           max_prefill_tokens=prompt, seed=1)
            else:
                eng = Engine(cfg, device=dev, seed=1, kv_pages=pages, max_prefill_tokens=prompt,
                             max_batch=batch)
                eng.warmup((batch,), ctx=ctx + new)
            t0 = time.perf_counter()
            m = measure(eng, cfg.vocab, prompt, batch, ctx, new, a.steps, a.warmup, dev,
                        getattr(a, "hybrid_phase", "both"))
            line = {"metric": "hybrid-vs-dense throughput", "model": cfg.name,
                    "params_m": round((params if hybrid else cfg.n_params()) / 1e6, 1),
                    "width": width, "layers": cfg.n_layers,
                    "layer_runs": len(cfg.runs()) if hybrid else cfg.n_layers, "dtype": "bf16",
                    "prompt_tokens": prompt, "decode_batch": batch, "decode_ctx": ctx,
                    "new_tokens": new, "steps": a.steps, "warmup": a.warmup,
                    "data": "random tokens; random-init weights",
                    "bench_s": round(time.perf_counter() - t0, 1)}
            line.update(m)
            print(json.dumps(line), flush=True)
            del eng
            torch.cuda.empty_cache()
