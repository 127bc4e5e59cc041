"""Merusun on the ragged engine: reader of its ``config.json`` and the map from checkpoint tensor names to
``LayerTensors``.

The design: a sandwich-norm decoder (x <- x + norm_b(f(norm_a(x))) around every mixer and feed-forward, plain RMS norms,
scaled embedding) whose token mixers are

* sliding-window attention with biased projections, unit-norm queries and keys, no rotation and a softmax whose
  normaliser carries one extra term (a sink of score 0); a layer may read another layer's keys and values,
* latent attention: one compressed row and one rotated key part per token are cached, queries and keys have an
  unrotated and a rotated (neighbouring pairs) part, sliding window, ordinary softmax,
* mLSTM: a matrix memory per head with soft-capped exponential gates and a running maximum,

and whose feed-forwards are mixtures of small relu-squared experts with a softmax router that picks the best experts
inside the best groups, plus an expert that every token uses.
"""
from __future__ import annotations

import json
import math
import os

import torch

from .ragged_engine import (LatentAttention, LayerTensors, Mlstm, RaggedConfig, RaggedDecoder, RoutedExperts,
                            WindowAttention, rotary_inv_freq)

ARCHITECTURE = "Merusun"
SINK_SCORE = 0.0           # fixed by the design: the normaliser of the windowed attention is 1 + sum exp(s)
MLSTM_M_START = 0.0        # the running maximum of a fresh sequence
MLSTM_DEN_FLOOR = 1e-6


def is_merusun(config: dict) -> bool:
    return config.get("architecture") == ARCHITECTURE


def read_config(config: dict) -> RaggedConfig:
    mixers, mlps = [], []
    for layer in config["layers"]:
        m, kind = layer["mixer"], layer["type"]
        mask = m.get("mask") or {}
        if kind == "attention":
            mixers.append(WindowAttention(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]), qk_norm=True, window=int(mask.get("size") or 0), kv_from=m.get("kv_from"),
                bias=True, sink=SINK_SCORE))
        elif kind == "latent_attention":
            rot = m.get("rot") or {}
            mixers.append(LatentAttention(
                heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                rank=int(m["kv_rank"]), scale=float(m["scale"]), rot_dims=int(rot.get("dims") or 0),
                rot_base=float(rot.get("base", 10000.0)), window=int(mask.get("size") or 0)))
        elif kind == "mlstm":
            mixers.append(Mlstm(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), gate_cap=float(m["gate_cap"]),
                                m_start=MLSTM_M_START, den_floor=MLSTM_DEN_FLOOR))
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        f = layer.get("mlp")
        if f is None:
            mlps.append(None)
        elif f.get("kind") == "moe":
            r = f["router"]
            g = r.get("groups") or {}
            mlps.append(RoutedExperts(experts=int(r["experts"]), top=int(r["top"]), ff=int(f["expert"]["ff"]),
                                      groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))),
                                      scale=float(r.get("scale", 1.0)), shared_ff=int((f.get("shared") or {}).get("ff", 0))))
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    return RaggedConfig(vocab=int(config["vocab"]), width=int(config["width"]), mixers=mixers, mlps=mlps,
                        norm_eps=float((config.get("norm") or {}).get("eps", 1e-6)), name=ARCHITECTURE,
                        embed_scale=float((config.get("embedding") or {}).get("scale", 1.0)), block="sandwich")


def build_engine(cfg: RaggedConfig, sd: dict, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """``sd``: checkpoint tensors by name ('l<i>.mix.q', 'l<i>.mlp.e<j>.up', ...).  Projection and expert weights take
    the activation type; norm weights, router rows and gate biases become float32 (what reads them computes in 32 bits)."""
    dev = torch.device(device)

    def act(*names):
        return torch.cat([sd[n] for n in names], 0).to(dev, dtype).contiguous()

    def f32(*names):
        return torch.cat([sd[n].float().reshape(-1) for n in names], 0).to(dev).contiguous()

    layers = []
    for li, (m, mlp) in enumerate(zip(cfg.mixers, cfg.mlps)):
        p = f"l{li}.mix."
        if isinstance(m, WindowAttention):
            proj = ["q", "k", "v"] if m.kv_from is None else ["q"]
            lt = LayerTensors(w_in=act(*[p + n for n in proj]), w_out=act(p + "o"), norm1=f32(f"l{li}.norm1"))
            lt.b_in = act(*[p + n + ".b" for n in proj])
            # unit norm over a head's channels: the kernel's weighted norm with a weight of ones
            lt.q_norm = lt.k_norm = torch.ones(m.dim, dtype=torch.float32, device=dev)
        elif isinstance(m, LatentAttention):
            lt = LayerTensors(w_in=act(p + "q", p + "dkv"), w_out=act(p + "o"), norm1=f32(f"l{li}.norm1"))
            lt.k_norm = f32(p + "dkv.norm")
            lt.w_uk = sd[p + "uk"].to(dev, dtype).view(m.heads, m.dim, m.rank).contiguous()
            lt.w_uv = sd[p + "uv"].to(dev, dtype).view(m.heads, m.vdim, m.rank).contiguous()
            if m.rot_dims:
                lt.inv_freq = rotary_inv_freq(m.rot_dims, m.rot_base, 1.0).to(dev)
        else:
            lt = LayerTensors(w_in=act(p + "q", p + "k", p + "v", p + "g", p + "i", p + "f"), w_out=act(p + "o"),
                              norm1=f32(f"l{li}.norm1"))
            lt.gate_bias = f32(p + "i.b", p + "f.b")
            lt.o_norm = f32(p + "norm")
        lt.norm1b = f32(f"l{li}.norm1b")
        if mlp is not None:
            q = f"l{li}.mlp."
            lt.norm2, lt.norm2b = f32(f"l{li}.norm2"), f32(f"l{li}.norm2b")
            lt.w_router = sd[q + "router"].float().to(dev).contiguous()
            lt.w_up = torch.stack([sd[q + f"e{e}.up"] for e in range(mlp.experts)]).to(dev, dtype).contiguous()
            lt.w_dn = torch.stack([sd[q + f"e{e}.down"] for e in range(mlp.experts)]).to(dev, dtype).contiguous()
            if mlp.shared_ff:
                lt.w_sup, lt.w_sdn = act(q + "shared.up"), act(q + "shared.down")
        layers.append(lt)
    return RaggedDecoder(cfg, sd["embed"].to(dev, dtype).contiguous(), layers, f32("final.norm"),
                         sd["head"].to(dev, dtype).contiguous(), act_dtype=dtype, device=dev)


def load(path: str, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """Engine for the checkpoint directory ``path`` (config.json + model.safetensors)."""
    from .arch import load_checkpoint_tensors
    with open(os.path.join(path, "config.json")) as f:
        config = json.load(f)
    if not is_merusun(config):
        raise ValueError(f"{path}: not a {ARCHITECTURE} checkpoint")
    return build_engine(read_config(config), load_checkpoint_tensors(path), dtype, device)


def example_config(width=2048, layers=16, heads=16, kv_heads=4, dim=128, ff=1408, experts=64, top=6, groups=8, keep=4,
                   shared_ff=2816, vocab=32000, window=1024, rank=512, rot_dim=64, latent_dim=128, rec_heads=8,
                   rec_dim=128, rec_vdim=256) -> dict:
    """A config.json of this design at the proportions of a real model: of every four layers one windowed attention
    layer with keys of its own, one latent attention layer, one attention layer that reads the first one's cache, one
    mLSTM layer; every layer has routed experts.  For benchmarks and smoke tests (random weights)."""
    moe = {"kind": "moe", "expert": {"ff": ff}, "shared": {"ff": shared_ff},
           "router": {"experts": experts, "top": top, "scale": 2.0, "groups": {"count": groups, "keep": keep}}}
    out = []
    for i in range(layers):
        if i % 4 == 1:
            m = {"heads": heads, "dim": latent_dim, "rot_dim": rot_dim, "vdim": latent_dim, "kv_rank": rank,
                 "scale": (latent_dim + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": 10000.0}, "mask": {"size": window}}
            out.append({"type": "latent_attention", "mixer": m, "mlp": moe})
        elif i % 4 == 3:
            m = {"heads": rec_heads, "dim": rec_dim, "vdim": rec_vdim, "gate_cap": 15.0}
            out.append({"type": "mlstm", "mixer": m, "mlp": moe})
        else:
            m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": 8.0 * dim ** -0.5, "mask": {"size": window}}
            if i % 4 == 2:
                m["kv_from"] = i - 2
            out.append({"type": "attention", "mixer": m, "mlp": moe})
    return {"architecture": ARCHITECTURE, "embedding": {"scale": math.sqrt(width)}, "layers": out, "norm": {"eps": 1e-6},
            "vocab": vocab, "width": width}


def random_state_dict(config: dict, device="cuda", seed: int = 0) -> dict:
    """Random checkpoint tensors (bfloat16, created on ``device``) with the names and shapes the design gives them."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)
    D = config["width"]

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, device=dev, generator=g) * (s / math.sqrt(k))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, device=dev, generator=g)).to(torch.bfloat16)

    sd = {"embed": mat(config["vocab"], D, 1.0), "final.norm": vec(D, 1.0), "head": mat(config["vocab"], D)}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.mix.", layer["mixer"]
        for n in ("norm1", "norm1b"):
            sd[f"l{li}.{n}"] = vec(D, 1.0)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in [("q", H * d)] + ([] if m.get("kv_from") is not None else [("k", G * d), ("v", G * e)]):
                sd[p + n], sd[p + n + ".b"] = mat(rows, D), vec(rows)
            sd[p + "o"] = mat(D, H * e)
        elif layer["type"] == "latent_attention":
            H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            sd[p + "q"], sd[p + "dkv"], sd[p + "dkv.norm"] = mat(H * (d + r), D), mat(R + r, D), vec(R, 1.0)
            sd[p + "uk"], sd[p + "uv"], sd[p + "o"] = mat(H * d, R), mat(H * e, R), mat(D, H * e)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            sd[p + "q"], sd[p + "k"], sd[p + "v"], sd[p + "g"] = mat(H * d, D), mat(H * d, D), mat(H * e, D), mat(H * e, D)
            sd[p + "o"], sd[p + "norm"] = mat(D, H * e), vec(H * e, 1.0)
            sd[p + "i"], sd[p + "f"], sd[p + "i.b"], sd[p + "f.b"] = mat(H, D), mat(H, D), vec(H, 0.0, 1.0), vec(H, 3.0, 1.0)
        f = layer.get("mlp")
        if f is not None:
            q = f"l{li}.mlp."
            for n in ("norm2", "norm2b"):
                sd[f"l{li}.{n}"] = vec(D, 1.0)
            sd[q + "router"] = mat(f["router"]["experts"], D, 2.0)
            for e in range(f["router"]["experts"]):
                sd[q + f"e{e}.up"], sd[q + f"e{e}.down"] = mat(f["expert"]["ff"], D), mat(D, f["expert"]["ff"])
            if f.get("shared"):
                sd[q + "shared.up"], sd[q + "shared.down"] = mat(f["shared"]["ff"], D), mat(D, f["shared"]["ff"])
    return sd


def build_random(config: dict, dtype=torch.bfloat16, device="cuda", seed: int = 0) -> RaggedDecoder:
    return build_engine(read_config(config), random_state_dict(config, device, seed), dtype, device)
