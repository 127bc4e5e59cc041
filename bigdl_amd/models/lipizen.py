"""Lipizen on the ragged engine: reader of its ``config.json`` and the map from checkpoint tensor names to
``LayerTensors``.

The design: a post-sum norm decoder (x <- norm(alpha * x + sublayer(x)), grouped RMS norm) whose token mixers are either
windowed differential attention (two score maps per head, short convolutions behind q / k / v, per-head query / key
norm, partial rotary with linear scaling, kept first tokens, per-head sigmoid gate, optional reuse of another layer's
keys and values) or HGRN2 recurrences, with clamped gated feed-forwards and soft-capped logits.
"""
from __future__ import annotations

import json
import math
import os

import torch

from .ragged_engine import ClampedGlu, Hgrn2, LayerTensors, RaggedConfig, RaggedDecoder, WindowAttention, rotary_inv_freq

ARCHITECTURE = "Lipizen"
GLU_SLOPE = 1.702          # fixed by the design


def is_lipizen(config: dict) -> bool:
    return config.get("architecture") == ARCHITECTURE


def read_config(config: dict) -> RaggedConfig:
    mixers, mlps = [], []
    for layer in config["layers"]:
        m, kind = layer["mixer"], layer["type"]
        if kind == "attention":
            rot = m.get("rot") or {}
            mask = m.get("mask") or {}
            diff = float(m.get("diff", 0.0))
            mixers.append(WindowAttention(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]), maps=2, lam=diff, out_scale=1.0 - diff, out_norm=True,
                conv_taps=int(m.get("conv") or 0), qk_norm=True, rot_dims=int(rot.get("dims") or 0),
                rot_base=float(rot.get("base", 10000.0)), rot_factor=float((rot.get("scaling") or {}).get("factor", 1.0)),
                window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0), gate=True,
                kv_from=m.get("kv_from")))
        elif kind == "hgrn2":
            mixers.append(Hgrn2(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"])))
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        f = layer.get("mlp")
        if f is None:
            mlps.append(None)
        elif f.get("kind", "dense") == "dense":
            mlps.append(ClampedGlu(ff=int(f["ff"]), limit=float(f["limit"]), slope=GLU_SLOPE))
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    norm = config.get("norm") or {}
    return RaggedConfig(vocab=int(config["vocab"]), width=int(config["width"]), mixers=mixers, mlps=mlps,
                        norm_eps=float(norm.get("eps", 1e-6)), norm_groups=int(norm.get("groups", 1)),
                        residual_alpha=float(config.get("postln_alpha", 1.0)),
                        logit_softcap=float(config.get("logit_softcap") or 0.0), name=ARCHITECTURE)


def build_engine(cfg: RaggedConfig, sd: dict, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """``sd``: checkpoint tensors by name ('l<i>.mix.q', 'l<i>.mlp.gate', ...).  Projection weights take the activation
    type; norm weights, convolution taps, biases and bounds become float32 (what reads them computes in 32 bits)."""
    dev = torch.device(device)

    def act(*names):
        return torch.cat([sd[n] for n in names], 0).to(dev, dtype).contiguous()

    def f32(*names):
        return torch.cat([sd[n].float().reshape(sd[n].shape[0], -1) for n in names], 0).to(dev).contiguous()

    layers = []
    for li, (m, mlp) in enumerate(zip(cfg.mixers, cfg.mlps)):
        p = f"l{li}."
        if isinstance(m, WindowAttention):
            own = m.kv_from is None
            proj = ["q", "k", "v"] if own else ["q"]
            lt = LayerTensors(w_in=act(*[p + "mix." + n for n in proj], p + "mix.g"), w_out=act(p + "mix.o"),
                              norm1=f32(p + "norm1").view(-1))
            if m.conv_taps:
                lt.conv_w = f32(*[p + f"mix.{n}.conv" for n in proj])
            lt.q_norm = f32(p + "mix.q.norm").view(-1)
            if own:
                lt.k_norm = f32(p + "mix.k.norm").view(-1)
            if m.rot_dims:
                lt.inv_freq = rotary_inv_freq(m.rot_dims, m.rot_base, m.rot_factor).to(dev)
            # the second map's weight: exp(<lq1, lk1>) - exp(<lq2, lk2>) + diff, one number per layer, in float32
            lq1, lk1, lq2, lk2 = (sd[p + "mix." + n].float() for n in ("lq1", "lk1", "lq2", "lk2"))
            m.lam = math.exp(float((lq1 * lk1).sum())) - math.exp(float((lq2 * lk2).sum())) + (1.0 - m.out_scale)
        else:
            lt = LayerTensors(w_in=act(p + "mix.q", p + "mix.f", p + "mix.v"), w_out=act(p + "mix.o"),
                              norm1=f32(p + "norm1").view(-1), f_bias=f32(p + "mix.f.b").view(-1),
                              lower=f32(p + "mix.lower").view(-1), o_norm=f32(p + "mix.norm").view(-1))
        if mlp is not None:
            lt.w_gu = act(p + "mlp.gate", p + "mlp.up")
            lt.w_down = act(p + "mlp.down")
            lt.norm2 = f32(p + "norm2").view(-1)
        layers.append(lt)
    return RaggedDecoder(cfg, sd["embed"].to(dev, dtype).contiguous(), layers, f32("final.norm").view(-1),
                         sd["head"].to(dev, dtype).contiguous(), act_dtype=dtype, device=dev)


def load(path: str, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """Engine for the checkpoint directory ``path`` (config.json + model.safetensors)."""
    from .arch import load_checkpoint_tensors
    with open(os.path.join(path, "config.json")) as f:
        config = json.load(f)
    if not is_lipizen(config):
        raise ValueError(f"{path}: not a {ARCHITECTURE} checkpoint")
    return build_engine(read_config(config), load_checkpoint_tensors(path), dtype, device)


def example_config(width=2048, layers=16, heads=16, kv_heads=4, dim=64, vdim=128, ff=5632, vocab=32000, window=1024,
                   keep_first=4, conv=4, rec_heads=16, rec_dim=128, groups=4) -> dict:
    """A config.json of this design at the proportions of a real model: of every four layers two attention layers with
    keys of their own, one HGRN2 layer without a feed-forward, one attention layer that reads the cache of the layer
    before the recurrence.  For benchmarks and smoke tests (random weights)."""
    def attn(kv_from=None):
        m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": 0.5, "scale": dim ** -0.5, "conv": conv,
             "mask": {"size": window, "keep_first": keep_first},
             "rot": {"dims": dim // 2, "base": 10000.0, "scaling": {"factor": 2.0}}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff, "limit": 7.0}}
    out = []
    for i in range(layers):
        if i % 4 == 2:
            out.append({"type": "hgrn2", "mixer": {"heads": rec_heads, "dim": rec_dim, "vdim": rec_dim}, "mlp": None})
        elif i % 4 == 3:
            out.append(attn(kv_from=i - 2))
        else:
            out.append(attn())
    return {"architecture": ARCHITECTURE, "layers": out, "logit_softcap": 30.0, "norm": {"eps": 1e-6, "groups": groups},
            "postln_alpha": 2.0, "vocab": vocab, "width": width}


def random_state_dict(config: dict, device="cuda", seed: int = 0) -> dict:
    """Random checkpoint tensors (bfloat16, created on ``device``) with the names and shapes the design gives them."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)
    D = config["width"]

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, device=dev, generator=g) * (s / math.sqrt(k))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, device=dev, generator=g)).to(torch.bfloat16)

    sd = {"embed": mat(config["vocab"], D, math.sqrt(D)), "final.norm": vec(D, 1.0), "head": mat(config["vocab"], D)}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.", layer["mixer"]
        sd[p + "norm1"] = vec(D, 1.0)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, rows in [("q", H * 2 * d)] + ([] if m.get("kv_from") is not None else [("k", G * 2 * d), ("v", G * e)]):
                sd[p + "mix." + n] = mat(rows, D)
                if m.get("conv"):
                    sd[p + f"mix.{n}.conv"] = (torch.randn(rows, m["conv"], device=dev, generator=g) * 0.5).to(torch.bfloat16)
                if n != "v":
                    sd[p + f"mix.{n}.norm"] = vec(d, 1.0)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                sd[p + "mix." + n] = vec(d)
            sd[p + "mix.g"], sd[p + "mix.o"] = mat(H, D), mat(D, H * e)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            sd[p + "mix.q"], sd[p + "mix.f"], sd[p + "mix.v"], sd[p + "mix.o"] = mat(H * d, D), mat(H * d, D), mat(H * e, D), mat(D, H * e)
            sd[p + "mix.f.b"] = vec(H * d, 1.0, 1.0)
            sd[p + "mix.lower"] = torch.sigmoid(torch.randn(H * d, device=dev, generator=g)).to(torch.bfloat16)
            sd[p + "mix.norm"] = vec(e, 1.0)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            sd[p + "norm2"] = vec(D, 1.0)
            sd[p + "mlp.gate"], sd[p + "mlp.up"], sd[p + "mlp.down"] = mat(ff, D), mat(ff, D), mat(D, ff)
    return sd


def build_random(config: dict, dtype=torch.bfloat16, device="cuda", seed: int = 0) -> RaggedDecoder:
    return build_engine(read_config(config), random_state_dict(config, device, seed), dtype, device)
