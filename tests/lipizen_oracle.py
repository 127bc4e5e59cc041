"""Plain, slow statement of the Lipizen design in float64, one function per mechanism, whole sequences only (no cache,
no pages, no batches).  The tests compare the engine with it; it shares no code with the engine.

Notation: T tokens, H query heads, G key/value heads, d per-map query/key size, e value size.  ``W`` maps checkpoint
tensor names to float64 tensors; ``m`` is a mixer's entry of config.json.
"""
import math

import torch

F64 = torch.float64


def rms_div(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis"""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """the vector in `groups` consecutive parts, each divided by its own root mean square, then times w"""
    T, D = x.shape
    parts = [rms_div(x[:, g * (D // groups):(g + 1) * (D // groups)], eps) for g in range(groups)]
    return torch.cat(parts, -1) * w


def short_conv(u, w):
    """y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start; u [T, C], w [C, taps]"""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotate(x, pos, dims, base, factor):
    """x [..., n] at integer position pos: pairs (i, i + dims/2), angle pos * base^(-2i/dims) / factor"""
    out = x.clone()
    half = dims // 2
    for i in range(half):
        a = pos * (base ** (-2.0 * i / dims)) / factor
        c, s = math.cos(a), math.sin(a)
        out[..., i] = x[..., i] * c - x[..., i + half] * s
        out[..., i + half] = x[..., i + half] * c + x[..., i] * s
    return out


def sees(i, j, size, keep_first):
    if j > i:
        return False
    if size is None:
        return True
    return i - j < size or j < keep_first


def softmax_attend(q, ks, vs, scale):
    """q [d], ks [n, d], vs [n, e] -> [e]"""
    s = (ks @ q) * scale
    p = torch.exp(s - s.max())
    return (p / p.sum()) @ vs


def mixer_lambda(W, p, diff):
    return math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum())) - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + diff


def attention_mixer(h, W, p, m, eps, kv_store, li):
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot")
    mask = m.get("mask")
    size = mask["size"] if mask else None
    keep = mask["keep_first"] if mask else 0

    def branch(name, heads, width, norm, rotated):
        u = h @ W[p + name].T
        if m.get("conv"):
            u = short_conv(u, W[p + name + ".conv"])
        u = u.view(T, heads, -1, width)                      # [T, heads, maps, width]
        if norm:
            u = rms_div(u, eps) * W[p + name + ".norm"]
        if rotated and rot:
            fac = (rot.get("scaling") or {}).get("factor", 1.0)
            u = torch.stack([rotate(u[t], t, rot["dims"], rot["base"], fac) for t in range(T)])
        return u

    q = branch("q", H, d, True, True)
    if m.get("kv_from") is not None:
        k, v = kv_store[m["kv_from"]]
    else:
        k = branch("k", G, d, True, True)
        v = branch("v", G, e, False, False)[:, :, 0]
        kv_store[li] = (k, v)
    lam = mixer_lambda(W, p, m["diff"])
    gate = torch.sigmoid(h @ W[p + "g"].T)                   # [T, H]
    out = torch.zeros(T, H, e, dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if sees(i, j, size, keep)]
        for hh in range(H):
            g = hh // (H // G)
            a1 = softmax_attend(q[i, hh, 0], k[js, g, 0], v[js, g], m["scale"])
            a2 = softmax_attend(q[i, hh, 1], k[js, g, 1], v[js, g], m["scale"])
            o = rms_div(a1 - lam * a2, eps) * (1.0 - m["diff"])
            out[i, hh] = o * gate[i, hh]
    return out.reshape(T, H * e) @ W[p + "o"].T


def hgrn2_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = torch.nn.functional.silu(h @ W[p + "q"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, e)
    low = W[p + "lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).view(T, H, d)
    S = torch.zeros(H, d, e, dtype=F64)
    out = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        for hh in range(H):
            S[hh] = f[t, hh][:, None] * S[hh] + torch.outer(1 - f[t, hh], v[t, hh])
            out[t, hh] = S[hh].T @ q[t, hh]
    out = rms_div(out, eps) * W[p + "norm"]
    return out.reshape(T, H * e) @ W[p + "o"].T


def feed_forward(h, W, p, f):
    lim = f["limit"]
    g = torch.clamp(h @ W[p + "gate"].T, max=lim)
    u = torch.clamp(h @ W[p + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[p + "down"].T


def forward(config, W, tokens, layers_out=None):
    """logits [T, vocab] for one sequence of token ids"""
    eps, groups, alpha = config["norm"]["eps"], config["norm"]["groups"], config["postln_alpha"]
    x = W["embed"][torch.tensor(tokens)]
    kv = {}
    for li, layer in enumerate(config["layers"]):
        p = f"l{li}."
        if layer["type"] == "attention":
            y = attention_mixer(x, W, p + "mix.", layer["mixer"], eps, kv, li)
        else:
            y = hgrn2_mixer(x, W, p + "mix.", layer["mixer"], eps)
        x = group_norm(alpha * x + y, W[p + "norm1"], groups, eps)
        if layer.get("mlp") is not None:
            x = group_norm(alpha * x + feed_forward(x, W, p + "mlp.", layer["mlp"]), W[p + "norm2"], groups, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = group_norm(x, W["final.norm"], groups, eps) @ W["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


# ---------------------------------------------------------------------------------------------------------------
# small random models

def attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, diff=0.3, size=12, keep_first=2, rot_dims=8,
                    factor=2.0, kv_from=None, ff=48, limit=1.5):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff, "scale": dim ** -0.5}
    if conv:
        m["conv"] = conv
    if size is not None:
        m["mask"] = {"size": size, "keep_first": keep_first}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": 10000.0, "scaling": {"factor": factor}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def hgrn2_layer(heads=2, dim=16, vdim=16, ff=0, limit=1.5):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def make_config(layers, vocab=96, width=64, groups=2, alpha=2.0, softcap=10.0, eps=1e-6):
    return {"architecture": "Lipizen", "layers": layers, "logit_softcap": softcap, "norm": {"eps": eps, "groups": groups},
            "postln_alpha": alpha, "vocab": vocab, "width": width}


def random_weights(config, seed=0):
    """checkpoint tensors (bfloat16, as a checkpoint stores them) by name"""
    g = torch.Generator().manual_seed(seed)
    D = config["width"]

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, generator=g) * s / math.sqrt(k)).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    sd = {"embed": mat(config["vocab"], D, math.sqrt(D)), "final.norm": vec(D, 1.0), "head": mat(config["vocab"], D, 2.0)}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.", layer["mixer"]
        sd[p + "norm1"] = vec(D, 1.0)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            names = [("q", H * 2 * d)] + ([] if m.get("kv_from") is not None else [("k", G * 2 * d), ("v", G * e)])
            for n, rows in names:
                sd[p + "mix." + n] = mat(rows, D, 2.0)
                if m.get("conv"):
                    sd[p + f"mix.{n}.conv"] = (torch.randn(rows, m["conv"], generator=g) * 0.6).to(torch.bfloat16)
                if n != "v":
                    sd[p + f"mix.{n}.norm"] = vec(d, 1.0, 0.2)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                sd[p + "mix." + n] = vec(d, 0.0, 0.15)
            sd[p + "mix.g"] = mat(H, D, 2.0)
            sd[p + "mix.o"] = mat(D, H * e, 2.0)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            sd[p + "mix.q"], sd[p + "mix.f"], sd[p + "mix.v"] = mat(H * d, D, 2.0), mat(H * d, D, 3.0), mat(H * e, D, 2.0)
            sd[p + "mix.f.b"] = vec(H * d, 0.5, 1.0)
            sd[p + "mix.lower"] = torch.sigmoid(torch.randn(H * d, generator=g)).to(torch.bfloat16)
            sd[p + "mix.norm"] = vec(e, 1.0, 0.2)
            sd[p + "mix.o"] = mat(D, H * e, 2.0)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            sd[p + "norm2"] = vec(D, 1.0)
            sd[p + "mlp.gate"], sd[p + "mlp.up"], sd[p + "mlp.down"] = mat(ff, D, 2.0), mat(ff, D, 2.0), mat(D, ff, 2.0)
    return sd


def as_f64(sd):
    return {k: v.to(F64) for k, v in sd.items()}
