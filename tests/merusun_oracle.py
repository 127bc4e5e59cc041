"""Plain, slow float64 statement of the Merusun design: one function per mechanism, token by token where a mechanism has
a memory, nothing shared with ``bigdl_amd``.  Weights are a dict of float64 tensors by checkpoint name.

Notation: x is the residual stream [T, width]; a layer is x <- x + N_1b(mixer(N_1(x))), x <- x + N_2b(ff(N_2(x))) with
N(u) = w * u / sqrt(mean(u^2) + eps).
"""
import math

import torch

F64 = torch.float64


def unit(u, eps):
    return u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps)


def norm(u, w, eps):
    return unit(u, eps) * w


def visible(i, j, size):
    return j <= i and (size is None or size <= 0 or i - j < size)


# ---------------------------------------------------------------------------------------- windowed attention with a sink
def sink_attend(q, keys, values, scale, sink):
    """one query against its visible keys: weights exp(s_j) / (exp(sink) + sum exp(s_j))"""
    s = (keys @ q) * scale
    top = max(float(s.max()), sink)
    e = torch.exp(s - top)
    return (e / (e.sum() + math.exp(sink - top))) @ values


def attention_mixer(h, W, p, m, eps, store, li, sink=0.0):
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit((h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d), eps)
    if m.get("kv_from") is None:
        k = unit((h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d), eps)
        v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, e)
        store[li] = (k, v)
    else:
        k, v = store[m["kv_from"]]
    size = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, e, dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if visible(i, j, size)]
        for hh in range(H):
            g = hh // (H // G)
            out[i, hh] = sink_attend(q[i, hh], k[js, g], v[js, g], m["scale"], sink)
    return out.reshape(T, H * e) @ W[p + "o"].T


# ---------------------------------------------------------------------------------------- latent attention
def turn_pairs(u, pos, dims, base):
    """neighbouring pairs (2 i, 2 i + 1) of the first ``dims`` channels of u [..., n] turned by pos * base^(-2 i / dims)"""
    out = u.clone()
    for i in range(dims // 2):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(ang), math.sin(ang)
        a, b = u[..., 2 * i], u[..., 2 * i + 1]
        out[..., 2 * i], out[..., 2 * i + 1] = a * c - b * s, b * c + a * s
    return out


def latent_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    dims, base = rot.get("dims", 0), rot.get("base", 10000.0)
    q = (h @ W[p + "q"].T).view(T, H, d + r)
    low = h @ W[p + "dkv"].T
    c = norm(low[:, :R], W[p + "dkv.norm"], eps)
    shared = torch.stack([turn_pairs(low[t, R:], t, dims, base) for t in range(T)])
    keys = torch.cat([(c @ W[p + "uk"].T).view(T, H, d), shared[:, None, :].expand(T, H, r)], -1)       # [T, H, d + r]
    vals = (c @ W[p + "uv"].T).view(T, H, e)
    size = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, e, dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if visible(i, j, size)]
        for hh in range(H):
            qi = torch.cat([q[i, hh, :d], turn_pairs(q[i, hh, d:], i, dims, base)])
            out[i, hh] = torch.softmax((keys[js, hh] @ qi) * m["scale"], 0) @ vals[js, hh]
    return out.reshape(T, H * e) @ W[p + "o"].T


# ---------------------------------------------------------------------------------------- mLSTM
def mlstm_mixer(h, W, p, m, eps, m0=0.0, floor=1e-6):
    T = h.shape[0]
    H, d, e, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W[p + "q"].T).view(T, H, d) / math.sqrt(d)
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, e)
    li = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    out = torch.zeros(T, H, e, dtype=F64)
    for hh in range(H):
        S, n, mm = torch.zeros(d, e, dtype=F64), torch.zeros(d, dtype=F64), m0
        for t in range(T):
            new = max(float(lf[t, hh]) + mm, float(li[t, hh]))
            a, b = math.exp(float(lf[t, hh]) + mm - new), math.exp(float(li[t, hh]) - new)
            S = a * S + b * torch.outer(k[t, hh], v[t, hh])
            n = a * n + b * k[t, hh]
            mm = new
            out[t, hh] = (S.T @ q[t, hh]) / (max(abs(float(n @ q[t, hh])), math.exp(-mm)) + floor)
    o = unit(out, eps).reshape(T, H * e) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


# ---------------------------------------------------------------------------------------- routed experts
def choose(scores, count, keep, top):
    """indices of the ``top`` best experts among the ``keep`` groups whose best expert scores highest"""
    E = scores.numel()
    size = E // count
    best = [float(scores[g * size:(g + 1) * size].max()) for g in range(count)]
    kept = sorted(range(count), key=lambda g: -best[g])[:keep]
    allowed = [e for e in range(E) if e // size in kept]
    return sorted(allowed, key=lambda e: -float(scores[e]))[:top]


def expert(u, up, down):
    return down @ torch.relu(up @ u).pow(2)


def routed_ff(h, W, p, f):
    r = f["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        s = torch.softmax(W[p + "router"] @ h[t], 0)
        for e in choose(s, g["count"], g["keep"], r["top"]):
            out[t] += s[e] * r.get("scale", 1.0) * expert(h[t], W[p + f"e{e}.up"], W[p + f"e{e}.down"])
        if f.get("shared"):
            out[t] += expert(h[t], W[p + "shared.up"], W[p + "shared.down"])
    return out


# ---------------------------------------------------------------------------------------- the model
def forward(config, W, tokens, layers_out=None):
    eps = config["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * config["embedding"]["scale"]
    store = {}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.", layer["mixer"]
        h = norm(x, W[p + "norm1"], eps)
        if layer["type"] == "attention":
            y = attention_mixer(h, W, p + "mix.", m, eps, store, li)
        elif layer["type"] == "latent_attention":
            y = latent_mixer(h, W, p + "mix.", m, eps)
        else:
            y = mlstm_mixer(h, W, p + "mix.", m, eps)
        x = x + norm(y, W[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            x = x + norm(routed_ff(norm(x, W[p + "norm2"], eps), W, p + "mlp.", layer["mlp"]), W[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm(x, W["final.norm"], eps) @ W["head"].T


# ---------------------------------------------------------------------------------------- small configurations
def moe(experts=8, top=2, ff=24, count=4, keep=2, scale=1.7, shared=40):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale,
                                                            "groups": {"count": count, "keep": keep}}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=24, size=12, scale=0.9, kv_from=None, mlp="default"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        m["mask"] = {"size": size}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": moe() if mlp == "default" else mlp}


def latent_layer(heads=3, dim=16, rot_dim=8, vdim=20, rank=24, size=15, scale=0.3, base=50.0, mlp="default"):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "rot": {"dims": rot_dim, "base": base}}
    if size:
        m["mask"] = {"size": size}
    return {"type": "latent_attention", "mixer": m, "mlp": moe() if mlp == "default" else mlp}


def mlstm_layer(heads=2, dim=16, vdim=24, cap=6.0, mlp="default"):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": moe() if mlp == "default" else mlp}


def make_config(layers, vocab=96, width=64, scale=3.0, eps=1e-5):
    return {"architecture": "Merusun", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps}, "vocab": vocab,
            "width": width}


def random_weights(config, seed=0):
    """bfloat16 checkpoint tensors; gate biases and router rows are wide enough that gates and choices vary"""
    g = torch.Generator().manual_seed(seed)
    D = config["width"]

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, generator=g) * (s / math.sqrt(k))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    sd = {"embed": mat(config["vocab"], D, 1.0), "final.norm": vec(D, 1.0), "head": mat(config["vocab"], D)}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.mix.", layer["mixer"]
        sd[f"l{li}.norm1"], sd[f"l{li}.norm1b"] = vec(D, 1.0), vec(D, 0.7)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            names = [("q", H * d)] + ([] if m.get("kv_from") is not None else [("k", G * d), ("v", G * e)])
            for n, rows in names:
                sd[p + n], sd[p + n + ".b"] = mat(rows, D, 2.0), vec(rows, 0.0, 0.3)
            sd[p + "o"] = mat(D, H * e)
        elif layer["type"] == "latent_attention":
            H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            sd[p + "q"], sd[p + "dkv"], sd[p + "dkv.norm"] = mat(H * (d + r), D, 2.0), mat(R + r, D, 2.0), vec(R, 1.0, 0.2)
            sd[p + "uk"], sd[p + "uv"], sd[p + "o"] = mat(H * d, R, 2.0), mat(H * e, R), mat(D, H * e)
        else:
            H, d, e = m["heads"], m["dim"], m["vdim"]
            sd[p + "q"], sd[p + "k"], sd[p + "v"], sd[p + "g"] = mat(H * d, D, 2.0), mat(H * d, D, 2.0), mat(H * e, D), mat(H * e, D)
            sd[p + "o"], sd[p + "norm"] = mat(D, H * e), vec(H * e, 1.0, 0.2)
            sd[p + "i"], sd[p + "f"] = mat(H, D, 3.0), mat(H, D, 3.0)
            sd[p + "i.b"], sd[p + "f.b"] = vec(H, 0.0, 2.0), vec(H, 2.0, 2.0)
        f = layer.get("mlp")
        if f is not None:
            q = f"l{li}.mlp."
            sd[f"l{li}.norm2"], sd[f"l{li}.norm2b"] = vec(D, 1.0), vec(D, 0.7)
            sd[q + "router"] = mat(f["router"]["experts"], D, 3.0)
            for e in range(f["router"]["experts"]):
                sd[q + f"e{e}.up"], sd[q + f"e{e}.down"] = mat(f["expert"]["ff"], D, 1.5), mat(D, f["expert"]["ff"], 1.5)
            if f.get("shared"):
                sd[q + "shared.up"], sd[q + "shared.down"] = mat(f["shared"]["ff"], D, 1.5), mat(D, f["shared"]["ff"], 1.5)
    return sd


def as_f64(sd):
    return {k: v.double() for k, v in sd.items()}
