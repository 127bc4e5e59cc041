"""The Lipizen design on the ragged engine against the plain float64 statement in ``lipizen_oracle.py``.

Every test runs twice: on the CPU (the engine's bookkeeping over the unfused statements of ``ops/ragged.py``) and,
marked ``gpu``, on the device (the HIP kernels of ``libbigdl_ragged.so``).  Models are small and random; where random
weights would hide a fault (one far key among many, a window's edge) the inputs are made so that one score stands out.
"""
import json
import math
import os
import random

import pytest
import torch

import lipizen_oracle as O
from bigdl_amd.models import lipizen
from bigdl_amd.models.paged import PagedStatePool, PoolExhausted
from bigdl_amd.ops import ragged as R

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32_TOL = 3e-4


def engine_for(config, sd, dtype, device):
    return lipizen.build_engine(lipizen.read_config(config), sd, dtype, device)


def full_model(**over):
    layers = [O.attention_layer(), O.attention_layer(conv=4, size=20, keep_first=3, rot_dims=16, factor=1.0),
              O.hgrn2_layer(), O.attention_layer(kv_from=1, conv=2, size=9, keep_first=0, rot_dims=16, factor=1.0),
              O.hgrn2_layer(heads=1, dim=40, vdim=24, ff=32), O.attention_layer(kv_from=0, ff=0)]
    return O.make_config(layers, **over)


def tokens(n, vocab, seed):
    rnd = random.Random(seed)
    return [rnd.randrange(vocab) for _ in range(n)]


def run_schedule(engine, prompts, schedule, max_tokens, slots=4, seen_pages=None):
    """schedule: steps of [(request, count)]; returns {request: logits of all its positions [T, V]} (float64, host)"""
    engine.pool = None
    pool = engine.ensure_pool(max_tokens, slots)
    at, slot, got = {}, {}, {k: [] for k in prompts}
    for step in schedule:
        entries, want = [], []
        for rid, n in step:
            if rid not in slot:
                slot[rid] = pool.admit()
            lo = at.get(rid, 0)
            entries.append((slot[rid], prompts[rid][lo:lo + n]))
            want.append(list(range(n)))
            at[rid] = lo + n
        logits = engine.step(entries, want).double().cpu()
        row = 0
        for rid, n in step:
            got[rid].append(logits[row:row + n])
            row += n
            if seen_pages is not None:
                seen_pages.setdefault(rid, set()).update(pool.pages_of[slot[rid]])
            if at[rid] == len(prompts[rid]):
                pool.release(slot.pop(rid))
    return {k: torch.cat(v) for k, v in got.items() if v}


def close(a, b, tol=F32_TOL):
    assert a.shape == b.shape
    err = float((a - b).abs().max())
    assert err <= tol, f"max difference {err}"


# ------------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layers", [
    [O.attention_layer(ff=0)], [O.hgrn2_layer()], [O.attention_layer()], [O.hgrn2_layer(ff=40)],
    [O.attention_layer(heads=3, kv_heads=3, dim=24, vdim=80, conv=0, size=None, rot_dims=24, factor=1.0, diff=0.8)],
    [O.attention_layer(heads=6, kv_heads=1, dim=20, vdim=12, conv=2, size=200, keep_first=0, rot_dims=0)],
    [O.attention_layer(heads=2, kv_heads=1, dim=18, vdim=15, conv=3, size=10, keep_first=1, rot_dims=6)],
    [O.attention_layer(heads=8, kv_heads=1, dim=32, vdim=272, conv=1, size=33, keep_first=70, rot_dims=32, ff=0)],
    [O.attention_layer(heads=8, kv_heads=1, dim=32, vdim=64, conv=2, size=70, keep_first=2, rot_dims=16, ff=0),
     O.attention_layer(heads=6, kv_heads=3, dim=64, vdim=192, conv=0, size=40, keep_first=0, rot_dims=0, ff=0)],
    [O.attention_layer(heads=4, kv_heads=2, dim=12, vdim=20, conv=3, size=30, keep_first=2, rot_dims=12, ff=0),
     O.attention_layer(heads=8, kv_heads=2, dim=24, vdim=200, conv=3, size=30, keep_first=2, rot_dims=8, ff=0)],
], ids=["attention", "hgrn2", "attention+ff", "hgrn2+ff", "full-mask-wide-values", "one-kv-head-no-rotation",
        "odd-sizes", "eight-heads-per-kv-head-very-wide-values", "shared-reads-of-8-and-2-heads",
        "key-rows-that-do-not-divide-a-wavefront"])
def test_each_layer_kind_alone(device, layers):
    cfg = O.make_config(layers, groups=1 if len(layers[0]["mixer"]) < 4 else 2)
    sd = O.random_weights(cfg, seed=1)
    toks = tokens(85, cfg["vocab"], 2)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 45)], [("a", 38)], [("a", 1)], [("a", 1)]], 128)["a"]
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_layer_outputs_one_by_one(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=3)
    toks = tokens(30, cfg["vocab"], 4)
    ref_layers = []
    O.forward(cfg, O.as_f64(sd), toks, ref_layers)
    eng = engine_for(cfg, sd, torch.float32, device)
    pool = eng.ensure_pool(64, 1)
    mine = []
    eng.step([(pool.admit(), toks)], collect=mine)
    for li, (a, b) in enumerate(zip(mine, ref_layers)):
        assert float((a.double().cpu() - b).abs().max()) < 1e-4, f"layer {li}"


@pytest.mark.parametrize("device", DEVICES)
def test_prompt_against_token_by_token_and_portions(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=5)
    toks = tokens(150, cfg["vocab"], 6)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.float32, device)
    whole = run_schedule(eng, {"a": toks}, [[("a", 150)]], 192)["a"]
    close(whole, want)
    one_by_one = run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in range(150)], 192)["a"]
    close(one_by_one, want)
    for sizes in ([2] * 75, [64, 2, 62, 3, 1, 1, 17], [63, 1, 1, 63, 2, 20], [5, 128, 2, 2, 13], [1, 2, 3, 4, 5, 64, 65, 6]):
        assert sum(sizes) == 150
        got = run_schedule(eng, {"a": toks}, [[("a", n)] for n in sizes], 192)["a"]
        close(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_requests_in_one_batch_and_reuse_of_pages_and_slots(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=7)
    W = O.as_f64(sd)
    lens = {"a": 130, "b": 7, "c": 70, "d": 1, "e": 66, "f": 90}
    prompts = {k: tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg, W, p) for k, p in prompts.items()}
    # three slots, pool of 5 pages (320 tokens) for 364 tokens in total: d, e, f run in what a, b, c gave back
    schedule = [[("a", 60), ("b", 2), ("c", 1)], [("a", 1), ("b", 5), ("c", 63)], [("a", 5), ("c", 6)],
                [("a", 64), ("d", 1)], [("e", 2), ("f", 30)], [("e", 64), ("f", 1)], [("f", 59)]]
    eng = engine_for(cfg, sd, torch.float32, device)
    seen = {}
    got = run_schedule(eng, prompts, schedule, 320, slots=3, seen_pages=seen)
    for k in prompts:
        close(got[k], want[k])
    assert (seen["e"] | seen["f"] | seen["d"]) & (seen["a"] | seen["b"] | seen["c"]), "no page was used twice"
    # each alone gives the same as inside the batch
    alone = run_schedule(eng, {"c": prompts["c"]}, [[("c", 70)]], 128)["c"]
    close(alone, got["c"], 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_long_and_short_portions_side_by_side_through_the_recurrence(device):
    """a portion long enough for the chunked scan next to a short one and a single token, then the long one goes on"""
    cfg = O.make_config([O.hgrn2_layer(heads=2, dim=24, vdim=20, ff=32), O.hgrn2_layer(heads=1, dim=70, vdim=33)])
    sd = O.random_weights(cfg, seed=17)
    W = O.as_f64(sd)
    prompts = {"a": tokens(1400, cfg["vocab"], 18), "b": tokens(41, cfg["vocab"], 19), "c": tokens(3, cfg["vocab"], 20)}
    want = {k: O.forward(cfg, W, p) for k, p in prompts.items()}
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, prompts, [[("c", 2), ("a", 700), ("b", 40)], [("a", 1), ("b", 1), ("c", 1)], [("a", 699)]], 1600)
    for k in prompts:
        close(got[k], want[k])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_windows_and_pages(device):
    cfg = O.make_config([O.attention_layer(size=16, keep_first=3), O.hgrn2_layer(),
                         O.attention_layer(size=70, keep_first=1, kv_from=0)])
    sd = O.random_weights(cfg, seed=9)
    toks = tokens(200, cfg["vocab"], 11)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)] for _ in range(195)], 256)["a"]
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("odd", [False, True])
def test_bfloat16_stays_near_the_exact_result(device, odd):
    cfg = full_model()
    if odd:          # sizes that take none of the vector or matrix-core paths
        cfg = O.make_config([O.attention_layer(heads=2, kv_heads=1, dim=20, vdim=30, rot_dims=10),
                             O.hgrn2_layer(heads=1, dim=36, vdim=20), O.attention_layer(heads=2, kv_heads=1, dim=20, vdim=30,
                                                                                        rot_dims=10, kv_from=0, conv=0)])
    sd = O.random_weights(cfg, seed=13)
    toks = tokens(100, cfg["vocab"], 14)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.bfloat16, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 70)], [("a", 2)]] + [[("a", 1)] for _ in range(28)], 128)["a"]
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    rel = d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    assert float(rel.max()) < 0.08, float(rel.max())


# ------------------------------------------------------------------------------------------------ mechanisms alone
def _meta_for(pool, slot, n, device):
    pages = list(pool.reserve(slot, n))
    return R.BatchMeta([(slot, pool.len_of[slot], n, pages)], torch.device(device))


def _attend_through_pages(device, q, k, v, portions, *, window, keep_first, scale, lam, page_order=None):
    """q [T, H, 2, d], k [T, G, 2, d], v [T, G, e] (float64) through the paged attention op in the given portions"""
    T, H, _, d = q.shape
    G, e = v.shape[1], v.shape[2]
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("kv", G, 2 * d, e)]}, 64 * ((T + 63) // 64 + 2), 2, torch.float32, device)
    if page_order:
        pool.free_pages = list(page_order)
    slot = pool.admit()
    out, at = [], 0
    for n in portions:
        meta = _meta_for(pool, slot, n, device)
        for i in range(n):                                   # place keys / values as the cache holds them
            pos = at + i
            pg = pool.pages_of[slot][pos // 64]
            pool.k[0][pg, :, pos % 64] = k[pos].reshape(G, 2 * d).float().to(device)
            pool.v[0][pg, :, pos % 64] = v[pos].float().to(device)
        qq = q[at:at + n].reshape(n, H * 2 * d).float().to(device).contiguous()
        out.append(ops.paged_attn(qq, pool.k[0], pool.v[0], meta, maps=2, H=H, G=G, d=d, vd=e, window=window,
                                  keep_first=keep_first, scale=scale, lam=lam, out_scale=1.0, out_norm=False, eps=1e-6))
        pool.commit(slot, n)
        at += n
    return torch.cat(out).double().cpu().view(T, H, e)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode_tail", [0, 12])
def test_window_edges_far_keys_and_page_borders_stand_out(device, decode_tail):
    """Query i and key j are made parallel and long, so key j takes all of the weight when it is visible; its value is
    a marker.  One position off in the window, the kept first tokens or a page's border swaps the marker in or out."""
    g = torch.Generator().manual_seed(21)
    T, H, G, d, e, window, keep = 210, 2, 1, 8, 4, 70, 3
    cases = []                                               # (query position, key position)
    for i in (140, 191, 192, 193, 209):
        cases += [(i, i - window + 1), (i, i - window), (i, keep - 1), (i, keep), (i, 0)]
    cases += [(100, 63), (100, 64), (130, 127), (130, 128), (64, 63), (64, 64), (69, 0), (70, 0), (70, 1), (72, 3)]
    for i, j in cases:
        q = torch.randn(T, H, 2, d, generator=g, dtype=O.F64) * 0.1
        k = torch.randn(T, G, 2, d, generator=g, dtype=O.F64) * 0.1
        v = torch.randn(T, G, e, generator=g, dtype=O.F64) * 0.1
        u = torch.randn(d, generator=g, dtype=O.F64)
        u = u / u.norm()
        q[i, :, 0], k[j, :, 0] = 8.0 * u, 8.0 * u            # map 1 only: score 64 where everything else is ~0
        v[j] = 5.0
        want = torch.zeros(H, e, dtype=O.F64)
        js = [x for x in range(T) if O.sees(i, x, window, keep)]
        for hh in range(H):
            want[hh] = O.softmax_attend(q[i, hh, 0], k[js, 0, 0], v[js, 0], 1.0) - 0.5 * O.softmax_attend(q[i, hh, 1], k[js, 0, 1], v[js, 0], 1.0)
        visible = O.sees(i, j, window, keep)
        assert (float(want.abs().max()) > 3.0) == visible
        portions = [T] if not decode_tail else [T - decode_tail - 40, 40] + [1] * decode_tail
        if decode_tail and i < T - decode_tail:
            continue                                         # this case's query is not a decoded token
        got = _attend_through_pages(device, q, k, v, portions, window=window, keep_first=keep, scale=1.0, lam=0.5,
                                    page_order=[1, 4, 0, 3, 2, 5][::-1])
        close(got[i], want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,portions", [(2, [1, 1, 5, 2, 64, 7]), (3, [1, 1, 1, 2, 70, 5]), (4, [1, 2, 1, 1, 1, 74]), (4, [80])])
def test_short_convolution_norm_rotation_and_state(device, taps, portions):
    g = torch.Generator().manual_seed(31)
    T, heads, width, rot = sum(portions), 3, 12, 8
    C = heads * width + 5                                   # the segment sits inside a wider convolved region
    u = torch.randn(T, C + 4, generator=g, dtype=O.F64)     # and that inside a wider projection matrix
    cw = torch.randn(C, taps, generator=g, dtype=O.F64)
    nw = 1 + 0.2 * torch.randn(width, generator=g, dtype=O.F64)
    col0, ch0 = 2 + 5, 5
    y = O.short_conv(u[:, 2:2 + C], cw)[:, ch0:ch0 + heads * width].reshape(T, heads, width)
    y = O.rms_div(y, 1e-6) * nw
    want = torch.stack([O.rotate(y[t], t, rot, 100.0, 2.0) for t in range(T)]).reshape(T, heads * width)
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("tail", taps - 1, C)]}, 128, 3, torch.float32, device)
    pool.admit()
    slot = pool.admit()                                      # not slot 0
    pool.tail[0].fill_(7.0)                                  # a slot that was used before holds anything
    inv = lipizen.rotary_inv_freq(rot, 100.0, 2.0).to(device)
    out, at = [], 0
    for n in portions:
        meta = _meta_for(pool, slot, n, device)
        P = u[at:at + n].float().to(device).contiguous()
        dense = torch.empty(n, heads * width, dtype=torch.float32, device=device)
        ops.conv_head(P, col0, meta, cw=cw.float().to(device).contiguous(), taps=taps, C=C, ch0=ch0, state=pool.tail[0],
                      ngroups=heads, gsize=width, normw=nw.float().to(device), eps=1e-6, rot=rot, inv_freq=inv, out_dense=dense)
        ops.conv_state(P, 2, pool.tail[0], taps, C, meta)
        pool.commit(slot, n)
        out.append(dense)
        at += n
    close(torch.cat(out).double().cpu(), want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,dim,vdim,portions", [(2, 16, 16, (1, 2, 64, 1, 22)), (1, 40, 24, (1, 2, 64, 1, 22)),
                                                     (3, 80, 70, (1, 2, 64, 1, 22)), (1, 8, 130, (1, 2, 64, 1, 22)),
                                                     (2, 48, 40, (530, 3, 700))])
def test_hgrn2_recurrence_and_its_state(device, heads, dim, vdim, portions):
    g = torch.Generator().manual_seed(41)
    cfg = O.make_config([O.hgrn2_layer(heads=heads, dim=dim, vdim=vdim)], width=32)
    sd = O.random_weights(cfg, seed=42)
    W = O.as_f64(sd)
    T = sum(portions)                      # (portions of 512 tokens and more run in chunks on the GPU)
    h = torch.randn(T, 32, generator=g, dtype=O.F64)
    m = cfg["layers"][0]["mixer"]
    # the oracle's mixer up to (not including) the output norm and projection
    q = torch.nn.functional.silu(h @ W["l0.mix.q"].T)
    fpre = h @ W["l0.mix.f"].T
    v = h @ W["l0.mix.v"].T
    low = W["l0.mix.lower"]
    f = (low + (1 - low) * torch.sigmoid(fpre + W["l0.mix.f.b"])).view(T, heads, dim)
    S = torch.zeros(heads, dim, vdim, dtype=O.F64)
    want = torch.zeros(T, heads, vdim, dtype=O.F64)
    for t in range(T):
        S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t].view(heads, 1, vdim)
        want[t] = torch.einsum("hde,hd->he", S, q[t].view(heads, dim))
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("matrix", heads, dim, vdim)]}, T + 64, 2, torch.float32, device)
    pool.admit()
    slot = pool.admit()
    pool.matrix[0].fill_(3.0)                                # left by an earlier sequence: must not leak in
    P = torch.cat([h @ W["l0.mix.q"].T, fpre, v], 1).float().to(device).contiguous()
    hd = heads * dim
    out, at = [], 0
    for n in portions:
        meta = _meta_for(pool, slot, n, device)
        Pn = P[at:at + n].contiguous()
        qf, ff = ops.hgrn2_gates(Pn, 0, hd, W["l0.mix.f.b"].float().to(device), low.float().to(device), hd)
        out.append(ops.hgrn2_scan(qf, ff, Pn, 2 * hd, pool.matrix[0], heads, dim, vdim, meta))
        pool.commit(slot, n)
        at += n
    close(torch.cat(out).double().cpu().view(T, heads, vdim), want, 1e-4)
    close(pool.matrix[0][slot].double().cpu(), S, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_grouped_norm_of_the_sum_and_clamped_unit(device):
    g = torch.Generator().manual_seed(51)
    ops = R.ops_for(device)
    for D, groups in ((48, 1), (48, 4), (520, 2)):
        x = torch.randn(9, D, generator=g, dtype=O.F64)
        y = torch.randn(9, D, generator=g, dtype=O.F64)
        w = 1 + 0.3 * torch.randn(D, generator=g, dtype=O.F64)
        want = O.group_norm(1.7 * x + y, w, groups, 1e-5)
        xd = x.float().to(device)
        xa = ops.sum_group_norm(xd, y.float().to(device), w.float().to(device), groups, 1.7, 1e-5, torch.float32)
        close(xd.double().cpu(), want, 1e-5)
        close(xa.double().cpu(), want, 1e-5)
    gu = torch.randn(7, 2 * 33, generator=g, dtype=O.F64) * 3
    gg, uu = gu[:, :33].clamp(max=1.25), gu[:, 33:].clamp(-1.25, 1.25)
    want = gg * torch.sigmoid(1.702 * gg) * (uu + 1)
    close(ops.clamped_glu(gu.float().to(device).contiguous(), 1.25, 1.702).double().cpu(), want, 1e-5)


# ------------------------------------------------------------------------------------------------ pool, scheduler, entry points
def test_pool_hands_pages_and_slots_out_again():
    pool = PagedStatePool({0: [("kv", 1, 4, 4)]}, 64 * 3, 2, torch.float32, "cpu")
    a, b = pool.admit(), pool.admit()
    with pytest.raises(PoolExhausted):
        pool.admit()
    pa = list(pool.reserve(a, 65))
    pool.commit(a, 65)
    assert len(pa) == 2 and len(pool.reserve(a, 63)) == 2 and len(pool.reserve(b, 64)) == 1
    with pytest.raises(PoolExhausted):
        pool.reserve(b, 65)
    pool.release(a)
    c = pool.admit()
    assert c == a and pool.len_of[c] == 0 and set(pool.reserve(b, 65)) & set(pa)


def _save_checkpoint(tmp_path, cfg, sd):
    from safetensors.torch import save_file
    path = str(tmp_path / "model")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    return path


def _greedy_is_consistent(cfg, W, sequence, n_prompt):
    """every generated token is the oracle's argmax given what came before it, or within a rounding-sized gap of it"""
    logits = O.forward(cfg, W, sequence[:-1])
    for t in range(n_prompt, len(sequence)):
        row = logits[t - 1]
        assert float(row.max() - row[sequence[t]]) < 1e-3, f"token {t}"


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_auto_class_and_the_scheduler(device, tmp_path):
    from bigdl_amd.serving.continuous import ContinuousBatcher, SeqRequest
    from bigdl_amd.transformers import AutoModelForCausalLM
    cfg = full_model()
    sd = O.random_weights(cfg, seed=61)
    W = O.as_f64(sd)
    path = _save_checkpoint(tmp_path, cfg, sd)
    model = AutoModelForCausalLM.from_pretrained(path).to(device, torch.float32)
    prompts = torch.tensor([tokens(9, cfg["vocab"], 62), tokens(9, cfg["vocab"], 63)])
    out = model.generate(prompts, max_new_tokens=10)
    assert out.shape == (2, 19) and bool((out[:, :9] == prompts).all())
    for row in out.tolist():
        _greedy_is_consistent(cfg, W, row, 9)
    # more requests than slots, a pool that cannot hold them all at once, prompts longer than the per-step budget
    eng = model.engine
    cb = ContinuousBatcher(eng, max_num_seqs=2, max_seq_len=128, max_prefill_tokens=24, max_live_tokens=192)
    reqs = [cb.submit(SeqRequest(str(i), tokens(n, cfg["vocab"], 70 + i), max_new_tokens=m))
            for i, (n, m) in enumerate([(70, 6), (3, 12), (30, 4), (1, 9), (50, 5)])]
    cb.run_until_done(500)
    assert all(r.finished and len(r.output_ids) == r.max_new_tokens for r in reqs)
    assert cb.mixed_steps > 0 and not cb.pool.len_of and len(cb.pool.free_pages) == cb.pool.num_pages
    for r in reqs:
        _greedy_is_consistent(cfg, W, r.input_ids + r.output_ids, len(r.input_ids))


def test_trace_runner_replays_steps(tmp_path):
    import subprocess
    import sys
    import numpy as np
    cfg = full_model()
    sd = O.random_weights(cfg, seed=81)
    path = _save_checkpoint(tmp_path, cfg, sd)
    toks = tokens(20, cfg["vocab"], 82)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[13:15], "want": []}, {"id": "y", "tokens": toks[:3], "want": [2]}],
              "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": toks[15:], "want": [4]}], "end": ["x"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", out,
                        "--max-tokens", "128", "--device", "cpu"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = O.forward(cfg, O.as_f64(sd), toks)
    got0 = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4")).view(2, -1).double()
    close(got0, want[[0, 12]])
    got1 = torch.from_numpy(np.fromfile(os.path.join(out, "1.f32"), dtype="<f4")).view(1, -1).double()
    close(got1, want[[2]])
    got2 = torch.from_numpy(np.fromfile(os.path.join(out, "2.f32"), dtype="<f4")).view(1, -1).double()
    close(got2, want[[19]])


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,e,window,keep", [(4, 2, 64, 128, 100, 5), (2, 2, 48, 96, 70, 0), (4, 1, 48, 96, 70, 3), (3, 1, 16, 32, 0, 0),
                                                 (2, 1, 128, 64, 300, 70), (2, 2, 40, 16, 64, 64)])
def test_matrix_core_attention_against_the_plain_statement(H, G, d, e, window, keep):
    """bfloat16 prompt portions take the MFMA kernel, single tokens the row-wise one: both against float64 attention
    over the same (bfloat16-rounded) queries, keys and values, in portions that cut pages and windows."""
    g = torch.Generator().manual_seed(91)
    T = 333
    bf = lambda x: x.to(torch.bfloat16).to(O.F64)                                   # noqa: E731
    q = bf(torch.randn(T, H, 2, d, generator=g, dtype=O.F64))
    k = bf(torch.randn(T, G, 2, d, generator=g, dtype=O.F64))
    v = bf(torch.randn(T, G, e, generator=g, dtype=O.F64))
    scale, lam = d ** -0.5 * 2.0, 0.6
    want = torch.zeros(T, H, e, dtype=O.F64)
    for i in range(T):
        js = [x for x in range(T) if O.sees(i, x, window or None, keep)]
        for hh in range(H):
            kk = hh // (H // G)
            want[i, hh] = O.softmax_attend(q[i, hh, 0], k[js, kk, 0], v[js, kk], scale) - \
                lam * O.softmax_attend(q[i, hh, 1], k[js, kk, 1], v[js, kk], scale)
    device = "cuda"
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("kv", G, 2 * d, e)]}, 64 * 8, 2, torch.bfloat16, device)
    pool.free_pages = [3, 0, 7, 5, 1, 6, 2, 4]
    slot = pool.admit()
    got, at = [], 0
    for n in (70, 9, 1, 130, 64, 8, 1, 50):
        meta = _meta_for(pool, slot, n, device)
        for i in range(n):
            pos = at + i
            pg = pool.pages_of[slot][pos // 64]
            pool.k[0][pg, :, pos % 64] = k[pos].reshape(G, 2 * d).to(device, torch.bfloat16)
            pool.v[0][pg, :, pos % 64] = v[pos].to(device, torch.bfloat16)
        qq = q[at:at + n].reshape(n, H * 2 * d).float().to(device).contiguous()
        got.append(ops.paged_attn(qq, pool.k[0], pool.v[0], meta, maps=2, H=H, G=G, d=d, vd=e, window=window,
                                  keep_first=keep, scale=scale, lam=lam, out_scale=1.0, out_norm=False, eps=1e-6))
        pool.commit(slot, n)
        at += n
    assert at == T
    got = torch.cat(got).double().cpu().view(T, H, e)
    # the output is rounded to bfloat16 (2^-9 relative); the 32-bit softmax weights add nothing visible to that
    assert float((got - want).abs().max()) < 0.02 * float(want.abs().max()), float((got - want).abs().max())


@pytest.mark.gpu
@pytest.mark.skip(reason="recording of decode steps is off by default (BIGDL_RAGGED_GRAPH=1): this test passed on the GPU, "
                         "but a long trace replayed with recording on left the GPU in a fault whose cause is not "
                         "established; the path stays off the GPU until it is")
def test_recorded_decode_steps_replay_like_eager_ones():
    """Steps with one token per sequence are recorded into a hipGraph on their second occurrence and replayed from
    then on.  Every replay is checked against the plain statement, with eager steps (prompt portions, another batch
    size) between the replays, and against an engine that never records."""
    cfg = full_model()
    sd = O.random_weights(cfg, seed=101)
    W = O.as_f64(sd)
    prompts = {k: tokens(n, cfg["vocab"], 110 + i) for i, (k, n) in enumerate({"a": 91, "b": 40, "c": 76}.items())}
    want = {k: O.forward(cfg, W, p) for k, p in prompts.items()}
    schedule = [[("a", 60), ("b", 3)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1)], [("c", 20)],
                [("a", 1), ("b", 1)], [("a", 1), ("b", 1), ("c", 1)], [("a", 1), ("b", 1), ("c", 1)], [("c", 30)],
                [("a", 1), ("b", 1), ("c", 1)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1)], [("a", 5), ("b", 1), ("c", 1)]]
    schedule += [[("a", 1), ("b", 1)] for _ in range(17)] + [[("c", 1)] for _ in range(22)] + [[("b", 10)]]
    eng = engine_for(cfg, sd, torch.float32, "cuda")
    eng.use_graph = True
    got = run_schedule(eng, prompts, schedule, 512, slots=3)
    assert eng.graph_replays >= 30
    plain = engine_for(cfg, sd, torch.float32, "cuda")
    plain.use_graph = False
    ref = run_schedule(plain, prompts, schedule, 512, slots=3)
    for k in prompts:
        close(got[k], want[k])
        close(got[k], ref[k], 1e-4)
