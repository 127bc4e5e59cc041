"""Prompt and decode throughput of the Merusun design on the ragged engine at sizes that resemble a real model's layers
(random weights), beside the closest model of the framework at equal size: Lipizen on the same engine with the same
width, depth, vocabulary, window and head layout, and a dense feed-forward with as many multiply-adds per token as the
experts that a Merusun token uses.

    python bench.py --bench merusun [--steps K] [--warmup W] [--in-len S]

Prints one JSON line: tokens/s of a prompt of S tokens in one step and of single-token steps behind it (batch 1 and
batch 8), for both designs and every size.  BIGDL_MERUSUN_SIZES=a,b picks sizes, BIGDL_MERUSUN_ONLY=prefill|decode and
BIGDL_MERUSUN_DESIGNS=merusun,lipizen narrow a run down for a profiler.
"""
import json
import os
import time

import torch

SIZES = {
    "a": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, ff=1024, experts=32, top=4, groups=4, keep=2,
              shared_ff=2048, vocab=32000, window=1024, rank=512, rot_dim=64, latent_dim=128, rec_heads=8, rec_dim=128,
              rec_vdim=256),
    "b": dict(width=3072, layers=12, heads=24, kv_heads=8, dim=128, ff=1408, experts=64, top=6, groups=8, keep=4,
              shared_ff=2816, vocab=32000, window=2048, rank=512, rot_dim=64, latent_dim=128, rec_heads=12, rec_dim=128,
              rec_vdim=256),
}


def _time(fn, warmup, steps):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def engine_numbers(eng, vocab, in_len, warmup, steps, only):
    g = torch.Generator().manual_seed(0)
    out = {"weights_gb": round(eng.weight_bytes() / 2 ** 30, 2)}
    for batch in (1, 8):
        prompts = [torch.randint(3, vocab, (in_len,), generator=g).tolist() for _ in range(batch)]
        eng.pool = None
        pool = eng.ensure_pool(batch * (in_len + 256), batch)
        slots = [pool.admit() for _ in range(batch)]

        def prefill():
            for s in slots:
                pool.len_of[s] = 0                                   # the same pages again
            eng.step([(s, p) for s, p in zip(slots, prompts)])
        if batch == 1 and only != "decode":
            out["prefill_tokens_per_s"] = round(in_len / _time(prefill, warmup, steps), 1)
        else:
            prefill()
        if only == "prefill":
            break
        n = 0

        def decode():
            nonlocal n
            n += 1
            eng.step([(s, [7 + n % 50]) for s in slots])
        out[f"decode_tokens_per_s_batch{batch}"] = round(batch / _time(decode, 3, 32), 1)
    return out


def merusun_engine(size, device):
    from bigdl_amd.models import merusun
    return merusun.build_random(merusun.example_config(**SIZES[size]), torch.bfloat16, device, seed=1)


def lipizen_engine(size, device):
    from bigdl_amd.models import lipizen
    s = SIZES[size]
    ff = (2 * (s["top"] * s["ff"] + s["shared_ff"]) // 3 + 127) // 128 * 128          # three matrices instead of two
    cfg = lipizen.example_config(width=s["width"], layers=s["layers"], heads=s["heads"], kv_heads=s["kv_heads"], dim=64, vdim=128,
                                 ff=ff, vocab=s["vocab"], window=s["window"], rec_heads=s["width"] // 128, rec_dim=128)
    return lipizen.build_random(cfg, torch.bfloat16, device, seed=1)


def main(args):
    device = torch.device("cuda", 0)
    in_len = args.in_len if args.in_len != 1024 else 2048
    only = os.environ.get("BIGDL_MERUSUN_ONLY", "")
    designs = (os.environ.get("BIGDL_MERUSUN_DESIGNS") or "merusun,lipizen").split(",")
    res = {}
    for size in (os.environ.get("BIGDL_MERUSUN_SIZES") or ",".join(SIZES)).split(","):
        res[size] = {}
        for name, make in (("merusun", merusun_engine), ("lipizen", lipizen_engine)):
            if name in designs:
                eng = make(size, device)
                res[size][name] = engine_numbers(eng, SIZES[size]["vocab"], in_len, args.warmup, args.steps, only)
                del eng
                torch.cuda.empty_cache()
    print(json.dumps({"bench": "merusun", "prompt_tokens": in_len, "dtype": "bf16", "data": "synthetic",
                      "sizes": {k: dict(v) for k, v in SIZES.items()}, "results": res}), flush=True)
