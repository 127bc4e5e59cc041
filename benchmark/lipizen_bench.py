"""Prompt and decode throughput of the Lipizen design on the ragged engine at sizes that resemble a real model's layers
(random weights), beside the closest model of the native engine at equal size: a llama-shaped decoder with the same
width, depth, feed-forward size and vocabulary in plain 16-bit weights (``NativeDecoder`` with dense fp16 linears,
flash prompt attention, captured decode step).

    python bench.py --bench lipizen [--steps K] [--warmup W] [--in-len S]

Prints one JSON line: tokens/s of a prompt of S tokens in one step and of single-token steps behind it (batch 1 and
batch 8), for both engines and every size.
"""
import json
import os
import time

import torch

SIZES = {
    "1b": dict(width=2048, layers=16, heads=16, kv_heads=4, dim=64, vdim=128, ff=5632, vocab=32000, window=1024,
               rec_heads=16, rec_dim=128),
    "3b": dict(width=3072, layers=24, heads=24, kv_heads=8, dim=64, vdim=128, ff=8192, vocab=32000, window=2048,
               rec_heads=24, rec_dim=128),
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


def lipizen_numbers(size, in_len, warmup, steps, device):
    from bigdl_amd.models import lipizen
    cfg = lipizen.example_config(**SIZES[size])
    eng = lipizen.build_random(cfg, torch.bfloat16, device, seed=1)
    g = torch.Generator().manual_seed(0)
    out = {"weights_gb": round(eng.weight_bytes() / 2 ** 30, 2)}
    for batch in (1, 8):
        prompts = [torch.randint(3, cfg["vocab"], (in_len,), generator=g).tolist() for _ in range(batch)]
        eng.pool = None
        pool = eng.ensure_pool(batch * (in_len + 256), batch)
        slots = [pool.admit() for _ in range(batch)]

        def prefill():
            for s in slots:
                pool.len_of[s] = 0                                   # the same pages again
            eng.step([(s, p) for s, p in zip(slots, prompts)])
        if batch == 1:
            out["prefill_tokens_per_s"] = round(in_len / _time(prefill, warmup, steps), 1)
        else:
            prefill()
        n = 0

        def decode():
            nonlocal n
            n += 1
            eng.step([(s, [7 + n % 50]) for s in slots])
        out[f"decode_tokens_per_s_batch{batch}"] = round(batch / _time(decode, 3, 32), 1)
    return out


def llama_numbers(size, in_len, warmup, steps, device):
    from bigdl_amd import qtypes as Q
    from bigdl_amd.models.decoder import DecoderConfig, build_random_decoder
    s = SIZES[size]
    cfg = DecoderConfig(vocab_size=s["vocab"], hidden_size=s["width"], intermediate_size=s["ff"], num_layers=s["layers"],
                        num_heads=s["width"] // 128, num_kv_heads=s["kv_heads"], head_dim=128, max_position=8192)
    out = {}
    for batch in (1, 8):
        model = build_random_decoder(cfg, Q.FP16, device=str(device), seed=1)
        prompt = torch.randint(3, s["vocab"], (batch, in_len)).to(device)
        model.generate(prompt, max_new_tokens=4)
        firsts, rests = [], []
        for _ in range(max(1, steps)):
            model.generate(prompt, max_new_tokens=33, min_new_tokens=33)
            firsts.append(model.first_cost)
            rests.append(model.rest_cost_mean)
        if batch == 1:
            out["weights_gb"] = round(model.weight_bytes() / 2 ** 30, 2)
            out["prefill_tokens_per_s"] = round(in_len / (sum(firsts) / len(firsts)), 1)
        out[f"decode_tokens_per_s_batch{batch}"] = round(batch / (sum(rests) / len(rests)), 1)
        del model
        torch.cuda.empty_cache()
    return out


def main(args):
    device = torch.device("cuda", 0)
    in_len = args.in_len if args.in_len != 1024 else 2048
    res = {}
    for size in (os.environ.get("BIGDL_LIPIZEN_SIZES") or ",".join(SIZES)).split(","):
        res[size] = {"lipizen": lipizen_numbers(size, in_len, args.warmup, args.steps, device),
                     "llama_fp16": llama_numbers(size, in_len, args.warmup, args.steps, device)}
    print(json.dumps({"bench": "lipizen", "prompt_tokens": in_len, "dtype": "bf16 (llama: fp16)", "data": "synthetic",
                      "sizes": {k: dict(v) for k, v in SIZES.items()}, "results": res}), flush=True)
