"""Prompt and decode throughput of the Dimelix design on the ragged engine at sizes that resemble a real model's layers
(random weights), beside the closest model of the framework at equal size: Merusun on the same engine (sink attention,
latent attention over a compressed cache and a matrix-memory recurrence are its mixers too), with as many layers as
Dimelix has layer executions (a looped layer counts every time), the same width, vocabulary, head layout, window and
latent rank, and routed experts plus a shared expert sized so that a token's multiply-adds in the feed-forwards are equal.

    python bench.py --bench dimelix [--steps K] [--warmup W] [--in-len S]

Prints one JSON line: tokens/s of a prompt of S tokens in one step and of single-token steps behind it (batch 1 and
batch 8), for both designs and every size.  BIGDL_DIMELIX_SIZES=a,b picks sizes, BIGDL_DIMELIX_ONLY=prefill|decode and
BIGDL_DIMELIX_DESIGNS=dimelix,merusun narrow a run down for a profiler.
"""
import json
import os

import torch

from merusun_bench import engine_numbers

SIZES = {
    "a": dict(width=2048, layers=6, loop=(1, 3, 2), heads=16, kv_heads=4, dim=128, ff=5632, vocab=32000, window=1024, rank=512,
              latent_dim=128, delta_heads=16, delta_dim=64, rot_dims=64, streams=2),
    "b": dict(width=3072, layers=9, loop=(3, 6, 2), heads=24, kv_heads=8, dim=128, ff=8192, vocab=32000, window=2048, rank=512,
              latent_dim=128, delta_heads=24, delta_dim=64, rot_dims=64, streams=4),
}
EXPERTS = dict(a=dict(experts=32, top=4, ff=1024, groups=4, keep=2), b=dict(experts=64, top=6, ff=1024, groups=8, keep=4))


def executions(s):
    a, b, times = s["loop"]
    return s["layers"] + (b - a) * (times - 1)


def dimelix_engine(size, device):
    from bigdl_amd.models import dimelix
    return dimelix.build_random(dimelix.example_config(**SIZES[size]), torch.bfloat16, device, seed=1)


def merusun_engine(size, device):
    from bigdl_amd.models import merusun
    s, e = SIZES[size], EXPERTS[size]
    # multiply-adds per token and width: Dimelix's dense feed-forward 2 ff; Merusun's two-matrix experts 2 (top ff_e + shared)
    shared = max(128, (s["ff"] - e["top"] * e["ff"]) // 128 * 128)
    cfg = merusun.example_config(width=s["width"], layers=executions(s), heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"],
                                 ff=e["ff"], experts=e["experts"], top=e["top"], groups=e["groups"], keep=e["keep"], shared_ff=shared,
                                 vocab=s["vocab"], window=s["window"], rank=s["rank"], rot_dim=64, latent_dim=s["latent_dim"],
                                 rec_heads=s["delta_heads"] // 2, rec_dim=128, rec_vdim=128)
    return merusun.build_random(cfg, torch.bfloat16, device, seed=1)


def main(args):
    device = torch.device("cuda", 0)
    in_len = args.in_len if args.in_len != 1024 else 2048
    only = os.environ.get("BIGDL_DIMELIX_ONLY", "")
    designs = (os.environ.get("BIGDL_DIMELIX_DESIGNS") or "dimelix,merusun").split(",")
    res = {}
    for size in (os.environ.get("BIGDL_DIMELIX_SIZES") or ",".join(SIZES)).split(","):
        res[size] = {}
        for name, make in (("dimelix", dimelix_engine), ("merusun", merusun_engine)):
            if name in designs:
                eng = make(size, device)
                res[size][name] = engine_numbers(eng, SIZES[size]["vocab"], in_len, args.warmup, args.steps, only)
                res[size][name]["layer_executions"] = len(eng.runs)
                del eng
                torch.cuda.empty_cache()
    print(json.dumps({"bench": "dimelix", "prompt_tokens": in_len, "dtype": "bf16", "data": "synthetic",
                      "sizes": {k: dict(v) for k, v in SIZES.items()}, "results": res}), flush=True)
