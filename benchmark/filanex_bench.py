"""Prompt and decode throughput of the Filanex design on the ragged engine at sizes that resemble a real model's layers
(random weights), beside the closest model of the framework at equal size: Merusun on the same engine, restricted to its
windowed attention layers, with as many layers as Filanex has layer executions (a looped layer counts every time), the
same width, vocabulary, head layout and window (= Filanex's block size), the same routed experts, and a shared expert
sized so that a token's multiply-adds in the feed-forwards are equal on average.

    python bench.py --bench filanex [--steps K] [--warmup W] [--in-len S]

Prints one JSON line: tokens/s of a prompt of S tokens in one step and of single-token steps behind it (batch 1 and
batch 8), for both designs and every size.  BIGDL_FILANEX_SIZES=a,b picks sizes, BIGDL_FILANEX_ONLY=prefill|decode and
BIGDL_FILANEX_DESIGNS=filanex,merusun narrow a run down for a profiler.
"""
import json
import os

import torch

from merusun_bench import engine_numbers

SIZES = {
    "a": dict(width=2048, layers=8, loop=(2, 6, 2), heads=16, kv_heads=4, dim=128, vdim=128, ff=5632, expert_ff=1024, experts=32,
              top=4, groups=4, keep=2, vocab=32000, block=1024, rot_dims=64),
    "b": dict(width=3072, layers=12, loop=(4, 10, 2), heads=24, kv_heads=8, dim=128, vdim=128, ff=8192, expert_ff=1408, experts=64,
              top=6, groups=8, keep=4, vocab=32000, block=2048, rot_dims=64),
}


def executions(s):
    a, b, times = s["loop"]
    return s["layers"] + (b - a) * (times - 1)


def filanex_engine(size, device):
    from bigdl_amd.models import filanex
    return filanex.build_random(filanex.example_config(**SIZES[size]), torch.bfloat16, device, seed=1)


def merusun_engine(size, device):
    from bigdl_amd.models import merusun
    s = SIZES[size]
    # multiply-adds per token and width: dense 2 ff, gated experts 3 top ff_e (every other layer each); Merusun's
    # two-matrix experts 2 (top ff_e + shared)
    mean = (2 * s["ff"] + 3 * s["top"] * s["expert_ff"]) / 2
    shared = max(128, int((mean / 2 - s["top"] * s["expert_ff"]) // 128 * 128))
    moe = {"kind": "moe", "expert": {"ff": s["expert_ff"]}, "shared": {"ff": shared},
           "router": {"experts": s["experts"], "top": s["top"], "scale": 2.0, "groups": {"count": s["groups"], "keep": s["keep"]}}}
    mixer = {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["vdim"], "scale": 8.0 * s["dim"] ** -0.5,
             "mask": {"size": s["block"]}}
    cfg = {"architecture": merusun.ARCHITECTURE, "embedding": {"scale": s["width"] ** 0.5}, "norm": {"eps": 1e-6},
           "layers": [{"type": "attention", "mixer": dict(mixer), "mlp": moe} for _ in range(executions(s))],
           "vocab": s["vocab"], "width": s["width"]}
    return merusun.build_random(cfg, torch.bfloat16, device, seed=1)


def main(args):
    device = torch.device("cuda", 0)
    in_len = args.in_len if args.in_len != 1024 else 2048
    only = os.environ.get("BIGDL_FILANEX_ONLY", "")
    designs = (os.environ.get("BIGDL_FILANEX_DESIGNS") or "filanex,merusun").split(",")
    res = {}
    for size in (os.environ.get("BIGDL_FILANEX_SIZES") or ",".join(SIZES)).split(","):
        res[size] = {}
        for name, make in (("filanex", filanex_engine), ("merusun", merusun_engine)):
            if name in designs:
                eng = make(size, device)
                res[size][name] = engine_numbers(eng, SIZES[size]["vocab"], in_len, args.warmup, args.steps, only)
                res[size][name]["layer_executions"] = len(eng.runs)
                del eng
                torch.cuda.empty_cache()
    print(json.dumps({"bench": "filanex", "prompt_tokens": in_len, "dtype": "bf16", "data": "synthetic",
                      "sizes": {k: dict(v) for k, v in SIZES.items()}, "results": res}), flush=True)
