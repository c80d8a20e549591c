"""Filanex on the ragged engine: reader of its ``config.json`` and the map from checkpoint tensor names to
``LayerTensors``.

The design: a pre-norm decoder with parallel blocks -- u = norm(x) (RMS norm with a weight), x <- x + mixer(u) + ff(u),
one norm per layer -- whose embedding adds a row of a hashed token-pair table (the hash of the previous and the current
token; a sequence's first token takes the table's last row), and whose layer list may contain a run of layers that is
executed ``times`` times with the same weights and a cache per pass; in front of every pass the stream is mixed with the
embedding output, x <- W [x ; e] (tensor ``loop.in``).

Mixer: attention with grouped key/value heads, no biases, rotation of neighbouring channel pairs (2 i, 2 i + 1) over the
first ``rot.dims`` channels of a head with frequencies stretched pair by pair for long contexts (``rot.scaling``) and
cosine / sine multiplied by 0.1 ln(factor) + 1, scores scaled and passed through cap * tanh(. / cap), a mask of blocks
(a query sees the keys of its own block of ``mask.size`` positions, counted from the sequence's start, up to itself),
ordinary softmax, and a sigmoid gate per output channel from a projection of the mixer's input in front of the output
projection.

Feed-forward: dense W_down gelu(W_up u + b) + b with the erf form of gelu, or a mixture of gated experts
W_down (silu(W_gate u) * W_up u) chosen by sigmoid scores of a 32-bit router: groups of neighbouring experts are worth
the sum of their two best scores, the ``top`` best experts inside the ``keep`` best groups are used with their scores
divided by the scores' sum; or none.
"""
from __future__ import annotations

import json
import math
import os

import torch

from .ragged_engine import (DenseMlp, LayerTensors, PairEmbedding, RaggedConfig, RaggedDecoder, RoutedExperts,
                            WindowAttention, rotary_inv_freq, yarn_inv_freq)

ARCHITECTURE = "Filanex"
GROUP_TOP = 2              # fixed by the design: a group of experts is worth its two best scores
DENSE_ACT = "gelu_erf"


def is_filanex(config: dict) -> bool:
    return config.get("architecture") == ARCHITECTURE


def layer_runs(config: dict):
    """(layer index of every execution in order, executions in front of which the embedding output is mixed in)"""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n)), ()
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop.get("times", 1))
    if not 0 <= start <= stop <= n or times < 0:
        raise ValueError(f"loop {loop!r} does not fit {n} layers")
    runs, mix = list(range(start)), []
    for _ in range(times):
        if stop > start:
            mix.append(len(runs))
        runs += range(start, stop)
    return runs + list(range(stop, n)), tuple(mix)


def _frequencies(rot: dict):
    """(float32 frequencies of the rotated pairs, amplitude of cosine and sine) from a mixer's ``rot`` entry"""
    dims, base = int(rot["dims"]), float(rot.get("base", 10000.0))
    sc = rot.get("scaling")
    if not sc:
        return rotary_inv_freq(dims, base, 1.0), 1.0
    return yarn_inv_freq(dims, base, float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"]))


def read_config(config: dict) -> RaggedConfig:
    mixers, mlps = [], []
    for layer in config["layers"]:
        m, kind = layer["mixer"], layer["type"]
        if kind != "attention":
            raise ValueError(f"unknown layer type {kind!r}")
        rot = m.get("rot") or {}
        dims = int(rot.get("dims") or 0)
        freqs, amp = _frequencies(rot) if dims else (None, 1.0)
        mixers.append(WindowAttention(
            heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
            rot_dims=dims, rot_base=float(rot.get("base", 10000.0)), rot_neighbours=True,
            rot_freqs=None if freqs is None else tuple(freqs.tolist()), rot_amp=amp, chunk=int((m.get("mask") or {}).get("size") or 0),
            softcap=float(m.get("softcap") or 0.0), gate=True, gate_channels=True))
        f = layer.get("mlp")
        if f is None:
            mlps.append(None)
        elif f.get("kind") == "dense":
            mlps.append(DenseMlp(ff=int(f["ff"]), act=DENSE_ACT, bias=True))
        elif f.get("kind") == "moe":
            r = f["router"]
            g = r.get("groups") or {}
            count = int(g.get("count", 1))
            mlps.append(RoutedExperts(experts=int(r["experts"]), top=int(r["top"]), ff=int(f["expert"]["ff"]), groups=count,
                                      keep=int(g.get("keep", count)), scale=1.0, score="sigmoid", group_top=GROUP_TOP,
                                      renorm=True, act="swiglu"))
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    runs, mix = layer_runs(config)
    table = (config.get("embedding") or {}).get("bigram")
    pairs = None if not table else PairEmbedding(buckets=int(table["buckets"]), mul_prev=int(table["mul_prev"]),
                                                 mul_cur=int(table["mul_cur"]))
    return RaggedConfig(vocab=int(config["vocab"]), width=int(config["width"]), mixers=mixers, mlps=mlps,
                        norm_eps=float((config.get("norm") or {}).get("eps", 1e-6)), name=ARCHITECTURE, block="parallel",
                        runs=runs, mix_in=mix, pair_embed=pairs)


def build_engine(cfg: RaggedConfig, sd: dict, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """``sd``: checkpoint tensors by name ('l<i>.mix.q', 'l<i>.mlp.e<j>.gate', ...).  Projection and expert weights take
    the activation type; norm weights and router rows become float32 (what reads them computes in 32 bits)."""
    dev = torch.device(device)

    def act(*names):
        return torch.cat([sd[n] for n in names], 0).to(dev, dtype).contiguous()

    def f32(name):
        return sd[name].float().reshape(-1).to(dev).contiguous()

    layers = []
    for li, (m, mlp) in enumerate(zip(cfg.mixers, cfg.mlps)):
        p, q = f"l{li}.mix.", f"l{li}.mlp."
        proj = [p + "q", p + "k", p + "v", p + "g"]
        if isinstance(mlp, DenseMlp):
            # the up projection rides behind the mixer's projections: one product reads the normed stream
            lt = LayerTensors(w_in=act(*proj, q + "up"), w_out=act(p + "o"), norm1=f32(f"l{li}.norm1"))
            rows = lt.w_in.shape[0] - mlp.ff
            lt.b_in = torch.cat([torch.zeros(rows, dtype=dtype, device=dev), sd[q + "up.b"].to(dev, dtype)]).contiguous()
            lt.w_down, lt.b_down = act(q + "down"), sd[q + "down.b"].to(dev, dtype).contiguous()
        else:
            lt = LayerTensors(w_in=act(*proj), w_out=act(p + "o"), norm1=f32(f"l{li}.norm1"))
        if isinstance(mlp, RoutedExperts):
            lt.w_router = sd[q + "router"].float().to(dev).contiguous()
            # gate and up rows of an inner channel next to each other: the product's epilogue (and a wavefront of the
            # row-wise kernel) holds both and writes silu(gate) * up
            lt.w_up = torch.stack([torch.stack([sd[q + f"e{e}.gate"], sd[q + f"e{e}.up"]], 1).reshape(2 * mlp.ff, -1)
                                   for e in range(mlp.experts)]).to(dev, dtype).contiguous()
            lt.w_dn = torch.stack([sd[q + f"e{e}.down"] for e in range(mlp.experts)]).to(dev, dtype).contiguous()
        if m.rot_dims:
            lt.inv_freq = (rotary_inv_freq(m.rot_dims, m.rot_base, 1.0) if m.rot_freqs is None else
                           torch.tensor(m.rot_freqs, dtype=torch.float32)).to(dev)
        layers.append(lt)
    return RaggedDecoder(cfg, sd["embed"].to(dev, dtype).contiguous(), layers, f32("final.norm"),
                         sd["head"].to(dev, dtype).contiguous(), act_dtype=dtype, device=dev,
                         pair_table=sd["bigram"].to(dev, dtype).contiguous() if cfg.pair_embed is not None else None,
                         w_mix=sd["loop.in"].to(dev, dtype).contiguous() if cfg.mix_in else None)


def load(path: str, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """Engine for the checkpoint directory ``path`` (config.json + model.safetensors)."""
    from .arch import load_checkpoint_tensors
    with open(os.path.join(path, "config.json")) as f:
        config = json.load(f)
    if not is_filanex(config):
        raise ValueError(f"{path}: not a {ARCHITECTURE} checkpoint")
    return build_engine(read_config(config), load_checkpoint_tensors(path), dtype, device)


def example_config(width=2048, layers=8, heads=16, kv_heads=4, dim=128, vdim=128, ff=5632, expert_ff=1024, experts=32, top=4,
                   groups=4, keep=2, vocab=32000, block=1024, rot_dims=64, loop=(2, 6, 2), softcap=30.0, buckets=65521) -> dict:
    """A config.json of this design at the proportions of a real model: dense and expert feed-forwards alternate, the
    layers ``loop[0] .. loop[1] - 1`` run ``loop[2]`` times.  For benchmarks and smoke tests (random weights)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": softcap,
             "mask": {"size": block},
             "rot": {"dims": rot_dims, "base": 10000.0,
                     "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    moe = {"kind": "moe", "expert": {"ff": expert_ff},
           "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    out = [{"type": "attention", "mixer": dict(mixer), "mlp": moe if i % 2 else {"kind": "dense", "ff": ff}}
           for i in range(layers)]
    cfg = {"architecture": ARCHITECTURE, "embedding": {"bigram": {"buckets": buckets, "mul_prev": 1000003, "mul_cur": 31}},
           "layers": out, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


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
    table = (config.get("embedding") or {}).get("bigram")
    if table:
        sd["bigram"] = mat(table["buckets"] + 1, D, 0.5 * math.sqrt(D))
    if config.get("loop"):
        sd["loop.in"] = mat(D, 2 * D, 1.4)
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.mix.", layer["mixer"]
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        sd[f"l{li}.norm1"] = vec(D, 1.0)
        sd[p + "q"], sd[p + "k"], sd[p + "v"], sd[p + "g"] = mat(H * d, D, 2.0), mat(G * d, D, 2.0), mat(G * e, D), mat(H * e, D)
        sd[p + "o"] = mat(D, H * e)
        f = layer.get("mlp")
        q = f"l{li}.mlp."
        if f is None:
            continue
        if f["kind"] == "dense":
            sd[q + "up"], sd[q + "up.b"], sd[q + "down"], sd[q + "down.b"] = mat(f["ff"], D), vec(f["ff"]), mat(D, f["ff"]), vec(D)
        else:
            sd[q + "router"] = mat(f["router"]["experts"], D, 2.0)
            for x in range(f["router"]["experts"]):
                n = f["expert"]["ff"]
                sd[q + f"e{x}.gate"], sd[q + f"e{x}.up"], sd[q + f"e{x}.down"] = mat(n, D), mat(n, D), mat(D, n)
    return sd


def build_random(config: dict, dtype=torch.bfloat16, device="cuda", seed: int = 0) -> RaggedDecoder:
    return build_engine(read_config(config), random_state_dict(config, device, seed), dtype, device)
