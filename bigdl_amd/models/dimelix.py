"""Dimelix on the ragged engine: reader of its ``config.json`` and the map from checkpoint tensor names to
``LayerTensors``.

The design: a pre-norm decoder, x <- x + mixer(N1(x)), x <- x + ff(N2(x)) with RMS norms whose weights are stored as
offsets from one (w = 1 + g), over a stream that is kept in ``streams`` copies: sublayer q of a layer reads
u = sum_s in_q[s] X[s] and writes X[t] <- sum_s mix_q[s, t] X[s] + out_q[t] f(N(u)); all copies start as the embedding
output (table row times ``embedding.scale``) and the model's output is their sum, normed, multiplied with the embedding
table itself and soft-capped.  The layer list may contain a run of layers that is executed ``times`` times with the same
weights and a cache per pass.

Mixers (``type`` of a layer):

* ``attention``: grouped key/value heads, queries and keys RMS-normed per head with a weight, neighbouring channel pairs
  (2 i, 2 i + 1) of the first ``rot.dims`` channels turned by position * base^(-2 i / dims), full causal softmax whose
  normaliser also holds exp(sink) of a learned number per head, a sigmoid gate per output channel from a projection of
  the mixer's input, output projection;
* ``latent_attention``: one RMS-normed row of ``kv_rank`` channels per token is cached; keys and values of all heads are
  products of that row; no positions; ordinary causal softmax; the same gate;
* ``parallel``: two mixers side by side whose outputs are summed with the weights ``left_scale`` / ``right_scale``.  Left:
  attention over a sliding window of ``mask.size`` positions with normed queries and keys, no rotation, scores lowered by
  slope_h * (i - j) with slope_h = 2^(-8 (h + 1) / heads), and the key projections (as they are before the norm) as
  values.  Right: a generalised delta rule (``DeltaRule``) with per-head output norm, weight and gate.

Feed-forward: W_down act(W_up u) with a two-curvature unit whose curvatures are softplus of two learned numbers per
layer (``DenseMlp(act="xielu")``).
"""
from __future__ import annotations

import json
import math
import os

import torch

from .ragged_engine import (DeltaRule, DenseMlp, LatentAttention, LayerTensors, RaggedConfig, RaggedDecoder, SideBySide,
                            WindowAttention, rotary_inv_freq)

ARCHITECTURE = "Dimelix"
DECAY_RATE = math.exp(-0.5)    # fixed by the design: the decay is exp(-e^(-1/2) sigmoid(.))
UNIT_EPS = 1e-6                # inside the root of the unit key's length
SLOPE_SPAN = 8.0               # head h's distance slope is 2^(-SLOPE_SPAN (h + 1) / heads)


def is_dimelix(config: dict) -> bool:
    return config.get("architecture") == ARCHITECTURE


def layer_runs(config: dict):
    """layer index of every execution, in order"""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop.get("times", 1))
    if not 0 <= start <= stop <= n or times < 0:
        raise ValueError(f"loop {loop!r} does not fit {n} layers")
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def distance_slopes(heads: int) -> tuple:
    return tuple(2.0 ** (-SLOPE_SPAN * (h + 1) / heads) for h in range(heads))


def _sink_attention(m: dict) -> WindowAttention:
    rot = m.get("rot") or {}
    return WindowAttention(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                           scale=float(m["scale"]), qk_norm=True, rot_dims=int(rot.get("dims") or 0),
                           rot_base=float(rot.get("base", 10000.0)), rot_neighbours=True, gate=True, gate_channels=True,
                           head_sinks=True)


def _latent_attention(m: dict) -> LatentAttention:
    return LatentAttention(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=0, vdim=int(m["vdim"]), rank=int(m["kv_rank"]),
                           scale=float(m["scale"]), gate=True)


def _window_branch(m: dict, out_scale: float) -> WindowAttention:
    H, d = int(m["heads"]), int(m["dim"])
    if int(m.get("vdim", d)) != d:
        raise ValueError("values that are the key projections have the keys' size")
    return WindowAttention(heads=H, kv_heads=int(m["kv_heads"]), dim=d, vdim=d, scale=float(m["scale"]), qk_norm=True,
                           window=int((m.get("mask") or {}).get("size") or 0), gate=True, gate_channels=True,
                           dist_slopes=distance_slopes(H), v_from_k=True, out_scale=out_scale)


def read_config(config: dict) -> RaggedConfig:
    """(the rank of the decay's low-rank pair is a tensor's shape, not a config entry: ``build_engine`` fills it in)"""
    mixers, mlps = [], []
    for li, layer in enumerate(config["layers"]):
        m, kind = layer["mixer"], layer["type"]
        if kind == "attention":
            mixers.append(_sink_attention(m))
        elif kind == "latent_attention":
            mixers.append(_latent_attention(m))
        elif kind == "parallel":
            r = m["right"]
            right = DeltaRule(heads=int(r["heads"]), dim=int(r["dim"]), decay_rank=0,
                              decay_rate=DECAY_RATE, unit_eps=UNIT_EPS, out_scale=float(m.get("right_scale", 1.0)))
            mixers.append(SideBySide(_window_branch(m["left"], float(m.get("left_scale", 1.0))), right))
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        f = layer.get("mlp")
        if f is None:
            mlps.append(None)
        elif f.get("kind") == "dense":
            mlps.append(DenseMlp(ff=int(f["ff"]), act="xielu", bias=False))
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    return RaggedConfig(vocab=int(config["vocab"]), width=int(config["width"]), mixers=mixers, mlps=mlps,
                        norm_eps=float((config.get("norm") or {}).get("eps", 1e-6)), name=ARCHITECTURE, block="pre_norm",
                        streams=int(config.get("streams") or 1), runs=layer_runs(config),
                        embed_scale=float((config.get("embedding") or {}).get("scale", 1.0)),
                        logit_softcap=float(config.get("logit_softcap") or 0.0))


def _softplus(z: float) -> float:
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def build_engine(cfg: RaggedConfig, sd: dict, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """``sd``: checkpoint tensors by name ('l<i>.mix.q', 'l<i>.mix.left.k', 'l<i>.hc1.mix', ...).  Projection weights take
    the activation type; norm weights (stored as offsets from one), sinks, biases of the recurrence and the coefficients
    of the stream copies become float32 (what reads them computes in 32 bits)."""
    dev = torch.device(device)
    S = cfg.streams

    def act(*names):
        return torch.cat([sd[n] for n in names], 0).to(dev, dtype).contiguous()

    def f32(name):
        return sd[name].float().reshape(-1).to(dev).contiguous()

    def one_plus(name):
        return (1.0 + sd[name].float()).reshape(-1).to(dev).contiguous()

    def copies(prefix):
        if prefix + "in" not in sd:
            return None
        c = torch.cat([sd[prefix + "in"].float().reshape(-1), sd[prefix + "out"].float().reshape(-1),
                       sd[prefix + "mix"].float().reshape(-1)])                 # mix is [from, to], row-major
        if c.numel() != 2 * S + S * S:
            raise ValueError(f"{prefix}*: coefficients do not fit {S} copies of the stream")
        return c.to(dev).contiguous()

    def attention_tensors(p, m, names):
        lt = LayerTensors(w_in=act(*[p + n for n in names]), w_out=None, norm1=None, q_norm=f32(p + "q.norm"),
                          k_norm=f32(p + "k.norm"))
        if m.rot_dims:
            lt.inv_freq = rotary_inv_freq(m.rot_dims, m.rot_base, 1.0).to(dev)
        if m.head_sinks:
            lt.sinks = f32(p + "sink")
        if m.dist_slopes is not None:
            lt.slopes = torch.tensor(m.dist_slopes, dtype=torch.float64).to(torch.float32).to(dev)
        return lt

    layers = []
    for li, (m, mlp) in enumerate(zip(cfg.mixers, cfg.mlps)):
        p, q = f"l{li}.mix.", f"l{li}.mlp."
        if isinstance(m, WindowAttention):
            lt = attention_tensors(p, m, ("q", "k", "v", "g"))
            lt.w_out = act(p + "o")
        elif isinstance(m, LatentAttention):
            lt = LayerTensors(w_in=act(p + "q", p + "dkv", p + "g"), w_out=act(p + "o"), norm1=None, k_norm=f32(p + "dkv.norm"))
            lt.w_uk = sd[p + "uk"].view(m.heads, m.dim, m.rank).to(dev, dtype).contiguous()
            lt.w_uv = sd[p + "uv"].view(m.heads, m.vdim, m.rank).to(dev, dtype).contiguous()
        else:
            a, b = p + "left.", p + "right."
            left = attention_tensors(a, m.left, ("q", "k", "g"))
            m.right.decay_rank = int(sd[b + "w1"].shape[0])
            right = LayerTensors(w_in=act(*[b + n for n in ("r", "k", "v", "g", "a", "w1")]), w_out=None, norm1=None,
                                 o_norm=f32(b + "norm"), w_decay=act(b + "w2"), decay_bias=f32(b + "w0"), remove_bias=f32(b + "a.b"))
            lt = LayerTensors(w_in=torch.cat([left.w_in, right.w_in], 0).contiguous(), w_out=torch.cat(
                [sd[a + "o"], sd[b + "o"]], 1).to(dev, dtype).contiguous(), norm1=None, left=left, right=right)
        lt.norm1, lt.hc1 = one_plus(f"l{li}.norm1"), copies(f"l{li}.hc1.")
        if isinstance(mlp, DenseMlp):
            lt.norm2, lt.hc2 = one_plus(f"l{li}.norm2"), copies(f"l{li}.hc2.")
            lt.w_ff, lt.w_down = act(q + "up"), act(q + "down")
            pq = sd[q + "act"].float().reshape(-1).tolist()
            lt.act_params = (_softplus(pq[0]), _softplus(pq[1]))
        layers.append(lt)
    embed = sd["embed"].to(dev, dtype).contiguous()
    return RaggedDecoder(cfg, embed, layers, one_plus("final.norm"), embed, act_dtype=dtype, device=dev)


def load(path: str, dtype=torch.bfloat16, device="cuda") -> RaggedDecoder:
    """Engine for the checkpoint directory ``path`` (config.json + model.safetensors)."""
    from .arch import load_checkpoint_tensors
    with open(os.path.join(path, "config.json")) as f:
        config = json.load(f)
    if not is_dimelix(config):
        raise ValueError(f"{path}: not a {ARCHITECTURE} checkpoint")
    return build_engine(read_config(config), load_checkpoint_tensors(path), dtype, device)


def example_config(width=2048, layers=6, heads=16, kv_heads=4, dim=128, ff=5632, vocab=32000, window=1024, rank=512,
                   latent_dim=128, delta_heads=16, delta_dim=64, rot_dims=64, streams=2, loop=(1, 3, 2), softcap=30.0) -> dict:
    """A config.json of this design at the proportions of a real model: the three kinds of layers in turn, the layers
    ``loop[0] .. loop[1] - 1`` run ``loop[2]`` times.  For benchmarks and smoke tests (random weights)."""
    def mlp():
        return {"kind": "dense", "ff": ff}
    side = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5, "mask": {"size": window}},
            "right": {"heads": delta_heads, "dim": delta_dim}, "left_scale": 1.0, "right_scale": 1.0}
    sink = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5,
            "rot": {"dims": rot_dims, "base": 10000.0}}
    latent = {"heads": heads, "dim": latent_dim, "vdim": latent_dim, "kv_rank": rank, "scale": latent_dim ** -0.5}
    kinds = [("parallel", side), ("attention", sink), ("latent_attention", latent)]
    out = [{"type": kinds[i % 3][0], "mixer": json.loads(json.dumps(kinds[i % 3][1])), "mlp": mlp()} for i in range(layers)]
    cfg = {"architecture": ARCHITECTURE, "embedding": {"scale": 1.0}, "layers": out, "norm": {"eps": 1e-5}, "vocab": vocab,
           "width": width, "logit_softcap": softcap}
    if streams:
        cfg["streams"] = streams
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def random_state_dict(config: dict, device="cuda", seed: int = 0, decay_rank: int = 64) -> dict:
    """Random checkpoint tensors (bfloat16, created on ``device``) with the names and shapes the design gives them."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)
    D, S = config["width"], int(config.get("streams") or 0)

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, device=dev, generator=g) * (s / math.sqrt(k))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, device=dev, generator=g)).to(torch.bfloat16)

    sd = {"embed": mat(config["vocab"], D, math.sqrt(D)), "final.norm": vec(D)}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.mix.", layer["mixer"]
        sd[f"l{li}.norm1"] = vec(D)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd.update({p + "q": mat(H * d, D, 2.0), p + "k": mat(G * d, D, 2.0), p + "v": mat(G * e, D), p + "g": mat(H * e, D),
                       p + "o": mat(D, H * e), p + "q.norm": vec(d, 1.0), p + "k.norm": vec(d, 1.0), p + "sink": vec(H, 0.0, 1.0)})
        elif layer["type"] == "latent_attention":
            H, d, e, r = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
            sd.update({p + "q": mat(H * d, D, 2.0), p + "dkv": mat(r, D), p + "dkv.norm": vec(r, 1.0), p + "uk": mat(H * d, r, 2.0),
                       p + "uv": mat(H * e, r), p + "g": mat(H * e, D), p + "o": mat(D, H * e)})
        else:
            a, b = m["left"], m["right"]
            H, G, d = a["heads"], a["kv_heads"], a["dim"]
            sd.update({p + "left.q": mat(H * d, D, 2.0), p + "left.k": mat(G * d, D, 2.0), p + "left.g": mat(H * d, D),
                       p + "left.o": mat(D, H * d), p + "left.q.norm": vec(d, 1.0), p + "left.k.norm": vec(d, 1.0)})
            n = b["heads"] * b["dim"]
            sd.update({p + "right." + k: mat(n, D) for k in ("r", "k", "v", "g", "a")})
            sd.update({p + "right.a.b": vec(n), p + "right.w1": mat(decay_rank, D), p + "right.w2": mat(n, decay_rank),
                       p + "right.w0": vec(n), p + "right.norm": vec(n, 1.0), p + "right.o": mat(D, n)})
        subs = ["1"]
        f = layer.get("mlp")
        if f is not None:
            sd.update({f"l{li}.norm2": vec(D), f"l{li}.mlp.up": mat(f["ff"], D), f"l{li}.mlp.down": mat(D, f["ff"]),
                       f"l{li}.mlp.act": vec(2, 0.0, 1.0)})
            subs.append("2")
        if S:
            for n in subs:
                sd[f"l{li}.hc{n}.in"] = vec(S, 1.0 / S)
                sd[f"l{li}.hc{n}.out"] = vec(S, 1.0)
                sd[f"l{li}.hc{n}.mix"] = (torch.eye(S, device=dev) + 0.1 * torch.randn(S, S, device=dev, generator=g)).to(torch.bfloat16)
    return sd


def build_random(config: dict, dtype=torch.bfloat16, device="cuda", seed: int = 0, decay_rank: int = 64) -> RaggedDecoder:
    return build_engine(read_config(config), random_state_dict(config, device, seed, decay_rank), dtype, device)
