"""Plain, slow float64 statement of the Dimelix design: one function per mechanism, whole sequences, token by token
where there is a recurrence, nothing shared with ``bigdl_amd``.  Weights are a dict of float64 tensors by checkpoint
name; ``config`` is the parsed ``config.json``.

Notation: N(u, w) = u / sqrt(mean(u^2) + eps) * w.  The stream is kept in ``streams`` copies X[s]; a sublayer f with
coefficients (alpha, beta, M) reads u = sum_s alpha[s] X[s] and writes X'[t] = sum_s M[s, t] X[s] + beta[t] f(N(u, 1 + g)).
Without coefficients there is one copy and X' = X + f(N(X, 1 + g)).
"""
import math
import random

import torch

F64 = torch.float64


def rms(u, eps):
    return u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps)


def norm_plain(u, w, eps):
    return rms(u, eps) * w


def norm_one_plus(u, g, eps):
    return rms(u, eps) * (1.0 + g)


# ---------------------------------------------------------------------------------------- stream
def read_streams(X, alpha):
    """X [S, T, D] -> [T, D]"""
    return sum(alpha[s] * X[s] for s in range(X.shape[0]))


def write_streams(X, y, beta, M):
    S = X.shape[0]
    return torch.stack([sum(M[s, t] * X[s] for s in range(S)) + beta[t] * y for t in range(S)])


# ---------------------------------------------------------------------------------------- attention pieces
def turn_pairs(u, pos, dims, base):
    """channels (2 i, 2 i + 1), i < dims / 2, of u [..., n] turned by the angle pos * base^(-2 i / dims)"""
    out = u.clone()
    for i in range(dims // 2):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(ang), math.sin(ang)
        a, b = u[..., 2 * i], u[..., 2 * i + 1]
        out[..., 2 * i], out[..., 2 * i + 1] = a * c - b * s, b * c + a * s
    return out


def softmax_rows(scores, extra=None):
    """weights of the keys of one query; ``extra``: one more score in the denominator that has no value"""
    top = scores.max() if extra is None else max(float(scores.max()), float(extra))
    e = torch.exp(scores - top)
    den = e.sum() + (0.0 if extra is None else math.exp(float(extra) - top))
    return e / den


def attend(q, k, v, scale, window=None, sinks=None, slopes=None):
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e].  Query i sees key j when j <= i and, with a window, i - j <
    window.  ``slopes[h] * (i - j)`` is subtracted from the scores of head h, ``sinks[h]`` joins the denominator."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for i in range(T):
        lo = 0 if not window else max(0, i - window + 1)
        js = list(range(lo, i + 1))
        dist = torch.tensor([i - j for j in js], dtype=F64)
        for h in range(H):
            g = h // (H // G)
            s = (k[js, g] @ q[i, h]) * scale
            if slopes is not None:
                s = s - slopes[h] * dist
            out[i, h] = softmax_rows(s, None if sinks is None else sinks[h]) @ v[js, g]
    return out


def sink_attention_mixer(u, W, p, m, eps):
    """grouped heads, q / k normed per head, leading channels turned pair by pair, a learned sink per head, gate"""
    T = u.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = norm_plain((u @ W[p + "q"].T).view(T, H, d), W[p + "q.norm"], eps)
    k = norm_plain((u @ W[p + "k"].T).view(T, G, d), W[p + "k.norm"], eps)
    v = (u @ W[p + "v"].T).view(T, G, e)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        q = torch.stack([turn_pairs(q[t], t, rot["dims"], rot["base"]) for t in range(T)])
        k = torch.stack([turn_pairs(k[t], t, rot["dims"], rot["base"]) for t in range(T)])
    o = attend(q, k, v, m["scale"], sinks=W[p + "sink"])
    return (o.reshape(T, H * e) * torch.sigmoid(u @ W[p + "g"].T)) @ W[p + "o"].T


def latent_attention_mixer(u, W, p, m, eps):
    """keys and values of all heads are made from one normed low-rank row per token; no positions"""
    T = u.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = (u @ W[p + "q"].T).view(T, H, d)
    c = norm_plain(u @ W[p + "dkv"].T, W[p + "dkv.norm"], eps)
    k = (c @ W[p + "uk"].T).view(T, H, d)
    v = (c @ W[p + "uv"].T).view(T, H, e)
    o = attend(q, k, v, m["scale"])
    return (o.reshape(T, H * e) * torch.sigmoid(u @ W[p + "g"].T)) @ W[p + "o"].T


def distance_slopes(H):
    return [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]


def window_branch(u, W, p, m, eps):
    """sliding window, scores lowered by slope * distance, the values are the key projections before their norm"""
    T = u.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = norm_plain((u @ W[p + "q"].T).view(T, H, d), W[p + "q.norm"], eps)
    kraw = (u @ W[p + "k"].T).view(T, G, d)
    k = norm_plain(kraw, W[p + "k.norm"], eps)
    o = attend(q, k, kraw, m["scale"], window=(m.get("mask") or {}).get("size"), slopes=distance_slopes(H))
    return (o.reshape(T, H * d) * torch.sigmoid(u @ W[p + "g"].T)) @ W[p + "o"].T


DECAY_RATE = math.exp(-0.5)


def delta_gates(u, W, p, H, d):
    """per token and key channel: decay w in (exp(-e^-1/2), 1) and removal rate a in (0, 1)"""
    T = u.shape[0]
    w = torch.exp(-DECAY_RATE * torch.sigmoid(torch.tanh(u @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"]))
    a = torch.sigmoid(u @ W[p + "a"].T + W[p + "a.b"])
    return w.view(T, H, d), a.view(T, H, d)


def delta_rule(r, k, v, w, a, S0=None):
    """one head, token by token: S [d, d] <- diag(w) S - (a * n)(n^T S) + k v^T with n = k / sqrt(|k|^2 + 1e-6), both
    S on the right the old state; output S^T r.  Returns (outputs [T, d], last state)."""
    T, d = r.shape
    S = torch.zeros(d, d, dtype=F64) if S0 is None else S0.clone()
    out = torch.zeros(T, d, dtype=F64)
    for t in range(T):
        n = k[t] / torch.sqrt(k[t].pow(2).sum() + 1e-6)
        S = w[t][:, None] * S - torch.outer(a[t] * n, n @ S) + torch.outer(k[t], v[t])
        out[t] = S.T @ r[t]
    return out, S


def delta_branch(u, W, p, m, eps):
    T = u.shape[0]
    H, d = m["heads"], m["dim"]
    r = (u @ W[p + "r"].T).view(T, H, d)
    k = (u @ W[p + "k"].T).view(T, H, d)
    v = (u @ W[p + "v"].T).view(T, H, d)
    w, a = delta_gates(u, W, p, H, d)
    o = torch.stack([delta_rule(r[:, h], k[:, h], v[:, h], w[:, h], a[:, h])[0] for h in range(H)], 1)
    o = rms(o, eps).reshape(T, H * d) * W[p + "norm"] * torch.sigmoid(u @ W[p + "g"].T)
    return o @ W[p + "o"].T


def side_by_side_mixer(u, W, p, m, eps):
    return m["left_scale"] * window_branch(u, W, p + "left.", m["left"], eps) + \
        m["right_scale"] * delta_branch(u, W, p + "right.", m["right"], eps)


def mixer(u, W, p, layer, eps):
    kind, m = layer["type"], layer["mixer"]
    if kind == "attention":
        return sink_attention_mixer(u, W, p, m, eps)
    if kind == "latent_attention":
        return latent_attention_mixer(u, W, p, m, eps)
    if kind == "parallel":
        return side_by_side_mixer(u, W, p, m, eps)
    raise ValueError(kind)


# ---------------------------------------------------------------------------------------- feed-forward
def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def xielu(z, p, q):
    """two branches with learned curvatures: sp(p) z^2 + z / 2 right of zero, (1/2 + sp(q)) (e^z - 1 - z) + z / 2 left"""
    pos = softplus(float(p)) * z * z + 0.5 * z
    neg = (0.5 + softplus(float(q))) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def dense_ff(u, W, p):
    return xielu(u @ W[p + "up"].T, W[p + "act"][0], W[p + "act"][1]) @ W[p + "down"].T


# ---------------------------------------------------------------------------------------- whole model
def layer_order(config):
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(tokens, W, config, layers_out=None):
    """logits [T, vocab] of one sequence; ``layers_out`` collects the sum of the stream copies behind every layer run"""
    eps = config["norm"]["eps"]
    S = int(config.get("streams") or 1)
    x = W["embed"][torch.tensor(tokens)] * (config.get("embedding") or {}).get("scale", 1.0)
    X = torch.stack([x] * S)
    for li in layer_order(config):
        layer = config["layers"][li]
        subs = [("1", lambda u: mixer(u, W, f"l{li}.mix.", layer, eps))]
        if layer.get("mlp") is not None:
            subs.append(("2", lambda u: dense_ff(u, W, f"l{li}.mlp.")))
        for n, f in subs:
            hc = f"l{li}.hc{n}."
            if hc + "in" in W:
                y = f(norm_one_plus(read_streams(X, W[hc + "in"]), W[f"l{li}.norm{n}"], eps))
                X = write_streams(X, y, W[hc + "out"], W[hc + "mix"])
            else:
                X = X + f(norm_one_plus(X[0], W[f"l{li}.norm{n}"], eps))[None]
        if layers_out is not None:
            layers_out.append(X.sum(0))
    z = norm_one_plus(X.sum(0), W["final.norm"], eps) @ W["embed"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


# ---------------------------------------------------------------------------------------- small random models
def sink_layer(heads=4, kv_heads=2, dim=16, vdim=24, rot=(8, 100.0), ff=48):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent_layer(heads=3, dim=12, vdim=20, rank=16, ff=48):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": dim ** -0.5},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def side_layer(heads=4, kv_heads=2, dim=16, window=9, rheads=2, rdim=16, scales=(1.3, 0.7), ff=48):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5}
    if window:
        left["mask"] = {"size": window}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "dim": rdim}, "left_scale": scales[0],
                                          "right_scale": scales[1]},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, loop=None, streams=2, width=40, vocab=67, softcap=12.0, embed_scale=0.6, eps=1e-5):
    cfg = {"architecture": "Dimelix", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps},
           "vocab": vocab, "width": width}
    if streams:
        cfg["streams"] = streams
    if softcap:
        cfg["logit_softcap"] = softcap
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tensor_shapes(config, decay_rank=6):
    """name -> shape of every checkpoint tensor of ``config``"""
    D, S = config["width"], int(config.get("streams") or 0)
    out = {"embed": (config["vocab"], D), "final.norm": (D,)}
    for li, layer in enumerate(config["layers"]):
        p, m = f"l{li}.mix.", layer["mixer"]
        out[f"l{li}.norm1"] = (D,)
        if layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({p + "q": (H * d, D), p + "k": (G * d, D), p + "v": (G * e, D), p + "q.norm": (d,), p + "k.norm": (d,),
                        p + "sink": (H,), p + "g": (H * e, D), p + "o": (D, H * e)})
        elif layer["type"] == "latent_attention":
            H, d, e, r = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
            out.update({p + "q": (H * d, D), p + "dkv": (r, D), p + "dkv.norm": (r,), p + "uk": (H * d, r), p + "uv": (H * e, r),
                        p + "g": (H * e, D), p + "o": (D, H * e)})
        else:
            a, b = m["left"], m["right"]
            H, G, d = a["heads"], a["kv_heads"], a["dim"]
            out.update({p + "left.q": (H * d, D), p + "left.k": (G * d, D), p + "left.q.norm": (d,), p + "left.k.norm": (d,),
                        p + "left.g": (H * d, D), p + "left.o": (D, H * d)})
            n = b["heads"] * b["dim"]
            out.update({p + "right." + k: (n, D) for k in ("r", "k", "v", "g", "a")})
            out.update({p + "right.a.b": (n,), p + "right.w1": (decay_rank, D), p + "right.w2": (n, decay_rank),
                        p + "right.w0": (n,), p + "right.norm": (n,), p + "right.o": (D, n)})
        subs = ["1"]
        if layer.get("mlp") is not None:
            f = layer["mlp"]["ff"]
            out.update({f"l{li}.norm2": (D,), f"l{li}.mlp.up": (f, D), f"l{li}.mlp.down": (D, f), f"l{li}.mlp.act": (2,)})
            subs.append("2")
        if S:
            for n in subs:
                out.update({f"l{li}.hc{n}.in": (S,), f"l{li}.hc{n}.out": (S,), f"l{li}.hc{n}.mix": (S, S)})
    return out


def random_weights(config, seed=0, decay_rank=6):
    """bfloat16-representable random tensors by name (so that an engine that stores bfloat16 reads the same numbers)"""
    g = torch.Generator().manual_seed(seed)
    S = int(config.get("streams") or 0)
    W = {}
    for name, shape in tensor_shapes(config, decay_rank).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if len(shape) == 2 and not leaf.startswith("hc"):
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[1]))
            if name == "embed":
                t = t * math.sqrt(shape[1]) / 1.5
        elif leaf.endswith(".in"):
            t = 1.0 / S + 0.2 * torch.randn(shape, generator=g)
        elif leaf.endswith(".out"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf.endswith(".mix"):
            t = torch.eye(S) + 0.2 * torch.randn(shape, generator=g)
        elif leaf.endswith("q.norm") or leaf.endswith("k.norm") or leaf.endswith("dkv.norm") or leaf == "mix.right.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf.endswith("sink"):
            t = torch.randn(shape, generator=g)
        elif leaf.endswith("act"):
            t = torch.randn(shape, generator=g)
        else:                                             # one-plus norm weights, biases of the decay and the removal rate
            t = 0.3 * torch.randn(shape, generator=g)
        W[name] = t.to(torch.bfloat16).to(F64)
    return W


def random_tokens(n, vocab, seed):
    rnd = random.Random(seed)
    return [rnd.randrange(vocab) for _ in range(n)]
