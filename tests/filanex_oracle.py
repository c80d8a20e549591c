"""Plain, slow float64 statement of the Filanex design: one function per mechanism, whole sequences, nothing shared with
``bigdl_amd``.  Weights are a dict of float64 tensors by checkpoint name; ``config`` is the parsed ``config.json``.

Notation: x is the residual stream [T, width], N(u) = w * u / sqrt(mean(u^2) + eps).  A layer reads one normed copy of
the stream for both of its sublayers: u = N(x), x <- x + mixer(u) + ff(u).  The layer list may hold a run of layers that
is executed several times with the same weights; in front of every such pass the stream is mixed with the embedding
output e: x <- W_in [x ; e].
"""
import math

import torch

F64 = torch.float64


def norm(u, w, eps):
    return u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w


# ---------------------------------------------------------------------------------------- embedding
def pair_rows(tokens, table):
    """row of the token-pair table for every position: a hash of (previous token, token); the first position has no
    previous token and takes the table's last row"""
    n, a, b = table["buckets"], table["mul_prev"], table["mul_cur"]
    return [n if t == 0 else (tokens[t - 1] * a + tokens[t] * b) % n for t in range(len(tokens))]


def embed(tokens, W, config):
    x = W["embed"][torch.tensor(tokens)]
    table = (config.get("embedding") or {}).get("bigram")
    if table:
        x = x + W["bigram"][torch.tensor(pair_rows(tokens, table))]
    return x


# ---------------------------------------------------------------------------------------- rotation
def pair_frequencies(rot):
    """angular frequency of every rotated pair and the amplitude of the rotation.  With a scaling entry, pairs whose
    wavelength is long against the original context are slowed by ``factor``, short ones stay, a linear ramp over the
    pair index joins the two, and cosine and sine grow by 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def index_of(turns):                 # the (real-valued) pair index whose wavelength makes `turns` turns in the original context
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(index_of(sc["fast"])), 0)
    hi = min(math.ceil(index_of(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / sc["factor"] * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def turn_neighbours(u, pos, freqs, amp):
    """channels (2 i, 2 i + 1) of u [..., n] turned by pos * freqs[i], cosine and sine times amp; the rest unchanged"""
    out = u.clone()
    for i, f in enumerate(freqs):
        c, s = amp * math.cos(pos * f), amp * math.sin(pos * f)
        a, b = u[..., 2 * i], u[..., 2 * i + 1]
        out[..., 2 * i], out[..., 2 * i + 1] = a * c - b * s, b * c + a * s
    return out


# ---------------------------------------------------------------------------------------- attention
def sees(i, j, size):
    """causal, and only inside the same block of ``size`` positions counted from the sequence's start"""
    return j <= i and (not size or i // size == j // size)


def capped(s, cap):
    return cap * torch.tanh(s / cap) if cap else s


def attend(q, k, v, scale, cap, size):
    """q [T, H, d], k [T, G, d], v [T, G, e] -> [T, H, e]: softmax over the visible keys of the capped, scaled scores"""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if sees(i, j, size)]
        for h in range(H):
            g = h // (H // G)
            out[i, h] = torch.softmax(capped((k[js, g] @ q[i, h]) * scale, cap), 0) @ v[js, g]
    return out


def attention_mixer(u, W, p, m):
    T = u.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (u @ W[p + "q"].T).view(T, H, d)
    k = (u @ W[p + "k"].T).view(T, G, d)
    v = (u @ W[p + "v"].T).view(T, G, e)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        freqs, amp = pair_frequencies(rot)
        q = torch.stack([turn_neighbours(q[t], t, freqs, amp) for t in range(T)])
        k = torch.stack([turn_neighbours(k[t], t, freqs, amp) for t in range(T)])
    out = attend(q, k, v, m["scale"], m.get("softcap"), (m.get("mask") or {}).get("size"))
    gate = torch.sigmoid(u @ W[p + "g"].T)
    return (out.reshape(T, H * e) * gate) @ W[p + "o"].T


# ---------------------------------------------------------------------------------------- feed-forwards
def dense_ff(u, W, p):
    a = u @ W[p + "up"].T + W[p + "up.b"]
    a = 0.5 * a * (1.0 + torch.erf(a / math.sqrt(2.0)))
    return a @ W[p + "down"].T + W[p + "down.b"]


def route(u, W, p, r):
    """chosen experts and their weights for one token: sigmoid scores; a group of neighbouring experts is worth the sum
    of its two best scores; the best experts inside the best groups; weights = scores over their sum"""
    s = torch.sigmoid(W[p + "router"] @ u)
    E, top = r["experts"], r["top"]
    g = r.get("groups") or {}
    count = g.get("count", 1)
    keep = g.get("keep", count)
    size = E // count
    worth = [float(s[c * size:(c + 1) * size].sort(descending=True).values[:2].sum()) for c in range(count)]
    kept = sorted(range(count), key=lambda c: -worth[c])[:keep]
    allowed = [e for e in range(E) if e // size in kept]
    chosen = sorted(allowed, key=lambda e: -float(s[e]))[:top]
    total = sum(float(s[e]) for e in chosen) + 1e-20
    return chosen, [float(s[e]) / total for e in chosen]


def expert(u, W, p):
    a = W[p + "gate"] @ u
    return W[p + "down"] @ (a * torch.sigmoid(a) * (W[p + "up"] @ u))


def moe_ff(u, W, p, f, choices=None):
    out = torch.zeros(u.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(u.shape[0]):
        chosen, weights = route(u[t], W, p, f["router"])
        if choices is not None:
            choices.append(chosen)
        for e, w in zip(chosen, weights):
            out[t] += w * expert(u[t], W, f"{p}e{e}.")
    return out


# ---------------------------------------------------------------------------------------- the stack
def layer_runs(config):
    """[(layer index, mix the embedding output in before it)] in execution order"""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def layer(x, W, li, spec, eps, choices=None):
    u = norm(x, W[f"l{li}.norm1"], eps)
    if spec["type"] != "attention":
        raise ValueError(spec["type"])
    y = attention_mixer(u, W, f"l{li}.mix.", spec["mixer"])
    f = spec.get("mlp")
    if f is not None:
        y = y + (moe_ff(u, W, f"l{li}.mlp.", f, choices) if f["kind"] == "moe" else dense_ff(u, W, f"l{li}.mlp."))
    return x + y


def forward(tokens, W, config, collect=None, choices=None):
    """logits [T, vocab] of one whole sequence; ``collect`` receives the stream after every layer run"""
    eps = config["norm"]["eps"]
    e = embed(tokens, W, config)
    x = e
    for li, mix_in in layer_runs(config):
        if mix_in:
            x = torch.cat([x, e], -1) @ W["loop.in"].T
        x = layer(x, W, li, config["layers"][li], eps, choices)
        if collect is not None:
            collect.append(x.clone())
    return norm(x, W["final.norm"], eps) @ W["head"].T


# ---------------------------------------------------------------------------------------- small models for the tests
def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, size=24, cap=8.0, scale=None, rot=(8, 500.0, (3.0, 64, 4.0, 0.5)),
                    mlp="dense"):
    """rot: (dims, base, scaling or None) with scaling = (factor, original, fast, slow); None: no rotation"""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or 2.0 * dim ** -0.5}
    if size:
        m["mask"] = {"size": size}
    if cap:
        m["softcap"] = cap
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
        if rot[2]:
            m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rot[2]))
    return {"type": "attention", "mixer": m, "mlp": dense(40) if mlp == "dense" else mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=12, count=3, keep=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def make_config(layers, vocab=80, width=48, loop=None, pairs=(37, 11, 5), eps=1e-5):
    """loop: (start, stop, times) or None; pairs: (buckets, mul_prev, mul_cur) or None"""
    cfg = {"architecture": "Filanex", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if pairs:
        cfg["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), pairs))}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def random_weights(config, seed=0):
    """bfloat16 checkpoint tensors; router rows are wide enough that the choices vary from token to token"""
    g = torch.Generator().manual_seed(seed)
    D = config["width"]

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, generator=g) * (s / math.sqrt(k))).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    sd = {"embed": mat(config["vocab"], D, math.sqrt(D)), "final.norm": vec(D, 1.0), "head": mat(config["vocab"], D)}
    table = (config.get("embedding") or {}).get("bigram")
    if table:
        sd["bigram"] = mat(table["buckets"] + 1, D, math.sqrt(D))
    if config.get("loop"):
        sd["loop.in"] = mat(D, 2 * D, 1.4)
    for li, spec in enumerate(config["layers"]):
        p, q, m = f"l{li}.mix.", f"l{li}.mlp.", spec["mixer"]
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        sd[f"l{li}.norm1"] = vec(D, 1.0, 0.2)
        sd[p + "q"], sd[p + "k"], sd[p + "v"], sd[p + "g"] = mat(H * d, D, 2.0), mat(G * d, D, 2.0), mat(G * e, D), mat(H * e, D, 2.0)
        sd[p + "o"] = mat(D, H * e)
        f = spec.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            sd[q + "up"], sd[q + "up.b"] = mat(f["ff"], D), vec(f["ff"], 0.0, 0.3)
            sd[q + "down"], sd[q + "down.b"] = mat(D, f["ff"]), vec(D, 0.0, 0.3)
        else:
            sd[q + "router"] = mat(f["router"]["experts"], D, 3.0)
            for x in range(f["router"]["experts"]):
                n = f["expert"]["ff"]
                sd[q + f"e{x}.gate"], sd[q + f"e{x}.up"], sd[q + f"e{x}.down"] = mat(n, D, 2.0), mat(n, D), mat(D, n)
    return sd


def as_f64(sd):
    return {k: v.double() for k, v in sd.items()}
