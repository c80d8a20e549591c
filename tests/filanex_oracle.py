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
    size = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, e, dtype=F64)
    for i in range(T):
        js = [j for j in range(T) if sees(i, j, size)]
        for h in range(H):
            g = h // (H // G)
            s = capped((k[js, g] @ q[i, h]) * m["scale"], m.get("softcap"))
            out[i, h] = torch.softmax(s, 0) @ v[js, g]
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
