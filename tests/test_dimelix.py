"""The Dimelix design on the ragged engine against the plain float64 statement in ``dimelix_oracle.py``.

Every test runs twice: on the CPU (the engine's bookkeeping over the unfused statements of ``ops/ragged.py``) and,
marked ``gpu``, on the device (the HIP kernels of ``libbigdl_ragged.so``).  Models are small and random; where random
weights would hide a fault (one key among many, a window's edge, a page's border, a sink) the inputs are made so that it
shows.
"""
import json
import math
import os

import pytest
import torch

import dimelix_oracle as O
from bigdl_amd.models import dimelix
from bigdl_amd.models.paged import PagedStatePool
from bigdl_amd.ops import ragged as R

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32_TOL = 3e-4


def engine_for(config, W, dtype, device):
    return dimelix.build_engine(dimelix.read_config(config), W, dtype, device)


def full_model():
    """all three kinds of layers, one without a feed-forward; layers 1 .. 2 run three times; three copies of the stream"""
    return O.make_config([O.side_layer(), O.sink_layer(), O.latent_layer(ff=None), O.side_layer(heads=2, kv_heads=1, dim=8, window=70,
                                                                                               rheads=3, rdim=10),
                          O.sink_layer(heads=3, kv_heads=3, dim=10, vdim=6, rot=(10, 50.0))], loop=(1, 3, 3), streams=3)


def run_schedule(engine, prompts, schedule, max_tokens, slots=4, seen=None):
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
            if seen is not None:
                seen.setdefault(rid, (set(), set()))[0].update(pool.pages_of[slot[rid]])
                seen[rid][1].add(slot[rid])
            if at[rid] == len(prompts[rid]):
                pool.release(slot.pop(rid))
    return {k: torch.cat(v) for k, v in got.items() if v}


def close(a, b, tol=F32_TOL):
    assert a.shape == b.shape
    err = float((a - b).abs().max())
    assert err <= tol, f"max difference {err}"


# ------------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layers,loop,streams", [
    ([O.sink_layer()], None, 2),
    ([O.latent_layer()], None, 2),
    ([O.side_layer()], None, 2),
    ([O.sink_layer(heads=1, kv_heads=1, dim=8, vdim=12, rot=(8, 7.0), ff=None)], (0, 1, 3), 1),   # one head, whole head turned
    ([O.sink_layer(heads=6, kv_heads=6, dim=12, vdim=10, rot=None)], None, None),                  # no rotation, no stream copies
    ([O.sink_layer(heads=8, kv_heads=1, dim=32, vdim=136, rot=(2, 1e4))], None, 4),                # values wider than keys
    ([O.latent_layer(heads=1, dim=7, vdim=5, rank=9, ff=None)], None, 2),                          # odd sizes
    ([O.latent_layer(heads=5, dim=16, vdim=16, rank=16)], (0, 1, 2), 3),                           # all sizes equal
    ([O.latent_layer(heads=2, dim=8, vdim=24, rank=160)], None, 2),                                # a row wider than a head
    ([O.side_layer(heads=1, kv_heads=1, dim=24, window=1, rheads=1, rdim=24)], None, 2),           # a window of one
    ([O.side_layer(heads=6, kv_heads=2, dim=12, window=None, rheads=5, rdim=6, scales=(1.0, 1.0))], (0, 1, 2), 1),   # no window
    ([O.side_layer(heads=4, kv_heads=4, dim=8, window=64, rheads=2, rdim=40, scales=(0.0, 2.0))], None, 2),
    ([O.side_layer(heads=2, kv_heads=1, dim=20, window=65, rheads=1, rdim=70, scales=(0.5, 0.0), ff=None)], None, 5),
])
def test_each_layer_kind_alone(device, layers, loop, streams):
    cfg = O.make_config(layers, loop=loop, streams=streams)
    W = O.random_weights(cfg, seed=1)
    toks = O.random_tokens(90, cfg["vocab"], 2)
    want = O.forward(toks, W, cfg)
    eng = engine_for(cfg, W, torch.float32, device)
    close(run_schedule(eng, {"a": toks}, [[("a", 60)], [("a", 2)]] + [[("a", 1)] for _ in range(28)], 128)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_layer_outputs_one_by_one(device):
    cfg = full_model()
    W = O.random_weights(cfg, seed=3)
    toks = O.random_tokens(40, cfg["vocab"], 4)
    want = []
    O.forward(toks, W, cfg, layers_out=want)
    assert len(want) == 1 + 2 * 3 + 2
    eng = engine_for(cfg, W, torch.float32, device)
    pool = eng.ensure_pool(64, 1)
    got = []
    eng.step([(pool.admit(), toks)], collect=got)
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        err = float((a.double().cpu() - b).abs().max()) / max(1.0, float(b.abs().max()))
        assert err < 2e-5, f"layer execution {i}: {err}"


@pytest.mark.parametrize("device", DEVICES)
def test_prompt_against_token_by_token_and_portions(device):
    cfg = full_model()
    W = O.random_weights(cfg, seed=5)
    toks = O.random_tokens(150, cfg["vocab"], 6)
    want = O.forward(toks, W, cfg)
    eng = engine_for(cfg, W, torch.float32, device)
    close(run_schedule(eng, {"a": toks}, [[("a", 150)]], 192)["a"], want)
    close(run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in range(150)], 192)["a"], want)
    for sizes in ([2] * 75, [64, 2, 62, 3, 1, 1, 17], [63, 1, 1, 63, 2, 20], [5, 128, 2, 2, 13], [1, 2, 3, 4, 5, 64, 65, 6],
                  [9, 1, 8, 2, 70, 60]):
        assert sum(sizes) == 150
        close(run_schedule(eng, {"a": toks}, [[("a", n)] for n in sizes], 192)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_requests_in_one_batch_and_reuse_of_pages_and_slots(device):
    cfg = full_model()
    W = O.random_weights(cfg, seed=7)
    lens = {"a": 130, "b": 7, "c": 70, "d": 1, "e": 66, "f": 90}
    prompts = {k: O.random_tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(p, W, cfg) for k, p in prompts.items()}
    # three slots, pool of 5 pages (320 tokens) for 364 tokens in total: d, e, f run in what a, b, c gave back
    schedule = [[("a", 60), ("b", 2), ("c", 1)], [("a", 1), ("b", 5), ("c", 63)], [("a", 5), ("c", 6)],
                [("a", 64), ("d", 1)], [("e", 2), ("f", 30)], [("e", 64), ("f", 1)], [("f", 59)]]
    eng = engine_for(cfg, W, torch.float32, device)
    seen = {}
    got = run_schedule(eng, prompts, schedule, 320, slots=3, seen=seen)
    for k in prompts:
        close(got[k], want[k])
    old, new = ("a", "b", "c"), ("d", "e", "f")
    assert set().union(*(seen[k][0] for k in new)) & set().union(*(seen[k][0] for k in old)), "no page was used twice"
    assert set().union(*(seen[k][1] for k in new)) & set().union(*(seen[k][1] for k in old)), "no slot was used twice"
    alone = run_schedule(eng, {"c": prompts["c"]}, [[("c", 70)]], 128)["c"]
    close(alone, got["c"], 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_windows_and_pages(device):
    cfg = O.make_config([O.side_layer(window=16), O.sink_layer(), O.side_layer(window=70, ff=None), O.latent_layer()], loop=(0, 2, 2))
    W = O.random_weights(cfg, seed=9)
    toks = O.random_tokens(200, cfg["vocab"], 11)
    want = O.forward(toks, W, cfg)
    eng = engine_for(cfg, W, torch.float32, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)] for _ in range(195)], 256)["a"]
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_long_portions_run_the_delta_rule_in_chunks(device):
    """a portion of several hundred tokens (the recurrence is cut into chunks that are scanned side by side and chained)
    beside a short one and a single token, into a state that an earlier portion has left"""
    cfg = O.make_config([O.side_layer(window=40, rheads=2, rdim=24), O.side_layer(heads=2, kv_heads=2, dim=8, window=None, rheads=3, rdim=40)],
                        loop=(0, 1, 2))
    W = O.random_weights(cfg, seed=15)
    prompts = {"a": O.random_tokens(420, cfg["vocab"], 16), "b": O.random_tokens(300, cfg["vocab"], 17), "c": O.random_tokens(9, cfg["vocab"], 18)}
    want = {k: O.forward(p, W, cfg) for k, p in prompts.items()}
    eng = engine_for(cfg, W, torch.float32, device)
    got = run_schedule(eng, prompts, [[("a", 30), ("c", 3)], [("a", 390), ("b", 257), ("c", 1)], [("b", 43), ("c", 5)]], 832)
    for k in prompts:
        close(got[k], want[k], 5e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("odd", [False, True, "wide"])
def test_bfloat16_stays_near_the_exact_result(device, odd):
    if odd == "wide":    # latent rows beyond a head's width, many heads on one cached row, eight query heads per key head
        layers = [O.latent_layer(heads=20, dim=16, vdim=16, rank=160), O.sink_layer(heads=8, kv_heads=1, dim=32, vdim=32, rot=(32, 1e4)),
                  O.latent_layer(heads=3, dim=24, vdim=8, rank=320, ff=None)]
    elif odd:        # sizes that take none of the vector or matrix-core paths
        layers = [O.side_layer(heads=3, kv_heads=1, dim=20, window=30, rheads=1, rdim=34), O.sink_layer(heads=3, kv_heads=1, dim=18, vdim=14, rot=(6, 90.0)),
                  O.latent_layer(heads=3, dim=10, vdim=6, rank=21)]
    else:            # sizes that the vector and matrix-core paths serve
        layers = [O.side_layer(heads=4, kv_heads=2, dim=32, window=40, rheads=2, rdim=32), O.sink_layer(heads=4, kv_heads=1, dim=64, vdim=48, rot=(16, 100.0)),
                  O.latent_layer(heads=4, dim=32, vdim=32, rank=64)]
    cfg = O.make_config(layers, width=64, loop=(0, 2, 2))
    W = O.random_weights(cfg, seed=13)
    toks = O.random_tokens(100, cfg["vocab"], 14)
    want = O.forward(toks, W, cfg)
    eng = engine_for(cfg, W, torch.bfloat16, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 70)], [("a", 2)]] + [[("a", 1)] for _ in range(28)], 128)["a"]
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    rel = d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    assert float(rel.median()) < 0.05 and float(rel.max()) < 0.15, (float(rel.median()), float(rel.max()))


def _random_design(seed):
    """a model of the design with everything drawn at random: kinds and order of layers, sizes, loop, copies, constants"""
    import random
    rnd = random.Random(seed)
    layers = []
    for _ in range(rnd.randint(2, 4)):
        kind = rnd.choice(["sink", "latent", "side"])
        ff = rnd.choice([None, 24, 56])
        kv = rnd.choice([1, 2, 3])
        heads = kv * rnd.choice([1, 2, 4])
        dim = rnd.choice([8, 12, 16, 24, 40, 48, 64])
        if kind == "sink":
            rot = rnd.choice([None, (rnd.choice([2, 4, 8]), rnd.choice([100.0, 1e4, 5e5])), (dim, 77.0)])
            layers.append(O.sink_layer(heads=heads, kv_heads=kv, dim=dim, vdim=rnd.choice([8, 16, 20, 48, 80]), rot=rot, ff=ff))
        elif kind == "latent":
            layers.append(O.latent_layer(heads=heads, dim=dim, vdim=rnd.choice([8, 16, 28]), rank=rnd.choice([8, 24, 64, 72, 144]), ff=ff))
        else:
            layers.append(O.side_layer(heads=heads, kv_heads=kv, dim=dim, window=rnd.choice([None, 1, 5, 33, 64, 100, 150]),
                                       rheads=rnd.randint(1, 4), rdim=rnd.choice([8, 16, 32, 40, 72]),
                                       scales=(rnd.choice([0.5, 1.0, 1.7]), rnd.choice([0.25, 1.0, 2.0])), ff=ff))
        layers[-1]["mixer"]["scale"] = layers[-1]["mixer"].get("scale", 1.0) * rnd.choice([0.5, 1.0, 2.0]) if kind != "side" else 1.0
        if kind == "side":
            layers[-1]["mixer"].pop("scale")
            layers[-1]["mixer"]["left"]["scale"] *= rnd.choice([0.5, 1.0, 2.0])
    n = len(layers)
    a = rnd.randrange(n)
    loop = rnd.choice([None, (a, rnd.randint(a, n), rnd.randint(0, 3))])
    return O.make_config(layers, loop=loop, streams=rnd.choice([None, 1, 2, 3, 4]), width=rnd.choice([24, 40, 64]), vocab=rnd.choice([50, 67, 128]),
                         softcap=rnd.choice([None, 8.0, 30.0]), embed_scale=rnd.choice([0.4, 1.0, 1.5]), eps=rnd.choice([1e-5, 1e-6, 1e-3]))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("seed", range(8))
def test_random_models_of_the_design(device, seed):
    """three unequal requests in mixed steps (two slots, pages used again) against the plain statement, in float32; in
    bfloat16 the same steps stay near it"""
    cfg = _random_design(seed)
    W = O.random_weights(cfg, seed=100 + seed, decay_rank=1 + seed)
    prompts = {"a": O.random_tokens(140, cfg["vocab"], 200 + seed), "b": O.random_tokens(30, cfg["vocab"], 300 + seed),
               "c": O.random_tokens(75, cfg["vocab"], 400 + seed)}
    want = {k: O.forward(p, W, cfg) for k, p in prompts.items()}
    schedule = [[("a", 66), ("b", 3)], [("a", 1), ("b", 27)], [("a", 2), ("c", 70)], [("a", 70), ("c", 1)], [("a", 1), ("c", 4)]]
    got = run_schedule(engine_for(cfg, W, torch.float32, device), prompts, schedule, 320, slots=2)
    for k in prompts:
        scale = max(1.0, float(want[k].abs().max()))
        close(got[k] / scale, want[k] / scale)
    got = run_schedule(engine_for(cfg, W, torch.bfloat16, device), prompts, schedule, 320, slots=2)
    for k in prompts:
        d = got[k] - want[k]
        d = d - d.mean(-1, keepdim=True)
        rel = d.pow(2).mean(-1).sqrt() / (want[k] - want[k].mean(-1, keepdim=True)).pow(2).mean().sqrt()
        assert float(rel.median()) < 0.06 and float(rel.max()) < 0.25, (k, float(rel.median()), float(rel.max()))


# ------------------------------------------------------------------------------------------------ mechanisms alone
def _meta_for(pool, slot, n, device):
    pages = list(pool.reserve(slot, n))
    return R.BatchMeta([(slot, pool.len_of[slot], n, pages)], torch.device(device))


def _attend_through_pages(device, q, k, v, portions, *, scale, window=0, sinks=None, slopes=None, gate=None, page_order=None,
                          dtype=torch.float32):
    """q [T, H, d], k [T, G, d], v [T, G, e] (float64) through the paged attention op in the given portions"""
    T, H, d = q.shape
    G, e = k.shape[1], v.shape[2]
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("kv", G, d, e)]}, 64 * ((T + 63) // 64 + 2), 2, dtype, device)
    if page_order:
        pool.free_pages = list(page_order)
    slot = pool.admit()
    out, at = [], 0
    f32 = lambda t: None if t is None else torch.as_tensor(t, dtype=torch.float64).float().to(device)      # noqa: E731
    for n in portions:
        meta = _meta_for(pool, slot, n, device)
        for i in range(n):                                   # place keys / values as the cache holds them
            pos = at + i
            pg = pool.pages_of[slot][pos // 64]
            pool.k[0][pg, :, pos % 64] = k[pos].to(dtype).to(device)
            pool.v[0][pg, :, pos % 64] = v[pos].to(dtype).to(device)
        qq = q[at:at + n].reshape(n, H * d).float().to(device).contiguous()
        gg = None if gate is None else torch.cat([torch.zeros(n, 8), gate[at:at + n].float()], 1).to(dtype).to(device)
        out.append(ops.paged_attn(qq, pool.k[0], pool.v[0], meta, maps=1, H=H, G=G, d=d, vd=e, window=window or 0, keep_first=0,
                                  scale=scale, lam=0.0, out_scale=1.0, out_norm=False, eps=1e-6, gate=gg, gate0=8,
                                  gate_wide=gate is not None, sinks=f32(sinks), slopes=f32(slopes)))
        pool.commit(slot, n)
        at += n
    return torch.cat(out).double().cpu().view(T, H, e)


def _portions_for(i, T, decode_tail):
    head = T - decode_tail
    if decode_tail == 0 or i >= head:
        return [n for n in [head // 3, head - head // 3] + [1] * decode_tail if n]
    return [n for n in [i + 1, head - i - 1] + [1] * decode_tail if n]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode_tail", [0, 12])
@pytest.mark.parametrize("window", [70, 64, 16, 128, 1, 129, None])
def test_window_edges_far_keys_and_page_borders_stand_out(device, decode_tail, window):
    """Query i and key j are made parallel and long, so key j takes all of the weight when it is visible; its value is a
    marker.  One position off at a window's edge or at a page's border swaps the marker in or out.  With distance slopes
    the far key of the no-window case still wins (its score is large against slope * distance)."""
    g = torch.Generator().manual_seed(21)
    T, H, G, d, e = 210, 2, 1, 12, 4
    cases = []                                               # (query position, key position)
    for i in (140, 191, 192, 193, 209, 69, 70, 127, 128):
        lo = i - window + 1 if window else 0
        cases += [(i, lo), (i, lo - 1), (i, lo + 1), (i, i), (i, 0), (i, i - 1)]
    cases += [(100, 63), (100, 64), (130, 127), (130, 128), (64, 63), (64, 64), (0, 0), (1, 0), (15, 0), (16, 0), (16, 15)]
    cases = [(i, j) for i, j in cases if 0 <= j <= i]
    slopes = [0.05, 0.001]
    for i, j in cases:
        q = torch.randn(T, H, d, generator=g).double() * 0.3
        k = torch.randn(T, G, d, generator=g).double() * 0.3
        v = torch.randn(T, G, e, generator=g).double()
        direction = torch.randn(d, generator=g).double()
        direction /= direction.norm()
        q[i, :] = 9.0 * direction
        k[j, 0] = 9.0 * direction
        v[j, 0] = torch.tensor([100.0, -100.0, 50.0, 25.0], dtype=O.F64)
        want = O.attend(q, k, v, 1.0, window=window, slopes=slopes)
        got = _attend_through_pages(device, q, k, v, _portions_for(i, T, decode_tail), scale=1.0, window=window, slopes=slopes,
                                    page_order=[5, 0, 3, 1, 4, 2])
        close(got[i], want[i], 2e-3)
        close(got, want, 2e-3)


@pytest.mark.parametrize("device", DEVICES)
def test_sinks_take_their_share_of_every_head(device):
    """a sink far above the scores leaves almost nothing to the values, one far below changes nothing, and every head has
    its own; the first token of a sequence shares its weight with the sink alone"""
    g = torch.Generator().manual_seed(23)
    T, H, G, d, e = 150, 4, 2, 16, 8
    q, k = torch.randn(T, H, d, generator=g).double(), torch.randn(T, G, d, generator=g).double()
    v = torch.randn(T, G, e, generator=g).double() + 2.0
    gate = torch.randn(T, H * e, generator=g).double() * 3
    sinks = [16.0, -40.0, 0.3, 2.5]
    want = O.attend(q, k, v, 0.5, sinks=sinks)
    plain = O.attend(q, k, v, 0.5)
    assert float(want[:, 0].abs().max()) < 0.05 and float((want[:, 1] - plain[:, 1]).abs().max()) < 1e-9
    assert float((want[:, 2] - plain[:, 2]).abs().max()) > 0.1
    close(want[0, 2], v[0, 1] / (1.0 + math.exp(0.3 - float(q[0, 2] @ k[0, 1]) * 0.5)), 1e-9)
    for portions in ([150], [1] * 20 + [130], [90, 2, 58], [64, 64] + [1] * 22):
        got = _attend_through_pages(device, q, k, v, portions, scale=0.5, sinks=sinks, gate=gate)
        close(got, want * torch.sigmoid(gate).view(T, H, e), 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_scores_fall_with_the_distance(device):
    """all keys alike: the weights are a softmax of -slope * distance alone, so the output is known in closed form; the
    form slope * key position would give the same weights here, but not beside a sink"""
    T, H, G, d, e = 100, 2, 1, 8, 2
    q, k = torch.ones(T, H, d, dtype=O.F64), torch.ones(T, G, d, dtype=O.F64)
    v = torch.zeros(T, G, e, dtype=O.F64)
    v[:, 0, 0] = torch.arange(T, dtype=O.F64)
    v[:, 0, 1] = 1.0
    slopes, sinks = [0.5, 0.02], [8.0, 7.0]
    for window in (None, 30):
        for sk in (None, sinks):
            want = torch.zeros(T, H, e, dtype=O.F64)
            for i in range(T):
                js = torch.arange(max(0, i - window + 1) if window else 0, i + 1, dtype=O.F64)
                for h in range(H):
                    w = torch.exp(8.0 - slopes[h] * (i - js))
                    w = w / (w.sum() + (math.exp(sk[h]) if sk else 0.0))
                    want[i, h, 0], want[i, h, 1] = (w * js).sum(), w.sum()
            close(O.attend(q, k, v, 1.0, window=window, sinks=sk, slopes=slopes), want, 1e-9)
            got = _attend_through_pages(device, q, k, v, [70, 3] + [1] * 27, scale=1.0, window=window, sinks=sk, slopes=slopes)
            close(got, want, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_values_are_the_keys_before_their_norm(device):
    """the window branch alone: the cache's value pages hold the raw key projections, its key pages the normed ones"""
    cfg = O.make_config([O.side_layer(heads=2, kv_heads=1, dim=8, window=20, scales=(1.0, 0.0), ff=None)], streams=None)
    W = O.random_weights(cfg, seed=27)
    W["l0.mix.left.k.norm"] = W["l0.mix.left.k.norm"] * 3.0           # normed and raw keys differ a lot
    toks = O.random_tokens(50, cfg["vocab"], 28)
    eng = engine_for(cfg, W, torch.float32, device)
    close(run_schedule(eng, {"a": toks}, [[("a", 30)], [("a", 20)]], 64)["a"], O.forward(toks, W, cfg))
    pool = eng.ensure_pool(64, 1)
    slot = pool.admit()
    eng.step([(slot, toks[:10])])
    u = O.norm_one_plus(W["embed"][torch.tensor(toks[:10])] * cfg["embedding"]["scale"], W["l0.norm1"], 1e-5)
    kraw = u @ W["l0.mix.left.k"].T
    page = pool.pages_of[slot][0]
    close(pool.v[0][page, 0, :10].double().cpu(), kraw, 1e-4)
    close(pool.k[0][page, 0, :10].double().cpu(), O.norm_plain(kraw, W["l0.mix.left.k.norm"], 1e-5), 1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,d", [(2, 16), (1, 48), (3, 40), (1, 130), (5, 6)])
def test_delta_rule_state_across_portions_and_in_a_used_slot(device, H, d):
    """the scan op alone against the token-by-token statement: portions of 1, 2 and many tokens, a second sequence in a
    slot that the first has left, and a long portion that is scanned in chunks"""
    g = torch.Generator().manual_seed(31)
    ops = R.ops_for(device)
    T, rank = 330, 5
    HD = H * d
    P = (torch.randn(T, 5 * HD + rank, generator=g) * 0.7)
    wl, w0, ab = torch.randn(T, HD, generator=g), torch.randn(HD, generator=g), torch.randn(HD, generator=g)
    r, k, v, a_logit = (P[:, i * HD:(i + 1) * HD].double().view(T, H, d) for i in (0, 1, 2, 4))
    w = torch.exp(-O.DECAY_RATE * torch.sigmoid(wl.double() + w0.double())).view(T, H, d)
    a = torch.sigmoid(a_logit + ab.double().view(H, d))

    def statement(lo, hi):
        return torch.stack([O.delta_rule(r[lo:hi, h], k[lo:hi, h], v[lo:hi, h], w[lo:hi, h], a[lo:hi, h])[0] for h in range(H)], 1)

    def scan(pool, slot, lo, hi):
        n = hi - lo
        meta = R.BatchMeta([(slot, pool.len_of[slot], n, [])], torch.device(device))
        rows = P[lo:hi].to(device)
        arrays = ops.delta_gates(rows, 0, HD, 4 * HD, wl[lo:hi].to(device).contiguous(), w0.to(device), ab.to(device), O.DECAY_RATE,
                                 1e-6, H, d)
        out = ops.delta_scan(arrays, rows, 2 * HD, pool.matrix[0], H, d, d, meta)
        pool.commit(slot, n)
        return out.double().cpu().view(n, H, d)

    pool = PagedStatePool({0: [("matrix", H, d, d)]}, 64, 1, torch.float32, device)
    slot = pool.admit()
    cuts = [0, 1, 3, 40, 41, 43, 330]
    got = torch.cat([scan(pool, slot, lo, hi) for lo, hi in zip(cuts, cuts[1:])])
    want = statement(0, T)
    scale = float(want.abs().max())
    close(got / scale, want / scale, 2e-5)
    pool.release(slot)
    slot = pool.admit()                                      # the same slot: its old state must not leak into a new sequence
    close(scan(pool, slot, 100, 160) / scale, statement(100, 160) / scale, 2e-5)
    pool.release(slot)
    slot = pool.admit()
    close(scan(pool, slot, 0, 300) / scale, want[:300] / scale, 2e-5)     # one long portion: chunks side by side
    if device == "cuda":                                     # the walk over the chunks as library products (very tall states)
        ops.delta_chain = False
        pool.release(slot)
        slot = pool.admit()
        close(torch.cat([scan(pool, slot, 0, 20), scan(pool, slot, 20, 330)]) / scale, want / scale, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_forgets_along_the_key(device):
    """with removal rate 1 and no decay, writing the same unit key twice replaces the first value by the second"""
    ops = R.ops_for(device)
    H, d = 1, 8
    k = torch.zeros(d)
    k[3] = 1.0
    v1, v2 = torch.arange(1.0, d + 1), -torch.arange(1.0, d + 1)
    P = torch.zeros(2, 5 * d)
    P[:, 0:d] = k                                            # r = k: the output reads the value stored under k
    P[:, d:2 * d] = k
    P[0, 2 * d:3 * d], P[1, 2 * d:3 * d] = v1, v2
    P[:, 4 * d:5 * d] = 40.0                                 # removal rate sigmoid(40) = 1
    wl = torch.full((2, d), -40.0)                           # decay exp(-rate * sigmoid(-40)) = 1
    pool = PagedStatePool({0: [("matrix", H, d, d)]}, 64, 1, torch.float32, device)
    slot = pool.admit()
    meta = R.BatchMeta([(slot, 0, 2, [])], torch.device(device))
    arrays = ops.delta_gates(P.to(device), 0, d, 4 * d, wl.to(device), torch.zeros(d, device=device), torch.zeros(d, device=device),
                             O.DECAY_RATE, 1e-6, H, d)
    out = ops.delta_scan(arrays, P.to(device), 2 * d, pool.matrix[0], H, d, d, meta).cpu()
    close(out[0].double(), v1.double(), 1e-4)
    close(out[1].double(), v2.double(), 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_stream_copies_gate_columns_and_the_two_curvature_unit(device):
    g = torch.Generator().manual_seed(43)
    ops = R.ops_for(device)
    for S, D in ((1, 48), (2, 1000), (3, 1500), (4, 5000), (8, 40)):
        T = 5
        X = torch.randn(T, S, D, generator=g)
        y, w = torch.randn(T, D, generator=g), torch.randn(D, generator=g)
        prev, nxt = torch.randn(2 * S + S * S, generator=g), torch.randn(2 * S + S * S, generator=g)
        Xd = X.double().permute(1, 0, 2)
        new = O.write_streams(Xd, y.double(), prev[S:2 * S].double(), prev[2 * S:].double().view(S, S))
        u = O.read_streams(new, nxt[:S].double())
        Xs = X.clone().to(device)
        xa, uo = ops.hc_step(Xs, y.to(device), prev.to(device), nxt.to(device), w.to(device), 1e-5, torch.float32, want_u=True)
        close(Xs.double().cpu().permute(1, 0, 2), new, 1e-4)
        close(uo.double().cpu(), u, 1e-4)
        close(xa.double().cpu(), O.norm_plain(u, w.double(), 1e-5), 1e-4)
        Xs = X.clone().to(device)                            # read-out alone: the copies stay as they are
        xa, _ = ops.hc_step(Xs, None, None, nxt.to(device), w.to(device), 1e-5, torch.float32)
        close(Xs.cpu(), X, 0.0)
        close(xa.double().cpu(), O.norm_plain(O.read_streams(Xd, nxt[:S].double()), w.double(), 1e-5), 1e-4)
        Xs = X.clone().to(device)                            # write-back alone
        assert ops.hc_step(Xs, y.to(device), prev.to(device), None, None, 1e-5, torch.float32) == (None, None)
        close(Xs.double().cpu().permute(1, 0, 2), new, 1e-4)
    for width, c0, n in ((50, 7, 40), (56, 8, 40), (1040, 16, 1024)):      # columns that are and are not 16-byte pieces
        P = torch.randn(11, width, generator=g) * 3
        z = P[:, c0:c0 + n].double()
        for p, q in ((0.8, -1.3), (-2.0, 4.0), (0.0, 0.0)):
            sp = (O.softplus(p), O.softplus(q))
            close(ops.act_cols(P.to(device), c0, n, "xielu", sp).double().cpu(), O.xielu(z, p, q), 2e-5)
        close(ops.act_cols(P.to(device), c0, n, "tanh").double().cpu(), torch.tanh(z), 1e-5)
        o = torch.randn(11, n, generator=g)
        close(ops.gate_cols(o.to(device), P.to(device), c0, torch.float32, 1.7).double().cpu(), 1.7 * o.double() * torch.sigmoid(z), 1e-5)
    z = torch.tensor([-1e-4, 0.0, 1e-4], dtype=O.F64)         # the two branches meet at zero with slope 1/2
    close(O.xielu(z, 0.3, 0.9), 0.5 * z, 1e-7)


def test_layer_executions_of_a_loop():
    layers = [O.sink_layer() for _ in range(5)]
    for loop, runs in [(None, [0, 1, 2, 3, 4]), ((0, 5, 1), [0, 1, 2, 3, 4]), ((1, 3, 3), [0, 1, 2, 1, 2, 1, 2, 3, 4]),
                       ((3, 5, 2), [0, 1, 2, 3, 4, 3, 4]), ((2, 2, 4), [0, 1, 2, 3, 4]), ((4, 5, 2), [0, 1, 2, 3, 4, 4])]:
        cfg = O.make_config(layers, loop=loop)
        assert dimelix.read_config(cfg).layer_runs() == runs and O.layer_order(cfg) == runs
    cfg = O.make_config([O.side_layer(), O.latent_layer(), O.sink_layer()], loop=(0, 2, 2))
    eng = engine_for(cfg, O.random_weights(cfg, 1), torch.float32, "cpu")
    specs = eng.state_specs()                                # every execution has a cache / a state of its own
    assert sorted(specs) == [0, 1, 2, 3, 4] and [s[0] for s in specs[0]] == ["kv", "matrix"] and specs[0] == specs[2]
    assert [s[0] for s in specs[1]] == ["k"] and [s[0] for s in specs[4]] == ["kv"]
    assert dimelix.distance_slopes(4) == tuple(O.distance_slopes(4)) and O.distance_slopes(8)[-1] == 2.0 ** -8


# ------------------------------------------------------------------------------------------------ entry points
def _save_checkpoint(tmp_path, cfg, W):
    from safetensors.torch import save_file
    path = str(tmp_path / "model")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path


def _greedy_is_consistent(cfg, W, sequence, n_prompt):
    """every generated token is the oracle's argmax given what came before it, or within a rounding-sized gap of it"""
    logits = O.forward(sequence[:-1], W, cfg)
    for t in range(n_prompt, len(sequence)):
        row = logits[t - 1]
        assert float(row.max() - row[sequence[t]]) < 1e-3, f"token {t}"


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_auto_class_and_the_scheduler(device, tmp_path):
    from bigdl_amd.serving.continuous import ContinuousBatcher, SeqRequest
    from bigdl_amd.transformers import AutoModelForCausalLM
    cfg = full_model()
    W = O.random_weights(cfg, seed=61)
    path = _save_checkpoint(tmp_path, cfg, W)
    model = AutoModelForCausalLM.from_pretrained(path).to(device, torch.float32)
    prompts = torch.tensor([O.random_tokens(9, cfg["vocab"], 62), O.random_tokens(9, cfg["vocab"], 63)])
    out = model.generate(prompts, max_new_tokens=10)
    assert out.shape == (2, 19) and bool((out[:, :9] == prompts).all())
    for row in out.tolist():
        _greedy_is_consistent(cfg, W, row, 9)
    # more requests than slots, a pool that cannot hold them all at once, prompts longer than the per-step budget
    cb = ContinuousBatcher(model.engine, max_num_seqs=2, max_seq_len=128, max_prefill_tokens=24, max_live_tokens=192)
    reqs = [cb.submit(SeqRequest(str(i), O.random_tokens(n, cfg["vocab"], 70 + i), max_new_tokens=m))
            for i, (n, m) in enumerate([(70, 6), (3, 12), (30, 4), (1, 9), (50, 5)])]
    cb.run_until_done(500)
    assert all(r.finished and len(r.output_ids) == r.max_new_tokens for r in reqs)
    assert cb.mixed_steps > 0 and not cb.pool.len_of and len(cb.pool.free_pages) == cb.pool.num_pages
    for r in reqs:
        _greedy_is_consistent(cfg, W, r.input_ids + r.output_ids, len(r.input_ids))


def test_command_line_and_sampling(tmp_path, capsys):
    """``llm-cli --prompt-ids`` on a checkpoint without a tokenizer (greedy), and sampled generation through the same
    scheduler: with a fixed seed it repeats itself, and top_k = 1 is the greedy answer"""
    from bigdl_amd.cli import llm_cli
    from bigdl_amd.transformers import AutoModelForCausalLM
    cfg = O.make_config([O.side_layer(), O.latent_layer()], loop=(0, 2, 2))
    W = O.random_weights(cfg, seed=91)
    path = _save_checkpoint(tmp_path, cfg, W)
    prompt = O.random_tokens(11, cfg["vocab"], 92)
    model = AutoModelForCausalLM.from_pretrained(path).to("cpu", torch.float32)
    greedy = model.generate(torch.tensor([prompt]), max_new_tokens=7)[0].tolist()
    _greedy_is_consistent(cfg, W, greedy, len(prompt))
    assert model.generate(torch.tensor([prompt]), max_new_tokens=7, do_sample=True, top_k=1)[0].tolist() == greedy
    torch.manual_seed(3)
    a = model.generate(torch.tensor([prompt]), max_new_tokens=7, do_sample=True, temperature=1.5)[0].tolist()
    torch.manual_seed(3)
    assert model.generate(torch.tensor([prompt]), max_new_tokens=7, do_sample=True, temperature=1.5)[0].tolist() == a
    if torch.cuda.is_available():
        return                                               # (the command line would take the GPU: covered by the gpu tests)
    served = AutoModelForCausalLM.from_pretrained(path).to("cpu").generate(torch.tensor([prompt]), max_new_tokens=7)[0].tolist()
    llm_cli.main(["-m", path, "--prompt-ids", " ".join(map(str, prompt)), "-n", "7"])     # (the default type: bfloat16)
    assert capsys.readouterr().out.split()[-7:] == [str(t) for t in served[len(prompt):]]


def test_trace_runner_replays_steps(tmp_path):
    import subprocess
    import sys
    import numpy as np
    cfg = full_model()
    W = O.random_weights(cfg, seed=81)
    path = _save_checkpoint(tmp_path, cfg, W)
    toks = O.random_tokens(20, cfg["vocab"], 82)
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
    want = O.forward(toks, W, cfg)
    for step, rows in ((0, [0, 12]), (1, [2]), (2, [19])):
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4")).view(len(rows), -1).double()
        close(got, want[rows])


# ------------------------------------------------------------------------------------------------ kernels of long bfloat16 portions
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,e,window,sink,slope", [(4, 2, 64, 128, 100, True, False), (2, 2, 48, 48, 70, False, True),
                                                       (3, 1, 16, 32, 0, True, True), (8, 2, 128, 64, 64, False, True),
                                                       (2, 1, 32, 16, 1, True, False), (6, 3, 96, 80, 0, True, False),
                                                       (8, 4, 48, 48, 130, False, True)])
def test_matrix_core_attention_with_sinks_slopes_and_channel_gates(H, G, d, e, window, sink, slope):
    """bfloat16 prompt portions (the MFMA kernel) and single tokens (the row-wise kernel) against the plain statement on
    the same bfloat16-rounded keys, values and gate logits"""
    g = torch.Generator().manual_seed(71)
    T = 200
    q = torch.randn(T, H, d, generator=g).double()
    k = torch.randn(T, G, d, generator=g).bfloat16().double()
    v = torch.randn(T, G, e, generator=g).bfloat16().double()
    gate = (torch.randn(T, H * e, generator=g) * 2).bfloat16().double()
    sinks = [float(x) for x in torch.randn(H, generator=g) * 3] if sink else None
    slopes = O.distance_slopes(H) if slope else None
    qr = q.clone()
    qr[:190] = q[:190].bfloat16().double()                   # the MFMA kernel rounds its queries
    want = O.attend(qr, k, v, 2.0 * d ** -0.5, window=window, sinks=sinks, slopes=slopes) * torch.sigmoid(gate).view(T, H, e)
    got = _attend_through_pages("cuda", q, k, v, [120, 64, 3, 3] + [1] * 10, scale=2.0 * d ** -0.5, window=window, sinks=sinks,
                                slopes=slopes, gate=gate, dtype=torch.bfloat16)
    assert float((got - want).abs().max()) < 0.03, float((got - want).abs().max())
