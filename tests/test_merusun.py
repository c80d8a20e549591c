"""The Merusun design on the ragged engine against the plain float64 statement in ``merusun_oracle.py``.

Every test runs twice: on the CPU (the engine's bookkeeping over the unfused statements of ``ops/ragged.py``) and,
marked ``gpu``, on the device (the HIP kernels of ``libbigdl_ragged.so``).  Models are small and random; where random
weights would hide a fault (one far key among many, a window's edge, the sink) the inputs are made so that it shows.
"""
import json
import math
import os
import random

import pytest
import torch

import merusun_oracle as O
from bigdl_amd.models import merusun
from bigdl_amd.models.paged import PagedStatePool
from bigdl_amd.ops import ragged as R

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32_TOL = 3e-4


def engine_for(config, sd, dtype, device):
    return merusun.build_engine(merusun.read_config(config), sd, dtype, device)


def full_model():
    return O.make_config([O.attention_layer(), O.latent_layer(), O.attention_layer(kv_from=0, size=7),
                          O.mlstm_layer(), O.mlstm_layer(heads=1, dim=40, vdim=12, mlp=None),
                          O.latent_layer(heads=2, dim=8, rot_dim=4, vdim=8, rank=12, size=70, mlp=O.moe(6, 3, 16, 1, 1, 0.5, 0))])


def tokens(n, vocab, seed):
    rnd = random.Random(seed)
    return [rnd.randrange(vocab) for _ in range(n)]


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
@pytest.mark.parametrize("layers", [
    [O.attention_layer(mlp=None)],
    [O.attention_layer(heads=3, kv_heads=3, dim=24, vdim=80, size=None, scale=0.2, mlp=None)],
    [O.attention_layer(heads=6, kv_heads=1, dim=20, vdim=15, size=200, scale=-0.7, mlp=None)],
    [O.attention_layer(heads=8, kv_heads=1, dim=32, vdim=272, size=33, mlp=None), O.attention_layer(heads=8, kv_heads=1, dim=32, vdim=272, size=1, kv_from=0, mlp=None)],
    [O.latent_layer(mlp=None)],
    [O.latent_layer(heads=1, dim=10, rot_dim=6, vdim=7, rank=9, size=None, mlp=None)],
    [O.latent_layer(heads=4, dim=32, rot_dim=16, vdim=16, rank=64, size=66, mlp=None)],
    [O.latent_layer(heads=2, dim=16, rot_dim=32, vdim=24, rank=288, size=40, mlp=None)],
    [O.mlstm_layer(mlp=None)],
    [O.mlstm_layer(heads=1, dim=70, vdim=33, cap=2.0, mlp=None)],
    [O.mlstm_layer(heads=3, dim=8, vdim=130, cap=30.0, mlp=None)],
    [O.attention_layer(mlp=O.moe())],
    [O.attention_layer(mlp=O.moe(experts=12, top=1, ff=10, count=1, keep=1, scale=1.0, shared=0))],
    [O.attention_layer(mlp=O.moe(experts=66, top=5, ff=33, count=6, keep=6, scale=0.4, shared=7))],
    [O.attention_layer(mlp=O.moe(experts=70, top=4, ff=16, count=35, keep=3, scale=2.5, shared=16))],
], ids=["attention", "full-mask-wide-values", "one-kv-head-negative-scale", "very-wide-values-shared-cache-window-1",
        "latent", "latent-one-head-odd-sizes", "latent-rows-of-80", "latent-wide-rank", "mlstm", "mlstm-one-head-odd-sizes",
        "mlstm-wide-values", "experts", "one-expert-of-one-group-no-shared", "all-groups-kept-over-64-experts", "groups-of-two"])
def test_each_layer_kind_alone(device, layers):
    cfg = O.make_config(layers)
    sd = O.random_weights(cfg, seed=1)
    toks = tokens(85, cfg["vocab"], 2)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 45)], [("a", 38)], [("a", 1)], [("a", 1)]], 128)["a"]
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
def test_layer_outputs_one_by_one(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=3)
    toks = tokens(30, cfg["vocab"], 4)
    ref_layers = []
    O.forward(cfg, O.as_f64(sd), toks, ref_layers)
    eng = engine_for(cfg, sd, torch.float32, device)
    pool = eng.ensure_pool(64, 1)
    mine = []
    eng.step([(pool.admit(), toks)], collect=mine)
    assert len(mine) == len(ref_layers)
    for li, (a, b) in enumerate(zip(mine, ref_layers)):
        assert float((a.double().cpu() - b).abs().max()) < 1e-4, f"layer {li}"


@pytest.mark.parametrize("device", DEVICES)
def test_prompt_against_token_by_token_and_portions(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=5)
    toks = tokens(150, cfg["vocab"], 6)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.float32, device)
    close(run_schedule(eng, {"a": toks}, [[("a", 150)]], 192)["a"], want)
    close(run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in range(150)], 192)["a"], want)
    for sizes in ([2] * 75, [64, 2, 62, 3, 1, 1, 17], [63, 1, 1, 63, 2, 20], [5, 128, 2, 2, 13], [1, 2, 3, 4, 5, 64, 65, 6]):
        assert sum(sizes) == 150
        close(run_schedule(eng, {"a": toks}, [[("a", n)] for n in sizes], 192)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dense_rows", [0, 10 ** 9], ids=["experts-as-dense-products", "experts-row-by-row"])
def test_unequal_requests_in_one_batch_and_reuse_of_pages_and_slots(device, dense_rows):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=7)
    W = O.as_f64(sd)
    lens = {"a": 130, "b": 7, "c": 70, "d": 1, "e": 66, "f": 90}
    prompts = {k: tokens(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg, W, p) for k, p in prompts.items()}
    # three slots, pool of 5 pages (320 tokens) for 364 tokens in total: d, e, f run in what a, b, c gave back
    schedule = [[("a", 60), ("b", 2), ("c", 1)], [("a", 1), ("b", 5), ("c", 63)], [("a", 5), ("c", 6)],
                [("a", 64), ("d", 1)], [("e", 2), ("f", 30)], [("e", 64), ("f", 1)], [("f", 59)]]
    eng = engine_for(cfg, sd, torch.float32, device)
    eng.moe_dense_rows = dense_rows
    seen = {}
    got = run_schedule(eng, prompts, schedule, 320, slots=3, seen=seen)
    for k in prompts:
        close(got[k], want[k])
    old, new = ("a", "b", "c"), ("d", "e", "f")
    assert set().union(*(seen[k][0] for k in new)) & set().union(*(seen[k][0] for k in old)), "no page was used twice"
    assert set().union(*(seen[k][1] for k in new)) & set().union(*(seen[k][1] for k in old)), "no slot was used twice"
    # alone as inside the batch: the library's products sum in an order that depends on their row count, so the two
    # differ by rounding (each is within F32_TOL of the float64 statement)
    alone = run_schedule(eng, {"c": prompts["c"]}, [[("c", 70)]], 128)["c"]
    close(alone, got["c"], 2e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_long_and_short_portions_side_by_side_through_the_recurrence(device):
    """a portion long enough for the chunked scan next to a short one and a single token, then the long one goes on"""
    cfg = O.make_config([O.mlstm_layer(heads=2, dim=24, vdim=20), O.mlstm_layer(heads=1, dim=70, vdim=33, cap=4.0, mlp=None)])
    sd = O.random_weights(cfg, seed=17)
    W = O.as_f64(sd)
    prompts = {"a": tokens(1400, cfg["vocab"], 18), "b": tokens(41, cfg["vocab"], 19), "c": tokens(3, cfg["vocab"], 20)}
    want = {k: O.forward(cfg, W, p) for k, p in prompts.items()}
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, prompts, [[("c", 2), ("a", 700), ("b", 40)], [("a", 1), ("b", 1), ("c", 1)], [("a", 699)]], 1600)
    for k in prompts:
        close(got[k], want[k])


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_windows_and_pages(device):
    cfg = O.make_config([O.attention_layer(size=16), O.mlstm_layer(), O.latent_layer(size=70), O.attention_layer(size=66, kv_from=0)])
    sd = O.random_weights(cfg, seed=9)
    toks = tokens(200, cfg["vocab"], 11)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)] for _ in range(195)], 256)["a"]
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("odd", [False, True])
def test_bfloat16_stays_near_the_exact_result(device, odd):
    """(every row uses all of its experts here: a choice between two experts of nearly equal score is a jump that
    rounding may take either way, not an error of the arithmetic)"""
    all_experts = O.moe(experts=3, top=3, ff=24, count=1, keep=1, shared=40)
    if odd:          # sizes that take none of the vector or matrix-core paths
        layers = [O.attention_layer(heads=3, kv_heads=1, dim=20, vdim=30), O.latent_layer(heads=1, dim=10, rot_dim=6, vdim=7, rank=9),
                  O.mlstm_layer(heads=1, dim=36, vdim=20), O.attention_layer(heads=3, kv_heads=1, dim=20, vdim=30, kv_from=0)]
    else:            # sizes that the vector and matrix-core paths serve
        layers = [O.attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, size=40),
                  O.latent_layer(heads=4, dim=32, rot_dim=16, vdim=16, rank=64, size=66), O.mlstm_layer(heads=2, dim=32, vdim=64),
                  O.attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, size=70, kv_from=0)]
    for layer in layers:
        layer["mlp"] = all_experts
    cfg = O.make_config(layers)
    sd = O.random_weights(cfg, seed=13)
    toks = tokens(100, cfg["vocab"], 14)
    want = O.forward(cfg, O.as_f64(sd), toks)
    eng = engine_for(cfg, sd, torch.bfloat16, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 70)], [("a", 2)]] + [[("a", 1)] for _ in range(28)], 128)["a"]
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    rel = d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    # (single rows may sit where the recurrence's normaliser is small and rounding is amplified: the bound is on most rows)
    assert float(rel.median()) < 0.05 and float(rel.quantile(0.9)) < 0.15, (float(rel.median()), float(rel.quantile(0.9)))


# ------------------------------------------------------------------------------------------------ mechanisms alone
def _meta_for(pool, slot, n, device):
    pages = list(pool.reserve(slot, n))
    return R.BatchMeta([(slot, pool.len_of[slot], n, pages)], torch.device(device))


def _attend_through_pages(device, q, k, v, portions, *, window, scale, sink, page_order=None, dtype=torch.float32):
    """q [T, H, d], k [T, G, d] (float64) through the paged attention op in the given portions.  v [T, G, e], or None:
    the values are then the leading e = ``v_lead`` channels of the key rows, read from the key pages"""
    T, H, d = q.shape
    G = k.shape[1]
    shared = isinstance(v, int)
    e = v if shared else v.shape[2]
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("k", G, d)] if shared else [("kv", G, d, e)]}, 64 * ((T + 63) // 64 + 2), 2, dtype, device)
    if page_order:
        pool.free_pages = list(page_order)
    slot = pool.admit()
    out, at = [], 0
    for n in portions:
        meta = _meta_for(pool, slot, n, device)
        for i in range(n):                                   # place keys / values as the cache holds them
            pos = at + i
            pg = pool.pages_of[slot][pos // 64]
            pool.k[0][pg, :, pos % 64] = k[pos].to(dtype).to(device)
            if not shared:
                pool.v[0][pg, :, pos % 64] = v[pos].to(dtype).to(device)
        qq = q[at:at + n].reshape(n, H * d).float().to(device).contiguous()
        out.append(ops.paged_attn(qq, pool.k[0], pool.k[0] if shared else pool.v[0], meta, maps=1, H=H, G=G, d=d, vd=e,
                                  window=window, keep_first=0, scale=scale, lam=0.0, out_scale=1.0, out_norm=False, eps=1e-6,
                                  sink=sink))
        pool.commit(slot, n)
        at += n
    return torch.cat(out).double().cpu().view(T, H, e)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode_tail", [0, 12])
@pytest.mark.parametrize("shared_rows", [False, True], ids=["sink-attention", "values-inside-the-key-rows"])
def test_window_edges_far_keys_and_page_borders_stand_out(device, decode_tail, shared_rows):
    """Query i and key j are made parallel and long, so key j takes all of the weight when it is visible; its value is
    a marker.  One position off in the window or at a page's border swaps the marker in or out."""
    g = torch.Generator().manual_seed(21)
    T, H, G, d, e, window = 210, 2, 1, 12, 4, 70
    sink = None if shared_rows else 0.0
    cases = []                                               # (query position, key position)
    for i in (140, 191, 192, 193, 209):
        cases += [(i, i - window + 1), (i, i - window), (i, i), (i, 0)]
    cases += [(100, 63), (100, 64), (130, 127), (130, 128), (64, 63), (64, 64), (69, 0), (70, 0), (70, 1), (0, 0), (1, 0)]
    for i, j in cases:
        q = torch.randn(T, H, d, generator=g, dtype=O.F64) * 0.1
        k = torch.randn(T, G, d, generator=g, dtype=O.F64) * 0.1
        u = torch.randn(d - e, generator=g, dtype=O.F64)
        u = u / u.norm()
        q[i, :, e:], k[j, :, e:] = 8.0 * u, 8.0 * u          # score 64 where everything else is ~0
        k[j, :, :e] = 5.0                                     # (the marker, when the values are the rows' first channels)
        v = k[:, :, :e].clone()
        if not shared_rows:
            v = torch.randn(T, G, e, generator=g, dtype=O.F64) * 0.1
            v[j] = 5.0
        js = [x for x in range(T) if O.visible(i, x, window)]
        want = torch.stack([O.sink_attend(q[i, hh], k[js, 0], v[js, 0], 1.0, 0.0) if not shared_rows else
                            torch.softmax(k[js, 0] @ q[i, hh], 0) @ v[js, 0] for hh in range(H)])
        assert (float(want.abs().max()) > 3.0) == O.visible(i, j, window)
        portions = [T] if not decode_tail else [T - decode_tail - 40, 40] + [1] * decode_tail
        if decode_tail and i < T - decode_tail:
            continue                                         # this case's query is not a decoded token
        got = _attend_through_pages(device, q, k, e if shared_rows else v, portions, window=window, scale=1.0, sink=sink,
                                    page_order=[1, 4, 0, 3, 2, 5][::-1])
        close(got[i], want, 1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_the_sink_takes_weight_and_gives_no_value(device):
    """all scores far below the sink's: the output nearly vanishes; all far above: an ordinary softmax; one key at the
    sink's own score: exactly half of its value"""
    T, H, d, e = 70, 2, 8, 6
    g = torch.Generator().manual_seed(5)
    k = torch.randn(T, 1, d, generator=g, dtype=O.F64)
    v = torch.randn(T, 1, e, generator=g, dtype=O.F64)
    q = torch.randn(T, H, d, generator=g, dtype=O.F64)
    for scale, sink in ((1.0, 0.0), (1.0, 40.0), (1.0, -40.0), (0.0, 0.0), (3.0, 2.5)):
        want = torch.zeros(T, H, e, dtype=O.F64)
        for i in range(T):
            js = [x for x in range(T) if O.visible(i, x, 9)]
            for hh in range(H):
                want[i, hh] = O.sink_attend(q[i, hh], k[js, 0], v[js, 0], scale, sink)
        got = _attend_through_pages(device, q, k, v, [50, 1, 1, 18], window=9, scale=scale, sink=sink)
        close(got, want, 1e-4)
    got = _attend_through_pages(device, q[:1] * 0, k[:1], v[:1], [1], window=9, scale=1.0, sink=0.0)
    close(got[0, 0], 0.5 * v[0, 0], 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,dim,vdim,cap,portions", [(2, 16, 16, 6.0, (1, 2, 64, 1, 22)), (1, 40, 24, 15.0, (1, 2, 64, 1, 22)),
                                                         (3, 64, 70, 3.0, (90,)), (2, 130, 8, 8.0, (1, 1, 1, 87)),
                                                         (1, 32, 64, 5.0, (600, 3, 1, 520))])
def test_mlstm_recurrence_and_its_state(device, heads, dim, vdim, cap, portions):
    """gates, running maximum, normaliser, matrix memory and the gated head norm against the recurrence written out; a
    used slot is handed to a second sequence, which must start from nothing"""
    g = torch.Generator().manual_seed(31)
    T, H, d, e = sum(portions), heads, dim, vdim
    D = 32
    m = {"heads": H, "dim": d, "vdim": e, "gate_cap": cap}
    W = {"q": torch.randn(H * d, D, generator=g), "k": torch.randn(H * d, D, generator=g), "v": torch.randn(H * e, D, generator=g),
         "g": torch.randn(H * e, D, generator=g), "i": torch.randn(H, D, generator=g) * 1.5, "f": torch.randn(H, D, generator=g) * 1.5,
         "i.b": torch.randn(H, generator=g), "f.b": torch.randn(H, generator=g) + 2.0, "norm": torch.randn(H * e, generator=g),
         "o": torch.eye(H * e)}
    W = {k: v.double() for k, v in W.items()}
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("matrix", H, d, e + 1), ("vector", H)]}, 64 * 40, 1, torch.float32, device)
    gate_bias = torch.cat([W["i.b"], W["f.b"]]).float().to(device)
    wcat = torch.cat([W["q"], W["k"], W["v"], W["g"], W["i"], W["f"]])
    for seq in range(2):
        h = torch.randn(T, D, generator=g, dtype=O.F64) * 0.5
        want = O.mlstm_mixer(h, W, "", m, 1e-5)
        P = (h @ wcat.T).float().to(device).contiguous()
        slot = pool.admit()
        out, at = [], 0
        for n in portions:
            meta = _meta_for(pool, slot, n, device)
            Pn = P[at:at + n].contiguous()
            a, b, em = ops.mlstm_gates(Pn, 2 * H * d + 2 * H * e, gate_bias, cap, 0.0, H, pool.vector[0], meta)
            qf, ff, gf = ops.mlstm_expand(Pn, 0, H * d, a, b, H, d)
            o = ops.hgrn2_scan(qf, ff, Pn, 2 * H * d, pool.matrix[0], H, d, e + 1, meta, gf=gf, ones_col=True)
            out.append(ops.head_norm_gate(o, W["norm"].float().to(device), Pn, 2 * H * d + H * e, H, e, 1e-5, torch.float32,
                                          em=em, den_floor=1e-6))
            pool.commit(slot, n)
            at += n
        close(torch.cat(out).double().cpu(), want, 2e-4)
        pool.release(slot)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("experts,top,count,keep", [(8, 2, 4, 2), (16, 3, 2, 1), (12, 1, 1, 1), (70, 6, 7, 7), (96, 4, 48, 5), (130, 8, 5, 2)])
def test_router_and_expert_rows(device, experts, top, count, keep):
    g = torch.Generator().manual_seed(41)
    T, D, ff = 37, 48, 20
    ops = R.ops_for(device)
    x = torch.randn(T, D, generator=g)
    wr = torch.randn(experts, D, generator=g) * 0.4
    up, dn = torch.randn(experts, ff, D, generator=g) * 0.2, torch.randn(experts, D, ff, generator=g) * 0.2
    base = torch.randn(T, D, generator=g)
    idx, wts = ops.moe_route(x.to(device), wr.to(device), count, keep, top, 1.3)
    y = ops.moe_rows(x.to(device), idx, wts, up.to(device), dn.to(device), base.to(device)).double().cpu()
    idx, wts = idx.cpu(), wts.double().cpu()
    for t in range(T):
        s = torch.softmax(wr.double() @ x[t].double(), 0)
        want = O.choose(s, count, keep, top)
        assert sorted(idx[t].tolist()) == sorted(want), f"row {t}"
        ref = base[t].double()
        for j, e in enumerate(idx[t].tolist()):
            assert abs(float(wts[t, j]) - 1.3 * float(s[e])) < 1e-5
            ref = ref + 1.3 * s[e] * O.expert(x[t].double(), up[e].double(), dn[e].double())
        close(y[t], ref, 1e-4)
    close(ops.relu2(x.to(device)).double().cpu(), torch.relu(x.double()).pow(2), 1e-6)


@pytest.mark.parametrize("device", DEVICES)
def test_norm_behind_a_sublayer_and_in_front_of_the_next(device):
    g = torch.Generator().manual_seed(51)
    ops = R.ops_for(device)
    for rows, D in ((5, 64), (3, 200), (2, 1030)):
        x = torch.randn(rows, D, generator=g)
        y = torch.randn(rows, D, generator=g) * 3
        wp, wn = torch.randn(D, generator=g), torch.randn(D, generator=g)
        want_x = x.double() + O.norm(y.double(), wp.double(), 1e-5)
        xd = x.clone().to(device)
        xa = ops.post_norm_add(xd, y.to(device), wp.to(device), wn.to(device), 1e-5, torch.float32)
        close(xd.double().cpu(), want_x, 1e-5)
        close(xa.double().cpu(), O.norm(want_x, wn.double(), 1e-5), 1e-5)
        xd = x.clone().to(device)
        assert ops.post_norm_add(xd, y.to(device), wp.to(device), None, 1e-5, torch.float32) is None
        close(xd.double().cpu(), want_x, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_latent_rows_norm_part_of_the_row_and_turn_neighbouring_pairs(device):
    """the cached row of the latent attention: leading channels normed with a weight, trailing ones turned by position"""
    g = torch.Generator().manual_seed(61)
    R_, r, T = 20, 6, 70
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("k", 1, R_ + r)]}, 128, 1, torch.float32, device)
    slot = pool.admit()
    P = torch.randn(T, 5 + R_ + r, generator=g)
    w = torch.randn(R_, generator=g)
    inv = torch.tensor([50.0 ** (-2.0 * i / r) for i in range(r // 2)], dtype=torch.float32).to(device)
    at = 0
    for n in (3, 1, 62, 4):
        meta = _meta_for(pool, slot, n, device)
        ops.conv_head(P[at:at + n].contiguous().to(device), 5, meta, cw=None, taps=0, C=0, ch0=0, state=None, ngroups=1,
                      gsize=R_ + r, normw=w.to(device), norm_n=R_, eps=1e-5, rot=r, rot0=R_, interleaved=True, inv_freq=inv,
                      pages=pool.k[0])
        pool.commit(slot, n)
        at += n
    for t in (0, 1, 3, 4, 63, 64, 69):
        row = pool.k[0][pool.pages_of[slot][t // 64], 0, t % 64].double().cpu()
        close(row[:R_], O.norm(P[t, 5:5 + R_].double(), w.double(), 1e-5), 1e-5)
        close(row[R_:], O.turn_pairs(P[t, 5 + R_:].double(), t, r, 50.0), 1e-5)


# ------------------------------------------------------------------------------------------------ entry points
def _save_checkpoint(tmp_path, cfg, sd):
    from safetensors.torch import save_file
    path = str(tmp_path / "model")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    return path


def _greedy_is_consistent(cfg, W, sequence, n_prompt):
    """every generated token is the oracle's argmax given what came before it, or within a rounding-sized gap of it"""
    logits = O.forward(cfg, W, sequence[:-1])
    for t in range(n_prompt, len(sequence)):
        row = logits[t - 1]
        assert float(row.max() - row[sequence[t]]) < 1e-3, f"token {t}"


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_auto_class_and_the_scheduler(device, tmp_path):
    from bigdl_amd.serving.continuous import ContinuousBatcher, SeqRequest
    from bigdl_amd.transformers import AutoModelForCausalLM
    cfg = full_model()
    sd = O.random_weights(cfg, seed=61)
    W = O.as_f64(sd)
    path = _save_checkpoint(tmp_path, cfg, sd)
    model = AutoModelForCausalLM.from_pretrained(path).to(device, torch.float32)
    prompts = torch.tensor([tokens(9, cfg["vocab"], 62), tokens(9, cfg["vocab"], 63)])
    out = model.generate(prompts, max_new_tokens=10)
    assert out.shape == (2, 19) and bool((out[:, :9] == prompts).all())
    for row in out.tolist():
        _greedy_is_consistent(cfg, W, row, 9)
    # more requests than slots, a pool that cannot hold them all at once, prompts longer than the per-step budget
    cb = ContinuousBatcher(model.engine, max_num_seqs=2, max_seq_len=128, max_prefill_tokens=24, max_live_tokens=192)
    reqs = [cb.submit(SeqRequest(str(i), tokens(n, cfg["vocab"], 70 + i), max_new_tokens=m))
            for i, (n, m) in enumerate([(70, 6), (3, 12), (30, 4), (1, 9), (50, 5)])]
    cb.run_until_done(500)
    assert all(r.finished and len(r.output_ids) == r.max_new_tokens for r in reqs)
    assert cb.mixed_steps > 0 and not cb.pool.len_of and len(cb.pool.free_pages) == cb.pool.num_pages
    for r in reqs:
        _greedy_is_consistent(cfg, W, r.input_ids + r.output_ids, len(r.input_ids))


def test_trace_runner_replays_steps(tmp_path):
    import subprocess
    import sys
    import numpy as np
    cfg = full_model()
    sd = O.random_weights(cfg, seed=81)
    path = _save_checkpoint(tmp_path, cfg, sd)
    toks = tokens(20, cfg["vocab"], 82)
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
    want = O.forward(cfg, O.as_f64(sd), toks)
    for step, rows in ((0, [0, 12]), (1, [2]), (2, [19])):
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4")).view(len(rows), -1).double()
        close(got, want[rows])


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,e,window,sink,shared", [(4, 2, 64, 128, 100, 0.0, False), (2, 2, 48, 96, 70, 1.5, False),
                                                       (3, 1, 16, 32, 0, -2.0, False), (4, 1, 80, 64, 66, None, True),
                                                       (2, 1, 128, 112, 300, None, True), (4, 1, 144, 128, 66, None, True),
                                                       (2, 1, 576, 512, 100, None, True), (2, 2, 200, 192, 0, 1.0, False),
                                                       (3, 1, 328, 256, 130, None, True)])
def test_matrix_core_attention_with_a_sink_and_with_values_inside_the_key_rows(H, G, d, e, window, sink, shared):
    """bfloat16 prompt portions (the MFMA kernel) and single tokens (the row-wise kernel) against the plain statement on
    the same bfloat16-rounded keys and values"""
    g = torch.Generator().manual_seed(71)
    T = 200
    q = torch.randn(T, H, d, generator=g).double()
    k = torch.randn(T, G, d, generator=g).bfloat16().double()
    v = k[:, :, :e].clone() if shared else torch.randn(T, G, e, generator=g).bfloat16().double()
    scale = d ** -0.5
    want = torch.zeros(T, H, e, dtype=O.F64)
    for i in range(T):
        js = [x for x in range(T) if O.visible(i, x, window)]
        for hh in range(H):
            gg = hh // (H // G)
            # the MFMA kernels round their queries; rows wider than 128 channels take them for single tokens too
            qq = q[i, hh].bfloat16().double() if i < 190 or d > 128 else q[i, hh]
            want[i, hh] = (torch.softmax((k[js, gg] @ qq) * scale, 0) @ v[js, gg]) if sink is None else \
                O.sink_attend(qq, k[js, gg], v[js, gg], scale, sink)
    got = _attend_through_pages("cuda", q, k, e if shared else v, [120, 64, 3, 3] + [1] * 10, window=window, scale=scale, sink=sink,
                                dtype=torch.bfloat16)
    assert float((got - want).abs().max()) < 0.03, float((got - want).abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("T,D,ff,experts,top,count,keep", [(300, 64, 48, 10, 3, 5, 2), (1000, 256, 112, 64, 6, 8, 4), (70, 80, 16, 3, 3, 1, 1),
                                                         (129, 128, 128, 40, 1, 1, 1)])
def test_grouped_expert_product_on_sorted_rows(T, D, ff, experts, top, count, keep):
    """bfloat16 long portions: every expert's run of sorted rows through the grouped matrix-core product, against float64
    on the same bfloat16 inputs and against the row-wise kernels"""
    g = torch.Generator().manual_seed(91)
    ops = R.ops_for("cuda")
    x = (torch.randn(T + 3, D + 8, generator=g)).bfloat16().cuda()[3:, :D]                    # rows with a stride of their own
    x = x if x.stride(0) % 8 == 0 else x.contiguous()
    wr = (torch.randn(experts, D, generator=g) * 0.4).cuda()
    up = (torch.randn(experts, ff, D, generator=g) * 0.2).bfloat16().cuda()
    dn = (torch.randn(experts, D, ff, generator=g) * 0.2).bfloat16().cuda()
    base = torch.randn(T, D, generator=g).bfloat16().cuda()
    idx, wts = ops.moe_route(x, wr, count, keep, top, 1.3)
    got = ops.moe_sorted(x, idx, wts, up, dn, base)
    assert got is not None
    assert ops.moe_sorted(x[:, :D - 4].contiguous(), idx, wts, up[:, :, :D - 4].contiguous(), dn[:, :D - 4].contiguous(), None) is None
    rows = ops.moe_rows(x, idx, wts, up, dn, base)
    ref = base.double().cpu()
    xd, upd, dnd = x.double().cpu(), up.double().cpu(), dn.double().cpu()
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            a = torch.relu(upd[e] @ xd[t]).pow(2).bfloat16().double()
            ref[t] += float(wts[t, j]) * (dnd[e] @ a).bfloat16().double()
    scale = float(ref.abs().max())
    assert float((got.double().cpu() - ref).abs().max()) < 0.02 * scale
    assert float((rows.double().cpu() - ref).abs().max()) < 0.02 * scale
