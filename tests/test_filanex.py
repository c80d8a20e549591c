"""The Filanex design on the ragged engine against the plain float64 statement in ``filanex_oracle.py``.

Every test runs twice: on the CPU (the engine's bookkeeping over the unfused statements of ``ops/ragged.py``) and,
marked ``gpu``, on the device (the HIP kernels of ``libbigdl_ragged.so``).  Models are small and random; where random
weights would hide a fault (one key among many, a block's edge, a page's border) the inputs are made so that it shows.
"""
import json
import math
import os
import random

import pytest
import torch

import filanex_oracle as O
from bigdl_amd.models import filanex
from bigdl_amd.models.paged import PagedStatePool
from bigdl_amd.models.ragged_engine import PairEmbedding, yarn_inv_freq
from bigdl_amd.ops import ragged as R

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F32_TOL = 3e-4


def engine_for(config, sd, dtype, device):
    return filanex.build_engine(filanex.read_config(config), sd, dtype, device)


def full_model():
    """dense, expert and no feed-forward; blocks of 24, 7 and 70 positions; layers 1 .. 3 run twice"""
    return O.make_config([O.attention_layer(), O.attention_layer(mlp=O.moe()), O.attention_layer(mlp=None, size=7),
                          O.attention_layer(heads=3, kv_heads=3, dim=10, vdim=6, size=70, rot=(10, 100.0, None), mlp=O.moe(4, 1, 8, 1, 1)),
                          O.attention_layer(heads=2, kv_heads=1, dim=24, vdim=40, size=None, cap=None, rot=None)], loop=(1, 4, 2))


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
@pytest.mark.parametrize("layers,loop,pairs", [
    ([O.attention_layer()], None, None),
    ([O.attention_layer(mlp=O.moe())], None, (37, 11, 5)),
    ([O.attention_layer(mlp=None)], (0, 1, 3), (1, 1, 1)),                       # one bucket: every pair shares a row
    ([O.attention_layer(heads=1, kv_heads=1, dim=8, vdim=12, size=1, rot=(8, 7.0, (2.0, 16, 3.0, 1.0)))], (0, 1, 1), (80, 3, 1)),
    ([O.attention_layer(heads=6, kv_heads=2, dim=12, vdim=10, size=64, rot=(4, 1e4, (8.0, 4096, 32.0, 1.0)), mlp=O.moe(8, 3, 10, 8, 3))],
     None, (7, 5, 3)),                                                         # groups of one expert
    ([O.attention_layer(size=None, cap=None, rot=(16, 50.0, (1.5, 20, 2.0, 1.0)), mlp=O.moe(70, 5, 6, 7, 7))], (0, 1, 2), None),
    ([O.attention_layer(heads=2, kv_heads=1, dim=40, vdim=136, size=100, mlp=O.moe(12, 4, 18, 2, 1))], None, (500, 131, 9)),
])
def test_each_layer_kind_alone(device, layers, loop, pairs):
    cfg = O.make_config(layers, loop=loop, pairs=pairs)
    sd = O.random_weights(cfg, seed=1)
    toks = tokens(90, cfg["vocab"], 2)
    want = O.forward(toks, O.as_f64(sd), cfg)
    eng = engine_for(cfg, sd, torch.float32, device)
    close(run_schedule(eng, {"a": toks}, [[("a", 60)], [("a", 2)]] + [[("a", 1)] for _ in range(28)], 128)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_layer_outputs_one_by_one(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=3)
    toks = tokens(40, cfg["vocab"], 4)
    want = []
    O.forward(toks, O.as_f64(sd), cfg, collect=want)
    assert len(want) == 1 + 2 * 3 + 1
    eng = engine_for(cfg, sd, torch.float32, device)
    pool = eng.ensure_pool(64, 1)
    got = []
    eng.step([(pool.admit(), toks)], collect=got)
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        err = float((a.double().cpu() - b).abs().max())
        assert err < 2e-4, f"layer execution {i}: {err}"


@pytest.mark.parametrize("device", DEVICES)
def test_prompt_against_token_by_token_and_portions(device):
    cfg = full_model()
    sd = O.random_weights(cfg, seed=5)
    toks = tokens(150, cfg["vocab"], 6)
    want = O.forward(toks, O.as_f64(sd), cfg)
    eng = engine_for(cfg, sd, torch.float32, device)
    close(run_schedule(eng, {"a": toks}, [[("a", 150)]], 192)["a"], want)
    close(run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in range(150)], 192)["a"], want)
    for sizes in ([2] * 75, [64, 2, 62, 3, 1, 1, 17], [63, 1, 1, 63, 2, 20], [5, 128, 2, 2, 13], [1, 2, 3, 4, 5, 64, 65, 6],
                  [23, 1, 24, 2, 20, 6, 74]):
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
    want = {k: O.forward(p, W, cfg) for k, p in prompts.items()}
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
def test_long_decoding_past_blocks_and_pages(device):
    cfg = O.make_config([O.attention_layer(size=16), O.attention_layer(size=70, mlp=O.moe()), O.attention_layer(size=64, mlp=None),
                         O.attention_layer(size=None)], loop=(0, 2, 2))
    sd = O.random_weights(cfg, seed=9)
    toks = tokens(200, cfg["vocab"], 11)
    want = O.forward(toks, O.as_f64(sd), cfg)
    eng = engine_for(cfg, sd, torch.float32, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)] for _ in range(195)], 256)["a"]
    close(got, want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("odd", [False, True])
def test_bfloat16_stays_near_the_exact_result(device, odd):
    """(every row uses all of its experts here: a choice between two experts of nearly equal score is a jump that
    rounding may take either way, not an error of the arithmetic)"""
    every = O.moe(experts=3, top=3, ff=24, count=1, keep=1)
    if odd:          # sizes that take none of the vector or matrix-core paths
        layers = [O.attention_layer(heads=3, kv_heads=1, dim=20, vdim=30, rot=(6, 90.0, None)), O.attention_layer(mlp=every, dim=18, vdim=14)]
    else:            # sizes that the vector and matrix-core paths serve
        layers = [O.attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, size=40),
                  O.attention_layer(heads=4, kv_heads=1, dim=64, vdim=48, size=66, mlp=O.moe(3, 3, 32, 1, 1))]
    cfg = O.make_config(layers, width=64, loop=(0, 2, 2))
    sd = O.random_weights(cfg, seed=13)
    toks = tokens(100, cfg["vocab"], 14)
    want = O.forward(toks, O.as_f64(sd), cfg)
    eng = engine_for(cfg, sd, torch.bfloat16, device)
    got = run_schedule(eng, {"a": toks}, [[("a", 70)], [("a", 2)]] + [[("a", 1)] for _ in range(28)], 128)["a"]
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    rel = d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    assert float(rel.median()) < 0.05 and float(rel.max()) < 0.15, (float(rel.median()), float(rel.max()))


# ------------------------------------------------------------------------------------------------ mechanisms alone
def _meta_for(pool, slot, n, device):
    pages = list(pool.reserve(slot, n))
    return R.BatchMeta([(slot, pool.len_of[slot], n, pages)], torch.device(device))


def _attend_through_pages(device, q, k, v, portions, *, chunk, scale, cap, gate=None, page_order=None, dtype=torch.float32):
    """q [T, H, d], k [T, G, d], v [T, G, e] (float64) through the paged attention op in the given portions; gate
    [T, H * e]: logits of a gate per output channel"""
    T, H, d = q.shape
    G, e = k.shape[1], v.shape[2]
    ops = R.ops_for(device)
    pool = PagedStatePool({0: [("kv", G, d, e)]}, 64 * ((T + 63) // 64 + 2), 2, dtype, device)
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
            pool.v[0][pg, :, pos % 64] = v[pos].to(dtype).to(device)
        qq = q[at:at + n].reshape(n, H * d).float().to(device).contiguous()
        gg = None if gate is None else torch.cat([torch.zeros(n, 8), gate[at:at + n].float()], 1).to(dtype).to(device)
        out.append(ops.paged_attn(qq, pool.k[0], pool.v[0], meta, maps=1, H=H, G=G, d=d, vd=e, window=0, keep_first=0, scale=scale,
                                  lam=0.0, out_scale=1.0, out_norm=False, eps=1e-6, chunk=chunk, softcap=cap or 0.0,
                                  gate=gg, gate0=8, gate_wide=gate is not None))
        pool.commit(slot, n)
        at += n
    return torch.cat(out).double().cpu().view(T, H, e)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode_tail", [0, 12])
@pytest.mark.parametrize("chunk,cap", [(70, None), (64, 25.0), (16, None), (128, 30.0), (1, None), (500, 40.0)])
def test_block_edges_far_keys_and_page_borders_stand_out(device, decode_tail, chunk, cap):
    """Query i and key j are made parallel and long, so key j takes all of the weight when it is visible; its value is
    a marker.  One position off at a block's edge or at a page's border swaps the marker in or out."""
    g = torch.Generator().manual_seed(21)
    T, H, G, d, e = 210, 2, 1, 12, 4
    cases = []                                               # (query position, key position)
    for i in (140, 191, 192, 193, 209, 69, 70, 127, 128):
        c0 = i - i % chunk
        cases += [(i, c0), (i, c0 - 1), (i, c0 + 1), (i, i), (i, 0), (i, i - 1)]
    cases += [(100, 63), (100, 64), (130, 127), (130, 128), (64, 63), (64, 64), (0, 0), (1, 0), (15, 0), (16, 0), (16, 15)]
    cases = [(i, j) for i, j in cases if 0 <= j <= i]
    for i, j in cases:
        q = torch.randn(T, H, d, generator=g).double() * 0.3
        k = torch.randn(T, G, d, generator=g).double() * 0.3
        v = torch.randn(T, G, e, generator=g).double()
        direction = torch.randn(d, generator=g).double()
        direction /= direction.norm()
        q[i, :] = 8.0 * direction
        k[j, 0] = 8.0 * direction
        v[j, 0] = torch.tensor([100.0, -100.0, 50.0, 25.0], dtype=O.F64)
        want = O.attend(q, k, v, 1.0, cap, chunk)
        head = T - decode_tail
        portions = [head // 3, head - head // 3] + [1] * decode_tail if i >= T - decode_tail or decode_tail == 0 else \
            [i + 1, head - i - 1] + [1] * decode_tail
        got = _attend_through_pages(device, q, k, v, [n for n in portions if n], chunk=chunk, scale=1.0, cap=cap,
                                    page_order=[5, 0, 3, 1, 4, 2])
        close(got[i], want[i], 2e-3)
        close(got, want, 2e-3)


@pytest.mark.parametrize("device", DEVICES)
def test_scores_are_capped_and_gates_act_on_every_channel(device):
    """scores far beyond the cap: without it the softmax would be one-hot, with it the weights stay spread; the gate of
    every channel is its own"""
    g = torch.Generator().manual_seed(23)
    T, H, G, d, e = 90, 4, 2, 16, 8
    q, k = torch.randn(T, H, d, generator=g).double() * 3, torch.randn(T, G, d, generator=g).double() * 3
    v = torch.randn(T, G, e, generator=g).double()
    gate = torch.randn(T, H * e, generator=g).double() * 3
    for cap in (2.0, 11.0, None):
        want = O.attend(q, k, v, 0.7, cap, 40) * torch.sigmoid(gate).view(T, H, e)
        got = _attend_through_pages(device, q, k, v, [50, 30] + [1] * 10, chunk=40, scale=0.7, cap=cap, gate=gate)
        close(got, want, 1e-4)
    assert float((O.attend(q, k, v, 0.7, 2.0, 40) - O.attend(q, k, v, 0.7, None, 40)).abs().max()) > 0.5


@pytest.mark.parametrize("device", DEVICES)
def test_pairs_turn_with_stretched_frequencies(device):
    """frequencies and amplitude against the plain statement for several scalings (ramp inside, below and above the
    pairs; no ramp width), then the turn of neighbouring channels of queries written densely and keys written to pages"""
    for rot in [(8, 500.0, (3.0, 64, 4.0, 0.5)), (16, 10000.0, (8.0, 4096, 32.0, 1.0)), (4, 7.0, (2.0, 16, 3.0, 1.0)),
                (12, 100.0, (4.0, 8, 0.001, 0.0001)), (6, 50.0, (1.5, 10 ** 6, 1.0, 1.0)), (32, 2e4, (40.0, 2048, 1.0, 1.0))]:
        spec = {"dims": rot[0], "base": rot[1], "scaling": dict(zip(("factor", "original", "fast", "slow"), rot[2]))}
        want_f, want_amp = O.pair_frequencies(spec)
        got_f, got_amp = yarn_inv_freq(rot[0], rot[1], *rot[2])
        assert abs(got_amp - want_amp) < 1e-12
        assert all(abs(float(a) - b) <= 1e-6 * b for a, b in zip(got_f, want_f))
    g = torch.Generator().manual_seed(25)
    ops = R.ops_for(device)
    n, heads, dim, dims = 70, 3, 14, 8
    freqs, amp = O.pair_frequencies({"dims": dims, "base": 300.0, "scaling": {"factor": 5.0, "original": 32, "fast": 4.0, "slow": 0.5}})
    P = torch.randn(n, heads * dim + 5, generator=g)
    pool = PagedStatePool({0: [("kv", heads, dim, 2)]}, 256, 1, torch.float32, device)
    slot = pool.admit()
    pool.reserve(slot, 100)
    pool.commit(slot, 100)                                   # the rows continue a sequence of 100 tokens
    meta = _meta_for(pool, slot, n, device)
    dense = torch.zeros(n, heads * dim, device=device)
    args = dict(cw=None, taps=0, C=0, ch0=0, state=None, ngroups=heads, gsize=dim, normw=None, eps=1e-6, rot=dims,
                inv_freq=torch.tensor(freqs, dtype=torch.float32, device=device), interleaved=True, rot_amp=amp)
    ops.conv_head(P.to(device), 5, meta, out_dense=dense, **args)
    ops.conv_head(P.to(device), 5, meta, pages=pool.k[0], **args)
    for t in (0, 1, 27, 28, 69):
        want = O.turn_neighbours(P[t, 5:].double().view(heads, dim), 100 + t, freqs, amp)
        close(dense[t].double().cpu().view(heads, dim), want, 2e-4)
        pos = 100 + t
        close(pool.k[0][pool.pages_of[slot][pos // 64], :, pos % 64].double().cpu(), want, 2e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("experts,top,count,keep", [(8, 2, 4, 2), (16, 3, 2, 1), (12, 1, 1, 1), (70, 6, 7, 7), (96, 4, 48, 5), (130, 8, 5, 2),
                                                    (6, 3, 6, 4), (9, 2, 3, 3)])
def test_router_and_gated_expert_rows(device, experts, top, count, keep):
    g = torch.Generator().manual_seed(41)
    T, D, ff = 37, 48, 20
    ops = R.ops_for(device)
    x = torch.randn(T, D, generator=g)
    W = {"router": torch.randn(experts, D, generator=g).double() * 0.4}
    for e in range(experts):
        W[f"e{e}.gate"], W[f"e{e}.up"] = torch.randn(ff, D, generator=g).double() * 0.3, torch.randn(ff, D, generator=g).double() * 0.2
        W[f"e{e}.down"] = torch.randn(D, ff, generator=g).double() * 0.2
    up = torch.stack([torch.stack([W[f"e{e}.gate"], W[f"e{e}.up"]], 1).reshape(2 * ff, D) for e in range(experts)]).float()
    dn = torch.stack([W[f"e{e}.down"] for e in range(experts)]).float()
    idx, wts = ops.moe_route(x.to(device), W["router"].float().to(device), count, keep, top, 1.0, "sigmoid", 2, True)
    y = ops.moe_rows(x.to(device), idx, wts, up.to(device), dn.to(device), None, True).double().cpu()
    idx, wts = idx.cpu(), wts.double().cpu()
    spec = {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}
    for t in range(T):
        chosen, weights = O.route(x[t].double(), W, "", spec)
        assert idx[t].tolist() == chosen, f"row {t}"
        ref = torch.zeros(D, dtype=O.F64)
        for j, (e, w) in enumerate(zip(chosen, weights)):
            assert abs(float(wts[t, j]) - w) < 1e-5
            ref = ref + w * O.expert(x[t].double(), W, f"e{e}.")
        close(y[t], ref, 1e-4)
        assert abs(float(wts[t].sum()) - 1.0) < 1e-5
    pairs = torch.randn(T, 2 * ff, generator=g)
    close(ops.glu_pairs(pairs.to(device)).double().cpu(), torch.nn.functional.silu(pairs[:, 0::2].double()) * pairs[:, 1::2].double(), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_a_group_is_worth_its_two_best_scores(device):
    """three groups of three: the group with the single best expert loses to a group with two good ones"""
    ops = R.ops_for(device)
    D = 8
    x = torch.zeros(1, D)
    x[0, 0] = 1.0
    logits = [4.0, -6.0, -6.0, 1.5, 1.4, -6.0, 1.0, 0.9, 0.8]
    wr = torch.zeros(9, D)
    wr[:, 0] = torch.tensor(logits)
    idx, wts = ops.moe_route(x.to(device), wr.to(device), 3, 1, 2, 1.0, "sigmoid", 2, True)
    assert idx.cpu().tolist() == [[3, 4]]
    s = torch.sigmoid(torch.tensor(logits[3:5]).double())
    close(wts.double().cpu(), (s / s.sum()).view(1, 2), 1e-6)
    idx, _ = ops.moe_route(x.to(device), wr.to(device), 3, 1, 2, 1.0, "sigmoid", 1, True)     # (worth of the best alone: group 0)
    assert idx.cpu().tolist() == [[0, 1]] or idx.cpu().tolist()[0][0] == 0


@pytest.mark.parametrize("device", DEVICES)
def test_embedding_sum_stream_update_and_activations(device):
    g = torch.Generator().manual_seed(43)
    ops = R.ops_for(device)
    for D in (48, 1000, 1500, 5000):
        T = 5
        x = torch.randn(T, D, generator=g)
        y1, y2, w = torch.randn(T, D, generator=g), torch.randn(T, D, generator=g), torch.randn(D, generator=g)
        for a, b in ((y1, y2), (y1, None), (None, None)):
            xs = x.clone().to(device)
            xa = ops.add_norm(xs, None if a is None else a.to(device), None if b is None else b.to(device), w.to(device), 1e-5,
                              torch.float32)
            s = x.double() + (0 if a is None else a.double()) + (0 if b is None else b.double())
            close(xs.double().cpu(), s, 1e-5)
            close(xa.double().cpu(), O.norm(s, w.double(), 1e-5), 1e-4)
        xs = x.clone().to(device)
        assert ops.add_norm(xs, y1.to(device), y2.to(device), None, 1e-5, torch.float32) is None
        close(xs.double().cpu(), x.double() + y1.double() + y2.double(), 1e-5)
    t1, t2 = torch.randn(20, 70, generator=g), torch.randn(9, 70, generator=g)
    i1, i2 = torch.randint(0, 20, (33,), generator=g), torch.randint(0, 9, (33,), generator=g)
    close(ops.embed_rows(i1.to(device), t1.to(device), i2.to(device), t2.to(device), 1.0).double().cpu(), t1[i1].double() + t2[i2].double(), 1e-6)
    close(ops.embed_rows(i1.to(device), t1.to(device), scale=3.0).double().cpu(), 3.0 * t1[i1].double(), 1e-5)
    for width, c0, n in ((50, 7, 40), (56, 8, 40), (1040, 16, 1024)):      # columns that are and are not 16-byte pieces
        P = torch.randn(11, width, generator=g) * 3
        z = P[:, c0:c0 + n].double()
        close(ops.act_cols(P.to(device), c0, n, "gelu_erf").double().cpu(), 0.5 * z * (1 + torch.erf(z / math.sqrt(2))), 1e-5)
        close(ops.act_cols(P.to(device), c0, n, "gelu_tanh").double().cpu(),
              0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))), 1e-5)
        Pb = P.bfloat16()
        zb = Pb[:, c0:c0 + n].double()
        close(ops.act_cols(Pb.to(device), c0, n, "gelu_erf").double().cpu(), 0.5 * zb * (1 + torch.erf(zb / math.sqrt(2))), 0.05)


def test_pair_rows_continue_across_steps_and_start_anew_in_a_used_slot():
    table = {"buckets": 37, "mul_prev": 11, "mul_cur": 5}
    pe = PairEmbedding(37, 11, 5)
    toks = tokens(30, 80, 44)
    want = O.pair_rows(toks, table)
    assert want[0] == 37 and all(0 <= r < 37 for r in want[1:])
    assert pe.rows(-1, toks) == want
    assert pe.rows(-1, toks[:7]) + pe.rows(toks[6], toks[7:8]) + pe.rows(toks[7], toks[8:]) == want
    big = PairEmbedding(65521, 1000003, 31)                 # products beyond 32 bits
    assert big.rows(49999, [49998]) == [(49999 * 1000003 + 49998 * 31) % 65521]
    # through the engine: a model without layers is norm(embedding) times the head; the slot is used again
    cfg = O.make_config([], pairs=(37, 11, 5))
    sd = O.random_weights(cfg, seed=45)
    eng = engine_for(cfg, sd, torch.float32, "cpu")
    other = tokens(9, 80, 46)
    got = run_schedule(eng, {"a": toks, "b": other}, [[("a", 7)], [("a", 1)], [("a", 22)], [("b", 4)], [("b", 5)]], 64, slots=1)
    close(got["a"], O.forward(toks, O.as_f64(sd), cfg), 1e-4)
    close(got["b"], O.forward(other, O.as_f64(sd), cfg), 1e-4)


def test_layer_executions_of_a_loop():
    layers = [O.attention_layer() for _ in range(5)]
    for loop, runs, mix in [(None, [0, 1, 2, 3, 4], ()), ((0, 5, 1), [0, 1, 2, 3, 4], (0,)), ((1, 3, 3), [0, 1, 2, 1, 2, 1, 2, 3, 4], (1, 3, 5)),
                            ((3, 5, 2), [0, 1, 2, 3, 4, 3, 4], (3, 5)), ((2, 2, 4), [0, 1, 2, 3, 4], ()), ((4, 5, 2), [0, 1, 2, 3, 4, 4], (4, 5))]:
        cfg = O.make_config(layers, loop=loop)
        rc = filanex.read_config(cfg)
        assert rc.layer_runs() == runs and tuple(rc.mix_in) == mix
        assert [li for li, _ in O.layer_runs(cfg)] == runs and tuple(i for i, (_, m) in enumerate(O.layer_runs(cfg)) if m) == mix
    # every execution has a cache of its own
    eng = engine_for(O.make_config(layers[:3], loop=(1, 3, 2)), O.random_weights(O.make_config(layers[:3], loop=(1, 3, 2)), 1), torch.float32, "cpu")
    assert sorted(eng.state_specs()) == [0, 1, 2, 3, 4]


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
    logits = O.forward(sequence[:-1], W, cfg)
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


def test_command_line_and_sampling(tmp_path, capsys):
    """``llm-cli --prompt-ids`` on a checkpoint without a tokenizer (greedy), and sampled generation through the same
    scheduler: with a fixed seed it repeats itself, and top_k = 1 is the greedy answer"""
    from bigdl_amd.cli import llm_cli
    from bigdl_amd.transformers import AutoModelForCausalLM
    cfg = O.make_config([O.attention_layer(), O.attention_layer(mlp=O.moe())], loop=(0, 2, 2))
    sd = O.random_weights(cfg, seed=91)
    path = _save_checkpoint(tmp_path, cfg, sd)
    prompt = tokens(11, cfg["vocab"], 92)
    model = AutoModelForCausalLM.from_pretrained(path).to("cpu", torch.float32)
    greedy = model.generate(torch.tensor([prompt]), max_new_tokens=7)[0].tolist()
    _greedy_is_consistent(cfg, O.as_f64(sd), greedy, len(prompt))
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
    want = O.forward(toks, O.as_f64(sd), cfg)
    for step, rows in ((0, [0, 12]), (1, [2]), (2, [19])):
        got = torch.from_numpy(np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4")).view(len(rows), -1).double()
        close(got, want[rows])


# ------------------------------------------------------------------------------------------------ kernels of long bfloat16 portions
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,e,chunk,cap", [(4, 2, 64, 128, 100, 18.0), (2, 2, 48, 96, 70, None), (3, 1, 16, 32, 0, 5.0),
                                               (8, 2, 128, 64, 64, 30.0), (2, 1, 32, 16, 1, None), (4, 4, 80, 112, 130, 50.0)])
def test_matrix_core_attention_with_blocks_caps_and_channel_gates(H, G, d, e, chunk, cap):
    """bfloat16 prompt portions (the MFMA kernel) and single tokens (the row-wise kernel) against the plain statement on
    the same bfloat16-rounded keys, values and gate logits"""
    g = torch.Generator().manual_seed(71)
    T = 200
    q = torch.randn(T, H, d, generator=g).double()
    k = torch.randn(T, G, d, generator=g).bfloat16().double()
    v = torch.randn(T, G, e, generator=g).bfloat16().double()
    gate = (torch.randn(T, H * e, generator=g) * 2).bfloat16().double()
    qr = q.clone()
    qr[:190] = q[:190].bfloat16().double()                   # the MFMA kernel rounds its queries
    want = O.attend(qr, k, v, 2.0 * d ** -0.5, cap, chunk) * torch.sigmoid(gate).view(T, H, e)
    got = _attend_through_pages("cuda", q, k, v, [120, 64, 3, 3] + [1] * 10, chunk=chunk, scale=2.0 * d ** -0.5, cap=cap, gate=gate,
                                dtype=torch.bfloat16)
    assert float((got - want).abs().max()) < 0.03, float((got - want).abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("T,D,ff,experts,top,count,keep", [(300, 64, 48, 10, 3, 5, 2), (1000, 256, 112, 64, 6, 8, 4), (70, 80, 16, 3, 3, 1, 1),
                                                         (129, 128, 128, 40, 1, 1, 1)])
def test_grouped_product_of_gated_experts_on_sorted_rows(T, D, ff, experts, top, count, keep):
    """bfloat16 long portions: every expert's run of sorted rows through the grouped matrix-core product with silu(gate) * up
    on the way out, against float64 on the same bfloat16 inputs and against the row-wise kernels"""
    g = torch.Generator().manual_seed(91)
    ops = R.ops_for("cuda")
    x = torch.randn(T, D, generator=g).bfloat16().cuda()
    wr = (torch.randn(experts, D, generator=g) * 0.4).cuda()
    gt = (torch.randn(experts, ff, D, generator=g) * 0.3).bfloat16()
    up = (torch.randn(experts, ff, D, generator=g) * 0.2).bfloat16()
    dn = (torch.randn(experts, D, ff, generator=g) * 0.2).bfloat16().cuda()
    both = torch.stack([gt, up], 2).reshape(experts, 2 * ff, D).contiguous().cuda()
    idx, wts = ops.moe_route(x, wr, count, keep, top, 1.0, "sigmoid", 2, True)
    got = ops.moe_sorted(x, idx, wts, both, dn, None, True)
    assert got is not None
    rows = ops.moe_rows(x, idx, wts, both, dn, None, True)
    ref = torch.zeros(T, D, dtype=O.F64)
    xd, gd, ud, dnd = x.double().cpu(), gt.double(), up.double(), dn.double().cpu()
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            a = gd[e] @ xd[t]
            a = (a * torch.sigmoid(a) * (ud[e] @ xd[t])).bfloat16().double()
            ref[t] += float(wts[t, j]) * (dnd[e] @ a).bfloat16().double()
    scale = float(ref.abs().max())
    assert float((got.double().cpu() - ref).abs().max()) < 0.02 * scale
    assert float((rows.double().cpu() - ref).abs().max()) < 0.02 * scale
