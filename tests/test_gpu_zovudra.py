"""Zovudra on the GPU against the plain implementation: each mechanism's kernel alone, then whole models under
every way of cutting the work, in float32 (tight) and bfloat16, and greedy generation through the engine."""

import copy
import json
import math
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_zovudra as plain
import trace_helpers as th
from zovudra_fixtures import BLOCK_SIZE, CONFIGS, load_plain, make_tensors, write_model

pytestmark = pytest.mark.gpu
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32) * scale


def close(got, want, rel, what=""):
    got, want = got.detach().cpu().to(F64), want.detach().cpu().to(F64)
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= rel, f"{what}: relative error {err:.3e} > {rel:.0e}"


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# ------------------------------------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("n", [20, 64, 101, 384, 2048, 5001])
def test_dynamic_tanh_kernel(n):
    from tie_amd import kernels

    x = rnd(9, n, seed=n, scale=2.0)
    alpha, w, b = torch.tensor([0.7]), 1 + 0.3 * rnd(n, seed=1), rnd(n, seed=2, scale=0.2)
    want = plain.dynamic_tanh(x.to(F64), 0.7, w.to(F64), b.to(F64))
    xd = x.cuda()
    out = torch.empty_like(xd)
    kernels.dynamic_tanh(xd, alpha.cuda(), w.cuda(), b.cuda(), out)
    close(out, want, 2e-6, "dynamic tanh")
    assert torch.equal(xd.cpu(), x), "the stream is left as it was"
    few = torch.empty(3, n, dtype=torch.bfloat16, device="cuda")
    kernels.dynamic_tanh(xd, alpha.cuda(), w.cuda(), b.cuda(), few, rows=i32([7, 0, 3]))
    close(few, want[[7, 0, 3]], 8e-3, "chosen rows")
    # partial sums still owed to the stream are added in the same pass, and the stream keeps the sum
    owed = rnd(3, 9, n, seed=5)
    kernels.dynamic_tanh(xd, alpha.cuda(), w.cuda(), b.cuda(), out, owed=owed.cuda())
    total = x.to(F64) + owed.to(F64).sum(0)
    close(xd, total, 1e-6, "the settled stream")
    close(out, plain.dynamic_tanh(total, 0.7, w.to(F64), b.to(F64)), 3e-6, "dynamic tanh of the settled stream")
    plain_rows = torch.empty(9, n, dtype=torch.bfloat16, device="cuda")
    kernels.dynamic_tanh(xd, None, None, None, plain_rows)
    assert torch.equal(plain_rows.cpu(), xd.cpu().to(torch.bfloat16)), "without alpha the rows are only converted"


@pytest.mark.parametrize("dim,first,columns", [(8, 16, 32), (20, 0, 20), (5, 7, 19)])
def test_token_gate_kernel(dim, first, columns):
    from tie_amd import kernels

    T, vocab = 11, 37
    gate, table = rnd(T, dim, seed=1, scale=2.0), rnd(vocab, columns, seed=2)
    tokens = [(5 * t + 3) % vocab for t in range(T)]
    want = plain.gelu_tanh(gate.to(F64)) * table.to(F64)[tokens][:, first:first + dim]
    out = torch.empty(T, dim, device="cuda")
    kernels.token_gate(gate.cuda(), i32(tokens), table.cuda(), first, out)
    close(out, want, 2e-6, "gelu_tanh(gate) * the token's columns")
    half = torch.empty(T, dim, dtype=torch.bfloat16, device="cuda")
    kernels.token_gate(gate.cuda(), i32(tokens), table.to(torch.bfloat16).cuda(), first, half)
    close(half, plain.gelu_tanh(gate.to(F64)) * table.to(torch.bfloat16).to(F64)[tokens][:, first:first + dim], 8e-3, "bfloat16")


def test_rms_norm_over_the_first_columns_of_wider_rows():
    from tie_amd import kernels

    x, w = rnd(13, 50, seed=3, scale=2.0).cuda(), (1 + 0.2 * rnd(20, seed=4)).cuda()
    out = torch.empty(13, 20, device="cuda")
    kernels.rms_norm_columns(x[:, :20], w, 1e-5, out)
    close(out, plain.rms_norm(x.cpu().to(F64)[:, :20], w.cpu().to(F64), 1e-5), 2e-6, "norm of columns")


@pytest.mark.parametrize("scaling", [None, (3.0, 1.0, 4.0, 256), (8.0, 2.0, 16.0, 64), (2.0, 0.5, 1.5, 10)])
def test_banded_frequencies(scaling):
    from tie_amd.parts.base import PartSpec, build_part

    rot = {"dims": 24, "base": 300000.0}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    part = build_part("position", PartSpec("rope_banded", {"head_dim": 32, "theta": rot["base"], "rotary_dim": 24,
                                                          "pairing": "rotate_half", "scaling": rot.get("scaling")}))
    part.load(lambda *a, **k: None, "float32", torch.device("cuda"))
    want = plain.banded_frequencies(rot)
    close(part.inv_freq, want, 1e-6, "frequencies")
    if scaling:
        plain_f = plain.banded_frequencies({"dims": 24, "base": 300000.0})
        if 2 * math.pi < scaling[3] / scaling[2]:          # the fastest pair's wavelength is short: it is left alone
            assert float(want[0]) == float(plain_f[0])
        assert abs(float(want[-1]) * scaling[0] - float(plain_f[-1])) < 1e-12      # the slowest is stretched in full
        assert any(1.0001 < float(a / b) < scaling[0] * 0.9999 for a, b in zip(plain_f, want)), "no pair lies between"


def paged(keys, values, bs, dtype, scatter_seed=0):
    """Keys [T, KVH, D] and values of one sequence in pages drawn out of order from a larger pool."""
    T, KVH, D = keys.shape
    blocks = -(-T // bs)
    pool = blocks + 5
    order = torch.randperm(pool, generator=torch.Generator().manual_seed(scatter_seed))[:blocks].tolist()
    k_cache = torch.full((pool, KVH, bs, D), 1e30, dtype=dtype)       # what no query may read is huge, not NaN: the
    v_cache = torch.full((pool, KVH, D, bs), 1e30, dtype=dtype)       # matrix cores multiply masked keys by zero
    for t in range(T):
        k_cache[order[t // bs], :, t % bs] = keys[t].to(dtype)
        v_cache[order[t // bs], :, :, t % bs] = values[t].to(dtype)
    return k_cache.cuda(), v_cache.cuda(), order


def attend(q, keys, values, new, bs, dtype, window, keep, scale, H, free_passed_pages=True):
    """The engine's dispatcher over one sequence whose last ``new`` positions are this step's rows."""
    from tie_amd import kernels

    T, KVH, D = keys.shape
    k_cache, v_cache, order = paged(keys, values, bs, dtype, scatter_seed=T)
    table = list(order)
    if free_passed_pages and window:       # pages no query of this step reads hold garbage: they were given back
        first_needed = max(0, (T - new) - window + 1) // bs
        for page in range(-(-keep // bs), first_needed):
            k_cache[table[page]] = 1e30
            v_cache[table[page]] = 1e30
            table[page] = -1
    step = SimpleNamespace(block_tables=i32([table + [0] * 3]), key_shares=None)
    batch = SimpleNamespace(query_start=i32([0, new]), context_lens=i32([T]), seq_of_row=i32([0] * new),
                            all_decode=new == 1, num_seqs=1, plan_context=max(1024, T), host_new_tokens=[new],
                            host_context_lens=[T], memo={}, num_tokens=new)
    qd = q[T - new:].reshape(new, H * D).to(dtype).cuda().contiguous()
    out = torch.empty_like(qd)
    scratch = {}

    def get(name, shape, dt=None):
        key = (name, tuple(shape), dt)
        if key not in scratch:
            scratch[key] = torch.empty(tuple(shape), dtype=dt or dtype, device="cuda")
        return scratch[key]

    kernels.paged_attention(qd, k_cache, v_cache, out, step, batch, H, scale, window, scratch=get, keep_first=keep)
    return out.float().cpu().view(new, H, D)


def plain_attend(q, keys, values, window, keep, scale, H):
    T, KVH, D = keys.shape
    mask = plain.visible(T, window, keep)
    return torch.stack([plain.softmax_attention(q[:, h].to(F64), keys[:, h // (H // KVH)].to(F64),
                                                values[:, h // (H // KVH)].to(F64), scale, mask) for h in range(H)], dim=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("new", [1, 2, 37, 300])
@pytest.mark.parametrize("H,KVH,D,bs,window,keep", [(4, 2, 16, 4, 9, 3), (8, 2, 48, 16, 120, 5), (2, 1, 128, 16, 64, 4),
                                                    (6, 1, 32, 16, 16, 16), (3, 3, 64, 32, 7, 40), (4, 4, 128, 16, 33, 1),
                                                    (20, 1, 16, 8, 1, 2), (4, 2, 64, 16, 50, 0)])
def test_a_window_beside_kept_first_positions(H, KVH, D, bs, window, keep, new, dtype):
    T = 300
    q, keys, values = rnd(T, H, D, seed=1, scale=1.5), rnd(T, KVH, D, seed=2), rnd(T, KVH, D, seed=3)
    if dtype == torch.bfloat16:
        q, keys, values = (t.to(dtype).float() for t in (q, keys, values))
    want = plain_attend(q, keys, values, window, keep, 0.2, H)[T - new:]
    got = attend(q, keys, values, new, bs, dtype, window, keep, 0.2, H)
    close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2, f"attention, the last {new} rows")


@pytest.mark.parametrize("new", [1, 3, 70])
@pytest.mark.parametrize("H,KVH,D,bs,window,keep", [(8, 2, 64, 16, 1500, 70), (4, 4, 128, 16, 2000, 5), (4, 1, 48, 32, 900, 129),
                                                    (40, 2, 64, 16, 1200, 33), (17, 1, 128, 16, 2000, 0)])
def test_kept_positions_where_the_keys_are_cut_into_shares(H, KVH, D, bs, window, keep, new):
    """A long context and few rows: the matrix-core kernels cut a row's keys into shares that are merged; the kept
    keys go with the first share. More than sixteen query heads on a key/value head are several waves of columns."""
    from tie_amd import kernels

    T = 2600
    assert kernels.decode_splits(1, KVH, T, bs) > 1
    q, keys, values = rnd(T, H, D, seed=1, scale=1.5), rnd(T, KVH, D, seed=2), rnd(T, KVH, D, seed=3)
    for h in range(H):                       # the last query leans towards a kept key, so that losing it would show
        q[T - 1, h] += 3.0 * keys[keep - 1, h // (H // KVH)]
    q, keys, values = (t.to(torch.bfloat16).float() for t in (q, keys, values))
    want = plain_attend(q, keys, values, window, keep, 0.2, H)[T - new:]
    if keep:
        lost = plain_attend(q, keys, values, window, keep - 1, 0.2, H)[T - new:]
        assert float((want - lost).abs().max()) > 0.05
    got = attend(q, keys, values, new, bs, torch.bfloat16, window, keep, 0.2, H)
    close(got, want, 1.5e-2, f"attention over shares, the last {new} rows")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("new", [1, 40])
def test_one_key_that_towers_at_every_edge(new, dtype):
    """One key is made to answer the last query alone, at the first position, the last kept one, the first one not
    kept, far back, at a page's border, one before the window and at its first position: the output is that key's
    value where it is visible and must not know of it where it is not."""
    T, H, KVH, D, bs, window, keep = 400, 4, 2, 64, 16, 50, 6
    for place, seen in [(0, True), (keep - 1, True), (keep, False), (15, False), (16, False), (200, False),
                        (T - window - 1, False), (T - window, True), (T - 1, True), (335, False), (352, True)]:
        q, keys, values = rnd(T, H, D, seed=1, scale=0.3), rnd(T, KVH, D, seed=2, scale=0.3), rnd(T, KVH, D, seed=3)
        for h in range(H):
            q[T - 1, h] = 4.0 * keys[place, h // 2] / keys[place, h // 2].norm()
        keys[place] *= 30.0 / keys[place].norm(dim=-1, keepdim=True)
        if dtype == torch.bfloat16:
            q, keys, values = (t.to(dtype).float() for t in (q, keys, values))
        want = plain_attend(q, keys, values, window, keep, 1.0, H)[T - new:]
        got = attend(q, keys, values, new, bs, dtype, window, keep, 1.0, H)
        close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2, f"towering key at {place}")
        alone = float((want[-1, 0] - values[place, 0].to(F64)).abs().max())
        assert (alone < 1e-3) == seen, f"the key at {place} should {'be' if seen else 'not be'} the answer"


@pytest.mark.parametrize("E,groups,keep,top,shared", [(16, 4, 1, 3, 2), (8, 4, 2, 3, 0), (6, 3, 1, 2, 1), (5, 1, 1, 2, 1),
                                                      (1, 1, 1, 1, 1), (64, 8, 3, 6, 0), (12, 12, 5, 4, 3)])
def test_the_sigmoid_router(E, groups, keep, top, shared):
    from tie_amd import kernels

    T = 50
    logits = rnd(T, E + (1 if shared else 0), seed=E, scale=2.0)
    r = {"experts": E, "top": top, "scale": 1.75, "groups": {"count": groups, "keep": keep}}
    chosen, weights = plain.route(logits[:, :E].to(F64), r)
    ids = torch.empty(T, top + shared, dtype=torch.int32, device="cuda")
    w = torch.empty(T, top + shared, device="cuda")
    kernels.moe_route(logits.cuda(), None, groups, keep, top, ids, w, scoring="sigmoid", group_top=2, renormalize=True,
                      renorm_eps=1e-20, weight_scale=1.75, shared=shared)
    assert torch.equal(ids.cpu()[:, :top].long(), chosen), "the chosen experts, best first"
    close(w[:, :top], weights, 2e-6, "weights")
    if shared:
        assert torch.equal(ids.cpu()[:, top:], torch.arange(E, E + shared, dtype=torch.int32).expand(T, shared))
        close(w[:, top:], torch.sigmoid(logits[:, E:].to(F64)).expand(T, shared), 2e-6, "the shared expert's gate")


def test_a_routing_choice_worked_out_by_hand():
    from tie_amd import kernels

    # scores by sigmoid: groups (0.9, 0.1 | 0.6, 0.6 | 0.8, 0.3): sums of the two best 1.0, 1.2, 1.1 -> groups 1 and 2
    # stay; of (0.6, 0.6, 0.8, 0.3) the best two are experts 4 and 2 (a tie goes to the lower index): 0.8, 0.6
    s = torch.tensor([[0.9, 0.1, 0.6, 0.6, 0.8, 0.3]])
    logits = torch.log(s / (1 - s))
    ids = torch.empty(1, 2, dtype=torch.int32, device="cuda")
    w = torch.empty(1, 2, device="cuda")
    kernels.moe_route(logits.cuda(), None, 3, 2, 2, ids, w, scoring="sigmoid", group_top=2, renormalize=True,
                      renorm_eps=1e-20, weight_scale=3.0)
    assert ids.cpu().tolist() == [[4, 2]]
    close(w, torch.tensor([[3.0 * 0.8 / 1.4, 3.0 * 0.6 / 1.4]]), 1e-6, "weights")
    kernels.moe_route(logits.cuda(), None, 3, 2, 2, ids, w, scoring="sigmoid", group_top=1)      # groups by their best
    assert ids.cpu().tolist() == [[0, 4]]
    close(w, torch.tensor([[0.9, 0.8]]), 1e-6, "plain weights")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top,F_,K", [(3, 4, 2, 24, 64), (70, 3, 2, 16, 40), (700, 4, 3, 64, 128), (200, 2, 2, 9, 100)])
def test_experts_without_a_gate(T, E, top, F_, K, dtype):
    """relu(up_e h)^2 over rows sorted by expert, then down_e, then the weighted sum: the float32 kernels and the
    matrix-core ones in all three tile sizes."""
    from tie_amd import kernels

    h, up, down = rnd(T, K, seed=1), rnd(E, F_, K, seed=2, scale=0.3), rnd(E, K, F_, seed=3, scale=0.3)
    if dtype == torch.bfloat16:
        h, up, down = (t.to(dtype).float() for t in (h, up, down))
    g = torch.Generator().manual_seed(4)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    weights = torch.rand(T, top, generator=g)
    want = torch.zeros(T, K, dtype=F64)
    for t in range(T):
        for k in range(top):
            e = int(ids[t, k])
            want[t] += weights[t, k].to(F64) * plain.expert(h[t].to(F64), up[e].to(F64), down[e].to(F64))
    scratch = {}

    def get(name, shape, dt):
        return scratch.setdefault((name, tuple(shape)), torch.empty(tuple(shape), dtype=dt, device="cuda"))

    hd, upd, downd = h.to(dtype).cuda(), up.to(dtype).cuda(), down.to(dtype).cuda()
    tile = kernels.moe_tile_rows(dtype, dtype, K, F_, T * top, E)
    rows = kernels.moe_align(ids.cuda(), E, tile, get)
    act = torch.empty(T * top, F_, dtype=dtype, device="cuda")
    kernels.moe_gate_up(hd, None, upd, rows, act)
    parts = torch.empty(T * top, K, device="cuda")
    kernels.moe_down(act, downd, rows, parts)
    out = torch.zeros(T, K, device="cuda")
    kernels.moe_combine(kernels.RoutedParts(parts, rows.where, weights.cuda(), hd), out)
    close(out, want, 1e-5 if dtype == torch.float32 else 2e-2, f"experts in tiles of {tile}")


# ------------------------------------------------------------------------------------------- whole models
LENGTHS = {"A": [1, 23, 60, 37, 5], "B": [70, 2, 41, 90], "C": [33, 50, 8], "D": [12, 30, 3, 21, 9], "E": [150, 1, 66, 97]}
TOLERANCE = {"float32": 3e-5, "bfloat16": 8e-2}        # of the largest logit; the queries are drawn wide


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            folder = tmp_path_factory.mktemp(f"zovudra_{name}_{dtype}")
            out[name, dtype] = write_model(folder, config, seed=61 + len(out), dtype=dtype)
    return out


def reference(folder, config, requests, streams=None):
    weights = load_plain(folder)
    out = {}
    for rid, toks in requests.items():
        logits, behind = plain.forward(config, weights, toks)
        out[rid] = logits.float()
        if streams is not None:
            streams[rid] = behind
    return out


def worst_error(got, want):
    worst = 0.0
    for rid, ref in want.items():
        mine = torch.stack([got[rid][p] for p in range(ref.shape[0])])
        worst = max(worst, float(((mine - ref).abs().amax(dim=1) / ref.abs().max()).max()))
    return worst


def check(got, want, tolerance, label):
    worst = 0.0
    for rid, ref in want.items():
        rows = got[rid]
        assert sorted(rows) == list(range(ref.shape[0])), f"{label}: request {rid} misses positions"
        mine = torch.stack([rows[p] for p in range(ref.shape[0])])
        assert torch.isfinite(mine).all(), f"{label}: request {rid} has non-finite logits"
        err = (mine - ref).abs().amax(dim=1) / ref.abs().max()
        bad = int(torch.argmax((err > tolerance).float())) if bool((err > tolerance).any()) else -1
        assert bad < 0, (f"{label}: request {rid} first differs at position {bad} "
                         f"(relative error {float(err[bad]):.3e}, allowed {tolerance:.0e})")
        worst = max(worst, float(err.max()))
    print(f"[observed] {label}: {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_every_way_of_cutting_the_work(folders, name, dtype):
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, dtype], CONFIGS[name]
    requests = th.make_requests(config["vocab"], LENGTHS[name], seed=5)
    want = reference(folder, config, requests)
    bs = BLOCK_SIZE[name]
    biggest = max(th.round64(len(t)) for t in requests.values())

    def replayer(max_tokens):
        return TraceReplayer.from_folder(folder, dtype, max_tokens, block_size=bs)

    results = {"whole": th.collect(replayer(biggest), th.whole(requests)),
               "prefill+decode": th.collect(replayer(biggest), th.prefill_then_decode(requests, tail=40)),
               "portions": th.collect(replayer(biggest), th.portions(requests)),
               "portions of two": th.collect(replayer(biggest), th.portions(requests, sizes=(2,))),
               "token by token": th.collect(replayer(biggest), th.portions(requests, sizes=(1,)))}
    steps, peak = th.mixed(requests, max_live=4, seed=3)
    assert max(len(s["entries"]) for s in steps) >= 3
    rep = replayer(peak)
    results["mixed"] = th.collect(rep, steps)
    assert rep.cache.all_free()                                   # every page came back
    for label, got in results.items():
        check(got, want, TOLERANCE[dtype], f"{name}/{dtype}/{label}")
    if dtype == "float32":       # the ways of cutting agree with each other beyond what they owe the plain one
        for label in results:
            for rid in requests:
                a = torch.stack([results["whole"][rid][p] for p in range(len(requests[rid]))])
                b = torch.stack([results[label][rid][p] for p in range(len(requests[rid]))])
                assert float((a - b).abs().max() / a.abs().max()) < 1e-5, f"{name}: whole vs {label}, request {rid}"


def random_config(seed):
    """A model of random layers and sizes: every choice the reader knows is drawn, present or absent."""
    import random

    rng = random.Random(seed)
    pick = rng.choice
    width = pick([40, 64, 72, 96, 128])

    def rot(dims_most, whole):
        dims = dims_most if whole or rng.random() < 0.4 else pick([d for d in range(2, dims_most + 1, 2)])
        out = {"dims": dims, "base": pick([50.0, 1000.0, 10000.0, 500000.0])}
        if rng.random() < 0.6:
            low = pick([0.5, 1.0, 2.0])
            out["scaling"] = {"factor": pick([2.0, 4.0, 8.0]), "low": low, "high": low * pick([2.0, 4.0, 8.0]),
                              "original": pick([16, 64, 256])}
        return out

    def mixer():
        if rng.random() < 0.6:
            kv = pick([1, 2, 3])
            dim = pick([8, 16, 24, 32, 48, 64])
            m = {"heads": kv * pick([1, 2, 4, 6]), "kv_heads": kv, "dim": dim, "vdim": pick([dim, dim, 16, 40]),
                 "scale": rng.uniform(0.1, 0.4), "rot": rot(dim, False)}
            if rng.random() < 0.8:
                m["mask"] = {"size": pick([1, 3, 8, 17, 32, 50])}
                if rng.random() < 0.75:
                    m["mask"]["keep_first"] = pick([1, 2, 5, 16, 33, 70])
            return {"type": "attention", "mixer": m}
        r = pick([4, 8, 16, 32])
        m = {"heads": pick([1, 2, 5, 8, 18]), "dim": pick([8, 16, 24, 40]), "rot_dim": r, "vdim": pick([8, 16, 24, 56]),
             "kv_rank": pick([12, 16, 40, 64]), "q_rank": pick([8, 20, 32]), "scale": rng.uniform(0.1, 0.3),
             "rot": rot(r, True)}
        if rng.random() < 0.8:
            m["mask"] = {"size": pick([1, 4, 9, 20, 45])}
        return {"type": "latent_attention", "mixer": m}

    def mlp():
        u = rng.random()
        if u < 0.15:
            return None
        if u < 0.5:
            return {"kind": "dense", "ff": pick([16, 40, 64, 100])}
        groups = pick([1, 1, 2, 3, 4])
        per = pick([1, 2, 3, 4])
        keep = rng.randint(1, groups)
        router = {"experts": groups * per, "top": rng.randint(1, min(keep * per, 4))}
        if groups > 1 or rng.random() < 0.3:
            router["groups"] = {"count": groups, "keep": keep}
        if rng.random() < 0.7:
            router["scale"] = pick([0.5, 1.5, 2.0, 3.0])
        out = {"kind": "moe", "expert": {"ff": pick([8, 16, 24, 40])}, "router": router}
        if rng.random() < 0.7:
            out["shared"] = {"ff": pick([8, 16, 30, 56])}
        return out

    config = {"architecture": "Zovudra", "vocab": pick([50, 97, 200]), "width": width,
              "norm": {"eps": pick([1e-6, 1e-5, 1e-4])},
              "layers": [{**mixer(), "mlp": mlp()} for _ in range(rng.randint(1, 5))]}
    if rng.random() < 0.7:
        config["embedding"] = {"scale": pick([0.5, 2.0, 4.0])}
    if rng.random() < 0.7:
        config["token_side"] = {"dim": pick([4, 8, 12, 32])}
    return config, pick([4, 8, 16, 32])


@pytest.mark.parametrize("dtype,seed", [("float32", s) for s in range(12)] + [("bfloat16", s) for s in (1, 4, 7, 10)])
def test_models_of_random_layers_and_sizes(tmp_path, seed, dtype):
    from tie_amd.engine.replay import TraceReplayer

    config, bs = random_config(seed)
    folder = write_model(tmp_path / "model", config, seed=100 + seed, dtype=dtype)
    requests = th.make_requests(config["vocab"], [75, 3, 41, 1, 58], seed=seed)
    want = reference(folder, config, requests)
    biggest = max(th.round64(len(t)) for t in requests.values())
    results = {"whole": th.collect(TraceReplayer.from_folder(folder, dtype, biggest, block_size=bs), th.whole(requests)),
               "prefill+decode": th.collect(TraceReplayer.from_folder(folder, dtype, biggest, block_size=bs),
                                            th.prefill_then_decode(requests, tail=35))}
    steps, peak = th.mixed(requests, max_live=4, seed=seed)
    rep = TraceReplayer.from_folder(folder, dtype, max(peak, bs), block_size=bs)
    results["mixed"] = th.collect(rep, steps)
    assert rep.cache.all_free()
    for label, got in results.items():
        check(got, want, TOLERANCE[dtype], f"random model {seed}/{dtype}/{label}: {json.dumps(config)}")


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_stream_after_every_layer(folders, name):
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, "float32"], CONFIGS[name]
    requests = th.make_requests(config["vocab"], [29], seed=8)
    streams = {}
    reference(folder, config, requests, streams)
    rep = TraceReplayer.from_folder(folder, "float32", 64, block_size=BLOCK_SIZE[name])
    seen = []
    rep.model.layer_hook = lambda index, x: seen.append(x.detach().double().cpu().clone())
    th.collect(rep, th.whole(requests))
    assert len(seen) == len(config["layers"])
    for i, (mine, ref) in enumerate(zip(seen, streams["r0"])):
        close(mine, ref, 1e-5, f"{name}: the stream after layer {i}")


def _altered(config, change):
    other = copy.deepcopy(config)
    change(other)
    return other


def test_a_fault_of_one_position_or_one_term_would_show(folders):
    """The engine agrees with the plain model, and the plain model with one mechanism slightly off does not agree
    with the engine by a wide margin."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["A", "float32"], CONFIGS["A"]
    requests = th.make_requests(config["vocab"], [48, 31], seed=21)
    got = th.collect(TraceReplayer.from_folder(folder, "float32", 128, block_size=BLOCK_SIZE["A"]),
                     th.prefill_then_decode(requests, tail=20))
    weights = load_plain(folder)
    assert worst_error(got, reference(folder, config, requests)) < TOLERANCE["float32"]

    def off(label, config_change=None, weight_change=None):
        cfg = _altered(config, config_change) if config_change else config
        w = dict(weights)
        if weight_change:
            weight_change(w)
        want = {rid: plain.forward(cfg, w, toks)[0].float() for rid, toks in requests.items()}
        err = worst_error(got, want)
        print(f"[observed] {label}: {err:.3e}")
        assert err > 100 * TOLERANCE["float32"], f"{label} does not show in the logits ({err:.3e})"

    for layer in (0, 1, 3):
        mask = config["layers"][layer]["mixer"]["mask"]
        off(f"layer {layer}: a window one longer", lambda c: c["layers"][layer]["mixer"]["mask"].update(size=mask["size"] + 1))
        off(f"layer {layer}: a window one shorter", lambda c: c["layers"][layer]["mixer"]["mask"].update(size=mask["size"] - 1))
    for layer in (0, 3):
        keep = config["layers"][layer]["mixer"]["mask"]["keep_first"]
        off(f"layer {layer}: one more position kept", lambda c: c["layers"][layer]["mixer"]["mask"].update(keep_first=keep + 1))
        off(f"layer {layer}: one position fewer kept", lambda c: c["layers"][layer]["mixer"]["mask"].update(keep_first=keep - 1))
    off("no kept positions", lambda c: c["layers"][0]["mixer"]["mask"].update(keep_first=0))
    off("frequencies left unscaled", lambda c: c["layers"][0]["mixer"]["rot"].pop("scaling"))
    off("a whole head rotated", lambda c: c["layers"][0]["mixer"]["rot"].update(dims=16))
    off("no shared expert", lambda c: c["layers"][0]["mlp"].pop("shared"))
    off("every group kept", lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=4))
    off("routing weights not scaled", lambda c: c["layers"][0]["mlp"]["router"].update(scale=1.0))
    off("no per-token side input", lambda c: c.pop("token_side"))
    off("the side input of another layer", None,
        lambda w: w.__setitem__("side.embed", torch.roll(w["side.embed"], 8, dims=1)))
    off("an embedding left unscaled", lambda c: c.pop("embedding"))
    off("a norm without its bias", None, lambda w: w.__setitem__("l2.norm1.b", torch.zeros_like(w["l2.norm1.b"])))
    off("a query latent left unnormed", None, lambda w: w.__setitem__("l1.mix.dq.norm", w["l1.mix.dq.norm"] * 1.1))


def test_a_far_key_decides_a_decoded_token(tmp_path):
    """A prompt of hundreds of tokens in which one of the kept first tokens alone answers the last query, far
    outside the window: a lost page or a kept range that is one short shows in the logits."""
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.safetensors_io import write_safetensors

    config = {"architecture": "Zovudra", "vocab": 50, "width": 32, "norm": {"eps": 1e-5},
              "layers": [{"type": "attention", "mlp": None,
                          "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 2.0,
                                    "mask": {"size": 24, "keep_first": 6}}}]}
    tensors = make_tensors(config, 77, "float32")
    w = {k: v.to(F64) for k, v in tensors.items()}
    asked, answer = 48, 49

    def mixer_input(token):             # the first layer's rows depend on the token alone
        return plain.dynamic_tanh(w["embed"][token], w["l0.norm1.alpha"], w["l0.norm1"], w["l0.norm1.b"])

    key = plain.rms_norm(w["l0.mix.k"] @ mixer_input(answer), w["l0.mix.k.norm"], 1e-5)
    target = torch.cat([key, key])                  # W_q h(asked), once normed, points along the key in both heads
    h = mixer_input(asked)
    tensors["l0.mix.q"] = (target[:, None] * h[None, :] / (h * h).sum()).float()
    tensors["l0.mix.q.norm"] = torch.full_like(tensors["l0.mix.q.norm"], 3.0)
    folder = tmp_path / "far"
    folder.mkdir()
    with open(folder / "config.json", "w") as f:
        json.dump(config, f)
    write_safetensors(str(folder / "model.safetensors"), list(tensors.items()))
    weights = load_plain(str(folder))
    g = torch.Generator().manual_seed(3)
    tokens = torch.randint(0, 48, (700,), generator=g).tolist()
    tokens[5], tokens[-1] = answer, asked
    full = plain.forward(config, weights, tokens)[0].float()
    without = plain.forward(config, weights, tokens[:5] + [0] + tokens[6:])[0].float()
    assert float((without[699] - full[699]).abs().max() / full[699].abs().max()) > 0.05     # position 5 decides
    for cut in (690, 699, 700):                                   # the last tokens decoded one by one, or none
        rep = TraceReplayer.from_folder(str(folder), "float32", 128, block_size=16)     # 8 pages for 700 tokens
        steps, at = [], 0
        while at < cut:                 # the prompt in portions the pool can hold beside the window's pages
            n = min(64, cut - at)
            steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": tokens[at:at + n],
                                                           "want": [699 - at] if at + n == 700 else []}], "end": []})
            at += n
        steps += [{"step": len(steps) + i - cut, "entries": [{"id": "a", "tokens": [tokens[i]], "want": [0]}], "end": []}
                  for i in range(cut, 700)]
        got = th.collect(rep, steps)
        err = float((got["a"][699] - full[699]).abs().max() / full[699].abs().max())
        assert err < TOLERANCE["float32"], f"cut at {cut}: {err:.3e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_windows_with_pages_given_back_and_used_again(folders, dtype):
    """Two requests decode 150 tokens each in a pool that holds them only because the windows' pages go back while the
    pages of the kept first positions stay; a third then runs in the pages they left."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["E", dtype], CONFIGS["E"]
    requests = th.make_requests(config["vocab"], [170, 165, 60], seed=9)
    want = reference(folder, config, requests)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": requests[r][:20 - i], "want": list(range(20 - i))}
                                    for i, r in enumerate(("r0", "r1"))], "end": []}]
    at = {"r0": 20, "r1": 19}
    while at:
        entries = [{"id": r, "tokens": [requests[r][p]], "want": [0]} for r, p in at.items()]
        at = {r: p + 1 for r, p in at.items()}
        ended = [r for r, p in at.items() if p == len(requests[r])]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        for r in ended:
            del at[r]
    steps.append({"step": len(steps), "entries": [{"id": "r2", "tokens": requests["r2"], "want": list(range(60))}],
                  "end": ["r2"]})
    rep = TraceReplayer.from_folder(folder, dtype, 256, block_size=16)       # 16 pages: far fewer than 335 tokens
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE[dtype], f"long decoding, {dtype}")


@pytest.mark.parametrize("name", ["A", "E"])
def test_decode_steps_replayed_from_recordings_give_the_eager_logits(folders, name):
    """bfloat16 decode-only steps are recorded into HIP graphs and replayed; every replay against the eager engine."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders[name, "bfloat16"], CONFIGS[name]
    requests = th.make_requests(config["vocab"], [50, 41, 47], seed=10)
    steps, peak = th.mixed(requests, max_live=3, seed=4, tail=30)
    eager = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=BLOCK_SIZE[name], use_graphs=False)
    recorded = TraceReplayer.from_folder(folder, "bfloat16", peak, block_size=BLOCK_SIZE[name])
    assert recorded.runner.use_graphs
    a, b = th.collect(eager, steps), th.collect(recorded, steps)
    assert recorded.runner.graph_replays > 10
    for rid, toks in requests.items():
        for p in range(len(toks)):
            assert torch.equal(a[rid][p], b[rid][p]), f"request {rid}, position {p}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    """The engine's own entry point and scheduler: several requests at once, prompts in portions, a small pool."""
    import tie_amd

    folder, config = folders[name, dtype], CONFIGS[name]
    weights = load_plain(folder)
    prompts = list(th.make_requests(config["vocab"], [7, 19, 3, 30], seed=12).values())
    new = 10
    engine = tie_amd.create_engine(folder, dtype=dtype, kv_blocks=64, block_size=BLOCK_SIZE[name], max_seqs=3,
                                   max_tokens_per_step=16, prefill_chunk=8)
    ids = [engine.add_request(p, tie_amd.SamplingParams(max_tokens=new)) for p in prompts]
    while engine.has_work():
        engine.step()
    for sid, prompt in zip(ids, prompts):
        generated = list(engine.sequence(sid).generated)
        assert len(generated) == new
        tokens = list(prompt)
        for i, token in enumerate(generated):       # every generated token is the plain model's best, or ties it
            logits = plain.forward(config, weights, tokens)[0][-1]
            best = float(logits.max())
            margin = 1e-4 * float(logits.abs().max()) if dtype == "float32" else 0.05 * float(logits.abs().max())
            assert float(logits[token]) >= best - margin, f"request {sid}: token {i} is not the plain model's choice"
            tokens.append(token)


def test_the_command_line_generates_the_plain_models_tokens(folders):
    from conftest import ROOT

    folder, config = folders["A", "float32"], CONFIGS["A"]
    weights = load_plain(folder)
    prompt = list(th.make_requests(config["vocab"], [11], seed=14).values())[0]
    tokens = list(prompt)
    for _ in range(6):
        tokens.append(int(plain.forward(config, weights, tokens)[0][-1].argmax()))
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "tie"), "generate", "-m", folder, "-p",
                           ",".join(map(str, prompt)), "--temp", "0", "--max-tokens", "6", "--dtype", "float32",
                           "--kv-mem", "16M"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == tokens[len(prompt):]


def test_the_trace_program_runs_the_design(folders, tmp_path):
    """JSON lines in, .f32 files and 'done' lines out; pages used again."""
    from conftest import ROOT

    folder, config = folders["B", "float32"], CONFIGS["B"]
    requests = th.make_requests(config["vocab"], [23, 40, 9, 31, 17], seed=2)
    steps, peak = th.mixed(requests, max_live=4, seed=1)
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out), "--max-tokens", str(peak)],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done")] == [f"done {s['step']}" for s in steps]
    want = reference(folder, config, requests)
    position = {}
    for s in steps:
        data = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, config["vocab"])
        r = 0
        for e in s["entries"]:
            start = position.get(e["id"], 0)
            for w in e["want"]:
                ref = want[e["id"]][start + w]
                assert float(np.abs(data[r] - ref.numpy()).max() / ref.abs().max()) < TOLERANCE["float32"]
                r += 1
            position[e["id"]] = start + len(e["tokens"])
        assert r == data.shape[0]
