"""Minerax on the GPU against the plain implementation: each mechanism's kernel alone, then whole models under
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

import plain_minerax as plain
import trace_helpers as th
from minerax_fixtures import BLOCK_SIZE, CONFIGS, load_plain, write_model

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


def step_batch(counts, slots):
    """What the kernels read of a step: ``counts[s]`` rows of sequence s, whose state lives in ``slots[s]``."""
    starts = [0]
    for n in counts:
        starts.append(starts[-1] + n)
    return SimpleNamespace(num_seqs=len(counts), query_start=i32(starts), state_slots=i32(slots),
                           seq_of_row=i32([s for s, n in enumerate(counts) for _ in range(n)]))


# ------------------------------------------------------------------------------------------- kernels alone
@pytest.mark.parametrize("n", [20, 64, 100, 384, 2048, 5000])
def test_layer_norm_kernel(n):
    from tie_amd import kernels

    x = (rnd(9, n, seed=n, scale=3.0) + 5.0).cuda()              # a mean far from zero
    w = (1 + 0.3 * rnd(n, seed=1)).cuda()
    out = torch.empty_like(x)
    kernels.layer_norm(x, w, 1e-5, out)
    close(out, plain.layer_norm(x.cpu().to(F64), w.cpu().to(F64), 1e-5), 2e-6, "layer norm")
    rows = i32([7, 0, 3])
    few = torch.empty(3, n, dtype=torch.bfloat16, device="cuda")
    kernels.layer_norm(x, w, 1e-5, few, rows=rows)
    close(few, plain.layer_norm(x.cpu().to(F64)[[7, 0, 3]], w.cpu().to(F64), 1e-5), 8e-3, "layer norm of chosen rows")
    half = x.to(torch.bfloat16)
    kernels.layer_norm(half, w, 1e-5, out)
    close(out, plain.layer_norm(half.cpu().to(F64), w.cpu().to(F64), 1e-5), 2e-6, "layer norm of bfloat16 rows")


@pytest.mark.parametrize("S,n,planes", [(1, 48, 0), (2, 64, 1), (3, 352, 0), (4, 100, 3), (8, 1000, 2), (4, 4100, 2), (2, 9000, 1)])
def test_hyper_connection_kernel(S, n, planes):
    from tie_amd import kernels

    T, eps = 6, 1e-5
    x = rnd(T, n, seed=S).cuda()
    streams = torch.full((S, T, n), float("nan"), device="cuda")
    w_in, w_out, mix = rnd(S, seed=2), rnd(S, seed=3), rnd(S, S, seed=4)
    norm_w = 1 + 0.2 * rnd(n, seed=5)
    h = torch.empty(T, n, device="cuda")
    kernels.hyper_connection(streams, x=x, from_x=True, read=(w_in.cuda(), "layer_norm", norm_w.cuda(), eps, h))
    old = [x.cpu().to(F64) for _ in range(S)]
    for s in range(S):
        close(streams[s], old[s], 0.0, "streams start as the embedding's rows")
    close(h, plain.layer_norm(sum(w_in[s].to(F64) * old[s] for s in range(S)), norm_w.to(F64), eps), 3e-6, "first read")
    y = rnd(max(planes, 1), T, n, seed=6)
    total = y.to(F64).sum(0)
    new = [sum(mix[s, t].to(F64) * old[s] for s in range(S)) + w_out[t].to(F64) * total for t in range(S)]
    w_next = rnd(S, seed=7)
    folded = torch.empty(T, n, device="cuda")
    half = torch.empty(T, n, dtype=torch.bfloat16, device="cuda")
    kernels.hyper_connection(streams, x=folded, fold=True, write=((y if planes else y[0]).cuda().contiguous(), mix.cuda(), w_out.cuda()),
                             read=(w_next.cuda(), "layer_norm", norm_w.cuda(), eps, half))
    for t in range(S):
        close(streams[t], new[t], 2e-6, f"stream {t} after a write (mix is indexed [from, to])")
    close(folded, sum(new), 2e-6, "the sum of the streams")
    close(half, plain.layer_norm(sum(w_next[s].to(F64) * new[s] for s in range(S)), norm_w.to(F64), eps), 8e-3, "next read")


def test_gelu_tanh_gate_kernel():
    from tie_amd import kernels

    T, I = 7, 50
    both = torch.cat([rnd(T, I, seed=1, scale=3.0), rnd(T, I, seed=2)], dim=1).cuda()
    out = torch.empty(T, I, device="cuda")
    kernels.swiglu(both, out, activation="gelu_tanh")
    close(out, plain.gelu_tanh(both[:, :I].cpu().to(F64)) * both[:, I:].cpu().to(F64), 2e-6, "gelu_tanh(gate) * up")


@pytest.mark.parametrize("pairing", ["interleaved", "rotate_half"])
def test_rotation_with_stretched_frequencies(pairing):
    """The position part's table and the kernel that turns pairs, at positions far beyond the original length."""
    from tie_amd import kernels
    from tie_amd.parts.base import PartSpec, build_part

    rot = {"dims": 12, "base": 300.0, "scaling": {"factor": 6.0, "original": 40, "fast": 8.0, "slow": 0.75}}
    part = build_part("position", PartSpec("rope_yarn", {"head_dim": 16, "theta": rot["base"], "rotary_dim": 12,
                                                        "pairing": pairing, "scaling": rot["scaling"]}))
    part.load(lambda *a, **k: None, "float32", torch.device("cuda"))
    freq, amplitude = plain.stretched_frequencies(rot)
    close(part.inv_freq, freq, 1e-6, "frequencies")
    assert abs(part.amplitude - amplitude) < 1e-12
    positions = i32([0, 1, 39, 40, 1000, 70000])
    angles = torch.empty(6, 12, device="cuda")
    kernels.rope_angles(positions, part.inv_freq, angles, part.amplitude)
    a = (positions.cpu().float()[:, None] * part.inv_freq.cpu()[None, :]).to(F64)       # angles are float32 products
    close(angles, torch.cat([torch.cos(a), torch.sin(a)], dim=1) * amplitude, 1e-5, "cos | sin")


@pytest.mark.parametrize("T", [1, 11, 200])
@pytest.mark.parametrize("H,K,N", [(3, 28, 24), (8, 64, 64), (20, 16, 48), (2, 100, 7), (4, 192, 72), (2, 264, 200)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_matrix_per_head(H, K, N, dtype, T):
    """Sizes in and out of the steps the matrix-core kernel takes (bfloat16, K in steps of 8), few rows and many."""
    from tie_amd import kernels

    wide = rnd(T, H, K + 8, seed=H).to(dtype).cuda()            # heads lie further apart than their width
    x = wide[:, :, :K]
    w = rnd(H, N, K, seed=K, scale=0.3).to(dtype).cuda()
    gate = rnd(T, H, N, seed=N).cuda()
    want = torch.einsum("thk,hnk->thn", x.cpu().to(F64), w.cpu().to(F64))
    out = torch.empty(T, H, N, dtype=dtype, device="cuda")
    kernels.head_linear(x, w, out)
    close(out, want, 1e-6 if dtype == torch.float32 else 8e-3, "a matrix per head")
    kernels.head_linear(x, w, out, gate)
    close(out, want * torch.sigmoid(gate.cpu().to(F64)), 1e-6 if dtype == torch.float32 else 8e-3, "gated")


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_convolution_and_the_norm_over_a_projection(taps):
    """Sequences cut into steps: the state carries the last inputs, also through steps shorter than the taps."""
    from tie_amd import kernels

    nq, nk, nv, eps = 24, 12, 20, 1e-5
    C = nq + nk + nv
    lengths = {0: 11, 1: 5, 2: 1}
    u = {s: rnd(n, C + 3, seed=10 + s) for s, n in lengths.items()}           # rows wider than what is convolved
    w = rnd(C, taps, seed=3)
    wq, wk = 1 + 0.2 * rnd(nq, seed=4), 1 + 0.2 * rnd(nk, seed=5)
    want = {}
    for s, rows in u.items():
        y = plain.short_convolution(rows[:, :C].to(F64), w.to(F64))
        want[s] = torch.cat([plain.rms_norm(y[:, :nq], wq.to(F64), eps), plain.rms_norm(y[:, nq:nq + nk], wk.to(F64), eps),
                             y[:, nq + nk:]], dim=1)
    state = torch.zeros(5, max(taps - 1, 1), C, device="cuda") if taps > 1 else None
    slots = {0: 3, 1: 0, 2: 4}
    # steps: (sequence, rows) lists; sequence 0 in portions of 1, 2, 1, 7; sequence 1 beside it
    plan = [[(0, 1), (1, 3)], [(0, 2)], [(1, 2), (0, 1), (2, 1)], [(0, 7)]]
    at = {s: 0 for s in lengths}
    got = {s: [] for s in lengths}
    for step in plan:
        rows = torch.cat([u[s][at[s]:at[s] + n] for s, n in step]).cuda()
        batch = step_batch([n for _, n in step], [slots[s] for s, _ in step])
        out = torch.empty(rows.shape[0], C, device="cuda")
        kernels.conv_qkv(rows, w.cuda(), taps, state, batch, (nq, nk, nv), out, wq.cuda(), wk.cuda(), eps=eps)
        if taps > 1:
            kernels.conv_state_update(rows, taps, state, batch, C)
        r = 0
        for s, n in step:
            got[s].append(out[r:r + n].cpu())
            r += n
            at[s] += n
    for s in lengths:
        close(torch.cat(got[s]), want[s], 3e-6, f"sequence {s}, {taps} taps")


def chunks_of(counts, rows):
    """A step's rows cut into chunks of at most ``rows``, as the engine hands them to the kernels."""
    from tie_amd import kernels

    items, first, row = [], [0], 0
    for s, n in enumerate(counts):
        pieces = -(-n // rows)
        items += [(s, row + n * i // pieces, row + n * (i + 1) // pieces) for i in range(pieces)]
        row += n
        first.append(len(items))
    return kernels.ScanChunks(i32(items), i32(first), len(items), max(b - a for _, a, b in items))


class Scratch:
    def __init__(self):
        self.memory = {}

    def __call__(self, name, shape, dtype):
        key = (name, tuple(shape), dtype)
        if key not in self.memory:
            self.memory[key] = torch.full(tuple(shape), float("nan"), dtype=dtype, device="cuda")
        return self.memory[key]


@pytest.mark.parametrize("chunk_rows", [None, 1, 3, 7])
@pytest.mark.parametrize("G,H,d,e,taps", [(2, 4, 8, 24, 3), (1, 1, 32, 64, 4), (2, 2, 40, 16, 2), (1, 3, 20, 9, 1),
                                          (2, 2, 64, 80, 3), (1, 2, 128, 128, 4), (1, 1, 200, 70, 2)])
def test_gated_delta_rule_kernels(G, H, d, e, taps, chunk_rows):
    """Rows of projections -> convolution, silu, unit vectors, beta, decays -> the recurrence, sequences cut anywhere
    and states in slots that are not in order, whole or chunk beside chunk; then the gated norm of the heads."""
    from tie_amd import kernels

    silu = torch.nn.functional.silu
    C = 2 * G * d + H * e
    lengths = {0: 37, 1: 6}
    slots = {0: 2, 1: 0}
    proj = {s: rnd(n, C + H, seed=20 + s, scale=1.5) for s, n in lengths.items()}
    arg = {s: rnd(n, H * d, seed=30 + s) for s, n in lengths.items()}
    w = rnd(C, taps, seed=1, scale=0.6)
    A_log, dt_bias = rnd(H, seed=2, scale=0.5), rnd(H * d, seed=3, scale=0.5)
    want = {}
    for s, n in lengths.items():
        y = silu(plain.short_convolution(proj[s][:, :C].to(F64), w.to(F64)))
        q, k, v = y[:, :G * d].view(n, G, d), y[:, G * d:2 * G * d].view(n, G, d), y[:, 2 * G * d:].view(n, H, e)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(proj[s][:, C:].to(F64))
        decay = torch.exp(-torch.exp(A_log.to(F64))[None, :, None] *
                          torch.nn.functional.softplus((arg[s].to(F64) + dt_bias.to(F64)).view(n, H, d)))
        want[s] = torch.cat([plain.delta_rule_scan(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], beta[:, h],
                                                   decay[:, h])[0] for h in range(H)], dim=1)
    conv_state = torch.zeros(3, taps - 1, C, device="cuda") if taps > 1 else None
    state = torch.zeros(3, H, d, e, device="cuda")
    plan = [[(0, 9), (1, 1)], [(1, 2), (0, 1)], [(0, 2)], [(0, 20), (1, 3)], [(0, 5)]]
    at = {s: 0 for s in lengths}
    got = {s: [] for s in lengths}
    for step in plan:
        rows = torch.cat([proj[s][at[s]:at[s] + n] for s, n in step]).cuda()
        a = torch.cat([arg[s][at[s]:at[s] + n] for s, n in step]).cuda()
        batch = step_batch([n for _, n in step], [slots[s] for s, _ in step])
        T = rows.shape[0]
        tok = torch.empty(T, C + H + H * d, device="cuda")
        kernels.delta_prepare(rows, w.cuda(), taps, conv_state, batch, a, A_log.cuda(), dt_bias.cuda(), G, H, d, e, tok)
        if taps > 1:
            kernels.conv_state_update(rows, taps, conv_state, batch, C)
        out = torch.empty(T, H * e, device="cuda")
        chunks = chunks_of([n for _, n in step], chunk_rows) if chunk_rows else None
        kernels.gated_delta_scan(tok, out, state, batch, G, H, d, e, chunks=chunks, scratch=Scratch())
        r = 0
        for s, n in step:
            got[s].append(out[r:r + n].cpu())
            r += n
            at[s] += n
    for s in lengths:
        close(torch.cat(got[s]), want[s], 2e-5, f"sequence {s}")
    assert float(state[1].abs().max()) == 0.0                    # a slot no sequence holds stays as it was
    o = torch.cat(got[0]).cuda()
    gate, nw = rnd(o.shape[0], H * e, seed=5).cuda(), (1 + 0.2 * rnd(e, seed=6)).cuda()
    normed = torch.empty_like(o)
    kernels.grouped_gated_rms_norm(o, nw, 1e-5, gate, normed, H)
    ref = plain.rms_norm(o.cpu().to(F64).view(-1, H, e), nw.cpu().to(F64), 1e-5).view(-1, H * e) * \
        torch.sigmoid(gate.cpu().to(F64))
    close(normed, ref, 3e-6, "gated norm a head")


# ------------------------------------------------------------------------------------------- whole models
LENGTHS = {"A": [1, 2, 9, 23, 40, 64, 37], "B": [5, 17, 33, 70, 128], "C": [1, 3, 30, 77, 18], "D": [2, 50, 21, 8],
           "E": [1, 45, 90, 6]}
TOLERANCE = {"float32": 3e-5, "bfloat16": 8e-2}        # of the largest logit; the queries are drawn wide


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, config in CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            folder = tmp_path_factory.mktemp(f"minerax_{name}_{dtype}")
            out[name, dtype] = write_model(folder, config, seed=41 + len(out), dtype=dtype)
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
        return TraceReplayer.from_folder(folder, dtype, max_tokens, block_size=bs, state_slots=4)

    results = {"whole": th.collect(replayer(biggest), th.whole(requests)),
               "prefill+decode": th.collect(replayer(biggest), th.prefill_then_decode(requests, tail=40)),
               "portions": th.collect(replayer(biggest), th.portions(requests)),
               "portions of two": th.collect(replayer(biggest), th.portions(requests, sizes=(2,))),
               "token by token": th.collect(replayer(biggest), th.portions(requests, sizes=(1,)))}
    steps, peak = th.mixed(requests, max_live=4, seed=3)
    assert max(len(s["entries"]) for s in steps) >= 3
    rep = replayer(peak)
    results["mixed"] = th.collect(rep, steps)
    assert rep.cache.all_free()                                   # every page and slot came back
    for label, got in results.items():
        check(got, want, TOLERANCE[dtype], f"{name}/{dtype}/{label}")
    if dtype == "float32":       # the ways of cutting agree with each other beyond what they owe the plain one
        for label in results:
            for rid in requests:
                a = torch.stack([results["whole"][rid][p] for p in range(len(requests[rid]))])
                b = torch.stack([results[label][rid][p] for p in range(len(requests[rid]))])
                assert float((a - b).abs().max() / a.abs().max()) < 1e-5, f"{name}: whole vs {label}, request {rid}"


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
        close(mine, ref, 1e-5, f"{name}: the streams' sum after layer {i}")


def _altered(config, change):
    other = copy.deepcopy(config)
    change(other)
    return other


def test_a_fault_of_one_position_or_one_term_would_show(folders):
    """The engine agrees with the plain model, and the plain model with one mechanism slightly off does not agree
    with the engine by a wide margin: a window one longer or shorter, a lost sink, a farthest key that is dropped, a
    convolution of one tap fewer, streams mixed the other way round."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["A", "float32"], CONFIGS["A"]
    requests = th.make_requests(config["vocab"], [48, 31], seed=21)
    got = th.collect(TraceReplayer.from_folder(folder, "float32", 128, block_size=BLOCK_SIZE["A"]),
                     th.prefill_then_decode(requests, tail=20))
    weights = load_plain(folder)
    right = worst_error(got, reference(folder, config, requests))
    assert right < TOLERANCE["float32"]

    def off(label, config_change=None, weight_change=None):
        cfg = _altered(config, config_change) if config_change else config
        w = dict(weights)
        if weight_change:
            weight_change(w)
        want = {rid: plain.forward(cfg, w, toks)[0].float() for rid, toks in requests.items()}
        err = worst_error(got, want)
        print(f"[observed] {label}: {err:.3e}")
        assert err > 100 * TOLERANCE["float32"], f"{label} does not show in the logits ({err:.3e})"

    for layer in (0, 2):
        size = config["layers"][layer]["mixer"]["mask"]["size"]
        off(f"layer {layer}: a window one longer", lambda c: c["layers"][layer]["mixer"]["mask"].update(size=size + 1))
        off(f"layer {layer}: a window one shorter", lambda c: c["layers"][layer]["mixer"]["mask"].update(size=size - 1))
        off(f"layer {layer}: no sink", None, lambda w: w.pop(f"l{layer}.mix.sink"))
    off("a left attention that sees only the last twenty keys",
        lambda c: c["layers"][1]["mixer"]["left"].update(mask={"size": 20}))
    off("a capped score left uncapped", lambda c: c["layers"][1]["mixer"]["left"].pop("softcap"))

    def drop_first_tap(w):
        for name in ("left.q", "left.k", "left.v", "right.q", "right.k", "right.v"):
            key = f"l1.mix.{name}.conv"
            w[key] = torch.cat([torch.zeros_like(w[key][:, :1]), w[key][:, 1:]], dim=1)

    off("a convolution that forgets its oldest input", None, drop_first_tap)
    off("streams mixed [to, from]", None,
        lambda w: [w.__setitem__(k, w[k].T.contiguous()) for k in list(w) if k.endswith(".mix") and ".hc" in k])
    off("a decay of one forgets nothing", None, lambda w: w.__setitem__("l1.mix.right.A_log", w["l1.mix.right.A_log"] - 30.0))


def test_a_far_key_decides_a_decoded_token(tmp_path):
    """A prompt of hundreds of tokens in which one early token alone answers the last query of the attention
    without a window: the query matrix is made so that the last token's query points along that token's key, so
    a lost or misplaced page shows in the logits."""
    from minerax_fixtures import make_tensors
    from tie_amd.engine.replay import TraceReplayer
    from tie_amd.weights.safetensors_io import write_safetensors

    config = {"architecture": "Minerax", "vocab": 50, "width": 32, "norm": {"eps": 1e-5}, "streams": 2,
              "layers": [{"type": "parallel", "mlp": None,
                          "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "conv": 1, "scale": 2.0},
                                    "right": {"heads": 1, "kv_heads": 1, "dim": 8, "vdim": 8, "conv": 2},
                                    "left_scale": 1.0, "right_scale": 0.1}}]}
    tensors = make_tensors(config, 77, "float32")
    w = {k: v.to(F64) for k, v in tensors.items()}
    eps, asked, answer = 1e-5, 48, 49

    def mixer_input(token):             # the first layer's rows depend on the token alone
        return plain.layer_norm(w["l0.hc1.in"].sum() * w["embed"][token], w["l0.norm1"], eps)

    key = plain.rms_norm(w["l0.mix.left.k.conv"][:, 0] * (w["l0.mix.left.k"] @ mixer_input(answer)),
                         w["l0.mix.left.k.norm"], eps)
    target = torch.cat([key, key]) / (w["l0.mix.left.q.conv"][:, 0] * w["l0.mix.left.q.norm"])
    h = mixer_input(asked)
    tensors["l0.mix.left.q"] = (target[:, None] * h[None, :] / (h * h).sum()).float()     # W_q h(asked) = target
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
        rep = TraceReplayer.from_folder(str(folder), "float32", 704, block_size=16)
        steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:cut], "want": [699] if cut == 700 else []}],
                  "end": []}]
        steps += [{"step": i, "entries": [{"id": "a", "tokens": [tokens[i]], "want": [0]}], "end": []}
                  for i in range(cut, 700)]
        got = th.collect(rep, steps)
        err = float((got["a"][699] - full[699]).abs().max() / full[699].abs().max())
        assert err < TOLERANCE["float32"], f"cut at {cut}: {err:.3e}"


def test_long_decoding_through_windows_with_pages_given_back_and_used_again(folders):
    """Two requests decode 150 tokens each in a pool that holds them only because the windows' pages go back;
    a third then runs in the pages and the slot they left."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["E", "float32"], CONFIGS["E"]
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
    rep = TraceReplayer.from_folder(folder, "float32", 192, block_size=16)       # 12 pages: far fewer than 335 tokens
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE["float32"], "long decoding")


def test_long_portions_run_the_delta_rule_chunk_beside_chunk(folders, monkeypatch):
    """Portions long enough for the three-launch walk (made to start at fewer rows here, in smaller chunks), beside a
    short one and a single token, against the plain model and against the same requests in short portions."""
    from tie_amd import kernels
    from tie_amd.engine.replay import TraceReplayer

    monkeypatch.setattr(kernels, "DELTA_CHUNKS_FROM", 400)
    monkeypatch.setattr(kernels, "DELTA_CHUNK_ROWS", 96)
    folder, config = folders["D", "float32"], CONFIGS["D"]
    requests = th.make_requests(config["vocab"], [700, 560, 40], seed=17)
    want = reference(folder, config, requests)
    a, b, c = requests["r0"], requests["r1"], requests["r2"]
    steps = [
        {"step": 0, "entries": [{"id": "r2", "tokens": c[:39], "want": list(range(39))}], "end": []},
        {"step": 1, "entries": [{"id": "r0", "tokens": a[:670], "want": list(range(670))},
                                {"id": "r2", "tokens": c[39:], "want": [0]},
                                {"id": "r1", "tokens": b[:10], "want": list(range(10))}], "end": ["r2"]},
        {"step": 2, "entries": [{"id": "r1", "tokens": b[10:], "want": list(range(550))},
                                {"id": "r0", "tokens": a[670:], "want": list(range(30))}], "end": ["r0", "r1"]},
    ]
    rep = TraceReplayer.from_folder(folder, "float32", 1408, block_size=BLOCK_SIZE["D"])
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE["float32"], "long portions")
    short = th.collect(TraceReplayer.from_folder(folder, "float32", 1408, block_size=BLOCK_SIZE["D"]),
                       th.portions({"r0": a}, sizes=(97, 150, 33)))
    mine = torch.stack([got["r0"][p] for p in range(len(a))])
    other = torch.stack([short["r0"][p] for p in range(len(a))])
    assert float((mine - other).abs().max() / mine.abs().max()) < 1e-5


def test_state_slots_are_cleared_when_they_are_used_again(folders):
    """Six requests through two state slots, one after another and side by side: every request starts from a zero
    state and an empty convolution history whatever its slot held before."""
    from tie_amd.engine.replay import TraceReplayer

    folder, config = folders["D", "float32"], CONFIGS["D"]
    requests = th.make_requests(config["vocab"], [30, 7, 19, 3, 26, 11], seed=13)
    want = reference(folder, config, requests)
    steps, peak = th.mixed(requests, max_live=2, seed=6, tail=5)
    rep = TraceReplayer.from_folder(folder, "float32", peak, block_size=BLOCK_SIZE["D"], state_slots=2)
    got = th.collect(rep, steps)
    assert rep.cache.all_free()
    check(got, want, TOLERANCE["float32"], "slots used again")


@pytest.mark.parametrize("name", ["A", "B"])
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
@pytest.mark.parametrize("name", ["A", "B", "D"])
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
    """JSON lines in, .f32 files and 'done' lines out; four slots, pages used again."""
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
