"""The plain Minerax pinned by cases worked out by hand, and the design's reader, spec and cache needs (CPU)."""

import copy
import math

import pytest
import torch

import plain_minerax as plain
from minerax_fixtures import CONFIGS

F64 = torch.float64


def test_layer_norm_by_hand():
    x = torch.tensor([[1.0, 3.0, 5.0, 7.0]], dtype=F64)
    out = plain.layer_norm(x, torch.tensor([1.0, 2.0, 1.0, 0.5], dtype=F64), 0.0)
    # mean 4, squared deviations 9 1 1 9: variance 5
    r = math.sqrt(5.0)
    assert torch.allclose(out, torch.tensor([[-3 / r, -2 / r, 1 / r, 1.5 / r]], dtype=F64))
    shifted = plain.layer_norm(x + 100.0, torch.ones(4, dtype=F64), 0.0)
    assert torch.allclose(shifted, plain.layer_norm(x, torch.ones(4, dtype=F64), 0.0))       # the mean goes


def test_gelu_tanh_by_hand():
    z = torch.tensor([0.0, 1.0, -2.0], dtype=F64)
    want = [0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in (0.0, 1.0, -2.0)]
    assert torch.allclose(plain.gelu_tanh(z), torch.tensor(want, dtype=F64))
    assert abs(float(plain.gelu_tanh(torch.tensor(1.0, dtype=F64))) - 0.8411919906082768) < 1e-12


def test_stretched_frequencies_by_hand():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 16, "fast": 2.0, "slow": 0.5}}
    freq, amplitude = plain.stretched_frequencies(rot)
    # dim(t) = 8 ln(16 / (2 pi t)) / (2 ln 100): dim(2) = 0.2098.., dim(0.5) = 1.4139..: lo 0, hi 2
    lo = math.floor(8 * math.log(16 / (4 * math.pi)) / (2 * math.log(100.0)))
    hi = math.ceil(8 * math.log(16 / math.pi) / (2 * math.log(100.0)))
    assert (lo, hi) == (0, 2)
    plain_f = [100.0 ** (-2 * i / 8) for i in range(4)]
    ramp = [0.0, 0.5, 1.0, 1.0]
    want = [f / 4.0 * r + f * (1 - r) for f, r in zip(plain_f, ramp)]
    assert torch.allclose(freq, torch.tensor(want, dtype=F64))
    assert amplitude == 0.1 * math.log(4.0) + 1.0
    freq, amplitude = plain.stretched_frequencies({"dims": 8, "base": 100.0})
    assert torch.allclose(freq, torch.tensor(plain_f, dtype=F64)) and amplitude == 1.0
    # a ramp whose ends meet: the divisor's floor keeps it a step
    tight = {"dims": 4, "base": 10.0, "scaling": {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}}
    freq, _ = plain.stretched_frequencies(tight)
    d = 4 * math.log(8 / (2 * math.pi)) / (2 * math.log(10.0))
    lo, hi = max(math.floor(d), 0), min(math.ceil(d), 3)
    ramp = [min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(2)]
    assert torch.allclose(freq, torch.tensor([10.0 ** (-i / 2) * (1 - r / 2) for i, r in zip(range(2), ramp)], dtype=F64))


def test_both_pairings_of_the_rotation():
    x = torch.arange(1, 7, dtype=F64).view(1, 1, 6).repeat(2, 1, 1)
    rot = {"dims": 4, "base": 100.0}
    a0, a1 = 1.0, 100.0 ** -0.5                          # position 1
    half = plain.rotate(x, rot, False)
    assert half[0].flatten().tolist() == [1, 2, 3, 4, 5, 6]
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5, 6]
    assert torch.allclose(half[1].flatten(), torch.tensor(want, dtype=F64))
    inter = plain.rotate(x, rot, True)
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 2 * math.cos(a0) + 1 * math.sin(a0),
            3 * math.cos(a1) - 4 * math.sin(a1), 4 * math.cos(a1) + 3 * math.sin(a1), 5, 6]
    assert torch.allclose(inter[1].flatten(), torch.tensor(want, dtype=F64))
    # the amplitude multiplies cosine and sine, so the rotated part grows and the rest does not
    scaled = plain.rotate(x, {**rot, "scaling": {"factor": math.e ** 5, "original": 1e9, "fast": 1e-9, "slow": 1e-9}}, True)
    assert torch.allclose(scaled[0].flatten(), torch.tensor([1.5, 3.0, 4.5, 6.0, 5, 6], dtype=F64))


def test_short_convolution_by_hand():
    u = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]], dtype=F64)
    w = torch.tensor([[100.0, 10.0, 1.0], [0.0, 0.0, 2.0]], dtype=F64)       # the last column is the current token's
    out = plain.short_convolution(u, w)
    assert out[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0]
    assert out[:, 1].tolist() == [20.0, 40.0, 60.0, 80.0]
    assert torch.equal(plain.short_convolution(u, torch.tensor([[3.0], [1.0]], dtype=F64)), u * torch.tensor([3.0, 1.0]))


def test_the_window_counts_the_token_itself():
    allowed = plain.visible(6, 3)
    assert allowed[0].tolist() == [True, False, False, False, False, False]
    assert allowed[4].tolist() == [False, False, True, True, True, False]
    assert plain.visible(4, 1).int().tolist() == torch.eye(4, dtype=torch.int32).tolist()
    assert plain.visible(4)[3].tolist() == [True] * 4


def test_the_sink_counts_once_unscaled_and_has_no_value():
    scores = torch.tensor([[[0.0, math.log(2.0)]]], dtype=F64)
    mask = torch.tensor([[True, True]])
    w = plain.softmax_with_sink(scores, mask, torch.tensor([math.log(5.0)], dtype=F64))
    assert torch.allclose(w, torch.tensor([[[1 / 8, 2 / 8]]], dtype=F64))
    assert torch.allclose(plain.softmax_with_sink(scores, mask), torch.tensor([[[1 / 3, 2 / 3]]], dtype=F64))
    w = plain.softmax_with_sink(scores, mask, torch.tensor([800.0], dtype=F64))
    assert float(w.sum()) < 1e-300


def test_one_step_of_the_delta_rule_by_hand():
    q = torch.tensor([[1.0, 0.0], [1.0, 1.0]], dtype=F64)
    k = torch.tensor([[1.0, 0.0], [1.0, 1.0]], dtype=F64)
    v = torch.tensor([[2.0, 4.0], [1.0, 1.0]], dtype=F64)
    beta = torch.tensor([0.5, 1.0], dtype=F64)
    decay = torch.tensor([[1.0, 1.0], [0.5, 0.25]], dtype=F64)
    out, S = plain.delta_rule_scan(q, k, v, beta, decay)
    # token 0: S = 0; u = 0.5 v = [1, 2]; S = k u^T = [[1, 2], [0, 0]]; o = S^T q = [1, 2]
    assert out[0].tolist() == [1.0, 2.0]
    # token 1: S <- rows times (0.5, 0.25) = [[0.5, 1], [0, 0]]; S^T k = [0.5, 1]; u = [0.5, 0]; S = [[1, 1], [0.5, 0]]
    assert S.tolist() == [[1.0, 1.0], [0.5, 0.0]]
    assert out[1].tolist() == [1.5, 1.0]                 # the read-out sees the current token's write
    again, S2 = plain.delta_rule_scan(q[1:], k[1:], v[1:], beta[1:], decay[1:],
                                      state=torch.tensor([[1.0, 2.0], [0.0, 0.0]], dtype=F64))
    assert torch.equal(again[0], out[1]) and torch.equal(S2, S)
    # beta 1 and no decay: the state then answers v for k exactly
    k1 = torch.tensor([[0.6, 0.8]], dtype=F64)
    _, S = plain.delta_rule_scan(k1, k1, torch.tensor([[3.0, -1.0]], dtype=F64), torch.ones(1, dtype=F64),
                                 torch.ones(1, 2, dtype=F64), state=torch.tensor([[1.0, 2.0], [3.0, 4.0]], dtype=F64))
    assert torch.allclose(S.T @ k1[0], torch.tensor([3.0, -1.0], dtype=F64))


def _tiny(streams):
    config = {"architecture": "Minerax", "vocab": 5, "width": 4, "norm": {"eps": 1e-5}, "layers": [
        {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 3},
         "mixer": {"heads": 1, "dim": 2, "rot_dim": 2, "vdim": 2, "kv_rank": 2, "scale": 1.0,
                   "rot": {"dims": 2, "base": 10.0}}}]}
    if streams:
        config["streams"] = streams
    g = torch.Generator().manual_seed(0)
    shapes = {"embed": (5, 4), "head": (5, 4), "final.norm": (4,), "l0.norm1": (4,), "l0.norm2": (4,),
              "l0.mix.q": (4, 4), "l0.mix.dkv": (4, 4), "l0.mix.dkv.norm": (2,), "l0.mix.uk": (2, 2),
              "l0.mix.uv": (2, 2), "l0.mix.sink": (1,), "l0.mix.g": (2, 4), "l0.mix.o": (4, 2),
              "l0.mlp.gate": (3, 4), "l0.mlp.up": (3, 4), "l0.mlp.down": (4, 3)}
    w = {n: torch.randn(*s, generator=g, dtype=F64) for n, s in shapes.items()}
    return config, w


def test_streams_that_only_pass_the_sum_are_the_plain_residual():
    """With ``in`` = (1, 0), ``mix`` = identity and ``out`` = (1, 0), stream 0 is the pre-norm residual and stream 1
    stays the embedding; the folded sum is their sum."""
    config, w = _tiny(None)
    want, _ = plain.forward(config, w, [1, 4, 2])
    config2, _ = _tiny(2)
    for q in (1, 2):
        w[f"l0.hc{q}.in"] = torch.tensor([1.0, 0.0], dtype=F64)
        w[f"l0.hc{q}.out"] = torch.tensor([1.0, 0.0], dtype=F64)
        w[f"l0.hc{q}.mix"] = torch.eye(2, dtype=F64)
    _, behind = plain.forward(config2, w, [1, 4, 2])
    _, single = plain.forward(config, w, [1, 4, 2])
    assert torch.allclose(behind[0], single[0] + w["embed"][torch.tensor([1, 4, 2])])
    # mix is indexed [from, to]: sending stream 1 into stream 0 only
    w["l0.hc1.mix"] = torch.tensor([[0.0, 0.0], [1.0, 0.0]], dtype=F64)
    w["l0.hc1.out"] = torch.zeros(2, dtype=F64)
    w["l0.hc2.mix"] = torch.eye(2, dtype=F64)
    w["l0.hc2.out"] = torch.zeros(2, dtype=F64)
    _, behind = plain.forward(config2, w, [3])
    assert torch.allclose(behind[0], w["embed"][torch.tensor([3])])      # stream 0 = old stream 1, stream 1 = 0
    assert want.shape == (3, 5)


# ----------------------------------------------------------------------------------- reader, registry, spec
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_reader_and_the_spec(name):
    import tie_amd  # noqa: F401
    from tie_amd.cache.spec import FixedState, PagedKV
    from tie_amd.models.builder import model_from_config

    config = CONFIGS[name]
    model = model_from_config(config)
    assert model.spec.architecture == "Minerax"
    names = {s.name for s in model.expected_tensors()}
    assert {"embed", "final.norm", "head"} <= names
    needs = [g.need for g in model.cache_plan.groups]
    for i, layer in enumerate(config["layers"]):
        m = layer["mixer"]
        p = f"l{i}.mix."
        if layer["type"] == "latent_attention":
            assert {p + k for k in ("q", "dkv", "dkv.norm", "uk", "uv", "sink", "g", "o")} <= names
            size = -(-(m["kv_rank"] + m["rot_dim"]) // 16) * 16
            assert PagedKV(1, size, (m.get("mask") or {}).get("size")) in needs        # one head: nothing per head
        else:
            left, right = m["left"], m["right"]
            assert {p + "left." + k for k in ("q", "k", "v", "o", "q.norm", "k.norm", "q.conv", "k.conv", "v.conv")} <= names
            assert {p + "right." + k for k in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o", "A_log", "dt_bias", "norm",
                                               "q.conv", "k.conv", "v.conv")} <= names
            assert FixedState((right["heads"], right["dim"], right["vdim"])) in needs
            channels = 2 * right["kv_heads"] * right["dim"] + right["heads"] * right["vdim"]
            if right["conv"] > 1:
                assert FixedState((right["conv"] - 1, channels)) in needs
            else:
                assert not any(isinstance(n, FixedState) and n.shape[-1] == channels for n in needs)
            assert any(isinstance(n, PagedKV) and n.num_kv_heads == left["kv_heads"] for n in needs)
        for q, part in ((1, True), (2, layer["mlp"] is not None)):
            assert (f"l{i}.norm{q}" in names) == part
            assert (f"l{i}.hc{q}.mix" in names) == (part and "streams" in config)
    assert model.capturable()


def test_what_does_not_fit_is_refused():
    import tie_amd  # noqa: F401
    from tie_amd.errors import LoadError, UnsupportedError
    from tie_amd.models.builder import model_from_config

    def changed(path, value):
        config = copy.deepcopy(CONFIGS["A"])
        node = config
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        return config

    for path, value, error in [
        (("layers", 0, "mixer", "kv_rank"), 0, LoadError),
        (("layers", 0, "mixer", "rot", "dims"), 10, LoadError),               # more than the rotated part holds
        (("layers", 0, "mixer", "mask", "size"), 0, LoadError),
        (("layers", 0, "mixer", "rot", "scaling", "factor"), 0.0, LoadError),
        (("layers", 1, "mixer", "left", "kv_heads"), 3, LoadError),
        (("layers", 1, "mixer", "left", "rot", "dims"), 7, LoadError),
        (("layers", 1, "mixer", "left", "rot", "dims"), 18, LoadError),
        (("layers", 1, "mixer", "left", "conv"), 0, LoadError),
        (("layers", 1, "mixer", "left", "softcap"), -2.0, LoadError),
        (("layers", 1, "mixer", "right", "kv_heads"), 3, LoadError),
        (("layers", 1, "mixer", "right", "conv"), 99, Exception),
        (("layers", 2, "type"), "lstm", UnsupportedError),
        (("layers", 0, "mlp", "kind"), "moe", UnsupportedError),
        (("norm", "eps"), 0.0, LoadError),
        (("streams",), 0, LoadError),
        (("streams",), 99, Exception),
        (("width",), 0, LoadError),
    ]:
        with pytest.raises(error):
            model_from_config(changed(path, value))


def test_the_frequencies_the_engine_makes_are_the_plain_ones():
    import tie_amd  # noqa: F401
    from tie_amd.parts.base import PartSpec, build_part

    for rot in ({"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 16, "fast": 2.0, "slow": 0.5}},
                {"dims": 32, "base": 5000.0, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}},
                {"dims": 4, "base": 10.0, "scaling": {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0}},
                {"dims": 16, "base": 1e6}):
        part = build_part("position", PartSpec("rope_yarn", {"head_dim": 64, "theta": rot["base"], "rotary_dim": rot["dims"],
                                                             "pairing": "interleaved", "scaling": rot.get("scaling")}))
        freq, amplitude = plain.stretched_frequencies(rot)
        assert torch.allclose(torch.from_numpy(part.host_inv_freq()).double(), freq, rtol=1e-6)
        assert abs(part.amplitude - amplitude) < 1e-12


def test_a_mixer_of_several_needs_gets_them_in_order():
    from tie_amd.cache.spec import CallCaches, FixedState, PagedKV, plan_cache

    pages, conv, state = PagedKV(2, 16), FixedState((2, 96)), FixedState((4, 8, 24))
    plan = plan_cache([PagedKV(1, 48, 9), (pages, conv, state, FixedState((2, 112))), None, (pages, conv)],
                      [None, None, None, None])
    first, second, third, fourth = plan.calls
    assert not isinstance(first, CallCaches) and third is None
    assert isinstance(second, CallCaches) and len(second) == 4 and isinstance(fourth, CallCaches) and len(fourth) == 2
    assert [plan.groups[c.group].need for c in second] == [pages, conv, state, FixedState((2, 112))]
    assert fourth[0].group == second[0].group and fourth[0].plane != second[0].plane       # same group, own plane
    assert fourth[1].group == second[1].group and fourth[1].plane != second[1].plane
    assert all(c.writes for c in second) and all(c.writes for c in fourth)


def test_windows_give_their_pages_back_and_slots_come_back():
    from tie_amd.cache.manager import FREED, CacheManager
    from tie_amd.cache.spec import FixedState, PagedKV, plan_cache

    need = PagedKV(1, 48, 9)
    assert [need.first_needed(p) for p in (0, 8, 9, 25)] == [0, 0, 1, 17]
    plan = plan_cache([need, (PagedKV(2, 16), FixedState((1, 96)), FixedState((4, 8, 24)))], [None, None])
    cache = CacheManager(plan, block_size=4, num_blocks=16, max_state_slots=2)
    a = cache.new_request()
    assert cache.reserve(a, 23)
    assert cache.trim(a, 23) == 3                       # positions 0..14 are out of every later window: 3 whole pages
    assert a.tables[0][:4] == [FREED] * 3 + [a.tables[0][3]] and FREED not in a.tables[1]
    b, c = cache.new_request(), cache.new_request()
    assert cache.reserve(b, 8) and b.state_slot != a.state_slot
    assert not cache.reserve(c, 4)                      # two slots, both taken
    slot = a.state_slot
    cache.release(a)
    assert cache.reserve(c, 4) and c.state_slot == slot
    cache.release(b)
    cache.release(c)
    assert cache.all_free()
