"""The plain Zovudra pinned by cases worked out by hand, and the design's reader, spec and cache needs (CPU)."""

import copy
import math

import pytest
import torch

import plain_zovudra as plain
from zovudra_fixtures import CONFIGS

F64 = torch.float64


def test_dynamic_tanh_by_hand():
    x = torch.tensor([[0.0, 1.0, -2.0]], dtype=F64)
    out = plain.dynamic_tanh(x, 0.5, torch.tensor([2.0, 2.0, 1.0], dtype=F64), torch.tensor([0.1, 0.0, -1.0], dtype=F64))
    assert torch.allclose(out, torch.tensor([[0.1, 2 * math.tanh(0.5), -math.tanh(1.0) - 1.0]], dtype=F64))
    # no statistics: a row's values do not know of each other
    wide = plain.dynamic_tanh(torch.tensor([[0.0, 1.0, 500.0]], dtype=F64), 0.5, torch.ones(3, dtype=F64), torch.zeros(3, dtype=F64))
    assert abs(float(wide[0, 1]) - math.tanh(0.5)) < 1e-15 and float(wide[0, 2]) == 1.0


def test_banded_frequencies_by_hand():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
    f = [100.0 ** (-2 * i / 8) for i in range(4)]                 # 1, 0.316, 0.1, 0.0316: wavelengths 6.3, 19.9, 62.8, 198.7
    # below 64 / 4 = 16: kept; above 64 / 1 = 64: divided by 4; 19.9 and 62.8 lie between
    blend = [(64 / (2 * math.pi / v) - 1.0) / 3.0 for v in f]
    want = [f[0], (1 - blend[1]) * f[1] / 4 + blend[1] * f[1], (1 - blend[2]) * f[2] / 4 + blend[2] * f[2], f[3] / 4]
    assert torch.allclose(plain.banded_frequencies(rot), torch.tensor(want, dtype=F64))
    assert 0 < blend[2] < blend[1] < 1
    assert torch.allclose(plain.banded_frequencies({"dims": 8, "base": 100.0}), torch.tensor(f, dtype=F64))


def test_both_pairings_of_the_rotation():
    x = torch.arange(1, 7, dtype=F64).view(1, 1, 6).repeat(2, 1, 1)
    rot = {"dims": 4, "base": 100.0}
    positions = torch.tensor([0, 1])
    a0, a1 = 1.0, 100.0 ** -0.5                          # the angles at position 1
    half = plain.rotate(x, positions, rot, False)
    assert half[0].flatten().tolist() == [1, 2, 3, 4, 5, 6]               # position 0 turns nothing
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5, 6]
    assert torch.allclose(half[1].flatten(), torch.tensor(want, dtype=F64))
    inter = plain.rotate(x, positions, rot, True)
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 2 * math.cos(a0) + 1 * math.sin(a0),
            3 * math.cos(a1) - 4 * math.sin(a1), 4 * math.cos(a1) + 3 * math.sin(a1), 5, 6]
    assert torch.allclose(inter[1].flatten(), torch.tensor(want, dtype=F64))


def test_the_window_counts_the_token_itself_and_kept_positions_stay():
    mask = plain.visible(8, 3, 2)
    assert mask[7].tolist() == [True, True, False, False, False, True, True, True]       # 0, 1 kept; 5, 6, 7 near
    assert mask[3].tolist() == [True, True, True, True, False, False, False, False]      # the two ranges meet
    assert mask[1].tolist() == [True, True] + [False] * 6
    assert plain.visible(5, 1)[4].tolist() == [False] * 4 + [True]                        # a window of one: itself
    assert plain.visible(4, None)[3].tolist() == [True] * 4
    assert plain.visible(6, 2, 9)[5].tolist() == [True] * 6                               # more kept than there are


def test_a_routing_choice_by_hand():
    s = torch.tensor([[0.9, 0.1, 0.6, 0.6, 0.8, 0.3]], dtype=F64)
    z = torch.log(s / (1 - s))
    # groups of two: sums of the two best 1.0, 1.2, 1.1: with two groups kept, experts 2..5 stay; the best two of them
    chosen, weights = plain.route(z, {"experts": 6, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 2}})
    assert sorted(chosen[0].tolist()) == [2, 4] or sorted(chosen[0].tolist()) == [3, 4]
    assert torch.allclose(weights.sort().values, torch.tensor([[3 * 0.6 / 1.4, 3 * 0.8 / 1.4]], dtype=F64))
    chosen, weights = plain.route(z, {"experts": 6, "top": 2})                           # no groups, no factor
    assert chosen[0].tolist() == [0, 4] and torch.allclose(weights, torch.tensor([[0.9 / 1.7, 0.8 / 1.7]], dtype=F64))
    chosen, _ = plain.route(z, {"experts": 6, "top": 1, "groups": {"count": 3, "keep": 1}})
    assert chosen[0].tolist() == [2]                     # the best expert's group lost to the group of two even ones


def test_an_expert_squares_what_relu_leaves():
    h = torch.tensor([1.0, -1.0], dtype=F64)
    up = torch.tensor([[2.0, 0.0], [0.0, 3.0], [1.0, 1.0]], dtype=F64)       # sums 2, -3, 0
    down = torch.tensor([[1.0, 1.0, 1.0], [0.5, 7.0, 7.0]], dtype=F64)
    assert plain.expert(h, up, down).tolist() == [4.0, 2.0]


def test_the_side_input_takes_the_layers_own_columns():
    w = {"side.embed": torch.arange(12, dtype=F64).view(2, 6), "l1.side.gate": torch.ones(3, 2, dtype=F64),
         "l1.side.proj": torch.eye(3, dtype=F64)[:2], "l1.side.norm": torch.tensor([2.0, 1.0], dtype=F64)}
    x = torch.tensor([[0.5, 0.5]], dtype=F64)
    out = plain.token_side(x, torch.tensor([1]), w, 1, 3, 0.0)
    g = float(plain.gelu_tanh(torch.tensor(1.0, dtype=F64)))
    y = torch.tensor([g * 9.0, g * 10.0], dtype=F64)                # token 1, columns 3..5: 9, 10, 11; proj keeps two
    want = y / torch.sqrt((y * y).mean()) * torch.tensor([2.0, 1.0], dtype=F64)
    assert torch.allclose(out, want[None])


# ----------------------------------------------------------------------------------- reader, registry, spec
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_the_reader_and_the_spec(name):
    import tie_amd  # noqa: F401
    from tie_amd.cache.spec import PagedKV
    from tie_amd.models.builder import model_from_config

    config = CONFIGS[name]
    model = model_from_config(config)
    assert model.spec.architecture == "Zovudra"
    names = {s.name for s in model.expected_tensors()}
    assert {"embed", "final.norm", "final.norm.b", "final.norm.alpha", "head"} <= names
    assert ("side.embed" in names) == ("token_side" in config)
    needs = [g.need for g in model.cache_plan.groups]
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        mask = m.get("mask") or {}
        if layer["type"] == "latent_attention":
            assert {p + k for k in ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "o")} <= names
            size = -(-(m["kv_rank"] + m["rot_dim"]) // 16) * 16
            assert PagedKV(1, size, mask.get("size")) in needs        # one head: nothing per head
        else:
            assert {p + k for k in ("q", "k", "v", "o", "q.norm", "k.norm")} <= names
            assert any(n.num_kv_heads == m["kv_heads"] and n.window == mask.get("size") and
                       n.keep_first == (mask.get("keep_first", 0) if mask.get("size") else 0) for n in needs)
        mlp = layer["mlp"]
        assert (f"l{i}.norm2.alpha" in names) == (mlp is not None)
        if mlp is not None and mlp["kind"] == "moe":
            experts = mlp["router"]["experts"]
            assert {f"l{i}.mlp.e{e}.{k}" for e in range(experts) for k in ("up", "down")} <= names
            assert f"l{i}.mlp.e{experts}.up" not in names and f"l{i}.mlp.router" in names
            assert (f"l{i}.mlp.shared.sg" in names) == ("shared" in mlp)
        assert (f"l{i}.side.gate" in names) == ("token_side" in config)
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
        (("layers", 0, "mixer", "kv_heads"), 3, LoadError),
        (("layers", 0, "mixer", "rot", "dims"), 18, LoadError),               # more than a head holds
        (("layers", 0, "mixer", "rot", "dims"), 7, LoadError),
        (("layers", 0, "mixer", "mask", "size"), 0, LoadError),
        (("layers", 0, "mixer", "mask", "keep_first"), -1, LoadError),
        (("layers", 0, "mixer", "rot", "scaling", "factor"), 0.0, LoadError),
        (("layers", 0, "mixer", "rot", "scaling", "high"), 2.0, LoadError),   # equal to low: no band between
        (("layers", 0, "mlp", "router", "top"), 5, LoadError),                # two groups of two stay: four experts
        (("layers", 0, "mlp", "router", "groups", "count"), 3, LoadError),
        (("layers", 0, "mlp", "shared", "ff"), 0, LoadError),
        (("layers", 0, "mlp", "kind"), "conv", UnsupportedError),
        (("layers", 1, "mixer", "q_rank"), 0, LoadError),
        (("layers", 1, "mixer", "rot", "dims"), 10, LoadError),               # more than the rotated part holds
        (("layers", 2, "type"), "lstm", UnsupportedError),
        (("norm", "eps"), 0.0, LoadError),
        (("token_side", "dim"), 0, LoadError),
        (("width",), 0, LoadError),
    ]:
        with pytest.raises(error):
            model_from_config(changed(path, value))


def test_keys_that_may_be_absent():
    import tie_amd  # noqa: F401
    from tie_amd.config.zovudra import ZovudraConfig

    config = copy.deepcopy(CONFIGS["A"])
    config.pop("embedding")
    config.pop("token_side")
    config["layers"][0]["mixer"]["mask"].pop("keep_first")
    config["layers"][0]["mixer"].pop("kv_heads")
    config["layers"][0]["mlp"]["router"].pop("groups")
    config["layers"][0]["mlp"]["router"].pop("scale")
    config["layers"][3]["mixer"]["mask"] = {"keep_first": 5}          # nothing to keep where every key is visible
    read = ZovudraConfig.from_json(config)
    assert read.embedding_scale == 1.0 and read.token_side_dim is None
    first = read.layers[0]
    assert first.mixer.keep_first == 0 and first.mixer.kv_heads == first.mixer.heads
    assert (first.mlp.groups, first.mlp.keep_groups, first.mlp.scale) == (1, 1, 1.0)
    assert read.layers[3].mixer.window is None and read.layers[3].mixer.keep_first == 0


def test_the_frequencies_the_engine_makes_are_the_plain_ones():
    import tie_amd  # noqa: F401
    from tie_amd.parts.base import PartSpec, build_part

    for rot in ({"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}},
                {"dims": 32, "base": 5000.0, "scaling": {"factor": 8.0, "low": 2.0, "high": 16.0, "original": 64}},
                {"dims": 6, "base": 70.0, "scaling": {"factor": 5.0, "low": 0.5, "high": 2.0, "original": 16}},
                {"dims": 16, "base": 1e6}):
        part = build_part("position", PartSpec("rope_banded", {"head_dim": 64, "theta": rot["base"], "rotary_dim": rot["dims"],
                                                               "pairing": "rotate_half", "scaling": rot.get("scaling")}))
        assert torch.allclose(torch.from_numpy(part.host_inv_freq()).double(), plain.banded_frequencies(rot), rtol=1e-6)
        assert part.amplitude == 1.0


def test_windows_give_their_pages_back_but_for_the_kept_first_positions():
    from tie_amd.cache.manager import FREED, CacheManager
    from tie_amd.cache.spec import PagedKV, plan_cache
    from tie_amd.errors import InvalidArgument

    need = PagedKV(2, 16, 9, None, 6)
    assert need.reach == 15 and [need.first_needed(p) for p in (0, 8, 9, 25)] == [0, 0, 1, 17]
    with pytest.raises(InvalidArgument):
        PagedKV(2, 16, None, None, 3)                       # nothing is kept without a window
    plan = plan_cache([need, PagedKV(1, 48, 9)], [None, None])
    cache = CacheManager(plan, block_size=4, num_blocks=16)
    a = cache.new_request()
    assert cache.reserve(a, 23)
    assert cache.trim(a, 23) == 1 + 3                   # positions 0..14 are out of every later window: three whole
    kept, plain_window = a.tables                       # pages, of which the two that hold positions 0..5 stay
    assert FREED not in kept[:2] and kept[2] == FREED and FREED not in kept[3:]
    assert plain_window[:3] == [FREED] * 3
    assert cache.reserve(a, 60) and cache.trim(a, 60) > 0
    assert FREED not in kept[:2] and kept[2:12] == [FREED] * 10          # the kept pages stay to the end
    assert cache.slots(a, 0, 0, 6) == [kept[0] * 4 + i for i in range(4)] + [kept[1] * 4, kept[1] * 4 + 1]
    cache.release(a)
    assert cache.all_free()
