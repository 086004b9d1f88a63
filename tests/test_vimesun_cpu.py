"""Vimesun on the host: its configuration reader, its plan, its caches, and the plain implementation's mechanisms."""

import math

import pytest
import torch

from kestrel_amd.cache.manager import CacheManager
from kestrel_amd.config.registry import read_model_dir, resolve
from kestrel_amd.models.decoder import DecoderModel
from kestrel_amd.models.vimesun import VimesunConfig, build_plan
from tests import vimesun_cases as cases
from tests.plain import vimesun_plain as plain


def test_config_names_the_architecture_and_round_trips():
    for name, config in cases.CONFIGS.items():
        assert resolve(config).name == "vimesun"
        typed = VimesunConfig.from_dict(config)
        again = VimesunConfig.from_dict(typed.to_dict())
        assert again.layers == typed.layers and (again.loop_start, again.loop_stop, again.loop_times) == \
            (typed.loop_start, typed.loop_stop, typed.loop_times), name


def test_schedule_follows_the_loop():
    plan = build_plan(VimesunConfig.from_dict(cases.CONFIGS["P"]))
    assert [(e.layer, e.before) for e in plan.schedule] == [(0, None), (1, "loop_in"), (1, "loop_in"), (1, "loop_in"), (2, None)]
    assert all(e.reads_cache_of is None for e in plan.schedule)          # every pass keeps a cache of its own
    plan = build_plan(VimesunConfig.from_dict(cases.CONFIGS["S"]))
    assert [(e.layer, e.before) for e in plan.schedule] == [(0, None), (1, "loop_in"), (1, "loop_in")]
    plan = build_plan(VimesunConfig.from_dict(cases.CONFIGS["R"]))
    assert [(e.layer, e.before) for e in plan.schedule] == [(0, None), (1, None)] and not plan.junctions
    assert [(i, s) for i, s in plain.layer_order(cases.CONFIGS["P"])] == [(0, False), (1, True), (1, True), (1, True), (2, False)]


def test_tensor_names_and_shapes():
    net = DecoderModel(build_plan(VimesunConfig.from_dict(cases.CONFIGS["Q"])))
    params = net.params()
    assert tuple(params["l1.mix.q"].shape) == (8 * 16, 96) and tuple(params["l1.mix.k"].shape) == (16, 96)
    assert tuple(params["l1.mix.v"].shape) == (20, 96) and tuple(params["l1.mix.o"].shape) == (96, 8 * 20)
    assert tuple(params["loop.in"].shape) == (96, 192) and tuple(params["pos"].shape) == (300, 96)
    assert "l0.mlp.up" not in params and "l0.norm2" not in params          # the layer without a feed-forward
    assert tuple(params["l2.mlp.up"].shape) == (200, 96) and "head" in params and "final.norm.b" in params
    assert "loop.in" not in DecoderModel(build_plan(VimesunConfig.from_dict(cases.CONFIGS["R"]))).params()


def test_model_folder_is_read_through_the_registry():
    spec, typed, plan = read_model_dir(cases.model_dir("P"))
    assert spec.name == "vimesun" and plan.dim == 64 and len(plan.schedule) == 5


@pytest.mark.parametrize("bad, message", [
    (lambda c: c["layers"][0].update(type="recurrent"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "dense"),
    (lambda c: c.update(loop={"start": 2, "stop": 1, "times": 1}), "loop"),
    (lambda c: c.pop("residual_mult"), "residual_mult"),
])
def test_config_errors_name_the_key(bad, message):
    import copy

    config = copy.deepcopy(cases.CONFIGS["P"])
    bad(config)
    with pytest.raises(ValueError, match=message):
        VimesunConfig.from_dict(config)


def test_cache_groups_follow_the_layers():
    """Layers of equal needs share a pool, a pass of a looped layer has tensors of its own, and a value size of its own
    gives the value pages their shape."""
    net = DecoderModel(build_plan(VimesunConfig.from_dict(cases.CONFIGS["P"])))
    cache = CacheManager(net.cache_needs(), 16, 8, 2)
    assert len(cache.groups) == 1 and len(cache.groups[0].entries) == 5
    assert cache.groups[0].spec.page_tensors(16) == {"k": (2, 16, 32), "v": (2, 64, 16)}
    net = DecoderModel(build_plan(VimesunConfig.from_dict(cases.CONFIGS["Q"])))
    cache = CacheManager(net.cache_needs(), 16, 32, 2)
    assert len(cache.groups) == 3
    assert [g.spec.window for g in cache.groups] == [7, 200, 1]
    # a window of 7 fed token by token never holds more than two pages; the window of 1 gives every page back but one
    slot = cache.admit()
    for length in range(1, 120):
        cache.ensure(slot, length)
        cache.trim(slot, length)
        held = [sum(1 for p in cache.block_table(g, slot) if p >= 0) for g in range(3)]
        assert held[0] <= 2 and held[2] <= 2 and held[1] == -(-length // 16)
    cache.release(slot)
    cache.check()


def test_plain_sink_softmax_and_slopes():
    scores = torch.tensor([[0.0, 1.0, -math.inf, 5.0]], dtype=torch.float64)
    w = plain.sink_softmax_weights(scores)
    direct = torch.exp(scores) / (1 + torch.exp(scores).sum())
    assert torch.allclose(w, direct, rtol=1e-12) and float(w.sum()) < 1.0
    assert float(plain.sink_softmax_weights(torch.full((1, 3), -40.0, dtype=torch.float64)).sum()) < 1e-16
    assert plain.head_slopes(4) == [0.25, 0.0625, 0.015625, 0.00390625]
    assert plain.head_slopes(1) == [2.0 ** -8]


def test_plain_window_and_distance():
    """One key stands out by construction: the output is that key's value while it is inside the window, and
    nothing of it once it is outside."""
    torch.manual_seed(0)
    n, d = 12, 8
    k = plain.unit_rms(torch.randn(n, 1, d, dtype=torch.float64), 0.0)
    v = torch.zeros(n, 1, 4, dtype=torch.float64)
    v[3, 0] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    q = k[3:4].expand(n, 1, d).clone()              # every query points at key 3
    out = plain.attention_core(q, k, v, scale=20.0, window=5)
    for i in range(n):
        expected_seen = 3 <= i < 3 + 5
        assert (float(out[i, 0, 0]) > 0.99) == expected_seen, i
        if not expected_seen:
            assert float(out[i, 0].abs().max()) < 1e-12
