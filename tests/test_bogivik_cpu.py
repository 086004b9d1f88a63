"""Bogivik on the host: its configuration reader, its plan, its caches, and the plain implementation's mechanisms."""

import copy
import math

import pytest
import torch

from kestrel_amd.cache.manager import CacheManager
from kestrel_amd.config.registry import read_model_dir, resolve
from kestrel_amd.models.bogivik import BogivikConfig, build_plan
from kestrel_amd.models.decoder import DecoderModel
from kestrel_amd.parts.rotary import rotary_frequencies
from kestrel_amd.parts.specs import CacheSpec, DistanceBuckets, WavelengthScaling
from tests import bogivik_cases as cases
from tests.plain import bogivik_plain as plain


def test_config_names_the_architecture_and_round_trips():
    for name, config in cases.CONFIGS.items():
        assert resolve(config).name == "bogivik"
        typed = BogivikConfig.from_dict(config)
        assert BogivikConfig.from_dict(typed.to_dict()).layers == typed.layers, name


def test_tensor_names_and_shapes():
    params = DecoderModel(build_plan(BogivikConfig.from_dict(cases.CONFIGS["Q"]))).params()
    assert tuple(params["l0.mix.left.q"].shape) == (120, 100) and tuple(params["l0.mix.left.q.b"].shape) == (120,)
    assert tuple(params["l0.mix.left.q.norm"].shape) == (24,) and tuple(params["l0.mix.left.o.b"].shape) == (100,)
    assert tuple(params["l0.mix.left.g"].shape) == (50, 100) and tuple(params["l0.mix.left.out"].shape) == (100,)
    assert tuple(params["l0.mix.right.v"].shape) == (108, 100) and tuple(params["l0.mix.right.i"].shape) == (3, 100)
    assert tuple(params["l0.mix.right.f.b"].shape) == (3,) and tuple(params["l0.mix.right.norm"].shape) == (108,)
    assert "l0.mlp.gate" not in params and tuple(params["l1.mlp.gate"].shape) == (50, 100)
    assert tuple(params["l1.mix.q.norm"].shape) == (120,) and tuple(params["l1.mix.k.norm"].shape) == (120,)
    assert tuple(params["l1.mix.rel"].shape) == (6, 5) and tuple(params["l1.mix.vmix"].shape) == ()
    assert "l2.mix.vmix" not in params and "l3.mix.vmix" in params and "l2.mix.q.b" not in params
    assert set(k for k in params if "." not in k or k.startswith("final")) == {"embed", "head", "final.norm"}


def test_the_number_of_buckets_may_come_from_the_weights_file():
    config = copy.deepcopy(cases.CONFIGS["P"])
    for layer in config["layers"]:
        layer["mixer"].pop("buckets", None)
    params = DecoderModel(build_plan(BogivikConfig.from_dict(config))).params()
    assert tuple(params["l0.mix.rel"].shape) == (-1, 4)


def test_blending_layers_are_one_source_and_followers():
    plan = build_plan(BogivikConfig.from_dict(cases.CONFIGS["Q"]))
    roles = [getattr(getattr(layer.mixer, "value_blend", None), "role", None) for layer in plan.layers]
    assert roles == [None, "source", None, "blend", None]


def test_caches_and_state_by_layer():
    net = DecoderModel(build_plan(BogivikConfig.from_dict(cases.CONFIGS["P"])))
    needs = net.cache_needs()
    assert [n[0].chunk for n in needs] == [None, 24, None, None] and [n[1] is not None for n in needs] == [False, True, False, False]
    assert needs[1][1].shape == (2 * (16 * 32 + 16 + 1),)
    cache = CacheManager(needs, page_size=16, n_pages=8, max_requests=2)
    assert len(cache.groups) == 3            # layers 0 and 2 share a pool; the chunked branch and the last layer have their own


def test_chunked_visibility_and_pages_given_back():
    spec = CacheSpec(1, 8, None, None, chunk=24)
    assert [spec.first_visible(p) for p in (0, 23, 24, 47, 48)] == [0, 0, 24, 24, 48]
    cache = CacheManager([(spec, None, None)], page_size=16, n_pages=4, max_requests=1)
    slot = cache.admit()
    held = []
    for length in range(1, 200):
        cache.ensure(slot, length)
        cache.trim(slot, length)
        cache.check()
        table = cache.block_table(0, slot)
        # every key the next query reads is still backed
        assert all(table[p // 16] >= 0 for p in range(spec.first_visible(length), length))
        held.append(sum(p >= 0 for p in table))
    assert max(held) <= 3
    cache.release(slot)
    assert cache.pages_available(0) == 4
    assert cache.pages_for(0, 1000, portion=1) <= 3 and cache.pages_for(0, 10) == 1


@pytest.mark.parametrize("bad, message", [
    (lambda c: c["layers"][0].update(type="recurrent"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "dense"),
    (lambda c: c["layers"][1]["mixer"]["left"].pop("mask"), "mask"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=33), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(gate_cap=0), "gate_cap"),
    (lambda c: c["layers"][0]["mixer"].pop("bias_max"), "bias_max"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=32), "one shape"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_config_errors_name_the_key(bad, message):
    config = copy.deepcopy(cases.CONFIGS["P"])
    bad(config)
    with pytest.raises(ValueError, match=message):
        BogivikConfig.from_dict(config)


def test_model_folder_is_read_through_the_registry():
    spec, typed, plan = read_model_dir(cases.model_dir("S"))
    assert spec.name == "bogivik" and plan.dim == 48 and len(plan.schedule) == 2


def test_buckets_of_the_product_and_of_the_plain_implementation_agree():
    for buckets, far in ((16, 40.0), (6, 9.5), (9, 400.0), (2, 3.0), (21, 400.0), (7, 30.0)):
        spec = DistanceBuckets(buckets, far)
        count = spec.distances()
        assert [spec.bucket(n) for n in range(count + 50)] == [plain.distance_bucket(n, buckets, far) for n in range(count + 50)]
        assert all(spec.bucket(n) == buckets - 1 for n in range(count - 1, count + 500))
        assert count == 1 or spec.bucket(count - 2) < buckets - 1
    half = 8
    assert [plain.distance_bucket(n, 16, 40.0) for n in range(half)] == list(range(half))
    assert plain.distance_bucket(39, 16, 40.0) < 16 and plain.distance_bucket(40, 16, 40.0) == 15


def test_frequencies_of_the_product_and_of_the_plain_implementation_agree():
    for dims, base, scaling in ((32, 10000.0, (8.0, 1.0, 4.0, 64)), (12, 500.0, None), (64, 1e6, (4.0, 1.0, 2.0, 128)),
                                (64, 1e4, (16.0, 0.5, 3.0, 256)), (40, 20.0, (2.0, 2.0, 8.0, 32))):
        rot = {"dims": dims, "base": base}
        if scaling:
            rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
        ours = rotary_frequencies(dims, base, WavelengthScaling(*scaling) if scaling else None)
        theirs = plain.rotary_frequencies(rot)
        assert len(ours) == dims // 2 and all(abs(a - b) <= 1e-12 * abs(b) for a, b in zip(ours, theirs))
    # all three regimes occur in one of them: kept, divided by the factor, blended
    rot = {"dims": 32, "base": 10000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}
    plainly = [10000.0 ** (-2.0 * i / 32) for i in range(16)]
    ratios = [a / b for a, b in zip(plain.rotary_frequencies(rot), plainly)]
    assert ratios[0] == 1.0 and abs(ratios[-1] - 1 / 8) < 1e-12 and any(1 / 8 + 1e-6 < r < 1 - 1e-6 for r in ratios)


def test_matrix_memory_carries_its_state_in_the_plain_implementation():
    """Token by token through a carried state equals the whole sequence; the running maximum starts at zero."""
    gen = torch.Generator().manual_seed(3)
    n, d, dv = 30, 6, 5
    q, k = torch.randn(n, d, generator=gen, dtype=torch.float64), torch.randn(n, d, generator=gen, dtype=torch.float64)
    v = torch.randn(n, dv, generator=gen, dtype=torch.float64)
    li, lf = torch.randn(n, generator=gen, dtype=torch.float64) * 3, -torch.rand(n, generator=gen, dtype=torch.float64)
    whole = plain.matrix_memory(q, k, v, li, lf)
    state = {"S": torch.zeros(d, dv, dtype=torch.float64), "n": torch.zeros(d, dtype=torch.float64), "m": torch.zeros((), dtype=torch.float64)}
    parts = [plain.matrix_memory(q[a:b], k[a:b], v[a:b], li[a:b], lf[a:b], state) for a, b in ((0, 1), (1, 2), (2, 17), (17, 30))]
    assert torch.allclose(torch.cat(parts), whole, rtol=1e-12, atol=1e-12)
    # with a very negative first input gate (and a forget gate of one) the maximum stays at its start, zero, not at the
    # gate's logarithm, and the denominator's floor is exp(0)
    one = plain.matrix_memory(q[:1], k[:1], v[:1], torch.tensor([-20.0], dtype=torch.float64), torch.zeros(1, dtype=torch.float64))
    weight = math.exp(-20.0)
    want = weight * (k[0] @ q[0]) * v[0] / (max(abs(weight * float(k[0] @ q[0])), 1.0) + 1e-6)
    assert torch.allclose(one[0], want, rtol=1e-9, atol=1e-30)


def test_chunk_mask_counts_from_position_zero():
    mask = plain.chunk_mask(10, 4)
    assert mask[5].tolist() == [False] * 4 + [True, True] + [False] * 4 and mask[8].tolist() == [False] * 8 + [True, False]
