"""Configuration, plan and cache bookkeeping of the Kamedra decoder (no GPU)."""

import copy

import pytest
import torch

from kamedra_helpers import KAMEDRA
from plain import kamedra_plain as plain
from somi_inference_amd.cache import RELEASED, CacheManager
from somi_inference_amd.config import ConfigError, KamedraConfig, config_from_dict
from somi_inference_amd.models import collect_weight_specs, kamedra_plan
from somi_inference_amd.parts import PAGE, FixedStateSpec, PagedSpec, PageTensor
from somi_inference_amd.parts.position import RotaryPosition
from somi_inference_amd.weights import ANY_SIZE, WeightSpec


@pytest.mark.parametrize("name", list(KAMEDRA))
def test_config_round_trips_through_its_json(name):
    config = KAMEDRA[name]["config"]
    raw = config.to_dict()
    assert raw["architecture"] == "Kamedra"
    arch, again = config_from_dict(copy.deepcopy(raw))
    assert arch.name == "Kamedra" and again == config and isinstance(again, KamedraConfig)


def test_config_errors_name_the_key():
    raw = KAMEDRA["A"]["config"].to_dict()
    for change, text in (
        (lambda r: r["layers"][0].__setitem__("type", "conv"), "'type'"),
        (lambda r: r["layers"][1]["mixer"].__setitem__("kv_heads", 3), "divisible"),
        (lambda r: r["layers"][1]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
        (lambda r: r["layers"][3]["mixer"].__setitem__("kv_from", 2), "kv_from"),
        (lambda r: r["layers"][3]["mixer"].__setitem__("dim", 32), "must agree"),
        (lambda r: r["layers"][1]["mixer"].pop("mask"), "mask"),
        (lambda r: r.pop("vocab"), "vocab"),
        (lambda r: r["layers"][1]["mlp"].__setitem__("kind", "experts"), "kind"),
    ):
        broken = copy.deepcopy(raw)
        change(broken)
        with pytest.raises(ConfigError, match=text):
            config_from_dict(broken)


def test_plan_names_tensors_and_cache_sharing():
    config = KAMEDRA["A"]["config"]
    plan = kamedra_plan(config)
    names = {spec.name: spec for spec in collect_weight_specs(plan)}
    assert {"embed", "final.norm", "l0.norm1", "l0.mix.a2.b", "l0.mix.norm", "l1.norm2", "l1.mix.lq1", "l1.mlp.down",
            "l3.mix.q", "l3.mix.o"} <= set(names)
    assert "l0.norm2" not in names and "l0.mlp.gate" not in names          # a layer without a feed-forward
    assert "l3.mix.k" not in names and "l3.mix.v" not in names              # the borrower has no key/value projections
    assert names["l1.mix.q"].shape == (4 * 2 * 16, 96) and names["l1.mix.k"].shape == (2 * 2 * 16, 96)
    assert names["l1.mix.v"].shape == (2 * 32, 96) and names["l0.mix.a2"].shape == (3 * 16, 8)
    assert plan.cache_from == {3: 1}
    assert not any(name.endswith(".weight") for name in names)


def test_rank_left_to_the_checkpoint():
    raw = KAMEDRA["A"]["config"].to_dict()
    for layer in raw["layers"]:
        layer["mixer"].pop("rank", None)
    _, config = config_from_dict(raw)
    names = {spec.name: spec for spec in collect_weight_specs(kamedra_plan(config))}
    assert names["l0.mix.a1"].shape == (ANY_SIZE, 96) and names["l0.mix.a2"].shape == (48, ANY_SIZE)
    assert names["l0.mix.a1"].fits((5, 96)) and not names["l0.mix.a1"].fits((5, 95))
    assert WeightSpec("x", (3, 4)).fits((3, 4)) and not WeightSpec("x", (3, 4)).fits((3, 4, 1))


def test_lenders_cache_keeps_what_its_borrowers_see():
    from somi_inference_amd.parts import build_part
    plan = kamedra_plan(KAMEDRA["A"]["config"])
    lender = build_part("block", plan.layers[1].block, prefix="l1").mixer
    spec = lender.cache_spec()
    assert isinstance(spec, PagedSpec) and spec.window == 40 and spec.keep_first == 5      # max over both masks
    assert build_part("block", plan.layers[3].block, prefix="l3").mixer.cache_spec() is None
    state = build_part("block", plan.layers[0].block, prefix="l0").mixer.cache_spec()
    assert isinstance(state, FixedStateSpec) and state.shape == (3, 16, 32) and state.dtype == torch.float32


def test_window_gives_pages_back_but_keeps_the_first_tokens():
    spec = PagedSpec((PageTensor("k", (1, PAGE, 4)),), window=10, page_size=4, keep_first=6)
    cache = CacheManager([spec, PagedSpec((PageTensor("k", (1, PAGE, 4)),), window=10, page_size=4)],
                         block_size=4, num_blocks=16, max_requests=2, dtype=torch.float32, device="cpu",
                         allocate_tensors=False)
    assert len(cache.groups) == 2 and [g.keep_first for g in cache.groups] == [6, 0]
    cache.register("r")
    for _ in range(30):
        cache.reserve("r", 1)
        cache.commit("r", 1)
    # the next token is at 30 and sees 21..30 and 0..5: pages 0, 1 (kept) and 5.. stay; 2, 3, 4 are given back
    kept, plain_window = cache.page_list(0, "r"), cache.page_list(1, "r")
    assert [p == RELEASED for p in kept] == [False, False, True, True, True, False, False, False]
    assert [p == RELEASED for p in plain_window] == [True] * 5 + [False] * 3
    assert cache.table_row(0, "r")[2] == 0 and cache.table_row(0, "r")[0] == kept[0]
    cache.check_invariants()
    cache.free("r")
    assert cache.free_pages() == [16, 16]


def test_rotary_frequencies_of_the_part_are_the_plain_ones():
    for dims, base, scaling in ((8, 1e4, dict(factor=4.0, low=1.0, high=4.0, original=64)), (24, 500.0, None),
                                (16, 3e4, dict(factor=8.0, low=1.0, high=4.0, original=512)),
                                (4, 10.0, dict(factor=2.0, low=2.0, high=8.0, original=16))):
        part = RotaryPosition("", head_dim=32, theta=base, rotary_dim=dims, pairing="neighbours", scaling=scaling)
        want = plain.rotary_frequencies(dims, base, scaling)
        torch.testing.assert_close(part.frequencies(), want, rtol=1e-6, atol=0.0)
    # all three regimes occur in the third case: kept, blended, divided
    f = [1e4 ** (-2.0 * i / 8) for i in range(4)]
    got = plain.rotary_frequencies(8, 1e4, dict(factor=4.0, low=1.0, high=4.0, original=64)).tolist()
    assert got[0] == pytest.approx(f[0]) and got[3] == pytest.approx(f[3] / 4.0) and f[1] / 4.0 < got[1] < f[1]


def test_plain_mask_and_recurrence_hold_together():
    # the mask as a matrix against its definition
    for size, keep in ((5, 2), (3, 7), (100, 0), (1, 0)):
        matrix = plain.visibility(20, size, keep)
        for i in range(20):
            for j in range(20):
                assert bool(matrix[i, j]) == plain.visible(i, j, size, keep)
    # the recurrence carried over a cut equals the whole
    torch.manual_seed(0)
    mixer = dict(heads=2, dim=6, vdim=5, tau=3.0)
    weights = {"l0.mix." + n: torch.randn(s) * 0.3 for n, s in (("q", (12, 10)), ("k", (12, 10)), ("v", (10, 10)),
               ("g", (10, 10)), ("o", (10, 10)), ("norm", (5,)), ("a1", (3, 10)), ("a2", (12, 3)), ("a2.b", (12,)))}
    h = torch.randn(9, 10)
    whole, _ = plain.gated_linear_attention(h, weights, "l0", mixer, 1e-6)
    first, state = plain.gated_linear_attention(h[:4], weights, "l0", mixer, 1e-6)
    second, _ = plain.gated_linear_attention(h[4:], weights, "l0", mixer, 1e-6, state)
    torch.testing.assert_close(torch.cat([first, second]), whole, rtol=1e-5, atol=1e-6)
