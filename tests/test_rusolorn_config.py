"""Configuration, plan and cache bookkeeping of the Rusolorn decoder, and the plain implementation against itself
(no GPU)."""

import copy

import pytest
import torch

from plain import rusolorn_plain as plain
from rusolorn_helpers import RUSOLORN
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.config import ConfigError, RusolornConfig, config_from_dict
from somi_inference_amd.models import collect_weight_specs, rusolorn_plan
from somi_inference_amd.models.decoder import DecoderModel
from somi_inference_amd.parts import CompositeSpec, FixedStateSpec, PagedSpec, Runtime


@pytest.mark.parametrize("name", list(RUSOLORN))
def test_config_round_trips_through_its_json(name):
    config = RUSOLORN[name]["config"]
    raw = config.to_dict()
    assert raw["architecture"] == "Rusolorn"
    arch, again = config_from_dict(copy.deepcopy(raw))
    assert arch.name == "Rusolorn" and again == config and isinstance(again, RusolornConfig)


def test_keys_a_config_may_leave_out():
    raw = RUSOLORN["A"]["config"].to_dict()
    del raw["token_side"], raw["embedding"], raw["residual_mult"]
    del raw["layers"][0]["mlp"]["router"]["groups"], raw["layers"][0]["mlp"]["shared"]
    raw["layers"][1]["mlp"] = None
    _, config = config_from_dict(raw)
    assert config.token_side_dim is None and config.embedding_scale == 1.0 and config.residual_mult == 1.0
    assert (config.layers[0].mlp.groups, config.layers[0].mlp.keep, config.layers[0].mlp.shared_ff) == (1, 1, None)
    names = {spec.name for spec in collect_weight_specs(rusolorn_plan(config))}
    assert "side.embed" not in names and "l0.side.gate" not in names and "l0.mlp.shared.gate" not in names
    assert "l1.mlp.router" not in names and "l0.mlp.e7.down" in names


def test_config_errors_name_the_key():
    raw = RUSOLORN["A"]["config"].to_dict()
    for change, text in (
        (lambda r: r["layers"][0].__setitem__("type", "serial"), "'type'"),
        (lambda r: r["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3), "divisible"),
        (lambda r: r["layers"][0]["mixer"]["left"].__setitem__("vdim", 8), "vdim"),
        (lambda r: r["layers"][0]["mixer"]["left"].pop("mask"), "mask"),
        (lambda r: r["layers"][0]["mixer"].pop("right"), "right"),
        (lambda r: r["layers"][0]["mlp"]["router"]["groups"].__setitem__("count", 3), "groups"),
        (lambda r: r["layers"][0]["mlp"]["router"].__setitem__("top", 5), "top"),
        (lambda r: r["layers"][0]["mlp"].__setitem__("kind", "dense"), "kind"),
        (lambda r: r.pop("vocab"), "vocab"),
    ):
        broken = copy.deepcopy(raw)
        change(broken)
        with pytest.raises(ConfigError, match=text):
            config_from_dict(broken)


def test_plan_names_tensors_and_composite_caches():
    config = RUSOLORN["A"]["config"]
    plan = rusolorn_plan(config)
    names = {spec.name: spec for spec in collect_weight_specs(plan)}
    assert {"embed", "side.embed", "final.norm", "final.norm.alpha", "final.norm.b", "l0.norm1.alpha", "l0.mix.left.q.norm",
            "l0.mix.left.out", "l0.mix.right.q.conv", "l0.mix.right.A_log", "l0.mix.right.dt_bias", "l1.mlp.e5.up",
            "l1.mlp.shared.down", "l2.side.proj", "l2.side.norm"} <= set(names)
    assert "l0.mix.left.v" not in names and "l0.norm2" not in names           # values are the keys; one norm a layer
    assert names["l1.mix.left.q"].shape == (6 * 32, 96) and names["l1.mix.left.k.norm"].shape == (32,)
    assert names["l0.mix.right.v.conv"].shape == (4 * 32, 4) and names["side.embed"].shape == (211, 3 * 8)
    assert names["final.norm.alpha"].shape == () and not any(name.endswith(".weight") for name in names)
    model = DecoderModel(plan, Runtime(torch.float32, torch.device("cpu")))
    needs = model.cache_needs()
    assert all(isinstance(need, CompositeSpec) for need in needs)
    left, right = dict(needs[1].parts)["left"], dict(needs[1].parts)["right"]
    assert isinstance(left, PagedSpec) and left.window == 36 and [t.name for t in left.tensors] == ["k", "v"]
    state, conv = (spec for _, spec in right.parts)
    assert isinstance(state, FixedStateSpec) and state.shape == (2, 32, 16) and conv.shape == (2, 2 * 32 + 2 * 16)
    # layers 0 and 2 share a window and so a pool of pages; every layer has tensors and state of its own
    cache = CacheManager(needs, block_size=16, num_blocks=8, max_requests=2, dtype=torch.float32, device="cpu",
                         allocate_tensors=False)
    assert [cache.layer_caches[i].children["left"].group for i in range(3)] == [0, 1, 0]
    assert [group.window for group in cache.groups] == [24, 36]
    assert len(cache.layer_caches[0].leaves()) == 3
    cache.register("a")
    cache.reserve("a", 70)
    cache.commit("a", 70)
    cache.check_invariants()
    # 70 tokens in pages of 16: the window of 24 has passed two pages (the next token sees from 47 on), and so has
    # the window of 36 (from 35 on)
    assert [len([p for p in cache.page_list(g, "a") if p >= 0]) for g in (0, 1)] == [3, 3]
    cache.free("a")
    assert cache.free_pages() == [8, 8]


# ------------------------------------------------------------------------------- the plain implementation against itself
def test_plain_delta_rule_cut_in_two_equals_the_whole():
    """The recurrence written with an explicit state and carried convolution inputs gives what the whole-sequence
    function gives: the state and the last taps - 1 inputs are all that a sequence's past leaves."""
    torch.manual_seed(0)
    mixer = dict(heads=4, kv_heads=2, dim=8, vdim=12, conv=3)
    width, tokens = 24, 19
    weights = {f"m.{n}": torch.randn(s) * 0.3 for n, s in {
        "q": (16, width), "k": (16, width), "v": (48, width), "g": (48, width), "o": (width, 48), "b": (4, width),
        "a": (4, width), "q.conv": (16, 3), "k.conv": (16, 3), "v.conv": (48, 3), "A_log": (4,), "dt_bias": (4,),
        "norm": (12,)}.items()}
    h = torch.randn(tokens, width)
    whole = plain.gated_delta_rule(h, weights, "m", mixer, 1e-5)
    # token by token with the definition's own steps
    q_in, k_in, v_in = (h @ weights[f"m.{n}"].T for n in "qkv")
    state = torch.zeros(4, 8, 12)
    rows = []
    for t in range(tokens):
        def conv(x, taps):
            past = torch.cat([torch.zeros(2, x.shape[1]), x])[t:t + 3]
            return plain.silu((past * taps.T).sum(0))
        q, k = conv(q_in, weights["m.q.conv"]).view(2, 8), conv(k_in, weights["m.k.conv"]).view(2, 8)
        v = conv(v_in, weights["m.v.conv"]).view(4, 12)
        q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * 8 ** -0.5
        k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(weights["m.b"] @ h[t])
        decay = torch.exp(-torch.exp(weights["m.A_log"]) * torch.nn.functional.softplus(weights["m.a"] @ h[t] + weights["m.dt_bias"]))
        out = []
        for a in range(4):
            state[a] = decay[a] * state[a]
            u = beta[a] * (v[a] - state[a].T @ k[a // 2])
            state[a] = state[a] + torch.outer(k[a // 2], u)
            out.append(plain.rms(state[a].T @ q[a // 2], 1e-5) * weights["m.norm"])
        rows.append((torch.cat(out) * plain.silu(weights["m.g"] @ h[t])) @ weights["m.o"].T)
    torch.testing.assert_close(torch.stack(rows), whole, rtol=1e-4, atol=1e-5)


def test_plain_router_keeps_the_best_groups_only():
    router = torch.eye(8)
    h = torch.tensor([[5.0, 0.0, 0.0, 4.0, 0.0, 0.0, 4.5, 4.4]])     # groups of two: best experts 0, 3, 6 (and 7)
    chosen, weight = plain.route(h, router, top=2, groups=4, keep=2)
    assert chosen.tolist() == [[0, 6]]                                # groups 0 and 3 stay; expert 3 is out with its group
    chosen, _ = plain.route(h, router, top=3, groups=4, keep=2)
    assert chosen.tolist() == [[0, 6, 7]]
    chosen, weight = plain.route(h, router, top=3, groups=1, keep=1)
    assert chosen.tolist() == [[0, 6, 7]] and abs(float(weight.sum()) - 1.0) < 1e-6
