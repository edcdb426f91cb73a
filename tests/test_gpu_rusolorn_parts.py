"""Each mechanism of the Rusolorn decoder alone: the part with its kernels and the engine's cache manager against the
plain function written from the equations."""

import pytest
import torch

from plain import rusolorn_plain as plain
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.engine.batch import StepEntry, build_step
from somi_inference_amd.kernels import ops
from somi_inference_amd.parts import PartSpec, Runtime, build_part

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DEV = torch.device("cuda:0")


def tol(dtype, loose=1.0):
    return dict(rtol=1e-4, atol=2e-5 * loose) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2 * loose)


def rounded(x: torch.Tensor, dtype) -> torch.Tensor:
    """float32 values that the dtype holds exactly, so that the kernel and the plain function start from the same."""
    return x.to(dtype).to(torch.float32)


def load_part(part, weights: dict, dtype):
    """Hand the part its tensors as the loader would: matrices in the compute dtype, vectors in float32."""
    roles = {spec.name: spec.role for spec in part.weight_specs()}
    assert set(roles) == set(weights), sorted(set(roles) ^ set(weights))
    part.load(lambda name: weights[name].to(dtype if roles[name] == "matrix" else torch.float32).to(DEV).contiguous(),
              Runtime(dtype, DEV))
    return part


def random_weights(part, dtype, seed, scale=None) -> dict:
    """float32 tensors for every tensor the part declares (matrices hold values the dtype has exactly)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for spec in part.weight_specs():
        value = torch.randn(spec.shape, generator=gen) * (scale or {}).get(spec.role, spec.init.std * (10 if spec.role == "matrix" else 1))
        value = value + spec.init.mean
        out[spec.name] = rounded(value, dtype) if spec.role == "matrix" else rounded(value, torch.bfloat16)
    return out


class Engine:
    """The cache manager and the step layout of the engine around one mixer."""

    def __init__(self, mixer, dtype, block_size, num_blocks=64, max_requests=4):
        self.mixer, self.dtype = mixer, dtype
        self.cache = CacheManager([mixer.cache_spec()], block_size=block_size, num_blocks=num_blocks,
                                  max_requests=max_requests, dtype=dtype, device=DEV)
        self.splits = () if mixer.entry_split is None else (mixer.entry_split,)

    def run(self, portions: list[tuple[str, torch.Tensor]]) -> list[torch.Tensor]:
        """One step of (request, its next input rows); the mixer's output rows per request."""
        entries = []
        for rid, x in portions:
            if not self.cache.has(rid):
                self.cache.register(rid)
            self.cache.reserve(rid, x.shape[0])
            entries.append(StepEntry(rid, [0] * x.shape[0], []))
        step = build_step(entries, self.cache, DEV, self.splits)
        y = self.mixer.forward(torch.cat([x for _, x in portions]).to(self.dtype).to(DEV).contiguous(), step,
                               self.cache.layer_caches[0])
        y = y.materialize() if hasattr(y, "materialize") else y
        for rid, x in portions:
            self.cache.commit(rid, x.shape[0])
        outs, at = [], 0
        for _, x in portions:
            outs.append(y[at:at + x.shape[0]].float().cpu())
            at += x.shape[0]
        return outs

    def run_cut(self, rid, x, sizes):
        outs, at, i = [], 0, 0
        while at < x.shape[0]:
            size = sizes[i % len(sizes)]
            outs.append(self.run([(rid, x[at:at + size])])[0])
            at += size
            i += 1
        self.cache.free(rid)
        return torch.cat(outs)


# ------------------------------------------------------------------------------------------ the norm and the joins
@pytest.mark.parametrize("dtype", DTYPES)
def test_dynamic_tanh_and_the_joins(dtype):
    torch.manual_seed(1)
    n, width = 37, 200
    h = torch.randn(n, width) * 3
    w, b, alpha = torch.randn(width), torch.randn(width), torch.tensor(0.37)
    got = ops.dynamic_tanh(h.to(DEV), w.to(DEV), b.to(DEV), alpha.reshape(1).to(DEV), dtype)
    want = plain.dynamic_tanh(h, {"n": w, "n.b": b, "n.alpha": alpha}, "n")
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype))
    left, right = rounded(torch.randn(n, width) * 5, dtype), rounded(torch.randn(n, width) * 0.01, dtype)
    got = ops.normed_pair_mean(left.to(dtype).to(DEV), right.to(dtype).to(DEV), w.to(DEV), b.to(DEV), 1e-5)
    torch.testing.assert_close(got.cpu(), 0.5 * (plain.rms(left, 1e-5) * w + plain.rms(right, 1e-5) * b), rtol=1e-5, atol=1e-5)
    a, c = torch.randn(n, width), torch.randn(n, width)
    stream = h.clone().to(DEV)
    copy = ops.scaled_add(stream, a.to(DEV), c.to(DEV), 0.7, dtype)
    torch.testing.assert_close(stream.cpu(), h + 0.7 * (a + c), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(copy.float().cpu(), stream.cpu(), **tol(dtype))
    ops.normed_add(stream, a.to(DEV), w.to(DEV), 1e-5, 1.3)
    torch.testing.assert_close(stream.cpu(), h + 0.7 * (a + c) + 1.3 * plain.rms(a, 1e-5) * w, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------------------ attention with tied values
def attention_part(width, heads, groups, dim, window, scale, eps=1e-5):
    spec = PartSpec("gqa_attention", {"hidden_size": width, "num_heads": heads, "num_kv_heads": groups, "head_dim": dim,
                                      "position": PartSpec("none", {}), "qkv_bias": False, "window": window, "scale": scale,
                                      "values": "keys", "qk_norm": "projection", "norm_eps": eps,
                                      "names": {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"},
                                      "suffix": ""})
    return build_part("mixer", spec, prefix="m")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,dim,window,page,tokens", [(4, 2, 16, 24, 16, 150), (3, 3, 24, 1000, 8, 70),
                                                               (6, 2, 48, 56, 16, 300), (2, 1, 20, 1, 4, 30),
                                                               (2, 2, 64, 7, 8, 90), (4, 1, 128, 100, 16, 300)])
def test_tied_value_attention_against_the_plain_function(dtype, heads, groups, dim, window, page, tokens):
    width = 64
    part = attention_part(width, heads, groups, dim, window, 0.9 * dim ** -0.5)
    weights = random_weights(part, dtype, seed=tokens)
    load_part(part, weights, dtype)
    x = rounded(torch.randn(tokens, width, generator=torch.Generator().manual_seed(3)), dtype)
    mixer = dict(heads=heads, kv_heads=groups, dim=dim, mask={"size": window}, scale=0.9 * dim ** -0.5)
    want = plain.tied_window_attention(x, weights, "m", mixer, 1e-5)
    engine = Engine(part, dtype, page)
    whole = engine.run_cut("w", x, [tokens])
    torch.testing.assert_close(whole, want, **tol(dtype, loose=4))
    for sizes in ([1], [2], [9, 2, 31, 1, 5], [window if window < tokens else 13]):
        cut = engine.run_cut("c", x, sizes)
        if dtype == torch.float32:
            assert torch.equal(cut, whole), f"float32 rows depend on the portions {sizes}"
        else:
            torch.testing.assert_close(cut, want, **tol(dtype, loose=4))
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page", [(44, 16), (33, 8), (9, 4), (16, 16), (1, 8)])
@pytest.mark.parametrize("decoded", [False, True])
def test_one_key_stands_out_exactly_inside_the_window(dtype, window, page, decoded):
    """The query and key projections pick disjoint channels of the input, so queries and keys are set at will: one key
    points where every query points.  A query's output is that key's value (its key as projected, before the norm)
    if and only if the key lies inside the query's window; decoded token by token or as one prompt."""
    dim, tokens = 32, 120
    width = 2 * dim
    part = attention_part(width, 1, 1, dim, window, 1.0)
    weights = {"m.q": torch.eye(width)[:dim], "m.k": torch.eye(width)[dim:], "m.o": torch.eye(width)[:, :dim].contiguous(),
               "m.q.norm": torch.ones(dim), "m.k.norm": torch.ones(dim)}
    load_part(part, weights, dtype)
    direction = torch.nn.functional.normalize(torch.randn(dim, generator=torch.Generator().manual_seed(5)), dim=0)
    for marked in sorted({0, 1, page - 1, page, 3 * page, 50, tokens - window, tokens - 1} & set(range(tokens))):
        gen = torch.Generator().manual_seed(marked)
        x = torch.randn(tokens, width, generator=gen) * 0.05
        x[:, :dim] += direction                               # every query points along the direction
        x[marked, dim:] = 4.0 * direction                     # and so does one key, whose value is four times as long
        x = rounded(x, dtype)
        mixer = dict(heads=1, kv_heads=1, dim=dim, mask={"size": window}, scale=1.0)
        want = plain.tied_window_attention(x, weights, "m", mixer, 1e-5)
        engine = Engine(part, dtype, page, num_blocks=tokens // page + 2)
        got = engine.run_cut("r", x, [1] if decoded else [tokens])
        torch.testing.assert_close(got, want, **tol(dtype, loose=4))
        seen = (got[:, :dim] @ direction) > 2.0               # the marked value is 4 long, the others 0.05 * sqrt(dim)
        for i in range(tokens):
            assert bool(seen[i]) == (0 <= i - marked < window), f"query {i}, marked key {marked}, window {window}"


# ------------------------------------------------------------------------------------------ the gated delta rule
def delta_part(width, heads, groups, dim, vdim, taps, eps=1e-5):
    names = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "b": "b", "a": "a", "norm": "norm", "a_log": "A_log",
             "dt_bias": "dt_bias", "conv": "conv"}
    spec = PartSpec("gated_delta_rule", {"hidden_size": width, "num_heads": heads, "num_groups": groups, "key_dim": dim,
                                         "value_dim": vdim, "taps": taps, "eps": eps, "names": names, "suffix": ""})
    return build_part("mixer", spec, prefix="m")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,groups,dim,vdim,taps,tokens", [(4, 2, 16, 32, 4, 130), (1, 1, 20, 24, 2, 60),
                                                              (2, 1, 64, 128, 1, 40), (3, 3, 12, 20, 3, 75),
                                                              (2, 2, 128, 16, 9, 50), (2, 1, 200, 8, 3, 30)])
def test_gated_delta_rule_against_the_plain_function(dtype, heads, groups, dim, vdim, taps, tokens):
    width = 48
    part = delta_part(width, heads, groups, dim, vdim, taps)
    weights = random_weights(part, dtype, seed=dim)
    weights["m.k"], weights["m.k.conv"] = weights["m.q"].clone(), weights["m.q.conv"].clone()     # k.q > 0: see the helpers
    load_part(part, weights, dtype)
    x = rounded(torch.randn(tokens, width, generator=torch.Generator().manual_seed(4)), dtype)
    mixer = dict(heads=heads, kv_heads=groups, dim=dim, vdim=vdim, conv=taps)
    want = plain.gated_delta_rule(x, weights, "m", mixer, 1e-5)
    engine = Engine(part, dtype, 16, max_requests=2)
    whole = engine.run_cut("w", x, [tokens])
    torch.testing.assert_close(whole, want, **tol(dtype, loose=4))
    # portions shorter than the convolution, single tokens, and a slot that another request used in between
    for sizes in ([1], [2], [1, 2, 1, 7, 3, 29], [taps], [max(1, taps - 1), 40]):
        engine.run_cut("other", x.flip(0), [17])
        cut = engine.run_cut("c", x, sizes)
        if dtype == torch.float32:
            assert torch.equal(cut, whole), f"float32 rows depend on the portions {sizes}"
        else:
            torch.testing.assert_close(cut, want, **tol(dtype, loose=4))


@pytest.mark.parametrize("lanes", [4, 16])
@pytest.mark.parametrize("heads,groups,dim,vdim", [(2, 1, 16, 32), (3, 3, 20, 24), (2, 2, 128, 16), (1, 1, 200, 40), (2, 1, 64, 130)])
def test_the_recurrence_with_either_number_of_lanes_a_column(lanes, heads, groups, dim, vdim):
    """The kernel of the recurrence alone, from a state that is not zero, with 4 and with 16 lanes a column."""
    gen = torch.Generator().manual_seed(dim + lanes)
    tokens, channels = 45, 2 * groups * dim + heads * vdim
    qkv = torch.randn(tokens, channels, generator=gen)
    qkv[:, :2 * groups * dim] = torch.nn.functional.normalize(qkv[:, :2 * groups * dim].view(tokens, 2 * groups, dim), dim=-1).view(tokens, -1)
    beta, decay = torch.rand(tokens, heads, generator=gen), 0.5 + 0.5 * torch.rand(tokens, heads, generator=gen)
    state = torch.randn(3, heads, dim, vdim, generator=gen)
    want_state, want = state.clone(), torch.zeros(tokens, heads, vdim)
    cuts = [0, 7, 45]                                      # two entries: slot 2 takes tokens 0..6, slot 0 the rest
    for (lo, hi), slot in zip(zip(cuts, cuts[1:]), (2, 0)):
        for t in range(lo, hi):
            for a in range(heads):
                g = a // (heads // groups)
                q, k = qkv[t, g * dim:(g + 1) * dim], qkv[t, (groups + g) * dim:(groups + g + 1) * dim]
                v = qkv[t, 2 * groups * dim + a * vdim:2 * groups * dim + (a + 1) * vdim]
                S = decay[t, a] * want_state[slot, a]
                S = S + torch.outer(k, beta[t, a] * (v - S.T @ k))
                want_state[slot, a], want[t, a] = S, S.T @ q
    on_device = state.to(DEV)
    got = ops.delta_scan(qkv.to(DEV), beta.to(DEV), decay.to(DEV), torch.tensor(cuts, dtype=torch.int32, device=DEV),
                         torch.tensor([2, 0], dtype=torch.int32, device=DEV), on_device, groups, lanes=lanes)
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(on_device.cpu(), want_state, rtol=1e-4, atol=1e-4)
    assert torch.equal(on_device[1].cpu(), state[1])              # a slot of no entry is left alone


def test_two_requests_side_by_side_keep_their_own_state():
    part = delta_part(32, 2, 1, 16, 16, 3)
    weights = random_weights(part, torch.float32, seed=9)
    load_part(part, weights, torch.float32)
    gen = torch.Generator().manual_seed(6)
    xa, xb = torch.randn(50, 32, generator=gen), torch.randn(21, 32, generator=gen)
    engine = Engine(part, torch.float32, 16, max_requests=2)
    alone_a, alone_b = engine.run_cut("a", xa, [50]), engine.run_cut("b", xb, [21])
    first = engine.run([("b", xb[:4]), ("a", xa[:30])])
    second = engine.run([("a", xa[30:31]), ("b", xb[4:])])
    third = engine.run([("a", xa[31:])])
    assert torch.equal(torch.cat([first[1], second[0], third[0]]), alone_a)
    assert torch.equal(torch.cat([first[0], second[1]]), alone_b)


# ------------------------------------------------------------------------------------------ mixture of experts
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,top,groups,keep,ff,shared,tokens", [(8, 2, 4, 2, 48, 64, 150), (5, 1, 1, 1, 40, None, 33),
                                                                      (4, 4, 2, 2, 24, 8, 1), (12, 4, 4, 3, 64, 96, 70),
                                                                      (6, 3, 3, 2, 20, None, 300)])
def test_routed_experts_against_the_plain_function(dtype, experts, top, groups, keep, ff, shared, tokens):
    width = 56
    spec = PartSpec("routed_experts", {"hidden_size": width, "num_experts": experts, "top": top, "expert_size": ff,
                                       "limit": 0.8, "groups": groups, "keep_groups": keep, "shared_size": shared,
                                       "shared_limit": 1.7 if shared else None, "suffix": ""})
    part = build_part("feed_forward", spec, prefix="f")
    weights = random_weights(part, dtype, seed=experts, scale={"matrix": 0.4, "vector": 0.5})
    load_part(part, weights, dtype)
    x = rounded(torch.randn(tokens, width, generator=torch.Generator().manual_seed(8)), dtype)
    mlp = {"router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}},
           "expert": {"ff": ff, "limit": 0.8}, "shared": {"ff": shared, "limit": 1.7} if shared else None}
    want = plain.mixture(x, weights, "f", mlp)
    got = part.forward(x.to(dtype).to(DEV)).cpu()
    assert got.dtype == torch.float32
    torch.testing.assert_close(got, want, **tol(dtype, loose=8))
    chosen, weight = ops.moe_route(x.to(dtype).to(DEV), weights["f.router"].to(DEV), top, groups, keep)
    want_chosen, want_weight = plain.route(x, weights["f.router"], top, groups, keep)
    assert torch.equal(chosen.cpu().long(), want_chosen)
    torch.testing.assert_close(weight.cpu(), want_weight, rtol=1e-4, atol=1e-6)
    # a token's row does not depend on its neighbours in the batch
    some = part.forward(x[tokens // 2:tokens // 2 + 1].to(dtype).to(DEV)).cpu()
    if dtype == torch.float32:
        assert torch.equal(some[0], got[tokens // 2])
    else:                                     # the shared expert's products pick their kernels by the number of rows
        torch.testing.assert_close(some[0], got[tokens // 2], **tol(dtype, loose=8))


# ------------------------------------------------------------------------------------------ the per-layer token input
@pytest.mark.parametrize("dtype", DTYPES)
def test_token_input_against_the_plain_function(dtype):
    width, vocab, dim, layers, layer = 40, 50, 12, 3, 1
    spec = PartSpec("gated_table", {"hidden_size": width, "vocab_size": vocab, "dim": dim, "table": "side.embed",
                                    "table_width": dim * layers, "offset": layer * dim, "eps": 1e-5})
    part = build_part("token_input", spec, prefix=f"l{layer}.side")
    weights = random_weights(part, dtype, seed=2, scale={"matrix": 0.5, "vector": 0.2})
    load_part(part, weights, dtype)
    gen = torch.Generator().manual_seed(7)
    tokens = torch.randint(0, vocab, (29,), generator=gen)
    h = torch.randn(29, width, generator=gen)
    x = rounded(h, dtype)

    class Step:
        token_ids = tokens.to(torch.int32).to(DEV)
    stream = h.clone().to(DEV)
    part.add_to(stream, x.to(dtype).to(DEV), Step, 0.6)
    want = h + 0.6 * plain.token_side(x, tokens, weights, layer, dim, 1e-5)
    torch.testing.assert_close(stream.cpu(), want, **tol(dtype, loose=2))
