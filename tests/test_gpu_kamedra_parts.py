"""Each mechanism of the Kamedra decoder alone: its kernels against the plain functions written from the equations."""

import math

import pytest
import torch

from plain import kamedra_plain as plain
from somi_inference_amd.kernels import ops

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def rounded(x: torch.Tensor, dtype) -> torch.Tensor:
    """float32 values that the dtype holds exactly, so that the kernel and the plain function start from the same."""
    return x.to(dtype).to(torch.float32)


# ------------------------------------------------------------------------------------------ rotation, page store
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nk,dk,nv,dv,dims,page", [(8, 4, 16, 2, 32, 8, 16), (12, 12, 24, 6, 40, 24, 8),
                                                      (4, 2, 8, 1, 16, 4, 4), (6, 0, 10, 0, 12, 6, 8)])
def test_pair_rotation_and_page_store(dtype, nq, nk, dk, nv, dv, dims, page):
    torch.manual_seed(1)
    n, pages = 37, 12
    width = (nq + nk) * dk + nv * dv
    rows = rounded(torch.randn(n, width), dtype)
    positions = torch.randint(0, 5000, (n,), dtype=torch.int32)
    slots = torch.randperm(pages * page)[:n].to(torch.int32)
    slots[5] = -1                                            # a token that stores nothing
    freqs = plain.rotary_frequencies(dims, 20000.0, dict(factor=8.0, low=1.0, high=4.0, original=2048))
    qkv = rows.to(dtype).cuda()
    kc = torch.zeros((pages, max(nk, 1), page, dk), dtype=dtype, device="cuda") if nk else None
    vc = torch.zeros((pages, max(nv, 1), dv, page), dtype=dtype, device="cuda") if nv else None
    ops.rope_kv_store_general(qkv, positions.cuda(), slots.cuda() if nk or nv else None, freqs.cuda(), dims, True,
                              nq, nk, dk, nv, dv, kc, vc)
    heads = rows[:, :(nq + nk) * dk].view(n, nq + nk, dk)
    want = plain.rotate_pairs(heads, positions, freqs)
    torch.testing.assert_close(qkv[:, :nq * dk].float().cpu().view(n, nq, dk), want[:, :nq], **tol(dtype))
    for t in range(n):
        slot = int(slots[t])
        if slot < 0 or not nk:
            continue
        torch.testing.assert_close(kc[slot // page, :, slot % page].float().cpu(), want[t, nq:], **tol(dtype))
        torch.testing.assert_close(vc[slot // page, :, :, slot % page].float().cpu(),
                                   rows[t, (nq + nk) * dk:].view(nv, dv), **tol(dtype))
    if nk:
        assert float(kc.float().abs().sum(dim=(1, 3)).flatten()[torch.tensor(
            [s for s in range(pages * page) if s not in set(slots.tolist())])].max()) == 0.0   # nothing written elsewhere


# ------------------------------------------------------------------------------------------ differential attention
def paged(keys: torch.Tensor, values: torch.Tensor, page: int, dtype, seed: int):
    """Pages in shuffled order for keys [T, 2G, dk] and values [T, G, dv] of one request: (k cache, v cache, table)."""
    t = keys.shape[0]
    count = (t + page - 1) // page
    order = torch.randperm(count + 3, generator=torch.Generator().manual_seed(seed))[:count]
    kc = torch.zeros((count + 3, keys.shape[1], page, keys.shape[2]), dtype=torch.float32)
    vc = torch.zeros((count + 3, values.shape[1], values.shape[2], page), dtype=torch.float32)
    for pos in range(t):
        kc[order[pos // page], :, pos % page] = keys[pos]
        vc[order[pos // page], :, :, pos % page] = values[pos]
    return kc.to(dtype).cuda(), vc.to(dtype).cuda(), order.to(torch.int32).view(1, -1).cuda()


def plain_differential(q, k, v, heads, scale, size, keep, lam, eps, out_scale):
    """q: [T, 2H, dk], k: [T, 2G, dk], v: [T, G, dv] -> [T, H * dv] by the plain functions."""
    g = v.shape[1]
    out = []
    for head in range(heads):
        kv = head // (heads // g)
        a1 = plain.masked_softmax_attention(q[:, 2 * head], k[:, 2 * kv], v[:, kv], scale, size, keep)
        a2 = plain.masked_softmax_attention(q[:, 2 * head + 1], k[:, 2 * kv + 1], v[:, kv], scale, size, keep)
        out.append(plain.rms(a1 - lam * a2, eps) * out_scale)
    return torch.cat(out, dim=1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,g,dk,dv,page,t,size,keep", [
    (4, 2, 16, 32, 16, 150, 24, 5), (6, 6, 24, 40, 8, 70, 1000, 0), (2, 1, 8, 16, 4, 90, 7, 9),
    (3, 1, 48, 32, 16, 300, 130, 17), (2, 2, 20, 130, 8, 40, 1, 0), (4, 4, 32, 16, 32, 260, 128, 128)])
def test_differential_attention_against_the_plain_maps(dtype, heads, g, dk, dv, page, t, size, keep):
    torch.manual_seed(2)
    q = rounded(torch.randn(t, 2 * heads, dk), dtype)
    k = rounded(torch.randn(t, 2 * g, dk), dtype)
    v = rounded(torch.randn(t, g, dv), dtype)
    kc, vc, table = paged(k, v, page, dtype, seed=t)
    scale, lam, eps, out_scale = 0.4, 0.55, 1e-5, 0.7
    want = plain_differential(q, k, v, heads, scale, size, keep, lam, eps, out_scale)
    positions = torch.arange(t, dtype=torch.int32).cuda()
    entry = torch.zeros(t, dtype=torch.int32).cuda()
    got = ops.diff_attention_plain(q.view(t, -1).to(dtype).cuda(), kc, vc, table, entry, positions, heads,
                                   size, keep, scale, lam, eps, out_scale)
    torch.testing.assert_close(got.float().cpu(), want, **tol(dtype))
    # a few tokens alone, in another order: the same rows
    some = torch.tensor([t - 1, 0, t // 2, min(t - 1, keep), min(t - 1, size)], dtype=torch.int32).cuda()
    out = torch.zeros_like(got)
    ops.diff_attention_plain(q.view(t, -1).to(dtype).cuda(), kc, vc, table, entry, positions, heads, size, keep, scale,
                             lam, eps, out_scale, out=out, token_list=some)
    assert torch.equal(out[some.long()], got[some.long()])


@pytest.mark.parametrize("dtype,kernel", [(torch.float32, "plain"), (torch.bfloat16, "plain"),
                                          (torch.bfloat16, "portion"), (torch.bfloat16, "listed")])
@pytest.mark.parametrize("page,size,keep", [(16, 40, 6), (8, 33, 16), (4, 9, 2), (16, 16, 16)])
def test_one_key_stands_out_exactly_where_the_mask_lets_it(dtype, kernel, page, size, keep):
    """One key carries a large score against every query: a query's output is that key's value (normed) if and only
    if the key is the query itself, within the window or among the kept first tokens."""
    torch.manual_seed(3)
    t, dk, dv = 200, 16, 32
    direction = torch.nn.functional.normalize(torch.randn(dk), dim=0)
    for marked in (0, keep - 1, keep, keep + 1, page - 1, page, 3 * page, 77, t - 1):
        q = rounded(torch.randn(t, 2, dk) * 0.1 + 6.0 * direction, dtype)
        k = rounded(torch.randn(t, 2, dk) * 0.1, dtype)
        k[marked] = rounded(6.0 * direction, dtype)
        v = rounded(torch.randn(t, 1, dv), dtype)
        kc, vc, table = paged(k, v, page, dtype, seed=marked)
        if kernel == "plain":
            got = ops.diff_attention_plain(q.view(t, -1).to(dtype).cuda(), kc, vc, table,
                                           torch.zeros(t, dtype=torch.int32).cuda(),
                                           torch.arange(t, dtype=torch.int32).cuda(),
                                           1, size, keep, 1.0, 0.0, 1e-6, 1.0).float().cpu()
        else:
            got = run_matrix_core(kernel, q, kc, vc, table, 1, size, keep, 1.0, 0.0, 1e-6, 1.0)
        marked_value = plain.rms(v[marked, 0], 1e-6)
        for i in range(t):
            sees = plain.visible(i, marked, size, keep)
            cosine = float(torch.nn.functional.cosine_similarity(got[i], marked_value, dim=0))
            assert (cosine > 0.999) == sees, f"key {marked}, query {i}: cosine {cosine:.4f}, visible {sees}"


def run_matrix_core(kind, q, kc, vc, table, heads, size, keep, scale, lam, eps, out_scale, first=0):
    """The matrix-core kernel on the tokens at positions first .. first + len(q) - 1 of the one request whose pages
    ``table`` lists: as one portion, or as listed tokens."""
    n = q.shape[0]
    flat = q.reshape(n, -1).to(torch.bfloat16).cuda()
    out = torch.zeros((n, heads * vc.shape[2]), dtype=torch.bfloat16, device="cuda")
    args = (flat, kc, vc, table, heads, size, keep, scale, lam, eps, out_scale, out)
    if kind == "portion":
        ops.diff_attention_mfma(*args, entry_start=torch.tensor([0, n], dtype=torch.int32).cuda(),
                                entry_first_position=torch.tensor([first], dtype=torch.int32).cuda(), max_entry_len=n)
    else:
        ops.diff_attention_mfma(*args, token_entry=torch.zeros(n, dtype=torch.int32).cuda(),
                                positions=torch.arange(first, first + n, dtype=torch.int32).cuda())
    return out.float().cpu()


@pytest.mark.parametrize("kind", ["portion", "listed"])
@pytest.mark.parametrize("heads,g,dk,dv,page,t,size,keep", [
    (4, 2, 16, 32, 16, 150, 24, 5), (3, 1, 48, 32, 16, 300, 130, 17), (4, 4, 32, 16, 32, 260, 128, 128),
    (8, 2, 64, 128, 8, 200, 50, 3), (2, 1, 16, 16, 4, 90, 7, 9), (16, 1, 128, 64, 16, 70, 1000, 0),
    (6, 1, 32, 48, 16, 130, 33, 40)])
def test_matrix_core_kernel_against_the_plain_maps(kind, heads, g, dk, dv, page, t, size, keep):
    dtype = torch.bfloat16
    torch.manual_seed(9)
    q = rounded(torch.randn(t, 2 * heads, dk), dtype)
    k = rounded(torch.randn(t, 2 * g, dk), dtype)
    v = rounded(torch.randn(t, g, dv), dtype)
    kc, vc, table = paged(k, v, page, dtype, seed=t)
    assert ops.diff_attention_mfma_supported(q.view(t, -1).to(dtype).cuda(), kc, vc)
    scale, lam, eps, out_scale = 0.4, 0.55, 1e-5, 0.7
    want = plain_differential(q, k, v, heads, scale, size, keep, lam, eps, out_scale)
    got = run_matrix_core(kind, q, kc, vc, table, heads, size, keep, scale, lam, eps, out_scale)
    torch.testing.assert_close(got, want, **tol(dtype))
    # the last tokens alone, from what is cached: a portion that starts in the middle of a page, a window and a tile
    for first in (t - 1, t - 7, t // 2 + 3):
        part = run_matrix_core(kind, q[first:], kc, vc, table, heads, size, keep, scale, lam, eps, out_scale, first=first)
        torch.testing.assert_close(part, want[first:], **tol(dtype))


# ------------------------------------------------------------------------------------------ gated linear attention
def test_decays():
    torch.manual_seed(4)
    z = torch.cat([torch.randn(50, 40) * 6, torch.tensor([[-80.0, -20.0, 0.0, 20.0, 80.0] * 8])])
    for tau in (16.0, 1.0, 0.5):
        got = ops.gla_alpha_(z.clone().cuda(), tau).cpu()
        want = torch.sigmoid(z.double()).pow(1.0 / tau).float()
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-30)
        assert float(got.min()) >= 0.0 and float(got.max()) <= 1.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(3, 16, 32), (1, 20, 24), (2, 64, 128), (2, 130, 70), (5, 8, 8), (2, 48, 64), (1, 256, 16), (2, 96, 40)])
def test_recurrence_over_entries_from_their_slots(dtype, heads, dim, vdim):
    torch.manual_seed(5)
    lengths, slots = [1, 37, 2, 16, 17], [3, 0, 5, 1, 4]
    n = sum(lengths)
    width = 2 * heads * dim + heads * vdim
    rows = rounded(torch.randn(n, width) * 0.5, dtype)
    alpha = torch.rand(n, heads * dim) * 0.5 + 0.5
    state = torch.randn(6, heads, dim, vdim)
    q, k, v = rows[:, :heads * dim], rows[:, heads * dim:2 * heads * dim], rows[:, 2 * heads * dim:]
    want_o = torch.zeros(n, heads, vdim)
    want_state = state.clone()
    at = 0
    for length, slot in zip(lengths, slots):
        s = want_state[slot].clone()
        for t in range(at, at + length):
            s = alpha[t].view(heads, dim, 1) * s + k[t].view(heads, dim, 1) * v[t].view(heads, 1, vdim)
            want_o[t] = torch.einsum("hdv,hd->hv", s, q[t].view(heads, dim) * dim ** -0.5)
        want_state[slot] = s
        at += length
    device_rows = rows.to(dtype).cuda()
    device_state = state.clone().cuda()
    starts = torch.tensor([0] + torch.tensor(lengths).cumsum(0).tolist(), dtype=torch.int32).cuda()
    got = ops.gla_scan(device_rows[:, :heads * dim], device_rows[:, heads * dim:2 * heads * dim],
                       device_rows[:, 2 * heads * dim:], alpha.cuda(), starts,
                       torch.tensor(slots, dtype=torch.int32).cuda(), device_state, dim ** -0.5)
    torch.testing.assert_close(got.cpu(), want_o, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(device_state.cpu(), want_state, rtol=1e-4, atol=1e-4)
    assert torch.equal(device_state[2].cpu(), state[2])       # a slot that no entry names is left alone


@pytest.mark.parametrize("dtype", DTYPES)
def test_recurrence_cut_anywhere_gives_the_same_bits(dtype):
    torch.manual_seed(6)
    heads, dim, vdim, n = 2, 24, 40, 53
    rows = (torch.randn(n, 2 * heads * dim + heads * vdim) * 0.5).to(dtype).cuda()
    alpha = (torch.rand(n, heads * dim) * 0.3 + 0.7).cuda()

    def run(cuts):
        state = torch.zeros(2, heads, dim, vdim, device="cuda")
        outs = []
        for lo, hi in zip([0] + cuts, cuts + [n]):
            part = rows[lo:hi].contiguous()
            outs.append(ops.gla_scan(part[:, :heads * dim], part[:, heads * dim:2 * heads * dim], part[:, 2 * heads * dim:],
                                     alpha[lo:hi].contiguous(), torch.tensor([0, hi - lo], dtype=torch.int32).cuda(),
                                     torch.tensor([1], dtype=torch.int32).cuda(), state, 0.2))
        return torch.cat(outs), state
    whole, state = run([])
    for cuts in ([1], [16], [17, 19], list(range(1, n))):
        again, state_again = run(cuts)
        assert torch.equal(again, whole) and torch.equal(state_again, state)


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_norm_and_gate(dtype):
    torch.manual_seed(7)
    n, heads, vdim, eps = 19, 3, 40, 1e-5
    o = torch.randn(n, heads, vdim) * 3
    weight = torch.randn(vdim)
    gate = rounded(torch.randn(n, heads * vdim) * 2, dtype)
    got = ops.gla_norm_gate(o.cuda(), weight.cuda(), gate.to(dtype).cuda(), eps).float().cpu()
    want = (plain.rms(o, eps) * weight).reshape(n, -1) * (gate * torch.sigmoid(gate))
    torch.testing.assert_close(got, want, **tol(dtype))


# ------------------------------------------------------------------------------------------ activation, soft cap
@pytest.mark.parametrize("dtype", DTYPES)
def test_gelu_gate_and_soft_cap(dtype):
    torch.manual_seed(8)
    gate_up = rounded(torch.randn(23, 2 * 56) * 3, dtype)
    got = ops.act_mul(gate_up.to(dtype).cuda(), "gelu_tanh").float().cpu()
    torch.testing.assert_close(got, plain.gelu_tanh(gate_up[:, :56]) * gate_up[:, 56:], **tol(dtype))
    mixed = gate_up.view(23, 2, 7, 8).transpose(1, 2).reshape(23, 112)          # gate and up in blocks of 8 columns
    again = ops.act_mul(mixed.to(dtype).cuda(), "gelu_tanh", block=8).float().cpu()
    assert torch.equal(again, got)
    silu = ops.act_mul(gate_up.to(dtype).cuda(), "silu").float().cpu()
    torch.testing.assert_close(silu, torch.nn.functional.silu(gate_up[:, :56]) * gate_up[:, 56:], **tol(dtype))
    logits = torch.randn(7, 301) * 40
    capped = ops.softcap_(logits.clone().cuda(), 30.0).cpu()
    torch.testing.assert_close(capped, 30.0 * torch.tanh(logits / 30.0), rtol=1e-5, atol=1e-5)
    assert float(capped.abs().max()) <= 30.0


@pytest.mark.parametrize("rows", [1, 5, 16, 40, 64, 100, 300])
@pytest.mark.parametrize("inter,hidden", [(64, 96), (160, 64), (2048, 256)])
def test_gelu_gate_in_the_products_ends(rows, inter, hidden):
    """The gated feed-forward's first product with the tanh form of GELU taken into its end, by every kernel that the
    row count and the sizes choose (few rows, split K, many rows; plain and with the norm taken in), against the plain
    functions."""
    from somi_inference_amd.kernels import linear as linear_kernels
    torch.manual_seed(10)
    x = rounded(torch.randn(rows, hidden), torch.bfloat16)
    gate = rounded(torch.randn(inter, hidden) * 0.2, torch.bfloat16)
    up = rounded(torch.randn(inter, hidden) * 0.2, torch.bfloat16)
    merged = torch.stack([gate.view(-1, 16, hidden), up.view(-1, 16, hidden)], dim=1).reshape(-1, hidden)
    want = plain.gelu_tanh(x @ gate.t()) * (x @ up.t())
    got = linear_kernels.linear_swiglu(x.bfloat16().cuda(), merged.bfloat16().cuda(), "gelu_tanh").float().cpu()
    torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)
    silu = linear_kernels.linear_swiglu(x.bfloat16().cuda(), merged.bfloat16().cuda(), "silu").float().cpu()
    torch.testing.assert_close(silu, torch.nn.functional.silu(x @ gate.t()) * (x @ up.t()), rtol=2e-2, atol=2e-2)
    # with the norm taken in: rows h whose weighted copy and sums of squares a product into the stream left
    h = torch.randn(rows, hidden, device="cuda")
    weight = (torch.rand(hidden, device="cuda") + 0.5)
    delta = torch.zeros(rows, 8, device="cuda").bfloat16()
    stats, weighted = linear_kernels.linear_residual(delta, torch.zeros(hidden, 8, device="cuda").bfloat16(), None, h, weight)
    # what the product multiplies: the weighted rows as bfloat16 holds them, scaled per row by the norm's factor
    normed = (weighted.float() / torch.sqrt(h.pow(2).mean(-1, keepdim=True) + 1e-6)).cpu()
    fused = linear_kernels.linear_scaled(weighted, 1e-6, stats, merged.bfloat16().cuda(), swiglu="gelu_tanh").float().cpu()
    torch.testing.assert_close(fused, plain.gelu_tanh(normed @ gate.t()) * (normed @ up.t()), rtol=2e-2, atol=2e-2)
