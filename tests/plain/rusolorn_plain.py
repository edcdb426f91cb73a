"""Plain Rusolorn decoder: one slow float32 function per mechanism, whole sequences at a time.

Written from the design's equations; it shares no code with the engine.  ``weights`` maps tensor names to
float32 tensors, ``config`` is the parsed config.json.  Notation: ``x`` the residual stream ``[T, width]``,
``h`` a sublayer's input, ``i`` a query's position and ``j`` a key's.
"""

from __future__ import annotations

import json
import math
import os

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def dynamic_tanh(x: torch.Tensor, weights: dict, name: str) -> torch.Tensor:
    """tanh(alpha x) * w + b: a norm without statistics."""
    return torch.tanh(weights[name + ".alpha"] * x) * weights[name] + weights[name + ".b"]


# ------------------------------------------------------------------------------------- windowed attention
def tied_window_attention(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float) -> torch.Tensor:
    """Softmax attention whose values are the keys as projected.  q and k are RMS-normed over their whole
    projection (all heads at once) with a weight of that size; the values are k before that norm.  Position i sees
    j with 0 <= i - j < size; no rotation."""
    heads, groups, dim = mixer["heads"], mixer["kv_heads"], mixer["dim"]
    size, scale = mixer["mask"]["size"], mixer["scale"]
    tokens = h.shape[0]
    q = h @ weights[prefix + ".q"].T
    k = h @ weights[prefix + ".k"].T
    v = k.view(tokens, groups, dim)
    q = (rms(q, eps) * weights[prefix + ".q.norm"]).view(tokens, heads, dim)
    k = (rms(k, eps) * weights[prefix + ".k.norm"]).view(tokens, groups, dim)
    out = torch.zeros(tokens, heads, dim)
    for i in range(tokens):
        lo = max(0, i - size + 1)
        for a in range(heads):
            g = a // (heads // groups)
            s = (k[lo:i + 1, g] @ q[i, a]) * scale
            out[i, a] = torch.softmax(s, dim=0) @ v[lo:i + 1, g]
    return out.reshape(tokens, heads * dim) @ weights[prefix + ".o"].T


# ------------------------------------------------------------------------------------- gated delta rule
def short_convolution(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """y[t, c] = sum_d taps[c, last - d] x[t - d, c] with zeros before the start, then SiLU."""
    tokens, width = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for d in range(min(width, tokens)):
        y[d:] += x[:tokens - d] * taps[:, width - 1 - d]
    return silu(y)


def gated_delta_rule(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float) -> torch.Tensor:
    heads, groups, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    tokens = h.shape[0]
    q = short_convolution(h @ weights[prefix + ".q"].T, weights[prefix + ".q.conv"]).view(tokens, groups, dim)
    k = short_convolution(h @ weights[prefix + ".k"].T, weights[prefix + ".k.conv"]).view(tokens, groups, dim)
    v = short_convolution(h @ weights[prefix + ".v"].T, weights[prefix + ".v.conv"]).view(tokens, heads, vdim)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ weights[prefix + ".b"].T)                                   # [T, heads]
    rate = torch.exp(weights[prefix + ".A_log"])
    decay = torch.exp(-rate * torch.nn.functional.softplus(h @ weights[prefix + ".a"].T + weights[prefix + ".dt_bias"]))
    gate = silu(h @ weights[prefix + ".g"].T).view(tokens, heads, vdim)
    out = torch.zeros(tokens, heads, vdim)
    for a in range(heads):
        g = a // (heads // groups)
        state = torch.zeros(dim, vdim)
        for t in range(tokens):
            state = decay[t, a] * state
            u = beta[t, a] * (v[t, a] - state.T @ k[t, g])
            state = state + torch.outer(k[t, g], u)
            out[t, a] = state.T @ q[t, g]
    out = rms(out, eps) * weights[prefix + ".norm"] * gate
    return out.reshape(tokens, heads * vdim) @ weights[prefix + ".o"].T


def parallel_mixer(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float) -> torch.Tensor:
    """Half the sum of the two mixers' outputs, each RMS-normed over the width with a weight of its own."""
    left = tied_window_attention(h, weights, prefix + ".left", mixer["left"], eps)
    right = gated_delta_rule(h, weights, prefix + ".right", mixer["right"], eps)
    return 0.5 * (rms(left, eps) * weights[prefix + ".left.out"] + rms(right, eps) * weights[prefix + ".right.out"])


# ------------------------------------------------------------------------------------- feed-forward
def clamped_expert(h: torch.Tensor, weights: dict, prefix: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ weights[prefix + ".gate"].T, max=limit)
    u = torch.clamp(h @ weights[prefix + ".up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ weights[prefix + ".down"].T


def route(h: torch.Tensor, router: torch.Tensor, top: int, groups: int, keep: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Chosen experts [T, top] and their weights: softmax scores over all experts; experts come in ``groups`` equal
    runs of neighbours, a run scores as its best expert, only the ``keep`` best runs stay; of those the ``top`` best
    experts, weighted by their scores over the scores' sum."""
    scores = torch.softmax(h @ router.T, dim=-1)
    tokens, experts = scores.shape
    chosen = torch.zeros(tokens, top, dtype=torch.long)
    weight = torch.zeros(tokens, top)
    per = experts // groups
    for t in range(tokens):
        best = sorted(range(groups), key=lambda g: (-float(scores[t, g * per:(g + 1) * per].max()), g))[:keep]
        allowed = [e for e in range(experts) if e // per in best]
        picks = sorted(allowed, key=lambda e: (-float(scores[t, e]), e))[:top]
        chosen[t] = torch.tensor(picks)
        weight[t] = scores[t, picks] / (scores[t, picks].sum() + 1e-20)
    return chosen, weight


def routing_margins(h: torch.Tensor, router: torch.Tensor, top: int, groups: int, keep: int) -> torch.Tensor:
    """Per token, how far the router's decisions are from a tie: the smaller of (the last chosen expert's score over
    the best allowed expert's that was not chosen) and (the last kept run's score over the best dropped run's), minus
    one.  A token with a small margin may be routed otherwise by rounding alone."""
    scores = torch.softmax(h @ router.T, dim=-1)
    tokens, experts = scores.shape
    per = experts // groups
    chosen, _ = route(h, router, top, groups, keep)
    out = torch.full((tokens,), float("inf"))
    for t in range(tokens):
        runs = sorted((float(scores[t, g * per:(g + 1) * per].max()) for g in range(groups)), reverse=True)
        if keep < groups:
            out[t] = min(float(out[t]), runs[keep - 1] / runs[keep] - 1.0)
        kept = sorted(range(groups), key=lambda g: (-float(scores[t, g * per:(g + 1) * per].max()), g))[:keep]
        rest = [float(scores[t, e]) for e in range(experts) if e // per in kept and e not in chosen[t].tolist()]
        if rest:
            out[t] = min(float(out[t]), float(scores[t, chosen[t]].min()) / max(rest) - 1.0)
    return out


def mixture(h: torch.Tensor, weights: dict, prefix: str, mlp: dict, margins: list | None = None) -> torch.Tensor:
    router = mlp["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    chosen, weight = route(h, weights[prefix + ".router"], router["top"], groups["count"], groups["keep"])
    if margins is not None:
        margins.append(routing_margins(h, weights[prefix + ".router"], router["top"], groups["count"], groups["keep"]))
    out = torch.zeros(h.shape[0], weights[prefix + ".e0.down"].shape[0])
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weight[t]):
            out[t] += w * clamped_expert(h[t:t + 1], weights, f"{prefix}.e{e}", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + clamped_expert(h, weights, prefix + ".shared", mlp["shared"]["limit"])
    return out


# ------------------------------------------------------------------------------------- the model
def token_side(x: torch.Tensor, tokens: torch.Tensor, weights: dict, layer: int, dim: int, eps: float) -> torch.Tensor:
    """What a layer adds from its slice of the second embedding table (before the residual multiplier)."""
    e = weights["side.embed"][tokens, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ weights[f"l{layer}.side.gate"].T) * e) @ weights[f"l{layer}.side.proj"].T
    return rms(y, eps) * weights[f"l{layer}.side.norm"]


def forward(config: dict, weights: dict, tokens: list[int], keep_layers: bool = False, margins: list | None = None):
    """Logits [T, vocab] of a whole sequence; with ``keep_layers`` also the residual stream after every layer;
    ``margins`` collects every routed layer's :func:`routing_margins`."""
    ids = torch.tensor(tokens, dtype=torch.long)
    eps, m = config["norm"]["eps"], config.get("residual_mult", 1.0)
    x = weights["embed"][ids] * config["embedding"]["scale"]
    side = config.get("token_side")
    kept = []
    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}"
        h = dynamic_tanh(x, weights, prefix + ".norm1")
        delta = parallel_mixer(h, weights, prefix + ".mix", layer["mixer"], eps)
        if layer.get("mlp"):
            delta = delta + mixture(h, weights, prefix + ".mlp", layer["mlp"], margins)
        x = x + m * delta
        if side:
            x = x + m * token_side(x, ids, weights, index, side["dim"], eps)
        kept.append(x.clone())
    logits = dynamic_tanh(x, weights, "final.norm") @ weights["embed"].T
    return (logits, torch.stack(kept)) if keep_layers else logits


def load_folder(folder: str) -> tuple[dict, dict]:
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: (t.to(torch.float32) if t.is_floating_point() else t)
               for name, t in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, weights
