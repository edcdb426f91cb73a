"""Plain Kamedra decoder: one slow float32 function per mechanism, whole sequences at a time.

Written from the design's equations; it shares no code with the engine.  ``weights`` maps tensor names to
float32 tensors, ``config`` is the parsed config.json.  Notation: ``h`` a mixer's input ``[T, width]``,
``p`` positions, ``i`` a query's position and ``j`` a key's.
"""

from __future__ import annotations

import json
import math
import os

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return rms(x, eps) * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z.pow(3))))


# ------------------------------------------------------------------------------------------ rotation
def rotary_frequencies(dims: int, base: float, scaling: dict | None) -> torch.Tensor:
    """f_i = base^(-2i/dims) for i < dims/2, then the wavelength-dependent rescaling: with l = 2 pi / f, f stays
    where l < original/high, becomes f/factor where l > original/low, and is blended linearly in between."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
            original = float(scaling["original"])
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float32)


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x: [T, heads, dim]; channels (2i, 2i+1) for i < len(freqs) turn by the angle p * f_i, the rest pass."""
    out = x.clone()
    angle = positions.to(torch.float32).unsqueeze(1) * freqs.unsqueeze(0)      # [T, dims/2]
    cos, sin = angle.cos().unsqueeze(1), angle.sin().unsqueeze(1)
    dims = 2 * freqs.numel()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ------------------------------------------------------------------------------------------ attention
def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def visibility(t: int, size: int, keep_first: int) -> torch.Tensor:
    """[T, T] booleans: row i, column j is ``visible(i, j, size, keep_first)``."""
    i, j = torch.arange(t).unsqueeze(1), torch.arange(t).unsqueeze(0)
    return (j <= i) & ((i - j < size) | (j < keep_first))


def masked_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, size: int,
                             keep_first: int) -> torch.Tensor:
    """q: [T, dim], k: [T, dim], v: [T, vdim] of one head and one map -> [T, vdim]."""
    scores = (q @ k.t()) * scale
    scores = scores.masked_fill(~visibility(q.shape[0], size, keep_first), float("-inf"))
    return torch.softmax(scores, dim=-1) @ v


def attention_keys_values(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, positions: torch.Tensor):
    """Rotated keys [T, 2 G, dim] and values [T, G, vdim] of a layer that has projections of its own."""
    g, dim, vdim = mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    t = h.shape[0]
    freqs = rotary_frequencies(mixer["rot"]["dims"], mixer["rot"]["base"], mixer["rot"].get("scaling"))
    k = (h @ weights[prefix + ".mix.k"].t()).view(t, 2 * g, dim)
    v = (h @ weights[prefix + ".mix.v"].t()).view(t, g, vdim)
    return rotate_pairs(k, positions, freqs), v


def differential_attention(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float,
                           positions: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Two softmax maps per head over the same values, joined as a1 - lambda a2, unit-normed per head, scaled by
    (1 - diff), then the output projection.  k, v: this layer's or the layer's it borrows them from."""
    heads, g, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    t = h.shape[0]
    freqs = rotary_frequencies(mixer["rot"]["dims"], mixer["rot"]["base"], mixer["rot"].get("scaling"))
    q = rotate_pairs((h @ weights[prefix + ".mix.q"].t()).view(t, 2 * heads, dim), positions, freqs)
    lam = (math.exp(float((weights[prefix + ".mix.lq1"] * weights[prefix + ".mix.lk1"]).sum()))
           - math.exp(float((weights[prefix + ".mix.lq2"] * weights[prefix + ".mix.lk2"]).sum())) + mixer["diff"])
    size, keep = mixer["mask"]["size"], mixer["mask"]["keep_first"]
    out = torch.zeros((t, heads, vdim), dtype=torch.float32)
    for head in range(heads):
        kv = head // (heads // g)
        a1 = masked_softmax_attention(q[:, 2 * head], k[:, 2 * kv], v[:, kv], mixer["scale"], size, keep)
        a2 = masked_softmax_attention(q[:, 2 * head + 1], k[:, 2 * kv + 1], v[:, kv], mixer["scale"], size, keep)
        out[:, head] = rms(a1 - lam * a2, eps) * (1.0 - mixer["diff"])
    return out.reshape(t, heads * vdim) @ weights[prefix + ".mix.o"].t()


# ------------------------------------------------------------------------------------------ gated linear attention
def gated_linear_attention(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float,
                           state: torch.Tensor | None = None):
    """Token by token: S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t, per head, S: [dim, vdim] from zero.
    Returns (output [T, width], final state [heads, dim, vdim])."""
    heads, dim, vdim, tau = mixer["heads"], mixer["dim"], mixer["vdim"], float(mixer["tau"])
    t = h.shape[0]
    q = (h @ weights[prefix + ".mix.q"].t()).view(t, heads, dim) * dim ** -0.5
    k = (h @ weights[prefix + ".mix.k"].t()).view(t, heads, dim)
    v = (h @ weights[prefix + ".mix.v"].t()).view(t, heads, vdim)
    z = (h @ weights[prefix + ".mix.a1"].t()) @ weights[prefix + ".mix.a2"].t() + weights[prefix + ".mix.a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / tau).view(t, heads, dim)
    s = torch.zeros((heads, dim, vdim), dtype=torch.float32) if state is None else state.clone()
    o = torch.zeros((t, heads, vdim), dtype=torch.float32)
    for step in range(t):
        s = alpha[step].unsqueeze(-1) * s + k[step].unsqueeze(-1) * v[step].unsqueeze(-2)
        o[step] = torch.einsum("hdv,hd->hv", s, q[step])
    o = rms(o, eps) * weights[prefix + ".mix.norm"]
    gate = h @ weights[prefix + ".mix.g"].t()
    y = o.reshape(t, heads * vdim) * (gate * torch.sigmoid(gate))
    return y @ weights[prefix + ".mix.o"].t(), s


# ------------------------------------------------------------------------------------------ feed-forward
def dense_feed_forward(x: torch.Tensor, weights: dict, prefix: str) -> torch.Tensor:
    gate = gelu_tanh(x @ weights[prefix + ".mlp.gate"].t())
    return (gate * (x @ weights[prefix + ".mlp.up"].t())) @ weights[prefix + ".mlp.down"].t()


# ------------------------------------------------------------------------------------------ the model
def forward(config: dict, weights: dict, tokens: list[int], return_layers: bool = False):
    """Logits [T, vocab] of a whole sequence from position 0 (and the residual stream after every layer)."""
    eps = float(config["norm"]["eps"])
    positions = torch.arange(len(tokens))
    x = weights["embed"][torch.tensor(tokens, dtype=torch.long)].clone()
    kept: dict[int, tuple] = {}
    after = []
    for index, layer in enumerate(config["layers"]):
        prefix, mixer = f"l{index}", layer["mixer"]
        h = rms_norm(x, weights[prefix + ".norm1"], eps)
        if layer["type"] == "attention":
            if mixer.get("kv_from") is None:
                kept[index] = attention_keys_values(h, weights, prefix, mixer, positions)
                k, v = kept[index]
            else:
                k, v = kept[mixer["kv_from"]]
            x = x + differential_attention(h, weights, prefix, mixer, eps, positions, k, v)
        elif layer["type"] == "gla":
            x = x + gated_linear_attention(h, weights, prefix, mixer, eps)[0]
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            x = x + dense_feed_forward(rms_norm(x, weights[prefix + ".norm2"], eps), weights, prefix)
        after.append(x.clone())
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["embed"].t()
    cap = config.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return (logits, torch.stack(after)) if return_layers else logits


def load_folder(folder: str):
    """(config, float32 weights) of a model folder."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: tensor.to(torch.float32) if tensor.is_floating_point() else tensor
               for name, tensor in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, weights
