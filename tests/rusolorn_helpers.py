"""Small Rusolorn configurations for the tests, with seeded random weights, and what the tests share."""

from __future__ import annotations

import os

import torch

from somi_inference_amd.config import (RusolornAttention, RusolornConfig, RusolornDeltaRule, RusolornExperts,
                                       RusolornLayer)


def layer(left, right, mlp=None) -> RusolornLayer:
    heads, kv, dim, window, scale = left
    rheads, rkv, rdim, rvdim, conv = right
    return RusolornLayer(left=RusolornAttention(heads=heads, kv_heads=kv, dim=dim, vdim=dim, scale=scale, window=window),
                         right=RusolornDeltaRule(heads=rheads, kv_heads=rkv, dim=rdim, vdim=rvdim, conv=conv),
                         mlp=None if mlp is None else RusolornExperts(**mlp))


# A: grouped heads in both mixers, experts in groups of which some are dropped, a shared expert with a limit of its
#    own, a token input, a residual multiplier and an embedding scale; layers that differ in window and sizes.
# B: as many key/value heads as heads, sizes that are no multiples of 16, a window longer than any test sequence, one
#    recurrent head, a convolution of two taps, a layer without a feed-forward, one expert a token, no groups, no
#    shared expert, no token input, multipliers of 1.
# C: windows of one and of seven tokens, no convolution (one tap), large recurrent heads, every expert chosen,
#    pages of 8 tokens, a width that is no multiple of 32.
# D: a width that is no multiple of 8, odd sizes everywhere, five taps, three q/k-sharing recurrent heads, experts
#    without groups beside a shared one, layers that differ in everything.
RUSOLORN = {
    "A": dict(block_size=16, seed=5, config=RusolornConfig(
        vocab=211, width=96, norm_eps=1e-5, embedding_scale=4.0, residual_mult=0.5, token_side_dim=8, layers=(
            layer((4, 2, 16, 24, 0.5), (4, 2, 16, 32, 4),
                  dict(experts=8, top=2, ff=48, limit=1.0, groups=4, keep=2, shared_ff=64, shared_limit=2.5)),
            layer((6, 1, 32, 36, 0.3), (2, 1, 32, 16, 3),
                  dict(experts=6, top=3, ff=32, limit=2.0, groups=3, keep=2, shared_ff=16, shared_limit=0.5)),
            layer((4, 2, 16, 24, 0.5), (4, 2, 16, 32, 4),
                  dict(experts=8, top=2, ff=48, limit=1.0, groups=4, keep=2, shared_ff=64, shared_limit=2.5)),
        ))),
    "B": dict(block_size=8, seed=6, config=RusolornConfig(
        vocab=130, width=72, norm_eps=1e-6, embedding_scale=1.0, residual_mult=1.0, token_side_dim=None, layers=(
            layer((3, 3, 24, 1000, 0.4), (1, 1, 20, 24, 2), dict(experts=5, top=1, ff=40, limit=3.0)),
            layer((3, 3, 24, 1000, 0.4), (3, 3, 12, 20, 2), None),
        ))),
    "C": dict(block_size=8, seed=7, config=RusolornConfig(
        vocab=97, width=80, norm_eps=1e-6, embedding_scale=9.0, residual_mult=1.3, token_side_dim=5, layers=(
            layer((2, 2, 48, 1, 0.2), (2, 1, 64, 128, 1), dict(experts=4, top=4, ff=24, limit=1.5, groups=2, keep=2)),
            layer((2, 1, 16, 7, 0.6), (2, 2, 8, 8, 1),
                  dict(experts=4, top=2, ff=24, limit=1.5, groups=4, keep=3, shared_ff=8, shared_limit=1.0)),
        ))),
    "D": dict(block_size=16, seed=8, config=RusolornConfig(
        vocab=77, width=100, norm_eps=1e-5, embedding_scale=2.5, residual_mult=0.8, token_side_dim=7, layers=(
            layer((5, 5, 12, 5, 0.7), (3, 1, 36, 28, 5), dict(experts=3, top=2, ff=20, limit=2.0, shared_ff=12, shared_limit=3.0)),
            layer((1, 1, 40, 50, 0.3), (1, 1, 10, 6, 2), None),
            layer((4, 2, 8, 9, 0.9), (6, 2, 6, 10, 3), dict(experts=7, top=3, ff=9, limit=0.7)),
        ))),
}


def write_rusolorn(name: str, folder: str, steady: bool = True) -> str:
    """The model folder of configuration ``name``.  Matrices of the feed-forward and of the token input are widened
    (random weights this small would leave them without a say), the norms' alphas set so that the tanh is neither
    linear nor saturated.

    ``steady``: the recurrent mixer's key projection and taps are set equal to the query's.  A recurrent head's
    output is divided by its own root mean square, so at a sequence's first tokens, where it is k.q times one value
    vector, only the sign of k.q survives: with independent random projections that product is now and then near
    zero, and rounding to bfloat16 flips the whole head.  With equal projections k.q is positive, and bfloat16
    results can be held to a bound.  float32 tests run on both kinds of model."""
    from safetensors.torch import load_file, save_file

    from somi_inference_amd.weights import write_random_model
    config = RUSOLORN[name]["config"]
    write_random_model(folder, config, seed=RUSOLORN[name]["seed"])
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key, tensor in list(tensors.items()):
        if tensor.dim() == 2 and (".mlp." in key or ".side." in key or key == "side.embed") and not key.endswith(".router"):
            tensors[key] = (tensor.float() * 8.0).to(tensor.dtype)
        if key.endswith(".router") or key.endswith(".right.b") or key.endswith(".right.a"):
            tensors[key] = (tensor.float() * 60.0).to(tensor.dtype)       # routers and gates that decide something
        if key == "embed":
            tensors[key] = (tensor.float() * 20.0).to(tensor.dtype)
    if steady:
        for index in range(len(config.layers)):
            tensors[f"l{index}.mix.right.k"] = tensors[f"l{index}.mix.right.q"].clone()
            tensors[f"l{index}.mix.right.k.conv"] = tensors[f"l{index}.mix.right.q.conv"].clone()
    save_file(tensors, path)
    return folder


def load_plain(folder: str):
    from plain import rusolorn_plain
    return rusolorn_plain.load_folder(folder)
