"""Small Kamedra configurations for the tests, with seeded random weights, and what the tests share."""

from __future__ import annotations

import json
import os
import shutil

import torch

from somi_inference_amd.config import KamedraAttention, KamedraConfig, KamedraGLA, KamedraLayer, RotaryScaling


def attention(heads, kv_heads, dim, vdim, size, keep_first, rot_dims, base=10000.0, scaling=None, diff=0.4,
              scale=0.25, kv_from=None) -> KamedraAttention:
    return KamedraAttention(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, diff=diff, mask_size=size,
                            mask_keep_first=keep_first, rot_base=base, rot_dims=rot_dims,
                            rot_scaling=RotaryScaling(*scaling) if scaling else None, kv_from=kv_from)


# A: both mixers with and without a feed-forward; a layer that borrows keys and values and sees further back than
#    its lender (a wider window, fewer kept tokens); rotation of half of a head with rescaled frequencies.
# B: as many key/value heads as heads and one only; sizes that are no multiples of 16; every channel rotated and no
#    rescaling; a window longer than any test sequence; more kept tokens than the window is long; one recurrent head;
#    tau = 1; no soft cap; attention first.
# C: large recurrent heads; attention without rotation and a window of a few tokens; lender and borrower alike.
# D: recurrent layers only (no paged cache at all), a width that is no multiple of 32.
# E: attention layers only (no state), one head, a lender with two borrowers of different masks, a window of one token.
KAMEDRA = {
    "A": dict(block_size=16, seed=5, config=KamedraConfig(vocab=211, width=96, norm_eps=1e-5, logit_softcap=20.0, layers=(
        KamedraLayer("gla", KamedraGLA(heads=3, dim=16, vdim=32, tau=8.0, rank=8)),
        KamedraLayer("attention", attention(4, 2, 16, 32, 24, 5, 8, scaling=(4.0, 1.0, 4.0, 64)), ff=160),
        KamedraLayer("gla", KamedraGLA(heads=3, dim=16, vdim=32, tau=8.0, rank=8), ff=64),
        KamedraLayer("attention", attention(4, 2, 16, 32, 40, 3, 8, scaling=(4.0, 1.0, 4.0, 64), diff=0.25, kv_from=1)),
    ))),
    "B": dict(block_size=8, seed=6, config=KamedraConfig(vocab=130, width=72, norm_eps=1e-6, logit_softcap=None, layers=(
        KamedraLayer("attention", attention(6, 6, 24, 40, 1000, 0, 24, base=500.0, diff=0.7, scale=0.2), ff=100),
        KamedraLayer("gla", KamedraGLA(heads=1, dim=20, vdim=24, tau=1.0, rank=4)),
        KamedraLayer("attention", attention(2, 1, 8, 16, 7, 9, 4, scaling=(2.0, 2.0, 8.0, 16), diff=0.1, scale=0.5)),
    ))),
    "C": dict(block_size=16, seed=7, config=KamedraConfig(vocab=97, width=64, norm_eps=1e-6, logit_softcap=8.0, layers=(
        KamedraLayer("gla", KamedraGLA(heads=2, dim=64, vdim=128, tau=32.0, rank=16), ff=96),
        KamedraLayer("attention", attention(2, 2, 48, 32, 16, 1, 0, diff=0.5, scale=0.15)),
        KamedraLayer("attention", attention(2, 2, 48, 32, 16, 1, 0, diff=0.5, scale=0.15, kv_from=1), ff=48),
    ))),
    "D": dict(block_size=16, seed=8, config=KamedraConfig(vocab=61, width=48, norm_eps=1e-6, logit_softcap=15.0, layers=(
        KamedraLayer("gla", KamedraGLA(heads=2, dim=12, vdim=20, tau=4.0, rank=6), ff=72),
        KamedraLayer("gla", KamedraGLA(heads=4, dim=8, vdim=16, tau=2.0, rank=3)),
    ))),
    "E": dict(block_size=8, seed=9, config=KamedraConfig(vocab=83, width=64, norm_eps=1e-5, logit_softcap=None, layers=(
        KamedraLayer("attention", attention(1, 1, 32, 32, 12, 2, 32, base=100.0, diff=0.3, scale=0.2)),
        KamedraLayer("attention", attention(1, 1, 32, 32, 1, 0, 32, base=100.0, diff=0.8, scale=0.3, kv_from=0), ff=40),
        KamedraLayer("attention", attention(1, 1, 32, 32, 50, 7, 32, base=100.0, diff=0.2, scale=0.1, kv_from=0)),
    ))),
}


def write_kamedra(name: str, folder: str, peaky: float = 1.0, steady: bool = False) -> str:
    """The model folder of configuration ``name``.  ``peaky`` scales the attention layers' query and key projections,
    so that scores spread over several units: single keys stand out and a wrong key, page, kept token or window
    edge changes the logits.

    ``steady``: the recurrent layers' key projection is set equal to their query projection.  A recurrent head's
    output is divided by its own root mean square, so at a sequence's first tokens, where it is k.q times one value
    vector, only the sign of k.q survives: with independent random projections that product is now and then near
    zero, and rounding to bfloat16 flips the whole head.  With equal projections k.q of a token with itself is
    positive, and bfloat16 results can be held to a bound.  float32 tests run on both kinds of model."""
    from safetensors.torch import load_file, save_file

    from somi_inference_amd.weights import write_random_model
    config = KAMEDRA[name]["config"]
    write_random_model(folder, config, seed=KAMEDRA[name]["seed"])
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for index, layer in enumerate(config.layers):
        # activations of a random model this small are tiny: widen every projection so that mixers matter
        for name_, tensor in list(tensors.items()):
            if name_.startswith(f"l{index}.mix.") and tensor.dim() == 2:
                boost = 4.0
                if layer.type == "attention" and name_.endswith((".q", ".k")):
                    boost *= peaky
                tensors[name_] = (tensor.float() * boost).to(tensor.dtype)
        if steady and layer.type == "gla":
            tensors[f"l{index}.mix.k"] = tensors[f"l{index}.mix.q"].clone()
    save_file(tensors, path)
    return folder


def load_plain(folder: str):
    from plain import kamedra_plain
    return kamedra_plain.load_folder(folder)
