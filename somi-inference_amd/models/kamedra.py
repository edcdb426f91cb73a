"""The Kamedra decoder as a plan: per layer a differential-attention or a gated-linear-attention mixer, an optional
dense feed-forward with the tanh form of GELU, a tied head with a soft cap on the logits.

Tensor names: ``embed``, ``final.norm``, and per layer ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>``,
``l<i>.mlp.{gate,up,down}``; no name carries a ``.weight`` suffix.
"""

from __future__ import annotations

from ..config.kamedra import KamedraConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .plan import LayerSpec, ModelPlan

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}
GLA_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}
BLOCK_NAMES = {"mixer_norm": "", "mixer": "mix", "ffn_norm": "", "feed_forward": "mlp"}


def kamedra_plan(config: KamedraConfig) -> ModelPlan:
    def norm(tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"hidden_size": config.width, "eps": config.norm_eps, "tensor": tensor})

    # what the layers that borrow a layer's keys and values see of them: the lender's cache keeps that much
    readers: dict[int, list[tuple[int | None, int]]] = {}
    for layer in config.layers:
        if layer.type == "attention" and layer.mixer.kv_from is not None:
            readers.setdefault(layer.mixer.kv_from, []).append((layer.mixer.mask_size, layer.mixer.mask_keep_first))
    layers, cache_from = [], {}
    for index, layer in enumerate(config.layers):
        m = layer.mixer
        if layer.type == "attention":
            scaling = None if m.rot_scaling is None else m.rot_scaling.to_dict()
            position = (PartSpec("rotary", {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims,
                                            "pairing": "neighbours", "scaling": scaling})
                        if m.rot_dims > 0 else PartSpec("none", {}))
            mixer = PartSpec("diff_attention", {
                "hidden_size": config.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                "value_dim": m.vdim, "position": position, "scale": m.scale, "diff": m.diff, "eps": config.norm_eps,
                "window": m.mask_size, "keep_first": m.mask_keep_first, "shares_cache": m.kv_from is not None,
                "reader_masks": tuple(readers.get(index, ())), "names": ATTENTION_NAMES, "suffix": ""})
            if m.kv_from is not None:
                cache_from[index] = m.kv_from
        else:
            mixer = PartSpec("gated_linear_attention", {
                "hidden_size": config.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
                "tau": m.tau, "eps": config.norm_eps, "rank": m.rank, "names": GLA_NAMES, "suffix": ""})
        feed_forward = None if layer.ff is None else PartSpec("swiglu", {
            "hidden_size": config.width, "intermediate_size": layer.ff, "activation": "gelu_tanh",
            "names": {"gate": "gate", "up": "up", "down": "down"}, "suffix": ""})
        block = PartSpec("pre_norm", {"mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm("norm1"),
                                      "ffn_norm": None if layer.ff is None else norm("norm2"), "names": BLOCK_NAMES})
        layers.append(LayerSpec(f"l{index}", block))
    return ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": config.width, "tensor": "embed"}),
        embedding_prefix="",
        layers=tuple(layers),
        final_norm=norm("norm"),
        final_norm_prefix="final",
        head=PartSpec("lm_head", {"vocab_size": config.vocab, "hidden_size": config.width, "tied": True,
                                  "softcap": config.logit_softcap}),
        head_prefix="",
        cache_from=cache_from,
        vocab_size=config.vocab,
    )


register_architecture(KamedraConfig.architecture, KamedraConfig, kamedra_plan, replace=True)
