"""The Rusolorn decoder as a plan: parallel layers (one norm without statistics, mixer and feed-forward side by side,
a scaled residual add), whose mixer is windowed attention with the keys as values beside a gated delta rule, whose
feed-forward is a mixture of experts, and which add a per-layer token input; a scaled embedding and a tied head.

Tensor names: ``embed``, ``side.embed``, ``final.norm`` (with ``.alpha`` and ``.b``), and per layer ``l<i>.norm1``,
``l<i>.mix.{left,right}.<name>``, ``l<i>.mlp.{router,e<j>.gate,...,shared.gate,...}``, ``l<i>.side.{gate,proj,norm}``;
no name carries a ``.weight`` suffix.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.rusolorn import RusolornConfig
from ..parts.base import PartSpec
from .plan import LayerSpec, ModelPlan

ATTENTION_NAMES = {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}
DELTA_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "b": "b", "a": "a", "norm": "norm", "a_log": "A_log",
               "dt_bias": "dt_bias", "conv": "conv"}
BLOCK_NAMES = {"norm": "", "mixer": "mix", "feed_forward": "mlp", "token_input": "side"}
SIDE_TABLE = "side.embed"


def rusolorn_plan(config: RusolornConfig) -> ModelPlan:
    def norm(tensor: str) -> PartSpec:
        return PartSpec("dynamic_tanh", {"hidden_size": config.width, "tensor": tensor})

    layers = []
    for index, layer in enumerate(config.layers):
        left, right, mlp = layer.left, layer.right, layer.mlp
        mixer = PartSpec("parallel", {
            "hidden_size": config.width, "eps": config.norm_eps,
            "left": PartSpec("gqa_attention", {
                "hidden_size": config.width, "num_heads": left.heads, "num_kv_heads": left.kv_heads, "head_dim": left.dim,
                "position": PartSpec("none", {}), "qkv_bias": False, "window": left.window, "scale": left.scale,
                "values": "keys", "qk_norm": "projection", "norm_eps": config.norm_eps, "names": ATTENTION_NAMES,
                "suffix": ""}),
            "right": PartSpec("gated_delta_rule", {
                "hidden_size": config.width, "num_heads": right.heads, "num_groups": right.kv_heads, "key_dim": right.dim,
                "value_dim": right.vdim, "taps": right.conv, "eps": config.norm_eps, "names": DELTA_NAMES, "suffix": ""})})
        feed_forward = None if mlp is None else PartSpec("routed_experts", {
            "hidden_size": config.width, "num_experts": mlp.experts, "top": mlp.top, "expert_size": mlp.ff,
            "limit": mlp.limit, "groups": mlp.groups, "keep_groups": mlp.keep, "shared_size": mlp.shared_ff,
            "shared_limit": mlp.shared_limit, "suffix": ""})
        token_input = None if config.token_side_dim is None else PartSpec("gated_table", {
            "hidden_size": config.width, "vocab_size": config.vocab, "dim": config.token_side_dim, "table": SIDE_TABLE,
            "table_width": config.token_side_dim * len(config.layers), "offset": index * config.token_side_dim,
            "eps": config.norm_eps})
        block = PartSpec("parallel", {"mixer": mixer, "feed_forward": feed_forward, "norm": norm("norm1"),
                                      "residual_mult": config.residual_mult, "token_input": token_input,
                                      "names": BLOCK_NAMES})
        layers.append(LayerSpec(f"l{index}", block))
    return ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": config.width, "tensor": "embed",
                                               "scale": config.embedding_scale}),
        embedding_prefix="",
        layers=tuple(layers),
        final_norm=norm("norm"),
        final_norm_prefix="final",
        head=PartSpec("lm_head", {"vocab_size": config.vocab, "hidden_size": config.width, "tied": True}),
        head_prefix="",
        vocab_size=config.vocab,
    )


register_architecture(RusolornConfig.architecture, RusolornConfig, rusolorn_plan, replace=True)
