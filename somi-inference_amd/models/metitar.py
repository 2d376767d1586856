"""The Metitar decoder as a plan: layers that norm their sublayers' outputs (layer norm with a bias), read their mixer's
input through a short causal convolution of the residual stream, and add a per-layer token input; the mixer is
attention over a shared low-rank latent (a layer may read the latent an earlier layer kept) or the HGRN2 recurrence,
the feed-forward a dense one with normed powers or a mixture of experts with sigmoid scores whose weights scale the
experts' inputs; a scaled embedding, an untied head and scaled logits.

Tensor names: ``embed``, ``side.embed``, ``final.norm`` (with ``.b``), ``head``, and per layer ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.canon1``, ``l<i>.mix.<name>``, ``l<i>.mlp.{up,down,act}`` or ``l<i>.mlp.{router,e<j>.gate,...,
shared.gate,...}``, ``l<i>.side.{gate,proj,norm}``; no name carries a ``.weight`` suffix.
"""

from __future__ import annotations

from ..config.metitar import MetitarConfig, MetitarDense
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .plan import LayerSpec, ModelPlan

BLOCK_NAMES = {"mixer_norm": "", "mixer": "mix", "ffn_norm": "", "feed_forward": "mlp", "input_conv": "canon1",
               "token_input": "side"}
SIDE_TABLE = "side.embed"


def metitar_plan(config: MetitarConfig) -> ModelPlan:
    def norm(tensor: str) -> PartSpec:
        return PartSpec("layer_norm", {"hidden_size": config.width, "eps": config.norm_eps, "tensor": tensor})

    layers, cache_from = [], {}
    for index, layer in enumerate(config.layers):
        m = layer.mixer
        if layer.type == "latent_attention":
            scaling = None if m.rot_scaling is None else m.rot_scaling.to_dict()
            position = (PartSpec("rotary", {"head_dim": m.rot_dim, "theta": m.rot_base, "rotary_dim": m.rot_dims,
                                            "pairing": "half", "scaling": scaling})
                        if m.rot_dims > 0 else PartSpec("none", {}))
            mixer = PartSpec("latent_attention", {
                "hidden_size": config.width, "num_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
                "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale, "eps": config.norm_eps, "position": position,
                "shares_cache": m.kv_from is not None, "suffix": ""})
            if m.kv_from is not None:
                cache_from[index] = m.kv_from
        else:
            mixer = PartSpec("hgrn2", {"hidden_size": config.width, "num_heads": m.heads, "key_dim": m.dim,
                                       "value_dim": m.vdim, "eps": config.norm_eps, "suffix": ""})
        mlp = layer.mlp
        if mlp is None:
            feed_forward = None
        elif isinstance(mlp, MetitarDense):
            feed_forward = PartSpec("poly_norm", {"hidden_size": config.width, "intermediate_size": mlp.ff,
                                                  "eps": config.norm_eps, "suffix": ""})
        else:
            feed_forward = PartSpec("routed_experts", {
                "hidden_size": config.width, "num_experts": mlp.experts, "top": mlp.top, "expert_size": mlp.ff,
                "limit": None, "alpha": 1.0, "shift": 0.0, "shared_size": mlp.shared_ff, "scores": "sigmoid",
                "normalize": False, "weight_on": "input", "suffix": ""})
        input_conv = (None if config.canon_taps is None
                      else PartSpec("short_causal", {"hidden_size": config.width, "taps": config.canon_taps}))
        token_input = None if config.token_side_dim is None else PartSpec("gated_table", {
            "hidden_size": config.width, "vocab_size": config.vocab, "dim": config.token_side_dim, "table": SIDE_TABLE,
            "table_width": config.token_side_dim * len(config.layers), "offset": index * config.token_side_dim,
            "eps": config.norm_eps})
        block = PartSpec("output_norm", {"mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm("norm1"),
                                         "ffn_norm": None if feed_forward is None else norm("norm2"),
                                         "input_conv": input_conv, "token_input": token_input, "names": BLOCK_NAMES})
        layers.append(LayerSpec(f"l{index}", block))
    return ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": config.width, "tensor": "embed",
                                               "scale": config.embedding_scale}),
        embedding_prefix="",
        layers=tuple(layers),
        final_norm=norm("norm"),
        final_norm_prefix="final",
        head=PartSpec("lm_head", {"vocab_size": config.vocab, "hidden_size": config.width, "tied": False, "tensor": "head",
                                  "scale": config.logit_scale}),
        head_prefix="",
        cache_from=cache_from,
        vocab_size=config.vocab,
    )


register_architecture(MetitarConfig.architecture, MetitarConfig, metitar_plan, replace=True)
