"""The Gizilorn decoder as a plan: pre-norm layers around several residual streams (hyper-connections); the mixer is
grouped-query attention with mixed heads (capped scores, a window, a softmax whose denominator holds an extra 1, values
rotated by their position) or attention over a shared low-rank latent (a window, a sigmoid gate on the heads' outputs;
a layer may read the latent an earlier layer kept); a dense feed-forward whose activation has two stored numbers;
RMS-normed embedded rows and an untied head.

Tensor names: ``embed``, ``embed.norm``, ``final.norm``, ``head``, and per layer ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.<name>`` (biases ``<name>.b``), ``l<i>.mlp.{up,down,act}`` (biases ``.b``), ``l<i>.hc1.{in,out,mix}`` and
``l<i>.hc2.{in,out,mix}``; no name carries a ``.weight`` suffix.
"""

from __future__ import annotations

from ..config.gizilorn import GizilornConfig
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .plan import LayerSpec, ModelPlan

BLOCK_NAMES = {"mixer_norm": "", "mixer": "mix", "ffn_norm": "", "feed_forward": "mlp", "mixer_streams": "hc1",
               "ffn_streams": "hc2"}


def gizilorn_plan(config: GizilornConfig) -> ModelPlan:
    def norm(tensor: str) -> PartSpec:
        return PartSpec("rmsnorm", {"hidden_size": config.width, "eps": config.norm_eps, "tensor": tensor})

    # a layer that lends its kept latent keeps a token's row for as long as the farthest-seeing reader needs it
    kept_for: dict[int, int | None] = {}
    for index, layer in enumerate(config.layers):
        if layer.type != "latent_attention":
            continue
        owner = index if layer.mixer.kv_from is None else layer.mixer.kv_from
        window = layer.mixer.window
        if owner not in kept_for:
            kept_for[owner] = window
        elif kept_for[owner] is not None:
            kept_for[owner] = None if window is None else max(kept_for[owner], window)

    layers, cache_from = [], {}
    for index, layer in enumerate(config.layers):
        m = layer.mixer
        if layer.type == "latent_attention":
            position = (PartSpec("rotary", {"head_dim": m.rot_dim, "theta": m.rot_base, "rotary_dim": m.rot_dims,
                                            "pairing": "neighbours"})
                        if m.rot_dims > 0 else PartSpec("none", {}))
            mixer = PartSpec("latent_attention", {
                "hidden_size": config.width, "num_heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "value_dim": m.vdim,
                "kv_rank": m.kv_rank, "q_rank": None, "scale": m.scale, "eps": config.norm_eps, "position": position,
                "shares_cache": m.kv_from is not None, "suffix": "", "sink": False, "window": m.window,
                "kept_window": kept_for[index] if m.kv_from is None else m.window, "gate": True})
            if m.kv_from is not None:
                cache_from[index] = m.kv_from
        else:
            position = (PartSpec("rotary", {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims,
                                            "pairing": "half"})
                        if m.rot_dims > 0 else PartSpec("none", {}))
            mixer = PartSpec("mixed_heads_attention", {
                "hidden_size": config.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "dim": m.dim,
                "value_dim": m.vdim, "position": position, "scale": m.scale, "softcap": m.softcap, "window": m.window,
                "sink_one": True, "head_mix": True, "value_rotation": {"theta": m.rot_base, "pairing": "half"},
                "qkv_bias": True, "suffix": "", "bias_suffix": "b"})
        feed_forward = None
        if layer.mlp is not None:
            feed_forward = PartSpec("activated", {"hidden_size": config.width, "intermediate_size": layer.mlp.ff,
                                                  "activation": "xielu", "bias": True, "suffix": "", "bias_suffix": "b"})
        block = PartSpec("hyper_connections", {
            "mixer": mixer, "feed_forward": feed_forward, "mixer_norm": norm("norm1"),
            "ffn_norm": None if feed_forward is None else norm("norm2"), "streams": config.streams or 1,
            "connections": config.streams is not None, "names": BLOCK_NAMES})
        layers.append(LayerSpec(f"l{index}", block))
    return ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab, "hidden_size": config.width, "tensor": "embed",
                                               "norm_tensor": "embed.norm", "norm_eps": config.norm_eps}),
        embedding_prefix="",
        layers=tuple(layers),
        final_norm=norm("norm"),
        final_norm_prefix="final",
        head=PartSpec("lm_head", {"vocab_size": config.vocab, "hidden_size": config.width, "tied": False, "tensor": "head"}),
        head_prefix="",
        cache_from=cache_from,
        vocab_size=config.vocab,
    )


register_architecture(GizilornConfig.architecture, GizilornConfig, gizilorn_plan, replace=True)
