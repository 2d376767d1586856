"""Small Metitar configurations for the tests, with seeded random weights, and what the tests share."""

from __future__ import annotations

import os

import torch

from somi_inference_amd.config import (MetitarConfig, MetitarDense, MetitarExperts, MetitarHGRN2, MetitarLatentAttention,
                                       MetitarLayer, RampedScaling)


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, dims=None, scaling=None, kv_from=None, mlp=None):
    return MetitarLayer("latent_attention", MetitarLatentAttention(
        heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale, rot_base=base,
        rot_dims=rot_dim if dims is None else dims, rot_scaling=scaling, kv_from=kv_from), mlp)


def hgrn2(heads, dim, vdim, mlp=None):
    return MetitarLayer("hgrn2", MetitarHGRN2(heads=heads, dim=dim, vdim=vdim), mlp)


# A: both mixers twice, a lender and a borrower with other heads and sizes, frequencies on a ramp, three taps, two
#    experts a token beside a shared one, a layer without a feed-forward, a token input, scaled embedding and logits.
# B: no input convolution, no token input, scales of one, no frequency scaling, one expert a token, no shared expert,
#    one recurrent head, pages of 8 tokens, a borrower right after its lender.
# C: a width that is no multiple of 8 and odd sizes everywhere, one tap (a convolution that only scales), fewer rotated
#    channels than the shared key part has, every expert chosen, five heads.
# D: a latent wider than a workgroup of the plain kernel, large recurrent heads, five taps, a ramp whose ends fall
#    outside the channels, only attention layers after the first.
METITAR = {
    "A": dict(block_size=16, seed=15, config=MetitarConfig(
        vocab=211, width=96, norm_eps=1e-5, embedding_scale=4.0, logit_scale=0.5, token_side_dim=8, canon_taps=3, layers=(
            latent(4, 16, 16, 24, 32, 40, 0.2, base=5000.0, scaling=RampedScaling(4.0, 64, 16.0, 2.0), mlp=MetitarDense(80)),
            hgrn2(3, 16, 24, MetitarExperts(experts=8, top=2, ff=32, shared_ff=48)),
            latent(2, 24, 16, 16, 32, 24, 0.25, base=5000.0, scaling=RampedScaling(4.0, 64, 16.0, 2.0), kv_from=0,
                   mlp=MetitarExperts(experts=6, top=3, ff=24, shared_ff=16)),
            hgrn2(2, 32, 16, None),
        ))),
    "B": dict(block_size=8, seed=16, config=MetitarConfig(
        vocab=130, width=72, norm_eps=1e-6, embedding_scale=1.0, logit_scale=1.0, token_side_dim=None, canon_taps=None, layers=(
            hgrn2(1, 24, 40, MetitarDense(56)),
            latent(3, 24, 4, 8, 16, 32, 0.3, base=100.0, mlp=MetitarExperts(experts=5, top=1, ff=40)),
            latent(6, 8, 4, 16, 16, 8, 0.5, base=100.0, kv_from=1, mlp=None),
        ))),
    "C": dict(block_size=8, seed=17, config=MetitarConfig(
        vocab=97, width=100, norm_eps=1e-6, embedding_scale=9.0, logit_scale=2.5, token_side_dim=5, canon_taps=1, layers=(
            latent(5, 12, 6, 20, 28, 20, 0.35, base=300.0, dims=2, mlp=MetitarExperts(experts=3, top=3, ff=24, shared_ff=8)),
            hgrn2(5, 12, 20, MetitarDense(36)),
        ))),
    "D": dict(block_size=16, seed=18, config=MetitarConfig(
        vocab=77, width=104, norm_eps=1e-5, embedding_scale=2.5, logit_scale=1.5, token_side_dim=7, canon_taps=5, layers=(
            hgrn2(1, 128, 64, MetitarExperts(experts=4, top=2, ff=16)),
            latent(2, 64, 32, 48, 160, 72, 0.1, base=1000.0, scaling=RampedScaling(8.0, 16, 64.0, 0.01), mlp=MetitarDense(40)),
            latent(3, 32, 32, 32, 160, 16, 0.12, base=1000.0, scaling=RampedScaling(8.0, 16, 64.0, 0.01), kv_from=1,
                   mlp=MetitarDense(24)),
        ))),
}


def write_metitar(name: str, folder: str, peaky: bool = False) -> str:
    """The model folder of configuration ``name``.  Matrices of the feed-forwards and of the token input are widened
    (random weights this small would leave them without a say), routers so that they decide something, the embedding so
    that tokens differ.  ``peaky``: the queries' and the latent's projections are widened further, so that attention
    scores spread over several units and single keys stand out."""
    from safetensors.torch import load_file, save_file

    from somi_inference_amd.weights import write_random_model
    write_random_model(folder, METITAR[name]["config"], seed=METITAR[name]["seed"])
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key, tensor in list(tensors.items()):
        factor = 1.0
        if tensor.dim() == 2 and (".mlp." in key or ".side." in key or key == "side.embed") and not key.endswith(".router"):
            factor = 8.0
        if key.endswith(".router"):
            factor = 60.0
        if key == "embed":
            factor = 20.0
        if tensor.dim() == 2 and ".mix." in key:
            factor = 4.0
        if peaky and (key.endswith(".mix.uq") or key.endswith(".mix.uk")):
            factor = 24.0
        if factor != 1.0:
            tensors[key] = (tensor.float() * factor).to(tensor.dtype)
    save_file(tensors, path)
    return folder


def load_plain(folder: str, dtype=torch.float32):
    from plain import metitar_plain
    return metitar_plain.load_folder(folder, dtype)
