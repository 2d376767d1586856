"""Small Gizilorn configurations for the tests, their model folders, and the harness that runs one part of the
engine (with the engine's cache manager and step layout) against a plain function."""

import os

import torch

from somi_inference_amd.config import (GizilornAttention, GizilornConfig, GizilornDense, GizilornLatentAttention,
                                       GizilornLayer)


def attention(heads, kv, dim, vdim, window, cap, rot_dims, base=10000.0, scale=None, mlp=None):
    return GizilornLayer("attention", GizilornAttention(heads=heads, kv_heads=kv, dim=dim, vdim=vdim,
                                                        scale=scale if scale is not None else dim ** -0.5, rot_base=base,
                                                        rot_dims=rot_dims, softcap=cap, window=window), mlp)


def latent(heads, dim, rot_dim, vdim, rank, window, base=10000.0, scale=None, kv_from=None, mlp=None):
    return GizilornLayer("latent_attention", GizilornLatentAttention(
        heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank,
        scale=scale if scale is not None else (dim + rot_dim) ** -0.5, rot_base=base, rot_dims=rot_dim, window=window,
        kv_from=kv_from), mlp)


# A: three streams; a latent layer whose reader sees further back than itself; partial rotation; value size unlike the
#    key size; a layer without a feed-forward; an attention layer without window and cap, one key/value head a query head.
# B: ONE stream that still has connection tensors; attention first; a window shorter than a page; one key/value head
#    for all query heads; a latent of a multiple of 16 channels without a window.
# C: no connection tensors at all (the plain residual sum); a latent layer read by two later layers.
# D: four streams; windows longer than the kernels' key tiles (64 and 128) and than several pages.
GIZILORN = {
    "A": dict(seed=11, block_size=8, config=GizilornConfig(vocab=301, width=96, norm_eps=1e-6, streams=3, layers=(
        latent(4, 16, 8, 24, 40, 20, base=5000.0, mlp=GizilornDense(64)),
        latent(4, 16, 8, 24, 40, 33, base=5000.0, kv_from=0, scale=0.3, mlp=None),
        attention(4, 2, 32, 16, 12, 15.0, 16, base=3000.0, mlp=GizilornDense(80)),
        attention(6, 6, 16, 32, None, None, 16, scale=0.2, mlp=GizilornDense(48)),
    ))),
    "B": dict(seed=12, block_size=16, config=GizilornConfig(vocab=130, width=64, norm_eps=1e-5, streams=1, layers=(
        attention(2, 1, 24, 24, 5, 8.0, 24, base=100.0, mlp=GizilornDense(40)),
        latent(3, 32, 16, 16, 48, None, base=250.0, mlp=GizilornDense(72)),
        attention(4, 4, 16, 8, 9, None, 8, mlp=None),
    ))),
    "C": dict(seed=13, block_size=4, config=GizilornConfig(vocab=97, width=80, norm_eps=1e-6, streams=None, layers=(
        latent(2, 8, 4, 8, 24, 7, base=40.0, mlp=GizilornDense(32)),
        attention(3, 3, 8, 12, 3, 4.0, 4, base=7.0, mlp=GizilornDense(56)),
        latent(5, 8, 4, 16, 24, 11, base=40.0, kv_from=0, mlp=GizilornDense(32)),
        latent(1, 24, 4, 8, 24, 2, base=40.0, kv_from=0, mlp=None),
    ))),
    "D": dict(seed=14, block_size=16, config=GizilornConfig(vocab=211, width=72, norm_eps=1e-6, streams=4, layers=(
        attention(4, 2, 16, 16, 70, 25.0, 8, base=800.0, mlp=GizilornDense(64)),
        latent(2, 16, 16, 32, 32, 131, base=1000.0, mlp=GizilornDense(64)),
    ))),
}


def write_gizilorn(name: str, folder: str, peaky: bool = False) -> str:
    """The model folder of configuration ``name``.  Random matrices this small would leave the sublayers without a say
    beside the streams, so the mixers' and feed-forwards' matrices are widened; the heads' mix becomes the identity
    plus what was drawn, so that every head mostly keeps its own weights and still gets some of every other's.
    ``peaky``: queries and keys are widened further, so that attention scores spread over several units and single
    keys stand out."""
    from safetensors.torch import load_file, save_file

    from somi_inference_amd.weights import write_random_model
    write_random_model(folder, GIZILORN[name]["config"], seed=GIZILORN[name]["seed"])
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key, tensor in list(tensors.items()):
        factor = 1.0
        if tensor.dim() == 2 and (".mlp." in key or ".mix." in key) and not key.endswith(".talk"):
            factor = 6.0
        if peaky and key.rsplit(".", 1)[-1] in ("q", "k", "uk"):
            factor = 18.0
        value = tensor.float() * factor
        if key.endswith(".talk"):
            value = value + torch.eye(tensor.shape[0])
        tensors[key] = value.to(tensor.dtype)
    save_file(tensors, path)
    return folder


def load_plain(folder: str, dtype=torch.float32):
    from plain import gizilorn_plain
    return gizilorn_plain.load_folder(folder, dtype)


# ------------------------------------------------------------------------------------------ one part in the engine
def rounded(x: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """float32 values that the dtype holds exactly, so that the kernel and the plain function start from the same."""
    return x.to(dtype).to(torch.float32)


def random_weights(part, seed, scale=None) -> dict:
    """float32 tensors for every tensor the part declares (all hold values bfloat16 has exactly)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for spec in part.weight_specs():
        std = (scale or {}).get(spec.name.rsplit(".", 1)[-1], spec.init.std * (10 if spec.role == "matrix" else 1))
        out[spec.name] = rounded(torch.randn(spec.shape, generator=gen) * std + spec.init.mean)
    return out


def load_part(part, weights: dict, dtype, device):
    """Hand the part its tensors as the loader would: matrices in the compute dtype, vectors in float32."""
    from somi_inference_amd.parts import Runtime
    roles = {spec.name: spec.role for spec in part.weight_specs()}
    assert set(roles) == set(weights), sorted(set(roles) ^ set(weights))
    part.load(lambda name: weights[name].to(dtype if roles[name] == "matrix" else torch.float32).to(device).contiguous(),
              Runtime(dtype, device))
    return part


class PartEngine:
    """The cache manager and the step layout of the engine around some mixers that run one after another on the same
    rows (``borrow``: mixer index -> the earlier mixer whose cache it reads)."""

    def __init__(self, mixers, dtype, device, block_size, num_blocks=64, max_requests=4, borrow=None):
        from somi_inference_amd.cache import CacheManager
        self.mixers, self.dtype, self.device = list(mixers), dtype, device
        needs = [(borrow or {}).get(i, m.cache_spec()) for i, m in enumerate(self.mixers)]
        self.cache = CacheManager(needs, block_size=block_size, num_blocks=num_blocks, max_requests=max_requests,
                                  dtype=dtype, device=device)

    def run(self, portions):
        """One step of (request, its next input rows); for every mixer, its output rows per request."""
        from somi_inference_amd.engine.batch import StepEntry, build_step
        entries = []
        for rid, x in portions:
            if not self.cache.has(rid):
                self.cache.register(rid)
            self.cache.reserve(rid, x.shape[0])
            entries.append(StepEntry(rid, [0] * x.shape[0], []))
        step = build_step(entries, self.cache, self.device, ())
        rows = torch.cat([x for _, x in portions]).to(self.dtype).to(self.device).contiguous()
        outs = []
        for index, mixer in enumerate(self.mixers):
            y = mixer.forward(rows, step, self.cache.layer_caches[index])
            y = y.materialize() if hasattr(y, "materialize") else y
            per, at = [], 0
            for _, x in portions:
                per.append(y[at:at + x.shape[0]].float().cpu())
                at += x.shape[0]
            outs.append(per)
        for rid, x in portions:
            self.cache.commit(rid, x.shape[0])
        return outs

    def run_cut(self, rid, x, sizes):
        """A whole sequence in portions of the given sizes (cycled); every mixer's rows for the sequence."""
        outs, at, i = [[] for _ in self.mixers], 0, 0
        while at < x.shape[0]:
            size = sizes[i % len(sizes)]
            for index, per in enumerate(self.run([(rid, x[at:at + size])])):
                outs[index].append(per[0])
            at += size
            i += 1
        self.cache.free(rid)
        return [torch.cat(o) for o in outs]
