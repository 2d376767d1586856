"""Plain Metitar decoder: one slow function per mechanism, whole sequences at a time.

Written from the design's equations; it shares no code with the engine.  ``weights`` maps tensor names to
tensors of one floating type (float32, or float64 for a sharper yardstick), ``config`` is the parsed config.json.
Notation: ``x`` the residual stream ``[T, width]``, ``h`` a sublayer's input, ``i`` a query's position and ``j`` a
key's.
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


def layer_norm(y: torch.Tensor, weights: dict, name: str, eps: float) -> torch.Tensor:
    """(y - mean) / sqrt(var + eps) * w + b with the variance as the mean of squared deviations."""
    mean = y.mean(dim=-1, keepdim=True)
    var = (y - mean).pow(2).mean(dim=-1, keepdim=True)
    return (y - mean) / torch.sqrt(var + eps) * weights[name] + weights[name + ".b"]


# ------------------------------------------------------------------------------------- input convolution
def input_convolution(h: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """h + conv(h): conv(h)[t, c] = sum_j taps[c, j] h[t - (n - 1) + j, c], zeros before the sequence's start."""
    tokens, n = h.shape[0], taps.shape[1]
    out = h.clone()
    for t in range(tokens):
        for j in range(n):
            src = t - (n - 1) + j
            if src >= 0:
                out[t] = out[t] + taps[:, j] * h[src]
    return out


# ------------------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict, dtype=torch.float64) -> tuple[torch.Tensor, float]:
    """The dims / 2 frequencies and the factor on cos and sin, with the wavelength-dependent rescaling if present."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    mult = 1.0
    scaling = rot.get("scaling")
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def where(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(where(float(scaling["fast"]))), 0)
        hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
        ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)],
                            dtype=torch.float64)
        f = f / factor * ramp + f * (1.0 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    return f.to(dtype), mult


def rotate(v: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """v: [T, ..., D]; the first rot.dims channels turn, channel i with i + dims / 2."""
    dims = int(rot["dims"])
    f, mult = rotary_frequencies(rot, torch.float64)
    angle = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = (torch.cos(angle) * mult).to(v.dtype), (torch.sin(angle) * mult).to(v.dtype)
    while cos.dim() < v.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    a, b = v[..., :dims // 2], v[..., dims // 2:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, v[..., dims:]], dim=-1)


# ------------------------------------------------------------------------------------- latent attention
def latent_keys(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float) -> tuple[torch.Tensor, torch.Tensor]:
    """What a latent-attention layer caches: the normed latent c [T, kv_rank] and the rotated shared key part
    [T, rot_dim]."""
    rank = mixer["kv_rank"]
    down = h @ weights[prefix + ".dkv"].T
    c = rms(down[:, :rank], eps) * weights[prefix + ".dkv.norm"]
    shared = rotate(down[:, rank:], torch.arange(h.shape[0]), mixer["rot"])
    return c, shared


def latent_attention(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float,
                     kept: tuple[torch.Tensor, torch.Tensor]) -> torch.Tensor:
    """Causal softmax attention with a sink, keys and values expanded from the latent ``kept`` = (c, shared rotated key
    part), which may be another layer's."""
    heads, dim, rot_dim, vdim = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"]
    tokens = h.shape[0]
    c, shared = kept
    cq = rms(h @ weights[prefix + ".dq"].T, eps) * weights[prefix + ".dq.norm"]
    q = (cq @ weights[prefix + ".uq"].T).view(tokens, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], rotate(q[..., dim:], torch.arange(tokens), mixer["rot"])
    k_plain = (c @ weights[prefix + ".uk"].T).view(tokens, heads, dim)
    v = (c @ weights[prefix + ".uv"].T).view(tokens, heads, vdim)
    sink = weights[prefix + ".sink"]
    out = torch.zeros(tokens, heads, vdim, dtype=h.dtype)
    for i in range(tokens):
        for a in range(heads):
            s = (k_plain[:i + 1, a] @ q_plain[i, a] + shared[:i + 1] @ q_turned[i, a]) * mixer["scale"]
            top = torch.maximum(s.max(), sink[a])
            e = torch.exp(s - top)
            out[i, a] = (e / (e.sum() + torch.exp(sink[a] - top))) @ v[:i + 1, a]
    return out.reshape(tokens, heads * vdim) @ weights[prefix + ".o"].T


# ------------------------------------------------------------------------------------- HGRN2
def hgrn2(h: torch.Tensor, weights: dict, prefix: str, mixer: dict, eps: float) -> torch.Tensor:
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t per head; f bounded below by a learned vector."""
    heads, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    tokens = h.shape[0]
    q = silu(h @ weights[prefix + ".q"].T).view(tokens, heads, dim)
    v = (h @ weights[prefix + ".v"].T).view(tokens, heads, vdim)
    lower = weights[prefix + ".lower"]
    f = (lower + (1.0 - lower) * torch.sigmoid(h @ weights[prefix + ".f"].T + weights[prefix + ".f.b"])).view(tokens, heads, dim)
    state = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    out = torch.zeros(tokens, heads, vdim, dtype=h.dtype)
    for t in range(tokens):
        state = f[t, :, :, None] * state + (1.0 - f[t])[:, :, None] * v[t, :, None, :]
        out[t] = torch.einsum("hkv,hk->hv", state, q[t])
    out = rms(out, eps) * weights[prefix + ".norm"]
    return out.reshape(tokens, heads * vdim) @ weights[prefix + ".o"].T


# ------------------------------------------------------------------------------------- feed-forwards
def poly_norm_ff(h: torch.Tensor, weights: dict, prefix: str, eps: float) -> torch.Tensor:
    """W_down (a N(z) + b N(z^2) + c N(z^3) + e) with z = W_up h and N the division by a row's root mean square."""
    z = h @ weights[prefix + ".up"].T
    a, b, c, e = weights[prefix + ".act"]
    return (a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e) @ weights[prefix + ".down"].T


def gated_unit(h: torch.Tensor, weights: dict, prefix: str) -> torch.Tensor:
    return (silu(h @ weights[prefix + ".gate"].T) * (h @ weights[prefix + ".up"].T)) @ weights[prefix + ".down"].T


def routing(h: torch.Tensor, weights: dict, prefix: str, mlp: dict) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(chosen experts [T, top], their weights [T, top], margin [T]): sigmoid scores, the ``top`` largest, weights are
    the scores as they are.  ``margin`` is how far the last chosen score is above the best one left out."""
    top = mlp["router"]["top"]
    s = torch.sigmoid(h @ weights[prefix + ".router"].T)
    order = torch.argsort(s, dim=-1, descending=True, stable=True)
    ranked = torch.gather(s, 1, order)
    margin = ranked[:, top - 1] - ranked[:, top] if s.shape[1] > top else torch.full((h.shape[0],), math.inf, dtype=h.dtype)
    return order[:, :top], ranked[:, :top], margin


def routed_experts(h: torch.Tensor, weights: dict, prefix: str, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """sum over the chosen experts of expert(w h): the weight multiplies the expert's input; plus the shared expert.
    ``margins`` collects, per layer, how far each token's choice is from a tie."""
    chosen, weight, margin = routing(h, weights, prefix, mlp)
    if margins is not None:
        margins.append(margin)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weight[t]):
            out[t] = out[t] + gated_unit((w * h[t])[None, :], weights, f"{prefix}.e{e}")[0]
    if mlp.get("shared"):
        out = out + gated_unit(h, weights, prefix + ".shared")
    return out


# ------------------------------------------------------------------------------------- token input
def token_input(x: torch.Tensor, tokens: torch.Tensor, weights: dict, index: int, dim: int, eps: float) -> torch.Tensor:
    e = weights["side.embed"][tokens][:, index * dim:(index + 1) * dim]
    y = (gelu_tanh(x @ weights[f"l{index}.side.gate"].T) * e) @ weights[f"l{index}.side.proj"].T
    return rms(y, eps) * weights[f"l{index}.side.norm"]


# ------------------------------------------------------------------------------------- the model
def forward(tokens, weights: dict, config: dict, want_layers: bool = False, margins: list | None = None):
    """Logits [T, vocab] of one whole sequence; with ``want_layers`` also the residual stream after every layer."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = config["norm"]["eps"]
    x = weights["embed"][tokens] * config.get("embedding", {}).get("scale", 1.0)
    side = config.get("token_side")
    canon = config.get("canon")
    kept: dict[int, tuple] = {}
    after = []
    for index, layer in enumerate(config["layers"]):
        p, mixer = f"l{index}", layer["mixer"]
        h = input_convolution(x, weights[p + ".canon1"]) if canon else x
        if layer["type"] == "latent_attention":
            source = mixer.get("kv_from")
            if source is None:
                kept[index] = latent_keys(h, weights, p + ".mix", mixer, eps)
                source = index
            y = latent_attention(h, weights, p + ".mix", mixer, eps, kept[source])
        elif layer["type"] == "hgrn2":
            y = hgrn2(h, weights, p + ".mix", mixer, eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + layer_norm(y, weights, p + ".norm1", eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = poly_norm_ff(x, weights, p + ".mlp", eps)
            else:
                y = routed_experts(x, weights, p + ".mlp", mlp, margins)
            x = x + layer_norm(y, weights, p + ".norm2", eps)
        if side:
            x = x + token_input(x, tokens, weights, index, side["dim"], eps)
        after.append(x.clone())
    logits = (layer_norm(x, weights, "final.norm", eps) @ weights["head"].T) * config.get("logit_scale", 1.0)
    return (logits, torch.stack(after)) if want_layers else logits


def load_folder(folder: str, dtype=torch.float32):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: (t.to(dtype) if t.is_floating_point() else t)
               for name, t in load_file(os.path.join(folder, "model.safetensors")).items()}
    return weights, config
