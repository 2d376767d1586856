"""Plain Gizilorn decoder: one slow function per mechanism, whole sequences at a time.

Written from the design's equations; it shares no code with the engine.  ``weights`` maps tensor names to
tensors of one floating type (float32, or float64 for a sharper yardstick), ``config`` is the parsed config.json.
Notation: ``x`` a stream ``[T, width]``, ``h`` a sublayer's input, ``i`` a query's position and ``j`` a key's.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


# ------------------------------------------------------------------------------------- rotation
def turn(v: torch.Tensor, positions: torch.Tensor, dims: int, base: float, layout: str, sign: float = 1.0) -> torch.Tensor:
    """v: [T, ..., D]; the first ``dims`` channels turn by ``sign * position * base^(-2 m / dims)``, pair m being
    (m, m + dims/2) in the ``halves`` layout and (2m, 2m + 1) in the ``interleaved`` one."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * m / dims) for m in range(half)], dtype=torch.float64)
    angle = sign * positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = torch.cos(angle).to(v.dtype), torch.sin(angle).to(v.dtype)
    while cos.dim() < v.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    out = v.clone()
    if layout == "halves":
        a, b = v[..., :half], v[..., half:dims]
        out[..., :half] = a * cos - b * sin
        out[..., half:dims] = b * cos + a * sin
    elif layout == "interleaved":
        a, b = v[..., 0:dims:2], v[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    else:
        raise ValueError(layout)
    return out


def visible(tokens: int, window: int | None) -> torch.Tensor:
    """[i, j] true where i sees j: j <= i and, with a window, i - j < window."""
    i = torch.arange(tokens)[:, None]
    j = torch.arange(tokens)[None, :]
    see = j <= i
    if window is not None:
        see = see & (i - j < window)
    return see


# ------------------------------------------------------------------------------------- attention with mixed heads
def attention(h: torch.Tensor, weights: dict, prefix: str, m: dict) -> torch.Tensor:
    """Grouped-query attention: biased q/k/v, partial rotation of q and k, values turned by their own position and
    the head's sum turned back by the query's, capped scores, a window, a softmax whose denominator has one added,
    and the heads' weights mixed by a matrix before they meet the values."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    rot = m["rot"]
    pos = torch.arange(T)
    q = (h @ weights[prefix + "q"].T + weights[prefix + "q.b"]).view(T, H, D)
    k = (h @ weights[prefix + "k"].T + weights[prefix + "k.b"]).view(T, G, D)
    v = (h @ weights[prefix + "v"].T + weights[prefix + "v.b"]).view(T, G, Dv)
    q = turn(q, pos, int(rot["dims"]), float(rot["base"]), "halves")
    k = turn(k, pos, int(rot["dims"]), float(rot["base"]), "halves")
    v = turn(v, pos, Dv, float(rot["base"]), "halves")
    see = visible(T, m["mask"]["size"] if m.get("mask") else None)
    cap = m.get("softcap")
    probs = torch.zeros(H, T, T, dtype=h.dtype)
    for a in range(H):
        s = (q[:, a] @ k[:, a // (H // G)].T) * float(m["scale"])
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        s = s.masked_fill(~see, float("-inf"))
        top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=0.0)
        e = torch.exp(s - top)
        probs[a] = e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))
    mixed = torch.einsum("ag,gij->aij", weights[prefix + "talk"], probs)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for a in range(H):
        out[:, a] = mixed[a] @ v[:, a // (H // G)]
    out = turn(out, pos, Dv, float(rot["base"]), "halves", sign=-1.0)
    return out.reshape(T, H * Dv) @ weights[prefix + "o"].T


# ------------------------------------------------------------------------------------- latent attention
def latent_of(h: torch.Tensor, weights: dict, prefix: str, m: dict, eps: float) -> tuple[torch.Tensor, torch.Tensor]:
    """What a layer keeps per token: the normed latent c [T, rank] and the turned shared key part r [T, rot_dim]."""
    rank, R = int(m["kv_rank"]), int(m["rot_dim"])
    d = h @ weights[prefix + "dkv"].T
    c = rms(d[:, :rank], eps) * weights[prefix + "dkv.norm"]
    r = turn(d[:, rank:rank + R], torch.arange(h.shape[0]), R, float(m["rot"]["base"]), "interleaved")
    return c, r


def latent_attention(h: torch.Tensor, weights: dict, prefix: str, m: dict, kept: tuple[torch.Tensor, torch.Tensor]) -> torch.Tensor:
    """Attention whose keys and values are per-head linear maps of the kept latent, plus one turned key part all
    heads share; a window, an ordinary softmax, a sigmoid gate on the concatenated heads."""
    T = h.shape[0]
    H, D, R, Dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    c, r = kept
    q = (h @ weights[prefix + "q"].T).view(T, H, D + R)
    q_plain = q[..., :D]
    q_turned = turn(q[..., D:].contiguous(), torch.arange(T), R, float(m["rot"]["base"]), "interleaved")
    keys = (c @ weights[prefix + "uk"].T).view(T, H, D)
    values = (c @ weights[prefix + "uv"].T).view(T, H, Dv)
    see = visible(T, m["mask"]["size"] if m.get("mask") else None)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for a in range(H):
        s = (q_plain[:, a] @ keys[:, a].T + q_turned[:, a] @ r.T) * float(m["scale"])
        s = s.masked_fill(~see, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ values[:, a]
    gate = torch.sigmoid(h @ weights[prefix + "g"].T)
    return (out.reshape(T, H * Dv) * gate) @ weights[prefix + "o"].T


# ------------------------------------------------------------------------------------- feed-forward
def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    p, q = softplus(pq[0]), softplus(pq[1])
    zn = torch.clamp(z, max=0.0)
    return torch.where(z > 0, p * z * z + 0.5 * z, (0.5 + q) * (torch.expm1(zn) - zn) + 0.5 * z)


def dense(h: torch.Tensor, weights: dict, prefix: str) -> torch.Tensor:
    z = h @ weights[prefix + "up"].T + weights[prefix + "up.b"]
    return xielu(z, weights[prefix + "act"]) @ weights[prefix + "down"].T + weights[prefix + "down.b"]


# ------------------------------------------------------------------------------------- the streams
def read_streams(streams: torch.Tensor, weights: dict, prefix: str) -> torch.Tensor:
    """u = sum_s in[s] x_s; streams: [S, T, width]."""
    return torch.einsum("s,stw->tw", weights[prefix + "in"], streams)


def write_streams(streams: torch.Tensor, y: torch.Tensor, weights: dict, prefix: str) -> torch.Tensor:
    """x_t <- sum_s mix[s, t] x_s + out[t] y, every new stream from the old ones."""
    return torch.einsum("st,sxw->txw", weights[prefix + "mix"], streams) + weights[prefix + "out"][:, None, None] * y[None]


# ------------------------------------------------------------------------------------- the model
def forward(config: dict, weights: dict, tokens: list[int], dtype=torch.float64) -> tuple[torch.Tensor, torch.Tensor]:
    """Logits [T, vocab] and the summed streams after every layer [layers, T, width]."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    S = int(config.get("streams") or 1)
    x = rms(w["embed"][torch.tensor(tokens)], eps) * w["embed.norm"]
    hyper = "l0.hc1.in" in w
    streams = x[None].repeat(S, 1, 1)
    kept: dict[int, tuple[torch.Tensor, torch.Tensor]] = {}
    after = []
    for n, layer in enumerate(config["layers"]):
        p, m = f"l{n}.", layer["mixer"]
        for sub in (1, 2):
            if sub == 2 and not layer.get("mlp"):
                continue
            u = read_streams(streams, w, f"{p}hc{sub}.") if hyper else streams[0]
            h = rms(u, eps) * w[f"{p}norm{sub}"]
            if sub == 2:
                y = dense(h, w, p + "mlp.")
            elif layer["type"] == "attention":
                y = attention(h, w, p + "mix.", m)
            elif layer["type"] == "latent_attention":
                if m.get("kv_from") is None:
                    kept[n] = latent_of(h, w, p + "mix.", m, eps)
                    mine = kept[n]
                else:
                    mine = kept[int(m["kv_from"])]
                y = latent_attention(h, w, p + "mix.", m, mine)
            else:
                raise ValueError(layer["type"])
            streams = write_streams(streams, y, w, f"{p}hc{sub}.") if hyper else streams + y[None]
        after.append(streams.sum(dim=0))
    x = rms(streams.sum(dim=0), eps) * w["final.norm"]
    return x @ w["head"].T, torch.stack(after)


def load_folder(folder: str, dtype=torch.float32) -> tuple[dict, dict]:
    """(weights, config) of a model folder, floating tensors in ``dtype``."""
    import json
    import os

    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {k: (v.to(dtype) if v.is_floating_point() else v)
               for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return weights, config
