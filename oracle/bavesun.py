"""Plain, slow CPU implementation of the Bavesun design: one function per mechanism, float64 by default.

It is the oracle the GPU kernels are tested against and shares no code with ``lit_gpt``. It takes the raw
``config.json`` dictionary and a ``{name: tensor}`` dictionary of weights, and walks a sequence token by token
wherever the design is recurrent or causal, so that nothing here depends on a chunking, a cache layout or a batch.

Notation: ``W`` model width, ``H`` heads, ``d`` key dim, ``dv`` value dim, ``r`` latent rank, ``dr`` rotated dims.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_offset(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight sits around zero: unit * (1 + w)."""
    return rms_unit(x, eps) * (1.0 + w)


def norm_plain(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def rope_angles(pos: int, dims: int, base: float) -> torch.Tensor:
    i = torch.arange(dims // 2, dtype=DT)
    return pos * base ** (-2.0 * i / dims)


def rope_half(x: torch.Tensor, pos: int, dims: int, base: float) -> torch.Tensor:
    """Rotate the first ``dims`` entries of a vector, entry i paired with entry i + dims/2."""
    a = rope_angles(pos, dims, base)
    u, v = x[: dims // 2], x[dims // 2: dims]
    out = x.clone()
    out[: dims // 2] = u * torch.cos(a) - v * torch.sin(a)
    out[dims // 2: dims] = v * torch.cos(a) + u * torch.sin(a)
    return out


def rope_interleaved(x: torch.Tensor, pos: int, dims: int, base: float) -> torch.Tensor:
    """Rotate the first ``dims`` entries of a vector, entry 2i paired with entry 2i + 1."""
    a = rope_angles(pos, dims, base)
    u, v = x[0:dims:2], x[1:dims:2]
    out = x.clone()
    out[0:dims:2] = u * torch.cos(a) - v * torch.sin(a)
    out[1:dims:2] = v * torch.cos(a) + u * torch.sin(a)
    return out


def retention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Decayed linear attention, one token after the other. h: (T, W) -> (T, W)."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    g = h @ w["g"].T
    out = torch.zeros(T, H, dv, dtype=DT)
    for hd in range(H):
        S = torch.zeros(d, dv, dtype=DT)
        lam = float(m["decay"][hd])
        for t in range(T):
            qt = rope_half(q[t, hd], t, rot["dims"], rot["base"])
            kt = rope_half(k[t, hd], t, rot["dims"], rot["base"]) * d ** -0.5
            S = lam * S + torch.outer(kt, v[t, hd])
            out[t, hd] = rms_unit(S.T @ qt, eps)
    gated = out.reshape(T, H * dv) * (g * torch.sigmoid(g))
    return gated @ w["o"].T


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Softmax attention over keys and values expanded from a low-rank latent, with a keyless sink."""
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, H, d + dr)
    dkv = h @ w["dkv"].T
    c = norm_plain(dkv[:, :r], w["dkv.norm"], eps)
    kr = torch.stack([rope_interleaved(dkv[t, r:], t, rot["dims"], rot["base"]) for t in range(T)])
    kn = (c @ w["uk"].T).view(T, H, d)
    val = (c @ w["uv"].T).view(T, H, dv)
    g = h @ w["g"].T
    out = torch.zeros(T, H, dv, dtype=DT)
    for t in range(T):
        for hd in range(H):
            qn = q[t, hd, :d]
            qr = rope_interleaved(q[t, hd, d:], t, rot["dims"], rot["base"])
            s = (kn[: t + 1, hd] @ qn + kr[: t + 1] @ qr) * m["scale"]
            sink = w["sink"][hd]
            mx = torch.maximum(s.max(), sink)
            e = torch.exp(s - mx)
            out[t, hd] = (e[:, None] * val[: t + 1, hd]).sum(0) / (e.sum() + torch.exp(sink - mx))
    gated = out.reshape(T, H * dv) * torch.sigmoid(g)
    return gated @ w["o"].T


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], spec: dict) -> torch.Tensor:
    """Top-k experts by router logit, weights = softmax over the chosen logits, expert = down(relu(up h)^2)."""
    E, top = spec["router"]["experts"], spec["router"]["top"]
    z = h @ w["router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        p = torch.softmax(torch.stack([z[t, e] for e in order]), 0)
        for pe, e in zip(p, order):
            a = torch.relu(w[f"e{e}.up"] @ h[t]) ** 2
            out[t] += pe * (w[f"e{e}.down"] @ a)
    return out


def token_side(x: torch.Tensor, tokens: torch.Tensor, layer: int, side_embed: torch.Tensor, w: Dict[str, torch.Tensor],
               dim: int, eps: float) -> torch.Tensor:
    """Per-layer token input: a gated slice of a second embedding table, projected, unit-normed and weighted."""
    e = side_embed[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return x + norm_plain(y, w["norm"], eps)


def _sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(DT) for k, v in weights.items() if k.startswith(prefix)}


def layer_order(cfg: dict) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int],
            residuals: Optional[list] = None) -> torch.Tensor:
    """Logits (T, vocab) of one whole sequence; ``residuals`` collects the stream after every layer run."""
    eps = cfg["norm"]["eps"]
    tok = torch.tensor(tokens, dtype=torch.long)
    embed = weights["embed"].to(DT)
    x = embed[tok] * cfg["embedding"]["scale"]
    for i in layer_order(cfg):
        spec = cfg["layers"][i]
        h = norm_offset(x, weights[f"l{i}.norm1"].to(DT), eps)
        mix = _sub(weights, f"l{i}.mix.")
        if spec["type"] == "retention":
            y = retention(h, mix, spec["mixer"], eps)
        elif spec["type"] == "latent_attention":
            y = latent_attention(h, mix, spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        ff = spec.get("mlp")
        if ff is not None:
            mw = _sub(weights, f"l{i}.mlp.")
            y = y + (dense_ff(h, mw) if ff["kind"] == "dense" else moe_ff(h, mw, ff))
        x = x + y
        if cfg.get("token_side") and f"l{i}.side.gate" in weights:
            x = token_side(x, tok, i, weights["side.embed"].to(DT), _sub(weights, f"l{i}.side."),
                           cfg["token_side"]["dim"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    x = norm_offset(x, weights["final.norm"].to(DT), eps)
    return x @ embed.T
