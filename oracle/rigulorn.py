"""Plain, slow CPU implementation of the Rigulorn design: one function per mechanism, float64 by default.

It is the oracle the GPU kernels are tested against and shares no code with ``lit_gpt``. It takes the raw
``config.json`` dictionary and a ``{name: tensor}`` dictionary of weights and walks a sequence token by token
wherever the design is recurrent or causal, so that nothing here depends on a chunking, a cache layout or a batch.

The design in short. The residual is kept in ``s`` parallel streams (hyper-connections): a sublayer reads a fixed
weighted sum of the streams, and its output is written back into every stream while the streams are mixed by a
small matrix. Layers are pre-norm (RMS norm with a plain weight): a sequence mixer, then an optional feed-forward.
Two mixers: *differential attention* (two softmax maps per head over the same values, the second subtracted with a
learned factor; grouped key/value heads; rotary positions on interleaved pairs; tanh soft-capped scores; a causal
mask confined to aligned chunks of positions; optional reuse of an earlier layer's keys and values) and a *Mamba-2*
selective state-space layer (short causal convolution, per-head scalar decay, grouped B / C, gated grouped norm).

Notation: ``W`` width, ``H`` heads, ``G`` key/value heads or groups, ``d`` key dim of one map, ``dv`` value dim,
``N`` state size.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

DT = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rope_interleaved(x: torch.Tensor, pos: int, dims: int, base: float) -> torch.Tensor:
    """Rotate the first ``dims`` entries of a vector, entry 2i paired with entry 2i + 1; the others are copied."""
    if dims == 0:
        return x.clone()
    i = torch.arange(dims // 2, dtype=x.dtype)
    a = pos * base ** (-2.0 * i / dims)
    u, v = x[0:dims:2], x[1:dims:2]
    out = x.clone()
    out[0:dims:2] = u * torch.cos(a) - v * torch.sin(a)
    out[1:dims:2] = v * torch.cos(a) + u * torch.sin(a)
    return out


def visible(i: int, j: int, mask: Optional[dict]) -> bool:
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    if mask and mask.get("size"):
        return i // int(mask["size"]) == j // int(mask["size"])
    return True


def attention_keys_values(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rotated keys (T, G, 2, d) and values (T, G, dv) of a layer that owns its projections."""
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    k = (h @ w["k"].T).view(T, G, 2, d)
    v = (h @ w["v"].T).view(T, G, dv)
    kr = torch.empty_like(k)
    for t in range(T):
        for g in range(G):
            for a in range(2):
                kr[t, g, a] = rope_interleaved(k[t, g, a], t, rot["dims"], rot["base"])
    return kr, v


def diff_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float,
                   kv: Tuple[torch.Tensor, torch.Tensor]) -> torch.Tensor:
    """Differential attention over the given keys and values, one query after the other. h: (T, W) -> (T, W)."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    keys, vals = kv
    q = (h @ w["q"].T).view(T, H, 2, d)
    lam = (math.exp(float((w["lq1"] * w["lk1"]).sum())) - math.exp(float((w["lq2"] * w["lk2"]).sum()))
           + float(m["diff"]))
    cap = m.get("softcap")
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        js = [j for j in range(t + 1) if visible(t, j, m.get("mask"))]
        for hd in range(H):
            g = hd // (H // G)
            maps = []
            for a in range(2):
                qt = rope_interleaved(q[t, hd, a], t, rot["dims"], rot["base"])
                s = (keys[js, g, a] @ qt) * float(m["scale"])
                if cap:
                    s = float(cap) * torch.tanh(s / float(cap))
                maps.append(torch.softmax(s, 0) @ vals[js, g])
            o = maps[0] - lam * maps[1]
            out[t, hd] = rms_unit(o, eps) * (1.0 - float(m["diff"]))
    return out.reshape(T, H * dv) @ w["o"].T


def causal_conv(u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """Per-channel causal convolution of u (T, C) with weight (C, taps): column taps - 1 weights the token itself,
    column 0 the oldest input."""
    T, C = u.shape
    taps = weight.shape[1]
    out = torch.zeros_like(u)
    for t in range(T):
        acc = bias.clone()
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                acc = acc + weight[:, j] * u[src]
        out[t] = acc
    return out


def mamba2(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Selective state-space layer, one token after the other. h: (T, W) -> (T, W)."""
    Hh, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = Hh * dv
    T = h.shape[0]
    proj = h @ w["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].view(T, Hh, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w["dt_bias"])
    decay = torch.exp(-torch.exp(w["A_log"]) * dt)  # (T, heads)
    y = torch.zeros(T, Hh, dv, dtype=h.dtype)
    for hd in range(Hh):
        g = hd // (Hh // G)
        S = torch.zeros(N, dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hd] * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + w["D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    parts = int(m.get("norm_groups", 1))
    y = rms_unit(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], f: dict) -> torch.Tensor:
    """Clamped gated unit: g = min(W_gate h, L), u = clamp(W_up h, -L, L); W_down (g sigmoid(1.702 g) (u + 1))."""
    lim = float(f["limit"])
    g = torch.clamp(h @ w["gate"].T, max=lim)
    u = torch.clamp(h @ w["up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def _sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=DT, layers_out: Optional[list] = None
            ) -> torch.Tensor:
    """Logits (T, vocab) of one sequence. ``layers_out``: a list that receives the sum of the streams after each layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    s = int(config.get("streams", 1))
    x0 = w["embed"][torch.tensor(tokens)] * float((config.get("embedding") or {}).get("scale", 1.0))
    xs = [x0.clone() for _ in range(s)]
    kv_of: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}

    def sublayer(xs, lw, q, fn):
        if s == 1 and f"hc{q}.in" not in lw:
            return [xs[0] + fn(norm_plain(xs[0], lw[f"norm{q}"], eps))]
        a, b, mix = lw[f"hc{q}.in"], lw[f"hc{q}.out"], lw[f"hc{q}.mix"]
        u = sum(a[i] * xs[i] for i in range(s))
        y = fn(norm_plain(u, lw[f"norm{q}"], eps))
        return [sum(mix[i, t] * xs[i] for i in range(s)) + b[t] * y for t in range(s)]

    for i, layer in enumerate(config["layers"]):
        lw, m = _sub(w, f"l{i}."), layer["mixer"]
        mw = _sub(lw, "mix.")
        if layer["type"] == "attention":
            def mixer(hh, i=i, m=m, mw=mw):
                if "kv_from" in m and m["kv_from"] is not None:
                    kv = kv_of[int(m["kv_from"])]
                else:
                    kv = kv_of[i] = attention_keys_values(hh, mw, m)
                return diff_attention(hh, mw, m, eps, kv)
        elif layer["type"] == "mamba2":
            def mixer(hh, m=m, mw=mw):
                return mamba2(hh, mw, m, eps)
        else:
            raise ValueError(layer["type"])
        xs = sublayer(xs, lw, 1, mixer)
        if layer.get("mlp") is not None:
            xs = sublayer(xs, lw, 2, lambda hh, lw=lw, f=layer["mlp"]: feed_forward(hh, _sub(lw, "mlp."), f))
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = norm_plain(sum(xs), w["final.norm"], eps)
    return x @ w["head"].T
