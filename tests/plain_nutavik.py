"""Nutavik, plainly: whole sequences in float64, dense masks, python loops over tokens for the
convolutions and the recurrences, every head's keys and values made from the latents in full.  One
function per mechanism, written from the design's equations; it shares nothing with the engine
(which never expands keys or values, keeps pages and state slots, and runs ragged batches).

``weights`` maps tensor names to tensors; ``cfg`` is the config.json dictionary.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rotation_tables(rot: dict, n: int):
    """cos and sin [n, dims / 2] with YaRN's ramp and magnitude where ``scaling`` is given."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        where = lambda turns: dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo, hi = max(math.floor(where(sc["fast"])), 0), min(math.ceil(where(sc["slow"])), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / sc["factor"] * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1.0
    angle = torch.arange(n, dtype=F)[:, None] * f[None, :]
    return torch.cos(angle) * mag, torch.sin(angle) * mag


def turn_pairs(x, cos, sin):
    """x [n, ..., dims]: pair (2i, 2i + 1) turned by the angle of position n and pair i."""
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [cos.shape[-1]]
    c, s = cos.view(shape), sin.view(shape)
    u, v = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


def latent_attention(W: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h, latents: dict, layer: int):
    n, H, d, r, vd, rank = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c_q = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (c_q @ W[p + "uq"].T).view(n, H, d + r)
    cos, sin = rotation_tables(m["rot"], n)
    q_plain, q_turned = q[..., :d], turn_pairs(q[..., d:], cos, sin)
    if m.get("kv_from") is not None:
        c, k_turned = latents[m["kv_from"]]
    else:
        both = h @ W[p + "dkv"].T
        c, k_turned = rms_norm(both[:, :rank], W[p + "dkv.norm"], eps), turn_pairs(both[:, rank:], cos, sin)
        latents[layer] = (c, k_turned)
    k = (c @ W[p + "uk"].T).view(n, H, d)
    v = (c @ W[p + "uv"].T).view(n, H, vd)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k) + torch.einsum("ihd,jd->hij", q_turned, k_turned)) * m["scale"]
    visible = torch.tril(torch.ones(n, n, dtype=torch.bool))
    prob = torch.softmax(scores.masked_fill(~visible, -math.inf), dim=-1)
    o = torch.einsum("hij,jhe->ihe", prob, v) * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(n, H * vd) @ W[p + "o"].T


def conv_silu(x, w):
    """Per channel over time, zeros before the start, the last tap on the current token; then silu."""
    n, taps = x.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x])
    y = torch.zeros_like(x)
    for t in range(n):
        for j in range(taps):
            y[t] += padded[t + j] * w[:, j]
    return y * torch.sigmoid(y)


def head_out(W, p, o, h, eps):
    """Each head's read-out over its root mean square, times the shared weight, times silu(W_g h)."""
    n = o.shape[0]
    y = rms_norm(o, W[p + "norm"], eps).reshape(n, -1)
    g = h @ W[p + "g"].T
    return (y * g * torch.sigmoid(g)) @ W[p + "o"].T


def delta(W, p: str, m: dict, eps: float, h):
    n, H, G, d, vd = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).view(n, G, d)
    k = conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).view(n, G, d)
    v = conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).view(n, H, vd)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k = unit(q) * d ** -0.5, unit(k)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    o = torch.zeros(n, H, vd, dtype=F)
    for head in range(H):
        S = torch.zeros(d, vd, dtype=F)
        kh = head // (H // G)
        for t in range(n):
            S = g[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, head] = S.T @ q[t, kh]
    return head_out(W, p, o, h, eps)


def gla(W, p: str, m: dict, eps: float, h):
    n, H, d, vd = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(n, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(n, H, d)
    v = (h @ W[p + "v"].T).view(n, H, vd)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(n, H, d)
    o = torch.zeros(n, H, vd, dtype=F)
    for head in range(H):
        S = torch.zeros(d, vd, dtype=F)
        for t in range(n):
            S = alpha[t, head][:, None] * S + torch.outer(k[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
    return head_out(W, p, o, h, eps)


def dense(W, p: str, h):
    return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: torch.Tensor, streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [tokens, vocab] (float64); ``streams`` collects the residual stream after every layer."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    ln = lambda x, name: layer_norm(x, W[name], W[name + ".b"], eps)
    x = W["embed"][tokens.long()]
    latents: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = ln(x, p + "norm1")
        if layer["type"] == "latent_attention":
            a = latent_attention(W, p + "mix.", layer["mixer"], eps, h, latents, i)
        elif layer["type"] == "delta":
            a = delta(W, p + "mix.", layer["mixer"], eps, h)
        else:
            a = gla(W, p + "mix.", layer["mixer"], eps, h)
        x = x + mult * ln(a, p + "norm1b")
        if layer.get("mlp") is not None:
            x = x + mult * ln(dense(W, p + "mlp.", ln(x, p + "norm2")), p + "norm2b")
        if streams is not None:
            streams.append(x.clone())
    return ln(x, "final.norm") @ W["embed"].T * cfg.get("logit_scale", 1.0)
