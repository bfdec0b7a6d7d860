"""A plain, slow implementation of the Suranex design, one function per mechanism, in
float64 on the CPU.  It shares no code with the engine: whole sequences at once, dense
masks, python loops.  Tests compare the engine with it on small random models.

A model is (config dict, {tensor name: torch tensor}); see ``yalis_amd/models/suranex.py``
for the keys of the configuration and the names of the tensors.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w.to(F))


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w.to(F)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def yarn_frequencies(dims, base, scaling):
    """Per-pair angular frequencies and the factor both cos and sin are multiplied with."""
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    if scaling is None:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(t):
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_halves(x, angles, mag=1.0):
    """x [..., T, d]; angles [T, r/2] turn the pairs (i, i + r/2) of the first r = 2 * angles.shape[1]
    elements; the rest passes."""
    half = angles.shape[-1]
    a, b, rest = x[..., :half], x[..., half: 2 * half], x[..., 2 * half:]
    c, s = torch.cos(angles) * mag, torch.sin(angles) * mag
    return torch.cat([a * c - b * s, b * c + a * s, rest], dim=-1)


def visible(T, size, keep_first):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def attention_mixer(h, m, w, pre, eps):
    """h [T, width] -> [T, width]; m the mixer's configuration, w the tensors, pre their prefix."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].to(F).T).view(T, H, d).transpose(0, 1)
    k = (h @ w[pre + "k"].to(F).T).view(T, G, d).transpose(0, 1)
    v = (h @ w[pre + "v"].to(F).T).view(T, G, dv).transpose(0, 1)
    q = norm_plain(q, w[pre + "q.norm"], eps)
    k = norm_plain(k, w[pre + "k.norm"], eps)
    pos = torch.arange(T, dtype=F)
    rot = m["rot"]
    f, mag = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    ang = pos[:, None] * f[None, :]
    q, k = rotate_halves(q, ang, mag), rotate_halves(k, ang, mag)
    v = rms_unit(v, eps)
    fv = rot["base"] ** (-2.0 * torch.arange(dv // 2, dtype=F) / dv)
    vang = pos[:, None] * fv[None, :]
    v = rotate_halves(v, vang)
    mask = m.get("mask") or {}
    mask = visible(T, mask.get("size") or T, mask.get("keep_first", 0))
    out = torch.empty(H, T, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[hh] @ k[g].T) * m["scale"]
        cap = m.get("softcap")
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~mask, -math.inf)
        out[hh] = torch.softmax(s, dim=-1) @ v[g]
    out = rotate_halves(out, -vang)
    gate = torch.sigmoid(h @ w[pre + "g"].to(F).T)  # [T, H]
    out = out * gate.T[:, :, None]
    return out.transpose(0, 1).reshape(T, H * dv) @ w[pre + "o"].to(F).T


def causal_conv(x, taps_w, bias):
    """x [T, C]; taps_w [C, taps], the last column meets the current token; zeros before the start."""
    T, C = x.shape
    taps = taps_w.shape[1]
    out = torch.zeros(T, C, dtype=F)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                out[t] += taps_w[:, j].to(F) * x[src]
        out[t] += bias.to(F)
    return out


def rglru_mixer(h, m, w, pre):
    T = h.shape[0]
    C, B = m["width"], m["blocks"]
    y = gelu_tanh(h @ w[pre + "y"].to(F).T + w[pre + "y.b"].to(F))
    u = causal_conv(h @ w[pre + "x"].to(F).T + w[pre + "x.b"].to(F), w[pre + "conv"], w[pre + "conv.b"])
    ub = u.view(T, B, C // B)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[pre + "ra"].to(F)) + w[pre + "ra.b"].to(F)).reshape(T, C)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[pre + "ri"].to(F)) + w[pre + "ri.b"].to(F)).reshape(T, C)
    log_a = -8.0 * r * torch.nn.functional.softplus(w[pre + "lam"].to(F))
    a = torch.exp(log_a)
    S = torch.zeros(C, dtype=F)
    out = torch.empty(T, C, dtype=F)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out[t] = S
    return (out * y) @ w[pre + "o"].to(F).T


def expert(h, w, pre, limit):
    g = (h @ w[pre + "gate"].to(F).T).clamp(max=limit)
    u = (h @ w[pre + "up"].to(F).T).clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].to(F).T


def table_moe(h, tokens, f, w, pre):
    top = f["router"]["top"]
    table = w[pre + "table"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in table[tokens[t]].tolist():
            out[t] += expert(h[t: t + 1], w, f"{pre}e{e}.", f["expert"]["limit"])[0] / top
    if f.get("shared"):
        out = out + expert(h, w, pre + "shared.", f["shared"]["limit"])
    return out


def forward(config, w, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (float64); with ``return_layers`` also the residual
    stream after every layer [layers, T, width]."""
    eps = config["norm"]["eps"]
    x = w["embed"].to(F)[tokens]
    layers = []
    for n, layer in enumerate(config["layers"]):
        pre = f"l{n}."
        if layer["type"] == "attention":
            a = attention_mixer(x, layer["mixer"], w, pre + "mix.", eps)
        elif layer["type"] == "rglru":
            a = rglru_mixer(x, layer["mixer"], w, pre + "mix.")
        else:
            raise ValueError(layer["type"])
        x = x + norm_one_plus(a, w[pre + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + norm_one_plus(table_moe(x, tokens, layer["mlp"], w, pre + "mlp."), w[pre + "norm2"], eps)
        layers.append(x)
    logits = norm_one_plus(x, w["final.norm"], eps) @ w["head"].to(F).T
    if return_layers:
        return logits, torch.stack(layers)
    return logits
