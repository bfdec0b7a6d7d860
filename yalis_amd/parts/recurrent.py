"""A recurrent mixer: the recurrent block of Griffin (De et al., "Griffin: Mixing Gated Linear
Recurrences with Local Attention for Efficient Language Models") with its real-gated linear
recurrent unit.

Two branches of ``width`` channels read the mixer's input h:
    y = gelu_tanh(W_y h + b_y)
    u = conv(W_x h + b_x)          a causal convolution per channel over ``conv_taps`` tokens
and per block b of width / blocks channels
    r = sigmoid(Ra[b] u_b + ba[b]),  i = sigmoid(Ri[b] u_b + bi[b])
    log a = -rate * r * softplus(lam),  S_t = a S_(t-1) + sqrt(1 - a^2) * i * u,  S = 0 before the first token
    out = W_o (S * y).
What a request remembers between steps is a state, not pages: S (float32) and the last
conv_taps - 1 inputs of the convolution; both live in the request's slot and start at zero.
Gates, decays and the recurrence are float32 in both engines.

params: prefix, hidden_size, width, blocks, conv_taps, rate (8.0: the constant in front of
r * softplus(lam)), scan_chunk (64: tokens of a chunk when a long span is scanned in chunks), names
(optional overrides of the tensor names below the prefix).
"""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..engine.batch import chunk_starts, span_chunks
from ..weights.loader import TensorSpec
from .base import Mixer, Runtime, StateNeed, register_mixer


@register_mixer("rglru")
class RecurrentGatedUnit(Mixer):
    graph_capturable = True

    def __init__(self, params, rt: Runtime):
        super().__init__(params, rt)
        self.prefix = params["prefix"]
        self.hidden = int(params["hidden_size"])
        self.width = int(params["width"])
        self.blocks = int(params["blocks"])
        self.taps = int(params["conv_taps"])
        self.rate = float(params.get("rate", 8.0))
        if self.width % self.blocks:
            raise ValueError(f"{self.prefix}: width={self.width} does not divide into {self.blocks} blocks")
        if self.taps < 1:
            raise ValueError(f"{self.prefix}: the convolution needs at least one tap")
        names = {"y": "y", "y_bias": "y.b", "x": "x", "x_bias": "x.b", "conv": "conv", "conv_bias": "conv.b",
                 "ra": "ra", "ra_bias": "ra.b", "ri": "ri", "ri_bias": "ri.b", "lam": "lam", "o": "o"}
        names.update(params.get("names", {}))
        self.names = {k: f"{self.prefix}.{v}" for k, v in names.items()}
        self.w_yx = self.b_yx = self.w_conv = self.b_conv = self.w_o = None
        self.wa_t = self.wi_t = self.ba = self.bi = self.lam = None
        self.wa = self.wi = None
        # long spans are scanned in chunks of this many tokens
        self.chunk = int(params.get("scan_chunk", 64))

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        c, bs, n = self.width, self.width // self.blocks, self.names
        small = ("normal", 0.02)
        return {
            n["y"]: TensorSpec((c, self.hidden)), n["y_bias"]: TensorSpec((c,), "float", small),
            n["x"]: TensorSpec((c, self.hidden)), n["x_bias"]: TensorSpec((c,), "float", small),
            n["conv"]: TensorSpec((c, self.taps), "float", ("normal", 0.3)), n["conv_bias"]: TensorSpec((c,), "float", small),
            n["ra"]: TensorSpec((self.blocks, bs, bs), "float", ("normal", 0.1)), n["ra_bias"]: TensorSpec((self.blocks, bs), "float", small),
            n["ri"]: TensorSpec((self.blocks, bs, bs), "float", ("normal", 0.1)), n["ri_bias"]: TensorSpec((self.blocks, bs), "float", small),
            n["lam"]: TensorSpec((c,), "float", ("normal", 1.0)),
            n["o"]: TensorSpec((self.hidden, c)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.names
        # one product for both branches: rows [y; x]
        self.w_yx = torch.cat([tensors[n["y"]], tensors[n["x"]]], dim=0).contiguous()
        self.b_yx = torch.cat([tensors[n["y_bias"]], tensors[n["x_bias"]]]).contiguous()
        self.w_conv, self.b_conv = tensors[n["conv"]].contiguous(), tensors[n["conv_bias"]].contiguous()
        # gate matrices [block, out, in] are kept [block, in, out]: the kernel's threads, one per output
        # channel, then read consecutive addresses
        self.wa, self.wi = tensors[n["ra"]].contiguous(), tensors[n["ri"]].contiguous()  # (what the matrix-core form reads)
        self.wa_t = self.wa.transpose(1, 2).contiguous()
        self.wi_t = self.wi.transpose(1, 2).contiguous()
        self.ba = tensors[n["ra_bias"]].reshape(-1).contiguous()
        self.bi = tensors[n["ri_bias"]].reshape(-1).contiguous()
        self.lam = tensors[n["lam"]].contiguous()
        self.w_o = tensors[n["o"]]
        same = {t.dtype for t in (self.wa_t, self.wi_t, self.ba, self.bi, self.lam)}
        if len(same) != 1:
            self.wa_t, self.wi_t, self.ba, self.bi, self.lam = (t.float() for t in (self.wa_t, self.wi_t, self.ba, self.bi, self.lam))
        if self.b_conv.dtype != self.w_conv.dtype:
            self.w_conv, self.b_conv = self.w_conv.float(), self.b_conv.float()

    def state_need(self):
        needs = [StateNeed((self.width,), torch.float32, 0.0)]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.width), self.rt.act_dtype, 0.0))
        return tuple(needs)

    def products(self):
        return ((2 * self.width, self.hidden), (self.hidden, self.width))

    def step_inputs(self):
        n = self.chunk
        return {f"span_chunks_{n}": lambda hb: span_chunks(hb, n), f"chunk_starts_{n}": lambda hb: chunk_starts(hb, n)}

    def forward(self, h: torch.Tensor, ctx, site) -> torch.Tensor:
        ops = self.rt.ops
        yx = ops.linear(h, self.w_yx, self.rt.act_dtype, bias=self.b_yx)
        y, x = yx[:, : self.width], yx[:, self.width:]
        conv_state = site.state(1) if self.taps > 1 else None
        u = ops.causal_conv(x, self.w_conv, self.b_conv, conv_state, ctx)
        s = ops.rglru(u, y, x, self.wa_t, self.ba, self.wi_t, self.bi, self.lam, self.rate, site.state(0), conv_state,
                      self.taps, ctx, wa=self.wa, wi=self.wi, chunks=ctx.arrays[f"span_chunks_{self.chunk}"],
                      seq_chunk0=ctx.arrays[f"chunk_starts_{self.chunk}"])
        return ops.linear(s, self.w_o, self.rt.act_dtype, partial_ok=True)
