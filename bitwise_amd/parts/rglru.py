"""A recurrent mixer with a real-gated linear recurrent unit: two branches of ``inner`` channels,

    y = gelu_tanh(W_y h + b_y)                                     the gate branch
    u = conv(W_x h + b_x)                                          a causal convolution over `taps` tokens, with a bias
    r = sigmoid(A_b u_b + a_b),  i = sigmoid(I_b u_b + i_b)        per block b of inner / blocks channels
    a = exp(-c r softplus(lambda)),  S <- a S + sqrt(1 - a^2) (i u)   per channel, S = 0 before the first token
    out = W_o (S y)

(the recurrent block of De et al., "Griffin: Mixing Gated Linear Recurrences with Local Attention for Efficient
Language Models").  The state of a request is S and the last taps - 1 inputs of the convolution, 32-bit; gates,
decays, the recurrence and both activations are 32-bit in both modes, and the projections' sums enter them unrounded.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import Mixer, StateSpec, TensorSpec, register_mixer
from .gated_attention import max_seq_rows
from .linear import Linear


@register_mixer("rglru")
class RealGatedLRU(Mixer):
    """params: width, inner, blocks, conv (taps), decay_scale (c; 8 by default).
    tensors: y, x [inner, width] with biases y.b, x.b; conv [inner, taps], conv.b; ra, ri [blocks, bs, bs] ([out, in] per
    block) with ra.b, ri.b [blocks, bs]; lam [inner]; o [width, inner]."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        p = params
        self.width, self.inner, self.blocks, self.taps = int(p["width"]), int(p["inner"]), int(p["blocks"]), int(p["conv"])
        self.decay_scale = float(p.get("decay_scale", 8.0))
        if self.inner % self.blocks:
            raise ValueError(f"rglru: {self.inner} channels do not split into {self.blocks} equal blocks")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"rglru: a convolution over {self.taps} tokens; the kernel takes 1 to {ops.CONV_MAX_TAPS}")
        self.bs = self.inner // self.blocks
        self.proj: Optional[Linear] = None
        self.o: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        R, B, bs = self.inner, self.blocks, self.bs
        return {
            "y": TensorSpec((R, self.width)), "y.b": TensorSpec((R,), "small_bias"),
            "x": TensorSpec((R, self.width)), "x.b": TensorSpec((R,), "small_bias"),
            "conv": TensorSpec((R, self.taps), "conv"), "conv.b": TensorSpec((R,), "small_bias"),
            "ra": TensorSpec((B, bs, bs), "gate_matrix"), "ra.b": TensorSpec((B, bs), "bias"),
            "ri": TensorSpec((B, bs, bs), "gate_matrix"), "ri.b": TensorSpec((B, bs), "bias"),
            "lam": TensorSpec((R,), "bias"),
            "o": TensorSpec((self.width, R)),
        }

    def bind(self, tensors) -> None:
        dev = self.rt.device
        wy, wx = tensors["y"], tensors["x"]
        if wy.dtype != wx.dtype:
            raise ValueError("the projections of one mixer must be stored in one dtype to be stacked")
        self.proj = Linear(torch.cat([wy, wx], dim=0), self.rt)
        # the projections' biases are added where their sums are first read: the convolution's inputs and the gate
        # branch's activation (one 32-bit addition behind the product's sum either way)
        self.y_bias = tensors["y.b"].to(dev).float().contiguous()
        self.x_bias = tensors["x.b"].to(dev).float().contiguous()
        self.o = Linear(tensors["o"], self.rt)
        self.conv_w = tensors["conv"].to(dev).float().contiguous()
        self.conv_b = tensors["conv.b"].to(dev).float().contiguous()
        # per block, input-major: [in][recurrence-gate outputs | input-gate outputs]
        ra, ri = tensors["ra"].to(dev).float(), tensors["ri"].to(dev).float()
        self.gate_w = torch.cat([ra.transpose(1, 2), ri.transpose(1, 2)], dim=2).contiguous()
        self.ra_b = tensors["ra.b"].to(dev).float().reshape(-1).contiguous()
        self.ri_b = tensors["ri.b"].to(dev).float().reshape(-1).contiguous()
        # log a = decay * r with decay = -c softplus(lambda): in double precision, rounded once
        lam = tensors["lam"].to(torch.float64)
        self.decay = (-self.decay_scale * torch.nn.functional.softplus(lam)).to(torch.float32).to(dev).contiguous()

    def weight_bytes(self) -> int:
        small = (self.conv_w.numel() + self.conv_b.numel() + self.gate_w.numel() + 5 * self.inner) * 4
        return self.proj.nbytes() + self.o.nbytes() + small

    def state_spec(self) -> StateSpec:
        return StateSpec((self.taps * self.inner,), "float32")          # [taps - 1][inner] inputs, then S

    def _run(self, ctx, call, h, target, add: bool) -> None:
        ws, rows, R = ctx.ws, ctx.rows, self.inner
        proj = ws.buffer("rglru_proj", 2 * R, torch.float32)
        self.proj.store(ws, h, proj, rows)
        u = ws.buffer("rglru_u", R, torch.float32)
        ops.causal_conv(proj[:, R:], self.conv_w, self.conv_b, call.state, ctx.seq_rows, ctx.slots, ctx.positions, ctx.nseq,
                        max_seq_rows(ctx), u, in_bias=self.x_bias)
        gates = ws.buffer("rglru_gates", 2 * R, torch.float32)
        ops.headwise_linear(u, 0, self.bs, self.gate_w, gates, 0, 2 * self.bs, rows)
        act = ws.buffer("rglru_out", R, self.rt.act_dtype)
        ops.rglru_scan(proj, u, gates, self.ra_b, self.ri_b, self.decay, call.state[:, (self.taps - 1) * R:], act,
                       ctx.seq_rows, ctx.slots, ctx.positions, ctx.nseq, rows, R, self.bs, y_bias=self.y_bias)
        if add:
            self.o.add_into(ws, act, target, rows)
        else:
            self.o.store(ws, act, target, rows)

    def forward(self, ctx, call, h, residual) -> None:
        self._run(ctx, call, h, residual, True)

    def forward_out(self, ctx, call, h, out) -> None:
        self._run(ctx, call, h, out, False)
