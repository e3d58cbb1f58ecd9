"""The recurrent block around a real-gated linear recurrent unit (RG-LRU; De et al., "Griffin: Mixing
Gated Linear Recurrences with Local Attention for Efficient Language Models", 2024).

Two branches of `width` channels read the input x: gate = gelu_tanh(Wy x + by) and
u = conv(Wx x + bx), a short causal convolution per channel with a bias and no activation. The
channels are cut into `blocks` equal parts with two square maps each:
r = sigmoid(Ra u + ba), i = sigmoid(Ri u + bi). With a = exp(-rate * r * softplus(lam)), rate = 8:
s_t = a s_(t-1) + sqrt(1 - a^2) (i u), from s = 0 (the first token is no special case). The
mixer's result is Wo (s * gate).

Kept per request: s (32-bit) and the convolution's last taps - 1 inputs. Gates, decay and the
recurrence are 32-bit.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import CacheSpec, Getter, ParamSpec, Placement
from .projected import ProjectedMixer
from .registry import register_part


class RGLRU(ProjectedMixer):
    RATE = 8.0

    def __init__(self, hidden_size: int, width: int, blocks: int, conv_taps: int):
        if width % blocks:
            raise ValueError(f"rglru: {width} channels do not divide into {blocks} blocks")
        self.hidden_size, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(conv_taps)
        self.out_width = self.width

    def input_names(self):
        return [("y", self.width), ("x", self.width)]

    def output_name(self):
        return "o"

    def param_specs(self):
        W, H, B = self.width, self.hidden_size, self.blocks
        bw = W // B
        return {"y": ParamSpec((W, H)), "y.b": ParamSpec((W,)), "x": ParamSpec((W, H)), "x.b": ParamSpec((W,)),
                "conv": ParamSpec((W, self.taps), "taps"), "conv.b": ParamSpec((W,)),
                "ra": ParamSpec((B, bw, bw)), "ra.b": ParamSpec((B, bw)), "ri": ParamSpec((B, bw, bw)),
                "ri.b": ParamSpec((B, bw)), "lam": ParamSpec((W,)), "o": ParamSpec((H, W))}

    def refusals(self):
        if not 1 <= self.taps <= ops.recurrent.MAX_TAPS:
            return [f"conv={self.taps}: the convolution kernel takes 1 to {ops.recurrent.MAX_TAPS} taps"]
        return []

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(state={"s": ((self.width,), torch.float32),
                                "conv": ((max(self.taps - 1, 0), self.width), torch.float32)})

    def load_core(self, get: Getter, placement: Placement) -> None:
        f32 = torch.float32
        self.y_bias = placement.place(get("y.b"), f32)
        # (the x branch's bias goes through the convolution with the values: the convolution kernel adds it to its input)
        self.x_bias = placement.place(get("x.b"), f32)
        self.conv_w = placement.place(get("conv"), f32)
        self.conv_b = placement.place(get("conv.b"), f32)
        self.ra, self.ri = placement.place(get("ra")), placement.place(get("ri"))
        if self.ra.dtype != self.ri.dtype:
            self.ra, self.ri = self.ra.float(), self.ri.float()
        self.ra_b = placement.place(get("ra.b"), f32).view(-1)
        self.ri_b = placement.place(get("ri.b"), f32).view(-1)
        self.lam = placement.place(get("lam"), f32)

    def core(self, p, step, cache, o, scale=1.0):
        if scale != 1.0:
            raise NotImplementedError("rglru: no scale on the result")
        T, W = p.shape[0], self.width
        y, x = p[:, :W], p[:, W:2 * W]
        u = step.buffer("rglru.u", (T, W), torch.float32)
        ops.short_conv(x, self.conv_w, self.conv_b, cache.state["conv"], step, u, silu=False, in_bias=self.x_bias)
        decay = step.buffer("rglru.decay", (T, W), torch.float32)
        drive = step.buffer("rglru.drive", (T, W), torch.float32)
        ops.rglru_gates(u, self.ra, self.ra_b, self.ri, self.ri_b, self.lam, self.RATE, decay, drive)
        ops.rglru_scan(decay, drive, y, self.y_bias, cache.state["s"], step, o)


register_part("mixer", "rglru", RGLRU)
