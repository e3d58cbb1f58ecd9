"""The gated delta rule: a fast-weight memory M [dim, vdim] per head that every token first lets decay,
then corrects towards its value and then reads.

q, k (kv_heads x dim) and v (heads x vdim) are projections of the input without biases; head h uses
q/k head h / (heads / kv_heads). Each passes a short causal convolution per channel (no bias) and
SiLU; q and k then become unit vectors per head, x / sqrt(sum(x^2) + 1e-6), q also times dim^-1/2.
beta = sigmoid(Wb x), one per head. Per head and token, in this order:

    M <- g * M;   w = beta (v - M^T k);   M <- M + k w^T;   o = M^T q

so that the token reads its own write. The decay g is either one number per head,
exp(-exp(A_log) softplus(Wa x + dt_bias)), or one per head and key channel, acting on the rows of M,
exp(-exp(A_log[head]) softplus(Wa2 (Wa1 x) + dt_bias)). Each head's o is divided by its root mean
square over vdim, multiplied by a weight of size vdim that the heads share and by a gate:
silu(Wg x) or sigmoid(Wg2 (Wg1 x)), heads x vdim. Then the output matrix.

Kept per request: M (32-bit) and the last taps - 1 inputs of the three convolutions. Everything
behind the convolutions' activation is 32-bit.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import CacheSpec, Getter, ParamSpec, Placement
from .projected import ProjectedMixer
from .registry import register_part


class GatedDeltaRule(ProjectedMixer):
    UNIT_EPS = 1e-6

    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, conv_taps: int, eps: float,
                 decay: str = "head", gate: str = "silu", decay_rank: int | None = None, gate_rank: int | None = None):
        if heads % kv_heads:
            raise ValueError(f"delta rule: {heads} heads do not divide into {kv_heads} key heads")
        if decay not in ("head", "channel"):
            raise ValueError(f"delta rule: decay {decay!r} is neither 'head' nor 'channel'")
        if gate not in ("silu", "sigmoid_lowrank"):
            raise ValueError(f"delta rule: gate {gate!r} is neither 'silu' nor 'sigmoid_lowrank'")
        self.hidden_size = int(hidden_size)
        self.heads, self.kv_heads, self.dim, self.vdim = int(heads), int(kv_heads), int(dim), int(vdim)
        self.taps, self.eps = int(conv_taps), float(eps)
        self.decay, self.gate = decay, gate
        # ranks of the two-stage maps: named by the configuration, or read off the checkpoint's tensors
        self.decay_rank = int(decay_rank) if decay_rank is not None else None
        self.gate_rank = int(gate_rank) if gate_rank is not None else None
        self.out_width = self.heads * self.vdim
        self.conv_channels = 2 * self.kv_heads * self.dim + self.heads * self.vdim

    # ---- tensors ----
    def _decay_in(self):
        return ("a1", self.decay_rank) if self.decay == "channel" else ("a", self.heads)

    def _gate_in(self):
        return ("g1", self.gate_rank) if self.gate == "sigmoid_lowrank" else ("g", self.heads * self.vdim)

    def input_names(self):
        qk = self.kv_heads * self.dim
        return [("q", qk), ("k", qk), ("v", self.heads * self.vdim), ("b", self.heads), self._decay_in(), self._gate_in()]

    def output_name(self):
        return "o"

    def param_specs(self):
        H, qk, hv = self.hidden_size, self.kv_heads * self.dim, self.heads * self.vdim
        specs = {"q": ParamSpec((qk, H)), "q.conv": ParamSpec((qk, self.taps), "taps"),
                 "k": ParamSpec((qk, H)), "k.conv": ParamSpec((qk, self.taps), "taps"),
                 "v": ParamSpec((hv, H)), "v.conv": ParamSpec((hv, self.taps), "taps"),
                 "b": ParamSpec((self.heads, H)), "A_log": ParamSpec((self.heads,)), "norm": ParamSpec((self.vdim,), "norm"),
                 "o": ParamSpec((H, hv))}
        if self.decay == "channel":
            specs.update({"a1": ParamSpec((self.decay_rank, H)), "a2": ParamSpec((self.heads * self.dim, self.decay_rank)),
                          "dt_bias": ParamSpec((self.heads * self.dim,))})
        else:
            specs.update({"a": ParamSpec((self.heads, H)), "dt_bias": ParamSpec((self.heads,))})
        if self.gate == "sigmoid_lowrank":
            specs.update({"g1": ParamSpec((self.gate_rank, H)), "g2": ParamSpec((hv, self.gate_rank))})
        else:
            specs["g"] = ParamSpec((hv, H))
        return specs

    def refusals(self):
        out = []
        if not 1 <= self.taps <= ops.recurrent.MAX_TAPS:
            out.append(f"conv={self.taps}: the convolution kernel takes 1 to {ops.recurrent.MAX_TAPS} taps")
        if self.dim > ops.recurrent.DELTA_MAX_DIM:
            out.append(f"dim={self.dim}: the delta-rule kernel takes key sizes up to {ops.recurrent.DELTA_MAX_DIM}")
        return out

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(state={"memory": ((self.heads, self.vdim, self.dim), torch.float32),
                                "conv": ((max(self.taps - 1, 0), self.conv_channels), torch.float32)})

    def load_core(self, get: Getter, placement: Placement) -> None:
        f32 = torch.float32
        self.conv_w = placement.place(torch.cat([get("q.conv").float(), get("k.conv").float(), get("v.conv").float()]), f32)
        self.A_log = placement.place(get("A_log"), f32)
        self.dt_bias = placement.place(get("dt_bias"), f32)
        self.norm_w = placement.place(get("norm"), f32)
        self.a2 = self.g2 = None
        if self.decay == "channel":
            a1, a2 = get("a1"), get("a2")
            if a1.shape[0] != a2.shape[1]:
                raise ValueError(f"delta rule: a1 {tuple(a1.shape)} and a2 {tuple(a2.shape)} disagree on the rank")
            self.decay_rank = int(a1.shape[0])
            self.a2 = placement.place(a2)
        if self.gate == "sigmoid_lowrank":
            g1, g2 = get("g1"), get("g2")
            if g1.shape[0] != g2.shape[1]:
                raise ValueError(f"delta rule: g1 {tuple(g1.shape)} and g2 {tuple(g2.shape)} disagree on the rank")
            self.gate_rank = int(g1.shape[0])
            self.g2 = placement.place(g2)

    def core(self, p, step, cache, o, scale=1.0):
        T = p.shape[0]
        C, heads, kvh, dim, vdim = self.conv_channels, self.heads, self.kv_heads, self.dim, self.vdim
        at = C
        b_in = p[:, at:at + heads]
        at += heads
        n_a = self._decay_in()[1]
        a_in = p[:, at:at + n_a]
        at += n_a
        g_in = p[:, at:at + self._gate_in()[1]]
        qkv = step.buffer("delta.qkv", (T, C), torch.float32)
        ops.short_conv(p[:, :C], self.conv_w, None, cache.state["conv"], step, qkv, silu=True)
        ops.unit_heads(qkv[:, :2 * kvh * dim], kvh, kvh, dim, float(dim) ** -0.5, 1.0, self.UNIT_EPS)
        beta = step.buffer("delta.beta", (T, heads), torch.float32)
        n_dec = heads * dim if self.decay == "channel" else heads
        decay = step.buffer("delta.decay", (T, n_dec), torch.float32)
        if self.a2 is not None:
            # the second stage of the two-stage map as a product of its own, its 32-bit input made contiguous first
            low = step.buffer("delta.decay_low", (T, self.decay_rank), torch.float32)
            ops.copy_cols(a_in, low)
            a_in = step.buffer("delta.decay_in", (T, n_dec), torch.float32)
            ops.gemm(low, self.a2, a_in, choices=step.choices)
        ops.delta_gates(b_in, a_in, None, self.A_log, self.dt_bias, beta, decay, heads, dim)
        read = step.buffer("delta.read", (T, heads * vdim), torch.float32)
        ops.delta_rule(qkv, beta, decay, cache.state["memory"], step, read, heads, kvh, dim, vdim,
                       per_channel=self.decay == "channel")
        if self.g2 is not None:
            low = step.buffer("delta.gate_low", (T, self.gate_rank), torch.float32)
            ops.copy_cols(g_in, low)
            g_in = step.buffer("delta.gate_in", (T, heads * vdim), torch.float32)
            ops.gemm(low, self.g2, g_in, choices=step.choices)
        ops.gated_head_norm(read, self.norm_w, g_in, None, o, heads, vdim, self.eps, scale,
                            activation="sigmoid" if self.gate == "sigmoid_lowrank" else "silu")


register_part("mixer", "gated_delta", GatedDeltaRule)
