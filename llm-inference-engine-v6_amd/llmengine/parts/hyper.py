"""A layer around a residual that is kept as several streams (hyper-connections; Zhu et al.,
"Hyper-Connections", 2024): x [S, T, H] instead of [T, H].

Sublayer q (the mixer, then the feed-forward) with its three small tensors in_q [S], out_q [S] and
mix_q [S, S] (indexed [from, to]):

    u = sum_s in_q[s] x_s;   y = sublayer(norm_q(u));   x_t <- sum_s mix_q[s, t] x_s + out_q[t] y

all streams at once from the old ones. The model starts every stream as the embedding and reads
their plain sum at the end. Sums and norms are 32-bit.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Block, FeedForward, Getter, Mixer, Norm, ParamSpec, Placement
from .registry import register_part


class HyperConnectionBlock(Block):
    graph_safe = True

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, ffn_norm: Norm | None,
                 streams: int, names: dict | None = None):
        if not 1 <= int(streams) <= ops.recurrent.MAX_STREAMS:
            raise ValueError(f"hyper-connections: 1 to {ops.recurrent.MAX_STREAMS} streams, got {streams}")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.ffn_norm = mixer_norm, ffn_norm
        self.streams = int(streams)
        self.names = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "feed_forward": "mlp",
                      "mixer_streams": "hc1", "ffn_streams": "hc2"}
        if names:
            self.names.update(names)
        self.coef: dict = {}
        # the block that runs behind this one when the model runs its layers in order (set by whoever composes the model;
        # None: unknown, the blocks then do not hand their inputs on)
        self.next_block = None

    def _subs(self):
        n = self.names
        out = [(n["mixer_streams"], self.mixer_norm, self.mixer)]
        if self.feed_forward is not None:
            out.append((n["ffn_streams"], self.ffn_norm, self.feed_forward))
        return out

    def children(self):
        n = self.names
        out = {n["mixer_norm"]: self.mixer_norm, n["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out.update({n["ffn_norm"]: self.ffn_norm, n["feed_forward"]: self.feed_forward})
        return out

    def param_specs(self):
        S = self.streams
        out = {}
        for prefix, _, _ in self._subs():
            out.update({f"{prefix}.in": ParamSpec((S,), "norm"), f"{prefix}.out": ParamSpec((S,), "norm"),
                        f"{prefix}.mix": ParamSpec((S, S), "identity")})
        return out

    def load_params(self, get: Getter, placement: Placement) -> None:
        for prefix, _, _ in self._subs():
            self.coef[prefix] = tuple(placement.place(get(f"{prefix}.{k}"), torch.float32) for k in ("in", "out", "mix"))

    def first_read(self):
        """(stream weights, norm weight, eps) of this block's first sublayer where its norm is the plain RMS formula, so that
        the block in front can make this block's first input in the kernel that stores its own last result; else None."""
        rms = self.mixer_norm.fused_rms()
        return None if rms is None else (self.coef[self.names["mixer_streams"]][0], rms[0], rms[1])

    def forward(self, h, step, cache, write_cache=True):
        S, T, H = h.shape
        x = step.buffer("block.normed", (T, H), step.act_dtype)
        y = step.buffer("block.sublayer", (T, H), torch.float32)
        subs = self._subs()
        # the block in front may have left this block's first input in x (see below)
        ready = step.extra.pop("block.normed is for", None) == id(self)
        for k, (prefix, norm, sub) in enumerate(subs):
            c_in, c_out, c_mix = self.coef[prefix]
            if not ready:
                rms = norm.fused_rms()
                if rms is not None:
                    ops.streams_read_norm(h, c_in, rms[0], rms[1], x)
                else:
                    u = step.buffer("block.mixed", (T, H), torch.float32)
                    ops.streams_read_norm(h, c_in, None, 0.0, u)
                    norm.forward(u, x)
            ready = False
            if sub is self.mixer:
                sub.forward(x, step, cache, y, False, write_cache)
            else:
                sub.forward(x, step, y, False)
            # what reads the streams next: this block's next sublayer, or the first sublayer of the block behind
            if k + 1 < len(subs):
                nxt_rms = subs[k + 1][1].fused_rms()
                nxt = None if nxt_rms is None else (self.coef[subs[k + 1][0]][0], nxt_rms[0], nxt_rms[1])
                owner = None
            else:
                behind = self.next_block
                nxt = behind.first_read() if isinstance(behind, HyperConnectionBlock) and behind.streams == S else None
                owner = behind
            if nxt is not None:
                # the streams' update and the next read of them in one pass over the rows
                ops.streams_write_read_norm(h, c_mix, c_out, y, nxt[0], nxt[1], nxt[2], x)
                if owner is not None:
                    step.extra["block.normed is for"] = id(owner)
                else:
                    ready = True
            else:
                ops.streams_write(h, c_mix, c_out, y)


register_part("block", "hyper", HyperConnectionBlock)
