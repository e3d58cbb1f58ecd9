"""Causal attention without a softmax, with the heads' scores mixed before the weights are made, over
the paged cache.

q (heads x dim), k (kv_heads x dim) and v (kv_heads x vdim) are projections without biases; query head
h reads key/value head h / (heads / kv_heads). q and k are rotated on their first `rot_dims` entries
(entry i with entry i + rot_dims / 2, by position * base^(-2 i / rot_dims)); k is cached rotated.
score[h, j] = scale q_h . k_j; the scores of all heads for one (query, key) pair are mixed by a matrix
[heads, heads]; a key at or before the query weighs sigmoid(mixed score + a bias per head), and the
weights are not normalised over the keys. Head h's sum of weighted values is multiplied by
sigmoid(Wg x)_h, one number per head, before the output matrix.

Angles, scores, their mixing, the weights and the sums over keys are 32-bit.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import PAGE, CacheSpec, Getter, ParamSpec, Placement
from .projected import ProjectedMixer
from .registry import register_part


class SigmoidAttention(ProjectedMixer):
    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 rot_dims: int = 0, rot_base: float = 10000.0):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads do not divide into {kv_heads} key/value heads")
        if rot_dims % 2 or not 0 <= rot_dims <= dim:
            raise ValueError(f"rot_dims {rot_dims} must be even and at most dim {dim}")
        self.hidden_size = int(hidden_size)
        self.heads, self.kv_heads, self.dim, self.vdim = int(heads), int(kv_heads), int(dim), int(vdim)
        self.scale, self.rot_dims, self.rot_base = float(scale), int(rot_dims), float(rot_base)
        self.out_width = self.heads * self.vdim
        self.inv_freq: torch.Tensor | None = None

    def input_names(self):
        return [("q", self.heads * self.dim), ("k", self.kv_heads * self.dim), ("v", self.kv_heads * self.vdim),
                ("g", self.heads)]

    def output_name(self):
        return "o"

    def param_specs(self):
        H, n = self.hidden_size, self.heads
        return {"q": ParamSpec((n * self.dim, H)), "k": ParamSpec((self.kv_heads * self.dim, H)),
                "v": ParamSpec((self.kv_heads * self.vdim, H)), "talk": ParamSpec((n, n), "identity"),
                "pb": ParamSpec((n,)), "g": ParamSpec((n, H)), "o": ParamSpec((H, n * self.vdim))}

    def refusals(self):
        if not ops.sigmoid_attention_fits(self.heads, self.dim, self.vdim):
            return [f"heads={self.heads}, dim={self.dim}, vdim={self.vdim}: beyond what the attention kernel without "
                    "softmax holds in a workgroup's memory"]
        return []

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(kind="full", paged={"k": (self.kv_heads, PAGE, self.dim), "v": (self.kv_heads, self.vdim, PAGE)})

    def load_core(self, get: Getter, placement: Placement) -> None:
        f32 = torch.float32
        self.talk = placement.place(get("talk"), f32)
        self.talk_t = self.talk.t().contiguous()        # [from, to], as the matrix-core kernel reads it
        self.bias = placement.place(get("pb"), f32)
        if self.rot_dims:
            # frequencies in 64-bit, stored in 32-bit; the angle is the kernel's 32-bit product with the position
            i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
            self.inv_freq = placement.place(torch.pow(torch.tensor(self.rot_base, dtype=torch.float64),
                                                      -2.0 * i / self.rot_dims).to(f32), f32)

    def core(self, p, step, cache, o, scale=1.0):
        T = p.shape[0]
        n, g, dim, vdim = self.heads, self.kv_heads, self.dim, self.vdim
        n_qkv = (n + g) * dim + g * vdim
        table = step.block_tables[cache.group]
        k_cache, v_cache = cache.paged["k"], cache.paged["v"]
        q = step.buffer("sigmoid_attention.q", (T, n * dim), step.act_dtype)
        ops.rotate_write(p[:, :n_qkv], self.inv_freq, step, table, q, k_cache, v_cache, n, g, dim, vdim)
        ops.sigmoid_attention(q, k_cache, v_cache, self.talk, self.bias, p[:, n_qkv:n_qkv + n], step, table, o,
                              n, g, dim, vdim, self.scale, scale, mix_t=self.talk_t)


register_part("mixer", "sigmoid_attention", SigmoidAttention)
