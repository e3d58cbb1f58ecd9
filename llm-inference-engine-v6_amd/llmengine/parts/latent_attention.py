"""Attention whose keys and values are expanded from a latent vector per token, over the paged cache.

The layer's input x goes down to a query latent (q_rank entries, RMS-normed with a plain weight) and up to
the heads' queries, each [dim unrotated | rot_dim rotated] entries. It also goes down to kv_rank + rot_dim
entries: the first kv_rank, RMS-normed, are the latent c; the last rot_dim, rotated at the token's position,
are a key part that every head shares. Head h's key is [Wuk_h c | shared part], its value Wuv_h c; scores are
scale * q . k over the keys the token may see (all earlier ones, or the last `window`), weights their softmax;
the heads' results side by side go through the output matrix.

Only c and the shared part are cached: a page holds rows of kv_rank + rot_dim entries. The kernels never
expand a key or a value either: a query takes Wuk_h^T onto itself and is scored against the rows as they
lie, the weighted sum runs over the rows' latent part, and Wuv_h is applied to that sum. A layer with
`keeps_latent=False` has no down map for keys and values and reads the rows another layer cached (if those
rows carry a rotated part and this layer has none, its queries score the latent entries alone).

Rotation: neighbours (2i, 2i + 1) of a part's first `dims` entries turn by position * f_i, with
f_i = base^(-2i / dims) and, where `scaling` is given, the frequencies blended towards f_i / factor over a ramp
of pairs (from the pair that makes `fast` turns over `original` positions to the one that makes `slow`) and cos
and sin times 0.1 ln(factor) + 1. Angles are 32-bit products in the kernels; the frequencies are made here in
64-bit and stored in 32-bit.
"""
from __future__ import annotations

import math

import torch

from .. import ops
from .base import PAGE, CacheSpec, Getter, Mixer, ParamSpec, Placement
from .projected import stack_rows
from .registry import register_part


def ramped_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """([dims / 2] float64 angular steps, the factor on cos and sin)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp_(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, heads: int, dim: int, vdim: int, kv_rank: int, q_rank: int, scale: float,
                 eps: float, rot_dim: int = 0, rot: dict | None = None, window: int = 0, keeps_latent: bool = True,
                 cache_window: int | None = None):
        if rot_dim % 2:
            raise ValueError(f"rot_dim {rot_dim} must be even")
        if rot_dim and not rot:
            raise ValueError("a rotated part needs the rotation's constants")
        self.hidden_size = int(hidden_size)
        self.heads, self.dim, self.rot_dim, self.vdim = int(heads), int(dim), int(rot_dim), int(vdim)
        self.kv_rank, self.q_rank = int(kv_rank), int(q_rank)
        self.scale, self.eps, self.window = float(scale), float(eps), int(window)
        self.keeps_latent = bool(keeps_latent)
        # how many of the last rows the cache keeps: the layer's window, or more where another layer reads further back
        self.cache_window = self.window if cache_window is None else int(cache_window)
        self.rot = dict(rot) if rot_dim else None
        self.rot_dims = int(self.rot["dims"]) if self.rot else 0
        if self.rot_dims % 2 or self.rot_dims > self.rot_dim:
            raise ValueError(f"rotated dims {self.rot_dims} must be even and at most rot_dim {self.rot_dim}")
        self.mag = 1.0
        self.freq: torch.Tensor | None = None

    @property
    def row(self) -> int:
        return self.kv_rank + self.rot_dim

    def param_specs(self):
        H, n = self.hidden_size, self.heads
        out = {"dq": ParamSpec((self.q_rank, H)), "dq.norm": ParamSpec((self.q_rank,), "norm"),
               "uq": ParamSpec((n * (self.dim + self.rot_dim), self.q_rank)),
               "uk": ParamSpec((n * self.dim, self.kv_rank)), "uv": ParamSpec((n * self.vdim, self.kv_rank)),
               "o": ParamSpec((H, n * self.vdim))}
        if self.keeps_latent:
            out.update({"dkv": ParamSpec((self.row, H)), "dkv.norm": ParamSpec((self.kv_rank,), "norm")})
        return out

    def refusals(self):
        if not ops.latent_attention_fits(self.kv_rank, self.rot_dim):
            return [f"kv_rank={self.kv_rank}, rot_dim={self.rot_dim}: the latent attention kernels take latents up to "
                    f"{ops.latent.LATENT_MAX_RANK} and cached rows up to {ops.latent.LATENT_MAX_ROW}"]
        return []

    def cache_spec(self) -> CacheSpec | None:
        if not self.keeps_latent:
            return None
        return CacheSpec(kind="window" if self.cache_window > 0 else "full", window=self.cache_window,
                         paged={"rows": (PAGE, self.row)})

    def load_params(self, get: Getter, placement: Placement) -> None:
        n, d, dv, R = self.heads, self.dim, self.vdim, self.kv_rank
        downs = [get("dq")] + ([get("dkv")] if self.keeps_latent else [])
        self.w_down, self.down_padded = stack_rows(downs, placement)
        self.q_norm = placement.place(get("dq.norm"))
        self.c_norm = placement.place(get("dkv.norm"), self.q_norm.dtype) if self.keeps_latent else None
        self.w_uq = placement.place_matrix(get("uq"))
        # per head: the key map transposed [kv_rank, dim] (it is applied to the query), the value map [vdim, kv_rank]
        uk = placement.place(get("uk"))
        self.w_uk_t = uk.view(n, d, R).transpose(1, 2).contiguous()
        self.w_uv = placement.place(get("uv")).view(n, dv, R).contiguous()
        self.w_o = placement.place_matrix(get("o"))
        if self.rot_dims:
            f, self.mag = ramped_frequencies(self.rot_dims, float(self.rot["base"]), self.rot.get("scaling"))
            self.freq = placement.place(f.to(torch.float32), torch.float32)

    def forward(self, x, step, cache, out, accumulate, write_cache=True):
        if bool(write_cache) != self.keeps_latent:
            raise NotImplementedError("a latent attention layer writes its own rows, or reads another layer's: "
                                      "the schedule and the layer disagree")
        T = x.shape[0]
        n, d, r, dv, R, Rq = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank, self.q_rank
        D, act = R + r, step.act_dtype
        rows = cache.paged["rows"]
        # A layer without rotated entries may read rows that hold some (the layer that cached them rotates): its queries
        # have zeros there, so that the rows are scored as they lie.
        pad = rows.shape[2] - D
        if pad and (pad < 0 or r or self.keeps_latent):
            raise ValueError(f"the cached rows hold {rows.shape[2]} entries, this layer reads {D}")
        D += pad
        table = step.block_tables[cache.group]
        p = step.buffer("latent.down", (T, self.down_padded), torch.float32)
        ops.gemm(x, self.w_down, p, choices=step.choices)
        cq = step.buffer("latent.cq", (T, Rq), act)
        ops.latent_prepare(p, Rq, R if write_cache else 0, r, self.rot_dims, self.q_norm, self.c_norm, self.freq, self.mag,
                           step, table, cq, rows, self.eps)
        q = step.buffer("latent.q", (T, n * (d + r)), act)
        ops.gemm(cq, self.w_uq, q, choices=step.choices)
        ol = step.buffer("latent.sum", (T, n * R), act)
        fast = ops.latent.latent_mfma_fits(rows, R, r + pad, step.choices) and act == torch.bfloat16
        if (fast and d % 8 == 0 and ops.latent.heads_gemm_fits(q, self.w_uk_t, step.choices)
                and ops.latent.heads_gemm_fits(ol, self.w_uv, step.choices)):
            # everything between the up map and the output map with the heads outermost ([heads, T, ..]): the two maps
            # that differ from head to head are then products of whole row tiles on the matrix cores
            qn = step.buffer("latent.qn", (n, T, d), act)
            qr = step.buffer("latent.qr", (n, T, r + pad), act) if r + pad else None
            if pad:
                ops.latent.zero_(qr)
            ops.latent.latent_q_split(q, self.freq, self.mag, step.positions, qn, qr if r else None, n, d, r, self.rot_dims)
            qa = step.buffer("latent.qa", (n, T, R), act)
            ops.latent.heads_gemm(qn, self.w_uk_t, qa)
            ol = ol.view(n, T, R)
            ops.latent.latent_attention_mfma(qa, qr, rows, ol, step, table, n, R, self.scale, self.window, head_major=True)
            oh = step.buffer("latent.oh", (n, T, dv), act)
            ops.latent.heads_gemm(ol, self.w_uv, oh)
            o = step.buffer("latent.o", (T, n * dv), act)
            ops.latent.heads_to_rows(oh, o)
            ops.gemm(o, self.w_o, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)
            return
        if fast:
            qa = step.buffer("latent.qa", (T, n * R), act)
            ops.head_gemm(q, d + r, self.w_uk_t, qa, R, n, choices=step.choices)
            qr = step.buffer("latent.qr", (T, n * (r + pad)), act) if r + pad else None
            if pad:
                ops.latent.zero_(qr)
            if r:
                ops.latent_q_rotate(q, self.freq, self.mag, step.positions, qr, n, d, r, self.rot_dims, 0)
            ops.latent.latent_attention_mfma(qa, qr, rows, ol, step, table, n, R, self.scale, self.window, head_major=False)
        else:
            qp = step.buffer("latent.qp", (T, n * D), act)
            if pad:
                ops.latent.zero_(qp)
            ops.head_gemm(q, d + r, self.w_uk_t, qp, D, n, choices=step.choices)
            if r:
                ops.latent_q_rotate(q, self.freq, self.mag, step.positions, qp, n, d, r, self.rot_dims, R)
            ops.latent_attention(qp, rows, ol, step, table, n, R, self.scale, self.window)
        o = step.buffer("latent.o", (T, n * dv), act)
        ops.head_gemm(ol, R, self.w_uv, o, dv, n, choices=step.choices)
        ops.gemm(o, self.w_o, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)


register_part("mixer", "latent_attention", LatentAttention)
