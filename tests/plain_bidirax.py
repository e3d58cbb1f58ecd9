"""A plain, slow implementation of the Bidirax design: whole sequences, float64, no cache, no batches,
one function per mechanism. It shares nothing with the engine and is what the engine's results are held
against. Weights come as a dict name -> torch tensor (any float type), the configuration as the dict
that config.json holds.

Notation: T tokens, D the residual width, n heads, d unrotated and r rotated query/key entries per head,
dv value entries per head, L the latent's size.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (the mean of its squares + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    """RMS norm whose weight multiplies as stored."""
    return rms_unit(x, eps) * w.to(F64)


def norm_centered(x, w, eps):
    """RMS norm whose stored weight is the distance from one."""
    return rms_unit(x, eps) * (1.0 + w.to(F64))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def linear(x, w):
    return x @ w.to(F64).T


def yarn_frequencies(rot: dict) -> tuple[torch.Tensor, float]:
    """The angular step of every pair and the factor on cos and sin."""
    n = int(rot["dims"])
    base = float(rot["base"])
    i = torch.arange(n // 2, dtype=F64)
    f = base ** (-2.0 * i / n)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_index(turns):       # the (fractional) pair that makes `turns` turns over the original length
        return n * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_index(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_index(float(sc["slow"]))), n - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., >= dims]: neighbours (2i, 2i + 1) of the first `dims` entries turn by position * f_i."""
    n = int(rot["dims"])
    f, m = yarn_frequencies(rot)
    ang = positions.to(F64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [n // 2]
    c, s = (torch.cos(ang) * m).view(shape), (torch.sin(ang) * m).view(shape)
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def visible(T: int, window: int = 0) -> torch.Tensor:
    """[T, T] True where query i may read key j: j <= i, and i - j < window where there is a window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j) < window
    return ok


def softmax_heads(q, k, v, scale, mask):
    """q [T, n, dk], k [T, n, dk], v [T, n, dv] -> [T, n * dv]."""
    s = torch.einsum("inc,jnc->nij", q, k) * scale
    s = s.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("nij,jnc->inc", p, v).reshape(q.shape[0], -1)


def latent_of(h, w, pre, m, eps):
    """The latent that a layer's keys and values are made from, and the shared rotated key part (None
    where the mixer has none)."""
    L = int(m["kv_rank"])
    a = linear(h, w[pre + "dkv"])
    c = norm_plain(a[:, :L], w[pre + "dkv.norm"], eps)
    return c, (a[:, L:] if a.shape[1] > L else None)


def latent_attention(h, w, pre, m, eps, latent=None, window=0):
    """Attention whose keys and values are expanded from a latent per token. latent: (c, shared part)
    of another layer, for a mixer that has no down map of its own."""
    T = h.shape[0]
    n, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    r = int(m.get("rot_dim", 0))
    pos = torch.arange(T)
    cq = norm_plain(linear(h, w[pre + "dq"]), w[pre + "dq.norm"], eps)
    q = linear(cq, w[pre + "uq"]).view(T, n, d + r)
    c, shared = latent if latent is not None else latent_of(h, w, pre, m, eps)
    k = linear(c, w[pre + "uk"]).view(T, n, d)
    v = linear(c, w[pre + "uv"]).view(T, n, dv)
    if r:
        qr = rotate_pairs(q[..., d:], pos, m["rot"])
        kr = rotate_pairs(shared.view(T, 1, r), pos, m["rot"]).expand(T, n, r)
        q = torch.cat([q[..., :d], qr], -1)
        k = torch.cat([k, kr], -1)
    o = softmax_heads(q, k, v, float(m["scale"]), visible(T, window))
    return linear(o, w[pre + "o"]), (c, shared)


def gated_ff(h, w, pre, act):
    return linear(act(linear(h, w[pre + "gate"])) * linear(h, w[pre + "up"]), w[pre + "down"])


def route(h, w_router, top, scale):
    """Per token: the chosen experts and their weights (softmax scores times scale, not renormalised)."""
    s = torch.softmax(linear(h, w_router), dim=-1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val * scale


def expert_ff(h, w, pre, mlp):
    r = mlp["router"]
    idx, wt = route(h, w[pre + "router"], int(r["top"]), float(r["scale"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            out[t] += a * gated_ff(h[t:t + 1], w, f"{pre}e{e}.", silu)[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, w, pre + "shared.", silu)
    return out


def forward(cfg: dict, w: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual after every layer)."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    latents, after = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = norm_centered(x, w[p + "norm1"], eps)
        src = m.get("kv_from")
        window = int(m["mask"]["size"]) if layer["type"] == "latent_attention_2" else 0
        y, latents[i] = latent_attention(h, w, p + "mix.", m, eps, latents[src] if src is not None else None, window)
        x = x + norm_centered(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_centered(x, w[p + "norm2"], eps)
            y = gated_ff(h, w, p + "mlp.", gelu_tanh) if mlp["kind"] == "dense" else expert_ff(h, w, p + "mlp.", mlp)
            x = x + norm_centered(y, w[p + "norm2b"], eps)
        after.append(x)
    logits = linear(norm_centered(x, w["final.norm"], eps), w["head"])
    return (logits, torch.stack(after)) if return_layers else logits
