"""Small Rilonex configurations for the tests, and weights for them that the tests draw themselves:
every kind of tensor gets values in a range where its mechanism shows (decays well inside (0, 1),
stream weights around one with a visible mix between streams, head-mixing matrices with off-diagonal
entries, convolution taps of order one)."""
from __future__ import annotations

import os

import torch


def rglru(width=48, blocks=3, conv=3, ff=40):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def channel_delta(heads=4, kv_heads=2, dim=24, vdim=20, conv=4, ff=40, decay_rank=6, gate_rank=5):
    return {"type": "channel_delta",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                      "decay_rank": decay_rank, "gate_rank": gate_rank},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def parallel(heads=6, kv_heads=2, dim=24, vdim=40, rot_dims=16, rot_base=100.0, scale=0.3, d_heads=2, d_kv=1, d_dim=16,
             d_vdim=24, conv=2, left_scale=0.7, right_scale=1.2, ff=40):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                               "rot": {"dims": rot_dims, "base": rot_base}},
                      "right": {"heads": d_heads, "kv_heads": d_kv, "dim": d_dim, "vdim": d_vdim, "conv": conv},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(layers, width=40, vocab=97, streams=2, eps=1e-5):
    cfg = {"architecture": "Rilonex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": list(layers)}
    if streams is not None:
        cfg["streams"] = streams
    return cfg


# all three mixers, sizes that are no powers of two, a layer without feed-forward, three streams
MIXED = config([rglru(), channel_delta(), parallel(), rglru(width=40, blocks=1, conv=2, ff=None),
                parallel(heads=2, kv_heads=2, dim=16, vdim=16, rot_dims=16, d_heads=3, d_kv=3, d_dim=8, d_vdim=8, conv=5)],
               width=40, vocab=97, streams=3)
# sizes that fit the matrix kernels (multiples of 32 and 16), one stream, as a model served in bfloat16 has them
ALIGNED = config([rglru(width=128, blocks=2, conv=4, ff=128), channel_delta(heads=2, kv_heads=2, dim=64, vdim=32, ff=128,
                                                                           decay_rank=16, gate_rank=16),
                  parallel(heads=4, kv_heads=2, dim=32, vdim=32, rot_dims=32, d_heads=2, d_kv=1, d_dim=32, d_vdim=64, conv=4,
                           ff=128)], width=64, vocab=128, streams=1)
# a plain residual (no streams key at all)
PLAIN = config([channel_delta(ff=None), rglru()], width=24, vocab=50, streams=None)


def make_weights(cfg: dict, seed: int, dtype=torch.bfloat16) -> dict:
    """name -> tensor for every tensor of the configuration's model (names and shapes as the engine's model
    tree lists them; the values are the tests' own)."""
    from llmengine.config.registry import architecture_name, parse_config, resolve
    model = resolve(architecture_name(cfg)).build_model(parse_config(cfg))
    g = torch.Generator().manual_seed(seed)
    out = {}

    def rnd(shape, std=1.0, mean=0.0):
        return torch.randn(shape, generator=g) * std + mean

    for name, spec in model.named_specs().items():
        shape = tuple(spec.shape)
        leaf = name.split(".")[-1]
        tail2 = ".".join(name.split(".")[-2:])
        if leaf in ("norm1", "norm2") or name == "final.norm" or tail2.endswith("mix.norm") or leaf == "norm":
            t = rnd(shape, 0.2, 1.0)
        elif leaf in ("in", "out") and ".hc" in name:
            t = rnd(shape, 0.3, 1.0)
        elif leaf == "mix" and ".hc" in name:
            t = torch.eye(shape[0]) + rnd(shape, 0.25)
        elif leaf == "conv":
            t = rnd(shape, 0.6)
        elif leaf == "talk":
            t = torch.eye(shape[0]) + rnd(shape, 0.4)
        elif leaf in ("pb", "dt_bias", "lam", "A_log"):
            t = rnd(shape, 0.7, -0.5 if leaf == "A_log" else 0.0)
        elif leaf == "b" and len(shape) == 1:                   # biases of the recurrent block
            t = rnd(shape, 0.3)
        elif len(shape) >= 2:
            t = rnd(shape, 1.4 / (shape[-1] ** 0.5))
        else:
            t = rnd(shape, 0.3)
        out[name] = t.to(dtype)
    return out


def write_model(tmp_path, cfg: dict, seed: int, dtype=torch.bfloat16, weights: dict | None = None) -> tuple[str, dict]:
    """Writes config.json and model.safetensors; returns (folder, the weights as stored)."""
    import json
    from llmengine.weights import write_state_dict
    weights = weights if weights is not None else make_weights(cfg, seed, dtype)
    os.makedirs(str(tmp_path), exist_ok=True)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(cfg, f)
    write_state_dict(os.path.join(str(tmp_path), "model.safetensors"), weights)
    return str(tmp_path), weights
