"""Small Bidirax configurations for the tests, and weights for them that the tests draw themselves (matrices
of order one over the root of their inputs, norm weights of the sublayers around zero, the latents' plain
norm weights around one). `sharp` multiplies an attention's scale so that its softmax stands on a few keys:
a key that is lost, or one too many, then moves the whole row."""
from __future__ import annotations

import json
import os

import torch


def rotated(heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, q_rank=14, scale=0.3, base=50.0, dims=None, scaling=True,
            mlp="dense", sharp=1.0, **more):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = scaling if isinstance(scaling, dict) else {"factor": 4.0, "original": 24, "fast": 3.0, "slow": 0.5}
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "scale": scale * sharp, "rot": rot, **more},
            "mlp": feed_forward(mlp)}


def windowed(heads=2, dim=10, vdim=14, kv_rank=12, q_rank=18, scale=0.35, window=9, kv_from=None, mlp="moe", sharp=1.0):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale * sharp,
         "mask": {"size": window}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention_2", "mixer": m, "mlp": feed_forward(mlp)}


def feed_forward(kind, ff=24, experts=5, top=2, scale=1.7, shared=20):
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": ff}
    if isinstance(kind, dict):
        return kind
    out = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def config(layers, width=28, vocab=61, eps=1e-5, embed_scale=2.5):
    return {"architecture": "Bidirax", "vocab": vocab, "width": width, "embedding": {"scale": embed_scale},
            "norm": {"eps": eps}, "layers": list(layers)}


# both mixers, a layer that reads the latent of the layer two in front of it through a wider window, sizes that are
# no powers of two, a layer without feed-forward, experts with and without a shared one
MIXED = config([rotated(), windowed(window=9), rotated(heads=2, dim=6, rot_dim=4, vdim=6, kv_rank=10, q_rank=8, scaling=None, mlp=None),
                windowed(heads=3, dim=8, vdim=6, window=13, kv_from=1, mlp=feed_forward("moe", experts=3, top=1, shared=None)),
                windowed(heads=1, dim=16, vdim=8, kv_rank=8, q_rank=8, window=20, mlp="dense")])
# sizes that the matrix kernels take (multiples of 16 and 32), as a model served in bfloat16 has them
ALIGNED = config([rotated(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64, q_rank=32, scale=0.12, base=10000.0,
                          scaling={"factor": 2.0, "original": 64, "fast": 8.0, "slow": 1.0}, mlp={"kind": "dense", "ff": 128}),
                  windowed(heads=4, dim=32, vdim=48, kv_rank=32, q_rank=64, scale=0.17, window=40,
                           mlp=feed_forward("moe", ff=64, experts=8, top=2, shared=64)),
                  windowed(heads=8, dim=16, vdim=16, kv_rank=32, q_rank=32, scale=0.25, window=24, kv_from=1,
                           mlp=feed_forward("moe", ff=32, experts=4, top=3, shared=None))], width=64, vocab=128)


def make_weights(cfg: dict, seed: int, dtype=torch.bfloat16) -> dict:
    """name -> tensor for every tensor of the configuration's model (names and shapes as the engine's model tree
    lists them; the values are the tests' own)."""
    from llmengine.config.registry import architecture_name, parse_config, resolve
    model = resolve(architecture_name(cfg)).build_model(parse_config(cfg))
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in model.named_specs().items():
        shape = tuple(spec.shape)
        leaf = name.split(".")[-1]
        if name.endswith("dq.norm") or name.endswith("dkv.norm"):
            t = torch.randn(shape, generator=g) * 0.2 + 1.0
        elif len(shape) == 1:
            t = torch.randn(shape, generator=g) * 0.25             # stored around zero
        elif leaf == "router":
            t = torch.randn(shape, generator=g) * 2.5 / shape[-1] ** 0.5
        else:
            t = torch.randn(shape, generator=g) * 1.3 / shape[-1] ** 0.5
        out[name] = t.to(dtype)
    return out


def write_model(tmp_path, cfg: dict, seed: int, dtype=torch.bfloat16, weights: dict | None = None) -> tuple[str, dict]:
    from llmengine.weights import write_state_dict
    weights = weights if weights is not None else make_weights(cfg, seed, dtype)
    os.makedirs(str(tmp_path), exist_ok=True)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(cfg, f)
    write_state_dict(os.path.join(str(tmp_path), "model.safetensors"), weights)
    return str(tmp_path), weights
