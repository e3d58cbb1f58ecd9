"""BidiraxConfig: the typed view of a Bidirax config.json.

The file names the vocabulary ("vocab"), the residual width ("width"), the embedding's multiplier
("embedding": {"scale"}), the norms' epsilon ("norm": {"eps"}) and a list "layers", one entry per layer:
"type" (which mixer), "mixer" (its sizes and constants) and "mlp" (the feed-forward: "kind" "dense" with
"ff", or "moe" with "router" {"experts", "top", "scale"}, "expert" {"ff"} and optionally "shared" {"ff"};
null for a layer without one). Nothing else is read. The design has no longest position and no
end-of-sequence token.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

from .base import ConfigError, KeyReader

MIXER_TYPES = ("latent_attention", "latent_attention_2")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class BidiraxLayer:
    type: str
    mixer: Mapping[str, Any]            # the mixer's sizes and constants, checked, as plain values
    mlp: Mapping[str, Any] | None       # {"kind": "dense", "ff"} or {"kind": "moe", "experts", "top", "scale", "ff", "shared_ff"}


def _rotation(m: KeyReader, rot_dim: int) -> dict | None:
    rot = m.mapping("rot")
    if rot is None or rot_dim == 0:
        if rot_dim:
            raise ConfigError(f"{m.where}: rot_dim={rot_dim} needs 'rot'")
        return None
    out = {"dims": rot.integer("dims", minimum=0), "base": rot.number("base"), "scaling": None}
    if out["dims"] % 2 or out["dims"] > rot_dim:
        raise ConfigError(f"{rot.where}: dims={out['dims']} must be even and at most rot_dim={rot_dim}")
    if out["base"] <= 0:
        raise ConfigError(f"{rot.where}: base must be > 0")
    sc = rot.mapping("scaling")
    if sc is not None:
        out["scaling"] = {"factor": sc.number("factor"), "original": sc.number("original"), "fast": sc.number("fast"),
                          "slow": sc.number("slow")}
        if out["scaling"]["factor"] <= 0 or out["scaling"]["original"] <= 0 or min(out["scaling"]["fast"], out["scaling"]["slow"]) <= 0:
            raise ConfigError(f"{sc.where}: factor, original, fast and slow must be > 0")
    return out


def _mixer(r: KeyReader, kind: str, index: int) -> dict:
    m = r.mapping("mixer")
    if m is None:
        raise ConfigError(f"{r.where}: required key 'mixer' is missing")
    out = {"heads": m.integer("heads", minimum=1), "dim": m.integer("dim", minimum=1), "vdim": m.integer("vdim", minimum=1),
           "kv_rank": m.integer("kv_rank", minimum=1), "q_rank": m.integer("q_rank", minimum=1), "scale": m.number("scale"),
           "rot_dim": m.integer("rot_dim", 0, minimum=0), "window": 0, "kv_from": None}
    if out["rot_dim"] % 2:
        raise ConfigError(f"{m.where}: rot_dim={out['rot_dim']} must be even")
    out["rot"] = _rotation(m, out["rot_dim"])
    mask = m.mapping("mask")
    if mask is not None:
        out["window"] = mask.integer("size", minimum=1)
    elif kind == "latent_attention_2":
        raise ConfigError(f"{m.where}: a mixer of type {kind!r} needs 'mask': {{'size'}}")
    if m.has("kv_from"):
        out["kv_from"] = m.integer("kv_from", minimum=0)
        if out["kv_from"] >= index:
            raise ConfigError(f"{m.where}: kv_from={out['kv_from']} must name an earlier layer than {index}")
    return out


def _mlp(r: KeyReader) -> dict | None:
    mlp = r.mapping("mlp")
    if mlp is None:
        return None
    kind = mlp.string("kind")
    if kind == "dense":
        return {"kind": kind, "ff": mlp.integer("ff", minimum=1)}
    if kind == "moe":
        router, expert, shared = mlp.mapping("router"), mlp.mapping("expert"), mlp.mapping("shared")
        if router is None or expert is None:
            raise ConfigError(f"{mlp.where}: a mixture of experts needs 'router' and 'expert'")
        out = {"kind": kind, "experts": router.integer("experts", minimum=1), "top": router.integer("top", minimum=1),
               "scale": router.number("scale", 1.0), "ff": expert.integer("ff", minimum=1),
               "shared_ff": shared.integer("ff", minimum=1) if shared is not None else None}
        if out["top"] > out["experts"]:
            raise ConfigError(f"{router.where}: top={out['top']} is more than experts={out['experts']}")
        return out
    raise ConfigError(f"{mlp.where}: kind {kind!r} is none of {list(MLP_KINDS)}")


@dataclass(frozen=True)
class BidiraxConfig:
    architecture: str
    vocab_size: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: tuple[BidiraxLayer, ...]
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def max_pos(self) -> int:
        """Positions are not limited by the design (angles are computed from the position)."""
        return 1 << 30

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], generation_cfg: Mapping[str, Any] | None = None,
                  architecture: str = "Bidirax") -> "BidiraxConfig":
        r = KeyReader(cfg)
        norm = r.mapping("norm")
        if norm is None:
            raise ConfigError("config.json: required key 'norm' is missing")
        raw = cfg.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw):
            lr = KeyReader(entry, f"config.json:layers[{i}]")
            kind = lr.string("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{lr.where}: mixer type {kind!r} is none of {list(MIXER_TYPES)}")
            layers.append(BidiraxLayer(kind, _mixer(lr, kind, i), _mlp(lr)))
        for i, layer in enumerate(layers):
            src = layer.mixer["kv_from"]
            if src is None:
                continue
            other = layers[src].mixer
            if other["kv_from"] is not None:
                raise ConfigError(f"config.json:layers[{i}]: kv_from={src} names a layer that keeps no latent of its own")
            if other["kv_rank"] != layer.mixer["kv_rank"] or layer.mixer["rot_dim"] not in (0, other["rot_dim"]):
                raise ConfigError(f"config.json:layers[{i}]: kv_rank must equal that of layer {src}, whose latent it reads "
                                  "(and rot_dim, unless it is 0)")
        emb = r.mapping("embedding")
        return cls(architecture=architecture, vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   embedding_scale=emb.number("scale", 1.0) if emb is not None else 1.0, norm_eps=norm.number("eps"),
                   layers=tuple(layers))
