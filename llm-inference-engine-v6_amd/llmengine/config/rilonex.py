"""RilonexConfig: the typed view of a Rilonex config.json.

The file names the vocabulary ("vocab"), the residual width ("width"), the number of residual
streams ("streams"; absent: a plain residual), the norms' epsilon ("norm": {"eps"}) and a list
"layers", one entry per layer: "type" (which mixer), "mixer" (its sizes) and "mlp" (the
feed-forward's kind and size, or null for a layer without one). Nothing else is read; every size
that the file does not name comes from a tensor's shape. The design has no longest position and no
end-of-sequence token.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

from .base import ConfigError, KeyReader

MIXER_TYPES = ("rglru", "channel_delta", "parallel")
MLP_KINDS = ("dense",)


@dataclass(frozen=True)
class RilonexLayer:
    type: str
    mixer: Mapping[str, Any]            # the mixer's sizes, checked, as plain values
    mlp_ff: int | None                  # the feed-forward's inner size; None: no feed-forward


def _delta_sizes(r: KeyReader) -> dict:
    out = {"heads": r.integer("heads", minimum=1), "kv_heads": r.integer("kv_heads", minimum=1),
           "dim": r.integer("dim", minimum=1), "vdim": r.integer("vdim", minimum=1), "conv": r.integer("conv", minimum=1)}
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{r.where}: heads={out['heads']} is no multiple of kv_heads={out['kv_heads']}")
    for key in ("decay_rank", "gate_rank"):         # only needed where no checkpoint gives the tensors' shapes
        if r.has(key):
            out[key] = r.integer(key, minimum=1)
    return out


def _attention_sizes(r: KeyReader) -> dict:
    out = {"heads": r.integer("heads", minimum=1), "kv_heads": r.integer("kv_heads", minimum=1),
           "dim": r.integer("dim", minimum=1), "vdim": r.integer("vdim", minimum=1), "scale": r.number("scale"),
           "rot_dims": 0, "rot_base": 10000.0}
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{r.where}: heads={out['heads']} is no multiple of kv_heads={out['kv_heads']}")
    rot = r.mapping("rot")
    if rot is not None:
        out["rot_dims"] = rot.integer("dims", minimum=0)
        out["rot_base"] = rot.number("base")
        if out["rot_dims"] % 2 or out["rot_dims"] > out["dim"]:
            raise ConfigError(f"{rot.where}: dims={out['rot_dims']} must be even and at most dim={out['dim']}")
        if out["rot_base"] <= 0:
            raise ConfigError(f"{rot.where}: base must be > 0")
    return out


def _layer(r: KeyReader) -> RilonexLayer:
    kind = r.string("type")
    m = r.mapping("mixer")
    if m is None:
        raise ConfigError(f"{r.where}: required key 'mixer' is missing")
    if kind == "rglru":
        mixer = {"width": m.integer("width", minimum=1), "blocks": m.integer("blocks", minimum=1),
                 "conv": m.integer("conv", minimum=1)}
        if mixer["width"] % mixer["blocks"]:
            raise ConfigError(f"{m.where}: width={mixer['width']} is no multiple of blocks={mixer['blocks']}")
    elif kind == "channel_delta":
        mixer = _delta_sizes(m)
    elif kind == "parallel":
        left, right = m.mapping("left"), m.mapping("right")
        if left is None or right is None:
            raise ConfigError(f"{m.where}: a parallel mixer needs 'left' and 'right'")
        mixer = {"left": _attention_sizes(left), "right": _delta_sizes(right),
                 "left_scale": m.number("left_scale"), "right_scale": m.number("right_scale")}
    else:
        raise ConfigError(f"{r.where}: mixer type {kind!r} is none of {list(MIXER_TYPES)}")
    mlp = r.mapping("mlp")
    ff = None
    if mlp is not None:
        mlp_kind = mlp.string("kind")
        if mlp_kind not in MLP_KINDS:
            raise ConfigError(f"{mlp.where}: kind {mlp_kind!r} is none of {list(MLP_KINDS)}")
        ff = mlp.integer("ff", minimum=1)
    return RilonexLayer(kind, mixer, ff)


@dataclass(frozen=True)
class RilonexConfig:
    architecture: str
    vocab_size: int
    width: int
    streams: int                        # 0: a plain residual
    norm_eps: float
    layers: tuple[RilonexLayer, ...]
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def max_pos(self) -> int:
        """Positions are not limited by the design (angles are computed, states have a fixed size)."""
        return 1 << 30

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], generation_cfg: Mapping[str, Any] | None = None,
                  architecture: str = "Rilonex") -> "RilonexConfig":
        r = KeyReader(cfg)
        norm = r.mapping("norm")
        if norm is None:
            raise ConfigError("config.json: required key 'norm' is missing")
        raw = cfg.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = tuple(_layer(KeyReader(entry, f"config.json:layers[{i}]")) for i, entry in enumerate(raw))
        streams = r.integer("streams", 0, minimum=0)
        return cls(architecture=architecture, vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   streams=streams, norm_eps=norm.number("eps"), layers=layers)
