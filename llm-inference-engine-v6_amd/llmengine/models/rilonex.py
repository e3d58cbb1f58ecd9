"""Rilonex as a list of layer specs: a residual in several streams (hyper-connections) around three
kinds of mixers (the RG-LRU recurrent block, the gated delta rule with a decay per key channel, and
an attention without softmax beside a gated delta rule with a decay per head) and a feed-forward
gated by a rectifier. Tensor names: "embed", "l<i>.norm1", "l<i>.mix.*", "l<i>.norm2", "l<i>.mlp.*",
"l<i>.hc1.*", "l<i>.hc2.*", "final.norm", "head".
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.rilonex import RilonexConfig, RilonexLayer
from ..parts import make_part
from .model import DecoderModel


def _delta(cfg: RilonexConfig, m: dict, decay: str, gate: str):
    return make_part("mixer", "gated_delta", hidden_size=cfg.width, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"],
                     vdim=m["vdim"], conv_taps=m["conv"], eps=cfg.norm_eps, decay=decay, gate=gate,
                     decay_rank=m.get("decay_rank"), gate_rank=m.get("gate_rank"))


def rilonex_mixer(cfg: RilonexConfig, layer: RilonexLayer):
    m = layer.mixer
    if layer.type == "rglru":
        return make_part("mixer", "rglru", hidden_size=cfg.width, width=m["width"], blocks=m["blocks"], conv_taps=m["conv"])
    if layer.type == "channel_delta":
        return _delta(cfg, m, "channel", "sigmoid_lowrank")
    if layer.type == "parallel":
        a = m["left"]
        left = make_part("mixer", "sigmoid_attention", hidden_size=cfg.width, heads=a["heads"], kv_heads=a["kv_heads"],
                         dim=a["dim"], vdim=a["vdim"], scale=a["scale"], rot_dims=a["rot_dims"], rot_base=a["rot_base"])
        return make_part("mixer", "parallel", left=left, right=_delta(cfg, m["right"], "head", "silu"),
                         left_scale=m["left_scale"], right_scale=m["right_scale"])
    raise ValueError(f"no mixer of type {layer.type!r}")


def build_rilonex(cfg: RilonexConfig) -> DecoderModel:
    names = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "feed_forward": "mlp"}
    layers = []
    for layer in cfg.layers:
        norm = lambda: make_part("norm", "rmsnorm", size=cfg.width, eps=cfg.norm_eps, tensor="")
        ff = None
        if layer.mlp_ff is not None:
            ff = make_part("feed_forward", "gated_mlp", hidden_size=cfg.width, intermediate_size=layer.mlp_ff,
                           activation="relu", names={"gate": "gate", "up": "up", "down": "down"})
        parts = dict(mixer=rilonex_mixer(cfg, layer), feed_forward=ff, mixer_norm=norm(),
                     ffn_norm=norm() if ff is not None else None, names=names)
        if cfg.streams:
            layers.append(make_part("block", "hyper", streams=cfg.streams, **parts))
        else:
            layers.append(make_part("block", "prenorm", **parts))
    embedding = make_part("embedding", "table", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="")
    head = make_part("head", "linear", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="")
    final_norm = make_part("norm", "rmsnorm", size=cfg.width, eps=cfg.norm_eps, tensor="")
    return DecoderModel(cfg, embedding, layers, final_norm, head, streams=cfg.streams,
                        names={"embedding": "embed", "layers": "l{}", "final_norm": "final.norm", "head": "head"})


register_architecture("Rilonex", RilonexConfig.from_dict, build_rilonex)
