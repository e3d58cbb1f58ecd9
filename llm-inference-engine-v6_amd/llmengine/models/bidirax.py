"""Bidirax as a list of layers: an embedding with a multiplier, layers with a norm in front of and behind
every sublayer, two kinds of latent attention (rotated with all earlier tokens visible; unrotated under a
sliding window, possibly reading the latent that an earlier layer cached) and a feed-forward that is dense
(gated by the tanh form of GELU) or a mixture of SiLU-gated experts beside a shared one. Tensor names:
"embed", "l<i>.norm1", "l<i>.norm1b", "l<i>.mix.*", "l<i>.norm2", "l<i>.norm2b", "l<i>.mlp.*", "final.norm", "head".
"""
from __future__ import annotations

from ..config.bidirax import BidiraxConfig, BidiraxLayer
from ..config.registry import register_architecture
from ..parts import make_part
from .model import DecoderModel, LayerCall

_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def bidirax_mixer(cfg: BidiraxConfig, layer: BidiraxLayer, keep: int):
    """keep: how many of the last tokens the layer's cache must hold (0: all), which is more than the layer's own
    window where a later layer reads the same rows through a wider one."""
    m = layer.mixer
    return make_part("mixer", "latent_attention", hidden_size=cfg.width, heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"],
                     vdim=m["vdim"], kv_rank=m["kv_rank"], q_rank=m["q_rank"], scale=m["scale"], eps=cfg.norm_eps,
                     rot=m["rot"], window=m["window"], keeps_latent=m["kv_from"] is None, cache_window=keep)


def bidirax_feed_forward(cfg: BidiraxConfig, layer: BidiraxLayer):
    mlp = layer.mlp
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return make_part("feed_forward", "gated_mlp", hidden_size=cfg.width, intermediate_size=mlp["ff"],
                         activation="gelu_tanh", names=_MLP_NAMES)
    shared = None
    if mlp["shared_ff"] is not None:
        shared = make_part("feed_forward", "gated_mlp", hidden_size=cfg.width, intermediate_size=mlp["shared_ff"],
                           activation="silu", names=_MLP_NAMES)
    return make_part("feed_forward", "mixture_of_experts", hidden_size=cfg.width, intermediate_size=mlp["ff"],
                     experts=mlp["experts"], top=mlp["top"], scale=mlp["scale"], renormalize=False, activation="silu",
                     shared=shared)


def build_bidirax(cfg: BidiraxConfig) -> DecoderModel:
    norm = lambda: make_part("norm", "rmsnorm_centered", size=cfg.width, eps=cfg.norm_eps, tensor="")
    # what a layer's cache must keep: the widest window among the layers that read it (0, everything, wins)
    keep = {i: layer.mixer["window"] for i, layer in enumerate(cfg.layers) if layer.mixer["kv_from"] is None}
    for layer in cfg.layers:
        src = layer.mixer["kv_from"]
        if src is not None:
            keep[src] = 0 if 0 in (keep[src], layer.mixer["window"]) else max(keep[src], layer.mixer["window"])
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        ff = bidirax_feed_forward(cfg, layer)
        layers.append(make_part("block", "sandwich", mixer=bidirax_mixer(cfg, layer, keep.get(i, 0)), feed_forward=ff,
                                mixer_norm=norm(), mixer_post_norm=norm(), ffn_norm=norm() if ff is not None else None,
                                ffn_post_norm=norm() if ff is not None else None))
        src = layer.mixer["kv_from"]
        schedule.append(LayerCall(i) if src is None else LayerCall(i, cache=src, write_cache=False))
    embedding = make_part("embedding", "table", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="",
                          scale=cfg.embedding_scale)
    head = make_part("head", "linear", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="")
    final_norm = make_part("norm", "rmsnorm_centered", size=cfg.width, eps=cfg.norm_eps, tensor="")
    return DecoderModel(cfg, embedding, layers, final_norm, head, schedule=schedule,
                        names={"embedding": "embed", "layers": "l{}", "final_norm": "final.norm", "head": "head"})


register_architecture("Bidirax", BidiraxConfig.from_dict, build_bidirax)
