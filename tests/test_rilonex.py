"""Rilonex without a GPU: the configuration reader, the model tree's tensor names, and the plain
implementation's mechanisms against facts that pin them independently of the engine."""
from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_rilonex as plain
import rilonex_models as rm


def _model(cfg):
    from llmengine.config.registry import architecture_name, parse_config, resolve
    return resolve(architecture_name(cfg)).build_model(parse_config(cfg))


def test_the_architecture_is_found_by_its_name():
    from llmengine.config import RilonexConfig, parse_config
    c = parse_config(rm.MIXED)
    assert isinstance(c, RilonexConfig) and c.streams == 3 and c.vocab_size == 97 and len(c.layers) == 5
    assert c.layers[3].mlp_ff is None and c.layers[2].mixer["left"]["rot_dims"] == 16
    assert parse_config(rm.PLAIN).streams == 0


@pytest.mark.parametrize("edit,needle", [
    (lambda c: c["layers"][0].update(type="lstm"), "lstm"),
    (lambda c: c["layers"][0]["mixer"].pop("blocks"), "blocks"),
    (lambda c: c["layers"][0]["mixer"].update(blocks=5), "blocks"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][2]["mixer"]["left"]["rot"].update(dims=30), "dims"),
    (lambda c: c["layers"][2]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "moe"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_bad_configuration_is_refused_by_the_name_of_its_key(edit, needle):
    from llmengine.config import ConfigError, parse_config
    cfg = copy.deepcopy(rm.MIXED)
    edit(cfg)
    with pytest.raises(ConfigError, match=needle):
        parse_config(cfg)


def test_tensor_names_and_shapes_of_the_model_tree():
    specs = _model(rm.MIXED).named_specs()
    shape = lambda n: tuple(specs[n].shape)
    assert shape("embed") == (97, 40) and shape("head") == (97, 40) and shape("final.norm") == (40,)
    assert shape("l0.norm1") == (40,) and shape("l0.hc1.mix") == (3, 3) and shape("l0.hc2.in") == (3,)
    assert shape("l0.mix.ra") == (3, 16, 16) and shape("l0.mix.conv") == (48, 3) and shape("l0.mix.y.b") == (48,)
    assert shape("l1.mix.q") == (48, 40) and shape("l1.mix.v.conv") == (80, 4) and shape("l1.mix.a2") == (96, 6)
    assert shape("l1.mix.dt_bias") == (96,) and shape("l1.mix.g2") == (80, 5) and shape("l1.mix.norm") == (20,)
    assert shape("l2.mix.left.q") == (144, 40) and shape("l2.mix.left.v") == (80, 40) and shape("l2.mix.left.talk") == (6, 6)
    assert shape("l2.mix.right.a") == (2, 40) and shape("l2.mix.right.dt_bias") == (2,) and shape("l2.mix.right.g") == (48, 40)
    assert shape("l2.mlp.gate") == (40, 40) and shape("l2.mlp.down") == (40, 40)
    # a layer without feed-forward has neither its norm nor its stream weights
    assert not any(n.startswith(("l3.mlp", "l3.norm2", "l3.hc2")) for n in specs) and "l3.hc1.in" in specs
    # a plain residual has no stream weights at all
    assert not any(".hc" in n for n in _model(rm.PLAIN).named_specs())


def test_a_rank_left_to_the_checkpoint_fits_any_size():
    from llmengine.weights import WeightError, check_names
    cfg = copy.deepcopy(rm.config([rm.channel_delta(ff=None)], streams=None))
    del cfg["layers"][0]["mixer"]["decay_rank"]
    model = _model(cfg)
    assert tuple(model.named_specs()["l0.mix.a1"].shape) == (None, 40)
    shapes = {n: tuple(7 if d is None else d for d in s.shape) for n, s in model.named_specs().items()}
    check_names(model, shapes, "here")
    shapes["l0.mix.a2"] = (95, 7)
    with pytest.raises(WeightError, match="a2"):
        check_names(model, shapes, "here")


def test_the_cache_spec_of_every_mixer():
    specs = _model(rm.MIXED).cache_specs()
    assert set(specs[0].state) == {"s", "conv"} and specs[0].state["conv"][0] == (2, 48) and not specs[0].paged
    assert specs[1].state["memory"][0] == (4, 20, 24) and specs[1].state["conv"][0] == (3, 2 * 48 + 80)
    assert set(specs[2].paged) == {"left.k", "left.v"} and set(specs[2].state) == {"right.memory", "right.conv"}
    assert all(dtype == torch.float32 for spec in specs.values() for _, dtype in spec.state.values())


# --- the plain implementation's mechanisms ---------------------------------------------------------
def test_plain_short_conv_is_a_causal_correlation():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(9, 5, generator=g, dtype=torch.float64), torch.randn(5, 4, generator=g, dtype=torch.float64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), w[:, None, :], groups=5)[0].T
    assert torch.allclose(plain.short_conv(x, w), want, atol=1e-12)


def test_plain_rotation_depends_on_the_distance_only():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 12, generator=g, dtype=torch.float64), torch.randn(1, 1, 12, generator=g, dtype=torch.float64)
    def score(i, j):
        return float((plain.rotate_half_pairs(q, torch.tensor([i]), 8, 50.0) * plain.rotate_half_pairs(k, torch.tensor([j]), 8, 50.0)).sum())
    assert abs(score(7, 3) - score(104, 100)) < 1e-9 and abs(score(7, 3) - score(7, 4)) > 1e-3
    # entries behind the rotated ones pass unchanged
    assert torch.equal(plain.rotate_half_pairs(q, torch.tensor([5]), 8, 50.0)[..., 8:], q[..., 8:])


def test_plain_delta_memory_stores_and_overwrites():
    """With unit keys, beta = 1 and no decay the memory returns the value last written under a key."""
    k = torch.eye(3, dtype=torch.float64)[[0, 1, 0]]
    v = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]], dtype=torch.float64)
    out = plain.delta_memory(k, k, v, torch.ones(3, dtype=torch.float64), torch.ones(3, 1, dtype=torch.float64))
    assert torch.allclose(out, v)
    # a decay of one half per token halves what an older write returns
    out = plain.delta_memory(torch.eye(3, dtype=torch.float64)[[0, 0, 0]], torch.eye(3, dtype=torch.float64)[[0, 1, 1]],
                             v, torch.tensor([1.0, 1.0, 1.0], dtype=torch.float64), torch.full((3, 1), 0.5, dtype=torch.float64))
    assert torch.allclose(out[2], 0.25 * v[0])


def test_plain_streams_reduce_to_a_residual():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 4, 6, generator=g, dtype=torch.float64)
    hc = {"in": torch.ones(1, dtype=torch.float64), "out": torch.ones(1, dtype=torch.float64), "mix": torch.ones(1, 1, dtype=torch.float64)}
    w = torch.ones(6, dtype=torch.float64)
    got = plain.hyper_sublayer(x, hc, w, 1e-5, lambda h: 2 * h)
    assert torch.allclose(got[0], x[0] + 2 * plain.rms_norm(x[0], w, 1e-5))


def test_plain_rglru_first_token_and_decay():
    """From an empty state the first token gives sqrt(1 - a^2) i u; a is in (0, 1) and falls with r."""
    W = 4
    p = {"y": torch.zeros(W, 3), "y.b": torch.full((W,), 10.0), "x": torch.zeros(W, 3), "x.b": torch.full((W,), 1.0),
         "conv": torch.tensor([[0.0, 1.0]] * W), "conv.b": torch.zeros(W), "ra": torch.zeros(2, 2, 2), "ra.b": torch.zeros(2, 2),
         "ri": torch.zeros(2, 2, 2), "ri.b": torch.zeros(2, 2), "lam": torch.zeros(W), "o": torch.eye(W)}
    p = {k: v.double() for k, v in p.items()}
    out = plain.rglru_mixer(torch.zeros(2, 3, dtype=torch.float64), p, 2)
    a = math.exp(-8.0 * 0.5 * math.log(2.0))
    first = math.sqrt(1 - a * a) * 0.5 * 1.0
    gate = float(plain.gelu_tanh(torch.tensor(10.0, dtype=torch.float64)))
    assert torch.allclose(out[0], torch.full((W,), first * gate, dtype=torch.float64))
    assert torch.allclose(out[1], torch.full((W,), (a * first + first) * gate, dtype=torch.float64))
