"""Bidirax on the CPU: the plain implementation's mechanisms pinned to independent facts, the configuration
reader, the tensor names and what the model asks of the cache manager."""
from __future__ import annotations

import copy
import math

import pytest
import torch

import bidirax_models as bm
import plain_bidirax as plain

F64 = torch.float64


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def test_centered_norm_is_the_plain_norm_with_one_added():
    x, w = _rand(5, 12), _rand(12, seed=1) * 0.1
    assert torch.allclose(plain.norm_centered(x, w, 1e-5), plain.norm_plain(x, w + 1.0, 1e-5))
    unit = plain.norm_plain(x, torch.ones(12, dtype=F64), 0.0)
    assert torch.allclose((unit * unit).mean(-1), torch.ones(5, dtype=F64))


def test_rotation_depends_on_distance_and_scales_by_the_factor():
    rot = {"dims": 8, "base": 50.0, "scaling": {"factor": 4.0, "original": 24, "fast": 3.0, "slow": 0.5}}
    q, k = _rand(1, 8), _rand(1, 8, seed=1)
    _, mag = plain.yarn_frequencies(rot)
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)

    def score(pq, pk):
        return float((plain.rotate_pairs(q, torch.tensor([pq]), rot) * plain.rotate_pairs(k, torch.tensor([pk]), rot)).sum())

    assert score(7, 3) == pytest.approx(score(104, 100), rel=1e-9)
    assert score(0, 0) == pytest.approx(float((q * k).sum()) * mag * mag, rel=1e-12)
    assert abs(score(7, 3) - score(7, 4)) > 1e-3
    # neighbours are partners: a vector with one pair set turns inside that pair only
    x = torch.zeros(1, 8, dtype=F64)
    x[0, 2] = 1.0
    y = plain.rotate_pairs(x, torch.tensor([5]), rot)
    assert torch.count_nonzero(y) == 2 and y[0, 2] != 0 and y[0, 3] != 0


def test_frequency_ramp():
    f, mag = plain.yarn_frequencies({"dims": 16, "base": 100.0})
    assert mag == 1.0 and torch.allclose(f, 100.0 ** (-torch.arange(8, dtype=F64) / 8))
    sc = {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 1.0}
    g, _ = plain.yarn_frequencies({"dims": 16, "base": 100.0, "scaling": sc})
    pair = lambda turns: 16 * math.log(64 / (2 * math.pi * turns)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(pair(4.0)), 0), min(math.ceil(pair(1.0)), 15)
    assert torch.allclose(g[:lo + 1], f[:lo + 1]) and torch.allclose(g[hi:], f[hi:] / 8.0)
    assert all(f[i] / 8.0 < g[i] < f[i] for i in range(lo + 1, hi))
    # the engine's frequencies are the same numbers
    from llmengine.parts.latent_attention import ramped_frequencies
    e, emag = ramped_frequencies(16, 100.0, sc)
    assert torch.allclose(e, g, rtol=1e-14) and emag == pytest.approx(0.1 * math.log(8.0) + 1.0)


def test_windows_and_softmax():
    m = plain.visible(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True] and m[1].tolist() == [True, True] + [False] * 4
    assert plain.visible(4).tolist() == torch.tril(torch.ones(4, 4)).bool().tolist()
    q, k, v = _rand(5, 2, 4), _rand(5, 2, 4, seed=1), _rand(5, 2, 3, seed=2)
    assert torch.allclose(plain.softmax_heads(q, k, v, 0.5, plain.visible(5, 1)), v.reshape(5, -1))      # a window of one: itself
    out = plain.softmax_heads(q, k, v, 0.5, plain.visible(5))
    s = (q[4, 1] @ k[:, 1].T) * 0.5
    assert torch.allclose(out[4, 3:], torch.softmax(s, 0) @ v[:, 1])


def _one_layer(layer, **kw):
    cfg = bm.config([layer], **kw)
    return cfg, {k: v.to(F64) for k, v in bm.make_weights(cfg, 5, torch.float32).items()}


def test_latent_attention_against_expanded_keys_and_values():
    cfg, w = _one_layer(bm.rotated(mlp=None))
    m = cfg["layers"][0]["mixer"]
    h = _rand(11, cfg["width"])
    y, (c, shared) = plain.latent_attention(h, w, "l0.mix.", m, 1e-5)
    # by hand for the last token and head 1
    n, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = plain.rms_unit(h @ w["l0.mix.dq"].T, 1e-5) * w["l0.mix.dq.norm"]
    q = (cq @ w["l0.mix.uq"].T).view(11, n, d + r)[10, 1]
    keys = (c @ w["l0.mix.uk"].T).view(11, n, d)[:, 1]
    pos = torch.arange(11)
    qr = plain.rotate_pairs(q[None, d:], pos[10:], m["rot"])[0]
    kr = plain.rotate_pairs(shared, pos, m["rot"])
    s = (keys @ q[:d] + kr @ qr) * m["scale"]
    o1 = torch.softmax(s, 0) @ (c @ w["l0.mix.uv"].T).view(11, n, dv)[:, 1]
    # the other heads' contribution removed: compare through the output matrix's columns of head 1
    full = plain.latent_attention(h, w, "l0.mix.", m, 1e-5)[0][10]
    w_o = w["l0.mix.o"].clone()
    w_o[:, dv:2 * dv] = 0
    w2 = dict(w)
    w2["l0.mix.o"] = w_o
    rest = plain.latent_attention(h, w2, "l0.mix.", m, 1e-5)[0][10]
    assert torch.allclose(full - rest, w["l0.mix.o"][:, dv:2 * dv] @ o1, atol=1e-10)
    assert c.shape == (11, m["kv_rank"]) and shared.shape == (11, r)
    # a window at least as long as the sequence is no window
    assert torch.allclose(plain.latent_attention(h, w, "l0.mix.", m, 1e-5, window=11)[0], y)
    assert not torch.allclose(plain.latent_attention(h, w, "l0.mix.", m, 1e-5, window=10)[0][10], y[10])


def test_router_and_experts():
    cfg, w = _one_layer(bm.windowed(mlp=bm.feed_forward("moe", experts=4, top=4, scale=1.0, shared=None)))
    h = _rand(3, cfg["width"])
    mlp = cfg["layers"][0]["mlp"]
    idx, wt = plain.route(h, w["l0.mlp.router"], 2, 3.0)
    s = torch.softmax(h @ w["l0.mlp.router"].T, -1)
    assert idx[0].tolist() == s[0].argsort(descending=True)[:2].tolist()
    assert torch.allclose(wt, 3.0 * s.gather(1, idx)) and float(wt[0].sum()) < 3.0          # not renormalised
    # every expert chosen: the softmax-weighted sum of all of them
    want = sum(s[:, e:e + 1] * plain.gated_ff(h, w, f"l0.mlp.e{e}.", plain.silu) for e in range(4))
    assert torch.allclose(plain.expert_ff(h, w, "l0.mlp.", mlp), want)
    z = torch.tensor([-1.0, 0.0, 2.0], dtype=F64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(plain.silu(z), torch.nn.functional.silu(z))


def test_a_layer_that_reads_another_layers_latent():
    cfg = bm.config([bm.windowed(window=4, mlp=None), bm.windowed(heads=3, dim=6, vdim=4, window=7, kv_from=0, mlp=None)])
    w = {k: v.to(F64) for k, v in bm.make_weights(cfg, 2, torch.float32).items()}
    assert "l1.mix.dkv" not in w and "l1.mix.dkv.norm" not in w and "l1.mix.uk" in w
    ids = list(range(12))
    _, after = plain.forward(cfg, w, ids, return_layers=True)
    # layer 1 by hand from layer 0's latent
    x0 = after[0]
    h0 = plain.norm_centered(w["embed"][ids] * 2.5, w["l0.norm1"], 1e-5)
    lat = plain.latent_of(h0, w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    h1 = plain.norm_centered(x0, w["l1.norm1"], 1e-5)
    y, _ = plain.latent_attention(h1, w, "l1.mix.", cfg["layers"][1]["mixer"], 1e-5, lat, 7)
    assert torch.allclose(after[1], x0 + plain.norm_centered(y, w["l1.norm1b"], 1e-5))


@pytest.mark.parametrize("sharp", [4.0, 8.0])
def test_the_sharp_configurations_show_a_key_too_few_or_too_many(sharp):
    """What the window tests rest on: with these weights the plain model itself moves by far more than the tolerance
    when a window is one key shorter or longer."""
    cfg = bm.config([bm.windowed(window=17, sharp=sharp, mlp=None)])
    weights = {k: v.float() for k, v in bm.make_weights(cfg, 3, torch.float32).items()}
    ids = torch.randint(0, cfg['vocab'], (60,), generator=torch.Generator().manual_seed(1)).tolist()
    ref = plain.forward(cfg, weights, ids)
    for delta in (-1, 1):
        other = copy.deepcopy(cfg)
        other["layers"][0]["mixer"]["mask"]["size"] += delta
        moved = plain.forward(other, weights, ids)
        rel = ((moved - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean(-1).sqrt())[20:]
        assert float(rel.max()) > 50 * 2e-4 and float((rel > 10 * 2e-4).float().mean()) > 0.15


def test_config_reader_names_and_cache_specs():
    from llmengine.config import ConfigError, parse_config
    from llmengine.config.registry import resolve
    cfg = parse_config(bm.MIXED)
    assert cfg.architecture == "Bidirax" and cfg.embedding_scale == 2.5 and len(cfg.layers) == 5
    assert cfg.layers[3].mixer["kv_from"] == 1 and cfg.layers[2].mlp is None and cfg.layers[3].mlp["shared_ff"] is None
    model = resolve("Bidirax").build_model(cfg)
    names = set(model.named_specs())
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm1b", "l0.norm2b", "l0.mix.dq.norm", "l0.mix.dkv", "l1.mlp.router",
            "l1.mlp.e4.down", "l1.mlp.shared.up", "l3.mix.uk"} <= names
    assert not {"l3.mix.dkv", "l3.mix.dkv.norm", "l2.norm2", "l2.mlp.gate", "l3.mlp.shared.gate"} & names
    specs = model.cache_specs()
    assert sorted(specs) == [0, 1, 2, 4]
    # layer 1 keeps what the wider window of layer 3, which reads its rows, reaches
    assert (specs[1].kind, specs[1].window) == ("window", 13) and specs[0].kind == "full"
    assert specs[1].paged["rows"] == (-1, 12) and specs[0].paged["rows"] == (-1, 28)
    assert [c.cache_id for c in model.schedule] == [0, 1, 2, 1, 4] and not model.schedule[3].write_cache
    for path, value, text in [(("layers", 1, "mixer", "mask"), None, "mask"), (("layers", 3, "mixer", "kv_from"), 3, "earlier"),
                              (("layers", 0, "type"), "attention", "none of"), (("layers", 0, "mixer", "rot", "dims"), 10, "dims"),
                              (("layers", 1, "mlp", "router", "top"), 9, "top"), (("layers", 3, "mixer", "kv_rank"), 16, "kv_rank"), (("layers", 3, "mixer", "rot_dim"), 4, "rot"),
                              (("norm",), None, "norm")]:
        bad = copy.deepcopy(bm.MIXED)
        at = bad
        for key in path[:-1]:
            at = at[key]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError, match=text):
            parse_config(bad)
