"""Rilonex on the GPU against the plain implementation (tests/plain_rilonex.py): every mixer alone and
together, under every way of cutting requests into steps, in 32-bit and in bfloat16."""
from __future__ import annotations

import copy

import numpy as np
import pytest
import torch

import plain_rilonex as plain
import replay
import rilonex_models as rm

pytestmark = pytest.mark.gpu

F32_TOL = 2e-4          # of a row's root mean square; honest 32-bit arithmetic is at 1e-5
# bfloat16 against the unrounded plain model: these narrow models with weights of order one move by 1 % of a row's
# root mean square on average and by up to 10 % in single rows (the same rows under every schedule); a fault of a
# kernel moves rows by their whole size. What a schedule changes is held much tighter, against the whole prompts' rows.
BF16_MEAN, BF16_WORST, BF16_BETWEEN_SCHEDULES = 3e-2, 0.25, 2e-2


def _engine(tmp_path, cfg, seed, dtype, weights=None, **kw):
    from llmengine import Engine
    store = torch.float32 if dtype == "fp32" else torch.bfloat16
    folder, weights = rm.write_model(tmp_path, cfg, seed, store, weights)
    return Engine(folder, dtype, deterministic=True, **kw), weights


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _reference(cfg, weights, requests):
    return {rid: plain.forward(cfg, weights, ids)[0].numpy() for rid, ids in requests.items()}


def _worst(got: dict, ref: dict) -> float:
    worst = 0.0
    for rid, rows in got.items():
        for pos, row in rows.items():
            want = ref[rid][pos]
            worst = max(worst, float(np.sqrt(np.mean((row - want) ** 2)) / np.sqrt(np.mean(want ** 2))))
    return worst


def _mean(got: dict, ref: dict) -> float:
    errs = [float(np.sqrt(np.mean((row - ref[rid][pos]) ** 2)) / np.sqrt(np.mean(ref[rid][pos] ** 2)))
            for rid, rows in got.items() for pos, row in rows.items()]
    return float(np.mean(errs))


def _covered(got: dict, requests: dict) -> bool:
    return all(sorted(got[rid]) == list(range(len(ids))) for rid, ids in requests.items())


ONE_LAYER = {
    "rglru": rm.config([rm.rglru(ff=None)], streams=None),
    "rglru_one_block_two_taps": rm.config([rm.rglru(width=40, blocks=1, conv=2, ff=None)], streams=None),
    "channel_delta": rm.config([rm.channel_delta(ff=None)], streams=None),
    "channel_delta_one_key_head": rm.config([rm.channel_delta(heads=3, kv_heads=1, dim=40, vdim=72, conv=5, ff=None)],
                                            streams=None),
    "parallel": rm.config([rm.parallel(ff=None)], streams=None),
    "parallel_no_rotation_left_only": rm.config([rm.parallel(rot_dims=0, right_scale=0.0, ff=None)], streams=None),
    "parallel_right_only": rm.config([rm.parallel(left_scale=0.0, ff=None)], streams=None),
    "parallel_key_size_of_20": rm.config([rm.parallel(heads=3, kv_heads=3, dim=20, vdim=12, rot_dims=10, ff=None)], streams=None),
    "feed_forward_and_streams": rm.config([rm.rglru(width=16, blocks=2, ff=56)], streams=4),
    "one_stream": rm.config([rm.channel_delta(ff=32)], streams=1),
    "width_of_30": rm.config([rm.rglru(width=18, blocks=3, ff=14), rm.parallel(heads=2, kv_heads=1, dim=6, vdim=10, rot_dims=4, d_heads=1,
                                                                             d_kv=1, d_dim=6, d_vdim=10, ff=None)],
                             width=30, vocab=33, streams=3),
    "five_streams": rm.config([rm.rglru(width=16, blocks=1, ff=24), rm.channel_delta(ff=24)], streams=5),
    "one_tap_and_wide_keys": rm.config([rm.channel_delta(heads=2, kv_heads=1, dim=136, vdim=8, conv=1, ff=None),
                                        rm.rglru(width=24, blocks=2, conv=1, ff=None)], streams=None),
}


@pytest.mark.parametrize("name", sorted(ONE_LAYER))
def test_each_mechanism_alone_whole_and_token_by_token(tmp_path, name):
    cfg = ONE_LAYER[name]
    engine, weights = _engine(tmp_path, cfg, 3, "fp32")
    requests = {"a": _tokens(37, cfg["vocab"], 1), "b": _tokens(1, cfg["vocab"], 2)}
    ref = _reference(cfg, weights, requests)
    for steps in (replay.whole(requests), replay.tail_one_by_one(requests, tail=36), replay.portions(requests)):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 8) // 8 + 1, 8, 2)
        got = replay.run_trace(engine, cache, steps)
        assert _covered(got, requests)
        assert _worst(got, ref) < F32_TOL


@pytest.mark.parametrize("name", ["width_of_30", "parallel_key_size_of_20", "one_tap_and_wide_keys", "five_streams"])
def test_sizes_that_no_fast_kernel_takes_in_bfloat16(tmp_path, name):
    """Widths, key sizes and stream counts that fall outside the vector and matrix-core kernels' limits, served in bfloat16:
    the plain kernels carry them, whole prompts and single tokens agree, and both are the plain model's within rounding."""
    cfg = ONE_LAYER[name]
    engine, weights = _engine(tmp_path, cfg, 4, "bf16")
    requests = {"a": _tokens(45, cfg["vocab"], 1), "b": _tokens(3, cfg["vocab"], 2)}
    ref = _reference(cfg, {k: v.float() for k, v in weights.items()}, requests)
    whole = replay.run_trace(engine, engine.new_cache(8, 16, 2), replay.whole(requests))
    tail = replay.run_trace(engine, engine.new_cache(8, 16, 2), replay.tail_one_by_one(requests, tail=40))
    assert _covered(whole, requests) and _covered(tail, requests)
    assert _mean(whole, ref) < BF16_MEAN and _worst(whole, ref) < BF16_WORST
    assert _worst(tail, {rid: np.stack([whole[rid][p] for p in sorted(whole[rid])]) for rid in requests}) < BF16_BETWEEN_SCHEDULES


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("cfg_name", ["MIXED", "ALIGNED", "PLAIN"])
def test_every_schedule_gives_the_plain_logits(tmp_path, cfg_name, dtype):
    cfg = getattr(rm, cfg_name)
    engine, weights = _engine(tmp_path, cfg, 11, dtype)
    V = cfg["vocab"]
    requests = {"long": _tokens(150, V, 5), "one": _tokens(1, V, 6), "two": _tokens(2, V, 7), "mid": _tokens(49, V, 8),
                "page": _tokens(32, V, 9), "more": _tokens(65, V, 10)}
    ref = _reference(cfg, {k: v.float() for k, v in weights.items()}, requests)
    schedules = {
        "whole": replay.whole(requests),
        "tail": replay.tail_one_by_one(requests, tail=40),
        "portions": replay.portions(requests),
        "portions of two": replay.portions(requests, sizes=(2,)),
        "mixed": replay.mixed(requests, max_live=3, seed=1),
        "mixed, other cuts": replay.mixed(requests, max_live=2, sizes=(2, 17, 3, 31), seed=2),
    }
    first = None
    for what, steps in schedules.items():
        for page in (16, 8):
            # as many pages as the live requests need and three slots: pages and slots are used again
            cache = engine.new_cache(replay.trace_peak_tokens(steps, page) // page, page, 3)
            got = replay.run_trace(engine, cache, steps)
            assert _covered(got, requests), what
            if dtype == "fp32":
                assert _worst(got, ref) < F32_TOL, (what, page)
            else:
                assert _mean(got, ref) < BF16_MEAN and _worst(got, ref) < BF16_WORST, (what, page)
                first = first or {rid: np.stack([rows[p] for p in sorted(rows)]) for rid, rows in got.items()}
                assert _worst(got, first) < BF16_BETWEEN_SCHEDULES, (what, page)
            assert not cache.manager.live_requests()


def test_a_slot_that_is_used_again_starts_from_nothing(tmp_path):
    """One slot, one request after the other: what the first left in the recurrent states, the convolutions'
    tails and the pages must not reach the second."""
    cfg = rm.MIXED
    engine, weights = _engine(tmp_path, cfg, 12, "fp32")
    cache = engine.new_cache(8, 16, 1)
    first, second = _tokens(100, cfg["vocab"], 1), _tokens(90, cfg["vocab"], 2)
    ref = _reference(cfg, weights, {"second": second})
    replay.run_trace(engine, cache, replay.tail_one_by_one({"first": first}, tail=5))
    got = replay.run_trace(engine, cache, replay.portions({"second": second}, sizes=(1, 1, 2, 40)))
    assert _worst(got, ref) < F32_TOL


def test_a_batch_gives_what_each_request_gives_alone(tmp_path):
    cfg = rm.MIXED
    engine, _ = _engine(tmp_path, cfg, 13, "bf16")
    V = cfg["vocab"]
    requests = {"a": _tokens(70, V, 1), "b": _tokens(9, V, 2), "c": _tokens(33, V, 3), "d": _tokens(2, V, 4)}
    alone = replay.run_trace(engine, engine.new_cache(16, 16, 1), replay.whole(requests))
    from llmengine import StepEntry
    cache = engine.new_cache(16, 16, 4)
    for rid in requests:
        cache.admit(rid)
    # prompts of unequal length in one step, then a portion of one beside single tokens of the others
    heads = {rid: max(1, len(ids) - 3) for rid, ids in requests.items()}
    logits = engine.step(cache, [StepEntry(rid, ids[:heads[rid]], list(range(heads[rid]))) for rid, ids in requests.items()])
    rows = logits.cpu().numpy()
    r = 0
    for rid, ids in requests.items():
        for p in range(heads[rid]):
            want = alone[rid][p]
            assert np.sqrt(np.mean((rows[r] - want) ** 2)) / np.sqrt(np.mean(want ** 2)) < 2e-2, (rid, p)
            r += 1
    entries = [StepEntry("a", requests["a"][heads["a"]:], [0, 1, 2])]
    entries += [StepEntry(rid, [requests[rid][heads[rid]]], [0]) for rid in ("b", "c") if heads[rid] < len(requests[rid])]
    rows = engine.step(cache, entries).cpu().numpy()
    r = 0
    for e in entries:
        for w in e.want:
            want = alone[e.request_id][heads[e.request_id] + w]
            assert np.sqrt(np.mean((rows[r] - want) ** 2)) / np.sqrt(np.mean(want ** 2)) < 2e-2
            r += 1


def _sharp_attention(cfg, weights, far_scale=6.0):
    """Weights under which single keys matter: large scores (weights near 0 or 1) in the attention without softmax."""
    weights = dict(weights)
    for name in weights:
        if name.endswith("left.q") or name.endswith("left.k"):
            weights[name] = (weights[name].float() * far_scale).to(weights[name].dtype)
    return weights


def test_far_keys_and_page_borders_show_in_the_logits(tmp_path):
    """A single attention layer with sharp weights: every position of a long prompt is checked, with prompts cut at
    and beside page borders and decoding across them, so a key lost at a border or far back changes a checked row.
    That a lost key would show is checked on the plain implementation first: another first token moves the last
    row by far more than the tolerance."""
    cfg = rm.config([rm.parallel(heads=4, kv_heads=2, dim=16, vdim=16, rot_dims=8, scale=0.5, right_scale=0.0, ff=None)],
                    streams=None, width=32)
    weights = _sharp_attention(cfg, rm.make_weights(cfg, 21, torch.float32))
    ids = _tokens(300, cfg["vocab"], 3)
    ref = plain.forward(cfg, weights, ids)[0].numpy()
    # the plain model itself: with another first token, the last row differs by that one key and value, 299 back
    other = [(ids[0] + 1) % cfg["vocab"]] + ids[1:]
    moved = plain.forward(cfg, weights, other)[0].numpy()[-1] - ref[-1]
    assert np.sqrt(np.mean(moved ** 2)) / np.sqrt(np.mean(ref[-1] ** 2)) > 100 * F32_TOL
    engine, _ = _engine(tmp_path, cfg, 21, "fp32", weights=weights)
    requests = {"r": ids}
    for sizes in ((15, 1, 1, 16, 17, 31, 2, 64, 1, 1, 1, 1), (16, 16, 1, 47, 33, 1, 1), (255, 1, 1, 1, 1)):
        steps = replay.portions(requests, sizes=sizes)
        cache = engine.new_cache(19, 16, 1)
        got = replay.run_trace(engine, cache, steps)
        assert _worst(got, {"r": ref}) < F32_TOL, sizes


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(8, 2, 64, 48), (16, 16, 32, 128), (4, 1, 128, 16)])
def test_the_matrix_core_attention_agrees_with_the_plain_kernel(tmp_path, heads, kv_heads, dim, vdim):
    """bfloat16 steps take the matrix-core kernel of the attention without softmax unless an engine is told not to: the same
    positions through both agree far below bfloat16's own rounding (they read the same rounded q, k and v and compute in
    32-bit), and both are the plain model's within that rounding. Requests of 100, 16 and 37 rows in one step, portions
    that start in the middle of a page, keys cut into several runs."""
    cfg = rm.config([rm.parallel(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, rot_dims=32, scale=0.4, right_scale=0.0,
                                 ff=None)], streams=None, width=64)
    weights = _sharp_attention(cfg, rm.make_weights(cfg, 22, torch.bfloat16), far_scale=3.0)
    engine, _ = _engine(tmp_path, cfg, 22, "bf16", weights=weights)
    V = cfg["vocab"]
    requests = {"a": _tokens(700, V, 1), "b": _tokens(16, V, 2), "c": _tokens(37, V, 3)}
    ref = _reference(cfg, {k: v.float() for k, v in weights.items()}, requests)
    from llmengine import StepEntry
    cache = engine.new_cache(60, 16, 3)
    for rid in requests:
        cache.admit(rid)
    fast = {}
    rows = engine.step(cache, [StepEntry(rid, ids[:len(ids) // 2 + 3], list(range(len(ids) // 2 + 3)))
                               for rid, ids in requests.items()]).cpu().numpy()
    r = 0
    for rid, ids in requests.items():
        n = len(ids) // 2 + 3
        fast[rid] = {p: rows[r + p].copy() for p in range(n)}
        r += n
    rows = engine.step(cache, [StepEntry(rid, ids[len(ids) // 2 + 3:], list(range(len(ids) - len(ids) // 2 - 3)))
                               for rid, ids in requests.items() if len(ids) - len(ids) // 2 - 3 > 0]).cpu().numpy()
    r = 0
    for rid, ids in requests.items():
        n0 = len(ids) // 2 + 3
        for p in range(n0, len(ids)):
            fast[rid][p] = rows[r].copy()
            r += 1
    for rid in requests:
        cache.release(rid)
    from llmengine.ops import KernelChoices
    plain_engine, _ = _engine(tmp_path / "plain", cfg, 22, "bf16", weights=weights, kernel_choices=KernelChoices(fast_attention=False))
    slow = replay.run_trace(plain_engine, plain_engine.new_cache(60, 16, 3), replay.portions(requests, sizes=(7, 5, 15, 2, 11)))
    small = replay.run_trace(engine, cache, replay.portions(requests, sizes=(1, 3, 16, 2, 40)))      # tiles of a few rows
    assert _worst(small, {rid: np.stack([slow[rid][p] for p in range(len(ids))]) for rid, ids in requests.items()}) < 3e-3
    assert _covered(fast, requests) and _covered(slow, requests)
    assert _worst(fast, {rid: np.stack([slow[rid][p] for p in range(len(ids))]) for rid, ids in requests.items()}) < 3e-3
    assert _mean(fast, ref) < BF16_MEAN and _worst(fast, ref) < BF16_WORST


def test_long_decoding_keeps_the_states(tmp_path):
    """300 tokens one by one after a short prompt (recorded decode steps replayed): the recurrent states and the
    convolutions' tails are carried in 32-bit without drift."""
    cfg = rm.MIXED
    engine, weights = _engine(tmp_path, cfg, 14, "fp32")
    ids = _tokens(310, cfg["vocab"], 4)
    ref = _reference(cfg, weights, {"r": ids})
    steps = replay.tail_one_by_one({"r": ids}, tail=300)
    got = replay.run_trace(engine, engine.new_cache(20, 16, 2), steps)
    assert _covered(got, {"r": ids}) and _worst(got, ref) < F32_TOL
    assert engine.runner.graph_replays >= 299


def test_first_tokens_of_a_sequence(tmp_path):
    """The first tokens see zeros in front of every convolution and an empty memory: prompts of 1 to 6 tokens, whole and
    one by one, against the plain model (convolutions of up to five taps reach back before the start in all of them)."""
    cfg = rm.MIXED
    engine, weights = _engine(tmp_path, cfg, 15, "fp32")
    requests = {f"n{n}": _tokens(n, cfg["vocab"], 30 + n) for n in range(1, 7)}
    ref = _reference(cfg, weights, requests)
    for steps in (replay.whole(requests), replay.tail_one_by_one(requests, tail=8), replay.mixed(requests, max_live=4, seed=3)):
        got = replay.run_trace(engine, engine.new_cache(8, 16, 4), steps)
        assert _worst(got, ref) < F32_TOL


def test_greedy_generation_through_the_entry_point_and_the_scheduler(tmp_path):
    cfg = rm.MIXED
    engine, weights = _engine(tmp_path, cfg, 16, "fp32")
    prompts = [_tokens(9, cfg["vocab"], 1), _tokens(30, cfg["vocab"], 2), _tokens(1, cfg["vocab"], 3)]
    new = 12

    def plain_greedy(ids):
        ids = list(ids)
        for _ in range(new):
            ids.append(int(plain.forward(cfg, weights, ids)[0][-1].argmax()))
        return ids

    want = [plain_greedy(p) for p in prompts]
    for p, w in zip(prompts, want):
        out, finish = engine.generate(p, new)
        assert out == w and finish == "length"
    from llmengine import BlockManager, ContinuousBatchScheduler
    sched = ContinuousBatchScheduler(engine, BlockManager(num_blocks=12, block_size=16), max_concurrent=2,
                                     max_prefill_tokens_per_step=16)
    for p in prompts:
        sched.enqueue(p, new)
    sched.run_until_idle()
    assert [r.token_ids for r in sched.results] == want


def test_a_model_without_pages_generates_again_and_again(tmp_path):
    """Recurrent layers only: no mixer keeps pages, the engine's own pool and the scheduler's have nothing to count."""
    cfg = rm.PLAIN
    engine, weights = _engine(tmp_path, cfg, 20, "fp32")
    prompt = _tokens(7, cfg["vocab"], 1)
    want = list(prompt)
    for _ in range(4):
        want.append(int(plain.forward(cfg, weights, want)[0][-1].argmax()))
    for _ in range(3):
        assert engine.generate(prompt, 4)[0] == want
    from llmengine import BlockManager, ContinuousBatchScheduler
    blocks = BlockManager(num_blocks=4, block_size=16)
    sched = ContinuousBatchScheduler(engine, blocks, max_concurrent=2, max_prefill_tokens_per_step=8)
    for _ in range(3):
        sched.enqueue(prompt, 4)
    sched.run_until_idle()
    assert [r.token_ids for r in sched.results] == [want] * 3 and blocks.free_blocks == 4


@pytest.mark.parametrize("dtype", ["bf16"])
def test_thirty_two_heads_on_the_matrix_cores(tmp_path, dtype):
    """32 query heads: eight wavefronts a workgroup and more LDS than a kernel gets without asking."""
    cfg = rm.config([rm.parallel(heads=32, kv_heads=8, dim=32, vdim=16, rot_dims=32, scale=0.4, right_scale=0.0, ff=None)],
                    streams=None, width=64)
    weights = _sharp_attention(cfg, rm.make_weights(cfg, 23, torch.bfloat16), far_scale=3.0)
    engine, _ = _engine(tmp_path, cfg, 23, dtype, weights=weights)
    requests = {"a": _tokens(200, cfg["vocab"], 1), "b": _tokens(21, cfg["vocab"], 2)}
    ref = _reference(cfg, {k: v.float() for k, v in weights.items()}, requests)
    whole = replay.run_trace(engine, engine.new_cache(16, 16, 2), replay.whole(requests))
    tail = replay.run_trace(engine, engine.new_cache(16, 16, 2), replay.tail_one_by_one(requests, tail=20))
    assert _mean(whole, ref) < BF16_MEAN and _worst(whole, ref) < BF16_WORST
    assert _worst(tail, {rid: np.stack([whole[rid][p] for p in sorted(whole[rid])]) for rid in requests}) < 3e-3


def test_the_models_trace_runner_replays_a_random_model(tmp_path):
    """bin/trace_run on a model folder of this design: mixed steps, four slots, logits as files."""
    import json
    import os
    import subprocess
    import sys
    cfg = rm.PLAIN
    folder, weights = rm.write_model(tmp_path / "model", cfg, 17, torch.float32)
    requests = {"a": _tokens(40, cfg["vocab"], 1), "b": _tokens(21, cfg["vocab"], 2)}
    steps = replay.mixed(requests, max_live=2, seed=5)
    ref = _reference(cfg, weights, requests)
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", str(replay.trace_peak_tokens(steps))],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    done = {rid: 0 for rid in requests}
    for s in steps:
        rows = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        r = 0
        for e in s["entries"]:
            for w in e["want"]:
                want = ref[e["id"]][done[e["id"]] + w]
                assert np.sqrt(np.mean((rows[r] - want) ** 2)) / np.sqrt(np.mean(want ** 2)) < F32_TOL
                r += 1
            done[e["id"]] += len(e["tokens"])


def test_the_command_line_generates_with_a_model_of_this_design(tmp_path):
    """bin/llmengine-cli: greedy tokens of a model folder as the plain model chooses them, and sampling from a configuration
    with random weights (which goes through the framework's own random initial values for this design's tensors)."""
    import json
    import os
    import subprocess
    import sys
    cfg = rm.MIXED
    folder, weights = rm.write_model(tmp_path / "model", cfg, 19, torch.float32)
    prompt = _tokens(11, cfg["vocab"], 1)
    want = list(prompt)
    for _ in range(5):
        want.append(int(plain.forward(cfg, weights, want)[0][-1].argmax()))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "llmengine-cli"), "--model", folder, "--dtype", "fp32",
                          "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert rec["token_ids"] == want and rec["finish_reason"] == "length"
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps(rm.ALIGNED))
    pf = tmp_path / "prompts.txt"
    pf.write_text("1 2 3\n7,8,9,10,11\n")
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "llmengine-cli"), "--random", str(cfgf), "--seed", "3",
                          "--prompt-file", str(pf), "--max-new-tokens", "4", "--temperature", "0.7"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    recs = [json.loads(line) for line in out.stdout.strip().splitlines()]
    assert [len(r["token_ids"]) for r in recs] == [7, 9] and all(r["finish_reason"] == "length" for r in recs)


def test_weights_with_a_rank_that_only_the_file_names(tmp_path):
    """The two-stage maps' inner sizes are read off the tensors when the configuration does not name them."""
    layer = rm.channel_delta(ff=None)
    cfg = rm.config([layer], streams=None)
    weights = rm.make_weights(cfg, 18, torch.float32)
    bare = copy.deepcopy(cfg)
    for key in ("decay_rank", "gate_rank"):
        del bare["layers"][0]["mixer"][key]
    engine, _ = _engine(tmp_path, bare, 18, "fp32", weights=weights)
    ids = _tokens(20, cfg["vocab"], 1)
    got = engine.forward_logits(ids)
    ref = plain.forward(cfg, weights, ids)[0].numpy()
    assert np.abs(got - ref).max() / np.abs(ref).max() < F32_TOL
