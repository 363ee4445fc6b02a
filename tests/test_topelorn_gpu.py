"""Topelorn through the engine on the GPU against the plain implementation: whole prompts,
decoding token by token, portions down to two tokens, mixed batches over pools that are used
again, long decoding past every window with pages going back, and greedy generation through
the entry point and its scheduler.  float32 is held to 1e-4; bfloat16 to 3 % of the largest
logit."""
import random

import numpy as np
import pytest
import torch

import plain_topelorn as plain
import replay_schedules as rs
from replay_harness import compare, replay_in_process, replay_program, tolerance
from servelab_amd import CacheConfig, LLMEngine, SamplingParams, SchedulerConfig, load_config
from servelab_amd.engine import ModelRunner
from topelorn_models import MODELS, make_weights, write_folder

pytestmark = pytest.mark.gpu


def reference(cfg, weights, requests):
    return {rid: plain.forward(cfg, weights, toks).float().numpy() for rid, toks in requests.items()}


def make_requests(vocab, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, tag, max_tokens=None, page=16, max_live=4):
    out = str(tmp_path / f"out_{tag}_{dtype}")
    replay_in_process(folder, steps, out, dtype, max_tokens or rs.max_tokens_needed(steps), block_size=page,
                      max_live=max_live)
    worst, where = compare(out, steps, ref, cfg["vocab"])
    bar = tolerance(dtype, ref)
    assert worst < bar, f"{tag}: max abs err {worst} at {where}, bar {bar}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(MODELS))
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, which, dtype):
    cfg = MODELS[which]
    folder, weights = write_folder(tmp_path, cfg, seed=11, tag=which)
    requests = make_requests(cfg["vocab"], [71, 1, 2, 40, 97, 23], seed=5)
    ref = reference(cfg, weights, requests)
    run_and_compare(tmp_path, folder, cfg, rs.whole(requests), ref, dtype, "whole")
    run_and_compare(tmp_path, folder, cfg, rs.tail_decoded(requests, tail=45), ref, dtype, "decode")
    run_and_compare(tmp_path, folder, cfg, rs.portions(requests), ref, dtype, "portions")
    run_and_compare(tmp_path, folder, cfg, rs.portions(requests, sizes=(2, 2, 3, 2, 64, 2)), ref, dtype, "twos")
    prompt_lens = {rid: max(1, len(t) - 20) for rid, t in requests.items()}
    for seed in (1, 2):
        steps = rs.mixed(requests, prompt_lens, max_live=3, seed=seed)
        run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, f"mixed{seed}")


@pytest.mark.parametrize("page", [16, 32, 64])
def test_pages_and_slots_are_used_again(tmp_path, page):
    """A pool no larger than the live requests need at their peak, four slots, ten requests one after the
    other and side by side: every page and slot serves several requests."""
    cfg = MODELS["A"]
    folder, weights = write_folder(tmp_path, cfg, seed=12, tag="A")
    requests = make_requests(cfg["vocab"], [50, 33, 80, 5, 64, 17, 129, 48, 2, 70], seed=6)
    ref = reference(cfg, weights, requests)
    prompt_lens = {rid: len(t) // 2 for rid, t in requests.items()}
    steps = rs.mixed(requests, prompt_lens, max_live=4, seed=3, max_portion=40)
    run_and_compare(tmp_path, folder, cfg, steps, ref, "float32", f"reuse{page}",
                    max_tokens=rs.max_tokens_needed(steps, max(64, page)), page=page, max_live=4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_past_every_window(tmp_path, dtype, monkeypatch):
    """Two requests decoded for 330 tokens through captured graphs whose capacity is outgrown twice; the
    windows (9 to 40 keys) pass over prompt and decoded tokens alike, pages behind them go back."""
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 128)
    cfg = MODELS["A"]
    folder, weights = write_folder(tmp_path, cfg, seed=13, tag="A")
    requests = make_requests(cfg["vocab"], [350, 341], seed=7)
    ref = reference(cfg, weights, requests)
    a, b = requests["r0"], requests["r1"]
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": a[:20], "want": [0, 19]},
                                     {"id": "r1", "tokens": b[:11], "want": [10]}], "end": []}]
    for i in range(330):
        steps.append({"step": i + 1, "entries": [{"id": "r0", "tokens": [a[20 + i]], "want": [0]},
                                                 {"id": "r1", "tokens": [b[11 + i]], "want": [0]}],
                      "end": ["r0", "r1"] if i == 329 else []})
    run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, "long")


def test_a_far_kept_token_decides_the_logits(tmp_path):
    """The first layer's weights are set so that every query looks at token 0 alone when it can (it is
    kept by keep_first, hundreds of tokens back) and token 0's value is large: dropping the kept tokens,
    or giving their page away, changes every logit."""
    cfg = {"architecture": "Topelorn", "width": 64, "vocab": 200, "norm": {"eps": 1e-5}, "layers": [
        {"type": "attention", "mlp": None,
         "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 24, "scale": 4.0,
                   "mask": {"size": 6, "keep_first": 1}, "v_mix": False}}]}
    weights = make_weights(cfg, 21)
    weights["l0.mix.sink"] = torch.full((2,), -20.0)
    folder, weights = write_folder(tmp_path, cfg, seed=21, tag="far", weights=weights)
    requests = make_requests(cfg["vocab"], [300], seed=8)
    full = reference(cfg, weights, requests)
    blind = dict(cfg, layers=[dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"],
                                                                   mask={"size": 6, "keep_first": 0}))])
    lost = reference(blind, weights, requests)
    assert np.abs(full["r0"][250:] - lost["r0"][250:]).max() > 0.05      # the kept token matters
    for name, steps in (("whole", rs.whole(requests)), ("decode", rs.tail_decoded(requests, tail=60)),
                        ("twos", rs.portions(requests, sizes=(33, 2, 64, 2, 2)))):
        run_and_compare(tmp_path, folder, cfg, steps, full, "float32", name)


def test_the_program_replays_a_trace(tmp_path):
    cfg = MODELS["C"]
    folder, weights = write_folder(tmp_path, cfg, seed=14, tag="C")
    requests = make_requests(cfg["vocab"], [30, 9], seed=9)
    ref = reference(cfg, weights, requests)
    steps = rs.tail_decoded(requests, tail=5)
    out = str(tmp_path / "out_prog")
    replay_program(folder, steps, out, "float32", rs.max_tokens_needed(steps))
    worst, where = compare(out, steps, ref, cfg["vocab"])
    assert worst < 1e-4, (worst, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_entry_point(tmp_path, which, dtype):
    cfg = MODELS[which]
    folder, weights = write_folder(tmp_path, cfg, seed=15, tag=which)
    prompts = list(make_requests(cfg["vocab"], [30, 4, 77, 1], seed=10).values())
    new = 24
    for budget, blocks in ((256, 64), (8, 64), (64, 24)):
        if dtype == "bfloat16" and budget != 256:
            continue
        engine = LLMEngine(load_config(folder), CacheConfig(num_blocks=blocks),
                           SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=budget), dtype=dtype)
        outs = engine.generate(prompts, SamplingParams.greedy(new))
        engine.runner.manager.check()
        for p, o in zip(prompts, outs):
            toks = o.outputs[0].token_ids
            assert o.finished and len(toks) == new
            logits = plain.forward(cfg, weights, list(p) + toks)
            slack = 1e-3 if dtype == "float32" else 2 * tolerance(dtype, {"x": logits.numpy()})
            for i, t in enumerate(toks):
                row = logits[len(p) - 1 + i]
                assert row[t] >= row.max() - slack, f"token {i}: {float(row[t])} vs best {float(row.max())}"


def test_command_line_samples_from_a_random_model(tmp_path, capsys):
    """bin/run_engine's entry with this design's config.json, seeded random weights made on the device,
    and a temperature with top-k and top-p cuts."""
    import json
    from servelab_amd import cli
    path = tmp_path / "config.json"
    path.write_text(json.dumps(MODELS["B"]))
    assert cli.main(["--config", str(path), "--random-weights", "3", "--prompt-ids", "5,6,7,8", "--max-tokens", "9",
                     "--temperature", "0.8", "--top-k", "20", "--top-p", "0.9", "--max-num-seqs", "4"]) == 0
    assert "finish=length" in capsys.readouterr().out
