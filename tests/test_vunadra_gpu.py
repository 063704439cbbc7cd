"""Vunadra through the engine on the GPU against the plain implementation: whole prompts, decoding
token by token, portions down to two tokens, mixed batches over pools and state slots that are
used again, long decoding through captured graphs, mixers whose output hangs on one marked token
(far back, at page borders, just inside and just outside a window), the replay program, and
greedy generation through the entry point and its scheduler."""
import random

import numpy as np
import pytest
import torch

import plain_vunadra as plain
import replay_schedules as rs
from replay_harness import compare, replay_in_process, replay_program
from servelab_amd import CacheConfig, LLMEngine, SamplingParams, SchedulerConfig, load_config
from servelab_amd.engine import ModelRunner
from vunadra_models import (MODELS, config, conv_attention, key_value_attention, latent, make_weights, rot,
                            write_folder)

pytestmark = pytest.mark.gpu


def reference(cfg, weights, requests):
    return {rid: plain.forward(cfg, weights, toks).float().numpy() for rid, toks in requests.items()}


def make_requests(vocab, lengths, seed, avoid=()):
    rng = random.Random(seed)
    ids = [t for t in range(vocab) if t not in avoid]
    return {f"r{i}": [rng.choice(ids) for _ in range(n)] for i, n in enumerate(lengths)}


def bar(dtype, ref):
    """float32: 2e-4 of the logits' range; bfloat16: 3 % of it (weights, projections, expert
    activations and pages rounded to 8 bits of mantissa)."""
    top = max(1.0, max(float(np.abs(r).max()) for r in ref.values()))
    return (2e-4 if dtype == "float32" else 0.03) * top


def emulated_bfloat16(tmp_path, folder, cfg, requests, ref):
    """(median, share of rows over the bar) of the row errors of a CPU computation that rounds to
    bfloat16 where the kernels do (tests/emulated_ops.py), every request whole: what rounding alone
    does to this model (repeated layers multiply it)."""
    from emulated_ops import EmulatedOps
    steps = rs.whole(requests)
    out = str(tmp_path / "out_emulated")
    replay_in_process(folder, steps, out, "bfloat16", rs.max_tokens_needed(steps), ops=EmulatedOps(torch.bfloat16),
                      device="cpu", max_live=max(16, len(requests)))
    errors = []
    compare(out, steps, ref, cfg["vocab"],
            score=lambda got, want: errors.append(float(np.abs(got - want).max())) or 0.0)
    errors = np.asarray(errors)
    return float(np.median(errors)), float((errors > bar("bfloat16", ref)).mean())


def run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, tag, max_tokens=None, page=16, max_live=4,
                    float32_bar=None, emulated=(0.0, 0.0)):
    """float32: every row within the bar.  bfloat16: a router's choice between two experts of
    nearly equal shares can fall the other way under rounding; so at most one row in four may lie
    over the bar, and the typical row (the median) must lie under a third of it, or, for a model
    that rounding alone moves further (``emulated``), no further than 1.5 times what rounding
    does.  The kernels' own bfloat16 tests are tight."""
    out = str(tmp_path / f"out_{tag}_{dtype}")
    replay_in_process(folder, steps, out, dtype, max_tokens or rs.max_tokens_needed(steps), block_size=page,
                      max_live=max_live)
    limit = bar(dtype, ref)
    if dtype == "float32":
        limit = max(limit, float32_bar or 0.0)
        worst, where = compare(out, steps, ref, cfg["vocab"])
        assert worst < limit, f"{tag}: max abs err {worst} at {where}, bar {limit}"
        return
    errors = []
    compare(out, steps, ref, cfg["vocab"],
            score=lambda got, want: errors.append(float(np.abs(got - want).max())) or 0.0)
    errors = np.asarray(errors)
    middle, over = max(limit / 3, 1.5 * emulated[0]), max(1 / 4, emulated[1] + 0.15)
    assert np.median(errors) < middle, f"{tag}: median row error {np.median(errors)}, bar {middle}"
    assert (errors > limit).mean() <= over, f"{tag}: {(errors > limit).mean():.3f} of the rows over {limit}"


def plain_float32_loss(cfg, weights, requests, ref):
    """Twice what the plain implementation itself loses in float32."""
    plain.F = torch.float32
    try:
        return 2.0 * max(float(np.abs(plain.forward(cfg, weights, toks).double().numpy() - ref[rid]).max())
                         for rid, toks in requests.items())
    finally:
        plain.F = torch.float64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(set(MODELS) - {"F"}))
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, which, dtype):
    cfg = MODELS[which]
    folder, weights = write_folder(tmp_path, cfg, seed=11, tag=which)
    requests = make_requests(cfg["vocab"], [71, 1, 2, 40, 97, 23], seed=5)
    ref = reference(cfg, weights, requests)
    kw = {"float32_bar": plain_float32_loss(cfg, weights, requests, ref)}
    if dtype == "bfloat16":
        kw["emulated"] = emulated_bfloat16(tmp_path, folder, cfg, requests, ref)
    run_and_compare(tmp_path, folder, cfg, rs.whole(requests), ref, dtype, "whole", **kw)
    run_and_compare(tmp_path, folder, cfg, rs.tail_decoded(requests, tail=45), ref, dtype, "decode", **kw)
    run_and_compare(tmp_path, folder, cfg, rs.portions(requests), ref, dtype, "portions", **kw)
    run_and_compare(tmp_path, folder, cfg, rs.portions(requests, sizes=(2, 2, 3, 2, 64, 2)), ref, dtype, "twos", **kw)
    prompt_lens = {rid: max(1, len(t) - 20) for rid, t in requests.items()}
    for seed in (1, 2):
        steps = rs.mixed(requests, prompt_lens, max_live=3, seed=seed)
        run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, f"mixed{seed}", max_live=3, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_of_the_widest_model(tmp_path, dtype):
    """Prompts of several hundred tokens: many pages a request, steps of enough rows for every product
    kernel and row tiles of every height, the attentions on the matrix cores in bfloat16, windows that
    release pages."""
    cfg = MODELS["F"]
    folder, weights = write_folder(tmp_path, cfg, seed=16, tag="F")
    requests = make_requests(cfg["vocab"], [613, 190], seed=12)
    ref = reference(cfg, weights, requests)
    kw = {"float32_bar": plain_float32_loss(cfg, weights, requests, ref)}
    if dtype == "bfloat16":
        kw["emulated"] = emulated_bfloat16(tmp_path, folder, cfg, requests, ref)
    run_and_compare(tmp_path, folder, cfg, rs.whole(requests), ref, dtype, "whole", **kw)
    run_and_compare(tmp_path, folder, cfg, rs.tail_decoded(requests, tail=40), ref, dtype, "decode", **kw)
    run_and_compare(tmp_path, folder, cfg, rs.portions(requests, sizes=(100, 2, 255, 64, 7)), ref, dtype, "portions", **kw)
    steps = rs.mixed(requests, {rid: len(t) - 30 for rid, t in requests.items()}, max_live=2, seed=5, max_portion=130)
    run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, "mixed", max_live=2, **kw)


@pytest.mark.parametrize("page", [16, 32, 64])
def test_pages_and_slots_are_used_again(tmp_path, page):
    """A pool no larger than the live requests need at their peak and three state slots for ten
    requests: every page and slot serves several requests, one after the other and side by side."""
    cfg = MODELS["A"]
    folder, weights = write_folder(tmp_path, cfg, seed=12, tag="A")
    requests = make_requests(cfg["vocab"], [50, 33, 80, 5, 64, 17, 129, 48, 2, 70], seed=6)
    ref = reference(cfg, weights, requests)
    prompt_lens = {rid: len(t) // 2 for rid, t in requests.items()}
    steps = rs.mixed(requests, prompt_lens, max_live=3, seed=3, max_portion=40)
    run_and_compare(tmp_path, folder, cfg, steps, ref, "float32", f"reuse{page}",
                    max_tokens=rs.max_tokens_needed(steps, max(64, page)), page=page, max_live=3,
                    float32_bar=plain_float32_loss(cfg, weights, requests, ref))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_captured_graphs(tmp_path, dtype, monkeypatch):
    """Two requests decoded for 330 tokens: the steps replay captured graphs whose capacity is
    outgrown twice; last inputs and pages are carried from replay to replay, every window is passed."""
    monkeypatch.setattr(ModelRunner, "GRAPH_MIN_CONTEXT", 128)
    cfg = MODELS["C"]
    folder, weights = write_folder(tmp_path, cfg, seed=13, tag="C")
    requests = make_requests(cfg["vocab"], [350, 341], seed=7)
    ref = reference(cfg, weights, requests)
    a, b = requests["r0"], requests["r1"]
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": a[:20], "want": [0, 19]},
                                     {"id": "r1", "tokens": b[:11], "want": [10]}], "end": []}]
    for i in range(330):
        steps.append({"step": i + 1, "entries": [{"id": "r0", "tokens": [a[20 + i]], "want": [0]},
                                                 {"id": "r1", "tokens": [b[11 + i]], "want": [0]}],
                      "end": ["r0", "r1"] if i == 329 else []})
    kw = {"float32_bar": plain_float32_loss(cfg, weights, requests, ref)}
    if dtype == "bfloat16":
        kw["emulated"] = emulated_bfloat16(tmp_path, folder, cfg, requests, ref)
    run_and_compare(tmp_path, folder, cfg, steps, ref, dtype, "long", **kw)


def test_graphs_are_in_use_for_decode_steps(tmp_path):
    cfg = MODELS["A"]
    folder, _ = write_folder(tmp_path, cfg, seed=14, tag="A")
    from servelab_amd.engine.session import load_model_on_device, make_runner
    from servelab_amd.engine import StepEntry
    _, model = load_model_on_device(folder, "bfloat16", "cuda:0")
    runner = make_runner(model, 64, 16, max_num_seqs=4)
    assert model.spec.graph_safe and runner.use_graphs
    runner.step([StepEntry("a", [1, 2, 3], [2])])
    for t in range(6):
        runner.step([StepEntry("a", [t], [0])])
    assert runner.graph_replays >= 4


MARK, WINDOW = 7, 48


def marked_token_model(kind):
    """One layer whose memory of one marked token decides every logit of a token that sees it: every
    query points at the key that only the token MARK makes, and that token's value is large."""
    if kind == "attention":        # no window: the key is seen 290 tokens later
        layers = [conv_attention(2, 1, 16, 24, 6.0, 3, rot(10000.0, 4), None)]
    elif kind == "attention_w":    # the same behind a window
        layers = [conv_attention(2, 1, 16, 24, 6.0, 3, rot(10000.0, 4), None, window=WINDOW)]
    elif kind == "attention_2":
        layers = [key_value_attention(2, 1, 16, 6.0, rot(10000.0, 4), None, window=WINDOW, softcap=25.0)]
    else:
        layers = [latent(2, 16, 4, 24, 12, 6.0, 10000.0, None, window=WINDOW)]
    cfg = config(64, 200, 1e-5, layers, embedding_scale=2.0, logit_scale=0.5)
    w = make_weights(cfg, 21)
    p = "l0.mix."
    w["l0.norm1"][:] = 1.0
    w["embed"][:, 0] = 0.0
    w["embed"][MARK, 0] = 8.0                        # only the marked token has anything in channel 0
    w["embed"][:, 1] = 2.0                           # channel 1 of the input is the same for all tokens
    if kind == "latent":
        w[p + "dkv"][:, 0] = 0.0
        w[p + "dkv"][3, 0] = 4.0                     # latent channel 3 is large for the marked token only
        w[p + "dkv.norm"][:] = 1.0
        w[p + "uk"][:] = 0.0
        w[p + "uk"][5::16, 3] = 2.0                  # key channel 5 of every head reads latent channel 3
        w[p + "q"][:] = 0.0
        w[p + "q"][5::20, 1] = 3.0                   # every query head asks for channel 5
        w[p + "uv"][:, 3] = 2.0                      # the marked token's values are large
        return cfg, {n: t.to(torch.bfloat16).float() for n, t in w.items()}
    w[p + "k"][:, 0] = 0.0
    w[p + "k"][15, 0] = 4.0                          # channel 15 (not rotated) of the one kv head
    w[p + "q"][15::16] = 0.0
    w[p + "q"][15::16, 1] = 3.0                      # every query head asks for channel 15
    if kind in ("attention", "attention_w"):
        for name in ("q.conv", "k.conv", "v.conv"):  # the marked token's own tap carries it; the other taps stay
            w[p + name][:, -1] = 1.0
        if kind == "attention_w":                    # (keys and values of the marked token alone, so that the
            w[p + "k.conv"][:, :-1] = 0.0            # window's edge is one token wide; the queries keep their taps)
            w[p + "v.conv"][:, :-1] = 0.0
        w[p + "v"][:, 0] = 3.0
    else:
        w[p + "q.norm"][:] = 1.0
        w[p + "k.norm"][:] = 1.0
    return cfg, {n: t.to(torch.bfloat16).float() for n, t in w.items()}


@pytest.mark.parametrize("kind", ["attention", "attention_w", "attention_2", "latent"])
@pytest.mark.parametrize("place", [0, 15, 16, 47, 64, 200])
def test_a_marked_token_decides_the_logits(tmp_path, kind, place):
    """The marked token at the start, and just before, at and after the borders of pages; in a prompt,
    among decoded tokens, in two-token portions.  With a window the last token that sees it and the
    first that does not are both checked: the plain logits differ by much at the one and not at all
    at the other."""
    cfg, weights = marked_token_model(kind)
    folder, weights = write_folder(tmp_path, cfg, seed=21, tag="far" + kind, weights=weights)
    requests = make_requests(cfg["vocab"], [300], seed=8, avoid=(MARK,))
    requests["r0"][place] = MARK
    full = reference(cfg, weights, requests)
    toks = list(requests["r0"])
    toks[place] = MARK + 1
    other = reference(cfg, weights, {"r0": toks})
    if kind == "attention":
        assert np.abs(full["r0"][250:] - other["r0"][250:]).min(0).max() > 0.5     # the token matters to the end
    else:
        last = place + WINDOW - 1
        assert np.abs(full["r0"][last] - other["r0"][last]).max() > 0.5
        assert np.abs(full["r0"][last + 1:] - other["r0"][last + 1:]).max() == 0.0
    for name, steps in (("whole", rs.whole(requests)), ("decode", rs.tail_decoded(requests, tail=60)),
                        ("twos", rs.portions(requests, sizes=(33, 2, 64, 2, 2)))):
        run_and_compare(tmp_path, folder, cfg, steps, full, "float32", name)
        run_and_compare(tmp_path, folder, cfg, steps, full, "bfloat16", name)


def test_the_first_tokens_and_a_window_of_two(tmp_path):
    """Sequences of one to five tokens (shorter than every convolution and window), and model D's window of
    two tokens, one by one and in portions of two."""
    for which in ("D", "E"):
        cfg = MODELS[which]
        folder, weights = write_folder(tmp_path, cfg, seed=17, tag=which)
        requests = make_requests(cfg["vocab"], [1, 2, 3, 4, 5, 1], seed=13)
        ref = reference(cfg, weights, requests)
        loss = plain_float32_loss(cfg, weights, requests, ref)
        run_and_compare(tmp_path, folder, cfg, rs.whole(requests), ref, "float32", "whole", float32_bar=loss)
        run_and_compare(tmp_path, folder, cfg, rs.tail_decoded(requests, tail=4), ref, "float32", "ones", float32_bar=loss)
        run_and_compare(tmp_path, folder, cfg, rs.portions(requests, sizes=(2,)), ref, "float32", "twos", float32_bar=loss)


def test_the_program_replays_a_trace(tmp_path):
    cfg = MODELS["B"]
    folder, weights = write_folder(tmp_path, cfg, seed=14, tag="B")
    requests = make_requests(cfg["vocab"], [30, 9], seed=9)
    ref = reference(cfg, weights, requests)
    steps = rs.tail_decoded(requests, tail=5)
    out = str(tmp_path / "out_prog")
    replay_program(folder, steps, out, "float32", rs.max_tokens_needed(steps))
    worst, where = compare(out, steps, ref, cfg["vocab"])
    assert worst < max(bar("float32", ref), plain_float32_loss(cfg, weights, requests, ref)), (worst, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "E"])
def test_greedy_generation_through_the_entry_point(tmp_path, which, dtype):
    cfg = MODELS[which]
    folder, weights = write_folder(tmp_path, cfg, seed=15, tag=which)
    prompts = list(make_requests(cfg["vocab"], [30, 4, 77, 1, 12, 50], seed=10).values())
    new = 24
    for budget, blocks in ((256, 64), (8, 64), (64, 24)):
        if dtype == "bfloat16" and budget != 256:
            continue
        engine = LLMEngine(load_config(folder), CacheConfig(num_blocks=blocks),
                           SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=budget), dtype=dtype)
        outs = engine.generate(prompts, SamplingParams.greedy(new))
        engine.runner.manager.check()
        for p, o in zip(prompts, outs):
            toks = o.outputs[0].token_ids
            assert o.finished and len(toks) == new
            logits = plain.forward(cfg, weights, list(p) + toks).float()
            slack = 2 * bar(dtype, {"x": logits.numpy()})
            near = [bool(logits[len(p) - 1 + i][t] >= logits[len(p) - 1 + i].max() - slack)
                    for i, t in enumerate(toks)]
            # (bfloat16: a routed choice that falls the other way moves a whole row)
            assert all(near) if dtype == "float32" else sum(near) >= 0.8 * len(near), near


def test_command_line_samples_from_a_random_model(tmp_path, capsys):
    import json
    from servelab_amd import cli
    path = tmp_path / "config.json"
    path.write_text(json.dumps(MODELS["B"]))
    assert cli.main(["--config", str(path), "--random-weights", "3", "--prompt-ids", "5,6,7,8", "--max-tokens", "9",
                     "--temperature", "0.8", "--top-k", "20", "--top-p", "0.9", "--max-num-seqs", "4"]) == 0
    assert "finish=length" in capsys.readouterr().out
