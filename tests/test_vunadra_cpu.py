"""Vunadra without a GPU: configuration and registry, declared tensors against a written
checkpoint, cache needs and the run list of repeated layers, the plain implementation's own
mechanisms against second closed forms, and the engine's host side (pages, state slots, run
list, batching, replay) over the kernel calls emulated in torch."""
import copy
import json
import math
import random

import pytest
import torch

import plain_vunadra as plain
import replay_schedules as rs
from emulated_ops import EmulatedOps
from replay_harness import compare, replay_in_process
from servelab_amd import ConfigError, load_config
from servelab_amd.config import VunadraConfig, resolve_architecture
from servelab_amd.parts import PagedKVSpec, StateSpec
from servelab_amd.parts.model import build_model_spec
from servelab_amd.weights.loader import Checkpoint, check_tensors
from vunadra_models import MODELS, make_weights, tensor_shapes, write_folder

F = torch.float64


def make_requests(vocab, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def reference(cfg, weights, requests):
    return {rid: plain.forward(cfg, weights, toks).float().numpy() for rid, toks in requests.items()}


def float32_bar(cfg, weights, requests, ref):
    """The bar for float32 logits: 2e-4 of the logits' range (at least 2e-4), or twice what the plain
    implementation itself loses when it runs in float32 where that is more."""
    plain.F = torch.float32
    try:
        lost = max(float((plain.forward(cfg, weights, toks).double() - torch.as_tensor(ref[rid]).double()).abs().max())
                   for rid, toks in requests.items())
    finally:
        plain.F = torch.float64
    top = max(float(abs(r).max()) for r in ref.values())
    return max(2e-4 * max(1.0, top), 2.0 * lost)


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("which", sorted(MODELS))
def test_config_round_trip_and_declared_tensors(tmp_path, which):
    cfg = MODELS[which]
    folder, _ = write_folder(tmp_path, cfg, seed=1, tag=which)
    assert resolve_architecture(json.load(open(folder + "/config.json"))).name == "Vunadra"
    config = load_config(folder)
    assert isinstance(config, VunadraConfig)
    again = VunadraConfig.from_hf(config.to_hf())
    assert again.layers == config.layers and again.loop == config.loop and again.to_hf() == config.to_hf()
    assert (again.embedding_scale, again.logit_scale) == (config.embedding_scale, config.logit_scale)
    spec = build_model_spec(config)
    check_tensors({n: s.shape for n, s in spec.param_specs().items()}, Checkpoint(folder).shapes())
    assert {n: tuple(s.shape) for n, s in spec.param_specs().items()} == tensor_shapes(cfg)


def test_missing_and_impossible_keys_name_themselves():
    base = MODELS["A"]
    for path, text in ((("width",), "width"), (("norm",), "norm"), (("embedding",), "embedding"),
                       (("logit_scale",), "logit_scale"), (("layers", 0, "mixer", "kv_heads"), "kv_heads"),
                       (("layers", 0, "mixer", "vdim"), "vdim"), (("layers", 2, "mixer", "kv_rank"), "kv_rank"),
                       (("layers", 0, "mixer", "rot", "scaling", "slow"), "slow"),
                       (("layers", 1, "mixer", "rot", "scaling", "high"), "high"),
                       (("layers", 1, "mlp", "router", "top"), "top"), (("layers", 1, "mlp", "expert", "limit"), "limit"),
                       (("layers", 1, "mlp", "router", "scale"), "scale"),
                       (("layers", 0, "mlp", "ff"), "ff"), (("loop", "times"), "times")):
        cfg = copy.deepcopy(base)
        node = cfg
        for k in path[:-1]:
            node = node[k]
        del node[path[-1]]
        with pytest.raises(ConfigError, match=text):
            VunadraConfig.from_hf(cfg)
    for change, text in ((lambda c: c["layers"][1].update(type="rnn"), "attention, attention_2, latent_attention"),
                         (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
                         (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
                         (lambda c: c["layers"][1]["mixer"].update(vdim=8), "equal"),
                         (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "dense, moe"),
                         (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top"),
                         (lambda c: c["loop"].update(stop=4), "loop")):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError, match=text):
            VunadraConfig.from_hf(cfg)


def test_keys_that_may_be_absent():
    """No mask: every earlier key; no softcap, no scaling, no convolution, no rotation, no loop, no
    feed-forward: each is a layer without that mechanism."""
    cfg = copy.deepcopy(MODELS["B"])
    config = VunadraConfig.from_hf(cfg)
    assert config.loop is None and config.layers[0].mlp is None
    assert [l.mixer.window for l in config.layers] == [0, 0, 0]
    assert config.layers[0].mixer.softcap == 0.0 and config.layers[0].mixer.rot.scaling is None
    cfg["layers"][1]["mixer"].pop("conv")
    cfg["layers"][1]["mixer"]["rot"] = None
    cfg["loop"] = None
    config = VunadraConfig.from_hf(cfg)
    assert config.layers[1].mixer.conv == 0 and config.layers[1].mixer.rot.dims == 0
    spec = build_model_spec(config)
    assert "l1.mix.q.conv" not in spec.param_specs() and "loop.in" not in spec.param_specs()
    assert len(spec.stream_specs()) == 3


def test_cache_needs_and_the_run_list_of_repeated_layers():
    spec = build_model_spec(VunadraConfig.from_hf(MODELS["A"]))
    # l0, then twice (entry, l1, l2); the entry block caches nothing and is the last block of the list
    entry = len(spec.layers) - 1
    assert [c.layer for c in spec.run] == [0, entry, 1, 2, entry, 1, 2]
    assert spec.keeps_embedding
    streams = spec.stream_specs()
    # the attention with a convolution keeps pages and the last two projected rows of q, k and v
    assert streams[0] == PagedKVSpec(2, 16, None, value_dim=24)
    assert streams[1] == StateSpec((2 * (4 * 16 + 2 * 16 + 2 * 24),), "float32")
    # every pass has streams of its own: keys that serve as values need value pages of the keys' width
    assert streams[2] == streams[4] == PagedKVSpec(2, 16, 9, value_dim=16)
    assert streams[3] == streams[5] == PagedKVSpec(1, 24 + 8, 13, value_dim=0)
    assert len(streams) == 6
    one_tap = build_model_spec(VunadraConfig.from_hf(MODELS["D"]))
    assert not any(isinstance(s, StateSpec) for s in one_tap.stream_specs().values())
    assert not build_model_spec(VunadraConfig.from_hf(MODELS["B"])).keeps_embedding


# ------------------------------------------------------------------ the plain mechanisms
def test_plain_rotation_of_neighbours_is_a_complex_product():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 2, 12, generator=g, dtype=F)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    freqs = plain.plain_frequencies(8, 50.0)
    got = plain.rotate_neighbours(x, pos, 8, freqs, 1.3)
    z = torch.view_as_complex(x[..., :8].reshape(5, 2, 4, 2).contiguous())
    turn = torch.polar(torch.full((5, 4), 1.3, dtype=F), pos.to(F)[:, None] * torch.tensor(freqs, dtype=F)[None, :])
    want = torch.view_as_real(z * turn[:, None, :]).reshape(5, 2, 8)
    assert torch.allclose(got[..., :8], want, atol=1e-12) and torch.equal(got[..., 8:], x[..., 8:])
    assert freqs[0] == 1.0 and math.isclose(freqs[3], 50.0 ** -0.75)


def test_plain_blended_frequencies_ramp_between_their_ends():
    dims, base, factor, original, fast, slow = 16, 10000.0, 4.0, 64, 8.0, 1.0
    plainf = plain.plain_frequencies(dims, base)
    got = plain.blended_frequencies(dims, base, factor, original, fast, slow)
    # a pair that turns more than `fast` times within `original` positions keeps its frequency, one that
    # turns less than `slow` times is slowed by the factor, the others lie between in the order of the pairs
    turns = [original * f / (2 * math.pi) for f in plainf]
    ratios = [g / f for g, f in zip(got, plainf)]
    assert all(r == 1.0 for r, t in zip(ratios, turns) if t > fast * base ** (2 / dims))
    assert all(math.isclose(r, 1 / factor) for r, t in zip(ratios, turns) if t < slow / base ** (2 / dims))
    assert all(a >= b for a, b in zip(ratios, ratios[1:])) and 1 / factor < ratios[2] < ratios[1] < 1.0
    assert math.isclose(plain.blended_magnitude(factor), 0.1 * math.log(4.0) + 1.0)


def test_plain_wavelength_frequencies_have_three_ranges():
    dims, base = 64, 10000.0
    plainf = plain.plain_frequencies(dims, base)
    got = plain.wavelength_frequencies(dims, base, 8.0, 1.0, 4.0, 256)
    kinds = set()
    for f, g in zip(plainf, got):
        wave = 2 * math.pi / f
        if wave < 256 / 4.0:
            assert g == f
            kinds.add("kept")
        elif wave > 256 / 1.0:
            assert math.isclose(g, f / 8.0)
            kinds.add("stretched")
        else:
            assert f / 8.0 < g < f
            kinds.add("between")
    assert kinds == {"kept", "stretched", "between"}


def test_plain_short_convolution_is_a_sum_over_taps():
    g = torch.Generator().manual_seed(1)
    u, taps = torch.randn(7, 3, generator=g, dtype=F), torch.randn(3, 4, generator=g, dtype=F)
    got = plain.short_convolution(u, taps)
    for t in range(7):
        want = sum(taps[:, j] * u[t - 3 + j] for j in range(4) if t - 3 + j >= 0)
        assert torch.allclose(got[t], want, atol=1e-12)
    assert torch.allclose(plain.short_convolution(u, taps[:, :1]), u * taps[:, 0], atol=1e-12)      # one tap


def test_plain_window_sees_itself_and_size_minus_one_before():
    seen = plain.visible(6, 3)
    assert seen[5].tolist() == [False, False, False, True, True, True]
    assert seen[1].tolist() == [True, True, False, False, False, False]
    assert plain.visible(4, None)[3].tolist() == [True] * 4 and plain.visible(4, 1)[3].tolist() == [False] * 3 + [True]


def test_plain_keys_serve_as_values_before_norm_and_rotation():
    """One head, one token: the softmax weight is 1, so the mixer returns W_o (W_k h + b_k) + b_o."""
    g = torch.Generator().manual_seed(2)
    w = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"q": (8, 6), "q.b": (8,), "k": (8, 6), "k.b": (8,), "q.norm": (8,), "k.norm": (8,), "o": (6, 8),
          "o.b": (6,)}.items()}
    m = {"heads": 1, "kv_heads": 1, "dim": 8, "scale": 0.3, "softcap": 2.0, "rot": {"base": 10.0, "dims": 8}}
    h = torch.randn(1, 6, generator=g, dtype=F)
    got = plain.keys_as_values_attention(h, m, w, "", 1e-5)
    assert torch.allclose(got, (h @ w["k"].T + w["k.b"]) @ w["o"].T + w["o.b"], atol=1e-12)


def test_plain_latent_attention_in_the_latents_space():
    """score_h(i, j) = (Wuk_h^T q_h) . c_j + q_h' . k'_j and sum_j p_ij Wuv_h c_j = Wuv_h sum_j p_ij c_j."""
    g = torch.Generator().manual_seed(3)
    m = {"heads": 2, "dim": 4, "rot_dim": 4, "vdim": 3, "kv_rank": 5, "scale": 0.4, "rot": {"base": 20.0, "dims": 4},
         "mask": {"size": 3}}
    w = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"q": (16, 6), "dkv": (9, 6), "dkv.norm": (5,), "uk": (8, 5), "uv": (6, 5), "o": (6, 6)}.items()}
    T = 6
    h = torch.randn(T, 6, generator=g, dtype=F)
    got = plain.latent_attention(h, m, w, "", 1e-5)
    q = (h @ w["q"].T).view(T, 2, 8)
    down = h @ w["dkv"].T
    c = plain.rms_norm(down[:, :5], w["dkv.norm"], 1e-5)
    pos = torch.arange(T)
    fr = plain.plain_frequencies(4, 20.0)
    kr = plain.rotate_neighbours(down[:, None, 5:], pos, 4, fr)[:, 0]
    qr = plain.rotate_neighbours(q[..., 4:], pos, 4, fr)
    out = torch.zeros(T, 2, 3, dtype=F)
    for hd in range(2):
        ql = q[:, hd, :4] @ w["uk"].view(2, 4, 5)[hd]                     # [T, 5]
        s = (ql @ c.T + qr[:, hd] @ kr.T) * 0.4
        p = torch.softmax(s.masked_fill(~plain.visible(T, 3), -math.inf), -1)
        out[:, hd] = (p @ c) @ w["uv"].view(2, 3, 5)[hd].T
    assert torch.allclose(got, out.reshape(T, 6) @ w["o"].T, atol=1e-10)


def test_plain_router_adds_the_correction_to_choose_and_not_to_weigh():
    w = {"router": torch.tensor([[1.0, 0], [0, 1.0], [-1.0, 0], [0.5, 0.5]], dtype=F),
         "correction": torch.tensor([0.0, 0.0, 1.0, 0.0], dtype=F)}
    h = torch.tensor([[3.0, -1.0]], dtype=F)            # logits 3, -1, -3, 1: shares fall 0, 3, 1, 2
    chosen, weights = plain.route(h, w, "", {"top": 2, "scale": 1.5})
    s = torch.softmax(torch.tensor([3.0, -1.0, -3.0, 1.0], dtype=F), 0)
    assert chosen[0].tolist() == [2, 0]                 # the correction lifts expert 2 over all others
    assert torch.allclose(weights[0], torch.stack([s[2], s[0]]) / (s[2] + s[0]) * 1.5, atol=1e-12)


def test_plain_experts_clamp_and_hand_through():
    w = {"router": torch.tensor([[4.0, 0], [0, 4.0], [0.0, 0.0]], dtype=F), "correction": torch.zeros(3, dtype=F),
         "e0.gate": torch.eye(2, dtype=F) * 5, "e0.up": -torch.eye(2, dtype=F) * 5, "e0.down": torch.eye(2, dtype=F),
         "e1.gate": torch.eye(2, dtype=F), "e1.up": torch.eye(2, dtype=F), "e1.down": torch.eye(2, dtype=F)}
    c = {"kind": "moe", "router": {"experts": 2, "identity": 1, "top": 3, "scale": 1.0}, "expert": {"ff": 2, "limit": 2.0}}
    h = torch.tensor([[1.0, -0.5]], dtype=F)
    got = plain.routed_ff(h, c, w, "")
    s = torch.softmax(torch.tensor([4.0, -2.0, 0.0], dtype=F), 0)
    g0, u0 = torch.tensor([2.0, -2.5], dtype=F), torch.tensor([-2.0, 2.0], dtype=F)     # 5 -> 2 above, -5 -> -2, 2.5 -> 2
    e0 = g0 * torch.sigmoid(1.702 * g0) * (u0 + 1)
    e1 = h[0] * torch.sigmoid(1.702 * h[0]) * (h[0] + 1)
    assert torch.allclose(got[0], s[0] * e0 + s[1] * e1 + s[2] * h[0], atol=1e-12)


def test_plain_loop_enters_every_pass_through_the_same_matrix():
    cfg = MODELS["C"]
    weights = make_weights(cfg, 3)
    toks = [5, 9, 100, 3, 77, 8]
    trace = []
    plain.forward(cfg, weights, toks, trace)
    assert len(trace) == 3 + 2                          # l0 three times, then l1 and l2
    w = {n: t.to(F) for n, t in weights.items()}
    x0 = w["embed"][torch.tensor(toks)] * cfg["embedding"]["scale"]
    x = x0
    for t in range(3):
        x = torch.cat([x, x0], -1) @ w["loop.in"].T + w["loop.step"][t]
        x = plain.layer(x, 0, cfg["layers"][0], w, cfg["norm"]["eps"])
        assert torch.equal(x, trace[t])


# ------------------------------------------------------------------ the engine's host side
@pytest.mark.parametrize("which", sorted(set(MODELS) - {"F"}))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "twos", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, which, schedule):
    cfg = MODELS[which]
    folder, weights = write_folder(tmp_path, cfg, seed=11, tag=which)
    requests = make_requests(cfg["vocab"], [37, 1, 2, 49, 5, 26], seed=5)
    ref = reference(cfg, weights, requests)
    steps = {"whole": lambda: rs.whole(requests), "tail": lambda: rs.tail_decoded(requests, tail=12),
             "portions": lambda: rs.portions(requests),
             "twos": lambda: rs.portions(requests, sizes=(2, 2, 3, 2, 17, 2)),
             "mixed": lambda: rs.mixed(requests, {r: max(1, len(t) - 8) for r, t in requests.items()},
                                       max_live=3, seed=2)}[schedule]()
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps),
                      ops=EmulatedOps(torch.float32), device="cpu", max_live=3)
    worst, where = compare(out, steps, ref, cfg["vocab"])
    bar = float32_bar(cfg, weights, requests, ref)
    assert worst < bar, f"max abs err {worst} at {where}, bar {bar}"


def test_slots_and_pages_that_held_another_request_start_afresh(tmp_path):
    """Two slots, seven requests: every slot and page serves several requests, and what the last
    one left there (last inputs of the convolution, keys) must not reach the next."""
    cfg = MODELS["A"]
    folder, weights = write_folder(tmp_path, cfg, seed=12, tag="A")
    requests = make_requests(cfg["vocab"], [20, 3, 31, 1, 12, 2, 25], seed=6)
    ref = reference(cfg, weights, requests)
    steps = rs.mixed(requests, {r: len(t) // 2 for r, t in requests.items()}, max_live=2, seed=4,
                     max_portion=7)
    out = str(tmp_path / "out")
    replay_in_process(folder, steps, out, "float32", rs.max_tokens_needed(steps),
                      ops=EmulatedOps(torch.float32), device="cpu", max_live=2)
    worst, where = compare(out, steps, ref, cfg["vocab"])
    assert worst < float32_bar(cfg, weights, requests, ref), f"max abs err {worst} at {where}"
