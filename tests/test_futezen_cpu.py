"""Futezen without a GPU: configuration and registry, declared tensors against a written
checkpoint, cache needs and the run list of repeated layers, the plain implementation's own
mechanisms against second closed forms, and the engine's host side (pages, state slots, run
list, batching, replay) over the kernel calls emulated in torch."""
import copy
import json
import math
import random

import pytest
import torch

import plain_futezen as plain
import replay_schedules as rs
from emulated_ops import EmulatedOps
from futezen_models import MODELS, make_weights, tensor_shapes, write_folder
from replay_harness import compare, replay_in_process
from servelab_amd import ConfigError, load_config
from servelab_amd.config import FutezenConfig, resolve_architecture
from servelab_amd.parts import PagedKVSpec, StateSpec
from servelab_amd.parts.model import build_model_spec
from servelab_amd.weights.loader import Checkpoint, check_tensors

F = torch.float64


def make_requests(vocab, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def reference(cfg, weights, requests):
    return {rid: plain.forward(cfg, weights, toks).float().numpy() for rid, toks in requests.items()}


def float32_bar(cfg, weights, requests, ref):
    """The bar for float32 logits: 2e-4, or twice what the plain implementation itself loses when it
    runs in float32 where that is more (a loop over many small layers multiplies rounding)."""
    plain.F = torch.float32
    try:
        lost = max(float((plain.forward(cfg, weights, toks).double() - torch.as_tensor(ref[rid]).double()).abs().max())
                   for rid, toks in requests.items())
    finally:
        plain.F = torch.float64
    return max(2e-4, 2.0 * lost)


# ------------------------------------------------------------------ configuration
@pytest.mark.parametrize("which", sorted(MODELS))
def test_config_round_trip_and_declared_tensors(tmp_path, which):
    cfg = MODELS[which]
    folder, _ = write_folder(tmp_path, cfg, seed=1, tag=which)
    assert resolve_architecture(json.load(open(folder + "/config.json"))).name == "Futezen"
    config = load_config(folder)
    assert isinstance(config, FutezenConfig)
    again = FutezenConfig.from_hf(config.to_hf())
    assert again.layers == config.layers and again.loop == config.loop and again.to_hf() == config.to_hf()
    spec = build_model_spec(config)
    check_tensors({n: s.shape for n, s in spec.param_specs().items()}, Checkpoint(folder).shapes())
    assert {n: tuple(s.shape) for n, s in spec.param_specs().items()} == tensor_shapes(cfg)


def test_missing_and_impossible_keys_name_themselves():
    base = MODELS["A"]
    for path, text in ((("width",), "width"), (("norm",), "norm"), (("layers", 0, "mixer", "kv_heads"), "kv_heads"),
                       (("layers", 1, "mixer", "q_rank"), "q_rank"), (("layers", 2, "mixer", "norm_groups"), "norm_groups"),
                       (("layers", 2, "mixer", "conv"), "conv"), (("layers", 1, "mlp", "router", "top"), "top"),
                       (("layers", 0, "mlp", "ff"), "ff"), (("loop", "times"), "times")):
        cfg = copy.deepcopy(base)
        node = cfg
        for k in path[:-1]:
            node = node[k]
        del node[path[-1]]
        with pytest.raises(ConfigError, match=text):
            FutezenConfig.from_hf(cfg)
    for change, text in ((lambda c: c["layers"][1].update(type="rnn"), "attention, latent_attention, mamba2"),
                         (lambda c: c["layers"][2]["mixer"].update(groups=3), "groups"),
                         (lambda c: c["layers"][2]["mixer"].update(norm_groups=3), "norm_groups"),
                         (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
                         (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "dense, moe"),
                         (lambda c: c["loop"].update(stop=4), "loop"),
                         (lambda c: c["loop"].update(times=0), "loop")):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError, match=text):
            FutezenConfig.from_hf(cfg)


def test_keys_that_may_be_null_or_absent():
    cfg = copy.deepcopy(MODELS["A"])
    cfg["loop"] = None
    cfg["layers"][1]["mlp"]["shared"] = None
    cfg["layers"][2]["mlp"] = None
    got = FutezenConfig.from_hf(cfg)
    assert got.loop is None and got.order() == [0, 1, 2]
    assert got.layers[1].mlp.shared_ff == 0 and got.layers[2].mlp is None
    spec = build_model_spec(got)
    names = set(spec.param_specs())
    assert "l1.mlp.shared.up" not in names and "l1.mlp.shared.sg" not in names and "l1.mlp.router.b" in names
    assert "l2.norm2" not in names and "l2.norm2b" not in names and "l2.norm1b" in names
    cfg["loop"] = {"start": 1, "stop": 1, "times": 3}                # an empty stretch
    assert FutezenConfig.from_hf(cfg).order() == [0, 1, 2]


def test_cache_needs_and_run_list():
    spec = build_model_spec(FutezenConfig.from_hf(MODELS["A"]))
    assert len(spec.layers) == 3 and [c.layer for c in spec.run] == [0, 1, 2, 1, 2]
    assert [c.streams for c in spec.run] == [(0,), (1,), (2,), (3,), (4,)]         # a pass has caches of its own
    needs = spec.stream_specs()
    assert needs[0] == PagedKVSpec(2, 16, None, value_dim=24)
    assert needs[1] == needs[3] == PagedKVSpec(1, 24 + 8, None, value_dim=0)       # the latent and the rotated part
    assert needs[2] == needs[4] == StateSpec((4 * 8 * 16 + 3 * (4 * 8 + 2 * 2 * 16),), "float32")
    none = copy.deepcopy(MODELS["A"])
    del none["loop"]
    assert [c.layer for c in build_model_spec(FutezenConfig.from_hf(none)).run] == [0, 1, 2]
    d = build_model_spec(FutezenConfig.from_hf(MODELS["D"]))
    assert [c.layer for c in d.run] == [0, 1, 2, 3, 4] * 2
    assert len({s for s in d.stream_specs().values() if isinstance(s, PagedKVSpec)}) == 3


# ------------------------------------------------------------------ the plain implementation itself
def test_plain_norm_weight_sits_around_zero():
    x = torch.tensor([[3.0, -4.0]], dtype=F)
    got = plain.offset_norm(x, torch.tensor([0.0, 0.5], dtype=F), 0.0)
    rms = math.sqrt(12.5)
    assert torch.allclose(got, torch.tensor([[3.0 / rms, -4.0 * 1.5 / rms]], dtype=F))


def test_plain_rotations_are_complex_multiplications():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 2, 10, generator=g, dtype=F)
    pos = torch.tensor([0, 1, 7, 300, 4095])
    dims, base = 6, 100.0
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(3)], dtype=F)
    turn = torch.polar(torch.ones(5, 3, dtype=F), pos.to(F)[:, None] * freq)[:, None, :]
    z = torch.complex(x[..., :3], x[..., 3:6]) * turn
    got = plain.rotate_halves(x, pos, dims, base)
    assert torch.allclose(got[..., :3], z.real) and torch.allclose(got[..., 3:6], z.imag)
    assert torch.equal(got[..., 6:], x[..., 6:]) and torch.equal(got[0], x[0])
    z = torch.complex(x[..., 0:6:2], x[..., 1:6:2]) * turn
    got = plain.rotate_neighbours(x, pos, dims, base)
    assert torch.allclose(got[..., 0:6:2], z.real) and torch.allclose(got[..., 1:6:2], z.imag)
    assert torch.equal(got[..., 6:], x[..., 6:])


def test_plain_latent_attention_is_attention_in_the_latents_space():
    """score = (Wuk^T q) . c + q' . k', output = Wuv (sum of weights times c): the form the engine runs."""
    g = torch.Generator().manual_seed(1)
    T, w = 7, 12
    m = {"heads": 2, "dim": 4, "rot_dim": 2, "vdim": 3, "q_rank": 5, "kv_rank": 6, "scale": 0.4,
         "rot": {"base": 50.0, "dims": 2}}
    W = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"dq": (5, w), "dq.norm": (5,), "uq": (12, 5), "dkv": (8, w), "dkv.norm": (6,), "uk": (8, 6), "uv": (6, 6),
          "o": (w, 6)}.items()}
    h = torch.randn(T, w, generator=g, dtype=F)
    got = plain.latent_attention(h, m, W, "", 1e-5)
    pos = torch.arange(T)
    cq = h @ W["dq"].T
    cq = cq / torch.sqrt((cq * cq).mean(-1, keepdim=True) + 1e-5) * W["dq.norm"]
    q = (cq @ W["uq"].T).view(T, 2, 6)
    down = h @ W["dkv"].T
    c = down[:, :6] / torch.sqrt((down[:, :6] ** 2).mean(-1, keepdim=True) + 1e-5) * W["dkv.norm"]
    kr = plain.rotate_neighbours(down[:, None, 6:], pos, 2, 50.0)[:, 0]
    qr = plain.rotate_neighbours(q[..., 4:], pos, 2, 50.0)
    out = torch.zeros(T, 2, 3, dtype=F)
    for hd in range(2):
        ql = q[:, hd, :4] @ W["uk"][4 * hd:4 * hd + 4]                       # [T, 6]
        for t in range(T):
            s = (c[:t + 1] @ ql[t] + kr[:t + 1] @ qr[t, hd]) * 0.4
            p = torch.softmax(s, 0)
            out[t, hd] = W["uv"][3 * hd:3 * hd + 3] @ (p @ c[:t + 1])
    assert torch.allclose(got, out.reshape(T, 6) @ W["o"].T, atol=1e-10)


def test_plain_state_space_mixer_is_the_sum_over_decayed_inputs():
    g = torch.Generator().manual_seed(2)
    T, w = 8, 10
    m = {"heads": 2, "vdim": 3, "state": 4, "groups": 1, "conv": 3, "norm_groups": 2}
    ch = 6 + 8
    W = {n: torch.randn(s, generator=g, dtype=F) for n, s in
         {"in": (12 + 8 + 2, w), "conv": (ch, 3), "conv.b": (ch,), "dt_bias": (2,), "A_log": (2,), "D": (2,),
          "norm": (6,), "o": (w, 6)}.items()}
    h = torch.randn(T, w, generator=g, dtype=F)
    got = plain.mamba2(h, m, W, "", 1e-5)
    proj = h @ W["in"].T
    z, raw, dt = proj[:, :6], proj[:, 6:6 + ch], proj[:, 6 + ch:]
    conv = torch.zeros(T, ch, dtype=F)
    for t in range(T):
        for j in range(3):
            if t - 2 + j >= 0:
                conv[t] += W["conv"][:, j] * raw[t - 2 + j]
    conv = conv + W["conv.b"]
    conv = conv * torch.sigmoid(conv)
    x, B, C = conv[:, :6].view(T, 2, 3), conv[:, 6:10], conv[:, 10:]
    dt = torch.log1p(torch.exp(dt + W["dt_bias"]))
    la = -torch.exp(W["A_log"]) * dt                                          # log decays [T, 2]
    y = torch.zeros(T, 2, 3, dtype=F)
    for t in range(T):
        for s in range(t + 1):
            decay = torch.exp(la[s + 1:t + 1].sum(0))                         # [2]
            y[t] += (decay * dt[s] * (C[t] @ B[s]))[:, None] * x[s]
        y[t] += W["D"][:, None] * x[t]
    y = y.reshape(T, 6) * (z * torch.sigmoid(z))
    y = y.view(T, 2, 3)
    y = (y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-5)).reshape(T, 6) * W["norm"]
    assert torch.allclose(got, y @ W["o"].T, atol=1e-9)


def test_plain_router_takes_the_largest_and_renormalises():
    w = {"router": torch.tensor([[1.0, 0], [0, 1.0], [-1.0, 0], [0.5, 0.5]], dtype=F),
         "router.b": torch.tensor([0.0, 0.0, 7.0, 0.0], dtype=F), "shared.sg": torch.tensor([[0.0, 2.0]], dtype=F),
         "shared.up": -torch.eye(2, dtype=F), "shared.down": torch.eye(2, dtype=F)}
    for e in range(4):
        w[f"e{e}.up"] = torch.eye(2, dtype=F) * (e + 1)
        w[f"e{e}.down"] = torch.eye(2, dtype=F)
    h = torch.tensor([[3.0, -1.0]], dtype=F)           # logits 3, -1, 4 (by its bias), 1: experts 2 and 0
    got = plain.experts(h, {"router": {"experts": 4, "top": 2}, "shared": {"ff": 2}}, w, "")
    share = torch.softmax(torch.tensor([4.0, 3.0], dtype=F), 0)
    routed = torch.tensor([9.0 * (share[0] * 9 + share[1] * 1), 0.0], dtype=F)   # the square of relu
    shared = torch.sigmoid(torch.tensor(-2.0, dtype=F)) * torch.tensor([0.0, 1.0], dtype=F)
    assert torch.allclose(got[0], routed + shared, atol=1e-9)


def test_plain_loop_runs_layers_again_with_the_same_weights():
    cfg = MODELS["C"]
    assert plain.layer_order(cfg) == [0, 0, 0, 1, 2]
    weights = make_weights(cfg, 3)
    once = copy.deepcopy(cfg)
    once["layers"] = [cfg["layers"][0]] * 3 + cfg["layers"][1:]
    del once["loop"]
    w2 = {}
    for n, t in weights.items():
        i, rest = n.split(".", 1) if n.startswith("l") else (None, None)
        if i == "l0":
            for j in range(3):
                w2[f"l{j}.{rest}"] = t
        elif i in ("l1", "l2"):
            w2[f"l{int(i[1:]) + 2}.{rest}"] = t
        else:
            w2[n] = t
    toks = [5, 9, 100, 3, 77, 8]
    assert torch.equal(plain.forward(cfg, weights, toks), plain.forward(once, w2, toks))


# ------------------------------------------------------------------ the engine's host side
@pytest.mark.parametrize("which", sorted(MODELS))
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
    one left there (state, last inputs of the convolution, keys) must not reach the next."""
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
    assert worst < 2e-4, f"max abs err {worst} at {where}"
