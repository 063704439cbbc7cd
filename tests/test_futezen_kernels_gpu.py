"""Each kernel call that the Futezen parts added or widened, alone, against the plain torch function
of the same name (tests/emulated_ops.py), in both activation types: steps of several sequences of
unequal length, some at their start in slots that hold another request's leftovers (NaN here),
some continuing; sizes that are no multiples of anything."""
import types

import pytest
import torch

from emulated_ops import EmulatedOps
from servelab_amd.kernels import HipOps
from servelab_amd.parts.base import RotaryTables
from test_vekanex_kernels_gpu import DEV, DTYPES, Q_LENS, SLOTS, STARTS, close, fake_batch, states, tables

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", DTYPES)
def test_output_norm_and_input_norm_in_one_call(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(0)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for T, H in ((1, 72), (33, 256), (5, 2048 + 8), (3, 5000)):
        resid = torch.randn(T, H, generator=g)
        y = (3 * torch.randn(T, H, generator=g)).to(dtype)
        wy, w = 1 + 0.3 * torch.randn(H, generator=g), 1 + 0.3 * torch.randn(H, generator=g)
        r1, r2 = resid.clone().to(DEV), resid.clone()
        o1 = hip.add_normed_rmsnorm(r1, y.to(DEV), wy.to(DEV), 1e-5, w.to(DEV), 1e-6)
        o2 = emu.add_normed_rmsnorm(r2, y, wy, 1e-5, w, 1e-6)
        close(r1, r2, 2e-6)
        close(o1, o2, tol)
        rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
        before = r1.clone()
        o1 = hip.add_normed_rmsnorm(r1, y.to(DEV), wy.to(DEV), 1e-5, w.to(DEV), 1e-6, rows=rows.to(DEV))
        o2 = emu.add_normed_rmsnorm(r2.clone(), y, wy, 1e-5, w, 1e-6, rows=rows)
        close(o1, o2, tol)
        assert torch.equal(r1, before)                      # listed rows: the stream stays as it is


@pytest.mark.parametrize("dtype", DTYPES)
def test_activations_and_gates(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(1)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for T, inter, block in ((3, 40, 8), (17, 96, None), (130, 24, 8), (2, 10, 5)):
        gu = torch.randn(T, 2 * inter, generator=g).to(dtype)
        for act in ("silu", "relu"):
            close(hip.gate_mul(gu.to(DEV), block, act), emu.gate_mul(gu, block, act), tol)
        for act in ("silu", "relu", "relu2"):
            close(hip.activate(gu.clone().to(DEV), act), emu.activate(gu.clone(), act), tol)


@pytest.mark.parametrize("rows", [1, 5, 16, 24, 64, 100, 200, 600])
def test_relu_gated_feed_forward_at_every_row_count(rows):
    """bfloat16: the row count decides which product kernel runs (few rows, two tiles, staged, tiles
    over the row-major copy, the library), and each has the gate's activation in its epilogue."""
    g = torch.Generator().manual_seed(2)
    width, inter = 256, 1536
    gate, up = torch.randn(inter, width, generator=g) * width ** -0.5, torch.randn(inter, width, generator=g) * width ** -0.5
    down = torch.randn(width, inter, generator=g) * inter ** -0.5
    x = torch.randn(rows, width, generator=g)
    for dtype in DTYPES:
        hip, emu = tables(dtype)
        b = hip.GATE_BLOCK
        gu = torch.stack([gate.reshape(inter // b, b, width), up.reshape(inter // b, b, width)], 1).reshape(2 * inter, width)
        w_gu, w_d = hip.prepare_weight(gu.to(dtype).to(DEV)), hip.prepare_weight(down.to(dtype).to(DEV))
        got = hip.materialize(hip.gated_mlp(x.to(dtype).to(DEV), w_gu, b, w_d, activation="relu"))
        want = emu.gated_mlp(x.to(dtype), gu.to(dtype), b, down.to(dtype), activation="relu")
        close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2)
        silu = emu.gated_mlp(x.to(dtype), gu.to(dtype), b, down.to(dtype))
        assert (want.float() - silu.float()).abs().max() > 0.05          # (the activations differ by more than the bar)


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_rows_with_queries_from_other_rows(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(3)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for T, nh, D, R, C, rot, Q in ((7, 3, 16, 8, 24, 8, 40), (33, 5, 12, 6, 10, 2, 7), (2, 2, 32, 32, 64, 32, 64)):
        page, pages = 16, 5
        buf = torch.randn(T, Q + C + R + 3, generator=g).to(dtype)
        q_rows = torch.randn(T, nh * (D + R), generator=g).to(dtype)
        gain, qgain = 1 + 0.2 * torch.randn(C, generator=g), 1 + 0.2 * torch.randn(Q, generator=g)
        ang = torch.rand(T, rot // 2, generator=g) * 6
        tb = RotaryTables(torch.cos(ang), torch.sin(ang))
        slots = torch.randperm(page * pages, generator=g)[:T].to(torch.int32)
        k1 = torch.zeros(pages, 1, page, C + R).to(dtype)
        k2 = k1.clone()
        q1, q2 = torch.zeros(T, nh * (C + R)).to(dtype), torch.zeros(T, nh * (C + R)).to(dtype)
        k1d, q1d = k1.to(DEV), q1.to(DEV)
        hip.latent_store(buf.to(DEV), nh, D, R, C, Q, rot, gain.to(DEV), 1e-5,
                         RotaryTables(tb.cos.to(DEV), tb.sin.to(DEV)), slots.to(DEV), k1d, page, q1d,
                         q_rows=q_rows.to(DEV))
        emu.latent_store(buf, nh, D, R, C, Q, rot, gain, 1e-5, tb, slots, k2, page, q2, q_rows=q_rows)
        close(k1d, k2, tol)
        close(q1d, q2, tol)
        close(hip.slice_rmsnorm(buf.to(DEV), 0, Q, qgain.to(DEV), 1e-5), emu.slice_rmsnorm(buf, 0, Q, qgain, 1e-5), tol)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotation_and_pages_without_a_norm_over_the_projection(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(4)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for T, H, G, D, Dv, rot in ((9, 4, 2, 16, 24, 8), (3, 5, 5, 12, 20, 2), (40, 2, 1, 64, 64, 64), (2, 3, 1, 8, 8, 0)):
        page, pages = 16, 4
        buf = torch.randn(T, (H + G) * D + G * Dv + 5, generator=g)
        ang = torch.rand(T, max(1, rot // 2), generator=g) * 6
        tb = RotaryTables(torch.cos(ang), torch.sin(ang)) if rot else None
        tbd = RotaryTables(tb.cos.to(DEV), tb.sin.to(DEV)) if rot else None
        slots = torch.randperm(page * pages, generator=g)[:T].to(torch.int32)
        k1, v1 = torch.zeros(pages, G, page, D).to(dtype), torch.zeros(pages, G, Dv, page).to(dtype)
        k2, v2 = k1.clone(), v1.clone()
        k1d, v1d = k1.to(DEV), v1.to(DEV)
        q1 = hip.projnorm_rope_store(buf.to(DEV), H, G, D, Dv, None, None, 1e-5, rot, tbd, slots.to(DEV), k1d, v1d, page)
        q2 = emu.projnorm_rope_store(buf, H, G, D, Dv, None, None, 1e-5, rot, tb, slots, k2, v2, page)
        close(q1, q2, tol)
        close(k1d, k2, tol)
        close(v1d, v2, tol)


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_conv_with_a_bias(taps):
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(5)
    C, off = 300, 11
    T = sum(Q_LENS)
    buf = torch.randn(T, 7 + C, generator=g)
    w, bias = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    st = states(6, off + (taps - 1) * C + 3, seed=3)
    batch_d, batch_h = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    s1, s2 = st.clone().to(DEV), st.clone()
    o1 = hip.short_conv(buf.to(DEV), 7, w.to(DEV), s1, off, batch_d, True, bias=bias.to(DEV))
    o2 = emu.short_conv(buf, 7, w, s2, off, batch_h, True, bias=bias)
    close(o1, o2, 2e-6)
    assert (o2 - emu.short_conv(buf, 7, w, st.clone(), off, batch_h, False)).abs().max() > 0.1
    if taps > 1:
        used = sorted(SLOTS)
        close(s1[used][:, off:off + (taps - 1) * C], s2[used][:, off:off + (taps - 1) * C], 0)


@pytest.mark.parametrize("H,G,N,P", [(2, 2, 8, 16), (4, 2, 24, 8), (4, 1, 72, 32), (1, 1, 136, 70), (3, 3, 40, 300),
                                     (6, 2, 48, 40), (5, 5, 4, 3)])
def test_state_space_scan(H, G, N, P):
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(6)
    T = sum(Q_LENS)
    inner = H * P
    src = torch.randn(T, inner + 2 * G * N + 3, generator=g) * 0.5
    steps = torch.randn(T, 9 + H, generator=g)
    rates, bias, skip = -1 + 0.5 * torch.randn(H, generator=g), 0.5 * torch.randn(H, generator=g), torch.randn(H, generator=g)
    st = states(6, inner * N + 5, seed=7)
    batch_d, batch_h = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    s1, s2 = st.clone().to(DEV), st.clone()
    args = (0, inner, inner + G * N, H, G, N, P)
    o1 = hip.ssd_scan(src.to(DEV), *args, steps.to(DEV), 9, rates.to(DEV), bias.to(DEV), skip.to(DEV), s1, batch_d, True)
    o2 = emu.ssd_scan(src, *args, steps, 9, rates, bias, skip, s2, batch_h, True)
    close(o1, o2, 1e-5)
    used = sorted(SLOTS)
    close(s1[used][:, :inner * N], s2[used][:, :inner * N], 1e-5)
    assert torch.equal(torch.nan_to_num(s1.cpu()[:, inner * N:], 9.0), torch.nan_to_num(st[:, inner * N:], 9.0))
    s3 = st.clone().to(DEV)
    hip.ssd_scan(src.to(DEV), *args, steps.to(DEV), 9, rates.to(DEV), bias.to(DEV), skip.to(DEV), s3, batch_d, False)
    assert torch.equal(torch.nan_to_num(s3.cpu(), 9.0), torch.nan_to_num(st, 9.0))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gate_before_the_norm_of_equal_parts(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(8)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for T, parts, per in ((5, 1, 200), (9, 3, 8), (2, 4, 1000), (33, 6, 32)):
        o = torch.randn(T, parts * per, generator=g)
        gate = torch.randn(T, 13 + parts * per, generator=g)
        w = 1 + 0.3 * torch.randn(parts * per, generator=g)
        got = hip.head_norm_gate(o.to(DEV), parts, per, w.to(DEV), True, 1e-5, gate.to(DEV), 13, "silu", gate_first=True)
        want = emu.head_norm_gate(o, parts, per, w, True, 1e-5, gate, 13, "silu", gate_first=True)
        close(got, want, tol)
        after = emu.head_norm_gate(o, parts, per, w, True, 1e-5, gate, 13, "silu")
        assert (want.float() - after.float()).abs().max() > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,E,top,ff,width,shared", [(7, 5, 2, 24, 64, True), (1, 12, 2, 80, 160, True),
                                                    (300, 8, 3, 32, 96, True), (40, 70, 9, 8, 40, False),
                                                    (2100, 4, 2, 64, 128, True), (9, 3, 3, 20, 36, True)])
def test_experts_without_a_gate_and_a_gated_shared_one(dtype, T, E, top, ff, width, shared):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(T, width, generator=g).to(dtype)
    up = (torch.randn(E, ff, width, generator=g) * width ** -0.5).to(dtype)
    down = (torch.randn(E, width, ff, generator=g) * ff ** -0.5).to(dtype)
    logits = torch.randn(T, E + 3, generator=g)
    base = torch.randn(T, width, generator=g).to(dtype) if shared else None
    r1 = hip.route_tokens(logits.to(DEV), E, top)
    r2 = emu.route_tokens(logits, E, top)
    assert torch.equal(r1.chosen.cpu(), r2[0])
    got = hip.routed_experts(x.to(DEV), r1, hip.prepare_expert_matrices(up.to(DEV), gated=False),
                             hip.prepare_expert_matrices(down.to(DEV)), base.to(DEV) if shared else None,
                             activation="relu2", gated=False, base_gate=logits.to(DEV) if shared else None,
                             base_gate_col=E)
    want = emu.routed_experts(x, r2, up, down, base, activation="relu2", gated=False,
                              base_gate=logits if shared else None, base_gate_col=E)
    close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2)
