"""Each kernel call that the Vunadra parts added or widened, alone, against the plain torch function
of the same name (tests/emulated_ops.py) or a float64 formula written here, in both activation
types: steps of several sequences of unequal length, some at their start in slots that hold
another request's leftovers (NaN here), some continuing; sizes that are no multiples of anything."""
import math
from types import SimpleNamespace

import pytest
import torch

from servelab_amd.parts.base import RotaryTables
from test_vekanex_kernels_gpu import DEV, DTYPES, Q_LENS, SLOTS, STARTS, close, fake_batch, states, tables
from test_window_kernels_gpu import fill_pages, paged

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_embedding_stream_pair_and_scaled_rows(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(0)
    for T, H, V in ((1, 72, 11), (33, 256, 300), (5, 1000, 7)):
        table = torch.randn(V, H, generator=g).to(dtype)
        ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
        x0 = hip.embed(ids.to(DEV), table.to(DEV), 2.5)
        close(x0, emu.embed(ids, table, 2.5), 0)
        assert torch.equal(hip.embed(ids.to(DEV), table.to(DEV)).cpu(), table[ids.long()].float())
        resid = torch.randn(T, H, generator=g) * 3
        delta = torch.randn(T, H, generator=g).to(dtype)
        for d in (None, delta):
            before = resid.clone().to(DEV)
            got = hip.stream_pair(before, None if d is None else d.to(DEV), x0)
            close(got, emu.stream_pair(resid, d, x0.cpu()), 0 if dtype == torch.float32 else 8e-3)
            assert torch.equal(before.cpu(), resid)               # neither stream is changed
        z = torch.randn(T, V, generator=g) * 5
        close(hip.scale_rows(z.clone().to(DEV), 1.75), z * 1.75, 1e-7)


def test_rotary_tables_with_a_magnitude():
    hip, emu = tables(torch.float32)
    pos = torch.tensor([0, 1, 2, 77, 1000, 30000], dtype=torch.int32)
    inv = torch.tensor([1.0, 0.31, 0.01, 1e-4], dtype=torch.float32)
    for mag in (1.0, 1.2079):
        cos, sin = hip.rope_tables(pos.to(DEV), inv.to(DEV), mag)
        ang = pos.double()[:, None] * inv.double()[None, :]
        # (the angle is a float32 product: at position 30,000 it is off by up to 2e-3 of a turn's 2 pi)
        tol = 30000 * 2 ** -24 * 1.5
        assert (cos.cpu().double() - mag * torch.cos(ang)).abs().max() < tol
        assert (sin.cpu().double() - mag * torch.sin(ang)).abs().max() < tol
        c2, s2 = emu.rope_tables(pos, inv, mag)
        close(cos, c2, 2e-6)
        close(sin, s2, 2e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gelu_gate_and_activation(dtype):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(1)
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    for T, inter, block in ((3, 40, 8), (17, 96, None), (130, 24, 8), (2, 10, 5)):
        gu = (2 * torch.randn(T, 2 * inter, generator=g)).to(dtype)
        close(hip.gate_mul(gu.to(DEV), block, "gelu_tanh"), emu.gate_mul(gu, block, "gelu_tanh"), tol)
        close(hip.activate(gu.clone().to(DEV), "gelu_tanh"), emu.activate(gu.clone(), "gelu_tanh"), tol)
    z = torch.linspace(-6, 6, 25, dtype=torch.float64)
    want = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))
    close(emu.activate(z.float().clone(), "gelu_tanh"), want, 1e-6)


@pytest.mark.parametrize("rows", [1, 5, 16, 24, 64, 100, 200, 600])
def test_biased_gelu_feed_forward_at_every_row_count(rows):
    """bfloat16: the row count decides which product kernel runs (few rows, two tiles, staged, tiles
    over the row-major copy, the library), and each adds the biases of gate and up in its epilogue."""
    g = torch.Generator().manual_seed(2)
    for width, inter in ((256, 1536), (72, 40)):
        gate, up = torch.randn(inter, width, generator=g) * width ** -0.5, torch.randn(inter, width, generator=g) * width ** -0.5
        down = torch.randn(width, inter, generator=g) * inter ** -0.5
        bg, bu, bd = torch.randn(inter, generator=g), torch.randn(inter, generator=g), torch.randn(width, generator=g)
        x = torch.randn(rows, width, generator=g)
        for dtype in DTYPES:
            hip, emu = tables(dtype)
            b = hip.GATE_BLOCK if inter % hip.GATE_BLOCK == 0 else inter
            gu = torch.stack([gate.reshape(inter // b, b, width), up.reshape(inter // b, b, width)], 1).reshape(2 * inter, width)
            bgu = torch.stack([bg.reshape(inter // b, b), bu.reshape(inter // b, b)], 1).reshape(2 * inter)
            w_gu, w_d = hip.prepare_weight(gu.to(dtype).to(DEV)), hip.prepare_weight(down.to(dtype).to(DEV))
            got = hip.materialize(hip.gated_mlp(x.to(dtype).to(DEV), w_gu, b, w_d, activation="gelu_tanh",
                                                bias_gate_up=bgu.to(DEV), bias_down=bd.to(DEV)))
            want = emu.gated_mlp(x.to(dtype), gu.to(dtype), b, down.to(dtype), activation="gelu_tanh", bias_gate_up=bgu,
                                 bias_down=bd)
            close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2)
            plain = gate.to(dtype).double(), up.to(dtype).double(), down.to(dtype).double()
            xd = x.to(dtype).double()
            z = xd @ plain[0].T + bg
            mid = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))) * (xd @ plain[1].T + bu)
            close(got, mid @ plain[2].T + bd, 2e-5 if dtype == torch.float32 else 2.5e-2)
            none = emu.gated_mlp(x.to(dtype), gu.to(dtype), b, down.to(dtype), activation="gelu_tanh")
            assert (want.float() - none.float()).abs().max() > 0.1            # (the biases matter)


@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_short_conv_without_an_activation(taps):
    hip, emu = tables(torch.float32)
    g = torch.Generator().manual_seed(3)
    C = 4 * 24 + 2 * 24 + 2 * 10 + 1
    T = sum(Q_LENS)
    buf = torch.randn(T, C + 5, generator=g)
    w = torch.randn(C, taps, generator=g)
    st = states(6, max(1, (taps - 1) * C) + 3, seed=4)
    batch_d, batch_h = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    s1, s2 = st.clone().to(DEV), st.clone()
    o1 = hip.short_conv(buf.to(DEV), 0, w.to(DEV), s1, 0, batch_d, True, activation=None)
    o2 = emu.short_conv(buf, 0, w, s2, 0, batch_h, True, activation=None)
    close(o1, o2, 2e-6)
    if taps > 1:
        close(s1[sorted(SLOTS)][:, :(taps - 1) * C], s2[sorted(SLOTS)][:, :(taps - 1) * C], 0)
    # against the sum written out, for a sequence that starts in the step
    a = Q_LENS[0] + Q_LENS[1]
    seq = buf[a:a + Q_LENS[2], :C].double()
    for t in range(Q_LENS[2]):
        want = sum(w[:, j].double() * seq[t - taps + 1 + j] for j in range(taps) if t - taps + 1 + j >= 0)
        assert (o1[a + t].cpu().double() - want).abs().max() < 1e-5
    silu = emu.short_conv(buf, 0, w, st.clone(), 0, batch_h, False)
    assert (silu - o2).abs().max() > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("normed", [True, False])
def test_keys_that_serve_as_values_reach_the_pages_unnormed(dtype, normed):
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(5)
    for H, G, D, rot, page in ((4, 2, 16, 16, 16), (6, 3, 10, 4, 32), (1, 1, 64, 0, 16), (8, 2, 64, 64, 64)):
        T = 21
        buf = torch.randn(T, (H + G) * D + 3, generator=g)
        qg = 1 + 0.3 * torch.randn(H * D, generator=g) if normed else None
        kg = 1 + 0.3 * torch.randn(G * D, generator=g) if normed else None
        ang = torch.rand(T, max(1, rot // 2), generator=g) * 6
        tb = RotaryTables(torch.cos(ang), torch.sin(ang)) if rot else None
        tbd = RotaryTables(tb.cos.to(DEV), tb.sin.to(DEV)) if rot else None
        slots = torch.randperm(4 * page, generator=g)[:T].to(torch.int32)
        kc1, vc1 = torch.zeros(4, G, page, D).to(dtype), torch.zeros(4, G, D, page).to(dtype)
        kc2, vc2 = kc1.clone(), vc1.clone()
        kd, vd = kc1.to(DEV), vc1.to(DEV)
        dev = lambda t: None if t is None else t.to(DEV)
        q1 = hip.projnorm_rope_store(buf.to(DEV), H, G, D, D, dev(qg), dev(kg), 1e-5, rot, tbd, slots.to(DEV), kd, vd, page,
                                     values_are_keys=True)
        q2 = emu.projnorm_rope_store(buf, H, G, D, D, qg, kg, 1e-5, rot, tb, slots, kc2, vc2, page, values_are_keys=True)
        tol = 3e-6 if dtype == torch.float32 else 8e-3
        close(q1, q2, tol)
        close(kd, kc2, tol)
        close(vd, vc2, tol)
        # the values are the rows' key columns as they came
        pg, off = (slots // page).long(), (slots % page).long()
        want = buf[:, H * D:(H + G) * D].view(T, G, D).to(dtype)
        assert torch.equal(vd.cpu()[pg, :, :, off], want)


def capped_attention(q, keys, values, q_pos, scale, window, cap):
    H, G, L = q.shape[1], keys.shape[1], keys.shape[0]
    kh, vh = keys.repeat_interleave(H // G, dim=1).double(), values.repeat_interleave(H // G, dim=1).double()
    sc = torch.einsum("ihd,jhd->hij", q.double(), kh) * scale
    if cap:
        sc = cap * torch.tanh(sc / cap)
    i, j = torch.as_tensor(q_pos)[:, None], torch.arange(L)[None, :]
    vis = (j <= i) & (i - j < (window or L + 1))
    p = torch.softmax(sc.masked_fill(~vis[None], -math.inf), -1)
    return torch.einsum("hij,jhd->ihd", p, vh)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,Dk,Dv", [(4, 2, 24, 16), (6, 1, 64, 64), (3, 3, 10, 10), (8, 2, 96, 96), (2, 1, 32, 48)])
def test_capped_scores(dtype, H, G, Dk, Dv):
    """Prompts, a portion deep in its sequence, portions of two tokens, single tokens (few keys, and enough
    for shares of the keys); scores several times the cap, so that leaving it out shows."""
    hip, _ = tables(dtype)
    g = torch.Generator().manual_seed(H + Dk)
    page, cap = 16, 2.0
    seqs = [(0, 70), (45, 19), (0, 2), (61, 2), (0, 1), (16, 1), (700, 1), (31, 1)]
    lens = [a + b for a, b in seqs]
    for window in (None, 9, 40):
        tbl, kc, vc = paged(lens, page, G, Dk, Dv, dtype, g)
        keys = [(1.5 * torch.randn(n, G, Dk, generator=g)).to(dtype) for n in lens]
        values = [torch.randn(n, G, Dv, generator=g).to(dtype) for n in lens]
        fill_pages(tbl, kc, vc, keys, values, page)
        T = sum(b for _, b in seqs)
        q = (1.5 * torch.randn(T, H * Dk, generator=g)).to(dtype)
        cu, pos, at, want, loose = [0], [], 0, [], []
        for s, (a, b) in enumerate(seqs):
            qs = q[at:at + b].reshape(b, H, Dk)
            want.append(capped_attention(qs, keys[s], values[s], list(range(a, a + b)), 0.5, window, cap))
            loose.append(capped_attention(qs, keys[s], values[s], list(range(a, a + b)), 0.5, window, None))
            pos += list(range(a, a + b))
            at += b
            cu.append(at)
        batch = SimpleNamespace(cu_q=torch.tensor(cu, dtype=torch.int32, device=DEV),
                                positions=torch.tensor(pos, dtype=torch.int32, device=DEV), num_seqs=len(seqs),
                                num_tokens=T, max_q_len=max(b for _, b in seqs), max_ctx_len=max(lens))
        for part in (slice(0, 4), slice(4, 8)):             # prompts and portions; then single tokens alone
            sub = seqs[part]
            t0, t1 = sum(b for _, b in seqs[:part.start]), sum(b for _, b in seqs[:part.stop])
            b2 = SimpleNamespace(cu_q=(batch.cu_q[part.start:part.stop + 1] - t0).contiguous(),
                                 positions=batch.positions[t0:t1].contiguous(), num_seqs=len(sub), num_tokens=t1 - t0,
                                 max_q_len=max(b for _, b in sub), max_ctx_len=max(a + b for a, b in sub))
            got = hip.window_attention(q[t0:t1].to(DEV), 0, H, G, Dk, Dv, kc.to(DEV), vc.to(DEV), page,
                                       tbl[part].contiguous().to(DEV), b2, 0.5, window, softcap=cap)
            w = torch.cat(want)[t0:t1]
            close(got.view(-1, H, Dv), w, 2e-5 if dtype == torch.float32 else 2e-2)
            assert (torch.cat(loose)[t0:t1] - w).abs().max() > 0.05


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("experts,through,top,T", [(5, 1, 2, 9), (3, 0, 1, 40), (70, 3, 9, 33), (1, 3, 4, 7), (8, 2, 3, 700),
                                                   (4, 1, 2, 1500)])
def test_experts_routed_by_shares_with_a_correction(dtype, experts, through, top, T):
    """The routing against the plain function, then the experts with their clamped gates and the ones
    that hand through; enough tokens for row tiles of 16, 64 and 128 rows."""
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(experts + T)
    width, ff, outputs = 64, 32, experts + through
    logits = torch.randn(T, outputs + 3, generator=g) * 2
    corr = torch.randn(outputs, generator=g) / outputs
    routing = hip.route_tokens(logits.to(DEV), outputs, top, over_all=True, correction=corr.to(DEV), scale=1.5,
                               with_matrices=experts)
    chosen, shares = emu.route_tokens(logits, outputs, top, over_all=True, correction=corr, scale=1.5)
    s = torch.softmax(logits[:, :outputs].double(), -1)
    pick = torch.topk(s + corr.double(), top, dim=-1).indices
    assert torch.equal(chosen.long(), pick)
    assert torch.equal(routing.chosen.cpu(), chosen)
    close(routing.shares, shares, 2e-6)
    wsum = torch.gather(s, 1, pick).sum(-1)
    close(routing.shares.sum(-1), 1.5 * wsum / (wsum + 1e-20), 2e-6)
    if through:
        assert (chosen >= experts).any()
    x = torch.randn(T, width, generator=g).to(dtype)
    w_gu = (2 * torch.randn(experts, 2 * ff, width, generator=g) * width ** -0.5).to(dtype)
    w_d = (torch.randn(experts, width, ff, generator=g) * ff ** -0.5).to(dtype)
    got = hip.routed_experts(x.to(DEV), routing, hip.prepare_expert_matrices(w_gu.to(DEV), gated=True),
                             hip.prepare_expert_matrices(w_d.to(DEV)), None, activation="clamped_swish", gated=True,
                             limit=0.8, pass_through=through > 0)
    want = emu.routed_experts(x, (chosen, shares), w_gu, w_d, None, activation="clamped_swish", gated=True, limit=0.8,
                              pass_through=through > 0)
    close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)
    loose = emu.routed_experts(x, (chosen, shares), w_gu, w_d, None, activation="clamped_swish", gated=True, limit=50.0,
                               pass_through=through > 0)
    assert (loose.float() - want.float()).abs().max() > 0.05                  # (the clamps matter)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 3, 4])
def test_convolution_inside_the_launch_that_turns_and_stores(dtype, taps):
    """q, k and v pass the convolution in the launch that norms, turns and stores them: the same rows,
    pages and last inputs as the two calls one after the other."""
    hip, emu = tables(dtype)
    g = torch.Generator().manual_seed(7 + taps)
    T = sum(Q_LENS)
    batch_d, batch_h = fake_batch(Q_LENS, STARTS, SLOTS, DEV), fake_batch(Q_LENS, STARTS, SLOTS, "cpu")
    for H, G, D, Dv, rot, normed in ((4, 2, 16, 24, 16, False), (3, 3, 10, 6, 4, True), (6, 3, 64, 32, 64, False)):
        C = (H + G) * D + G * Dv
        buf = torch.randn(T, C + 5, generator=g)
        w = 0.6 * torch.randn(C, taps, generator=g)
        qg = 1 + 0.3 * torch.randn(H * D, generator=g) if normed else None
        kg = 1 + 0.3 * torch.randn(G * D, generator=g) if normed else None
        ang = torch.rand(T, rot // 2, generator=g) * 6
        tb = RotaryTables(torch.cos(ang), torch.sin(ang))
        tbd = RotaryTables(tb.cos.to(DEV), tb.sin.to(DEV))
        page = 16
        slots = torch.randperm(8 * page, generator=g)[:T].to(torch.int32)
        kc2, vc2 = torch.zeros(8, G, page, D).to(dtype), torch.zeros(8, G, Dv, page).to(dtype)
        kd, vd = kc2.clone().to(DEV), vc2.clone().to(DEV)
        st = states(6, max(1, (taps - 1) * C) + 2, seed=8)
        s1, s2 = st.clone().to(DEV), st.clone()
        dev = lambda t: None if t is None else t.to(DEV)
        q1 = hip.projnorm_rope_store(buf.to(DEV), H, G, D, Dv, dev(qg), dev(kg), 1e-5, rot, tbd, slots.to(DEV), kd, vd,
                                     page, conv=(w.to(DEV), s1, 0, batch_d, True))
        q2 = emu.projnorm_rope_store(buf, H, G, D, Dv, qg, kg, 1e-5, rot, tb, slots, kc2, vc2, page,
                                     conv=(w, s2, 0, batch_h, True))
        tol = 3e-6 if dtype == torch.float32 else 8e-3
        close(q1, q2, tol)
        close(kd, kc2, tol)
        close(vd, vc2, tol)
        if taps > 1:
            close(s1[sorted(SLOTS)][:, :(taps - 1) * C], s2[sorted(SLOTS)][:, :(taps - 1) * C], 0)
        # and the two calls one after the other on the device give the same bits
        s3 = st.clone().to(DEV)
        k3, v3 = torch.zeros_like(kd), torch.zeros_like(vd)
        rows = hip.short_conv(buf.to(DEV), 0, w.to(DEV), s3, 0, batch_d, True, activation=None)
        q3 = hip.projnorm_rope_store(rows, H, G, D, Dv, dev(qg), dev(kg), 1e-5, rot, tbd, slots.to(DEV), k3, v3, page)
        assert torch.equal(q1, q3) and torch.equal(kd, k3) and torch.equal(vd, v3)


def test_rows_a_norm_left_unfinished_reach_a_matrix_of_odd_rows():
    """A product deferred to the norm that adds it leaves un-normalised rows for the next product to
    finish; a reader whose matrix has rows of a length the fused kernels do not take gets them finished."""
    hip, emu = tables(torch.bfloat16)
    g = torch.Generator().manual_seed(11)
    for M in (1, 3, 16):
        x = torch.randn(M, 64, generator=g).to(torch.bfloat16)
        down = (torch.randn(72, 64, generator=g) / 8).to(torch.bfloat16)
        head = (torch.randn(100, 72, generator=g) / 8).to(torch.bfloat16)
        gate_up = (torch.randn(48, 72, generator=g) / 8).to(torch.bfloat16)
        gain = 1 + 0.3 * torch.randn(72, generator=g)
        resid = torch.randn(M, 72, generator=g)
        r2 = resid.clone()
        want_rows = emu.add_rmsnorm(r2, emu.linear(x, down, None), gain, 1e-5)
        for reader in ("linear", "gated", "rows"):
            r1 = resid.clone().to(DEV)
            d = hip.linear(x.to(DEV), hip.prepare_weight(down.to(DEV), residual_delta=True), None, defer=True)
            if reader == "rows":
                rows = torch.tensor([M - 1, 0], dtype=torch.int32)
                normed = hip.rows_add_rmsnorm(r1, d, rows.to(DEV), gain.to(DEV), 1e-5, fuse=True)
                got = hip.linear(normed, hip.prepare_weight(head.to(DEV)), None, out_f32=True)
                close(got, emu.linear(want_rows[rows.long()], head, None, out_f32=True), 2e-2)
                continue
            normed = hip.add_rmsnorm(r1, d, gain.to(DEV), 1e-5, fuse=True)
            close(r1, r2, 1e-2)
            if reader == "linear":
                got = hip.linear(normed, hip.prepare_weight(head.to(DEV)), None, out_f32=True)
                close(got, emu.linear(want_rows, head, None, out_f32=True), 2e-2)
            else:
                got = hip.gated_linear(normed, hip.prepare_weight(gate_up.to(DEV)), 8)
                close(got, emu.gated_linear(want_rows, gate_up, 8), 2e-2)
