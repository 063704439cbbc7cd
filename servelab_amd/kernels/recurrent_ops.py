"""Calls for mixers that keep a matrix per head in a state slot, for a softmax attention whose q
and k are normed over the whole projection, for an RMS norm on a sublayer's output, and for
routed experts.  Their libraries (``recurrent``, ``routed``) are compiled when a model first
asks for them.

What is float32 here in both activation types: the input projections' sums as these calls read
them, gates, decays and their logarithms, unit norms, states, read-outs, router logits and
shares, the experts' weighted sum."""
import ctypes
from typing import NamedTuple

import torch

from .values import KernelError, _c_float, _p, activation_code

_ll = ctypes.c_longlong

_EXPAND_MODES = {"plain": 0, "log_sigmoid": 1, "rate_softplus": 2}
_SCAN_DECAY, _SCAN_DELTA, _SCAN_LSTM, _SCAN_SSD = 0, 1, 2, 3
_TILE_ROWS = (16, 64, 128)    # rows of a row tile of the grouped products (routed.hip)


class Routing(NamedTuple):
    """A step's routing on the device: per token the chosen experts [T, top] (int32) and their
    shares (float32); the (token, choice) pairs sorted by expert (``order`` [T top], ``place_of``
    its inverse) and the row tiles [max_tiles, 3] = (expert, first row, rows) of at most
    ``tile_rows`` rows that the grouped products walk."""
    chosen: torch.Tensor
    shares: torch.Tensor
    order: torch.Tensor
    place_of: torch.Tensor
    tiles: torch.Tensor
    tile_rows: int


class ExpertMatrices:
    """The stacked matrices [E, N, K] of a set of experts as the grouped products read them:
    row-major, or (bfloat16, N in steps of 16, K in steps of 32) every expert's matrix in the tiled
    layout of the few-rows products, in which a wavefront's load is 1 KB of consecutive memory."""
    __slots__ = ("data", "shape", "tiled")

    def __init__(self, data, shape, tiled):
        self.data, self.shape, self.tiled = data, tuple(shape), bool(tiled)


class RecurrentOps:
    ROUTED_WIDE_TILE_ROWS = 48    # rows an expert has on average from which row tiles hold 64 rows

    # ------------------------------------------------- norm on an output
    def add_postnorm(self, resid, y, weight, eps, mult):
        """resid += mult * y / sqrt(mean(y^2) + eps) * weight in place (float32); returns the
        stream's rows in the activation dtype.  ``y`` None: only those rows."""
        T, H = resid.shape
        self._check(resid, torch.float32, None, "residual stream")
        self._check(weight, torch.float32, (H,), "norm weight")
        if y is not None:
            self._check(y, self.act_dtype, (T, H), "sublayer output")
        out = self._new((T, H))
        self._call("norm", "sl_add_postnorm", _p(resid), _p(y), _p(weight), _p(out), T, H, _c_float(eps),
                   _c_float(mult))
        return out

    def scaled_sum(self, a, sa, b, sb):
        self._check(a, self.act_dtype, None, "a")
        self._check(b, self.act_dtype, tuple(a.shape), "b")
        out = self._new(tuple(a.shape))
        self._call("norm", "sl_scaled_sum", _p(a), _c_float(sa), _p(b), _c_float(sb), _p(out), _ll(a.numel()))
        return out

    def softcap(self, logits, cap):
        """logits <- cap * tanh(logits / cap), in place (float32)."""
        self._check(logits, torch.float32, None, "logits")
        self._call("norm", "sl_softcap", _p(logits), _c_float(cap), _ll(logits.numel()))
        return logits

    # ------------------------------------------------- what a scan reads
    def _f32_rows(self, t, name):
        self._check(t, torch.float32, None, name)
        if t.dim() != 2:
            raise KernelError(f"{name} must be rows [T, width]")
        return t.shape

    def _sequences(self, batch, T):
        self._check(batch.cu_q, torch.int32, (batch.num_seqs + 1,), "cu_q")
        self._check(batch.positions, torch.int32, (T,), "positions")
        self._check(batch.tok_seq, torch.int32, (T,), "tok_seq")
        self._check(batch.state_slots, torch.int32, (batch.num_seqs,), "state slots")
        if T != batch.num_tokens:
            raise KernelError(f"{T} rows for a batch of {batch.num_tokens} tokens")

    def _state(self, state, need):
        self._check(state, torch.float32, None, "state")
        if state.dim() != 2 or state.shape[1] < need:
            raise KernelError(f"state slots of {list(state.shape[1:])} values, {need} needed")
        return state.shape[1]

    def lowrank_expand(self, buf, col, w2, bias, mode, heads=1, divisor=1.0, rates=None):
        """z = buf[:, col:col + rank] w2^T + bias as float32 [T, C]: "plain" z, "log_sigmoid"
        logsigmoid(z) / divisor, "rate_softplus" -exp(rates[h]) softplus(z) with h = c // (C / heads)."""
        T, stride = self._f32_rows(buf, "projected rows")
        C, rank = w2.shape
        self._check(w2, torch.float32, None, "expansion matrix")
        if bias is not None:
            self._check(bias, torch.float32, (C,), "bias")
        if rates is not None:
            self._check(rates, torch.float32, (heads,), "rates")
        if mode not in _EXPAND_MODES:
            raise KernelError(f"lowrank_expand: unknown mode {mode!r}")
        out = self._new((T, C), torch.float32)
        self._call(self._lazy("recurrent"), "sl_lowrank_expand", _p(buf), stride, col, rank, _p(w2), _p(bias), T, C,
                   _EXPAND_MODES[mode], _c_float(divisor), _p(rates), heads, _p(out))
        return out

    def short_conv(self, buf, col, taps, state, state_off, batch, write, unit_heads=0, unit_dim=0,
                   unit_eps=1e-6, scaled_heads=0, scale=1.0, bias=None, activation="silu"):
        """silu (``activation`` None: nothing) of a causal convolution over time per channel of buf[:, col:col + C] (``taps``
        [C, n], the last one the token's own; ``bias`` [C] is added before the silu).  The n - 1 inputs before a step come from the
        sequence's state slot at ``state_off`` ([n - 1, C], zeros at a sequence's start), and the
        step's last n - 1 inputs go back there.  The first ``unit_heads`` heads of ``unit_dim``
        channels are divided by sqrt(sum x^2 + unit_eps), the first ``scaled_heads`` of them also
        multiplied by ``scale``.  Returns float32 [T, C]."""
        T, stride = self._f32_rows(buf, "projected rows")
        C, n = taps.shape
        self._check(taps, torch.float32, None, "taps")
        if activation not in (None, "silu"):
            raise KernelError("short_conv: the activation is silu or None")
        if bias is not None:
            self._check(bias, torch.float32, (C,), "convolution bias")
        self._sequences(batch, T)
        slot_size = self._state(state, state_off + (n - 1) * C)
        out = self._new((T, C), torch.float32)
        self._call(self._lazy("recurrent"), "sl_short_conv", _p(buf), stride, col, C, n, _p(taps), _p(bias), _p(state),
                   _ll(slot_size), state_off, _p(batch.cu_q), _p(batch.positions), _p(batch.tok_seq),
                   _p(batch.state_slots), batch.num_seqs, T, int(bool(write)), unit_heads, unit_dim,
                   _c_float(unit_eps), scaled_heads, _c_float(scale), int(activation == "silu"), _p(out))
        return out

    def _scan(self, mode, src, q_col, k_col, v_col, H, G, D, Dv, log_decay, q_scale, gates, i_col, f_col,
              cap, state, batch, write, rates=None, step_bias=None, skip=None):
        T, stride = self._f32_rows(src, "q, k, v rows")
        self._sequences(batch, T)
        need = H * Dv * D + (H * D + H if mode == _SCAN_LSTM else 0)
        slot_size = self._state(state, need)
        if log_decay is not None:
            self._check(log_decay, torch.float32, (T, H * D), "log decays")
        gate_stride = 0
        if gates is not None:
            gate_stride = self._f32_rows(gates, "gates")[1]
            if gates.shape[0] != T:
                raise KernelError("gates for another number of tokens")
        out = self._new((T, H * Dv), torch.float32)
        self._call(self._lazy("recurrent"), "sl_matrix_scan", mode, _p(src), stride, q_col, k_col, v_col, H, G,
                   D, Dv, _p(log_decay), _c_float(q_scale), _p(gates), gate_stride, i_col, f_col, _c_float(cap),
                   _p(rates), _p(step_bias), _p(skip), _p(state), _ll(slot_size), _p(batch.cu_q), _p(batch.positions), _p(batch.state_slots),
                   batch.num_seqs, T, int(bool(write)), _p(out))
        return out

    def decay_scan(self, src, q_col, k_col, v_col, H, G, D, Dv, log_decay, q_scale, beta_src, beta_col,
                   state, batch, write):
        """Per head S' = diag(exp(log_decay)) S + k v^T, o = S'^T (q_scale q); with ``beta_src``
        (float32 rows holding beta before its sigmoid at column ``beta_col`` + head) the delta rule:
        S' = diag(..) S, u = sigmoid(beta) (v - S'^T k), S' += k u^T.  q and k have G heads in
        ``src`` (head h reads h // (H / G)).  The slot holds S as [H, Dv, D] from 0 on; a sequence
        whose first token is in the step starts from zero.  Returns float32 [T, H Dv]."""
        if beta_src is None:
            return self._scan(_SCAN_DECAY, src, q_col, k_col, v_col, H, G, D, Dv, log_decay, q_scale, None,
                              0, 0, 1.0, state, batch, write)
        return self._scan(_SCAN_DELTA, src, q_col, k_col, v_col, H, G, D, Dv, log_decay, q_scale, beta_src,
                          beta_col, 0, 1.0, state, batch, write)

    def mlstm_scan(self, buf, q_col, k_col, v_col, i_col, f_col, H, D, Dv, cap, q_scale, state, batch, write):
        """The matrix LSTM: i = cap tanh(i~ / cap), f = logsigmoid(cap tanh(f~ / cap)), m' = max(f + m, i),
        S' = e^(f + m - m') S + e^(i - m') k v^T, n' likewise with k; returns S'^T q / (max(|n' . q|,
        e^-m') + 1e-6) as float32 [T, H Dv].  The slot holds S [H, Dv, D], n [H, D], m [H]; m starts at 0."""
        return self._scan(_SCAN_LSTM, buf, q_col, k_col, v_col, H, H, D, Dv, None, q_scale, buf, i_col, f_col,
                          cap, state, batch, write)

    def ssd_scan(self, src, x_col, b_col, c_col, H, G, N, P, steps, step_col, rates, step_bias, skip,
                 state, batch, write):
        """The state-space recurrence with one decay per head: with dt = softplus(steps[:, step_col + h]
        + step_bias[h]), S' = exp(-exp(rates[h]) dt) S + dt B x^T and y = S'^T C + skip[h] x, where x
        [H, P] lies at column ``x_col`` of ``src`` (float32 rows) and B and C, [G, N] each, at ``b_col``
        and ``c_col`` (head h reads group h // (H / G)).  The slot holds S as [H, P, N] from 0 on; a
        sequence whose first token is in the step starts from zero.  Returns float32 [T, H P]."""
        for name, v in (("rates", rates), ("step biases", step_bias), ("skips", skip)):
            self._check(v, torch.float32, (H,), name)
        return self._scan(_SCAN_SSD, src, c_col, b_col, x_col, H, G, N, P, None, 1.0, steps, step_col, 0, 1.0,
                          state, batch, write, rates=rates, step_bias=step_bias, skip=skip)

    def head_norm_gate(self, o, H, Dv, weight, per_head, eps, gate, gate_col, activation, gate_first=False):
        """Each head of ``o`` [T, H Dv] (float32) divided by its root mean square, times ``weight``
        ([H Dv] when ``per_head``, else [Dv] for every head), times sigmoid or silu of
        gate[:, gate_col + h Dv + d] (float32 rows).  ``gate_first``: the gate is applied before the
        norm (a "head" is then any equal part of the row that is normed by itself).  Returns rows in
        the activation dtype."""
        T, width = self._f32_rows(o, "read-out")
        if width != H * Dv:
            raise KernelError("head_norm_gate: the read-out is not [T, heads * channels]")
        self._check(weight, torch.float32, (H * Dv if per_head else Dv,), "gain")
        gate_stride = self._f32_rows(gate, "gates")[1]
        if gate.shape[0] != T or activation not in ("sigmoid", "silu"):
            raise KernelError("head_norm_gate: gates for another number of tokens, or an unknown activation")
        out = self._new((T, H * Dv))
        self._call(self._lazy("recurrent"), "sl_head_norm_gate", _p(o), T, H, Dv, _p(weight), int(bool(per_head)),
                   _c_float(eps), _p(gate), gate_stride, gate_col, 0 if activation == "sigmoid" else 1,
                   int(bool(gate_first)), _p(out))
        return out

    # ------------------------------- attention: norm over the projection, rotation, pages
    CONV_IN_STORE_MAX_CHANNELS = 12288    # (a token's convolved row waits in 48 KB of LDS)

    def projnorm_rope_store(self, buf, H, G, D, Dv, q_gain, k_gain, eps, rot, tables, slots, k_cache, v_cache,
                            page_size, values_are_keys=False, conv=None):
        """``buf`` (float32) holds q [H D], k [G D] and v [G Dv] side by side.  q and k are
        RMS-normed over all their heads at once (gains of that size; both None: no norm), the first ``rot`` channels of
        every head rotated in halves by ``tables``; k and v go to the token's place in the pages
        (``slots`` None: no write); q comes back as [T, H D] in the activation dtype.
        ``values_are_keys``: there is no v in ``buf``; the values cached are the keys as they lie
        in ``buf``, before norm and rotation (Dv = D).  ``conv`` = (taps [C, n], state, state_off, batch,
        write): q, k and v (the row's first C channels) first pass the short causal convolution of
        ``short_conv`` without bias and activation, in the same launch; the state's last inputs are
        renewed when ``write``."""
        T, stride = self._f32_rows(buf, "projected rows")
        if conv is not None and conv[0].shape[0] > self.CONV_IN_STORE_MAX_CHANNELS:
            taps, state, state_off, batch, write = conv
            buf = self.short_conv(buf, 0, taps, state, state_off, batch, write, activation=None)
            stride, conv = buf.shape[1], None
        if values_are_keys and Dv != D:
            raise KernelError("projnorm_rope_store: keys that serve as values have the values' width")
        if (q_gain is None) != (k_gain is None):
            raise KernelError("projnorm_rope_store: both gains or neither")
        if q_gain is not None:
            self._check(q_gain, torch.float32, (H * D,), "q gain")
            self._check(k_gain, torch.float32, (G * D,), "k gain")
        cos = sin = None
        if rot:
            cos, sin = tables.cos, tables.sin
            self._check(cos, torch.float32, (T, rot // 2), "cos")
            self._check(sin, torch.float32, (T, rot // 2), "sin")
        if slots is not None:
            pages = k_cache.shape[0]
            self._check(k_cache, self.act_dtype, (pages, G, page_size, D), "K pages")
            self._check(v_cache, self.act_dtype, (pages, G, Dv, page_size), "V pages")
            self._check(slots, torch.int32, (T,), "slots")
        q = self._new((T, H * D))
        self._call(self._lazy("recurrent"), "sl_projnorm_rope_store", _p(buf), stride, T, H, G, D, Dv, _p(q_gain),
                   _p(k_gain), _c_float(eps), rot, _p(cos), _p(sin), _p(slots),
                   _p(k_cache) if slots is not None else None, _p(v_cache) if slots is not None else None,
                   page_size, _p(q), H * D if values_are_keys else (H + G) * D, *self._conv_args(conv, T, stride))
        return q

    def _conv_args(self, conv, T, stride):
        """The convolution's part of ``sl_projnorm_rope_store``'s arguments."""
        if conv is None:
            return (None, 0, 0, None, _ll(0), 0, None, None, None, None, 0, 0)
        taps, state, state_off, batch, write = conv
        C, n = taps.shape
        self._check(taps, torch.float32, None, "taps")
        self._sequences(batch, T)
        slot_size = self._state(state, state_off + (n - 1) * C)
        if C > stride:
            raise KernelError("projnorm_rope_store: the convolution's channels do not fit the rows")
        return (_p(taps), n, C, _p(state), _ll(slot_size), state_off, _p(batch.cu_q), _p(batch.positions),
                _p(batch.tok_seq), _p(batch.state_slots), batch.num_seqs, int(bool(write)))

    # ------------------------------------------------------- routed experts
    def route_tokens(self, logits, experts, top, over_all=False, correction=None, scale=1.0, with_matrices=None):
        """The ``top`` largest of each row's first ``experts`` logits (float32; among equals the
        lower index) with the softmax over them, and the step's (token, choice) pairs sorted by
        expert for the grouped products.  ``over_all``: what is compared is the softmax over all
        ``experts`` logits plus ``correction`` [experts] (None: nothing), and a chosen expert's
        share is its softmax value over the sum of the chosen ones' (+ 1e-20), times ``scale``.
        ``with_matrices``: only the first so many experts have matrices (the others get no row
        tiles; ``routed_experts`` hands their input through)."""
        T, stride = self._f32_rows(logits, "router logits")
        n = T * top
        # larger row tiles once an expert has that many rows on average: its matrices are then read
        # once per 64 or 128 rows instead of once per 16
        per_expert = n / (experts if with_matrices is None else max(1, int(with_matrices)))
        tile_rows = _TILE_ROWS[2] if per_expert >= 2 * self.ROUTED_WIDE_TILE_ROWS else \
            (_TILE_ROWS[1] if per_expert >= self.ROUTED_WIDE_TILE_ROWS else _TILE_ROWS[0])
        max_tiles = -(-n // tile_rows) + experts
        chosen = self._new((T, top), torch.int32)
        shares = self._new((T, top), torch.float32)
        order = self._new((n,), torch.int32)
        place_of = self._new((n,), torch.int32)
        tiles = self._new((max_tiles, 3), torch.int32)
        if correction is not None:
            self._check(correction, torch.float32, (experts,), "correction")
        real = experts if with_matrices is None else int(with_matrices)
        self._call(self._lazy("routed"), "sl_route_tokens", _p(logits), stride, T, experts, top, _p(chosen),
                   _p(shares), _p(order), _p(place_of), _p(tiles), max_tiles, tile_rows, int(bool(over_all)),
                   _p(correction), _c_float(scale), real)
        return Routing(chosen, shares, order, place_of, tiles, tile_rows)

    def prepare_expert_matrices(self, w, gated=False):
        """Called once per stack of expert matrices [E, N, K] at load: what ``routed_experts`` takes.
        ``gated``: the stack holds every expert's gate rows before its up rows."""
        E, N, K = w.shape
        self._check(w, self.act_dtype, None, "expert matrices")
        if self.act_dtype != torch.bfloat16 or (N // 2 if gated else N) % 16 or K % 32:
            return ExpertMatrices(w, w.shape, False)
        tiled = torch.empty((E, N * K), dtype=torch.bfloat16, device=self.device)
        for e in range(E):
            self._call("gemm", "sl_tile_weight", _p(w[e]), _p(tiled[e]), N, K, 16)
        return ExpertMatrices(tiled, w.shape, True)

    def routed_experts(self, x, routing, w_gate_up, w_down, base=None, activation="silu", gated=True,
                       base_gate=None, base_gate_col=0, limit=0.0, pass_through=False):
        """sum over a token's choices of share * down_e(act(gate_e x) * up_e x), plus ``base``;
        ``w_gate_up`` [E, 2 ff, width] holds an expert's gate rows before its up rows, ``w_down``
        [E, width, ff].  ``gated`` False: an expert is down_e(act(up_e x)) and ``w_gate_up`` is
        [E, ff, width].  ``base_gate`` (float32 rows): ``base`` is multiplied by the sigmoid of
        base_gate[t, base_gate_col].  ``activation`` "clamped_swish" (gated only): with g = min(gate_e x,
        limit) and u = clamp(up_e x, -limit, limit) the product is g sigmoid(1.702 g) (u + 1).
        ``pass_through``: a chosen expert beyond the E with matrices adds share * x.  Sums are
        float32; what lies between the two products is rounded to the activation dtype."""
        code = activation_code(activation)
        if not isinstance(w_gate_up, ExpertMatrices):
            w_gate_up = ExpertMatrices(w_gate_up, w_gate_up.shape, False)
        if not isinstance(w_down, ExpertMatrices):
            w_down = ExpertMatrices(w_down, w_down.shape, False)
        T, K = x.shape
        E, two_ff, K2 = w_gate_up.shape
        ff = two_ff // 2 if gated else two_ff
        self._check(x, self.act_dtype, None, "x")
        if w_gate_up.shape != (E, two_ff, K) or (gated and two_ff % 2) or w_down.shape != (E, K, ff):
            raise KernelError(f"routed_experts: matrices of {list(w_gate_up.shape)} and {list(w_down.shape)} "
                              f"for rows of {K} values")
        for m in (w_gate_up, w_down):
            self._check(m.data, self.act_dtype, None, "expert matrices")
            if m.data.numel() != E * m.shape[1] * m.shape[2]:
                raise KernelError("routed_experts: expert matrices of another size than they say")
        top = routing.chosen.shape[1]
        n = T * top
        max_tiles = routing.tiles.shape[0]
        if activation == "clamped_swish" and not gated:
            raise KernelError("routed_experts: the clamped form is a gate's")
        if routing.chosen.shape[0] != T or max_tiles < -(-n // routing.tile_rows) + E:
            raise KernelError("routed_experts: the routing is for another step or other experts")
        if base is not None:
            self._check(base, self.act_dtype, (T, K), "base")
        gate_stride = 0
        if base_gate is not None:
            gate_stride = self._f32_rows(base_gate, "base gate")[1]
            if base is None or base_gate.shape[0] != T or not 0 <= base_gate_col < gate_stride:
                raise KernelError("routed_experts: the base's gate does not fit its rows, or there is no base")
        lib = self._lazy("routed")
        mid = self._new((n, ff))
        self._call(lib, "sl_grouped_product", _p(x), _p(routing.order), top, _p(w_gate_up.data),
                   _p(routing.tiles), int(w_gate_up.tiled), max_tiles, routing.tile_rows, ff, K, int(bool(gated)), code,
                   _c_float(limit), _p(mid))
        y = self._new((n, K), torch.float32)
        self._call(lib, "sl_grouped_product", _p(mid), None, 1, _p(w_down.data), _p(routing.tiles),
                   int(w_down.tiled), max_tiles, routing.tile_rows, K, ff, 0, 0, _c_float(0.0), _p(y))
        out = self._new((T, K))
        gate_at = None
        if base_gate is not None:
            gate_at = ctypes.c_void_p(base_gate.data_ptr() + 4 * base_gate_col)
        self._call(lib, "sl_routed_combine", _p(y), _p(routing.place_of), _p(routing.shares), T, top, _p(base),
                   gate_at, gate_stride, K, _p(out), _p(routing.chosen) if pass_through else None, E,
                   _p(x) if pass_through else None)
        return out
