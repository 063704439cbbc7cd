"""Mixers whose memory is a matrix per head, carried from token to token in a state slot.

All of them keep, per head, S [dim, vdim] in float32 and read a token's output as S^T q:

``MatrixLSTM``: scalar gates per head with a running maximum m (m_0 = 0):
    i = cap tanh(i~ / cap), f = logsigmoid(cap tanh(f~ / cap)), m' = max(f + m, i),
    S' = e^(f + m - m') S + e^(i - m') k v^T, n' likewise with k alone,
    o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6);
each head's o divided by its root mean square, a gain over all heads, a sigmoid output gate.

``GatedLinearAttention``: a decay per key channel, alpha = sigmoid(z)^(1/tau) with z from a
low-rank projection plus bias: S' = diag(alpha) S + k v^T; o RMS-normed per head with a gain
shared by the heads, times silu of a full-rank gate.

``GatedDeltaRule``: q, k, v pass a short causal convolution over time and silu; q and k become
unit vectors per head; S' = diag(g) S, u = beta (v - S'^T k), S' += k u^T, o = S'^T q (the
read-out sees the token's own write); g = exp(-exp(A_log_h) softplus(a + dt_bias)) per head and
key channel, a from a low-rank projection; the gain is shared by the heads and the sigmoid
output gate comes from a low-rank projection.  The convolution's last taps - 1 inputs are part
of the state.

``StateSpaceMixer``: one projection gives a gate z, the inputs x, B and C (B and C shared by the
heads of a group) and a step size per head; x, B and C pass a short causal convolution with a bias
and silu; dt = softplus(dt~ + dt_bias_h); S' = exp(-exp(A_log_h) dt) S + dt B x^T (one decay for
the whole head), y = S'^T C + D_h x; y times silu(z), then RMS-normed in equal parts with a gain
over the whole row.  The convolution's last taps - 1 inputs are part of the state.

Gates, decays, unit norms, state and read-out are float32 in both activation types; the input
projection (one product for everything a mixer projects from its input) returns float32 sums.
A state starts from zero at a sequence's first token, whatever the slot held.  Every size and
constant is a constructor parameter, checkpoint names too (``names``).
"""
import torch

from .base import Mixer, ParamSpec, StateSpec


def _rows(blocks):
    """Row-concatenated matrices and where each starts: ({name: first row}, matrix)."""
    at, n = {}, 0
    for name, t in blocks:
        at[name] = n
        n += t.shape[0]
    return at, torch.cat([t for _, t in blocks], 0)


class _MatrixMemoryMixer(Mixer):
    graph_safe = True

    def _project(self, x):
        return self.rt.ops.linear(x, self.w_in, self.b_in, out_f32=True)

    def _load_in(self, blocks, rt, biases=None):
        """One input matrix out of ``blocks`` [(name, tensor)], padded to a multiple of 8 rows;
        ``biases`` {name: tensor} are the rows' biases (others zero)."""
        self.at, w = _rows(blocks)
        extra = -w.shape[0] % 8
        if extra:
            w = torch.cat([w, w.new_zeros(extra, w.shape[1])], 0)
        self.w_in = rt.linear_weight(w)
        self.b_in = None
        if biases:
            b = torch.zeros(w.shape[0], dtype=torch.float32, device=w.device)
            for name, t in biases.items():
                b[self.at[name]:self.at[name] + t.shape[0]] = t.float()
            self.b_in = rt.vector(b)


class MatrixLSTM(_MatrixMemoryMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "norm": "norm",
             "i": "i", "i_bias": "i.b", "f": "f", "f_bias": "f.b"}

    def __init__(self, hidden_size, heads, dim, vdim, gate_cap, norm_eps, names=None):
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(heads), int(dim), int(vdim)
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))

    def param_specs(self):
        n, h, H, D, Dv = self.names, self.hidden_size, self.heads, self.dim, self.vdim
        return {n["q"]: ParamSpec((H * D, h)), n["k"]: ParamSpec((H * D, h)), n["v"]: ParamSpec((H * Dv, h)),
                n["gate"]: ParamSpec((H * Dv, h)), n["out"]: ParamSpec((h, H * Dv)),
                n["norm"]: ParamSpec((H * Dv,), init="gain"),
                n["i"]: ParamSpec((H, h)), n["i_bias"]: ParamSpec((H,)),
                n["f"]: ParamSpec((H, h)), n["f_bias"]: ParamSpec((H,))}

    def cache_spec(self):
        H, D, Dv = self.heads, self.dim, self.vdim
        return StateSpec((H * D * Dv + H * D + H,), "float32")        # S, n, m

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        self._load_in([(x, tensors(n[x])) for x in ("q", "k", "v", "gate", "i", "f")], rt,
                      {"i": tensors(n["i_bias"]), "f": tensors(n["f_bias"])})
        self.gain = rt.vector(tensors(n["norm"]))
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)

    def forward(self, x, batch, cache, shared):
        ops, at = self.rt.ops, self.at
        H, D, Dv = self.heads, self.dim, self.vdim
        buf = self._project(x)
        o = ops.mlstm_scan(buf, at["q"], at["k"], at["v"], at["i"], at["f"], H, D, Dv, self.gate_cap,
                           D ** -0.5, cache.state, batch, cache.write)
        y = ops.head_norm_gate(o, H, Dv, self.gain, True, self.norm_eps, buf, at["gate"], "sigmoid")
        return ops.linear(y, self.w_o, None)


class GatedLinearAttention(_MatrixMemoryMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "norm": "norm",
             "decay_in": "a1", "decay_out": "a2", "decay_bias": "a2.b"}

    def __init__(self, hidden_size, heads, dim, vdim, tau, decay_rank, norm_eps, names=None):
        self.hidden_size, self.heads, self.dim, self.vdim = int(hidden_size), int(heads), int(dim), int(vdim)
        self.tau, self.decay_rank, self.norm_eps = float(tau), int(decay_rank), float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))

    def param_specs(self):
        n, h, H, D, Dv, r = self.names, self.hidden_size, self.heads, self.dim, self.vdim, self.decay_rank
        return {n["q"]: ParamSpec((H * D, h)), n["k"]: ParamSpec((H * D, h)), n["v"]: ParamSpec((H * Dv, h)),
                n["gate"]: ParamSpec((H * Dv, h)), n["out"]: ParamSpec((h, H * Dv)),
                n["norm"]: ParamSpec((Dv,), init="gain"),
                n["decay_in"]: ParamSpec((r, h)), n["decay_out"]: ParamSpec((H * D, r)),
                n["decay_bias"]: ParamSpec((H * D,))}

    def cache_spec(self):
        return StateSpec((self.heads * self.dim * self.vdim,), "float32")

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        self._load_in([(x, tensors(n[x])) for x in ("q", "k", "v", "gate", "decay_in")], rt)
        self.decay_out = rt.vector(tensors(n["decay_out"]))
        self.decay_bias = rt.vector(tensors(n["decay_bias"]))
        self.gain = rt.vector(tensors(n["norm"]))
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)

    def forward(self, x, batch, cache, shared):
        ops, at = self.rt.ops, self.at
        H, D, Dv = self.heads, self.dim, self.vdim
        buf = self._project(x)
        log_decay = ops.lowrank_expand(buf, at["decay_in"], self.decay_out, self.decay_bias,
                                       "log_sigmoid", heads=H, divisor=self.tau)
        o = ops.decay_scan(buf, at["q"], at["k"], at["v"], H, H, D, Dv, log_decay, D ** -0.5,
                           None, 0, cache.state, batch, cache.write)
        y = ops.head_norm_gate(o, H, Dv, self.gain, False, self.norm_eps, buf, at["gate"], "silu")
        return ops.linear(y, self.w_o, None)


class GatedDeltaRule(_MatrixMemoryMixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
             "beta": "b", "rate": "A_log", "norm": "norm", "decay_in": "a1", "decay_out": "a2",
             "decay_bias": "dt_bias", "gate_in": "g1", "gate_out": "g2", "out": "o"}

    def __init__(self, hidden_size, heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank, norm_eps,
                 unit_eps=1e-6, names=None):
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.hidden_size, self.heads, self.kv_heads = int(hidden_size), int(heads), int(kv_heads)
        self.dim, self.vdim, self.conv = int(dim), int(vdim), int(conv)
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.names = dict(self.NAMES, **(names or {}))

    @property
    def channels(self):
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    def param_specs(self):
        n, h = self.names, self.hidden_size
        H, G, D, Dv, taps = self.heads, self.kv_heads, self.dim, self.vdim, self.conv
        return {n["q"]: ParamSpec((G * D, h)), n["q_conv"]: ParamSpec((G * D, taps)),
                n["k"]: ParamSpec((G * D, h)), n["k_conv"]: ParamSpec((G * D, taps)),
                n["v"]: ParamSpec((H * Dv, h)), n["v_conv"]: ParamSpec((H * Dv, taps)),
                n["beta"]: ParamSpec((H, h)), n["rate"]: ParamSpec((H,)),
                n["norm"]: ParamSpec((Dv,), init="gain"),
                n["decay_in"]: ParamSpec((self.decay_rank, h)), n["decay_out"]: ParamSpec((H * D, self.decay_rank)),
                n["decay_bias"]: ParamSpec((H * D,)),
                n["gate_in"]: ParamSpec((self.gate_rank, h)), n["gate_out"]: ParamSpec((H * Dv, self.gate_rank)),
                n["out"]: ParamSpec((h, H * Dv))}

    def cache_spec(self):
        H, D, Dv = self.heads, self.dim, self.vdim
        return StateSpec((H * D * Dv + (self.conv - 1) * self.channels,), "float32")   # S, last inputs

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        self._load_in([(x, tensors(n[x])) for x in ("q", "k", "v", "beta", "decay_in", "gate_in")], rt)
        self.taps = rt.vector(torch.cat([tensors(n[x]) for x in ("q_conv", "k_conv", "v_conv")], 0))
        self.rate = rt.vector(tensors(n["rate"]))
        self.decay_out = rt.vector(tensors(n["decay_out"]))
        self.decay_bias = rt.vector(tensors(n["decay_bias"]))
        self.gate_out = rt.vector(tensors(n["gate_out"]))
        self.gain = rt.vector(tensors(n["norm"]))
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)

    def forward(self, x, batch, cache, shared):
        ops, at = self.rt.ops, self.at
        H, G, D, Dv = self.heads, self.kv_heads, self.dim, self.vdim
        buf = self._project(x)
        # q, k and v lie side by side in the projection: one convolution over all their channels,
        # then q and k heads made unit vectors (q also times dim^-1/2)
        qkv = ops.short_conv(buf, at["q"], self.taps, cache.state, H * D * Dv, batch, cache.write,
                             unit_heads=2 * G, unit_dim=D, unit_eps=self.unit_eps,
                             scaled_heads=G, scale=D ** -0.5)
        log_decay = ops.lowrank_expand(buf, at["decay_in"], self.decay_out, self.decay_bias,
                                       "rate_softplus", heads=H, rates=self.rate)
        o = ops.decay_scan(qkv, 0, G * D, 2 * G * D, H, G, D, Dv, log_decay, 1.0,
                           buf, at["beta"], cache.state, batch, cache.write)
        gate = ops.lowrank_expand(buf, at["gate_in"], self.gate_out, None, "plain", heads=H)
        y = ops.head_norm_gate(o, H, Dv, self.gain, False, self.norm_eps, gate, 0, "sigmoid")
        return ops.linear(y, self.w_o, None)


class StateSpaceMixer(_MatrixMemoryMixer):
    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "step_bias": "dt_bias", "rate": "A_log",
             "skip": "D", "norm": "norm", "out": "o"}

    def __init__(self, hidden_size, heads, vdim, state, groups, conv, norm_groups, norm_eps, names=None):
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("heads must be a multiple of groups, heads * vdim of norm_groups")
        self.hidden_size, self.heads, self.vdim, self.state = int(hidden_size), int(heads), int(vdim), int(state)
        self.groups, self.conv, self.norm_groups = int(groups), int(conv), int(norm_groups)
        self.norm_eps = float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))

    @property
    def inner(self):
        return self.heads * self.vdim

    @property
    def channels(self):
        """What passes the convolution: x, B and C."""
        return self.inner + 2 * self.groups * self.state

    def param_specs(self):
        n, h, H = self.names, self.hidden_size, self.heads
        return {n["in"]: ParamSpec((2 * self.inner + 2 * self.groups * self.state + H, h)),
                n["conv"]: ParamSpec((self.channels, self.conv)), n["conv_bias"]: ParamSpec((self.channels,)),
                n["step_bias"]: ParamSpec((H,)), n["rate"]: ParamSpec((H,)), n["skip"]: ParamSpec((H,)),
                n["norm"]: ParamSpec((self.inner,), init="gain"), n["out"]: ParamSpec((h, self.inner))}

    def cache_spec(self):
        return StateSpec((self.inner * self.state + (self.conv - 1) * self.channels,), "float32")   # S, last inputs

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        w = tensors(n["in"])
        # the projection's rows are [z | x | B | C | dt]
        self._load_in([("z", w[:self.inner]), ("xbc", w[self.inner:self.inner + self.channels]),
                       ("dt", w[self.inner + self.channels:])], rt)
        self.taps = rt.vector(tensors(n["conv"]))
        self.conv_bias = rt.vector(tensors(n["conv_bias"]))
        self.step_bias = rt.vector(tensors(n["step_bias"]))
        self.rate = rt.vector(tensors(n["rate"]))
        self.skip = rt.vector(tensors(n["skip"]))
        self.gain = rt.vector(tensors(n["norm"]))
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)

    def forward(self, x, batch, cache, shared):
        ops, at = self.rt.ops, self.at
        H, P, N, G = self.heads, self.vdim, self.state, self.groups
        buf = self._project(x)
        xbc = ops.short_conv(buf, at["xbc"], self.taps, cache.state, self.inner * N, batch, cache.write,
                             bias=self.conv_bias)
        y = ops.ssd_scan(xbc, 0, self.inner, self.inner + G * N, H, G, N, P, buf, at["dt"], self.rate,
                         self.step_bias, self.skip, cache.state, batch, cache.write)
        # the gate comes before the norm, which takes the row in `norm_groups` equal parts
        y = ops.head_norm_gate(y, self.norm_groups, self.inner // self.norm_groups, self.gain, True,
                               self.norm_eps, buf, at["z"], "silu", gate_first=True)
        return ops.linear(y, self.w_o, None)


class SideBySide(Mixer):
    """Two mixers that read the same rows; the result is left_scale * left + right_scale *
    right.  Each keeps a cache of its own kind: the block hands over one binding for each
    (``cache_specs``)."""

    def __init__(self, left, right, left_scale, right_scale, names=("left.", "right.")):
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.names = tuple(names)

    @property
    def graph_safe(self):
        return self.left.graph_safe and self.right.graph_safe

    def _sides(self):
        return list(zip(self.names, (self.left, self.right)))

    def param_specs(self):
        specs = {}
        for prefix, part in self._sides():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def cache_specs(self):
        return [s for s in (self.left.cache_spec(), self.right.cache_spec()) if s is not None]

    def load(self, tensors, rt):
        from .base import prefixed
        self.rt = rt
        for prefix, part in self._sides():
            part.load(prefixed(prefix, tensors), rt)

    def forward(self, x, batch, caches, shared):
        ops = self.rt.ops
        caches = list(caches)
        a = self.left.forward(x, batch, caches.pop(0) if self.left.cache_spec() is not None else None, shared)
        b = self.right.forward(x, batch, caches.pop(0) if self.right.cache_spec() is not None else None, shared)
        return ops.scaled_sum(ops.materialize(a), self.left_scale, ops.materialize(b), self.right_scale)
