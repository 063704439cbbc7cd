"""A feed-forward of routed experts: every token goes through the ``top`` experts with the
largest router logits, weighted by the softmax over those logits only, plus an optional shared
expert that every token takes.  An expert is the gated feed-forward down(act(gate x) * up x)
without biases (``gated`` False: down(act(up x)), from two matrices).  Router logits are float32
sums, with a bias when ``router_bias``.  ``shared_gate``: the shared expert's output is multiplied
by the sigmoid of one number per token, a projection of the input by a [1, width] matrix.

``routing`` "shares": the router's softmax runs over all experts; the ``top`` experts are those
with the largest share + correction_e (``correction``: a stored vector; False: none), and a chosen
expert weighs in with its share (without the correction) over the sum of the chosen shares
(+ 1e-20), times ``route_scale``.  ``pass_through`` n: the router has n more outputs behind the
experts', for experts without matrices whose output is their input.  ``activation``
"clamped_swish" (gated only), with ``limit`` c: g = min(gate x, c), u = clamp(up x, -c, c), and the
expert is down(g sigmoid(1.702 g) (u + 1)).

The experts' matrices are stacked at load ([experts, 2 ff, width] with an expert's gate rows
before its up rows, and [experts, width, ff]); the kernel table sorts the step's (token,
choice) pairs by expert on the device and runs one grouped product over all experts, so a step
is a fixed list of launches whatever the routing.
"""
import torch

from .base import FeedForward, ParamSpec
from .feedforward import GatedMLP, PlainMLP


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size, experts, top, ff, shared_ff=0, names=None, activation="silu", gated=True,
                 router_bias=False, shared_gate=False, routing="top", correction=False, route_scale=1.0,
                 pass_through=0, limit=0.0):
        if not 1 <= top <= experts + int(pass_through):
            raise ValueError("top must be between 1 and the number of experts")
        if activation not in (("silu", "relu", "clamped_swish") if gated else ("silu", "relu", "relu2")):
            raise ValueError(f"RoutedExperts: activation '{activation}' is not supported")
        if routing not in ("top", "shares"):
            raise ValueError("routing is 'top' (softmax over the chosen logits) or 'shares' (over all)")
        if routing == "top" and (correction or pass_through or float(route_scale) != 1.0):
            raise ValueError("a correction, a scale and experts that hand through belong to routing by shares")
        if shared_ff and activation == "clamped_swish":
            raise ValueError("RoutedExperts: a shared expert has no clamped form")
        self.routing, self.correction, self.route_scale = routing, bool(correction), float(route_scale)
        self.pass_through, self.limit = int(pass_through), float(limit)
        self.hidden_size, self.experts, self.top, self.ff = int(hidden_size), int(experts), int(top), int(ff)
        self.activation, self.gated, self.router_bias = activation, bool(gated), bool(router_bias)
        self.names = dict({"router": "router", "router_bias": "router.b", "correction": "correction",
                           "expert": "e{}.", "shared": "shared.",
                           "shared_gate": "shared.sg", "gate": "gate", "up": "up", "down": "down"}, **(names or {}))
        n = self.names
        self.shared = None
        if shared_ff:
            self.shared = GatedMLP(hidden_size, shared_ff, activation, names=(n["gate"], n["up"], n["down"])) \
                if gated else PlainMLP(hidden_size, shared_ff, activation, names=(n["up"], n["down"]))
        self.shared_gate = bool(shared_gate) and self.shared is not None

    @property
    def outputs(self):
        """The router's outputs: the experts and those that hand their input through."""
        return self.experts + self.pass_through

    def param_specs(self):
        n, h, f = self.names, self.hidden_size, self.ff
        specs = {}
        for e in range(self.experts):
            p = n["expert"].format(e)
            if self.gated:
                specs[p + n["gate"]] = ParamSpec((f, h))
            specs[p + n["up"]] = ParamSpec((f, h))
            specs[p + n["down"]] = ParamSpec((h, f))
        specs[n["router"]] = ParamSpec((self.outputs, h))
        if self.router_bias:
            specs[n["router_bias"]] = ParamSpec((self.outputs,))
        if self.correction:
            specs[n["correction"]] = ParamSpec((self.outputs,))
        if self.shared is not None:
            for name, spec in self.shared.param_specs().items():
                specs[n["shared"] + name] = spec
        if self.shared_gate:
            specs[n["shared_gate"]] = ParamSpec((1, h))
        return specs

    def load(self, tensors, rt):
        from .base import prefixed
        self.rt = rt
        n = self.names
        router = tensors(n["router"])
        if self.shared_gate:           # the shared expert's gate is one more row of the router's product
            router = torch.cat([router, tensors(n["shared_gate"]).reshape(1, -1)], 0)
        extra = -router.shape[0] % 8
        if extra:
            router = torch.cat([router, router.new_zeros(extra, router.shape[1])], 0)
        self.w_router = rt.linear_weight(router)
        self.b_router = None
        if self.router_bias:
            b = torch.zeros(router.shape[0], dtype=torch.float32, device=router.device)
            b[:self.outputs] = tensors(n["router_bias"]).float()
            self.b_router = rt.vector(b)
        self.route_correction = rt.vector(tensors(n["correction"])) if self.correction else None
        gate_up, down = [], []
        for e in range(self.experts):
            p = n["expert"].format(e)
            up = tensors(p + n["up"])
            gate_up.append(torch.cat([tensors(p + n["gate"]), up], 0) if self.gated else up)
            down.append(tensors(p + n["down"]))
        prepare = getattr(rt.ops, "prepare_expert_matrices", lambda w, gated=False: w)   # (the kernel table's layout)
        self.w_gate_up = prepare(rt.matrix(torch.stack(gate_up)), gated=self.gated)      # [E, 2 ff | ff, width]
        self.w_down = prepare(rt.matrix(torch.stack(down)))                 # [E, width, ff]
        if self.shared is not None:
            self.shared.load(prefixed(n["shared"], tensors), rt)

    def forward(self, x):
        ops = self.rt.ops
        logits = ops.linear(x, self.w_router, self.b_router, out_f32=True)
        if self.routing == "shares":
            routing = ops.route_tokens(logits, self.outputs, self.top, over_all=True,
                                       correction=self.route_correction, scale=self.route_scale,
                                       with_matrices=self.experts)
            base = ops.materialize(self.shared.forward(x)) if self.shared is not None else None
            return ops.routed_experts(x, routing, self.w_gate_up, self.w_down, base, activation=self.activation,
                                      gated=self.gated, base_gate=logits if self.shared_gate else None,
                                      base_gate_col=self.outputs, limit=self.limit,
                                      pass_through=self.pass_through > 0)
        routing = ops.route_tokens(logits, self.experts, self.top)
        base = ops.materialize(self.shared.forward(x)) if self.shared is not None else None
        if self.gated and self.activation == "silu" and not self.shared_gate:
            return ops.routed_experts(x, routing, self.w_gate_up, self.w_down, base)
        return ops.routed_experts(x, routing, self.w_gate_up, self.w_down, base, activation=self.activation,
                                  gated=self.gated, base_gate=logits if self.shared_gate else None,
                                  base_gate_col=self.experts)
