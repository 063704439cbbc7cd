"""Gated feed-forward: down(act(gate(x)) * up(x)), act = silu (SwiGLU), relu or the tanh form of
gelu, without biases or with one on each of the three products; and the
plain one, down(act(up(x))), act = silu, relu or the square of relu.

Reference: servelab/parallel/tp_model.py:56-68 (two GEMMs, silu, multiply, one
GEMM).  Here gate and up are one GEMM over a matrix that holds the rows of Wg
and Wu interleaved in blocks of 8 (so that one output tile of the few-rows
kernel has a channel's gate and up and can apply silu-multiply itself), then
the down GEMM.
"""
import torch

from .base import FeedForward, ParamSpec


class GatedMLP(FeedForward):
    graph_safe = True
    takes_scaled_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), bias_names=None):
        """``bias_names``: checkpoint names of the gate, up and down biases (None: no biases)."""
        if activation not in ("silu", "relu", "gelu_tanh"):
            raise ValueError(f"GatedMLP: activation '{activation}' is not supported")
        self.activation = activation
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = tuple(names)          # checkpoint names of the gate, up and down matrices
        self.bias_names = None if bias_names is None else tuple(bias_names)

    def param_specs(self):
        h, i = self.hidden_size, self.intermediate_size
        specs = {self.names[0]: ParamSpec((i, h)),
                 self.names[1]: ParamSpec((i, h)),
                 self.names[2]: ParamSpec((h, i))}
        if self.bias_names is not None:
            specs.update({self.bias_names[0]: ParamSpec((i,)), self.bias_names[1]: ParamSpec((i,)),
                          self.bias_names[2]: ParamSpec((h,))})
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        gate, up = tensors(self.names[0]), tensors(self.names[1])
        i, h = self.intermediate_size, self.hidden_size
        self.block = getattr(rt.ops, "GATE_BLOCK", i)
        if i % self.block:
            self.block = i                       # plain [Wg; Wu]
        b = self.block
        self.w_gate_up = rt.linear_weight(torch.stack(
            [gate.reshape(i // b, b, h), up.reshape(i // b, b, h)], 1).reshape(2 * i, h))
        self.w_down = rt.linear_weight(tensors(self.names[2]), delta=True)
        self.b_gate_up = self.b_down = None
        if self.bias_names is not None:      # the biases of gate and up lie as their rows do
            bg, bu = tensors(self.bias_names[0]).float(), tensors(self.bias_names[1]).float()
            self.b_gate_up = rt.vector(torch.stack([bg.reshape(i // b, b), bu.reshape(i // b, b)], 1).reshape(2 * i))
            self.b_down = rt.vector(tensors(self.bias_names[2]))

    def forward(self, x):
        ops = self.rt.ops
        if self.bias_names is not None:
            return ops.gated_mlp(x, self.w_gate_up, self.block, self.w_down, defer=True, activation=self.activation,
                                 bias_gate_up=self.b_gate_up, bias_down=self.b_down)
        if self.activation == "silu":
            return ops.gated_mlp(x, self.w_gate_up, self.block, self.w_down, defer=True)
        return ops.gated_mlp(x, self.w_gate_up, self.block, self.w_down, defer=True, activation=self.activation)


class PlainMLP(FeedForward):
    """down(act(up(x))) without a gate and without biases; ``activation``: "silu", "relu" or
    "relu2" (the square of relu).  ``names``: checkpoint names of the up and down matrices."""
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu",
                 names=("up", "down")):
        if activation not in ("silu", "relu", "relu2"):
            raise ValueError(f"PlainMLP: activation '{activation}' is not supported")
        self.activation = activation
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.names = tuple(names)

    def param_specs(self):
        h, i = self.hidden_size, self.intermediate_size
        return {self.names[0]: ParamSpec((i, h)), self.names[1]: ParamSpec((h, i))}

    def load(self, tensors, rt):
        self.rt = rt
        self.w_up = rt.linear_weight(tensors(self.names[0]))
        self.w_down = rt.linear_weight(tensors(self.names[1]), delta=True)

    def forward(self, x):
        ops = self.rt.ops
        return ops.linear(ops.activate(ops.linear(x, self.w_up, None), self.activation), self.w_down, None)
