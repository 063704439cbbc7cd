"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w in float32; LayerNorm with a gain and
no bias: y = (x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations.

Reference: servelab/attention/triton/paged_attention.py:76-91 and the vector
in tests/test_triton_kernels.py:57-59.  Here the residual add that precedes
every use (servelab/parallel/tp_model.py:131-133) is fused in.
"""
from .base import Norm, ParamSpec


class NormedDelta:
    """A sublayer's output that joins the stream through an RMS norm of its own:
    stream += y / sqrt(mean(y^2) + eps) * weight.  A block hands it on as its pending delta, and
    the RMS norm that reads the stream next does the add and its own norm in one kernel call."""
    __slots__ = ("y", "weight", "eps")

    def __init__(self, y, weight, eps):
        self.y, self.weight, self.eps = y, weight, float(eps)


class RMSNorm(Norm):
    """``offset``: the stored weight w acts as the gain offset + w (1 for weights kept around
    zero); the sum is taken once at load, in float32."""
    graph_safe = True

    def __init__(self, size: int, eps: float, name: str = "weight", offset: float = 0.0):
        self.size = int(size)
        self.eps = float(eps)
        self.name = name
        self.offset = float(offset)

    def param_specs(self):
        return {self.name: ParamSpec((self.size,), init="gain" if not self.offset else "normal")}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.vector(tensors(self.name))
        if self.offset:
            self.weight = (self.weight + self.offset).contiguous()

    def forward(self, resid, delta, fuse=False):
        if isinstance(delta, NormedDelta):
            return self.rt.ops.add_normed_rmsnorm(resid, delta.y, delta.weight, delta.eps, self.weight, self.eps)
        return self.rt.ops.add_rmsnorm(resid, delta, self.weight, self.eps, fuse=fuse)

    def forward_rows(self, resid, delta, rows, fuse=False):
        if isinstance(delta, NormedDelta):
            return self.rt.ops.add_normed_rmsnorm(resid, delta.y, delta.weight, delta.eps, self.weight, self.eps,
                                                  rows=rows)
        return self.rt.ops.rows_add_rmsnorm(resid, delta, rows, self.weight, self.eps, fuse=fuse)

    def normed(self, y):
        """``y`` as a delta that joins the stream through this norm."""
        return NormedDelta(self.rt.ops.materialize(y), self.weight, self.eps)


class LayerNorm(Norm):
    """Layer norm with a gain and no bias, in float32, fused with the residual
    add before it.  ``delta`` may be a tuple of values that are all added (the
    outputs of sublayers that ran side by side).  Its rows are plain normed rows
    (``fuse`` is not taken up)."""
    graph_safe = True

    def __init__(self, size: int, eps: float, name: str = "weight"):
        self.size = int(size)
        self.eps = float(eps)
        self.name = name

    def param_specs(self):
        return {self.name: ParamSpec((self.size,), init="gain")}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.vector(tensors(self.name))

    def forward(self, resid, delta, fuse=False):
        return self.rt.ops.add_layernorm(resid, delta, self.weight, self.eps)

    def forward_rows(self, resid, delta, rows, fuse=False):
        return self.rt.ops.add_layernorm(resid, delta, self.weight, self.eps, rows=rows)


class PostRMSNorm(RMSNorm):
    """An RMS norm on a sublayer's output instead of its input: the stream takes
    ``mult`` times the normed output, and the sublayers read the stream itself.
    ``forward_post(resid, y)`` adds mult * norm(y) into the float32 stream in
    place and returns the stream's rows in the activation dtype, which is what
    the next sublayer reads (``y`` None: only those rows)."""

    def __init__(self, size: int, eps: float, mult: float = 1.0, name: str = "weight"):
        super().__init__(size, eps, name)
        self.mult = float(mult)

    def forward_post(self, resid, y):
        return self.rt.ops.add_postnorm(resid, y, self.weight, self.eps, self.mult)
