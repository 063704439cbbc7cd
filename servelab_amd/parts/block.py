"""Arrangements of parts in a block.

PreNormBlock: h += Mixer(Norm1(h)); h += FeedForward(Norm2(h))
(servelab/parallel/tp_model.py:124-133).  The adds are fused into the norm
that follows them, so a block returns its feed-forward output as a pending
delta for the next norm to add.

ParallelBlock: with x = Norm(h), h += Mixer(x) + FeedForward(x): one norm, both
sublayers read its output; the block returns both outputs as its pending delta
(a tuple), which the next norm adds to the stream in float32.

SandwichBlock: h += Norm1b(Mixer(Norm1(h))); h += Norm2b(FeedForward(Norm2(h))): a norm before and
after each sublayer.  The norm on an output and the norm before the next sublayer are one kernel
call, so a block returns its last output with the norm that is still to be applied to it.

StreamReentry: no sublayers; the stream is rewritten as a product of itself and the step's kept
embedding output side by side, plus a vector of the pass: what a stretch of layers that is walked
several times starts every pass with.
"""
from .base import Block, prefixed


class PreNormBlock(Block):
    """``feedforward`` may be None (then there is no second norm either, and the mixer's output is
    the pending delta).  A mixer that keeps caches of several kinds declares them as a list
    (``cache_specs``) and gets the list of bindings."""

    def __init__(self, norm1, mixer, norm2, feedforward,
                 names=("input_layernorm.", "self_attn.", "post_attention_layernorm.", "mlp.")):
        self.norm1, self.mixer, self.norm2, self.feedforward = norm1, mixer, norm2, feedforward
        self.names = tuple(names)

    @property
    def graph_safe(self):
        return all(part.graph_safe for _, part in self._children())

    def _children(self):
        parts = list(zip(self.names, (self.norm1, self.mixer, self.norm2, self.feedforward)))
        return parts if self.feedforward is not None else parts[:2]

    def cache_specs(self):
        several = getattr(self.mixer, "cache_specs", None)
        if several is not None:
            return list(several())
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def param_specs(self):
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        for prefix, part in self._children():
            part.load(prefixed(prefix, tensors), rt)

    def forward(self, resid, delta, batch, caches, shared):
        x = self.norm1.forward(resid, delta, fuse=self.mixer.takes_scaled_rows)
        if hasattr(self.mixer, "cache_specs"):
            a = self.mixer.forward(x, batch, caches, shared)
        else:
            a = self.mixer.forward(x, batch, caches[0] if caches else None, shared)
        if self.feedforward is None:
            return a
        x2 = self.norm2.forward(resid, a, fuse=self.feedforward.takes_scaled_rows)
        return self.feedforward.forward(x2)


class StreamReentry(Block):
    """What stands before every pass over a run of layers that is walked several times: the
    stream becomes W [x; x0] + step[t], x the stream as the layers before left it, x0 the
    embedding output of the same tokens, W [width, 2 width] (x's columns first), step [passes,
    width] and t = 0, 1, ... the number of the pass.  The run list calls the block once per
    pass; which pass it is, the block counts in the step's ``shared`` dict.  It needs
    ``ModelSpec.keeps_embedding`` and caches nothing.  The product's sums are float32 and become
    the stream as they are."""
    graph_safe = True

    def __init__(self, hidden_size, passes, names=("in", "step")):
        self.hidden_size, self.passes = int(hidden_size), int(passes)
        self.names = tuple(names)

    def param_specs(self):
        from .base import ParamSpec
        h = self.hidden_size
        return {self.names[0]: ParamSpec((h, 2 * h)), self.names[1]: ParamSpec((self.passes, h))}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.linear_weight(tensors(self.names[0]))
        self.steps = rt.vector(tensors(self.names[1]))

    def forward(self, resid, delta, batch, caches, shared):
        ops = self.rt.ops
        t = shared.get(("pass", id(self)), 0)
        if t >= self.passes:
            raise RuntimeError("the run list enters a repeated stretch more often than it has passes")
        shared[("pass", id(self))] = t + 1
        x0 = shared.get("embedding output")
        if x0 is None:
            raise RuntimeError("the embedding output was not kept for this step")
        rows = ops.stream_pair(resid, delta, x0)
        resid.copy_(ops.linear(rows, self.weight, self.steps[t], out_f32=True))
        shared.pop("stream rows", None)
        return None


class ParallelBlock(Block):
    """``feedforward`` may be None: the mixer alone."""

    def __init__(self, norm, mixer, feedforward, names=("norm.", "mixer.", "mlp.")):
        self.norm, self.mixer, self.feedforward = norm, mixer, feedforward
        self.names = tuple(names)

    @property
    def graph_safe(self):
        return all(part.graph_safe for _, part in self._children())

    def _children(self):
        parts = [(self.names[0], self.norm), (self.names[1], self.mixer)]
        if self.feedforward is not None:
            parts.append((self.names[2], self.feedforward))
        return parts

    def cache_specs(self):
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def param_specs(self):
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        for prefix, part in self._children():
            part.load(prefixed(prefix, tensors), rt)

    def forward(self, resid, delta, batch, caches, shared):
        x = self.norm.forward(resid, delta)
        a = self.mixer.forward(x, batch, caches[0] if caches else None, shared)
        if self.feedforward is None:
            return a
        return (a, self.feedforward.forward(x))


class PostNormBlock(Block):
    """h += m * Norm1(Mixer(h)); h += m * Norm2(FeedForward(h)): the norms sit on the sublayers'
    outputs (``PostRMSNorm`` parts, which hold m), and the sublayers read the stream itself, as
    rows in the activation dtype that the norm's kernel writes along with its add.  The block
    leaves no pending delta.  ``feedforward`` may be None.  A mixer made of several mixers
    declares its cache needs as a list (``cache_specs``) and gets the list of bindings.

    The rows of the stream travel from block to block in the step's ``shared`` dict; a block of
    another kind that changes the stream has to drop the entry ``"stream rows"``."""

    def __init__(self, norm1, mixer, norm2, feedforward, names=("norm1.", "mix.", "norm2.", "mlp.")):
        self.norm1, self.mixer, self.norm2, self.feedforward = norm1, mixer, norm2, feedforward
        self.names = tuple(names)

    @property
    def graph_safe(self):
        return all(part.graph_safe for _, part in self._children())

    def _children(self):
        parts = [(self.names[0], self.norm1), (self.names[1], self.mixer)]
        if self.feedforward is not None:
            parts += [(self.names[2], self.norm2), (self.names[3], self.feedforward)]
        return parts

    def cache_specs(self):
        several = getattr(self.mixer, "cache_specs", None)
        if several is not None:
            return list(several())
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def param_specs(self):
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        for prefix, part in self._children():
            part.load(prefixed(prefix, tensors), rt)

    def forward(self, resid, delta, batch, caches, shared):
        ops = self.rt.ops
        x = shared.get("stream rows")
        if delta is not None:                 # what a block of another kind left to be added
            for d in (delta if isinstance(delta, (tuple, list)) else (delta,)):
                if d is not None:
                    ops.add_into(resid, ops.materialize(d))
            x = None
        if x is None:
            x = self.norm1.forward_post(resid, None)
        if hasattr(self.mixer, "cache_specs"):
            y = self.mixer.forward(x, batch, caches, shared)
        else:
            y = self.mixer.forward(x, batch, caches[0] if caches else None, shared)
        x = self.norm1.forward_post(resid, ops.materialize(y))
        if self.feedforward is not None:
            x = self.norm2.forward_post(resid, ops.materialize(self.feedforward.forward(x)))
        shared["stream rows"] = x
        return None


class SandwichBlock(Block):
    """A norm before and a norm after each sublayer: h += Norm1b(Mixer(Norm1(h))), then
    h += Norm2b(FeedForward(Norm2(h))), all four of them ``RMSNorm`` parts.  A sublayer's output
    waits, with the norm it has to pass, for the norm that reads the stream next
    (``RMSNorm.normed`` -> ``NormedDelta``), which adds it.  ``feedforward`` may be None (then
    there are no second norms).  Blocks of this kind follow each other or a block that leaves a
    plain delta."""

    def __init__(self, norm1, mixer, norm1b, norm2, feedforward, norm2b,
                 names=("norm1.", "mix.", "norm1b.", "norm2.", "mlp.", "norm2b.")):
        self.norm1, self.mixer, self.norm1b = norm1, mixer, norm1b
        self.norm2, self.feedforward, self.norm2b = norm2, feedforward, norm2b
        self.names = tuple(names)

    @property
    def graph_safe(self):
        return all(part.graph_safe for _, part in self._children())

    def _children(self):
        parts = [(self.names[0], self.norm1), (self.names[1], self.mixer), (self.names[2], self.norm1b)]
        if self.feedforward is not None:
            parts += [(self.names[3], self.norm2), (self.names[4], self.feedforward), (self.names[5], self.norm2b)]
        return parts

    def cache_specs(self):
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def param_specs(self):
        specs = {}
        for prefix, part in self._children():
            for name, spec in part.param_specs().items():
                specs[prefix + name] = spec
        return specs

    def load(self, tensors, rt):
        self.rt = rt
        for prefix, part in self._children():
            part.load(prefixed(prefix, tensors), rt)

    def forward(self, resid, delta, batch, caches, shared):
        x = self.norm1.forward(resid, delta)
        a = self.mixer.forward(x, batch, caches[0] if caches else None, shared)
        pending = self.norm1b.normed(a)
        if self.feedforward is None:
            return pending
        x2 = self.norm2.forward(resid, pending)
        return self.norm2b.normed(self.feedforward.forward(x2))
