"""Token embedding and output head.

Embedding lookup servelab/parallel/tp_model.py:123; head = embedding table when
tied, else its own matrix, no bias, logits returned in float32
(servelab/parallel/tp_model.py:115-119, servelab/engine/engine.py:218).
"""
from .base import Embedding, Part, ParamSpec


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, name: str = "weight", scale: float = 1.0):
        """``scale``: the rows of the table enter the stream multiplied by it (in float32)."""
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.name = name
        self.scale = float(scale)

    def param_specs(self):
        return {self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.matrix(tensors(self.name))

    def forward(self, batch):
        """The rows of the table at ``batch.ids`` (int32 [T]) as the float32
        residual stream [T, H]."""
        if self.scale != 1.0:
            return self.rt.ops.embed(batch.ids, self.weight, self.scale)
        return self.rt.ops.embed(batch.ids, self.weight)


class OutputHead(Part):
    graph_safe = True
    takes_scaled_rows = True

    """``tied_to`` is the embedding part whose table the head shares, or None.
    ``softcap`` c: the logits become c * tanh(logits / c), in float32.  ``scale``: the logits
    are multiplied by it, in float32 (a tied table is used as it is stored, whatever scale the
    embedding applies to its rows)."""

    def __init__(self, vocab_size: int, hidden_size: int, tied_to=None, name: str = "weight",
                 softcap=None, scale=None):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to
        self.name = name
        self.softcap = float(softcap) if softcap else None
        self.scale = None if scale is None or float(scale) == 1.0 else float(scale)

    def param_specs(self):
        if self.tied_to is not None:
            return {}
        return {self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors, rt):
        self.rt = rt
        if self.tied_to is not None:
            self.weight = rt.linear_weight(self.tied_to.weight, shared=True)
        else:
            self.weight = rt.linear_weight(tensors(self.name))

    def forward(self, rows):
        """normed rows [R, H] -> float32 logits [R, V]."""
        logits = self.rt.ops.linear(rows, self.weight, None, out_f32=True)
        if self.scale is not None:
            logits = self.rt.ops.scale_rows(logits, self.scale)
        if self.softcap is not None:
            logits = self.rt.ops.softcap(logits, self.softcap)
        return logits
