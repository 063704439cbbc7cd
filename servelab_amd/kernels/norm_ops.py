"""Embedding gather, residual add + RMSNorm (with the products the norm runs or adds up itself),
the activation of a gate times its up product, and plain activations."""
import ctypes

import torch

from .values import (Deferred, KernelError, PartialSums, ScaledRows, TiledRows, _c_float, _p,
                     activation_code)


class NormOps:
    # ------------------------------------------------------------ embedding
    def embed(self, ids, table, scale=1.0):
        """The rows of ``table`` at ``ids`` times ``scale``, as the float32 stream [T, H]."""
        T = ids.shape[0]
        V, H = table.shape
        self._check(ids, torch.int32, (T,), "ids")
        self._check(table, self.act_dtype, None, "embedding table")
        out = self._new((T, H), torch.float32)
        self._call("elementwise", "sl_embed", _p(ids), _p(table), _p(out), T, H, V, _c_float(scale))
        return out

    def stream_pair(self, resid, delta, other):
        """[resid + delta | other] as rows [T, 2 H] in the activation dtype: the float32 stream with
        what is still to be added to it (``delta``, or None; a deferred product is run) beside a
        second float32 stream.  Neither stream is changed."""
        T, H = resid.shape
        self._check(resid, torch.float32, None, "residual stream")
        self._check(other, torch.float32, (T, H), "second stream")
        delta = self.materialize(self._fold_deltas(resid, delta))
        if delta is not None:
            self._check(delta, self.act_dtype, (T, H), "delta")
        out = self._new((T, 2 * H))
        self._call("elementwise", "sl_stream_pair", _p(resid), _p(delta), _p(other), _p(out), T, H)
        return out

    def scale_rows(self, x, factor):
        """x *= factor in place (float32 rows, e.g. logits)."""
        self._check(x, torch.float32, None, "rows")
        self._call("norm", "sl_scale", _p(x), _c_float(factor), ctypes.c_longlong(x.numel()))
        return x

    # ---------------------------------------------------------------- norms
    def add_rmsnorm(self, resid, delta, weight, eps, fuse=False):
        """resid += delta (in place, float32); returns the normed rows.  A
        ``Deferred`` delta is run here; with ``fuse`` (the reader takes
        ``ScaledRows``) the product, the add and the norm are one kernel."""
        T, H = resid.shape
        self._check(resid, torch.float32, None, "residual stream")
        self._check(weight, torch.float32, (H,), "norm weight")
        delta = self._fold_deltas(resid, delta)
        if isinstance(delta, Deferred):
            if fuse:
                return self._produce_scaled_rows(resid, delta, weight, eps)
            delta = self.materialize(delta)
        out = self._new((T, H))
        self._call("norm", "sl_add_rmsnorm", _p(resid), *self._delta_args(delta, T, H), None,
                   _p(weight), _p(out), T, H, _c_float(eps))
        return out

    def _fold_deltas(self, resid, delta):
        """A tuple of deltas (sublayers that ran side by side): all but the last are added into
        the stream here; the last is returned for the norm's own add."""
        if not isinstance(delta, (tuple, list)):
            return delta
        values = [d for d in delta if d is not None]
        for d in values[:-1]:
            self.add_into(resid, self.materialize(d))
        return values[-1] if values else None

    def _delta_args(self, delta, T, H):
        """(delta, parts, nparts, T, bias) of the norm kernels for any kind of delta."""
        if isinstance(delta, PartialSums):
            ks = delta.parts.shape[0]
            self._check(delta.parts, torch.float32, (ks, T, H), "partial sums")
            if delta.bias is not None:
                self._check(delta.bias, torch.float32, (H,), "bias")
            return None, _p(delta.parts), ks, T, _p(delta.bias)
        if delta is not None:
            self._check(delta, self.act_dtype, (T, H), "delta")
        return _p(delta), None, 0, T, None

    def rows_add_rmsnorm(self, resid, delta, rows, weight, eps, fuse=False):
        """The normed rows ``rows`` of resid + delta.  The stream is left as it
        is, except that a fused ``Deferred`` delta is added into it."""
        T, H = resid.shape
        R = rows.shape[0]
        self._check(resid, torch.float32, None, "residual stream")
        self._check(weight, torch.float32, (H,), "norm weight")
        self._check(rows, torch.int32, (R,), "rows")
        delta = self._fold_deltas(resid, delta)
        if isinstance(delta, Deferred):
            if fuse and R <= self._fused_rows(H):
                scaled = self._produce_scaled_rows(resid, delta, weight, eps)
                scaled.rows = rows
                return scaled
            delta = self.materialize(delta)
        out = self._new((R, H))
        self._call("norm", "sl_add_rmsnorm", _p(resid), *self._delta_args(delta, T, H), _p(rows),
                   _p(weight), _p(out), R, H, _c_float(eps))
        return out

    def materialize(self, value):
        """The plain tensor of a ``Deferred`` product (anything else is returned as it is)."""
        if isinstance(value, Deferred):
            return self.linear(value.x, value.weight, value.bias)
        if isinstance(value, PartialSums):
            ks, M, N = value.parts.shape
            y = self._new((M, N))
            self._call("gemm", "sl_splitk_reduce", _p(value.parts), _p(value.bias), _p(y), M, N, ks, 0)
            return y
        return value

    def _produce_scaled_rows(self, resid, d, gain, eps):
        x, weight = d.x, d.weight
        M, K = x.shape
        N = weight.shape[0]
        if tuple(resid.shape) != (M, N):
            raise KernelError(f"a delta of shape {[M, N]} does not fit the stream {list(resid.shape)}")
        self._check(x.data if isinstance(x, TiledRows) else x, self.act_dtype, None, "x")
        if d.bias is not None:
            self._check(d.bias, torch.float32, (N,), "bias")
        out = self._new((M, N))
        th = self._producer_copy(weight, M)[1]
        parts = self._new((-(-N // th), 16), torch.float32)
        tiled = M if self.tile_few_rows and M > 1 and N % 32 == 0 else 0     # for the products that read the rows
        self._skinny(x, weight, d.bias, out, M, N, K, resid=resid, next_gain=gain, out_parts=parts,
                     y_tiled=bool(tiled))
        return ScaledRows(out, parts, eps, tiled=tiled)

    def silu_mul(self, gate_up, block=None):
        return self.gate_mul(gate_up, block, "silu")

    def gate_mul(self, gate_up, block=None, activation="silu"):
        """act(gate) * up of rows that hold gate and up interleaved in blocks of ``block`` columns
        (default: halves); ``activation``: "silu", "relu" or "gelu_tanh"."""
        code = activation_code(activation, ("silu", "relu", "gelu_tanh"))
        T, two_i = gate_up.shape
        if two_i % 2:
            raise KernelError("silu_mul: the row must hold gate and up of equal width")
        inter = two_i // 2
        block = inter if block is None else int(block)
        if block < 1 or inter % block:
            raise KernelError(f"silu_mul: block {block} does not divide the width {inter}")
        self._check(gate_up, self.act_dtype, None, "gate_up")
        out = self._new((T, inter))
        self._call("elementwise", "sl_gate_mul", _p(gate_up), _p(out), T, inter, block, code)
        return out

    def activate(self, x, activation):
        """act(x) in place, in float; ``activation``: "silu", "relu", "relu2" (relu squared) or
        "gelu_tanh"."""
        self._check(x, self.act_dtype, None, "x")
        self._call("elementwise", "sl_activate", _p(x), _p(x), ctypes.c_longlong(x.numel()),
                   activation_code(activation, ("silu", "relu", "relu2", "gelu_tanh")))
        return x

    def add_normed_rmsnorm(self, resid, y, y_weight, y_eps, weight, eps, rows=None):
        """A sublayer's output ``y`` joins the float32 stream through an RMS norm of its own, and the
        norm of the sublayer that reads the stream next follows in the same kernel:
        v = resid + y / sqrt(mean(y^2) + y_eps) * y_weight, returned v / sqrt(mean(v^2) + eps) * weight.
        ``rows`` None: every row, and v goes back into ``resid``; else (int32) only those rows are
        computed and returned, and the stream stays as it is."""
        T, H = resid.shape
        self._check(resid, torch.float32, None, "residual stream")
        self._check(y, self.act_dtype, (T, H), "sublayer output")
        self._check(y_weight, torch.float32, (H,), "output norm weight")
        self._check(weight, torch.float32, (H,), "norm weight")
        if rows is not None:
            self._check(rows, torch.int32, (rows.shape[0],), "rows")
        R = T if rows is None else rows.shape[0]
        out = self._new((R, H))
        self._call("norm", "sl_add_normed_rmsnorm", _p(resid), _p(y), _p(y_weight), _c_float(y_eps), _p(rows),
                   _p(weight), _c_float(eps), _p(out), R, H)
        return out
