"""Layer norm with its residual add, products with one matrix per head, and attention with a window that
keeps the first tokens, a distance bias, a sink and an output gate, with what runs before it (per-head
norms and the cache write of keys and mixed values, or of a latent row with its rotated part).  Their
libraries are compiled when a model first asks for them."""
import ctypes

import torch

from . import build
from .values import KernelError, _c_float, _c_void_p, _p

_ll = ctypes.c_longlong


class WindowOps:
    # shares of the keys for steps of single tokens: one share per this many keys a token sees
    # (the float kernel, the matrix-core kernel)
    WINDOW_SHARE_KEYS = 256
    WINDOW_MAX_SHARES = 16
    WINDOW_MFMA_MAX_SHARES = 32
    WINDOW_MFMA_LDS_BYTES = 160 * 1024

    def _window_mfma_fits(self, q, q_col, Dk, Dv):
        """The matrix-core kernel takes bfloat16, key widths in steps of 32 and value widths in steps
        of 16 whose staged block fits LDS, and q rows that are 16-byte aligned; everything else goes
        to the float kernel."""
        if self.act_dtype != torch.bfloat16 or not self.use_mfma_attention:
            return False
        if Dk % 32 or Dv % 16 or Dk > 1024 or Dv > 512:
            return False
        if 2 * (32 * (Dk + 8) + Dv * 40) > self.WINDOW_MFMA_LDS_BYTES:
            return False
        return q.shape[1] % 8 == 0 and q_col % 8 == 0 and q.data_ptr() % 16 == 0

    def _window_mfma_lib(self, Dk, Dv, in_keys):
        key = ("window_attention_mfma", Dk, Dv, in_keys)
        if key not in self._lib:
            self._lib[key] = build.load(build.unit("window_attention_mfma", "bfloat16", SL_DK=Dk, SL_DV=Dv,
                                                   SL_VK=int(in_keys)))
        return key

    def _lazy(self, stem):
        """The library of ``stem`` for this table's dtype, compiled and loaded at first use."""
        if stem not in self._lib:
            self._lib[stem] = build.load(build.unit(stem, self.dtype_name))
        return stem

    # ---------------------------------------------------------------- norms
    def _plain_deltas(self, deltas):
        """Up to two plain tensors out of what parts hand a norm: nothing, one value, or a tuple of
        values that are all to be added (deferred products are run)."""
        if deltas is None:
            return []
        if not isinstance(deltas, (tuple, list)):
            deltas = [deltas]
        return [self.materialize(d) for d in deltas if d is not None]

    def add_into(self, resid, delta):
        """resid += delta in place (float32 stream, delta in the activation dtype)."""
        self._check(resid, torch.float32, None, "residual stream")
        self._check(delta, self.act_dtype, tuple(resid.shape), "delta")
        self._call("norm", "sl_add_into", _p(resid), _p(delta), _ll(resid.numel()))

    def add_layernorm(self, resid, deltas, weight, eps, rows=None):
        """resid += sum of ``deltas`` (in place, float32), then the layer norm of every row with
        gain ``weight`` and no bias.  ``rows`` (int32): only those rows are normed and returned, and
        the stream is left as it is."""
        T, H = resid.shape
        self._check(resid, torch.float32, None, "residual stream")
        self._check(weight, torch.float32, (H,), "norm weight")
        ds = self._plain_deltas(deltas)
        for d in ds:
            self._check(d, self.act_dtype, (T, H), "delta")
        if len(ds) > 2:
            raise KernelError("a layer norm adds at most two deltas")
        if rows is not None:
            self._check(rows, torch.int32, (rows.shape[0],), "rows")
        R = T if rows is None else rows.shape[0]
        out = self._new((R, H))
        self._call("norm", "sl_add_layernorm", _p(resid), _p(ds[0]) if ds else None,
                   _p(ds[1]) if len(ds) > 1 else None, _p(rows), _p(weight), _p(out), R, H, _c_float(eps))
        return out

    # ------------------------------------------------- one matrix per head
    def head_products(self, x, x_col, heads, x_head, A, y=None, y_col=0, y_head=None):
        """y[t, h, :] = A[h] x[t, h, :]: ``x`` [T, width] holds head h's K values from column
        ``x_col + h * x_head`` on, ``A`` is [heads, N, K].  The result goes to columns
        ``y_col + h * y_head`` of ``y`` (made here as [T, heads * N] when None)."""
        T = x.shape[0]
        H, N, K = A.shape
        if H != heads:
            raise KernelError(f"head_products: {H} matrices for {heads} heads")
        self._check(x, self.act_dtype, None, "x")
        self._check(A, self.act_dtype, None, "head matrices")
        if x.dim() != 2 or x_col < 0 or x_col + (heads - 1) * x_head + K > x.shape[1] or x_head < K:
            raise KernelError("head_products: the heads do not fit the rows of x")
        if y is None:
            y_head = N if y_head is None else y_head
            y = self._new((T, y_col + heads * y_head))
        else:
            self._check(y, self.act_dtype, None, "y")
            y_head = N if y_head is None else y_head
        if y.dim() != 2 or y.shape[0] != T or y_col < 0 or y_col + (heads - 1) * y_head + N > y.shape[1] or y_head < N:
            raise KernelError("head_products: the heads do not fit the rows of y")
        lib = self._lazy("head_gemm")
        item = x.element_size()
        self._call(lib, "sl_head_products", _c_void_p(x.data_ptr() + x_col * item), _ll(x.shape[1]), x_head,
                   _p(A), _c_void_p(y.data_ptr() + y_col * item), _ll(y.shape[1]), y_head, T, heads, N, K)
        return y

    # ------------------------------------------------ before the attention
    def headnorm_store(self, buf, nh, nkv, Dk, Dv, q_gain, k_gain, eps, v_first, lam, slots,
                       k_cache, v_cache, page_size):
        """``buf`` [T, >= (nh + nkv) Dk + nkv Dv] holds q, k and v side by side.  q heads are
        divided by their root mean square and multiplied by ``q_gain`` in place (None: left as they
        are), k heads likewise with ``k_gain`` on their way into the cache; v goes to the cache as
        (1 - lam) v + lam v_first when ``v_first`` (a [T, nkv Dv] view, rows may be strided) is
        given.  ``slots`` None: nothing is written to the cache."""
        T, stride = buf.shape
        self._check(buf, self.act_dtype, None, "q/k/v rows")
        for name, gain in (("q gain", q_gain), ("k gain", k_gain)):
            if gain is not None:
                self._check(gain, torch.float32, (Dk,), name)
        vf_stride = 0
        if v_first is not None:
            if (v_first.dtype != self.act_dtype or v_first.dim() != 2 or v_first.shape != (T, nkv * Dv)
                    or v_first.stride(1) != 1 or not v_first.is_cuda):
                raise KernelError("the other layer's values must be [T, nkv * Dv] rows of this step")
            vf_stride = v_first.stride(0)
        if slots is not None:
            pages = k_cache.shape[0]
            self._check(k_cache, self.act_dtype, (pages, nkv, page_size, Dk), "K pages")
            self._check(v_cache, self.act_dtype, (pages, nkv, Dv, page_size), "V pages")
            self._check(slots, torch.int32, (T,), "slots")
        lib = self._lazy("window_attention")
        self._call(lib, "sl_headnorm_store", _p(buf), stride, T, nh, nkv, Dk, Dv, _p(q_gain), _p(k_gain),
                   _c_float(eps), _p(v_first), vf_stride, _c_float(lam), _p(slots),
                   _p(k_cache) if slots is not None else None, _p(v_cache) if slots is not None else None,
                   page_size)

    def slice_rmsnorm(self, buf, col, n, gain, eps):
        """The RMS norm of columns col .. col + n of every row, times ``gain`` [n], in float32;
        returns [T, n] in the activation dtype."""
        T, stride = buf.shape
        self._check(buf, self.act_dtype, None, "rows")
        self._check(gain, torch.float32, (n,), "gain")
        if col < 0 or col + n > stride:
            raise KernelError("slice_rmsnorm: the slice does not fit the rows")
        out = self._new((T, n))
        self._call(self._lazy("window_attention"), "sl_slice_rmsnorm", _p(buf), stride, col, n, _p(gain),
                   _c_float(eps), T, _p(out))
        return out

    def latent_store(self, buf, nh, D, R, C, down_off, rot, gain, eps, tables, slots, k_cache,
                     page_size, q_out, q_rows=None):
        """``buf`` [T, width] holds nh query heads of D + R channels (``q_rows`` given: those rows
        hold them instead, from column 0) and, from column ``down_off``,
        C + R channels: the first C, RMS-normed with ``gain``, and the last R with their first
        ``rot`` channels rotated by ``tables`` (cos and sin [T, rot / 2]) go to the token's key row
        (``slots`` None: no write); the last R channels of every query head are rotated the same
        way into ``q_out`` [T, nh, C + R] at channel C."""
        T, stride = buf.shape
        self._check(buf, self.act_dtype, None, "projected rows")
        q_rows = buf if q_rows is None else q_rows
        self._check(q_rows, self.act_dtype, None, "query rows")
        if q_rows.dim() != 2 or q_rows.shape[0] != T or q_rows.shape[1] < nh * (D + R):
            raise KernelError("latent_store: the query rows do not hold the heads")
        self._check(gain, torch.float32, (C,), "latent gain")
        self._check(q_out, self.act_dtype, (T, nh * (C + R)), "q in the latent's space")
        cos = sin = None
        if rot:
            cos, sin = tables.cos, tables.sin
            self._check(cos, torch.float32, (T, rot // 2), "cos")
            self._check(sin, torch.float32, (T, rot // 2), "sin")
        if slots is not None:
            self._check(k_cache, self.act_dtype, (k_cache.shape[0], 1, page_size, C + R), "latent pages")
            self._check(slots, torch.int32, (T,), "slots")
        lib = self._lazy("window_attention")
        self._call(lib, "sl_latent_store", _p(q_rows), q_rows.shape[1], _p(buf), stride, T, nh, D, R, C, down_off,
                   rot, _p(gain),
                   _c_float(eps), _p(cos), _p(sin), _p(slots), _p(k_cache) if slots is not None else None,
                   page_size, _p(q_out))

    # ------------------------------------------------------------ attention
    def window_attention(self, q, q_col, nh, nkv, Dk, Dv, k_cache, v_cache, page_size, block_tables,
                         batch, scale, window, keep_first=0, slopes=None, sinks=None, gate=None,
                         gate_col=0, softcap=None):
        """Attention of every token of the batch over its sequence's pages.  ``q`` [T, width]
        holds head h of a token at column ``q_col + h * Dk``; ``v_cache`` None: values are the
        first Dv channels of the key rows.  ``window`` (None: all keys) and ``keep_first``: the
        query at position i sees key j <= i when i - j < window or j < keep_first.  ``slopes``
        [nh]: slope_h * (i - j) is taken off the scaled score; ``sinks`` [nh]: exp(sink_h) joins
        the denominator; ``gate`` [T, width] with head h's gate at column ``gate_col + h``: the
        output is multiplied by its sigmoid.  ``softcap`` c: the scaled score s becomes
        c tanh(s / c).  Returns [T, nh * Dv]."""
        T = q.shape[0]
        S, max_pages = block_tables.shape
        self._check(q, self.act_dtype, None, "q")
        if q.dim() != 2 or q_col < 0 or q_col + nh * Dk > q.shape[1]:
            raise KernelError("window_attention: the heads do not fit the rows of q")
        pages = k_cache.shape[0]
        self._check(k_cache, self.act_dtype, (pages, nkv, page_size, Dk), "K pages")
        if v_cache is not None:
            self._check(v_cache, self.act_dtype, (pages, nkv, Dv, page_size), "V pages")
        elif Dv > Dk:
            raise KernelError("window_attention: values read from key rows cannot be wider than a key")
        self._check(block_tables, torch.int32, None, "block tables")
        self._check(batch.cu_q, torch.int32, (S + 1,), "cu_q")
        self._check(batch.positions, torch.int32, (T,), "positions")
        if S != batch.num_seqs or T != batch.num_tokens:
            raise KernelError(f"block tables hold {S} sequences, the batch {batch.num_seqs}")
        if batch.max_ctx_len > max_pages * page_size:
            raise KernelError("block table is shorter than the context")
        for name, v in (("slopes", slopes), ("sinks", sinks)):
            if v is not None:
                self._check(v, torch.float32, (nh,), name)
        gate_stride = 0
        if gate is not None:
            self._check(gate, self.act_dtype, None, "gate")
            if gate.dim() != 2 or gate.shape[0] != T or gate_col < 0 or gate_col + nh > gate.shape[1]:
                raise KernelError("window_attention: the gates do not fit their rows")
            gate_stride = gate.shape[1]
        window = int(window or 0)
        # shares of the keys: for steps of single tokens only, by the number of keys a token can see
        # there; fixed by sizes that a captured step keeps.  (A prompt's tiles are not cut: measured at
        # 2,048 tokens, two shares a tile save 35 us of attention over four layers and their merging
        # costs 186 us.)
        mfma = self._window_mfma_fits(q, q_col, Dk, Dv)
        nsplit = 1
        if batch.max_q_len == 1:
            span = batch.max_ctx_len if not window else min(batch.max_ctx_len, window + int(keep_first))
            if mfma:
                # a workgroup for every CU, a block of 32 keys a share at least
                nsplit = max(1, min(self.WINDOW_MFMA_MAX_SHARES, span // 32, self._num_cus // max(1, S * nkv)))
            else:
                nsplit = max(1, min(self.WINDOW_MAX_SHARES, span // self.WINDOW_SHARE_KEYS))
        part_o = part_ml = None
        if nsplit > 1:
            part_o = self._new((T, nh, nsplit, Dv), torch.float32)
            part_ml = self._new((T, nh, nsplit, 2), torch.float32)
        out = self._new((T, nh * Dv))
        item = q.element_size()
        if mfma:
            lib = self._window_mfma_lib(Dk, Dv, v_cache is None)
            name = f"sl_window_attention_mfma@{Dk}.{Dv}.{int(v_cache is None)}"
            if name not in self._fn:
                fn = self._lib[lib].sl_window_attention_mfma
                fn.restype = ctypes.c_char_p
                self._fn[name] = fn
        else:
            lib, name = self._lazy("window_attention"), "sl_window_attention"
        self._call(lib, name, _c_void_p(q.data_ptr() + q_col * item), q.shape[1], _p(k_cache),
                   _p(v_cache), _p(block_tables), max_pages, _p(batch.cu_q), _p(batch.positions),
                   S, batch.max_q_len, T, nh, nkv, Dk, Dv, page_size, _c_float(scale),
                   _c_float(float(softcap or 0.0)), window,
                   int(keep_first), _p(slopes), _p(sinks),
                   _c_void_p(gate.data_ptr() + gate_col * item) if gate is not None else None, gate_stride,
                   _p(out), nsplit, _p(part_o), _p(part_ml))
        return out
