"""Grouped-query attention over a paged cache.

Reference math: q/k/v projections with optional bias, head-major views
(servelab/parallel/tp_model.py:43-53); rotary on q and k before k is cached
(:128-129); per sequence scores * 1/sqrt(D), causal mask, softmax and PV in
float32 with kv head = head // g (:136-157).  The reference runs three GEMMs
and a Python loop over sequences; here q, k and v come from one GEMM over the
row-concatenated weight, the kernel table applies the position encoding (a
parameter this mixer never looks inside) and writes the pages, and one call
attends for all sequences of the batch through their block tables.  The
window (keys p - W < r <= p) is this build's own.

``ProjectionNormAttention`` and ``ShortConvAttention`` are the attention of designs whose softmax
weights stay float32 and whose keys and values differ in width: a norm over the whole projection,
biases, keys that serve as values, capped scores and a short convolution before the rotation are
switches of theirs.
"""
import math

import torch

from .base import Mixer, PagedKVSpec, ParamSpec, StateSpec


class PagedAttention(Mixer):
    graph_safe = True
    takes_scaled_rows = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, position,
                 qkv_bias=True, window=None, scale=None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.position = position
        self.qkv_bias = bool(qkv_bias)
        self.window = None if not window else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)

    # ---- declarations
    def param_specs(self):
        h, d = self.hidden_size, self.head_dim
        specs = {
            "q_proj.weight": ParamSpec((self.num_heads * d, h)),
            "k_proj.weight": ParamSpec((self.num_kv_heads * d, h)),
            "v_proj.weight": ParamSpec((self.num_kv_heads * d, h)),
            "o_proj.weight": ParamSpec((h, self.num_heads * d)),
        }
        if self.qkv_bias:
            specs["q_proj.bias"] = ParamSpec((self.num_heads * d,))
            specs["k_proj.bias"] = ParamSpec((self.num_kv_heads * d,))
            specs["v_proj.bias"] = ParamSpec((self.num_kv_heads * d,))
        return specs

    def cache_spec(self):
        return PagedKVSpec(self.num_kv_heads, self.head_dim, self.window)

    def load(self, tensors, rt):
        self.rt = rt
        self.position.load(tensors, rt)
        # [Wq; Wk; Wv] -> one [(nh + 2 nkv) D, H] matrix, one GEMM.  The kernel table says in
        # which order it wants the channels of every q and k head for this position encoding
        # (q . k does not depend on the order as long as both agree); v keeps its own.
        self.rotation = rt.ops.plan_rotation(self.head_dim, self.position.layout())
        order = self.rotation.order

        def reorder(t, heads):
            if order is None:
                return t
            by_head = t.reshape(heads, self.head_dim, *t.shape[1:])
            return by_head[:, order.to(t.device)].reshape(t.shape)
        self.w_qkv = rt.linear_weight(torch.cat(
            [reorder(tensors("q_proj.weight"), self.num_heads),
             reorder(tensors("k_proj.weight"), self.num_kv_heads), tensors("v_proj.weight")], 0))
        self.b_qkv = None
        if self.qkv_bias:
            self.b_qkv = rt.vector(torch.cat(
                [reorder(tensors("q_proj.bias").float(), self.num_heads),
                 reorder(tensors("k_proj.bias").float(), self.num_kv_heads),
                 tensors("v_proj.bias").float()], 0))
        self.w_o = rt.linear_weight(tensors("o_proj.weight"), delta=True)
        # a kernel table may want part of the score scale applied to q where q is made
        split = getattr(rt.ops, "split_attention_scale", None)
        self.q_scale, self.score_scale = split(self.scale) if split is not None else (1.0, self.scale)

    # ---- compute
    def forward(self, x, batch, cache, shared):
        ops = self.rt.ops
        group = batch.groups[cache.group]
        slots, kc, vc = (group.slots, cache.k, cache.v) if cache.write else (None, None, None)
        qkv = ops.project_qkv(x, self.w_qkv, self.b_qkv, self.num_heads, self.num_kv_heads,
                              self.head_dim, self.rotation, self.position.tables(batch, shared),
                              slots, kc, vc, cache.page_size, q_scale=self.q_scale)
        return ops.attend_and_project(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v,
            cache.page_size, group.block_tables, batch, self.score_scale, self.window,
            self.w_o, None, defer=True)


def _turning_order(rot: int, width: int, pairing: str) -> torch.Tensor:
    """The order that puts ``width`` channels whose first ``rot`` turn in ``pairing`` pairs into
    the order in which they turn in halves (a score does not depend on the order of its terms as
    long as q and k agree)."""
    if pairing == "half" or not rot:
        return torch.arange(width)
    return torch.cat([torch.arange(0, rot, 2), torch.arange(1, rot, 2), torch.arange(rot, width)])


class ProjectionNormAttention(Mixer):
    """Grouped-query softmax attention whose q and k are RMS-normed over the whole projection
    (all heads of a token at once, a gain of that size) before the rotation, with biases on q,
    k, v and the output, keys of ``key_dim`` and values of ``value_dim`` channels, a score
    scale given from outside and float32 softmax weights.  The position encoding turns the
    leading channels of a head, in halves or in neighbouring pairs (the rows that make q and k
    are then put into the order of halves at load).  Causal; ``window`` None keeps every key.
    ``projection_norm`` False: q and k go to the rotation as the projection left them (no gains
    in the checkpoint); ``bias`` False: no biases.  ``values`` "keys": there is no value
    projection; a token's values are its keys as the projection left them (with their bias),
    before norm and rotation.  ``softcap`` c: a scaled score s becomes c tanh(s / c).
    The input goes to nothing but the input product and the output product's result only joins the
    stream, so in steps of few rows a pre-norm block's norms can run the products around them."""
    graph_safe = True
    takes_scaled_rows = True

    NAMES = {"q": "q", "k": "k", "v": "v", "out": "o", "q_bias": "q.b", "k_bias": "k.b",
             "v_bias": "v.b", "out_bias": "o.b", "q_norm": "q.norm", "k_norm": "k.norm"}

    def __init__(self, hidden_size, num_heads, num_kv_heads, key_dim, value_dim, scale, position,
                 norm_eps, bias=True, window=None, names=None, projection_norm=True, values="projected",
                 softcap=None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if values not in ("projected", "keys"):
            raise ValueError("values are 'projected' or 'keys'")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.values_are_keys = values == "keys"
        if self.values_are_keys and self.value_dim != self.key_dim:
            raise ValueError("keys that serve as values have the values' width")
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.position = position
        self.bias = bool(bias)
        self.projection_norm = bool(projection_norm)
        self.window = None if not window else int(window)
        self.softcap = float(softcap) if softcap else None
        self.names = dict(self.NAMES, **(names or {}))

    @property
    def in_channels(self):
        """Channels of the input projection: q, k and (with a value projection) v."""
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        return (H + G) * D + (0 if self.values_are_keys else G * Dv)

    def param_specs(self):
        n, h = self.names, self.hidden_size
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        specs = {n["q"]: ParamSpec((H * D, h)), n["k"]: ParamSpec((G * D, h)), n["out"]: ParamSpec((h, H * Dv))}
        if not self.values_are_keys:
            specs[n["v"]] = ParamSpec((G * Dv, h))
        if self.projection_norm:
            specs.update({n["q_norm"]: ParamSpec((H * D,), init="gain"),
                          n["k_norm"]: ParamSpec((G * D,), init="gain")})
        if self.bias:
            specs.update({n["q_bias"]: ParamSpec((H * D,)), n["k_bias"]: ParamSpec((G * D,)),
                          n["out_bias"]: ParamSpec((h,))})
            if not self.values_are_keys:
                specs[n["v_bias"]] = ParamSpec((G * Dv,))
        return specs

    def cache_spec(self):
        return PagedKVSpec(self.num_kv_heads, self.key_dim, self.window, value_dim=self.value_dim)

    def _by_head(self, t, heads):
        """Rows (or entries) of q or k, every head's channels in the order the rotation wants."""
        by_head = t.reshape(heads, self.key_dim, *t.shape[1:])
        return by_head[:, self.order.to(t.device)].reshape(t.shape)

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        self.position.load(tensors, rt)
        layout = self.position.layout()
        if layout is not None and (layout.pairing not in ("half", "interleaved") or layout.rot_dim > D):
            raise ValueError("the rotation must turn leading channels of a head, in halves or in neighbouring pairs")
        self.rot = 0 if layout is None else int(layout.rot_dim)
        self.order = _turning_order(self.rot, D, "half" if layout is None else layout.pairing)
        rows = [self._by_head(tensors(n["q"]), H), self._by_head(tensors(n["k"]), G)]
        if not self.values_are_keys:
            rows.append(tensors(n["v"]))
        w = torch.cat(rows, 0)
        extra = -w.shape[0] % 8
        if extra:
            w = torch.cat([w, w.new_zeros(extra, w.shape[1])], 0)
        self.w_in = rt.linear_weight(w)
        self.b_in = self.b_o = None
        if self.bias:
            b = [self._by_head(tensors(n["q_bias"]).float(), H), self._by_head(tensors(n["k_bias"]).float(), G)]
            if not self.values_are_keys:
                b.append(tensors(n["v_bias"]).float())
            self.b_in = rt.vector(torch.cat(b + [torch.zeros(extra, device=w.device)], 0))
            self.b_o = rt.vector(tensors(n["out_bias"]))
        self.q_gain = rt.vector(self._by_head(tensors(n["q_norm"]), H)) if self.projection_norm else None
        self.k_gain = rt.vector(self._by_head(tensors(n["k_norm"]), G)) if self.projection_norm else None
        w_o = tensors(n["out"])
        if self.values_are_keys:
            # the values arrive in the keys' order: the output projection's columns follow them
            w_o = w_o.reshape(w_o.shape[0], H, Dv)[:, :, self.order.to(w_o.device)].reshape(w_o.shape)
        self.w_o = rt.linear_weight(w_o, delta=True)

    def forward(self, x, batch, cache, shared):
        buf = self.rt.ops.linear(x, self.w_in, self.b_in, out_f32=True)
        return self._attend(buf, batch, cache, shared)

    def _attend(self, buf, batch, cache, shared, conv=None):
        """``buf``: float32 rows that hold q, k and (with a value projection) v side by side;
        ``conv``: a short convolution they pass first, in the launch that norms, turns and stores."""
        ops = self.rt.ops
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        group = batch.groups[cache.group]
        tables = self.position.tables(batch, shared) if self.rot else None
        store = (buf, H, G, D, Dv, self.q_gain, self.k_gain, self.norm_eps, self.rot,
                 tables, group.slots if cache.write else None, cache.k, cache.v, cache.page_size)
        more = {}
        if self.values_are_keys:
            more["values_are_keys"] = True
        if conv is not None:
            more["conv"] = conv
        q = ops.projnorm_rope_store(*store, **more)
        attend = (q, 0, H, G, D, Dv, cache.k, cache.v, cache.page_size, group.block_tables, batch, self.scale,
                  self.window)
        attn = ops.window_attention(*attend, softcap=self.softcap) if self.softcap else ops.window_attention(*attend)
        return ops.linear(attn, self.w_o, self.b_o, defer=True)


class ShortConvAttention(ProjectionNormAttention):
    """``ProjectionNormAttention`` whose q, k and v pass a short causal convolution over time, per
    channel and without a bias or an activation, right after the projection:
    y_t = sum_j taps[:, j] u_(t - n + 1 + j), zeros before the sequence's start.  The last n - 1
    projected rows of a sequence are state, so the mixer keeps pages and a state slot
    (``cache_specs``; ``forward`` takes both bindings)."""

    NAMES = dict(ProjectionNormAttention.NAMES, q_conv="q.conv", k_conv="k.conv", v_conv="v.conv")

    def __init__(self, *args, conv=4, **kwargs):
        super().__init__(*args, **kwargs)
        self.conv = int(conv)
        if self.conv < 1:
            raise ValueError("the convolution has at least one tap")

    def param_specs(self):
        specs = super().param_specs()
        n = self.names
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        specs[n["q_conv"]] = ParamSpec((H * D, self.conv))
        specs[n["k_conv"]] = ParamSpec((G * D, self.conv))
        if not self.values_are_keys:
            specs[n["v_conv"]] = ParamSpec((G * Dv, self.conv))
        return specs

    def cache_specs(self):
        specs = [self.cache_spec()]
        if self.conv > 1:
            specs.append(StateSpec(((self.conv - 1) * self.in_channels,), "float32"))
        return specs

    def load(self, tensors, rt):
        super().load(tensors, rt)
        n = self.names
        taps = [self._by_head(tensors(n["q_conv"]), self.num_heads), self._by_head(tensors(n["k_conv"]), self.num_kv_heads)]
        if not self.values_are_keys:
            taps.append(tensors(n["v_conv"]))
        self.taps = rt.vector(torch.cat(taps, 0))
        self.no_state = torch.zeros((1, 1), dtype=torch.float32, device=rt.device)

    def forward(self, x, batch, caches, shared):
        ops = self.rt.ops
        caches = caches if isinstance(caches, (list, tuple)) else [caches]
        pages = caches[0]
        buf = ops.linear(x, self.w_in, self.b_in, out_f32=True)
        if self.conv > 1:
            state = caches[1]
            conv = (self.taps, state.state, 0, batch, state.write)
        else:                  # one tap: a factor per channel, nothing carried
            conv = (self.taps, self.no_state, 0, batch, False)
        return self._attend(buf, batch, pages, shared, conv=conv)
