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
"""
import math

import torch

from .base import Mixer, PagedKVSpec, ParamSpec


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


class ProjectionNormAttention(Mixer):
    """Grouped-query softmax attention whose q and k are RMS-normed over the whole projection
    (all heads of a token at once, a gain of that size) before the rotation, with biases on q,
    k, v and the output, keys of ``key_dim`` and values of ``value_dim`` channels, a score
    scale given from outside and float32 softmax weights.  The position encoding turns the
    leading channels of a head in halves.  Causal; ``window`` None keeps every key.
    ``projection_norm`` False: q and k go to the rotation as the projection left them (no gains
    in the checkpoint); ``bias`` False: no biases."""
    graph_safe = True

    NAMES = {"q": "q", "k": "k", "v": "v", "out": "o", "q_bias": "q.b", "k_bias": "k.b",
             "v_bias": "v.b", "out_bias": "o.b", "q_norm": "q.norm", "k_norm": "k.norm"}

    def __init__(self, hidden_size, num_heads, num_kv_heads, key_dim, value_dim, scale, position,
                 norm_eps, bias=True, window=None, names=None, projection_norm=True):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.position = position
        self.bias = bool(bias)
        self.projection_norm = bool(projection_norm)
        self.window = None if not window else int(window)
        self.names = dict(self.NAMES, **(names or {}))

    def param_specs(self):
        n, h = self.names, self.hidden_size
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        specs = {n["q"]: ParamSpec((H * D, h)), n["k"]: ParamSpec((G * D, h)), n["v"]: ParamSpec((G * Dv, h)),
                 n["out"]: ParamSpec((h, H * Dv))}
        if self.projection_norm:
            specs.update({n["q_norm"]: ParamSpec((H * D,), init="gain"),
                          n["k_norm"]: ParamSpec((G * D,), init="gain")})
        if self.bias:
            specs.update({n["q_bias"]: ParamSpec((H * D,)), n["k_bias"]: ParamSpec((G * D,)),
                          n["v_bias"]: ParamSpec((G * Dv,)), n["out_bias"]: ParamSpec((h,))})
        return specs

    def cache_spec(self):
        return PagedKVSpec(self.num_kv_heads, self.key_dim, self.window, value_dim=self.value_dim)

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        self.position.load(tensors, rt)
        layout = self.position.layout()
        if layout is not None and (layout.pairing != "half" or layout.rot_dim > self.key_dim):
            raise ValueError("the rotation must turn leading channels of a head in halves")
        self.rot = 0 if layout is None else int(layout.rot_dim)
        w = torch.cat([tensors(n["q"]), tensors(n["k"]), tensors(n["v"])], 0)
        extra = -w.shape[0] % 8
        if extra:
            w = torch.cat([w, w.new_zeros(extra, w.shape[1])], 0)
        self.w_in = rt.linear_weight(w)
        self.b_in = self.b_o = None
        if self.bias:
            b = torch.cat([tensors(n["q_bias"]).float(), tensors(n["k_bias"]).float(),
                           tensors(n["v_bias"]).float(), torch.zeros(extra, device=w.device)], 0)
            self.b_in = rt.vector(b)
            self.b_o = rt.vector(tensors(n["out_bias"]))
        self.q_gain = rt.vector(tensors(n["q_norm"])) if self.projection_norm else None
        self.k_gain = rt.vector(tensors(n["k_norm"])) if self.projection_norm else None
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)

    def forward(self, x, batch, cache, shared):
        ops = self.rt.ops
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        group = batch.groups[cache.group]
        buf = ops.linear(x, self.w_in, self.b_in, out_f32=True)
        tables = self.position.tables(batch, shared) if self.rot else None
        q = ops.projnorm_rope_store(buf, H, G, D, Dv, self.q_gain, self.k_gain, self.norm_eps, self.rot,
                                    tables, group.slots if cache.write else None, cache.k, cache.v,
                                    cache.page_size)
        attn = ops.window_attention(q, 0, H, G, D, Dv, cache.k, cache.v, cache.page_size,
                                    group.block_tables, batch, self.scale, self.window)
        return ops.linear(attn, self.w_o, self.b_o)
