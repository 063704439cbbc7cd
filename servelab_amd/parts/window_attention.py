"""Two attention mixers over a paged cache whose softmax sees a window.

``GatedWindowAttention``: grouped-query attention without rotation.  Per head,
q and k are divided by their root mean square and multiplied by a gain shared
by the heads; score = (q . k) * scale - slope_h * (i - j) with slope_h =
2^(-8 (h + 1) / heads) (``distance_bias``); the query at position i sees key
j <= i when i - j < window or j < keep_first; the softmax's denominator also
holds exp(sink_h) (``sink``); values may be mixed with those an earlier layer
made for the same token, v <- (1 - lambda) v + lambda v_first, before they are
cached (``value_mix``: "give" keeps this layer's own values for later layers
of the same ``mix_group``, "take" mixes them in); a head's output is multiplied
by sigmoid(Wg x)_h (``gate``) before the output projection.  Keys have
``key_dim`` channels and values ``value_dim``.

``LatentWindowAttention``: keys and values of every head are made from a latent
c = RMSNorm(Wdkv x)[:rank] of few channels, k_h = Wuk_h c and v_h = Wuv_h c,
plus one rotated key part shared by the heads; score = (q_h . k_h + q_h' . k')
* scale over a window.  Only c and the rotated part are cached, as one key row
[c | k'] of one kv head, and the attention runs in the latent's space: the
query becomes [Wuk_h^T q_h | q_h'], the weighted sum of the cached c comes back
through Wuv_h (both are products with one small matrix per head), so neither
keys nor values of the heads are ever formed for cached tokens.  With ``q_rank`` the queries
pass a latent of their own: q = Wuq RMSNorm(Wdq x), the norm with a gain of ``q_rank`` channels.
The rotation may pair halves or neighbouring channels: the rows that make the rotated channels
are put into the order of halves at load (a score does not depend on the order of its terms).

Every constant is a constructor parameter; checkpoint names are a parameter
too (``names``).
"""
import torch

from .base import Mixer, PagedKVSpec, ParamSpec

def _padded_rows(rows):
    """[rows...] concatenated, with zero rows added up to a multiple of 8: the product's output
    rows then start 16-byte aligned in both activation types."""
    w = torch.cat(rows, 0)
    extra = -w.shape[0] % 8
    return torch.cat([w, w.new_zeros(extra, w.shape[1])], 0) if extra else w


_WINDOW_NAMES = {"q": "q", "k": "k", "v": "v", "q_norm": "q.norm", "k_norm": "k.norm",
                 "mix": "vmix", "sink": "sink", "gate": "g", "out": "o"}


def distance_slopes(num_heads: int) -> torch.Tensor:
    """slope_h = 2^(-8 (h + 1) / heads), float32 [heads]."""
    h = torch.arange(1, num_heads + 1, dtype=torch.float64)
    return torch.pow(torch.tensor(2.0, dtype=torch.float64), -8.0 * h / num_heads).to(torch.float32)


class GatedWindowAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, key_dim, value_dim, scale, window,
                 keep_first=0, norm_eps=1e-6, qk_norm=True, distance_bias=True, sink=True,
                 value_mix=None, mix_group="values", gate=True, names=None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if value_mix not in (None, "give", "take"):
            raise ValueError("value_mix is None, 'give' or 'take'")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale = float(scale)
        self.window = None if not window else int(window)
        self.keep_first = int(keep_first) if self.window else 0
        self.norm_eps = float(norm_eps)
        self.qk_norm, self.distance_bias, self.sink, self.gate = bool(qk_norm), bool(distance_bias), bool(sink), bool(gate)
        self.value_mix, self.mix_group = value_mix, mix_group
        self.names = dict(_WINDOW_NAMES, **(names or {}))

    # ---- declarations
    def param_specs(self):
        n, h = self.names, self.hidden_size
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        specs = {n["q"]: ParamSpec((H * D, h)), n["k"]: ParamSpec((G * D, h)), n["v"]: ParamSpec((G * Dv, h))}
        if self.qk_norm:
            specs[n["q_norm"]] = ParamSpec((D,), init="gain")
            specs[n["k_norm"]] = ParamSpec((D,), init="gain")
        if self.value_mix is not None:
            specs[n["mix"]] = ParamSpec(())           # (the giving layer holds one too, unused)
        if self.sink:
            specs[n["sink"]] = ParamSpec((H,))
        if self.gate:
            specs[n["gate"]] = ParamSpec((H, h))
        specs[n["out"]] = ParamSpec((h, H * Dv))
        return specs

    def cache_spec(self):
        return PagedKVSpec(self.num_kv_heads, self.key_dim, self.window, value_dim=self.value_dim,
                           keep_first=self.keep_first)

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        rows = [tensors(n["q"]), tensors(n["k"]), tensors(n["v"])]
        if self.gate:
            rows.append(tensors(n["gate"]))
        self.w_in = rt.linear_weight(_padded_rows(rows))          # [q; k; v; gate] in one product
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)
        self.q_gain = rt.vector(tensors(n["q_norm"])) if self.qk_norm else None
        self.k_gain = rt.vector(tensors(n["k_norm"])) if self.qk_norm else None
        self.sinks = rt.vector(tensors(n["sink"])) if self.sink else None
        self.slopes = distance_slopes(self.num_heads).to(rt.device) if self.distance_bias else None
        self.mix = float(tensors(n["mix"]).float()) if self.value_mix is not None else 0.0

    # ---- compute
    def forward(self, x, batch, cache, shared):
        ops = self.rt.ops
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        group = batch.groups[cache.group]
        buf = ops.linear(x, self.w_in, None)
        v_col, g_col = (H + G) * D, (H + G) * D + G * Dv
        key = ("first values", self.mix_group)
        v_first = None
        if self.value_mix == "take":
            if key not in shared:
                raise RuntimeError("a layer mixes in the values of an earlier layer that has not run")
            v_first = shared[key]
        ops.headnorm_store(buf, H, G, D, Dv, self.q_gain, self.k_gain, self.norm_eps, v_first, self.mix,
                           group.slots if cache.write else None, cache.k, cache.v, cache.page_size)
        if self.value_mix == "give":
            shared[key] = buf[:, v_col:v_col + G * Dv]
        attn = ops.window_attention(buf, 0, H, G, D, Dv, cache.k, cache.v, cache.page_size,
                                    group.block_tables, batch, self.scale, self.window, self.keep_first,
                                    self.slopes, self.sinks, buf if self.gate else None, g_col)
        return ops.linear(attn, self.w_o, None, defer=True)


_LATENT_NAMES = {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_k": "uk", "up_v": "uv",
                 "gate": "g", "out": "o", "q_down": "dq", "q_down_norm": "dq.norm", "q_up": "uq"}


def _halves_order(rot: int, width: int, pairing: str) -> torch.Tensor:
    """The order that puts ``width`` channels whose first ``rot`` turn in ``pairing`` pairs into
    the order in which they turn in halves."""
    if pairing == "half":
        return torch.arange(width)
    return torch.cat([torch.arange(0, rot, 2), torch.arange(1, rot, 2), torch.arange(rot, width)])


class LatentWindowAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size, num_heads, head_dim, rot_dim, value_dim, rank, scale, window,
                 position, norm_eps=1e-6, gate=True, names=None, q_rank=None):
        """``position``: the encoding of the ``rot_dim`` rotated channels (a
        ``PositionEncoding`` whose layout rotates leading channels of them).
        ``q_rank``: the width of the queries' latent (None: q is one projection
        of the input)."""
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim, self.rot_dim = int(head_dim), int(rot_dim)
        self.value_dim, self.rank = int(value_dim), int(rank)
        self.scale = float(scale)
        self.window = None if not window else int(window)
        self.position = position
        self.norm_eps = float(norm_eps)
        self.gate = bool(gate)
        self.q_rank = None if not q_rank else int(q_rank)
        self.names = dict(_LATENT_NAMES, **(names or {}))

    def param_specs(self):
        n, h = self.names, self.hidden_size
        H, D, R, Dv, C = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank
        specs = {n["down"]: ParamSpec((C + R, h)),
                 n["down_norm"]: ParamSpec((C,), init="gain"),
                 n["up_k"]: ParamSpec((H * D, C)), n["up_v"]: ParamSpec((H * Dv, C))}
        if self.q_rank:
            specs.update({n["q_down"]: ParamSpec((self.q_rank, h)),
                          n["q_down_norm"]: ParamSpec((self.q_rank,), init="gain"),
                          n["q_up"]: ParamSpec((H * (D + R), self.q_rank))})
        else:
            specs[n["q"]] = ParamSpec((H * (D + R), h))
        if self.gate:
            specs[n["gate"]] = ParamSpec((H, h))
        specs[n["out"]] = ParamSpec((h, H * Dv))
        return specs

    def cache_spec(self):
        # one key row [latent | rotated part] per token; the values are its first `rank` channels
        return PagedKVSpec(1, self.rank + self.rot_dim, self.window, value_dim=0)

    def load(self, tensors, rt):
        self.rt = rt
        n = self.names
        H, D, Dv, C = self.num_heads, self.head_dim, self.value_dim, self.rank
        self.position.load(tensors, rt)
        layout = self.position.layout()
        if layout is None:
            self.rot = 0
        else:
            if layout.pairing not in ("half", "interleaved") or layout.rot_dim > self.rot_dim:
                raise ValueError("the rotated part takes an encoding that turns leading channels of it, in "
                                 "halves or in neighbouring pairs")
            self.rot = int(layout.rot_dim)
        R = self.rot_dim
        order = _halves_order(self.rot, R, "half" if layout is None else layout.pairing)
        w_q = tensors(n["q_up"] if self.q_rank else n["q"])
        by_head = w_q.reshape(H, D + R, w_q.shape[1])
        w_q = torch.cat([by_head[:, :D], by_head[:, D:][:, order.to(w_q.device)]], 1).reshape(w_q.shape)
        w_down = tensors(n["down"])
        w_down = torch.cat([w_down[:C], w_down[C:][order.to(w_down.device)]], 0)
        if self.q_rank:
            # [q's latent; down; gate] in one product, the queries in a second one from the normed latent
            rows = [tensors(n["q_down"]), w_down]
            self.w_q = rt.linear_weight(w_q)
            self.q_gain = rt.vector(tensors(n["q_down_norm"]))
        else:
            rows = [w_q, w_down]
        if self.gate:
            rows.append(tensors(n["gate"]))
        self.w_in = rt.linear_weight(_padded_rows(rows))          # [q; down; gate] in one product
        self.w_o = rt.linear_weight(tensors(n["out"]), delta=True)
        self.gain = rt.vector(tensors(n["down_norm"]))
        # per head: Wuk_h^T [C, D] takes q to the latent's space, Wuv_h [Dv, C] brings the output back
        self.to_latent = rt.matrix(tensors(n["up_k"]).reshape(H, D, C).transpose(1, 2))
        self.from_latent = rt.matrix(tensors(n["up_v"]).reshape(H, Dv, C))

    def forward(self, x, batch, cache, shared):
        ops = self.rt.ops
        H, D, R, Dv, C = self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank
        group = batch.groups[cache.group]
        buf = ops.linear(x, self.w_in, None)
        if self.q_rank:
            down_col = self.q_rank
            q_rows = ops.linear(ops.slice_rmsnorm(buf, 0, self.q_rank, self.q_gain, self.norm_eps), self.w_q, None)
        else:
            down_col = H * (D + R)
            q_rows = buf
        g_col = down_col + C + R
        T = buf.shape[0]
        q_lat = torch.empty((T, H * (C + R)), dtype=buf.dtype, device=buf.device)
        tables = self.position.tables(batch, shared) if self.rot else None
        ops.latent_store(buf, H, D, R, C, down_col, self.rot, self.gain, self.norm_eps, tables,
                         group.slots if cache.write else None, cache.k, cache.page_size, q_lat,
                         q_rows=q_rows if self.q_rank else None)
        ops.head_products(q_rows, 0, H, D + R, self.to_latent, y=q_lat, y_col=0, y_head=C + R)
        attn = ops.window_attention(q_lat, 0, H, 1, C + R, C, cache.k, None, cache.page_size,
                                    group.block_tables, batch, self.scale, self.window, 0, None, None,
                                    buf if self.gate else None, g_col)
        heads = ops.head_products(attn, 0, H, C, self.from_latent)
        return ops.linear(heads, self.w_o, None, defer=True)
