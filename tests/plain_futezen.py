"""A slow, whole-sequence implementation of the Futezen design in float64, one function per
mechanism, written from the design's equations.  It shares no code with servelab_amd: the tests
hold the engine to it.

config: the dict of config.json.  weights: {tensor name: torch tensor}.  Everything runs on the
CPU, token by token where the design is a recurrence.

The design in short.  A layer is x += N1b(Mixer(N1(x))), then x += N2b(FF(N2(x))), every N an RMS
norm whose stored weight w acts as the gain 1 + w.  Mixers: softmax attention over grouped heads
with a rotation of leading channels in halves; attention whose keys and values are made from a
cached latent and whose queries pass a normed latent of their own, with one rotated key part
shared by the heads (pairs of neighbouring channels); a state-space mixer with a scalar decay per
head.  Feed-forwards: a relu-gated dense one, or routed experts (squared relu, no gate) with a
shared expert behind a sigmoid of one number per token.  A run of layers may be repeated with
the same weights.  The final norm is followed by the embedding table as the head."""
import math

import torch

F = torch.float64


def rms_norm(x, gain, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if gain is None else y * gain


def offset_norm(x, w, eps):
    """The design's layer norms: the stored weight sits around zero."""
    return rms_norm(x, 1.0 + w, eps)


def linear(x, w, b=None):
    y = x @ w.T
    return y if b is None else y + b


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def angles(pos, dims, base):
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    return pos.to(F)[:, None] * freq[None, :]


def rotate_halves(x, pos, dims, base):
    """x [T, heads, D]: channel i turns with channel i + dims / 2, i < dims / 2; the rest pass."""
    half = dims // 2
    ang = angles(pos, dims, base)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def rotate_neighbours(x, pos, dims, base):
    """x [T, heads, D]: channel 2i turns with channel 2i + 1, i < dims / 2; the rest pass."""
    ang = angles(pos, dims, base)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def causal_softmax(scores):
    """scores [H, T, T] -> weights with every key after the query shut out."""
    T = scores.shape[-1]
    seen = torch.ones(T, T, dtype=torch.bool).tril()
    return torch.softmax(scores.masked_fill(~seen, -math.inf), -1)


# --------------------------------------------------------------------------- mixers
def attention(h, m, w, p, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate_halves(linear(h, w[p + "q"]).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_halves(linear(h, w[p + "k"]).view(T, G, D), pos, m["rot"]["dims"], m["rot"]["base"])
    v = linear(h, w[p + "v"]).view(T, G, Dv)
    k = k.repeat_interleave(H // G, 1)
    v = v.repeat_interleave(H // G, 1)
    weights = causal_softmax(torch.einsum("qhd,khd->hqk", q, k) * m["scale"])
    out = torch.einsum("hqk,khd->qhd", weights, v).reshape(T, H * Dv)
    return linear(out, w[p + "o"])


def latent_attention(h, m, w, p, eps):
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    dims, base = m["rot"]["dims"], m["rot"]["base"]
    cq = rms_norm(linear(h, w[p + "dq"]), w[p + "dq.norm"], eps)
    q = linear(cq, w[p + "uq"]).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_neighbours(q[..., D:], pos, dims, base)
    down = linear(h, w[p + "dkv"])
    c = rms_norm(down[:, :C], w[p + "dkv.norm"], eps)
    k_rot = rotate_neighbours(down[:, None, C:], pos, dims, base)[:, 0]            # [T, R], one for all heads
    k_plain = linear(c, w[p + "uk"]).view(T, H, D)
    v = linear(c, w[p + "uv"]).view(T, H, Dv)
    scores = (torch.einsum("qhd,khd->hqk", q_plain, k_plain)
              + torch.einsum("qhr,kr->hqk", q_rot, k_rot)) * m["scale"]
    out = torch.einsum("hqk,khd->qhd", causal_softmax(scores), v).reshape(T, H * Dv)
    return linear(out, w[p + "o"])


def causal_conv(x, taps, bias):
    """x [T, C]; taps [C, n], the last column is the token's own; zeros before the start."""
    T, n = x.shape[0], taps.shape[1]
    full = torch.cat([torch.zeros(n - 1, x.shape[1], dtype=F), x], 0)
    return sum(full[j:j + T] * taps[:, j] for j in range(n)) + bias


def mamba2(h, m, w, p, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = linear(h, w[p + "in"])
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, 1)
    Cm = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, 1)
    dt = softplus(dt + w[p + "dt_bias"])                                        # [T, H]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * dt)
    S = torch.zeros(H, N, P, dtype=F)
    y = torch.zeros(T, H, P, dtype=F)
    for t in range(T):
        S = decay[t][:, None, None] * S + dt[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, Cm[t]) + w[p + "D"][:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    groups = m["norm_groups"]
    y = rms_norm(y.view(T, groups, inner // groups), None, eps).reshape(T, inner) * w[p + "norm"]
    return linear(y, w[p + "o"])


MIXERS = {"attention": attention, "latent_attention": latent_attention, "mamba2": mamba2}


# --------------------------------------------------------------------------- feed-forwards
def dense(h, w, p):
    return linear(torch.relu(linear(h, w[p + "gate"])) * linear(h, w[p + "up"]), w[p + "down"])


def expert(h, w, p):
    return linear(torch.relu(linear(h, w[p + "up"])) ** 2, w[p + "down"])


def experts(h, c, w, p):
    n, top = c["router"]["experts"], c["router"]["top"]
    logits = linear(h, w[p + "router"], w[p + "router.b"])
    best = torch.topk(logits, top, dim=-1)
    shares = torch.softmax(best.values, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(best.indices[t].tolist(), shares[t]):
            out[t] += s * expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if c.get("shared"):
        out = out + torch.sigmoid(linear(h, w[p + "shared.sg"])) * expert(h, w, p + "shared.")
    return out


# --------------------------------------------------------------------------- the model
def layer_order(config):
    """Indices of the layers in the order they run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(config, weights, tokens, streams=None):
    """Logits [T, vocab] (float64) of one sequence.  ``streams``: a list that receives the
    residual stream after every layer run."""
    w = {k: v.to(F) for k, v in weights.items() if v.is_floating_point()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i in layer_order(config):
        layer, p = config["layers"][i], f"l{i}."
        y = MIXERS[layer["type"]](offset_norm(x, w[p + "norm1"], eps), layer["mixer"], w, p + "mix.", eps)
        x = x + offset_norm(y, w[p + "norm1b"], eps)
        c = layer.get("mlp")
        if c:
            hn = offset_norm(x, w[p + "norm2"], eps)
            y = dense(hn, w, p + "mlp.") if c["kind"] == "dense" else experts(hn, c, w, p + "mlp.")
            x = x + offset_norm(y, w[p + "norm2b"], eps)
        if streams is not None:
            streams.append(x.clone())
    return linear(offset_norm(x, w["final.norm"], eps), w["embed"])
