"""A slow, whole-sequence implementation of the Vunadra design in float64, one function per
mechanism, written from the design's equations.  It shares no code with servelab_amd: the tests
hold the engine to it.

config: the dict of config.json.  weights: {tensor name: torch tensor}.  Everything runs on the
CPU over one whole sequence.

The design in short.  The embedding is multiplied by a constant.  A layer is x += Mixer(N1(x)),
then x += FF(N2(x)), N an RMS norm with a plain gain.  Mixers: grouped-query attention whose q, k
and v pass a short causal convolution over time, with neighbouring channels turning by angles
whose frequencies are blended between plain and stretched ones (and cos and sin enlarged);
grouped-query attention whose values are the keys as projected, with biases, a norm over the whole
projection, frequencies stretched by wavelength, capped scores and a window; attention over a
cached latent with one rotated key part shared by the heads, over a window.  Feed-forwards: a dense
one with biases and the tanh form of gelu as gate, or routed experts chosen by softmax shares
plus a correction, some of which hand their input through, with clamped products.  A run of
layers may be repeated with the same weights; each pass starts from a product of the stream and
the embedding output side by side, plus a vector of the pass.  The final norm is followed by the
embedding table as the head, times a constant."""
import math

import torch

F = torch.float64


def rms_norm(x, gain, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if gain is None else y * gain


def linear(x, w, b=None):
    y = x @ w.T
    return y if b is None else y + b


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# --------------------------------------------------------------------------- rotation
def plain_frequencies(dims, base):
    return [base ** (-2.0 * i / dims) for i in range(dims // 2)]


def blended_frequencies(dims, base, factor, original, fast, slow):
    """Between a fast and a slow number of turns within the original length the frequency goes
    over from itself to itself / factor."""
    def turn_index(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(turn_index(fast)), 0)
    hi = min(math.ceil(turn_index(slow)), dims - 1)
    out = []
    for i, f in enumerate(plain_frequencies(dims, base)):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return out


def blended_magnitude(factor):
    return 0.1 * math.log(factor) + 1.0


def wavelength_frequencies(dims, base, factor, low, high, original):
    """Short waves stay, long waves are stretched by factor, those between are interpolated."""
    out = []
    for f in plain_frequencies(dims, base):
        wave = 2.0 * math.pi / f
        if wave < original / high:
            out.append(f)
        elif wave > original / low:
            out.append(f / factor)
        else:
            s = (original / wave - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


def rotation_of(rot):
    """(dims, frequencies, magnitude) of a mixer's ``rot`` section; dims 0 when there is none."""
    if not rot or not rot.get("dims"):
        return 0, [], 1.0
    dims, base, sc = rot["dims"], rot["base"], rot.get("scaling")
    if not sc:
        return dims, plain_frequencies(dims, base), 1.0
    if "fast" in sc:
        return dims, blended_frequencies(dims, base, sc["factor"], sc["original"], sc["fast"], sc["slow"]), \
            blended_magnitude(sc["factor"])
    return dims, wavelength_frequencies(dims, base, sc["factor"], sc["low"], sc["high"], sc["original"]), 1.0


def rotate_neighbours(x, pos, dims, freqs, magnitude=1.0):
    """x [T, heads, D]: channel 2i turns with channel 2i + 1, i < dims / 2; the rest pass."""
    if not dims:
        return x
    ang = pos.to(F)[:, None] * torch.tensor(freqs, dtype=F)[None, :]
    c, s = (torch.cos(ang) * magnitude)[:, None, :], (torch.sin(ang) * magnitude)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# --------------------------------------------------------------------------- softmax over what is seen
def visible(T, window):
    """[T, T] bool: query i sees key j when 0 <= i - j (< window, if there is one)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if window:
        seen &= (i - j) < window
    return seen


def masked_softmax(scores, window):
    """scores [H, T, T]."""
    T = scores.shape[-1]
    return torch.softmax(scores.masked_fill(~visible(T, window), -math.inf), -1)


def short_convolution(u, taps):
    """u [T, C], taps [C, n]: y_t = sum_j taps[:, j] u_(t - n + 1 + j), zeros before the start."""
    T, C = u.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(n):
        y = y + taps[:, j][None, :] * padded[j:j + T]
    return y


def grouped_attention(q, k, v, scale, window, softcap=None):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H * Dv]; query head h reads kv head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    kh = k.repeat_interleave(rep, 1)
    vh = v.repeat_interleave(rep, 1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * scale
    if softcap:
        scores = softcap * torch.tanh(scores / softcap)
    p = masked_softmax(scores, window)
    return torch.einsum("hij,jhd->ihd", p, vh).reshape(T, -1)


def _window(m):
    mask = m.get("mask")
    return int(mask["size"]) if mask and mask.get("size") else None


# --------------------------------------------------------------------------- mixers
def conv_attention(h, m, w, p, eps):
    """Attention whose projections pass a short convolution before the rotation."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = linear(h, w[p + "q"]), linear(h, w[p + "k"]), linear(h, w[p + "v"])
    if m.get("conv"):
        q = short_convolution(q, w[p + "q.conv"])
        k = short_convolution(k, w[p + "k.conv"])
        v = short_convolution(v, w[p + "v.conv"])
    pos = torch.arange(T)
    dims, freqs, mag = rotation_of(m.get("rot"))
    q = rotate_neighbours(q.reshape(T, H, D), pos, dims, freqs, mag)
    k = rotate_neighbours(k.reshape(T, G, D), pos, dims, freqs, mag)
    o = grouped_attention(q, k, v.reshape(T, G, Dv), m["scale"], _window(m), m.get("softcap"))
    return linear(o, w[p + "o"])


def keys_as_values_attention(h, m, w, p, eps):
    """Attention without a value projection: the values are the keys as the projection left them."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = linear(h, w[p + "q"], w[p + "q.b"])
    k = linear(h, w[p + "k"], w[p + "k.b"])
    v = k.reshape(T, G, D)
    q = rms_norm(q, w[p + "q.norm"], eps)          # over all heads at once
    k = rms_norm(k, w[p + "k.norm"], eps)
    pos = torch.arange(T)
    dims, freqs, mag = rotation_of(m.get("rot"))
    q = rotate_neighbours(q.reshape(T, H, D), pos, dims, freqs, mag)
    k = rotate_neighbours(k.reshape(T, G, D), pos, dims, freqs, mag)
    o = grouped_attention(q, k, v, m["scale"], _window(m), m.get("softcap"))
    return linear(o, w[p + "o"], w[p + "o.b"])


def latent_attention(h, m, w, p, eps):
    """Keys and values of every head from a normed latent, one rotated key part for all heads."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = linear(h, w[p + "q"]).reshape(T, H, D + R)
    down = linear(h, w[p + "dkv"])
    c = rms_norm(down[:, :C], w[p + "dkv.norm"], eps)
    pos = torch.arange(T)
    dims, freqs, mag = rotation_of(m.get("rot"))
    k_rot = rotate_neighbours(down[:, None, C:], pos, dims, freqs, mag)            # [T, 1, R]
    q_rot = rotate_neighbours(q[..., D:], pos, dims, freqs, mag)
    k_plain = linear(c, w[p + "uk"]).reshape(T, H, D)
    v = linear(c, w[p + "uv"]).reshape(T, H, Dv)
    scores = (torch.einsum("ihd,jhd->hij", q[..., :D], k_plain)
              + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * m["scale"]
    pw = masked_softmax(scores, _window(m))
    o = torch.einsum("hij,jhd->ihd", pw, v).reshape(T, -1)
    return linear(o, w[p + "o"])


MIXERS = {"attention": conv_attention, "attention_2": keys_as_values_attention,
          "latent_attention": latent_attention}


# --------------------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p):
    gate = linear(h, w[p + "gate"], w[p + "gate.b"])
    up = linear(h, w[p + "up"], w[p + "up.b"])
    return linear(gelu_tanh(gate) * up, w[p + "down"], w[p + "down.b"])


def clamped_expert(h, w, p, limit):
    g = torch.clamp(linear(h, w[p + "gate"]), max=limit)
    u = torch.clamp(linear(h, w[p + "up"]), min=-limit, max=limit)
    return linear(g * torch.sigmoid(1.702 * g) * (u + 1.0), w[p + "down"])


def route(h, w, p, router):
    """Per token the chosen experts and their weights: ([T, top] long, [T, top])."""
    shares = torch.softmax(linear(h, w[p + "router"]), -1)
    choice = shares + w[p + "correction"]
    chosen = torch.topk(choice, router["top"], dim=-1).indices
    picked = torch.gather(shares, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20) * router["scale"]


def routed_ff(h, c, w, p):
    router = c["router"]
    real = router["experts"]
    chosen, weights = route(h, w, p, router)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, share in zip(chosen[t].tolist(), weights[t]):
            if e >= real:                           # an expert that hands its input through
                out[t] += share * h[t]
            else:
                out[t] += share * clamped_expert(h[t:t + 1], w, f"{p}e{e}.", c["expert"]["limit"])[0]
    return out


def feed_forward(h, c, w, p):
    return dense_ff(h, w, p) if c["kind"] == "dense" else routed_ff(h, c, w, p)


# --------------------------------------------------------------------------- the model
def layer(x, i, entry, w, eps):
    p = f"l{i}."
    x = x + MIXERS[entry["type"]](rms_norm(x, w[p + "norm1"], eps), entry["mixer"], w, p + "mix.", eps)
    if entry.get("mlp"):
        x = x + feed_forward(rms_norm(x, w[p + "norm2"], eps), entry["mlp"], w, p + "mlp.")
    return x


def pass_start(x, x0, w, t):
    return linear(torch.cat([x, x0], -1), w["loop.in"]) + w["loop.step"][t]


def forward(config, weights, tokens, trace=None):
    """tokens: list of ids of one sequence -> logits [T, vocab] (float64).  ``trace`` (a list)
    receives the stream after every layer run."""
    w = {n: t.to(F) if t.is_floating_point() else t for n, t in weights.items()}
    eps = config["norm"]["eps"]
    entries = config["layers"]
    x0 = w["embed"][torch.tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    x = x0

    def run(i):
        nonlocal x
        x = layer(x, i, entries[i], w, eps)
        if trace is not None:
            trace.append(x.clone())
    loop = config.get("loop")
    if not loop:
        for i in range(len(entries)):
            run(i)
    else:
        for i in range(loop["start"]):
            run(i)
        for t in range(loop["times"]):
            x = pass_start(x, x0, w, t)
            for i in range(loop["start"], loop["stop"]):
                run(i)
        for i in range(loop["stop"], len(entries)):
            run(i)
    return linear(rms_norm(x, w["final.norm"], eps), w["embed"]) * config["logit_scale"]
