"""Vunadra: a pre-norm decoder whose config.json lists its layers.

    x = embed[token] * embedding.scale
    x += Mixer(Norm1(x));  x += FeedForward(Norm2(x))          (RMS norms with plain gains)
    logits = embed Norm(x) * logit_scale

Mixers: grouped-query attention whose q, k and v pass a short causal convolution, with channels
turning in neighbouring pairs at frequencies blended between plain and stretched ones
(``ShortConvAttention``); grouped-query attention whose values are the keys as projected, with
biases, a norm over the whole projection, frequencies stretched by wavelength, capped scores and
a window (``ProjectionNormAttention(values="keys")``); attention over a cached latent with one
rotated key part shared by the heads, over a window (``LatentWindowAttention``).  Feed-forward:
dense with biases and the tanh form of gelu as gate (``GatedMLP``), or experts routed by their
softmax shares plus a correction, some of which hand their input through, with clamped products
(``RoutedExperts(routing="shares")``), or absent.  ``loop`` walks a stretch of layers several
times: the run list calls those blocks again, each call with cache streams of its own, and
enters every pass through a ``StreamReentry`` block (stream and embedding output side by side
through one matrix, plus a vector of the pass).  Checkpoint names: ``embed``, ``loop.in``,
``loop.step``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``.
"""
from ..config import VunadraConfig, register_architecture
from ..config.vunadra import BiasedDenseConfig
from ..parts.attention import ProjectionNormAttention, ShortConvAttention
from ..parts.block import PreNormBlock, StreamReentry
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.feedforward import GatedMLP
from ..parts.model import LayerCall, ModelSpec
from ..parts.norm import RMSNorm
from ..parts.position import (NoPosition, RotaryPosition, blended_frequencies, blended_magnitude,
                              wavelength_frequencies)
from ..parts.routed import RoutedExperts
from ..parts.window_attention import LatentWindowAttention


def _position(rot, head_dim):
    """The encoding of a mixer's ``rot`` section over heads (or a shared part) of ``head_dim``."""
    if not rot.dims:
        return NoPosition()
    frequencies, magnitude = None, 1.0
    if rot.scaling is not None:
        kind, factor, original, a, b = rot.scaling
        if kind == "blended":
            frequencies = blended_frequencies(rot.dims, rot.base, factor, original, a, b)
            magnitude = blended_magnitude(factor)
        else:
            frequencies = wavelength_frequencies(rot.dims, rot.base, factor, a, b, original)
    else:
        # (the plain frequencies in double precision, rounded once)
        from ..parts.position import plain_frequencies
        frequencies = plain_frequencies(rot.dims, rot.base)
    return RotaryPosition(head_dim, rot.base, rotary_dim=rot.dims, pairing="interleaved",
                          frequencies=frequencies, magnitude=magnitude)


def _mixer(cfg: VunadraConfig, layer):
    m, w, eps = layer.mixer, cfg.width, cfg.norm_eps
    if layer.kind == "latent_attention":
        return LatentWindowAttention(w, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, m.window or None,
                                     _position(m.rot, m.rot_dim), norm_eps=eps, gate=False)
    common = dict(bias=m.values_are_keys, window=m.window or None, projection_norm=m.values_are_keys,
                  values="keys" if m.values_are_keys else "projected", softcap=m.softcap or None)
    args = (w, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, _position(m.rot, m.dim), eps)
    if m.conv:
        return ShortConvAttention(*args, conv=m.conv, **common)
    return ProjectionNormAttention(*args, **common)


def _feedforward(cfg: VunadraConfig, c):
    if c is None:
        return None
    if isinstance(c, BiasedDenseConfig):
        return GatedMLP(cfg.width, c.ff, "gelu_tanh", names=("gate", "up", "down"),
                        bias_names=("gate.b", "up.b", "down.b"))
    return RoutedExperts(cfg.width, c.experts, c.top, c.ff, activation="clamped_swish", gated=True,
                         routing="shares", correction=True, route_scale=c.scale, pass_through=c.identity,
                         limit=c.limit)


def build_vunadra(cfg: VunadraConfig) -> ModelSpec:
    embedding = TokenEmbedding(cfg.vocab, cfg.width, name="embed", scale=cfg.embedding_scale)

    def norm(name):
        return RMSNorm(cfg.width, cfg.norm_eps, name=name)
    layers = []
    for i, layer in enumerate(cfg.layers):
        block = PreNormBlock(norm("norm1"), _mixer(cfg, layer), norm("norm2"), _feedforward(cfg, layer.mlp),
                             names=("", "mix.", "", "mlp."))
        layers.append((f"l{i}.", block))
    before, stretch, passes, behind = cfg.stretches()
    run, streams = [], 0

    def call(i):                                # a repeated layer is a further call with streams of its own
        nonlocal streams
        n = len(layers[i][1].cache_specs())
        run.append(LayerCall(i, tuple(range(streams, streams + n))))
        streams += n
    for i in before:
        call(i)
    if passes:
        layers.append(("loop.", StreamReentry(cfg.width, passes)))
        entry = len(layers) - 1
        for _ in range(passes):
            run.append(LayerCall(entry))
            for i in stretch:
                call(i)
    for i in behind:
        call(i)
    return ModelSpec(
        embedding=("", embedding),
        layers=layers,
        run=run,
        final_norm=("final.", norm("norm")),
        head=("", OutputHead(cfg.vocab, cfg.width, tied_to=embedding, scale=cfg.logit_scale)),
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        eos_token_id=-1,
        keeps_embedding=passes > 0,
    )


register_architecture("Vunadra", VunadraConfig.from_hf, build_vunadra, model_type="vunadra")
