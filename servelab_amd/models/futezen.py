"""Futezen: a decoder whose config.json lists its layers, each a block with a norm before and
after each sublayer.

    h += Norm1b(Mixer(Norm1(h)));  h += Norm2b(FeedForward(Norm2(h)))

Every norm is an RMS norm whose stored weight w acts as the gain 1 + w.  The mixer is a softmax
attention over grouped heads whose leading channels turn in halves (``parts/attention.py``), an
attention over a cached latent whose queries pass a normed latent of their own and whose shared
rotated key part turns in neighbouring pairs (``parts/window_attention.py``, here without a
window), or a state-space mixer with one decay per head (``parts/recurrent.py``).  The
feed-forward is relu-gated and dense, or routed experts without a gate whose activation is the
square of relu, with a router bias and a shared expert behind a sigmoid of one number per token
(``parts/routed.py``), or absent.  ``loop`` repeats a stretch of layers: the run list calls those
blocks again, each call with cache streams of its own.  The final norm is followed by the
embedding table as the head.  Checkpoint names: ``embed``, ``l<i>.norm1``, ``l<i>.norm1b``,
``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``.
"""
from ..config import FutezenConfig, register_architecture
from ..config.futezen import DenseFfConfig
from ..parts.attention import ProjectionNormAttention
from ..parts.block import SandwichBlock
from ..parts.embedding import OutputHead, TokenEmbedding
from ..parts.feedforward import GatedMLP
from ..parts.model import LayerCall, ModelSpec
from ..parts.norm import RMSNorm
from ..parts.position import NoPosition, RotaryPosition
from ..parts.recurrent import StateSpaceMixer
from ..parts.routed import RoutedExperts
from ..parts.window_attention import LatentWindowAttention


def _mixer(cfg: FutezenConfig, layer):
    m, w, eps = layer.mixer, cfg.width, cfg.norm_eps
    if layer.kind == "attention":
        position = RotaryPosition(m.dim, m.rot_base, rotary_dim=m.rot_dims) if m.rot_dims else NoPosition()
        return ProjectionNormAttention(w, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, position, eps,
                                       bias=False, projection_norm=False)
    if layer.kind == "latent_attention":
        position = RotaryPosition(m.rot_dim, m.rot_base, rotary_dim=m.rot_dims, pairing="interleaved") \
            if m.rot_dims else NoPosition()
        return LatentWindowAttention(w, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.scale, None, position,
                                     norm_eps=eps, gate=False, q_rank=m.q_rank)
    return StateSpaceMixer(w, m.heads, m.vdim, m.state, m.groups, m.conv, m.norm_groups, eps)


def _feedforward(cfg: FutezenConfig, c):
    if c is None:
        return None
    if isinstance(c, DenseFfConfig):
        return GatedMLP(cfg.width, c.ff, "relu", names=("gate", "up", "down"))
    return RoutedExperts(cfg.width, c.experts, c.top, c.ff, c.shared_ff, activation="relu2", gated=False,
                         router_bias=True, shared_gate=True)


def build_futezen(cfg: FutezenConfig) -> ModelSpec:
    embedding = TokenEmbedding(cfg.vocab, cfg.width, name="embed")

    def norm(name):
        return RMSNorm(cfg.width, cfg.norm_eps, name=name, offset=1.0)
    layers = []
    for i, layer in enumerate(cfg.layers):
        block = SandwichBlock(norm("norm1"), _mixer(cfg, layer), norm("norm1b"), norm("norm2"),
                              _feedforward(cfg, layer.mlp), norm("norm2b"),
                              names=("", "mix.", "", "", "mlp.", ""))
        layers.append((f"l{i}.", block))
    run, streams = [], 0
    for i in cfg.order():                       # a repeated layer is a further call with streams of its own
        n = len(layers[i][1].cache_specs())
        run.append(LayerCall(i, tuple(range(streams, streams + n))))
        streams += n
    return ModelSpec(
        embedding=("", embedding),
        layers=layers,
        run=run,
        final_norm=("final.", norm("norm")),
        head=("", OutputHead(cfg.vocab, cfg.width, tied_to=embedding)),
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        eos_token_id=-1,
    )


register_architecture("Futezen", FutezenConfig.from_hf, build_futezen, model_type="futezen")
