"""Small Vunadra configurations and weights for the tests.  The configurations differ from each
other in every size, in the order of their layers and in which options they use; the weights are
drawn so that every mechanism matters (corrections of the size of the shares, biases of the size
of their sums, products that reach their clamps, scores that reach their cap)."""
import json
import os

import torch

from servelab_amd.weights.safetensors_io import write_safetensors


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit, scale):
    return {"kind": "moe", "router": {"experts": experts, "identity": identity, "top": top, "scale": scale},
            "expert": {"ff": ff, "limit": limit}}


def rot(base, dims, **scaling):
    out = {"base": base, "dims": dims}
    if scaling:
        out["scaling"] = scaling
    return out


def blended(factor, original, fast, slow):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def by_wavelength(factor, original, low, high):
    return {"factor": factor, "original": original, "low": low, "high": high}


def conv_attention(heads, kv_heads, dim, vdim, scale, conv, rotation, mlp, window=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "conv": conv,
         "rot": rotation}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": mlp}


def key_value_attention(heads, kv_heads, dim, scale, rotation, mlp, window=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": rotation}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base, mlp, window=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def config(width, vocab, eps, layers, loop=None, embedding_scale=1.0, logit_scale=1.0):
    out = {"architecture": "Vunadra", "width": width, "vocab": vocab, "norm": {"eps": eps},
           "embedding": {"scale": embedding_scale}, "logit_scale": logit_scale, "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


def _a():
    # the last two layers run twice; groups of two heads; blended frequencies whose ramp lies inside the
    # pairs; windows shorter than the prompts; one expert that hands its input through
    layers = [
        conv_attention(4, 2, 16, 24, 0.3, 3, rot(10000.0, 16, **blended(4.0, 64, 8.0, 1.0)), dense(48)),
        key_value_attention(4, 2, 16, 0.25, rot(5000.0, 16, **by_wavelength(4.0, 64, 1.0, 4.0)),
                            moe(5, 1, 2, 24, 0.7, 2.0), window=9, softcap=5.0),
        latent(3, 16, 8, 24, 24, 0.2, 5000.0, moe(5, 1, 2, 24, 0.7, 2.0), window=13),
    ]
    return config(64, 300, 1e-5, layers, (1, 3, 2), embedding_scale=2.5, logit_scale=0.5)


def _b():
    # a width that is no multiple of 32; constants that are 1; no loop; no masks (every earlier key); no cap;
    # plain frequencies; part of a head rotated; one choice per token, no expert that hands through; a layer
    # without a feed-forward; one kv head; a convolution of two taps; a last feed-forward whose output product
    # takes the fused few-rows kernel while the head's rows of 72 values do not
    layers = [
        key_value_attention(3, 1, 8, 0.5, rot(500.0, 8), None),
        conv_attention(3, 3, 8, 8, 0.4, 2, rot(100.0, 4), moe(3, 0, 1, 16, 1.0, 1.0)),
        latent(2, 24, 4, 8, 40, 0.15, 100.0, dense(64)),
    ]
    return config(72, 257, 1e-6, layers)


def _c():
    # sizes the matrix-core kernels take in bfloat16; the first layer alone runs three times; a window on the
    # attention with the convolution; eight heads on two kv heads; frequencies stretched by wavelength with
    # pairs in all three ranges
    layers = [
        conv_attention(4, 4, 32, 16, 0.2, 4, rot(50000.0, 32, **blended(8.0, 128, 16.0, 2.0)),
                       moe(8, 2, 3, 32, 1.5, 1.25), window=20),
        latent(4, 32, 32, 32, 32, 0.125, 1000000.0, dense(128), window=33),
        key_value_attention(8, 2, 64, 0.125, rot(10000.0, 64, **by_wavelength(8.0, 256, 1.0, 4.0)),
                            moe(8, 2, 3, 32, 1.5, 1.25), window=17, softcap=10.0),
    ]
    return config(96, 128, 1e-5, layers, (0, 1, 3), embedding_scale=4.0, logit_scale=1.5)


def _d():
    # a convolution of one tap (nothing kept); head counts that are no powers of two; channel counts that are
    # no multiples of four; two rotated channels; more router outputs than a wavefront has lanes; a cap on the
    # attention with the convolution; a window of two; a loop over all layers
    layers = [
        conv_attention(5, 5, 12, 20, 0.4, 1, rot(100.0, 2), moe(70, 3, 9, 8, 0.5, 3.0), softcap=3.0),
        key_value_attention(6, 3, 10, 0.3, rot(7.0, 10, **by_wavelength(2.0, 16, 0.5, 2.0)), dense(20), window=2),
        latent(5, 12, 2, 20, 6, 0.3, 10.0, moe(2, 2, 2, 12, 2.0, 0.75), window=5),
    ]
    return config(40, 97, 1e-4, layers, (0, 3, 2), embedding_scale=0.5, logit_scale=3.0)


def _e():
    # every router output chosen, most of them experts that hand through; a loop of one pass; one head; a
    # convolution of five taps; no rotation on one layer
    layers = [
        conv_attention(2, 1, 16, 8, 0.25, 5, rot(30.0, 16, **blended(2.0, 32, 4.0, 1.0)), moe(1, 3, 4, 32, 1.0, 1.0)),
        key_value_attention(1, 1, 32, 0.2, None, moe(6, 1, 3, 16, 0.8, 1.5), softcap=2.0),
    ]
    return config(48, 200, 1e-5, layers, (0, 2, 1), embedding_scale=1.5, logit_scale=2.5)


def _f():
    # wider layers and prompts of several hundred tokens: keys of 64 and 96 channels, a latent of 64, twelve
    # experts; the two middle layers run twice
    layers = [
        latent(4, 32, 32, 48, 64, 0.14, 1000000.0, dense(384), window=50),
        conv_attention(6, 3, 64, 32, 0.125, 4, rot(10000.0, 64, **blended(8.0, 512, 32.0, 1.0)),
                       moe(12, 2, 3, 64, 1.0, 1.5)),
        key_value_attention(4, 1, 96, 0.1, rot(250000.0, 96, **by_wavelength(8.0, 512, 1.0, 4.0)),
                            moe(12, 2, 3, 64, 1.0, 1.5), window=70, softcap=20.0),
        conv_attention(2, 2, 64, 64, 0.125, 3, rot(10000.0, 32), dense(256), window=90),
    ]
    return config(256, 512, 1e-5, layers, (1, 3, 2), embedding_scale=2.0, logit_scale=1.25)


MODELS = {"A": _a(), "B": _b(), "C": _c(), "D": _d(), "E": _e(), "F": _f()}


def tensor_shapes(cfg):
    """{name: shape} of every tensor a checkpoint of ``cfg`` holds (written from the design)."""
    w, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    if cfg.get("loop"):
        out["loop.in"] = (w, 2 * w)
        out["loop.step"] = (cfg["loop"]["times"], w)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        x = p + "mix."
        if layer["type"] == "attention":
            H, G, D, Dv, n = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            out.update({x + "q": (H * D, w), x + "k": (G * D, w), x + "v": (G * Dv, w), x + "o": (w, H * Dv),
                        x + "q.conv": (H * D, n), x + "k.conv": (G * D, n), x + "v.conv": (G * Dv, n)})
        elif layer["type"] == "attention_2":
            H, G, D = m["heads"], m["kv_heads"], m["dim"]
            out.update({x + "q": (H * D, w), x + "q.b": (H * D,), x + "k": (G * D, w), x + "k.b": (G * D,),
                        x + "q.norm": (H * D,), x + "k.norm": (G * D,), x + "o": (w, H * D), x + "o.b": (w,)})
        else:
            H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out.update({x + "q": (H * (D + R), w), x + "dkv": (C + R, w), x + "dkv.norm": (C,),
                        x + "uk": (H * D, C), x + "uv": (H * Dv, C), x + "o": (w, H * Dv)})
        c = layer["mlp"]
        if c is not None:
            out[p + "norm2"] = (w,)
            y = p + "mlp."
            if c["kind"] == "dense":
                out.update({y + "gate": (c["ff"], w), y + "gate.b": (c["ff"],), y + "up": (c["ff"], w),
                            y + "up.b": (c["ff"],), y + "down": (w, c["ff"]), y + "down.b": (w,)})
            else:
                ff, r = c["expert"]["ff"], c["router"]
                for e in range(r["experts"]):
                    out.update({f"{y}e{e}.gate": (ff, w), f"{y}e{e}.up": (ff, w), f"{y}e{e}.down": (w, ff)})
                out[y + "router"] = (r["experts"] + r["identity"], w)
                out[y + "correction"] = (r["experts"] + r["identity"],)
    return out


def make_weights(cfg, seed):
    """Values that are exact in bfloat16, as float32 tensors."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1", "norm2"):
            t = 1.0 + 0.25 * torch.randn(shape, generator=g)           # plain gains
        elif last == "b":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif last == "correction":
            t = torch.randn(shape, generator=g) / shape[0]             # of the size of a share
        elif last == "step":
            t = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif last == "router":
            t = 2.0 * torch.randn(shape, generator=g) * shape[1] ** -0.5
        elif last == "in":
            t = torch.randn(shape, generator=g) * shape[-1] ** -0.5
        else:
            t = 1.5 * torch.randn(shape, generator=g) * shape[-1] ** -0.5
        out[name] = t.to(torch.bfloat16).float()
    return out


def write_folder(tmp_path, cfg, seed, tag, weights=None):
    """(folder, weights): config.json and model.safetensors in bfloat16."""
    folder = os.path.join(str(tmp_path), f"vunadra_{tag}")
    os.makedirs(folder, exist_ok=True)
    weights = weights if weights is not None else make_weights(cfg, seed)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: t.to(torch.bfloat16) for n, t in weights.items()})
    return folder, weights
