"""Small Futezen configurations and weights for the tests.  The configurations differ from each
other in every size, in the order of their layers and in which options they use; the weights are
drawn so that every mechanism matters (step sizes and decays well inside their ranges, biases of
the size of their sums, norm weights away from zero)."""
import json
import os

import torch

from servelab_amd.weights.safetensors_io import write_safetensors


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=0):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def attention(heads, kv_heads, dim, vdim, scale, base, dims, mlp):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      "rot": {"base": base, "dims": dims}}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, mlp):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
                      "kv_rank": kv_rank, "scale": scale, "rot": {"base": base, "dims": rot_dim}}}


def mamba2(heads, vdim, state, groups, conv, norm_groups, mlp):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                      "norm_groups": norm_groups}}


def config(width, vocab, eps, layers, loop=None):
    out = {"architecture": "Futezen", "width": width, "vocab": vocab, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


def _a():
    # the last two layers run twice; groups of two heads; the read-out normed in two parts; part of
    # a head rotated
    layers = [
        attention(4, 2, 16, 24, 0.3, 10000.0, 8, dense(48)),
        latent(3, 16, 8, 24, 40, 24, 0.2, 5000.0, moe(5, 2, 24, 40)),
        mamba2(4, 8, 16, 2, 4, 2, moe(5, 2, 24, 40)),
    ]
    return config(64, 300, 1e-5, layers, (1, 3, 2))


def _b():
    # a width that is no multiple of 32; one choice per token; no shared expert; a convolution of two
    # taps; every head its own group; a layer without a feed-forward; no loop; one kv head; the whole
    # head rotated
    layers = [
        mamba2(3, 24, 8, 3, 2, 1, moe(3, 1, 16)),
        attention(3, 1, 8, 8, 0.5, 500.0, 8, None),
        latent(2, 24, 4, 8, 16, 40, 0.15, 100.0, dense(40)),
    ]
    return config(72, 257, 1e-6, layers)


def _c():
    # sizes the matrix-core kernels take in bfloat16; a state wider than one lane group's reach; the
    # first layer alone runs three times; every head its own kv head
    layers = [
        latent(4, 32, 32, 32, 64, 32, 0.125, 1000000.0, dense(128)),
        attention(4, 4, 32, 16, 0.2, 50000.0, 16, moe(8, 3, 32, 16)),
        mamba2(2, 32, 72, 1, 3, 1, moe(8, 3, 32, 16)),
    ]
    return config(96, 128, 1e-5, layers, (0, 1, 3))


def _d():
    # a convolution of one tap (no inputs kept); head counts that are no powers of two; channel
    # counts that are no multiples of four; two rotated channels; more experts than a wavefront has
    # lanes; every expert chosen; a loop over all layers; two attentions whose pages differ in size
    layers = [
        attention(5, 5, 12, 20, 0.4, 100.0, 2, moe(70, 9, 8)),
        mamba2(5, 12, 20, 5, 1, 5, moe(2, 2, 12, 4)),
        latent(5, 12, 2, 20, 10, 6, 0.3, 10.0, moe(2, 1, 12, 4)),
        attention(2, 1, 16, 8, 0.25, 7.0, 16, None),
        mamba2(6, 4, 4, 2, 5, 3, dense(20)),
    ]
    return config(40, 97, 1e-4, layers, (0, 5, 2))


def _e():
    # no attention at all: the engine holds states and not one page; a feed-forward of one expert
    # that every token takes; a loop that runs once
    layers = [
        mamba2(2, 16, 16, 1, 4, 1, moe(1, 1, 32)),
        mamba2(4, 8, 32, 4, 3, 4, moe(6, 3, 16, 16)),
    ]
    return config(48, 200, 1e-5, layers, (0, 2, 1))


def _f():
    # wider layers: keys of 96 channels over a latent of 80, six heads on three kv heads, eight state-space
    # heads in two groups, twelve experts; the two middle layers run twice
    layers = [
        latent(4, 32, 16, 48, 96, 80, 0.14, 1000000.0, dense(384)),
        mamba2(8, 16, 64, 2, 3, 2, moe(12, 3, 64, 96)),
        attention(6, 3, 64, 32, 0.125, 10000.0, 32, dense(384)),
        latent(4, 32, 16, 48, 96, 80, 0.14, 1000000.0, moe(12, 3, 64, 96)),
    ]
    return config(256, 512, 1e-5, layers, (1, 3, 2))


MODELS = {"A": _a(), "B": _b(), "C": _c(), "D": _d(), "E": _e(), "F": _f()}


def tensor_shapes(cfg):
    """{name: shape} of every tensor a checkpoint of ``cfg`` holds (written from the design)."""
    w, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (w,)
        x = p + "mix."
        if layer["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({x + "q": (H * D, w), x + "k": (G * D, w), x + "v": (G * Dv, w), x + "o": (w, H * Dv)})
        elif layer["type"] == "latent_attention":
            H, D, R, Dv, Q, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            out.update({x + "dq": (Q, w), x + "dq.norm": (Q,), x + "uq": (H * (D + R), Q), x + "dkv": (C + R, w),
                        x + "dkv.norm": (C,), x + "uk": (H * D, C), x + "uv": (H * Dv, C), x + "o": (w, H * Dv)})
        else:
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = H * P + 2 * G * N
            out.update({x + "in": (2 * H * P + 2 * G * N + H, w), x + "conv": (ch, m["conv"]), x + "conv.b": (ch,),
                        x + "dt_bias": (H,), x + "A_log": (H,), x + "D": (H,), x + "norm": (H * P,),
                        x + "o": (w, H * P)})
        c = layer["mlp"]
        if c is not None:
            out[p + "norm2"] = out[p + "norm2b"] = (w,)
            y = p + "mlp."
            if c["kind"] == "dense":
                out.update({y + "gate": (c["ff"], w), y + "up": (c["ff"], w), y + "down": (w, c["ff"])})
            else:
                for e in range(c["router"]["experts"]):
                    out.update({f"{y}e{e}.up": (c["expert"]["ff"], w), f"{y}e{e}.down": (w, c["expert"]["ff"])})
                out[y + "router"] = (c["router"]["experts"], w)
                out[y + "router.b"] = (c["router"]["experts"],)
                if c.get("shared"):
                    ff = c["shared"]["ff"]
                    out.update({y + "shared.up": (ff, w), y + "shared.down": (w, ff), y + "shared.sg": (1, w)})
    return out


def make_weights(cfg, seed):
    """Values that are exact in bfloat16, as float32 tensors."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith("dq.norm") or name.endswith("dkv.norm") or name.endswith("mix.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)            # plain gains
        elif last in ("norm", "norm1", "norm1b", "norm2", "norm2b"):
            t = 0.3 * torch.randn(shape, generator=g)                  # weights around zero: gain 1 + w
        elif last in ("b", "dt_bias", "D"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "A_log":
            t = -1.0 + 0.5 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif last in ("router", "sg"):
            t = 2.0 * torch.randn(shape, generator=g) * shape[1] ** -0.5
        else:
            t = 1.5 * torch.randn(shape, generator=g) * shape[-1] ** -0.5
        out[name] = t.to(torch.bfloat16).float()
    return out


def write_folder(tmp_path, cfg, seed, tag, weights=None):
    """(folder, weights): config.json and model.safetensors in bfloat16."""
    folder = os.path.join(str(tmp_path), f"futezen_{tag}")
    os.makedirs(folder, exist_ok=True)
    weights = weights if weights is not None else make_weights(cfg, seed)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: t.to(torch.bfloat16) for n, t in weights.items()})
    return folder, weights
