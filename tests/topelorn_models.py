"""Small Topelorn configurations and weights for the tests.  The configurations
differ from each other in every size and in the order of their layers; the
weights are drawn so that every mechanism matters (sinks of the size of a
score, mixing factors well inside (0, 1), gains away from 1)."""
import json
import os

import torch

from servelab_amd.weights.safetensors_io import write_safetensors


def attention(heads, kv_heads, dim, vdim, size, keep_first, v_mix, ff, scale=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                      "scale": scale if scale is not None else dim ** -0.5,
                      "mask": {"size": size, "keep_first": keep_first}, "v_mix": v_mix},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent(heads, dim, rot_dim, vdim, kv_rank, size, ff, base=10000.0, dims=None, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
                      "mask": {"size": size}, "rot": {"base": base, "dims": dims or rot_dim}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(width, vocab, eps, layers):
    return {"architecture": "Topelorn", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "layers": layers}


# two kinds of mixer interleaved; a layer without feed-forward; value mixing across layers whose
# heads differ (same total width of the values)
MODEL_A = config(64, 300, 1e-5, [
    attention(4, 2, 24, 16, 9, 3, True, 96),
    latent(3, 16, 8, 24, 40, 13, 0),
    attention(4, 2, 24, 16, 9, 3, True, 96),
    attention(2, 2, 8, 16, 40, 0, True, 32, scale=0.5),
])
# a latent layer first, rotating fewer channels than its rotated part has; one kv head for six heads;
# a window longer than any test sequence; more kept tokens than a page holds; a layer that mixes no
# values before the first that does; heads without groups; a width that is no multiple of 32
MODEL_B = config(72, 257, 1e-6, [
    latent(2, 32, 16, 16, 48, 5, 72, base=500.0, dims=8),
    attention(6, 1, 16, 40, 1000, 20, False, 72),
    attention(3, 3, 40, 8, 17, 1, True, 40),
    attention(3, 3, 40, 8, 33, 2, True, 40),
])
# one layer of each kind, for tests that look at one mechanism
MODEL_C = config(96, 128, 1e-5, [
    attention(8, 4, 32, 32, 6, 2, True, 128),
    latent(4, 24, 8, 40, 32, 7, 64),
])
# widths the matrix-core attention takes in bfloat16 (keys in steps of 32, values in steps of 16)
MODEL_D = config(64, 211, 1e-5, [
    attention(4, 2, 32, 16, 9, 3, True, 96),
    latent(3, 16, 16, 24, 48, 13, 0),
    attention(4, 2, 32, 16, 40, 0, True, 64),
])
# sizes that are multiples of nothing convenient: a width of 100, a vocabulary of 97, heads of 12 and 20 channels,
# a latent of 22 with 6 rotated channels of which 4 turn
MODEL_E = config(100, 97, 1e-5, [
    attention(5, 5, 12, 20, 7, 2, True, 52),
    latent(2, 10, 6, 14, 22, 9, 36, base=77.0, dims=4),
    attention(10, 5, 12, 20, 64, 1, True, 0),
])
MODELS = {"A": MODEL_A, "B": MODEL_B, "C": MODEL_C, "D": MODEL_D, "E": MODEL_E}


def tensor_shapes(cfg):
    w, shapes = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        shapes[p + "norm1"] = (w,)
        if layer["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes.update({p + "mix.q": (H * D, w), p + "mix.k": (G * D, w), p + "mix.v": (G * Dv, w),
                           p + "mix.q.norm": (D,), p + "mix.k.norm": (D,), p + "mix.vmix": (),
                           p + "mix.sink": (H,), p + "mix.g": (H, w), p + "mix.o": (w, H * Dv)})
        else:
            H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            shapes.update({p + "mix.q": (H * (D + R), w), p + "mix.dkv": (C + R, w),
                           p + "mix.dkv.norm": (C,), p + "mix.uk": (H * D, C), p + "mix.uv": (H * Dv, C),
                           p + "mix.g": (H, w), p + "mix.o": (w, H * Dv)})
        if layer["mlp"]:
            ff = layer["mlp"]["ff"]
            shapes.update({p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return shapes


def make_weights(cfg, seed=0, dtype=torch.float32):
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("norm") or name.endswith("norm1"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif name.endswith("vmix"):
            t = 0.2 + 0.6 * torch.rand(shape, generator=gen)
        elif name.endswith("sink"):
            t = torch.randn(shape, generator=gen)
        elif name == "embed":
            t = torch.randn(shape, generator=gen)
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / shape[1] ** 0.5)
        out[name] = t.to(dtype)
    return out


def write_folder(tmp_path, cfg, seed=0, tag="m", dtype=torch.float32, weights=None):
    folder = os.path.join(str(tmp_path), f"topelorn_{tag}_{seed}")
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    weights = weights if weights is not None else make_weights(cfg, seed, dtype)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return folder, weights
