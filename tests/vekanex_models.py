"""Small Vekanex configurations and weights for the tests.  The configurations differ from each
other in every size, in the order of their layers and in which options they use; the weights are
drawn so that every mechanism matters (gates and decays well inside their ranges, biases of the
size of their sums, gains away from 1)."""
import json
import os

import torch

from servelab_amd.weights.safetensors_io import write_safetensors


def moe(experts, top, ff, shared=0):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def mlstm(heads, dim, vdim, cap, mlp):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def gla(heads, dim, vdim, tau, rank, mlp):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": rank},
            "mlp": mlp}


def parallel(left, right, left_scale, right_scale, mlp):
    heads, kv, dim, vdim, scale, base, dims = left
    rh, rkv, rdim, rvdim, conv, decay_rank, gate_rank = right
    return {"type": "parallel", "mlp": mlp, "mixer": {
        "left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                 "rot": {"base": base, "dims": dims}},
        "right": {"heads": rh, "kv_heads": rkv, "dim": rdim, "vdim": rvdim, "conv": conv,
                  "decay_rank": decay_rank, "gate_rank": gate_rank},
        "left_scale": left_scale, "right_scale": right_scale}}


def again(layers, j):
    return dict(json.loads(json.dumps(layers[j])), weights_of=j)


def config(width, vocab, eps, mult, softcap, layers):
    return {"architecture": "Vekanex", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "residual_mult": mult, "logit_softcap": softcap, "layers": layers}


def _a():
    layers = [
        parallel((4, 2, 16, 24, 0.3, 10000.0, 8), (4, 2, 16, 8, 4, 8, 12), 1.2, 0.7, moe(5, 2, 24, 40)),
        mlstm(3, 8, 16, 6.0, moe(5, 2, 24, 40)),
        gla(2, 24, 8, 4.0, 4, None),
    ]
    return config(64, 300, 1e-5, 0.7, 12.0, layers + [again(layers, 0), again(layers, 2)])


def _b():
    # a width that is no multiple of 32; one choice per token; no shared expert; a convolution of
    # two taps; every head with its own q and k on the right and one kv head on the left; the whole
    # head rotated
    layers = [
        gla(3, 8, 24, 9.0, 16, moe(3, 1, 16)),
        parallel((3, 1, 8, 8, 0.5, 500.0, 8), (2, 2, 24, 16, 2, 4, 4), 0.5, 1.5, moe(4, 4, 8, 8)),
        mlstm(1, 40, 24, 15.0, None),
    ]
    return config(72, 257, 1e-6, 1.0, 50.0, layers)


def _c():
    # sizes the matrix-core attention takes in bfloat16; key channels beyond one lane group's reach
    layers = [
        mlstm(2, 32, 32, 10.0, moe(8, 3, 32, 16)),
        parallel((4, 4, 32, 16, 0.2, 50000.0, 16), (4, 1, 72, 32, 3, 8, 8), 1.0, 1.0, moe(8, 3, 32, 16)),
        gla(2, 136, 16, 2.0, 8, moe(8, 3, 32, 16)),
    ]
    return config(96, 128, 1e-5, 0.5, 20.0, layers)


def _d():
    # a convolution of one tap (no inputs kept); head counts that are no powers of two; channel
    # counts that are no multiples of four; two rotated channels; more experts than a wavefront has
    # lanes; a layer that borrows from one behind it; two attentions whose pages differ in size
    layers = [
        parallel((5, 5, 12, 20, 0.4, 100.0, 2), (5, 1, 20, 12, 1, 2, 3), 0.3, 1.1, moe(70, 9, 8)),
        gla(5, 20, 12, 1.0, 2, moe(2, 2, 12, 4)),
        mlstm(5, 12, 20, 3.0, moe(2, 1, 12, 4)),
        parallel((2, 1, 16, 8, 0.25, 7.0, 16), (3, 3, 8, 8, 5, 1, 1), 1.0, -0.5, None),
    ]
    return config(40, 97, 1e-4, 0.25, 5.0, [dict(again(layers, 2), weights_of=3)] + layers[:2] + layers[2:])


def _e():
    # no attention at all: the engine holds states and not one page; the decay's projection as wide
    # as a head's key; a feed-forward of one expert that every token takes
    layers = [
        gla(2, 16, 16, 6.0, 16, moe(1, 1, 32)),
        mlstm(2, 16, 8, 8.0, moe(6, 3, 16, 16)),
    ]
    return config(48, 200, 1e-5, 1.5, 8.0, layers + [again(layers, 0)])


MODELS = {"A": _a(), "B": _b(), "C": _c(), "D": _d(), "E": _e()}


def tensor_shapes(cfg):
    """{name: shape} of every tensor a checkpoint of ``cfg`` holds (written from the design)."""
    w, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "head": (cfg["vocab"], cfg["width"]),
                            "final.norm": (cfg["width"],)}
    for i, layer in enumerate(cfg["layers"]):
        if "weights_of" in layer:
            continue
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        x = p + "mix."
        if layer["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            out.update({x + "q": (H * D, w), x + "k": (H * D, w), x + "v": (H * Dv, w), x + "g": (H * Dv, w),
                        x + "o": (w, H * Dv), x + "norm": (H * Dv,), x + "i": (H, w), x + "i.b": (H,),
                        x + "f": (H, w), x + "f.b": (H,)})
        elif layer["type"] == "gla":
            H, D, Dv, r = m["heads"], m["dim"], m["vdim"], m["decay_rank"]
            out.update({x + "q": (H * D, w), x + "k": (H * D, w), x + "v": (H * Dv, w), x + "g": (H * Dv, w),
                        x + "o": (w, H * Dv), x + "norm": (Dv,), x + "a1": (r, w), x + "a2": (H * D, r),
                        x + "a2.b": (H * D,)})
        else:
            l, r = m["left"], m["right"]
            H, G, D, Dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            y = x + "left."
            out.update({y + "q": (H * D, w), y + "q.b": (H * D,), y + "k": (G * D, w), y + "k.b": (G * D,),
                        y + "v": (G * Dv, w), y + "v.b": (G * Dv,), y + "q.norm": (H * D,),
                        y + "k.norm": (G * D,), y + "o": (w, H * Dv), y + "o.b": (w,)})
            H, G, D, Dv = r["heads"], r["kv_heads"], r["dim"], r["vdim"]
            y = x + "right."
            out.update({y + "q": (G * D, w), y + "q.conv": (G * D, r["conv"]), y + "k": (G * D, w),
                        y + "k.conv": (G * D, r["conv"]), y + "v": (H * Dv, w), y + "v.conv": (H * Dv, r["conv"]),
                        y + "b": (H, w), y + "A_log": (H,), y + "norm": (Dv,),
                        y + "a1": (r["decay_rank"], w), y + "a2": (H * D, r["decay_rank"]),
                        y + "dt_bias": (H * D,), y + "g1": (r["gate_rank"], w),
                        y + "g2": (H * Dv, r["gate_rank"]), y + "o": (w, H * Dv)})
        if layer["mlp"] is not None:
            c = layer["mlp"]
            out[p + "norm2"] = (w,)
            y = p + "mlp."
            names = [f"e{e}." for e in range(c["router"]["experts"])]
            sizes = [c["expert"]["ff"]] * len(names)
            if c.get("shared"):
                names.append("shared.")
                sizes.append(c["shared"]["ff"])
            for n, ff in zip(names, sizes):
                out.update({y + n + "gate": (ff, w), y + n + "up": (ff, w), y + n + "down": (w, ff)})
            out[y + "router"] = (c["router"]["experts"], w)
    return out


def make_weights(cfg, seed):
    """Values that are exact in bfloat16, as float32 tensors."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith("norm") or last in ("norm1", "norm2"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "b" and len(shape) == 1 or last == "dt_bias":
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "A_log":
            t = -1.0 + 0.5 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif name in ("embed",):
            t = torch.randn(shape, generator=g)
        elif last == "router":
            t = 2.0 * torch.randn(shape, generator=g) * shape[1] ** -0.5
        else:
            t = 1.5 * torch.randn(shape, generator=g) * shape[-1] ** -0.5
        out[name] = t.to(torch.bfloat16).float()
    return out


def write_folder(tmp_path, cfg, seed, tag, weights=None):
    """(folder, weights): config.json without the low-rank widths (they are read from the
    tensors' shapes, as for a model from outside) and model.safetensors in bfloat16."""
    folder = os.path.join(str(tmp_path), f"vekanex_{tag}")
    os.makedirs(folder, exist_ok=True)
    weights = weights if weights is not None else make_weights(cfg, seed)
    raw = json.loads(json.dumps(cfg))
    for layer in raw["layers"]:
        m = layer["mixer"]
        m.pop("decay_rank", None)
        if "right" in m:
            m["right"].pop("decay_rank", None)
            m["right"].pop("gate_rank", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: t.to(torch.bfloat16) for n, t in weights.items()})
    return folder, weights
