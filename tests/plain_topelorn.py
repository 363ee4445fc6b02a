"""Plain, slow implementation of the Topelorn decoder.

Whole sequences, no cache, one function per mechanism, torch on the CPU in the
precision of the tensors it is given (float32 or float64).  It shares no code
with ``servelab_amd``: configurations are the plain dicts of config.json and
weights a {name: tensor} dict.  Every engine test of this design compares
against it.

Notation: T tokens at positions 0..T-1, rows of ``h`` are tokens; a weight
matrix W [out, in] is applied as h @ W.T.
"""
import math

import torch


# ------------------------------------------------------------------- norms
def layer_norm_gain(x, gain, eps):
    """(x - mean) / sqrt(var + eps) * gain, var = mean of squared deviations."""
    mu = x.mean(dim=-1, keepdim=True)
    dev = x - mu
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * gain


def rms_norm_gain(x, gain, eps):
    """x / sqrt(mean(x^2) + eps) * gain."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x / torch.sqrt(ms + eps) * gain


# --------------------------------------------------------------- visibility
def window_mask(T, size, keep_first=0):
    """[T, T] bool: query i sees key j iff j <= i and (i - j < size or
    j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def distance_slopes(heads, dtype):
    """slope_h = 2^(-8 (h + 1) / heads), h = 0 .. heads-1."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=dtype)


def softmax_with_sink(scores, visible, sink=None):
    """Softmax over the visible keys of each row; ``sink`` [heads] adds
    exp(sink_h) to the denominator (no key, no value).  scores [heads, T, T]."""
    s = scores.masked_fill(~visible[None], -math.inf)
    top = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None, None])
    e = torch.exp(s - top)
    denom = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink[:, None, None] - top)
    return e / denom


# ------------------------------------------------------------------ mixers
def biased_attention(h, w, m, eps, v_first=None):
    """The 'attention' mixer.  ``w``: the mixer's tensors by short name,
    ``m``: its config dict.  Returns (output [T, width], the values this layer
    computed before mixing [T, G * vdim])."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, D)
    k = (h @ w["k"].T).view(T, G, D)
    v_own = h @ w["v"].T
    q = rms_norm_gain(q, w["q.norm"], eps)
    k = rms_norm_gain(k, w["k.norm"], eps)
    v = v_own
    if v_first is not None:
        lam = w["vmix"]
        v = (1 - lam) * v_own + lam * v_first
    v = v.view(T, G, Dv)
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1)          # head h uses kv head h // rep
    vh = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"]
    pos = torch.arange(T, dtype=h.dtype)
    dist = pos[:, None] - pos[None, :]
    scores = scores - distance_slopes(H, h.dtype)[:, None, None] * dist[None]
    mask = m.get("mask") or {}
    visible = window_mask(T, mask.get("size", T), mask.get("keep_first", 0))
    p = softmax_with_sink(scores, visible, w["sink"].to(h.dtype))
    out = torch.einsum("hij,jhd->ihd", p, vh)
    gate = torch.sigmoid(h @ w["g"].T)            # [T, H]
    out = out * gate[:, :, None]
    return out.reshape(T, H * Dv) @ w["o"].T, v_own


def rotate_pairs(x, positions, base, dims):
    """Rotary positions on the first ``dims`` channels of the last axis of x
    [T, ..., D]: channel i pairs with i + dims/2, angle p * base^(-2i/dims)."""
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=x.dtype) / dims)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def latent_attention(h, w, m, eps):
    """The 'latent_attention' mixer, in its direct form: keys and values of
    every head are made from the latent."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ w["q"].T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    down = h @ w["dkv"].T
    latent = rms_norm_gain(down[:, :C], w["dkv.norm"], eps)
    k_rot = down[:, C:]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q_rot = rotate_pairs(q_rot, pos, base, dims)
    k_rot = rotate_pairs(k_rot, pos, base, dims)
    k_plain = (latent @ w["uk"].T).view(T, H, D)
    v = (latent @ w["uv"].T).view(T, H, Dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain)
              + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * m["scale"]
    mask = m.get("mask") or {}
    visible = window_mask(T, mask.get("size", T))
    p = softmax_with_sink(scores, visible)
    out = torch.einsum("hij,jhd->ihd", p, v)
    gate = torch.sigmoid(h @ w["g"].T)
    out = out * gate[:, :, None]
    return out.reshape(T, H * Dv) @ w["o"].T


def dense_ff(h, w):
    """down(silu(gate h) * (up h))."""
    a = h @ w["gate"].T
    return (a * torch.sigmoid(a) * (h @ w["up"].T)) @ w["down"].T


# ------------------------------------------------------------------- model
def sub(weights, prefix):
    return {n[len(prefix):]: t for n, t in weights.items() if n.startswith(prefix)}


def forward(config, weights, tokens, dtype=torch.float64, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the stream after each layer)."""
    w = {n: t.to(dtype) for n, t in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    v_first = None
    after = []
    for i, layer in enumerate(config["layers"]):
        h = layer_norm_gain(x, w[f"l{i}.norm1"], eps)
        mw = sub(w, f"l{i}.mix.")
        m = layer["mixer"]
        if layer["type"] == "attention":
            if m.get("v_mix"):
                y, v_own = biased_attention(h, mw, m, eps, v_first)
                if v_first is None:
                    v_first = v_own
            else:
                y, _ = biased_attention(h, mw, m, eps, None)
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, mw, m, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp"):
            y = y + dense_ff(h, sub(w, f"l{i}.mlp."))
        x = x + y
        after.append(x)
    logits = layer_norm_gain(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, torch.stack(after)) if return_layers else logits
