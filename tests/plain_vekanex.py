"""A slow, whole-sequence implementation of the Vekanex design in float64, one function per
mechanism, written from the design's equations.  It shares no code with servelab_amd: the tests
hold the engine to it.

config: the dict of config.json.  weights: {tensor name: torch tensor}.  Everything runs on the
CPU, token by token where the design is a recurrence."""
import math

import torch

F = torch.float64


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis (w None: no gain)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def linear(x, w, b=None):
    y = x @ w.T
    return y if b is None else y + b


def silu(z):
    return z * torch.sigmoid(z)


def logsigmoid(z):
    return -torch.nn.functional.softplus(-z)


def softcap(z, cap):
    return cap * torch.tanh(z / cap)


# --------------------------------------------------------------------------- mixers
def mlstm(h, m, w, p, eps):
    """Matrix memory with exponential gating and a running maximum that starts at 0."""
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = linear(h, w[p + "q"]).view(T, H, D) * D ** -0.5
    k = linear(h, w[p + "k"]).view(T, H, D)
    v = linear(h, w[p + "v"]).view(T, H, Dv)
    i_gate = softcap(linear(h, w[p + "i"], w[p + "i.b"]), cap)                  # [T, H]
    f_gate = logsigmoid(softcap(linear(h, w[p + "f"], w[p + "f.b"]), cap))
    S = torch.zeros(H, D, Dv, dtype=F)
    n = torch.zeros(H, D, dtype=F)
    mx = torch.zeros(H, dtype=F)
    out = torch.zeros(T, H, Dv, dtype=F)
    for t in range(T):
        new = torch.maximum(f_gate[t] + mx, i_gate[t])
        keep = torch.exp(f_gate[t] + mx - new)
        add = torch.exp(i_gate[t] - new)
        S = keep[:, None, None] * S + add[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + add[:, None] * k[t]
        mx = new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    out = rms_norm(out, None, eps).reshape(T, H * Dv) * w[p + "norm"]
    out = out * torch.sigmoid(linear(h, w[p + "g"]))
    return linear(out, w[p + "o"])


def rotate(x, pos, dims, base):
    """x [T, heads, D]: the first ``dims`` channels turn, channel i with channel i + dims/2."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = pos.to(F)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def softmax_attention(h, m, w, p, eps):
    """Grouped heads, biases, a norm over the whole q (and k) projection, rotation of the leading
    channels, causal softmax."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(linear(h, w[p + "q"], w[p + "q.b"]), w[p + "q.norm"], eps).view(T, H, D)
    k = rms_norm(linear(h, w[p + "k"], w[p + "k.b"]), w[p + "k.norm"], eps).view(T, G, D)
    v = linear(h, w[p + "v"], w[p + "v.b"]).view(T, G, Dv)
    pos = torch.arange(T)
    q = rotate(q, pos, m["rot"]["dims"], float(m["rot"]["base"]))
    k = rotate(k, pos, m["rot"]["dims"], float(m["rot"]["base"]))
    out = torch.zeros(T, H, Dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(pos[None, :] > pos[:, None], float("-inf"))
        out[:, head] = torch.softmax(s, -1) @ v[:, g]
    return linear(out.reshape(T, H * Dv), w[p + "o"], w[p + "o.b"])


def short_conv(x, taps):
    """x [T, C], taps [C, n]: y_t = sum_j taps[:, j] x_(t - (n - 1) + j), zeros before the start."""
    n = taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, x.shape[1], dtype=F), x], 0)
    return sum(padded[j:j + x.shape[0]] * taps[:, j] for j in range(n))


def gated_delta(h, m, w, p, eps):
    """Gated delta rule with a decay per key channel."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(linear(h, w[p + "q"]), w[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(linear(h, w[p + "k"]), w[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(linear(h, w[p + "v"]), w[p + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(linear(h, w[p + "b"]))                                # [T, H]
    a = linear(linear(h, w[p + "a1"]), w[p + "a2"]) + w[p + "dt_bias"]
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None]
                      * torch.nn.functional.softplus(a).view(T, H, D))          # [T, H, D]
    S = torch.zeros(H, D, Dv, dtype=F)
    out = torch.zeros(T, H, Dv, dtype=F)
    for t in range(T):
        for head in range(H):
            g = head // (H // G)
            Sh = decay[t, head][:, None] * S[head]
            u = beta[t, head] * (v[t, head] - Sh.T @ k[t, g])
            Sh = Sh + k[t, g][:, None] * u[None, :]
            S[head] = Sh
            out[t, head] = Sh.T @ q[t, g]
    out = rms_norm(out, w[p + "norm"], eps)
    out = out.reshape(T, H * Dv) * torch.sigmoid(linear(linear(h, w[p + "g1"]), w[p + "g2"]))
    return linear(out, w[p + "o"])


def parallel(h, m, w, p, eps):
    return float(m["left_scale"]) * softmax_attention(h, m["left"], w, p + "left.", eps) \
        + float(m["right_scale"]) * gated_delta(h, m["right"], w, p + "right.", eps)


def gla(h, m, w, p, eps):
    """Gated linear attention: a decay per key channel, alpha = sigmoid(z)^(1/tau)."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = linear(h, w[p + "q"]).view(T, H, D) * D ** -0.5
    k = linear(h, w[p + "k"]).view(T, H, D)
    v = linear(h, w[p + "v"]).view(T, H, Dv)
    z = linear(linear(h, w[p + "a1"]), w[p + "a2"], w[p + "a2.b"]).view(T, H, D)
    alpha = torch.exp(logsigmoid(z) / float(m["tau"]))
    S = torch.zeros(H, D, Dv, dtype=F)
    out = torch.zeros(T, H, Dv, dtype=F)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = rms_norm(out, w[p + "norm"], eps).reshape(T, H * Dv)
    return linear(out * silu(linear(h, w[p + "g"])), w[p + "o"])


MIXERS = {"mlstm": mlstm, "parallel": parallel, "gla": gla}


# --------------------------------------------------------------------------- feed-forward
def expert(h, w, p):
    return linear(silu(linear(h, w[p + "gate"])) * linear(h, w[p + "up"]), w[p + "down"])


def routed_experts(h, mlp, w, p):
    top = mlp["router"]["top"]
    z = linear(h, w[p + "router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        best = torch.topk(z[t], top).indices
        share = torch.softmax(z[t][best], -1)
        for e, s in zip(best.tolist(), share):
            out[t] += s * expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared") is not None:
        out = out + expert(h, w, p + "shared.")
    return out


# --------------------------------------------------------------------------- model
def forward(config, weights, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` (a list) receives the stream after every
    layer run."""
    w = {n: t.to(F) for n, t in weights.items()}
    eps, mult = float(config["norm"]["eps"]), float(config["residual_mult"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', i)}."
        y = MIXERS[layer["type"]](x, layer["mixer"], w, p + "mix.", eps)
        x = x + mult * rms_norm(y, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = routed_experts(x, layer["mlp"], w, p + "mlp.")
            x = x + mult * rms_norm(y, w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = linear(rms_norm(x, w["final.norm"], eps), w["head"])
    return softcap(logits, float(config["logit_softcap"]))
