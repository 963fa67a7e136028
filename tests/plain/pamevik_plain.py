"""Pamevik, the slow way: every mechanism of the design as one plain function over a whole sequence.

Double precision on the CPU, token by token where the design is recurrent, full score matrices where it
attends.  Shares nothing with the package: it is what the package's parts and kernels are held against.

A model is ``(config, weights)``: the config.json mapping and name -> tensor.  A layer's tensors start with
``l<i>.``; a mixer's with ``l<i>.mix.``; linear weights are ``[out, in]``.
"""
import math

import torch

F = torch.float64


def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b over the last axis; var is the mean squared deviation."""
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def causal_taps(h, w):
    """out[t, c] = sum_j w[c, j] * h[t - (taps - 1) + j, c], with zeros before the first row.
    The last tap meets the current row."""
    steps, taps = h.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, h.shape[1], dtype=h.dtype), h], dim=0)
    out = torch.zeros_like(h)
    for j in range(taps):
        out += padded[j:j + steps] * w[:, j]
    return out


def input_convolution(h, w):
    """What a sublayer reads: h + conv(h)."""
    return h + causal_taps(h, w)


def rotate_half(x, positions, dims, base):
    """x [steps, heads, size]: the first ``dims`` elements of every head turn in pairs (i, i + dims/2) by the
    angle position * base^(-2i/dims); the rest is left alone."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = torch.tensor(positions, dtype=F)[:, None] * freq[None, :]          # [steps, half]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., dims:]], dim=-1)


def soft_capped(z, cap):
    return cap * torch.tanh(z / cap)


def log_sigmoid(z):
    return -torch.nn.functional.softplus(-z)


# ---- mixers ----------------------------------------------------------------------------------------------

def mlstm(h, w, p, m, eps):
    """Matrix memory with exponential gates and a running maximum that starts at 0."""
    heads, dim, vdim, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    steps = h.shape[0]
    q = (h @ w[p + "q"].T).view(steps, heads, dim) * dim ** -0.5
    k = (h @ w[p + "k"].T).view(steps, heads, dim)
    v = (h @ w[p + "v"].T).view(steps, heads, vdim)
    log_i = soft_capped(h @ w[p + "i"].T + w[p + "i.b"], cap)                 # [steps, heads]
    log_f = log_sigmoid(soft_capped(h @ w[p + "f"].T + w[p + "f.b"], cap))
    memory = torch.zeros(heads, dim, vdim, dtype=F)
    norm = torch.zeros(heads, dim, dtype=F)
    top = torch.zeros(heads, dtype=F)
    out = torch.zeros(steps, heads, vdim, dtype=F)
    for t in range(steps):
        new_top = torch.maximum(log_f[t] + top, log_i[t])
        keep = torch.exp(log_f[t] + top - new_top)
        take = torch.exp(log_i[t] - new_top)
        memory = keep[:, None, None] * memory + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        norm = keep[:, None] * norm + take[:, None] * k[t]
        top = new_top
        read = torch.einsum("hdv,hd->hv", memory, q[t])
        floor = torch.maximum((norm * q[t]).sum(dim=-1).abs(), torch.exp(-top))
        out[t] = read / (floor[:, None] + 1e-6)
    out = unit_rms(out, eps).reshape(steps, heads * vdim) * w[p + "norm"]
    out = out * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def softmax_attention(h, w, p, m, positions):
    """Grouped-query causal softmax attention, rotary on part of a head, one sigmoid gate a head."""
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    steps = h.shape[0]
    q = (h @ w[p + "q"].T).view(steps, heads, dim)
    k = (h @ w[p + "k"].T).view(steps, groups, dim)
    v = (h @ w[p + "v"].T).view(steps, groups, vdim)
    q = rotate_half(q, positions, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half(k, positions, m["rot"]["dims"], m["rot"]["base"])
    gate = torch.sigmoid(h @ w[p + "g"].T)                                   # [steps, heads]
    out = torch.zeros(steps, heads, vdim, dtype=F)
    visible = torch.tril(torch.ones(steps, steps, dtype=torch.bool))
    for head in range(heads):
        g = head // (heads // groups)
        scores = (q[:, head] @ k[:, g].T) * m["scale"]
        scores = scores.masked_fill(~visible, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, g]
    out = out * gate[:, :, None]
    return out.reshape(steps, heads * vdim) @ w[p + "o"].T


def retention(h, w, p, m, positions, eps):
    """Linear attention with one fixed decay a head: S <- decay S + k v^T, o = S^T q."""
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    steps = h.shape[0]
    q = (h @ w[p + "q"].T).view(steps, heads, dim)
    k = (h @ w[p + "k"].T).view(steps, heads, dim)
    v = (h @ w[p + "v"].T).view(steps, heads, vdim)
    q = rotate_half(q, positions, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half(k, positions, m["rot"]["dims"], m["rot"]["base"]) * dim ** -0.5
    decay = torch.tensor(m["decay"], dtype=F)
    memory = torch.zeros(heads, dim, vdim, dtype=F)
    out = torch.zeros(steps, heads, vdim, dtype=F)
    for t in range(steps):
        memory = decay[:, None, None] * memory + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", memory, q[t])
    out = unit_rms(out, eps).reshape(steps, heads * vdim)
    out = out * torch.nn.functional.silu(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def parallel(h, w, p, m, positions, eps):
    """Two mixers on the same input; each result RMS-normed over the width with a plain gain; half their sum."""
    left = softmax_attention(h, w, p + "left.", m["left"], positions)
    right = retention(h, w, p + "right.", m["right"], positions, eps)
    return 0.5 * (unit_rms(left, eps) * w[p + "left.out"] + unit_rms(right, eps) * w[p + "right.out"])


def channel_delta(h, w, p, m, eps):
    """Gated delta rule with one decay per head and key channel."""
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    steps = h.shape[0]
    silu = torch.nn.functional.silu
    q = silu(causal_taps(h @ w[p + "q"].T, w[p + "q.conv"])).view(steps, groups, dim)
    k = silu(causal_taps(h @ w[p + "k"].T, w[p + "k.conv"])).view(steps, groups, dim)
    v = silu(causal_taps(h @ w[p + "v"].T, w[p + "v.conv"])).view(steps, heads, vdim)
    q = q / torch.sqrt((q * q).sum(dim=-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(dim=-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)                                   # [steps, heads]
    rate = torch.exp(w[p + "A_log"])                                         # [heads]
    step = torch.nn.functional.softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"])
    decay = torch.exp(-rate[None, :, None] * step.view(steps, heads, dim))   # [steps, heads, dim]
    memory = torch.zeros(heads, dim, vdim, dtype=F)
    out = torch.zeros(steps, heads, vdim, dtype=F)
    share = heads // groups
    for t in range(steps):
        kt = k[t].repeat_interleave(share, dim=0)                            # [heads, dim]
        qt = q[t].repeat_interleave(share, dim=0)
        memory = decay[t][:, :, None] * memory
        seen = torch.einsum("hdv,hd->hv", memory, kt)
        write = beta[t][:, None] * (v[t] - seen)
        memory = memory + kt[:, :, None] * write[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", memory, qt)
    out = unit_rms(out, eps) * w[p + "norm"]
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(steps, heads, vdim)
    return (out * gate).reshape(steps, heads * vdim) @ w[p + "o"].T


def dense_feed_forward(h, w, p):
    """down(relu(up h)^2)."""
    return torch.relu(h @ w[p + "up"].T) ** 2 @ w[p + "down"].T


# ---- the model -------------------------------------------------------------------------------------------

def mixer(kind, h, w, p, m, positions, eps):
    if kind == "mlstm":
        return mlstm(h, w, p, m, eps)
    if kind == "parallel":
        return parallel(h, w, p, m, positions, eps)
    if kind == "channel_delta":
        return channel_delta(h, w, p, m, eps)
    raise ValueError(kind)


def forward(config, weights, tokens, layers_out=None):
    """Logits [steps, vocab] of one sequence from position 0; ``layers_out`` (a list) receives the stream
    after every layer."""
    w = {name: t.to(F) if t.is_floating_point() else t for name, t in weights.items()}
    eps = config["norm"]["eps"]
    positions = list(range(len(tokens)))
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = input_convolution(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), w[p + "canon1"])
        y = mixer(layer["type"], h, w, p + "mix.", layer["mixer"], positions, eps)
        x = x + layer_norm(y, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        if layer.get("mlp") is not None:
            h = input_convolution(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps), w[p + "canon2"])
            y = dense_feed_forward(h, w, p + "mlp.")
            x = x + layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["head"].T
