"""Zukinex, the slow way: every mechanism of the design as one plain function over a whole sequence.

Double precision on the CPU, full score matrices, experts walked token by token.  Shares nothing with the
package: it is what the package's parts and kernels are held against.

A model is ``(config, weights)``: the config.json mapping and name -> tensor.  A layer's tensors start with
``l<i>.``; a mixer's with ``l<i>.mix.``, a feed-forward's with ``l<i>.mlp.``; linear weights are ``[out, in]``.
"""
import math

import torch

F = torch.float64


def unit_rms(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_adjacent(x, positions, dims, base):
    """x [steps, heads, size]: elements 2i and 2i+1 (2i+1 < dims) turn together by position * base^(-2i/dims);
    elements from ``dims`` on are left alone."""
    if not dims:
        return x
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = torch.tensor(positions, dtype=F)[:, None] * freq[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).reshape(*x.shape[:-1], dims)
    return torch.cat([turned, x[..., dims:]], dim=-1)


def visible(steps, size, keep_first):
    """mask[i, j]: position i sees j if j <= i and (i - j < size or j < keep_first); size None: every j <= i."""
    i = torch.arange(steps)[:, None]
    j = torch.arange(steps)[None, :]
    causal = j <= i
    if size is None:
        return causal
    return causal & ((i - j < size) | (j < keep_first))


def keys_and_values(h, m, w, p, eps, positions):
    """What a layer's cache holds: keys after head norm and rotation [steps, kv_heads, dim], values
    [steps, kv_heads, vdim]."""
    steps = h.shape[0]
    k = (h @ w[p + "k"].T).view(steps, m["kv_heads"], m["dim"])
    v = (h @ w[p + "v"].T).view(steps, m["kv_heads"], m["vdim"])
    k = rms_norm(k, w[p + "k.norm"], eps)
    rot = m.get("rot") or {}
    k = rotate_adjacent(k, positions, int(rot.get("dims", 0)), float(rot.get("base", 1.0)))
    return k, v


def attention(h, m, w, p, eps, positions, kv):
    """The attention mixer on input ``h`` [steps, width]; ``kv`` = (keys, values) it reads (its own or another
    layer's)."""
    steps = h.shape[0]
    heads, groups, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(steps, heads, dim)
    q = rms_norm(q, w[p + "q.norm"], eps)
    rot = m.get("rot") or {}
    q = rotate_adjacent(q, positions, int(rot.get("dims", 0)), float(rot.get("base", 1.0)))
    k, v = kv
    mask = m.get("mask")
    see = visible(steps, None if not mask else int(mask["size"]), 0 if not mask else int(mask.get("keep_first", 0)))
    out = torch.zeros(steps, heads, vdim, dtype=F)
    for head in range(heads):
        g = head // (heads // groups)
        score = (q[:, head] @ k[:, g].T) * m["scale"]
        score = score.masked_fill(~see, float("-inf"))
        out[:, head] = torch.softmax(score, dim=-1) @ v[:, g]
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return (out.reshape(steps, heads * vdim) * gate) @ w[p + "o"].T


def glu(h, w, p, act):
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, router, correction, r):
    """For every row: the chosen outputs of the router and their weights.  ``r`` is the config's router."""
    total = int(r["experts"]) + int(r.get("identity", 0))
    s = torch.softmax(h @ router.T, dim=-1)
    choice = s + correction
    groups = r.get("groups")
    if groups and int(groups["count"]) > 1:
        count, keep = int(groups["count"]), int(groups["keep"])
        size = total // count
        best = choice.view(-1, count, size).max(dim=-1).values
        kept = torch.topk(best, keep, dim=-1).indices
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        allowed = allowed[:, :, None].expand(-1, -1, size).reshape(-1, total)
        choice = choice.masked_fill(~allowed, float("-inf"))
    chosen = torch.topk(choice, int(r["top"]), dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)


def mixture(h, mlp, w, p):
    r = mlp["router"]
    experts = int(r["experts"])
    chosen, weight = route(h, w[p + "router"], w[p + "correction"], r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weight[t]):
            if e >= experts:
                out[t] += a * h[t]                      # an identity expert hands the input on
            else:
                out[t] += a * glu(h[t:t + 1], w, f"{p}e{e}.", silu)[0]
    if mlp.get("shared"):
        out = out + glu(h, w, p + "shared.", silu)
    return out


def feed_forward(h, mlp, w, p):
    if mlp["kind"] == "dense":
        return glu(h, w, p, gelu_tanh)
    return mixture(h, mlp, w, p)


def forward(config, weights, tokens, layers_out=None):
    """Logits [steps, vocab] of one sequence from position 0; ``layers_out`` (a list) receives the stream
    after every layer."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    positions = list(range(len(tokens)))
    x = w["embed"][torch.tensor(tokens)] + w["pos"][torch.tensor(positions)]
    caches = {}
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        if m.get("kv_from") is None:
            caches[i] = keys_and_values(x, m, w, p, eps, positions)
            kv = caches[i]
        else:
            kv = caches[int(m["kv_from"])]
        x = x + rms_norm(attention(x, m, w, p, eps, positions, kv), w[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            x = x + rms_norm(feed_forward(x, layer["mlp"], w, f"l{i}.mlp."), w[f"l{i}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
