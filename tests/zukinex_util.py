"""Small Zukinex configurations and weights for the tests, made here from the design's naming alone (the product's
list of tensors is checked against this, not used to make it)."""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, rot=None, mask=None, kv_from=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if rot is not None:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    if mask is not None:
        m["mask"] = {"size": mask[0], "keep_first": mask[1]}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0, groups=None, shared=None):
    router = {"experts": experts, "top": top, "identity": identity}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer, mlp=None):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5, max_positions=512):
    return {"architecture": "Zukinex", "vocab": vocab, "width": width, "max_positions": max_positions, "norm": {"eps": eps},
            "layers": layers}


# Sizes unlike one another: one head and several, grouped and ungrouped heads, values wider and narrower than keys,
# rotations of the whole head, of a part and none, windows below, at and above a page of 16 with and without kept
# first keys, no window, a reader of another layer's keys with a wider and with a narrower mask than the owner's,
# layers without feed-forward, dense ones, mixtures with and without identity experts, groups and a shared expert,
# one expert chosen and several, widths that are no multiples of 64.
SMALL = {
    "A": config(64, 211, [
        layer(attention(4, 2, 16, 24, rot=(8, 10000.0), mask=(20, 3)), moe(6, 3, 24, identity=2, groups=(4, 2), shared=40)),
        layer(attention(4, 2, 16, 24, rot=(8, 10000.0), mask=(33, 5), kv_from=0), dense(72)),
        layer(attention(2, 2, 32, 32, rot=(32, 500.0))),
        layer(attention(2, 2, 32, 32, rot=(32, 500.0), mask=(7, 0), kv_from=2), moe(5, 1, 20)),
    ]),
    "B": config(96, 130, [
        layer(attention(3, 1, 24, 16, mask=(16, 1)), dense(100)),
        layer(attention(1, 1, 40, 48, rot=(16, 77.0), mask=(40, 17)), moe(4, 2, 40, identity=4, groups=(2, 1), shared=24)),
        layer(attention(3, 1, 24, 16, mask=(5, 2), kv_from=0), moe(9, 4, 8, identity=1, groups=(5, 3))),
    ], eps=1e-6),
    # keys and values of one size, a multiple of 16: in bfloat16 attention goes to the matrix-core kernels
    "C": config(128, 257, [
        layer(attention(4, 2, 64, 64, rot=(64, 1000.0), mask=(24, 4)), dense(160)),
        layer(attention(4, 2, 64, 64, rot=(64, 1000.0), mask=(50, 2), kv_from=0), moe(8, 2, 64, identity=2, groups=(2, 2), shared=64)),
        layer(attention(8, 1, 32, 32, rot=(16, 1000.0)), moe(4, 4, 32, shared=32)),
    ]),
}


def tensor_shapes(raw: dict) -> Dict[str, tuple]:
    w, shapes = raw["width"], {}
    shapes["embed"] = (raw["vocab"], w)
    shapes["pos"] = (raw["max_positions"], w)
    for i, entry in enumerate(raw["layers"]):
        p, m, f = f"l{i}.", entry["mixer"], entry["mlp"]
        shapes[p + "norm1"] = (w,)
        x = p + "mix."
        shapes.update({x + "q": (m["heads"] * m["dim"], w), x + "q.norm": (m["dim"],), x + "g": (m["heads"] * m["vdim"], w),
                       x + "o": (w, m["heads"] * m["vdim"])})
        if m.get("kv_from") is None:
            shapes.update({x + "k": (m["kv_heads"] * m["dim"], w), x + "v": (m["kv_heads"] * m["vdim"], w),
                           x + "k.norm": (m["dim"],)})
        if f is None:
            continue
        shapes[p + "norm2"] = (w,)
        y = p + "mlp."
        if f["kind"] == "dense":
            shapes.update({y + "gate": (f["ff"], w), y + "up": (f["ff"], w), y + "down": (w, f["ff"])})
            continue
        r = f["router"]
        total = r["experts"] + r.get("identity", 0)
        shapes[y + "router"] = (total, w)
        shapes[y + "correction"] = (total,)
        for e in range(r["experts"]):
            ff = f["expert"]["ff"]
            shapes.update({f"{y}e{e}.gate": (ff, w), f"{y}e{e}.up": (ff, w), f"{y}e{e}.down": (w, ff)})
        if f.get("shared"):
            ff = f["shared"]["ff"]
            shapes.update({y + "shared.gate": (ff, w), y + "shared.up": (ff, w), y + "shared.down": (w, ff)})
    shapes["final.norm"] = (w,)
    shapes["head"] = (raw["vocab"], w)
    return shapes


def make_weights(raw: dict, seed: int, dtype=torch.bfloat16, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    """Weights at which every mechanism matters: projections that keep activations of order 1, gains around 1, a
    router whose scores spread, corrections of both signs that are of the scores' size.  ``sharpen`` scales the gain
    of the queries' head norm, so that scores spread and a misplaced key moves the logits.  Rounded to ``dtype``."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw).items():
        last = name.split(".")[-1]
        if name.endswith("q.norm"):
            t = (1.0 + 0.2 * torch.randn(shape, generator=gen)) * sharpen
        elif last in ("norm1", "norm2", "norm") or name.endswith("k.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif name == "embed":
            t = torch.randn(shape, generator=gen)
        elif name == "pos":
            t = 0.5 * torch.randn(shape, generator=gen)
        elif last == "router":
            t = torch.randn(shape, generator=gen) * (3.0 / math.sqrt(shape[-1]))
        elif last == "correction":
            t = 0.15 * torch.randn(shape, generator=gen)
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / math.sqrt(shape[-1]))
        out[name] = t.to(dtype)
    return out


def write_dir(path: str, raw: dict, weights: Dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as handle:
        json.dump(raw, handle)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return path


def relative_error(have: np.ndarray, want: np.ndarray) -> np.ndarray:
    """Per row: root mean square of the difference (its mean taken off, as a logit's shift means nothing) over
    the root mean square of the expected logits."""
    d = have.astype(np.float64) - want.astype(np.float64)
    d = d - d.mean(axis=-1, keepdims=True)
    scale = np.sqrt((want.astype(np.float64) ** 2).mean()) + 1e-30
    return np.sqrt((d * d).mean(axis=-1)) / scale
