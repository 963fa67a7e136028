"""Small Pamevik configurations and weights for the tests, made here from the design's naming alone (the
product's list of tensors is checked against this, not used to make it)."""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import numpy as np
import torch


def mlstm(heads, dim, vdim, cap=8.0, ff=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def delta(heads, kv_heads, dim, vdim, conv, ff=None):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def parallel(heads, kv_heads, dim, vdim, rot_dims, r_heads, r_dim, r_vdim, r_rot, decay, ff=None, scale=None,
             base=10000.0, r_base=500000.0):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "scale": scale if scale is not None else dim ** -0.5, "rot": {"dims": rot_dims, "base": base}},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": list(decay),
                                "rot": {"dims": r_rot, "base": r_base}}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def config(width, vocab, taps, layers, eps=1e-5):
    return {"architecture": "Pamevik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "layers": layers}


# Sizes unlike one another: one head and several, grouped and ungrouped heads, values wider and narrower than
# keys, rotations of the whole head and of a part, two to five taps, widths and feed-forwards that are no
# multiples of 8 or 64, every layer order.
SMALL = {
    "P": config(64, 300, 3, [mlstm(2, 16, 24, 6.0), parallel(4, 2, 16, 8, 8, 2, 24, 16, 24, [0.9, 0.99], ff=96),
                             delta(4, 2, 16, 8, 4)]),
    "Q": config(96, 211, 5, [delta(3, 3, 24, 40, 2, ff=100), parallel(3, 1, 32, 48, 32, 3, 16, 40, 8, [1.0, 0.5, 0.97]),
                             mlstm(1, 40, 16, 15.0, ff=72), mlstm(3, 8, 8, 3.0)], eps=1e-6),
    "R": config(40, 97, 2, [parallel(2, 2, 8, 16, 4, 1, 72, 24, 40, [0.995], scale=0.5), delta(2, 1, 72, 12, 3),
                            mlstm(2, 72, 70, 10.0)]),
    "S": config(48, 130, 4, [mlstm(2, 16, 16, 12.0), delta(2, 2, 16, 16, 4)]),          # no paged cache at all
    # keys and values of one size, a multiple of 64: in bfloat16 the attention branch goes to the matrix-core kernels
    "T": config(128, 257, 3, [parallel(4, 2, 64, 64, 32, 2, 32, 64, 32, [0.96, 0.999], ff=160), mlstm(2, 48, 80, 9.0),
                              parallel(2, 1, 128, 128, 128, 1, 64, 32, 16, [0.9])]),
}
RANKS = {"P": (8, 16), "Q": (12, 8), "R": (5, 8), "S": (8, 8), "T": (8, 8)}      # (a_rank, g_rank); 12 and 5: inner sizes off the runs of 8


def tensor_shapes(raw: dict, ranks=(8, 8)) -> Dict[str, tuple]:
    w, shapes = raw["width"], {}
    shapes["embed"] = (raw["vocab"], w)
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        subs = ["norm1", "norm1b"] + (["norm2", "norm2b"] if layer["mlp"] else [])
        for n in subs:
            shapes[p + n] = (w,)
            shapes[p + n + ".b"] = (w,)
        shapes[p + "canon1"] = (w, raw["canon"]["taps"])
        if layer["mlp"]:
            shapes[p + "canon2"] = (w, raw["canon"]["taps"])
            shapes[p + "mlp.up"] = (layer["mlp"]["ff"], w)
            shapes[p + "mlp.down"] = (w, layer["mlp"]["ff"])
        x = p + "mix."
        if layer["type"] == "mlstm":
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({x + "q": (qk, w), x + "k": (qk, w), x + "v": (vv, w), x + "g": (vv, w), x + "o": (w, vv),
                           x + "norm": (vv,), x + "i": (m["heads"], w), x + "i.b": (m["heads"],),
                           x + "f": (m["heads"], w), x + "f.b": (m["heads"],)})
        elif layer["type"] == "channel_delta":
            qk, vv = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({x + "q": (qk, w), x + "k": (qk, w), x + "v": (vv, w), x + "q.conv": (qk, m["conv"]),
                           x + "k.conv": (qk, m["conv"]), x + "v.conv": (vv, m["conv"]), x + "b": (m["heads"], w),
                           x + "A_log": (m["heads"],), x + "dt_bias": (m["heads"] * m["dim"],), x + "a1": (ranks[0], w),
                           x + "a2": (m["heads"] * m["dim"], ranks[0]), x + "g1": (ranks[1], w), x + "g2": (vv, ranks[1]),
                           x + "norm": (m["vdim"],), x + "o": (w, vv)})
        else:
            l, r = m["left"], m["right"]
            shapes.update({x + "left.q": (l["heads"] * l["dim"], w), x + "left.k": (l["kv_heads"] * l["dim"], w),
                           x + "left.v": (l["kv_heads"] * l["vdim"], w), x + "left.g": (l["heads"], w),
                           x + "left.o": (w, l["heads"] * l["vdim"]), x + "left.out": (w,),
                           x + "right.q": (r["heads"] * r["dim"], w), x + "right.k": (r["heads"] * r["dim"], w),
                           x + "right.v": (r["heads"] * r["vdim"], w), x + "right.g": (r["heads"] * r["vdim"], w),
                           x + "right.o": (w, r["heads"] * r["vdim"]), x + "right.out": (w,)})
    shapes["final.norm"] = (w,)
    shapes["final.norm.b"] = (w,)
    shapes["head"] = (raw["vocab"], w)
    return shapes


def make_weights(raw: dict, seed: int, ranks=(8, 8), dtype=torch.bfloat16, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    """Weights at which every mechanism matters: projections that keep activations of order 1, gains around 1,
    biases and gate biases that are not 0, decays away from 0 and 1.  ``sharpen`` scales the softmax branch's
    queries, so that scores spread and a misplaced key moves the logits.  Rounded to ``dtype`` (what a file holds)."""
    gen = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(raw, ranks).items():
        last = name.split(".")[-1]
        if name.endswith(".b") and len(shape) == 1 and "mix" not in name.split(".")[:-1]:      # a norm's bias
            t = 0.1 * torch.randn(shape, generator=gen)
        elif last in ("norm1", "norm1b", "norm2", "norm2b", "out") or name in ("final.norm",) or name.endswith("mix.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=gen)
        elif last in ("canon1", "canon2", "conv"):
            t = 0.4 * torch.randn(shape, generator=gen)
        elif name.endswith("i.b") or name.endswith("f.b"):
            t = torch.randn(shape, generator=gen) + (2.0 if name.endswith("f.b") else 0.0)
        elif last == "A_log":
            t = torch.randn(shape, generator=gen) * 0.5 - 1.0
        elif last == "dt_bias":
            t = torch.randn(shape, generator=gen)
        elif name == "embed":
            t = torch.randn(shape, generator=gen)
        else:
            t = torch.randn(shape, generator=gen) * (1.5 / math.sqrt(shape[-1]))
            if name.endswith("left.q"):
                t = t * sharpen
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
