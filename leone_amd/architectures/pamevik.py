"""Pamevik: how its configuration becomes parts.

A small decoder-only design whose layers are listed one by one in config.json.  Every layer is a "sandwich"
block: layer norm, input convolution, mixer, layer norm, residual sum, and the same around a squared-ReLU
feed-forward if the layer has one.  The mixer is an mLSTM cell, a gated delta rule with a decay per key channel,
or softmax attention and retention side by side (``config/pamevik.py`` lists the keys).  Embedding, then the
layers, a final layer norm and an untied output head.  Tensor names: ``embed``, ``head``, ``final.norm[.b]``,
and per layer ``l<i>.norm1[.b]``, ``l<i>.norm1b[.b]``, ``l<i>.canon1``, ``l<i>.mix.*`` (and ``norm2``,
``norm2b``, ``canon2``, ``mlp.up``, ``mlp.down`` with a feed-forward).
"""
from __future__ import annotations

from ..config.pamevik import ChannelDeltaConfig, MlstmConfig, PamevikConfig, ParallelConfig
from ..parts.base import PartSpec
from ..parts.model import ModelSpec, default_schedule
from .registry import register_architecture


def _norm(config: PamevikConfig, name: str) -> PartSpec:
    return PartSpec("layernorm", {"size": config.width, "eps": config.eps, "weight": name, "bias": name + ".b"})


def _canon(config: PamevikConfig, name: str) -> PartSpec:
    return PartSpec("causal_conv", {"channels": config.width, "taps": config.taps, "weights": [name], "add_input": True})


def _mixer(config: PamevikConfig, i: int, positions: dict) -> PartSpec:
    m, p = config.layers[i].mixer, f"l{i}.mix."
    if isinstance(m, MlstmConfig):
        return PartSpec("mlstm", {"hidden": config.width, "heads": m.heads, "dim": m.dim, "vdim": m.vdim,
                                  "gate_cap": m.gate_cap, "eps": config.eps, "q": p + "q", "k": p + "k", "v": p + "v",
                                  "g": p + "g", "o": p + "o", "norm": p + "norm", "i": p + "i", "i_bias": p + "i.b",
                                  "f": p + "f", "f_bias": p + "f.b"})
    if isinstance(m, ChannelDeltaConfig):
        if m.a_rank is None or m.g_rank is None:
            raise ValueError(f"layer {i}: the ranks of the low-rank projections are read from the tensors "
                             f"(PamevikConfig.with_shapes) or given (with_ranks)")
        return PartSpec("channel_delta", {"hidden": config.width, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim,
                                          "vdim": m.vdim, "taps": m.conv, "eps": config.eps, "a_rank": m.a_rank,
                                          "g_rank": m.g_rank, "q": p + "q", "k": p + "k", "v": p + "v",
                                          "q_conv": p + "q.conv", "k_conv": p + "k.conv", "v_conv": p + "v.conv",
                                          "b": p + "b", "A_log": p + "A_log", "dt_bias": p + "dt_bias", "a1": p + "a1",
                                          "a2": p + "a2", "g1": p + "g1", "g2": p + "g2", "norm": p + "norm", "o": p + "o"})
    assert isinstance(m, ParallelConfig)

    def rope(dims: int, base: float) -> str:
        name = f"rope_{dims}_{base!r}"
        positions.setdefault(name, PartSpec("rope_half_split", {"rotary_dim": dims, "theta": base}))
        return name

    l, r = m.left, m.right
    left = PartSpec("gqa_attention", {"hidden": config.width, "q_heads": l.heads, "kv_heads": l.kv_heads, "head_dim": l.dim,
                                      "value_dim": l.vdim, "qk_norm_eps": None, "window": None, "scale": l.scale,
                                      "position": rope(l.rot_dims, l.rot_base), "float_output": True,
                                      "q": p + "left.q", "k": p + "left.k", "v": p + "left.v", "o": p + "left.o",
                                      "gate": p + "left.g"})
    right = PartSpec("retention", {"hidden": config.width, "heads": r.heads, "dim": r.dim, "vdim": r.vdim,
                                   "decay": list(r.decay), "eps": config.eps, "position": rope(r.rot_dims, r.rot_base),
                                   "q": p + "right.q", "k": p + "right.k", "v": p + "right.v", "g": p + "right.g",
                                   "o": p + "right.o"})
    return PartSpec("parallel", {"hidden": config.width, "eps": config.eps, "branches": {"left": left, "right": right},
                                 "gains": {"left": p + "left.out", "right": p + "right.out"}, "scale": 0.5})


def pamevik_model_spec(config: PamevikConfig) -> ModelSpec:
    positions: dict = {}
    layers = []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        params = {"norm1": _norm(config, p + "norm1"), "conv1": _canon(config, p + "canon1"),
                  "mixer": _mixer(config, i, positions), "norm1b": _norm(config, p + "norm1b")}
        if layer.ff is not None:
            params.update(norm2=_norm(config, p + "norm2"), conv2=_canon(config, p + "canon2"),
                          feed_forward=PartSpec("relu2", {"hidden": config.width, "intermediate": layer.ff,
                                                          "up": p + "mlp.up", "down": p + "mlp.down"}),
                          norm2b=_norm(config, p + "norm2b"))
        layers.append(PartSpec("sandwich", params))
    return ModelSpec(hidden_size=config.width, vocab_size=config.vocab, max_positions=config.max_positions,
                     embedding="embed", layers=layers, schedule=default_schedule(len(layers)),
                     final_norm=_norm(config, "final.norm"), head="head", positions=positions)


register_architecture(PamevikConfig.ARCHITECTURE, PamevikConfig.from_dict, pamevik_model_spec)
