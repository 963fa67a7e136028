"""Zukinex: how its configuration becomes parts.

A small decoder-only design of attention layers listed one by one in config.json.  The token's vector and a learned
vector of its position make the stream.  In a layer the norms stand behind the sublayers, which read the stream itself
(``postnorm`` block).  The mixer is grouped-query softmax attention with a head norm on queries and keys, a rotation of
neighbouring pairs on the first elements of a head, a window that keeps the first positions in sight, and an output
gate for every element; a layer may read the keys and values of an earlier layer instead of making its own.  The
feed-forward is a gated one (tanh form of gelu), a mixture of gated experts (silu) with identity experts and a shared
expert, or absent.  A final RMS norm and an untied output head.  Tensor names: ``embed``, ``pos``, ``head``,
``final.norm`` and per layer ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.{q,k,v,g,o,q.norm,k.norm}``,
``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,correction,e<j>.{gate,up,down},shared.{gate,up,down}}``.
"""
from __future__ import annotations

from ..config.zukinex import DenseConfig, MoeConfig, ZukinexConfig
from ..parts.base import PartSpec
from ..parts.model import LayerRun, ModelSpec
from .registry import register_architecture


def _norm(config: ZukinexConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": config.width, "eps": config.eps, "weight": name})


def _mixer(config: ZukinexConfig, i: int, positions: dict) -> PartSpec:
    m, p = config.layers[i].mixer, f"l{i}.mix."
    position = None
    if m.rot_dims:
        position = f"rope_{m.rot_dims}_{m.rot_base!r}"
        positions.setdefault(position, PartSpec("rope_adjacent", {"rotary_dim": m.rot_dims, "theta": m.rot_base}))
    params = {"hidden": config.width, "q_heads": m.heads, "kv_heads": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim,
              "qk_norm_eps": config.eps, "scale": m.scale, "window": m.window, "keep_first": m.keep_first,
              "position": position, "float_output": True, "gate": p + "g", "gate_each": True,
              "q": p + "q", "o": p + "o", "q_norm": p + "q.norm"}
    if m.kv_from is None:
        window, first = config.kv_retention(i)
        params.update(k=p + "k", v=p + "v", k_norm=p + "k.norm", retain_window=window, retain_first=first)
    else:
        window, first = config.kv_retention(m.kv_from)
        params.update(shared_kv=True, retain_window=window, retain_first=first)
    return PartSpec("gqa_attention", params)


def _feed_forward(config: ZukinexConfig, i: int):
    f, p = config.layers[i].mlp, f"l{i}.mlp."
    if f is None:
        return None
    if isinstance(f, DenseConfig):
        return PartSpec("swiglu", {"hidden": config.width, "intermediate": f.ff, "activation": "gelu_tanh", "float_output": True,
                                   "gate": p + "gate", "up": p + "up", "down": p + "down"})
    assert isinstance(f, MoeConfig)
    shared = None
    if f.shared_ff is not None:
        shared = PartSpec("swiglu", {"hidden": config.width, "intermediate": f.shared_ff, "activation": "silu", "float_output": True,
                                     "gate": p + "shared.gate", "up": p + "shared.up", "down": p + "shared.down"})
    return PartSpec("routed_glu", {"hidden": config.width, "experts": f.experts, "identity": f.identity, "top": f.top,
                                   "group_count": f.group_count, "group_keep": f.group_keep, "intermediate": f.expert_ff,
                                   "activation": "silu", "router": p + "router", "correction": p + "correction",
                                   "expert": p + "e{e}", "shared": shared})


def zukinex_model_spec(config: ZukinexConfig) -> ModelSpec:
    positions: dict = {}
    layers, schedule = [], []
    for i, layer in enumerate(config.layers):
        p = f"l{i}."
        params = {"mixer": _mixer(config, i, positions), "norm1": _norm(config, p + "norm1")}
        feed_forward = _feed_forward(config, i)
        if feed_forward is not None:
            params.update(feed_forward=feed_forward, norm2=_norm(config, p + "norm2"))
        layers.append(PartSpec("postnorm", params))
        # a layer without keys of its own runs on the cache slot of the layer whose keys it reads, and writes nothing
        source = layer.mixer.kv_from
        schedule.append(LayerRun(i, i if source is None else source, source is None))
    return ModelSpec(hidden_size=config.width, vocab_size=config.vocab, max_positions=config.max_positions,
                     embedding="embed", layers=layers, schedule=schedule, final_norm=_norm(config, "final.norm"),
                     head="head", positions=positions, position_table="pos")


register_architecture(ZukinexConfig.ARCHITECTURE, ZukinexConfig.from_dict, zukinex_model_spec)
