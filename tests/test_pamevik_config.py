"""Pamevik on the CPU: configuration, registry, the list of tensors, cache needs, and the plain implementation's
own consistency (a sequence and its prefix, each mechanism's recurrence against its closed form)."""
import copy

import pytest
import torch

from tests import pamevik_util as pu
from tests.plain import pamevik_plain as plain


def test_configuration_reads_back_and_is_chosen_by_name():
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.config.pamevik import PamevikConfig
    for name, raw in pu.SMALL.items():
        config = config_from_dict(raw)
        assert isinstance(config, PamevikConfig) and config.architecture == "Pamevik"
        assert config.width == raw["width"] and config.vocab == raw["vocab"] and config.taps == raw["canon"]["taps"]
        assert config.eps == raw["norm"]["eps"] and len(config.layers) == len(raw["layers"])
        assert config.to_dict() == raw
        ranked = config.with_ranks(*pu.RANKS[name])
        assert config_from_dict(ranked.to_dict()) == ranked
        with pytest.raises(ValueError):
            if any(layer["type"] == "channel_delta" for layer in raw["layers"]):
                model_spec_for(config)          # the ranks come from the tensors
            else:
                raise ValueError


@pytest.mark.parametrize("path, value, field", [
    (("canon", "taps"), 1, "canon.taps"), (("norm", "eps"), 0.0, "eps"), (("vocab",), -3, "vocab"),
    (("layers", 0, "type"), "lstm", "type"), (("layers", 0, "mixer", "heads"), 0, "heads"),
    (("layers", 1, "mixer", "left", "kv_heads"), 3, "kv_heads"), (("layers", 1, "mixer", "left", "rot", "dims"), 7, "rot.dims"),
    (("layers", 1, "mixer", "right", "decay"), [0.5], "decay"), (("layers", 1, "mlp", "kind"), "moe", "mlp.kind"),
    (("layers", 2, "mixer", "kv_heads"), 3, "kv_heads"), (("layers", 2, "mixer", "conv"), 1, "conv"),
])
def test_configuration_errors_name_the_key(path, value, field):
    from leone_amd.architectures import config_from_dict
    from leone_amd.config.base import ConfigError
    raw = copy.deepcopy(pu.SMALL["P"])
    at = raw
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as caught:
        config_from_dict(raw)
    assert field in str(caught.value)


def test_unknown_architecture_is_refused_by_name():
    from leone_amd.architectures import config_from_dict
    from leone_amd.config.base import UnsupportedArchitecture
    with pytest.raises(UnsupportedArchitecture):
        config_from_dict({"architecture": "Pamevic"})


@pytest.mark.parametrize("name", list(pu.SMALL))
def test_the_model_asks_for_exactly_the_designs_tensors(name):
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.parts.model import DecoderModel
    raw = pu.SMALL[name]
    shapes = pu.tensor_shapes(raw, pu.RANKS[name])
    config = config_from_dict(raw).with_shapes(shapes)
    model = DecoderModel(model_spec_for(config), torch.float32, "cpu")
    assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == shapes


def test_cache_needs_of_every_layer_kind():
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.parts import KvNeed, StateNeed
    from leone_amd.parts.model import DecoderModel
    raw = pu.SMALL["P"]
    config = config_from_dict(raw).with_ranks(*pu.RANKS["P"])
    needs = DecoderModel(model_spec_for(config), torch.float32, "cpu").cache_needs()
    taps, width = raw["canon"]["taps"], raw["width"]
    assert needs[(0, "mixer")] == StateNeed((2, 16 * 24 + 16 + 1))
    assert needs[(0, "conv1")] == StateNeed((taps - 1, width)) and (0, "conv2") not in needs
    assert needs[(1, "mixer", "left")] == KvNeed(2, 16, value_dim=8)
    assert needs[(1, "mixer", "right")] == StateNeed((2, 24 * 16))
    assert needs[(1, "conv2")] == StateNeed((taps - 1, width))
    assert needs[(2, "mixer", "memory")] == StateNeed((4, 16, 8))
    assert needs[(2, "mixer", "conv")] == StateNeed((3, 2 * 2 * 16 + 4 * 8))


def test_cache_manager_without_paged_groups_hands_out_and_reuses_slots():
    """A model whose layers all keep state only has no pages at all: requests still get slots, lengths advance,
    and a slot that is given back is handed out again."""
    from leone_amd.cache.manager import CacheManager, OutOfSlots
    manager = CacheManager([], 2, 512)
    a, b = manager.admit("a"), manager.admit("b")
    assert {a, b} == {0, 1}
    with pytest.raises(OutOfSlots):
        manager.admit("c")
    manager.reserve("a", 5)
    manager.commit("a", 5)
    assert manager.length("a") == 5 and manager.length("b") == 0
    manager.release("a")
    assert manager.admit("c") == a and manager.length("c") == 0
    manager.check()


# ---- the plain implementation against itself ------------------------------------------------------------------

def test_plain_logits_of_a_prefix_do_not_depend_on_what_follows():
    raw = pu.SMALL["P"]
    w = pu.make_weights(raw, 3, pu.RANKS["P"])
    tokens = torch.randint(0, raw["vocab"], (40,), generator=torch.Generator().manual_seed(1)).tolist()
    whole = plain.forward(raw, w, tokens)
    part = plain.forward(raw, w, tokens[:17])
    assert torch.allclose(whole[:17], part, atol=1e-10)


def test_plain_retention_equals_its_closed_form():
    """o_t = sum_{s<=t} decay^(t-s) (q_t . k_s) v_s."""
    torch.manual_seed(0)
    m = {"heads": 2, "dim": 6, "vdim": 5, "decay": [0.8, 0.95], "rot": {"dims": 4, "base": 100.0}}
    width, steps = 12, 9
    w = {"x.q": torch.randn(12, width, dtype=plain.F), "x.k": torch.randn(12, width, dtype=plain.F),
         "x.v": torch.randn(10, width, dtype=plain.F), "x.g": torch.randn(10, width, dtype=plain.F),
         "x.o": torch.eye(10, dtype=plain.F)}
    h = torch.randn(steps, width, dtype=plain.F)
    got = plain.retention(h, w, "x.", m, list(range(steps)), 1e-5)
    q = plain.rotate_half((h @ w["x.q"].T).view(steps, 2, 6), list(range(steps)), 4, 100.0)
    k = plain.rotate_half((h @ w["x.k"].T).view(steps, 2, 6), list(range(steps)), 4, 100.0) * 6 ** -0.5
    v = (h @ w["x.v"].T).view(steps, 2, 5)
    o = torch.zeros(steps, 2, 5, dtype=plain.F)
    for t in range(steps):
        for s in range(t + 1):
            for head in range(2):
                o[t, head] += m["decay"][head] ** (t - s) * (q[t, head] @ k[s, head]) * v[s, head]
    want = plain.unit_rms(o, 1e-5).reshape(steps, 10) * torch.nn.functional.silu(h @ w["x.g"].T)
    assert torch.allclose(got, want, atol=1e-10)


def test_plain_mlstm_equals_its_unstabilised_form_for_small_gates():
    """With gates of moderate size the running maximum only rescales: S = sum_s exp(F_t - F_s + i_s) k_s v_s^T with
    F the running sum of log forget gates, the denominator max(|n . q|, exp(-m)) scaled alike."""
    torch.manual_seed(1)
    m = {"heads": 1, "dim": 4, "vdim": 3, "gate_cap": 5.0}
    width, steps = 8, 7
    w = {"x." + n: torch.randn(s, dtype=plain.F) * 0.5 for n, s in
         (("q", (4, width)), ("k", (4, width)), ("v", (3, width)), ("g", (3, width)), ("i", (1, width)), ("f", (1, width)))}
    w.update({"x.i.b": torch.tensor([0.3], dtype=plain.F), "x.f.b": torch.tensor([1.0], dtype=plain.F),
              "x.norm": torch.ones(3, dtype=plain.F), "x.o": torch.eye(3, dtype=plain.F)})
    h = torch.randn(steps, width, dtype=plain.F)
    got = plain.mlstm(h, w, "x.", m, 1e-5)
    q, k, v = (h @ w["x.q"].T) * 4 ** -0.5, h @ w["x.k"].T, h @ w["x.v"].T
    li = plain.soft_capped(h @ w["x.i"].T + w["x.i.b"], 5.0)[:, 0]
    lf = plain.log_sigmoid(plain.soft_capped(h @ w["x.f"].T + w["x.f.b"], 5.0))[:, 0]
    out = torch.zeros(steps, 3, dtype=plain.F)
    top = torch.zeros((), dtype=plain.F)
    for t in range(steps):
        top = torch.maximum(lf[t] + top, li[t])
        S, n = torch.zeros(4, 3, dtype=plain.F), torch.zeros(4, dtype=plain.F)
        for s in range(t + 1):
            weight = torch.exp(lf[s + 1:t + 1].sum() + li[s])
            S += weight * torch.outer(k[s], v[s])
            n += weight * k[s]
        scale = torch.exp(-top)                     # what the stabilised state is multiplied by
        out[t] = (S.T @ q[t]) * scale / (torch.maximum((n @ q[t]).abs() * scale, torch.exp(-top)) + 1e-6)
    want = plain.unit_rms(out[:, None, :], 1e-5).reshape(steps, 3) * torch.sigmoid(h @ w["x.g"].T)
    assert torch.allclose(got, want, atol=1e-9)


def test_plain_delta_rule_overwrites_a_key_it_has_seen():
    """With beta = 1 and no decay, writing (k, v2) after (k, v1) leaves exactly v2 behind k: the rule's point."""
    S = torch.zeros(4, 3, dtype=plain.F)
    k = torch.tensor([0.5, 0.5, 0.5, 0.5], dtype=plain.F)
    for v in (torch.tensor([1.0, 2.0, 3.0], dtype=plain.F), torch.tensor([-4.0, 0.0, 9.0], dtype=plain.F)):
        S = S + torch.outer(k, 1.0 * (v - S.T @ k))
    assert torch.allclose(S.T @ k, torch.tensor([-4.0, 0.0, 9.0], dtype=plain.F))
