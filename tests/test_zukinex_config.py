"""Zukinex on the CPU: the configuration reader, what the builder makes of it, the cache manager's kept first
positions, and the plain implementation against itself."""
import copy

import pytest
import torch

from leone_amd.architectures import config_from_dict, model_spec_for
from leone_amd.cache.manager import CacheManager, GroupSpec
from leone_amd.config.base import ConfigError
from leone_amd.config.zukinex import DenseConfig, MoeConfig, ZukinexConfig
from leone_amd.engine.trace_check import PoolFigures
from leone_amd.parts.model import DecoderModel
from tests import zukinex_util as zu
from tests.plain import zukinex_plain as plain


@pytest.mark.parametrize("name", list(zu.SMALL))
def test_configuration_reads_back(name):
    raw = zu.SMALL[name]
    config = config_from_dict(raw)
    assert isinstance(config, ZukinexConfig) and len(config.layers) == len(raw["layers"])
    again = config.to_dict()
    for mine, theirs in zip(again["layers"], raw["layers"]):
        assert mine["mixer"] == theirs["mixer"]
        if theirs["mlp"] is None or theirs["mlp"]["kind"] == "dense":
            assert mine["mlp"] == theirs["mlp"]
        else:
            assert mine["mlp"]["router"]["experts"] == theirs["mlp"]["router"]["experts"]
            assert mine["mlp"].get("shared") == theirs["mlp"].get("shared")
    assert config_from_dict(again) == config


def test_what_config_json_leaves_out():
    raw = zu.config(32, 50, [zu.layer(zu.attention(2, 1, 8, 8), zu.moe(3, 2, 8))])
    config = config_from_dict(raw)
    mixer, mlp = config.layers[0].mixer, config.layers[0].mlp
    assert mixer.rot_dims == 0 and mixer.window is None and mixer.keep_first == 0 and mixer.kv_from is None
    assert isinstance(mlp, MoeConfig) and (mlp.identity, mlp.group_count, mlp.group_keep, mlp.shared_ff) == (0, 1, 1, None)
    assert isinstance(config_from_dict(zu.SMALL["A"]).layers[1].mlp, DenseConfig)


@pytest.mark.parametrize("change,field", [
    (lambda r: r.pop("vocab"), "vocab"),
    (lambda r: r.pop("max_positions"), "max_positions"),
    (lambda r: r["norm"].update(eps=0.0), "eps"),
    (lambda r: r["layers"][0].update(type="conv"), "layers[0].type"),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), "layers[0].mixer.kv_heads"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=9), "layers[0].mixer.rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "layers[0].mixer.mask.size"),
    (lambda r: r["layers"][1]["mixer"].update(kv_from=1), "layers[1].mixer.kv_from"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=1), "layers[3].mixer.kv_from"),
    (lambda r: r["layers"][1]["mixer"].update(dim=32), "layers[1].mixer.kv_from"),
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=9), "layers[0].mlp.router.top"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=3), "layers[0].mlp.router.groups"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(keep=1), "layers[0].mlp.router.groups"),
    (lambda r: r["layers"][1]["mlp"].update(kind="sparse"), "layers[1].mlp.kind"),
    (lambda r: r["layers"][0]["mlp"]["expert"].pop("ff"), "layers[0].mlp.ff"),
])
def test_errors_name_the_key(change, field):
    raw = copy.deepcopy(zu.SMALL["A"])
    change(raw)
    with pytest.raises(ConfigError) as caught:
        config_from_dict(raw)
    assert caught.value.field == field, caught.value.field


@pytest.mark.parametrize("name", list(zu.SMALL))
def test_the_model_asks_for_exactly_the_designs_tensors(name):
    raw = zu.SMALL[name]
    model = DecoderModel(model_spec_for(config_from_dict(raw)), torch.float32, "cpu")
    asked = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert asked == zu.tensor_shapes(raw)


def test_a_reader_of_another_layers_keys_runs_on_its_slot_and_widens_what_it_keeps():
    config = config_from_dict(zu.SMALL["A"])
    spec = model_spec_for(config)
    assert [(run.layer, run.cache, run.writes) for run in spec.schedule] == [(0, 0, True), (1, 0, False), (2, 2, True), (3, 2, False)]
    assert config.kv_retention(0) == (33, 5)          # the reader's mask is wider than the owner's
    assert config.kv_retention(2) == (None, 0)        # the owner sees everything, whatever the reader's window
    model = DecoderModel(spec, torch.float32, "cpu")
    needs = model.cache_needs()
    assert needs[0].window == 33 and needs[0].keep_first == 5 and needs[2].window is None
    owner, reader = model.layers[0].mixer, model.layers[1].mixer
    assert (owner.window, owner.keep_first, reader.window, reader.keep_first) == (20, 3, 33, 5)
    assert reader.shared_kv and not owner.shared_kv


def test_a_window_that_passes_leaves_the_kept_first_pages():
    cache = CacheManager([GroupSpec(12, 4, window=6, keep_first=5), GroupSpec(12, 4, window=6)], max_requests=3, max_context=48)
    cache.admit("a")
    for tokens in (3, 7, 9, 1, 1, 10):
        cache.reserve("a", tokens)
        cache.commit("a", tokens)
        cache.check()
    # 31 positions: the next row reads keys from 26 on, pages 0..5 lie behind; two pages hold the first five positions
    assert [page >= 0 for page in cache.table("a", 0)] == [True, True, False, False, False, False, True, True]
    assert [page >= 0 for page in cache.table("a", 1)] == [False] * 6 + [True, True]
    assert cache.free_pages(0) == 8 and cache.free_pages(1) == 10
    # a request that takes over another's 24 positions shares the kept first pages and the window's, nothing between
    cache.admit("c")
    cache.reserve("c", 24)
    cache.commit("c", 24)
    assert cache.fork("c", "d", 24) == 24
    mine, theirs = cache.table("c", 0), cache.table("d", 0)
    assert mine[2] == mine[3] == -1 and theirs == [mine[0], mine[1], -1, -1, mine[4], mine[5]]
    assert cache.holders(0, mine[0]) == 2 and cache.holders(0, mine[5]) == 2
    cache.check()
    cache.release("c")
    cache.check()
    cache.release("d")
    assert cache.free_pages(0) == 8
    cache.release("a")
    assert cache.free_pages(0) == 12
    cache.check()
    pools = PoolFigures(12, 4, 6, 5)
    assert pools.pages_for(31, 31) == 4 and PoolFigures(12, 4, 6).pages_for(31, 31) == 2 and pools.pages_for(0, 3) == 1


def test_what_a_position_sees():
    see = plain.visible(12, 4, 2)
    assert see[11].tolist() == [True, True] + [False] * 6 + [True] * 4
    assert see[3].tolist() == [True] * 4 + [False] * 8                       # the window still covers the first keys
    assert see[5].tolist() == [True, True, True, True, True, True] + [False] * 6   # 0, 1 kept; 2..5 in the window
    assert see[6].tolist() == [True, True, False, True, True, True, True] + [False] * 5
    assert plain.visible(5, None, 0).tolist() == torch.ones(5, 5).tril().bool().tolist()


def test_the_router_of_the_plain_implementation():
    r = {"experts": 4, "identity": 2, "top": 2, "groups": {"count": 3, "keep": 2}}
    logits = torch.log(torch.tensor([[0.05, 0.10, 0.30, 0.05, 0.20, 0.30]], dtype=torch.float64))
    router = torch.eye(6, dtype=torch.float64)
    # without a correction groups (0,1) (2,3) (4,5) score .10 .30 .30: the first is shut; 2 and 5 win
    chosen, weight = plain.route(logits, router, torch.zeros(6, dtype=torch.float64), r)
    assert sorted(chosen[0].tolist()) == [2, 5] and torch.allclose(weight.sum(), torch.tensor(1.0, dtype=torch.float64))
    # a correction opens the first group and shuts the second; the weights are the scores without it
    correction = torch.tensor([0.0, 0.5, -0.4, -0.4, 0.0, 0.0], dtype=torch.float64)
    chosen, weight = plain.route(logits, router, correction, r)
    assert chosen[0].tolist() == [1, 5]
    assert torch.allclose(weight[0], torch.tensor([0.25, 0.75], dtype=torch.float64))
    # negative choice scores everywhere: a shut group must not win by counting as 0
    chosen, _ = plain.route(logits, router, torch.full((6,), -1.0, dtype=torch.float64), r)
    assert sorted(chosen[0].tolist()) == [2, 5]


def test_plain_forward_is_causal_and_cut_free():
    raw = zu.SMALL["A"]
    weights = zu.make_weights(raw, 3, torch.float32)
    tokens = torch.randint(0, raw["vocab"], (60,), generator=torch.Generator().manual_seed(1)).tolist()
    whole = plain.forward(raw, weights, tokens)
    part = plain.forward(raw, weights, tokens[:41])
    assert torch.allclose(whole[:41], part, atol=1e-9)
