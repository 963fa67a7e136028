"""Zukinex on the GPU against the plain implementation: each mechanism alone, whole models of several sizes under
every way of cutting the work, pages and slots that are used again, keys planted far away and at the edges of
windows, long decoding, and generation through the scheduler."""
import json
import math
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

from tests import schedules
from tests import zukinex_util as zu
from tests.plain import zukinex_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F = torch.float64
# float32: sums of a few hundred float products: every position must keep the bound.  bfloat16: 8 significant bits
# wherever an activation is stored; beside that a rounded router input now and then gives a row another expert
# than the plain implementation chooses (two choice scores within the rounding of one another), which moves that
# position by an expert's whole output: so the median must keep the bound and at most one position in twelve may
# be beyond five times it.  A fault (a wrong key, a window off by one, a sink left out) moves most positions.
TOLERANCE = {"float32": 3e-5, "bfloat16": 3e-2}
LENGTHS = {"A": [1, 2, 37, 130, 64, 9], "B": [70, 3, 150, 33, 81], "C": [90, 17, 65, 2, 48]}


def widened(weights):
    return {k: v.float() if v.is_floating_point() else v for k, v in weights.items()}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    cache = {}

    def get(name, dtype_name):
        key = (name, dtype_name)
        if key not in cache:
            raw = zu.SMALL[name]
            weights = zu.make_weights(raw, 17 + len(cache), DTYPES[dtype_name], sharpen=2.5 if dtype_name == "float32" else 1.0)
            folder = zu.write_dir(str(tmp_path_factory.mktemp(f"zukinex_{name}_{dtype_name}")), raw, weights)
            gen = np.random.default_rng(5 + len(cache))
            requests = {f"r{i}": gen.integers(0, raw["vocab"], size=n).tolist() for i, n in enumerate(LENGTHS[name])}
            expected = {rid: plain.forward(raw, widened(weights), toks).numpy() for rid, toks in requests.items()}
            cache[key] = (folder, requests, expected)
        return cache[key]
    return get


def make_engine(folder, dtype_name, **options):
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model
    options.setdefault("page_tokens", 16)
    options.setdefault("max_requests", 4)
    return Engine(load_model(folder, dtype_name), **options)


def run_steps(engine, steps):
    from leone_amd.engine.engine import StepEntry
    outputs = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if out.logits is not None:
            outputs[s["step"]] = out.logits.float().cpu().numpy()
        for rid in s["end"]:
            engine.release(rid)
        engine.cache.check()
    return outputs


def compare(steps, outputs, expected, dtype_name, what):
    tol = TOLERANCE[dtype_name]
    got = schedules.collect(steps, outputs)
    assert set(got) == set(expected)
    errors = []
    for rid, rows in got.items():
        have, want = np.stack(rows), expected[rid]
        assert have.shape == want.shape and np.isfinite(have).all(), (what, rid, have.shape, want.shape)
        err = zu.relative_error(have, want)
        errors.append(err)
        if dtype_name == "float32":
            assert err.max() <= tol, (f"{what}: request {rid}, first position over the bound {int(np.argmax(err > tol))} of "
                                      f"{len(err)}, worst {int(err.argmax())}: {err.max():.3e}, bound {tol}")
    errors = np.concatenate(errors)
    if dtype_name != "float32":
        far = int((errors > 5 * tol).sum())
        assert np.median(errors) <= tol and far <= max(1, len(errors) // 12), (
            f"{what}: median {np.median(errors):.3e}, {far} of {len(errors)} positions beyond five times the bound {tol}")
    return float(errors.max())


SCHEDULES = {"whole": schedules.whole, "tail_decoded": lambda r: schedules.tail_decoded(r, 45),
             "portions": schedules.portions, "mixed": schedules.mixed}


@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(zu.SMALL))
def test_engine_agrees_with_plain_however_the_work_is_cut(cases, name, dtype_name, schedule):
    """Whole prompts, tails decoded token by token (windows of 5 to 40 pass over decoded tokens), portions down to
    two tokens, and four requests at a time with portions beside single tokens, on an engine with four slots and
    just enough pages of 16 tokens: pages are used again, also those a window has passed.  Logits at every position."""
    folder, requests, expected = cases(name, dtype_name)
    steps = SCHEDULES[schedule](requests)
    engine = make_engine(folder, dtype_name, max_tokens=schedules.max_live_tokens(steps, 16), poison_freed=True)
    outputs = run_steps(engine, steps)
    worst = compare(steps, outputs, expected, dtype_name, f"{name} {dtype_name} {schedule}")
    print(f"{name} {dtype_name} {schedule}: worst relative error {worst:.2e}")
    assert all(engine.cache.free_pages(g) == engine.cache.groups[g].num_pages for g in range(len(engine.cache.groups)))


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_pages_and_slots_that_held_another_request(cases, dtype_name):
    """One slot and pages enough for one request: every request runs where the one before it ran, and what freed
    pages hold is overwritten with NaN here, as a fault would leave it."""
    folder, requests, expected = cases("A", dtype_name)
    engine = make_engine(folder, dtype_name, max_tokens=144, max_requests=1)
    for rid, toks in requests.items():
        steps = schedules.portions({rid: toks}, sizes=(3, 1, 2, 40))
        outputs = run_steps(engine, steps)
        compare(steps, outputs, {rid: expected[rid]}, dtype_name, f"page reuse {rid}")
        for storage in engine.pools.paged.values():
            for pool in storage:
                pool.fill_(float("nan"))


def test_long_decoding_through_recorded_steps():
    """A short prompt, then 300 tokens one by one (steps replayed from a recording), two requests side by side:
    every window passes over decoded tokens many times, pages behind them are handed back and used again."""
    raw = zu.SMALL["B"]
    weights = zu.make_weights(raw, 91, torch.float32, sharpen=2.0)
    gen = np.random.default_rng(2)
    requests = {"a": gen.integers(0, raw["vocab"], size=310).tolist(), "b": gen.integers(0, raw["vocab"], size=305).tolist()}
    expected = {rid: plain.forward(raw, weights, toks).numpy() for rid, toks in requests.items()}
    with tempfile.TemporaryDirectory() as folder:
        zu.write_dir(folder, raw, weights)
        for graphs in (True, False):
            engine = make_engine(folder, "float32", max_tokens=256, graphs=graphs, poison_freed=True)
            steps = [{"step": 0, "entries": [{"id": "a", "tokens": requests["a"][:10], "want": list(range(10))},
                                             {"id": "b", "tokens": requests["b"][:5], "want": list(range(5))}], "end": []}]
            for i in range(300):
                steps.append({"step": i + 1, "entries": [{"id": "a", "tokens": [requests["a"][10 + i]], "want": [0]},
                                                         {"id": "b", "tokens": [requests["b"][5 + i]], "want": [0]}],
                              "end": ["a", "b"] if i == 299 else []})
            assert engine.graphs == graphs
            outputs = run_steps(engine, steps)
            compare(steps, outputs, expected, "float32", f"long decoding, graphs {graphs}")


def test_greedy_generation_through_the_scheduler():
    """The framework's own entry point: prompts in, greedy tokens out, scheduled in portions with more requests
    than slots, against the plain implementation's argmax token by token."""
    from leone_amd.api import Runtime
    from leone_amd.engine.scheduler import SchedulerPolicy
    raw = zu.SMALL["A"]
    weights = zu.make_weights(raw, 23, torch.float32, sharpen=2.0)
    gen = np.random.default_rng(8)
    prompts = [gen.integers(0, raw["vocab"], size=n).tolist() for n in (3, 40, 21, 9, 57)]
    with tempfile.TemporaryDirectory() as folder:
        zu.write_dir(folder, raw, weights)
        runtime = Runtime.load(folder, "float32", max_tokens=512, page_tokens=16, max_requests=2,
                               policy=SchedulerPolicy(max_live_requests=2, prefill_chunk_tokens=16, max_step_tokens=24))
        results = runtime.generate_tokens(prompts, 12, eos_token_id=None)
    for prompt, result in zip(prompts, results):
        tokens = list(prompt)
        for i in range(12):
            logits = plain.forward(raw, weights, tokens)[-1]
            best = int(logits.argmax())
            if result.tokens[i] != best:       # a near tie may fall either way; anything else is a fault
                assert float(logits[best] - logits[result.tokens[i]]) < 1e-4, (i, best, result.tokens[i])
            tokens.append(result.tokens[i])
        assert len(result.tokens) == 12


def test_trace_replay_as_a_user_runs_it(cases, tmp_path):
    folder, requests, expected = cases("B", "float32")
    steps = schedules.mixed(requests)
    out_dir = str(tmp_path / "out")
    process = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                                "--out", out_dir, "--max-tokens", str(schedules.max_live_tokens(steps, 64))],
                               stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    outputs = {}
    for s in steps:
        process.stdin.write(json.dumps(s) + "\n")
        process.stdin.flush()
        assert process.stdout.readline().strip() == f"done {s['step']}"
        wanted = sum(len(e["want"]) for e in s["entries"])
        if wanted:
            outputs[s["step"]] = np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4").reshape(wanted, -1)
    process.stdin.close()
    assert process.wait(timeout=60) == 0
    compare(steps, outputs, expected, "float32", "trace replay")


def test_command_line_generates_from_token_ids(tmp_path):
    """``leone generate`` on a Zukinex folder: greedy tokens as the plain implementation picks them; ``leone
    random-model`` writes a folder of the design that loads again."""
    from leone_amd import cli
    raw = zu.SMALL["B"]
    weights = zu.make_weights(raw, 61, torch.float32, sharpen=2.0)
    folder = zu.write_dir(str(tmp_path / "model"), raw, weights)
    prompt = [5, 17, 3, 99, 42, 7]
    out = str(tmp_path / "tokens.json")
    assert cli.main(["generate", "-m", folder, "--prompt-tokens", ",".join(map(str, prompt)), "-n", "8", "--dtype", "float32",
                     "--ignore-eos", "--debug-tokens", out]) == 0
    with open(out) as handle:
        got = json.load(handle)
    tokens = list(prompt)
    for token in got:
        logits = plain.forward(raw, weights, tokens)[-1]
        assert token == int(logits.argmax()) or float(logits.max() - logits[token]) < 1e-4
        tokens.append(token)
    assert len(got) == 8
    config_path = str(tmp_path / "config.json")
    with open(config_path, "w") as handle:
        json.dump(zu.SMALL["A"], handle)
    made = str(tmp_path / "made")
    assert cli.main(["random-model", "--config", config_path, "--seed", "3", "--out", made]) == 0
    engine = make_engine(made, "bfloat16", max_tokens=64)
    from leone_amd.engine.engine import StepEntry
    logits = engine.step([StepEntry("a", [1, 2, 3], [2])]).logits
    assert logits.shape == (1, zu.SMALL["A"]["vocab"]) and torch.isfinite(logits).all()


def test_which_attention_kernels_a_layer_gets(cases):
    """Keys and values of one size that the matrix-core kernels take go to them in bfloat16, kept first keys and the
    gate for every element included; values of another size, and float32, go to the row kernel."""
    folder, _, _ = cases("C", "bfloat16")
    engine = make_engine(folder, "bfloat16", max_tokens=256)
    owner, reader = engine.model.layers[0].mixer, engine.model.layers[1].mixer
    assert owner.keep_first == 4 and reader.keep_first == 2 and reader.shared_kv and owner.gate_each
    assert owner.attention_kernels(torch.bfloat16, 16, 16) == {"decode": "split_kv", "prompt": "flash"}
    assert reader.attention_kernels(torch.bfloat16, 16, 16) == {"decode": "split_kv", "prompt": "flash"}
    assert owner.attention_kernels(torch.float32, 16, 16) == {"decode": "rows", "prompt": "rows"}
    folder, _, _ = cases("A", "bfloat16")
    other = make_engine(folder, "bfloat16", max_tokens=256).model.layers[0].mixer
    assert other.value_dim != other.head_dim
    assert other.attention_kernels(torch.bfloat16, 16, 16) == {"decode": "rows", "prompt": "rows"}


# ---- each mechanism alone ---------------------------------------------------------------------------------------

def close(have, want, tol, what):
    have, want = have.double().cpu(), want.double().cpu()
    scale = float(want.abs().max()) + 1e-30
    worst = float((have - want).abs().max()) / scale
    assert worst <= tol, f"{what}: off by {worst:.3e} of the largest value, bound {tol}"


@pytest.mark.parametrize("hidden", [40, 90, 192, 1000])
def test_norm_behind_a_sublayer(hidden):
    """The norm of a sublayer's result, the sum into the stream and what the next product reads, in one kernel; at the
    model's end with the final norm on picked rows."""
    from leone_amd import ops
    gen = torch.Generator().manual_seed(hidden)
    rows, eps = 9, 1e-5
    x = torch.randn(rows, hidden, generator=gen)
    planes = torch.randn(3, rows, hidden, generator=gen)
    gain, gain2 = 1 + 0.3 * torch.randn(hidden, generator=gen), 1 + 0.3 * torch.randn(hidden, generator=gen)
    want = x.double() + plain.rms_norm(planes.double().sum(0), gain.double(), eps)
    stream = x.to(DEV)
    out = ops.add_normed(stream, planes[0].to(DEV) + planes[1].to(DEV) + planes[2].to(DEV), gain.to(DEV), eps, out_dtype=torch.bfloat16)
    close(stream, want, 2e-6, "stream")
    close(out.float(), want, 5e-3, "rows as the product reads them")
    stream = x.to(DEV)
    same = ops.add_normed(stream, planes.to(DEV), gain.to(DEV), eps, out_dtype=torch.float32)
    assert same is stream
    close(stream, want, 2e-6, "stream from planes")
    stream = x.to(DEV)
    picked = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    normed = ops.add_normed(stream, planes.to(DEV), gain.to(DEV), eps, then=(gain2.to(DEV), 1e-6, torch.float32), rows=picked)
    close(normed, plain.rms_norm(want, gain2.double(), 1e-6)[[7, 0, 3]], 3e-6, "final norm of picked rows")
    assert torch.equal(stream.cpu(), x), "with picked rows the stream is left alone"
    plainly = ops.add_normed(stream, None, None, 0.0, out_dtype=torch.bfloat16)
    assert torch.equal(plainly.cpu(), x.to(torch.bfloat16))


def test_embedding_with_a_learned_position_table():
    from leone_amd import ops
    gen = torch.Generator().manual_seed(4)
    for dtype in (torch.float32, torch.bfloat16):
        table = torch.randn(50, 72, generator=gen).to(dtype)
        places = torch.randn(30, 72, generator=gen).to(dtype)
        tokens = torch.tensor([3, 49, 0, 3, 17], dtype=torch.int32)
        positions = torch.tensor([0, 29, 5, 6, 6], dtype=torch.int32)
        out = ops.embed(table.to(DEV), tokens.to(DEV), position_table=places.to(DEV), positions=positions.to(DEV))
        close(out, table.double()[tokens.long()] + places.double()[positions.long()], 1e-6, f"embed {dtype}")


@pytest.mark.parametrize("rows", [3, 40, 200])
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_feed_forward_with_either_activation(rows, activation, dtype):
    """Few rows (the products with the activation folded in), some more (the multi-row products) and many (the
    library's products with the activation kernel)."""
    from leone_amd.parts import FEED_FORWARDS, PartSpec
    gen = torch.Generator().manual_seed(rows)
    width, ff = 64, 100
    w = {"gate": torch.randn(ff, width, generator=gen) / 8, "up": torch.randn(ff, width, generator=gen) / 8,
         "down": torch.randn(width, ff, generator=gen) / 10}
    w = {k: v.to(dtype) for k, v in w.items()}
    part = FEED_FORWARDS.build(PartSpec("swiglu", {"hidden": width, "intermediate": ff, "activation": activation,
                                                   "float_output": True, "gate": "gate", "up": "up", "down": "down"}))
    part.bind({k: v.to(DEV) for k, v in w.items()})
    h = (2 * torch.randn(rows, width, generator=gen)).to(dtype)
    out = part.forward(h.to(DEV), None)
    assert out.dtype == torch.float32
    act = plain.silu if activation == "silu" else plain.gelu_tanh
    close(out, plain.glu(h.double(), {k: v.double() for k, v in w.items()}, "", act), 2e-6 if dtype == torch.float32 else 2e-2,
          f"{activation} {rows} rows")


ROUTERS = [{"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}},
           {"experts": 5, "identity": 0, "top": 1},
           {"experts": 9, "identity": 1, "top": 4, "groups": {"count": 5, "keep": 3}},
           {"experts": 60, "identity": 12, "top": 6, "groups": {"count": 8, "keep": 3}},
           {"experts": 140, "identity": 10, "top": 8, "groups": {"count": 10, "keep": 4}},
           {"experts": 70, "identity": 3, "top": 2, "groups": {"count": 73, "keep": 22}},
           {"experts": 200, "identity": 0, "top": 5, "groups": {"count": 100, "keep": 30}},
           {"experts": 4, "identity": 0, "top": 4, "groups": {"count": 1, "keep": 1}}]


@pytest.mark.parametrize("r", ROUTERS, ids=lambda r: f"{r['experts']}+{r['identity']}")
def test_router_choice_and_weights(r):
    """Scores, corrections of both signs (all choice scores negative in some rows), groups, the best few: the same
    outputs in the same order as the plain router, and its weights."""
    from leone_amd import ops
    total = r["experts"] + r["identity"]
    gen = torch.Generator().manual_seed(total)
    logits = 2 * torch.randn(150, total, generator=gen)
    correction = 0.2 * torch.randn(total, generator=gen)
    correction[::2] -= 1.5                                   # far below any score: shut groups must not count as 0
    chosen, weight = ops.route_topk(logits.to(DEV), correction.to(DEV), r["top"], (r.get("groups") or {}).get("count", 1),
                                    (r.get("groups") or {}).get("keep", 1))
    want_chosen, want_weight = plain.route(logits.double(), torch.eye(total, dtype=F), correction.double(), r)
    assert torch.equal(chosen.cpu().long(), want_chosen), "the chosen outputs differ"
    close(weight, want_weight, 1e-5, "weights")
    close(weight.sum(dim=1), torch.ones(150), 1e-5, "weights add up to one")


@pytest.mark.parametrize("rows", [1, 7, 300])
@pytest.mark.parametrize("sizes", [(64, 24, 6, 2, 3), (40, 20, 3, 0, 2), (96, 8, 9, 5, 4)], ids=str)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_experts(rows, sizes, dtype):
    """Rows sorted by expert on the device, the experts' products, identity experts, a shared result added; inner
    sizes that are no multiples of 8; one row and many."""
    from leone_amd import ops
    width, ff, experts, identity, top = sizes
    gen = torch.Generator().manual_seed(rows + width)
    w = {}
    for e in range(experts):
        w[f"e{e}.gate"] = (torch.randn(ff, width, generator=gen) / math.sqrt(width)).to(dtype)
        w[f"e{e}.up"] = (torch.randn(ff, width, generator=gen) / math.sqrt(width)).to(dtype)
        w[f"e{e}.down"] = (torch.randn(width, ff, generator=gen) / math.sqrt(ff)).to(dtype)
    h = torch.randn(rows, width, generator=gen).to(dtype)
    chosen = torch.stack([torch.randperm(experts + identity, generator=gen)[:top] for _ in range(rows)]).to(torch.int32)
    weight = torch.rand(rows, top, generator=gen)
    extra = torch.randn(rows, width, generator=gen)
    gate_up = torch.stack([torch.stack([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(experts)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(experts)]).to(DEV)
    out = ops.routed_experts(h.to(DEV), chosen.to(DEV), weight.to(DEV), gate_up, down, "silu", extra=extra.to(DEV))
    want = extra.double()
    wide = {k: v.double() for k, v in w.items()}
    for t in range(rows):
        for e, a in zip(chosen[t].tolist(), weight[t].double()):
            want[t] += a * (h[t].double() if e >= experts else plain.glu(h[t:t + 1].double(), wide, f"e{e}.", plain.silu)[0])
    close(out, want, 3e-6 if dtype == torch.float32 else 2e-2, f"{sizes} {rows} rows")


@pytest.mark.parametrize("rows", [1, 9, 64, 65, 300])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixture_part_against_plain(rows, dtype):
    """The whole feed-forward part: router product, choice, tiles (in one launch up to 64 rows), experts, identity
    experts and the shared expert, against the plain mixture; in bfloat16 rows whose choice is a close call are left
    out of the comparison (the plain router sees the unrounded product)."""
    from leone_amd.parts import FEED_FORWARDS, PartSpec
    width = 64
    mlp = zu.moe(6, 3, 24, identity=2, groups=(4, 2), shared=40)
    raw = zu.config(width, 50, [zu.layer(zu.attention(2, 1, 8, 8), mlp)])
    weights = {k[len("l0.mlp."):]: v for k, v in zu.make_weights(raw, 12, dtype).items() if k.startswith("l0.mlp.")}
    shared = PartSpec("swiglu", {"hidden": width, "intermediate": 40, "float_output": True, "gate": "shared.gate",
                                 "up": "shared.up", "down": "shared.down"})
    part = FEED_FORWARDS.build(PartSpec("routed_glu", {"hidden": width, "experts": 6, "identity": 2, "top": 3, "group_count": 4,
                                                       "group_keep": 2, "intermediate": 24, "router": "router",
                                                       "correction": "correction", "expert": "e{e}", "shared": shared}))
    part.bind({k: v.to(DEV) for k, v in weights.items()})
    h = torch.randn(rows, width, generator=torch.Generator().manual_seed(rows)).to(dtype)
    out = part.forward(h.to(DEV), None)
    wide = {k: v.double() for k, v in weights.items()}
    want = plain.mixture(h.double(), mlp, wide, "")
    keep = torch.ones(rows, dtype=torch.bool)
    if dtype == torch.bfloat16:
        s = torch.softmax(h.double() @ wide["router"].T, dim=-1) + wide["correction"]
        ranked = s.sort(dim=-1, descending=True).values
        keep = (ranked[:, :-1] - ranked[:, 1:]).min(dim=-1).values > 2e-3      # no two choice scores close to each other
        assert keep.sum() >= rows // 2
    close(out.cpu()[keep], want[keep], 3e-6 if dtype == torch.float32 else 2e-2, f"mixture of {rows} rows")


def planted(n, heads, dim, vdim, seed):
    """Keys and values of one request of ``n`` positions: random keys of one length, so that a query along one key
    stands out against all others."""
    gen = torch.Generator().manual_seed(seed)
    k = torch.randn(n, heads, dim, generator=gen)
    k = k / k.norm(dim=-1, keepdim=True)
    v = torch.randn(n, heads, vdim, generator=gen)
    return k, v


def paged(k, v, page_tokens, dtype, seed):
    """The cache of one request over scattered pages, the rest filled with NaN."""
    from leone_amd import ops
    n, heads, dim = k.shape
    blocks = -(-n // page_tokens)
    pages = 2 * blocks + 3
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(seed))[:blocks]
    k_pool = torch.full((pages, heads, dim // 8, page_tokens, 8), float("nan"), dtype=dtype)
    v_pool = torch.full((pages, heads, page_tokens // 8, v.shape[2], 8), float("nan"), dtype=dtype)
    for b in range(blocks):
        # what lies beyond the request's end is not the request's
        kp = torch.full((page_tokens, heads, dim), float("nan"))
        vp = torch.full((page_tokens, heads, v.shape[2]), float("nan"))
        rows = min(page_tokens, n - b * page_tokens)
        kp[:rows], vp[:rows] = k[b * page_tokens:b * page_tokens + rows], v[b * page_tokens:b * page_tokens + rows]
        packed_k, packed_v = ops.pack_keys(kp.transpose(0, 1)).to(dtype), ops.pack_values(vp.transpose(0, 1)).to(dtype)
        k_pool[order[b]], v_pool[order[b]] = packed_k, packed_v
    return k_pool.to(DEV), v_pool.to(DEV), order.to(torch.int32).view(1, -1).to(DEV)


def attend_plainly(q, k, v, positions, scale, window, keep_first, group):
    n = k.shape[0]
    see = plain.visible(n, window or None, keep_first)
    out = torch.zeros(len(positions), q.shape[1], v.shape[2], dtype=F)
    for r, p in enumerate(positions):
        for head in range(q.shape[1]):
            score = (k[:, head // group].double() @ q[r, head].double()) * scale
            score = score.masked_fill(~see[p], float("-inf"))
            out[r, head] = torch.softmax(score, dim=0) @ v[:, head // group].double()
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,keep_first", [(40, 5), (16, 1), (33, 0), (0, 0), (7, 20)])
def test_planted_keys_far_away_and_at_every_edge(dtype, window, keep_first):
    """Queries made so that one key stands out: the key just inside and just outside the window, the last kept first
    key and the first one that is not kept, the very first key, a key hundreds of positions back, keys on both sides
    of a page border; as the rows of one long portion and as single rows.  A wrong edge flips which key wins."""
    from leone_amd import ops
    n, heads, q_heads, dim, vdim, page_tokens = 300, 2, 4, 16, 24, 16
    k, v = planted(n, heads, dim, vdim, 3 + window)
    kd, vd = k.to(dtype).float(), v.to(dtype).float()
    k_pool, v_pool, table = paged(k, v, page_tokens, dtype, 7)
    targets = []
    for i in (299, 200, 64, 63, 47, 48, 21, 6, 0):
        edge = [i, i - 1, 0, keep_first - 1, keep_first, 15, 16, 17]
        if window:
            edge += [i - window, i - window + 1, i - window - 1]
        targets += [(i, j) for j in edge if 0 <= j <= i]
    positions = [i for i, _ in targets]
    q = torch.zeros(len(targets), q_heads, dim)
    for r, (i, j) in enumerate(targets):
        for head in range(q_heads):
            key = kd[j, head // 2]
            q[r, head] = key / (key @ key) * 60.0        # a score of 60 for key j, 60 times a cosine for any other
    want = attend_plainly(q.to(dtype).float(), kd, vd, positions, 1.0, window, keep_first, 2)
    flat_q = q.reshape(len(targets), -1).to(dtype).to(DEV)
    rows_at = torch.tensor(positions, dtype=torch.int32, device=DEV)
    entry = torch.zeros(len(targets), dtype=torch.int32, device=DEV)
    out = ops.attention_rows(flat_q, k_pool, v_pool, rows_at, entry, table, q_heads, 1.0, window, keep_first=keep_first)
    close(out.float().view(len(targets), q_heads, vdim), want, 2e-5 if dtype == torch.float32 else 1.5e-2, "rows side by side")
    for r in (0, 5, len(targets) - 1):
        one = ops.attention_rows(flat_q[r:r + 1], k_pool, v_pool, rows_at[r:r + 1], entry[:1], table, q_heads, 1.0, window,
                                 keep_first=keep_first)
        assert torch.equal(one[0], out[r]), "a row alone and the same row beside others"
    # what the planted key decides: its value comes out if the key is in sight, something else if not
    see = plain.visible(n, window or None, keep_first)
    for r, (i, j) in enumerate(targets):
        hit = float((out[r].float().cpu().view(q_heads, vdim)[0] - vd[j, 0]).abs().max())
        assert (hit < 0.25) == bool(see[i, j]), f"position {i}, key {j}: in sight {bool(see[i, j])}, distance {hit:.3f}"


@pytest.mark.parametrize("page_tokens", [16, 64])
@pytest.mark.parametrize("window,keep_first", [(40, 5), (64, 3), (100, 70), (33, 0), (0, 0), (7, 20), (150, 40), (130, 129)])
def test_matrix_core_attention_with_kept_first_keys(window, keep_first, page_tokens):
    """The prompt kernel (a portion of 420 rows that continues a request of 100) and the split-KV kernel (the same
    rows one by one, and cut into several parts) with planted keys: for every row a key at one of the edges (just
    inside and outside the window, the last kept key and the first that is not, the first key, the row's own, one
    far back).  Kept keys lie in tiles and stages of their own, before the window's; with 70 and 129 of them they
    take several."""
    from leone_amd import ops
    n, first, heads, q_heads, dim = 520, 100, 2, 4, 32
    k, v = planted(n, heads, dim, dim, 11 + window)
    kd, vd = k.bfloat16().float(), v.bfloat16().float()
    k_pool, v_pool, table = paged(k, v, page_tokens, torch.bfloat16, 9)
    positions = list(range(first, n))
    q = torch.zeros(len(positions), q_heads, dim)
    targets = []
    for r, i in enumerate(positions):
        kinds = [i, i - 1, 0, keep_first - 1, keep_first, i // 2, i - window, i - window + 1, i - window - 1, 63, 64]
        j = kinds[r % len(kinds)] if window else kinds[r % 6]
        j = min(max(j, 0), i)
        targets.append(j)
        for head in range(q_heads):
            key = kd[j, head // 2]
            q[r, head] = key / (key @ key) * 60.0
    want = attend_plainly(q.bfloat16().float(), kd, vd, positions, 1.0, window, keep_first, 2)
    flat_q = q.reshape(len(positions), -1).bfloat16().to(DEV)
    rows_at = torch.tensor(positions, dtype=torch.int32, device=DEV)
    entry = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
    out = torch.full_like(flat_q, float("nan"))
    tiles = ops.prefill_tiles([(0, 0, len(positions))]).to(DEV)
    ops.attention_prefill(flat_q, out, k_pool, v_pool, rows_at, tiles, table, q_heads, 1.0, window, mean_keys=300,
                          keep_first=keep_first)
    close(out.float().view(len(positions), q_heads, dim), want, 1.5e-2, "prompt kernel")
    for splits in (None, 1, 3):
        one = ops.attention_decode(flat_q, k_pool, v_pool, rows_at, entry, table, q_heads, 1.0, window, max_context=n,
                                   splits=splits, keep_first=keep_first)
        close(one.float().view(len(positions), q_heads, dim), want, 1.5e-2, f"split-KV kernel, splits {splits}")
    see = plain.visible(n, window or None, keep_first)
    for r, (i, j) in enumerate(zip(positions, targets)):
        hit = float((out[r].float().cpu().view(q_heads, dim)[0] - vd[j, 0]).abs().max())
        assert (hit < 0.25) == bool(see[i, j]), f"position {i}, key {j}: in sight {bool(see[i, j])}, distance {hit:.3f}"


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_attention_layers_alone_with_a_reader_of_the_owners_keys(dtype_name):
    """Two attention parts on one cache slot, the owner of the keys and a reader with a wider mask, fed two
    sequences in cuts (portions beside single rows, a sequence sitting a step out, interleaved pages); each against
    the plain mixer, which for the reader takes the owner's keys and values."""
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.parts.base import BLOCKS, POSITIONS
    from leone_amd.parts.context import StepContext
    dtype = DTYPES[dtype_name]
    raw = zu.config(48, 60, [zu.layer(zu.attention(4, 2, 16, 8, rot=(12, 300.0), mask=(9, 2))),
                             zu.layer(zu.attention(4, 2, 16, 8, rot=(12, 300.0), mask=(21, 4), kv_from=0))], max_positions=128)
    weights = zu.make_weights(raw, 5, dtype, sharpen=2.0)
    spec = model_spec_for(config_from_dict(raw))
    positions = {name: POSITIONS.build(s) for name, s in spec.positions.items()}
    for part in positions.values():
        part.prepare(128, DEV)
    blocks = [BLOCKS.build(s, positions=positions) for s in spec.layers]
    on_device = {k: v.to(DEV) for k, v in weights.items()}
    for block in blocks:
        block.bind(dict(on_device))
    owner, reader = blocks[0].mixer, blocks[1].mixer
    need = owner.cache_need()
    assert need == reader.cache_need() and need.window == 21 and need.keep_first == 4
    storage = need.allocate(24, 16, dtype, DEV)
    for pool in storage:
        pool.fill_(float("nan"))
    gen = torch.Generator().manual_seed(1)
    hs = [torch.randn(63, 48, generator=gen).to(dtype), torch.randn(66, 48, generator=gen).to(dtype)]
    pages = {0: list(range(1, 24, 2)), 1: list(range(0, 24, 2))}
    cuts = [(5, 1), (1, 1), (2, 0), (1, 3), (17, 1), (1, 16), (0, 2), (33, 1), (1, 1), (2, 40)]
    at, outs = [0, 0], {"owner": [[], []], "reader": [[], []]}
    for cut in cuts:
        present = [s for s in (0, 1) if cut[s]]
        meta, rows = [], []
        for e, s in enumerate(present):
            meta += [(e, at[s] + i) for i in range(cut[s])]
            rows.append(hs[s][at[s]:at[s] + cut[s]])
        table = torch.tensor([pages[s] for s in present], dtype=torch.int32, device=DEV)
        step = StepContext(rows=len(meta), dtype=dtype, device=torch.device(DEV),
                           positions=torch.tensor([p for _, p in meta], dtype=torch.int32, device=DEV),
                           row_entry=torch.tensor([e for e, _ in meta], dtype=torch.int32, device=DEV), entries=[],
                           entry_slots=torch.zeros(len(present), dtype=torch.int32, device=DEV), want_rows=None,
                           block_tables={0: table}, max_position=max(p for _, p in meta))
        h = torch.cat(rows).to(DEV)
        view = need.view(storage, table, 16)
        results = {"owner": owner.forward(h, step, view),
                   "reader": reader.forward(h, step, type(view)(**{**view.__dict__, "writes": False}))}
        for who, result in results.items():
            first = 0
            for s in present:
                outs[who][s].append(result[first:first + cut[s]].float().cpu())
                first += cut[s]
        for s in present:
            at[s] += cut[s]
    wide = {k: v.double() for k, v in weights.items()}
    tol = 2e-5 if dtype_name == "float32" else 3e-2
    for s in (0, 1):
        h, n = hs[s].double(), hs[s].shape[0]
        kv = plain.keys_and_values(h, raw["layers"][0]["mixer"], wide, "l0.mix.", 1e-5, list(range(n)))
        close(torch.cat(outs["owner"][s]), plain.attention(h, raw["layers"][0]["mixer"], wide, "l0.mix.", 1e-5, list(range(n)), kv),
              tol, f"owner, sequence {s}")
        close(torch.cat(outs["reader"][s]), plain.attention(h, raw["layers"][1]["mixer"], wide, "l1.mix.", 1e-5, list(range(n)), kv),
              tol, f"reader, sequence {s}")
