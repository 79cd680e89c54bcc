"""Zederax through the framework's step function, cache manager and parts on the CPU with the emulated kernels, against
the plain implementation: what differs here is a fault of the host logic (tables, pages, the order of the parts, what
layers hand each other within a step), not of a kernel."""
import json
import os

import pytest
import torch

import plain_zederax as Z
import traces as TR
from emulated_kernels import EmulatedKernels
from levanter_amd.config import ConfigError, InferenceEngineConfig, LmConfig, ZederaxConfig
from levanter_amd.engine import ModelRunner, StepEntry
from levanter_amd.engine.loading import load_model, make_cache
from levanter_amd.parts import BuildEnv
from levanter_amd.weights import WeightsError
from zederax_configs import ZED


def build(name, tmp, dtype=torch.float32):
    raw, seed = ZED[name]
    W = Z.random_weights(raw, seed)
    d = Z.write_folder(raw, W, os.path.join(str(tmp), name), torch.float32)
    env = BuildEnv(dtype, torch.device("cpu"), EmulatedKernels())
    config, model = load_model(d, env)
    return raw, W, model, env, config


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def setup(request, tmp_path_factory):
    raw, W, model, env, _ = build(request.param, tmp_path_factory.mktemp("zed"))
    lengths = {"A": [70, 45, 100, 37, 64, 33], "B": [90, 130, 41, 17, 64], "C": [40, 12, 30], "D": [66, 21, 80, 5]}[request.param]
    reqs = TR.random_requests(raw["vocab"], lengths, 5)
    plain = {rid: Z.plain_logits(W, raw, torch.tensor(t)) for rid, t in reqs.items()}
    return raw, W, model, env, reqs, plain


def replay(model, env, steps, max_tokens, ps=16, max_seqs=4):
    cfg = InferenceEngineConfig(max_pages=max(1, max_tokens // ps), max_seqs=max_seqs, page_size=ps, max_pages_per_seq=16, compute_dtype="float32")
    cache = make_cache(model, cfg)
    runner = ModelRunner(model, cache, env)
    live, out = {}, {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in live:
                live[e["id"]] = cache.open(e["id"])
            entries.append(StepEntry(live[e["id"]], e["tokens"], e["want"]))
        logits = runner.step(entries)
        cache.check_invariants()
        if logits.shape[0]:
            out[s["step"]] = logits
        for rid in s["end"]:
            cache.close(live.pop(rid))
    cache.check_invariants()
    assert all(g.pool.n_free == g.pool.n_pages for g in cache.groups)
    return out, cache


@pytest.mark.parametrize("mode", ["whole", "singles", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(setup, mode):
    raw, W, model, env, reqs, plain = setup
    steps = {"whole": TR.trace_whole, "singles": TR.trace_prefill_then_singles, "portions": TR.trace_portions,
             "mixed": lambda r: TR.trace_mixed(r, seed=4)}[mode](reqs)
    TR.number(steps)
    got, _ = replay(model, env, steps, TR.peak_tokens(steps))
    want = TR.expected_rows(steps, lambda rid: plain[rid[1:]])
    assert set(got) == set(want)
    for k in want:
        torch.testing.assert_close(got[k].double(), want[k], rtol=1e-4, atol=1e-4)


def test_the_registry_finds_the_architecture_by_its_name(tmp_path):
    raw, W, model, env, config = build("A", tmp_path)
    assert isinstance(config, ZederaxConfig) and config.model_type_name == "zederax"
    assert LmConfig.from_dict(config.to_hf_config()) == config
    assert [b.kind for b in model.blocks] == ["parallel"] * 4
    # groups of the cache: layers differ in their windows and head sizes, so each has a group of its own here
    reqs = [r for _, r in model.cache_requirements()]
    assert [(r.n_kv_heads, r.head_dim, r.v_dim, r.window) for r in reqs] == [(2, 16, 8, 24), (2, 24, 8, 37), (2, 8, 8, None), (1, 16, 16, 5)]
    # which layer leaves its values and which ones blend: the first with v_mix is the source, the layer between has none
    assert [b.mixer.value_mix for b in model.blocks] == ["source", None, "blend", None]
    assert model.blocks[1].feed_forward is None and model.blocks[0].feed_forward is not None


def test_bad_configurations_and_checkpoints_are_refused(tmp_path):
    raw = json.loads(json.dumps(ZED["A"][0]))
    for change, match in ((lambda c: c["layers"][0].update(type="recurrent"), "type"),
                          (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
                          (lambda c: c["layers"][2]["mixer"].update(vdim=16), "value heads differ"),
                          (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "mlp.kind"),
                          (lambda c: c.pop("norm"), "norm.eps"),
                          (lambda c: c["layers"][1]["mixer"].update(mask={"size": 0}), "mask")):
        bad = json.loads(json.dumps(raw))
        change(bad)
        with pytest.raises(ConfigError, match=match):
            LmConfig.from_dict(bad)
    with pytest.raises(ConfigError, match="neither"):
        LmConfig.from_dict({"vocab": 3})
    W = Z.random_weights(raw, 0)
    del W["l1.dwa"]
    W["l2.mix.talk"] = torch.zeros(3, 3, dtype=torch.float64)
    W["l0.extra"] = torch.zeros(2, dtype=torch.float64)
    d = Z.write_folder(raw, W, str(tmp_path / "bad"), torch.float32)
    with pytest.raises(WeightsError) as e:
        load_model(d, BuildEnv(torch.float32, torch.device("cpu"), EmulatedKernels()))
    assert e.value.missing == ["l1.dwa"] and e.value.unexpected == ["l0.extra"] and "l2.mix.talk" in e.value.wrong_shape[0]


def test_the_stream_after_every_layer(tmp_path):
    """The residual stream that each layer hands on, through the parts themselves, against the plain implementation."""
    raw, W, model, env, _ = build("A", tmp_path)
    tokens = TR.random_requests(raw["vocab"], [53], 9)["r0"]
    want = Z.plain_streams(W, raw, torch.tensor(tokens))
    cache = make_cache(model, InferenceEngineConfig(max_pages=8, max_seqs=2, page_size=16, max_pages_per_seq=8, compute_dtype="float32"))
    runner = ModelRunner(model, cache, env)
    h = cache.open("a")
    got = []
    for blk in model.blocks:  # record what every block leaves in x
        fwd = blk.forward

        def spy(x, ctx, unit, writes, fwd=fwd):
            fwd(x, ctx, unit, writes)
            got.append(x.clone())

        blk.forward = spy
    try:
        runner.step([StepEntry(h, tokens[:31], []), ])
        runner.step([StepEntry(h, tokens[31:], [0])])
    finally:
        for blk in model.blocks:
            del blk.forward
    n = len(model.blocks)
    for i in range(n):
        torch.testing.assert_close(torch.cat([got[i], got[n + i]]).double(), want[i], rtol=1e-4, atol=1e-4)


def test_windowed_layers_give_pages_back_and_take_used_ones(tmp_path):
    """A request far longer than its windows holds few pages in the windowed groups; the pages it gave back are handed to
    the next request, whose logits are those of the plain implementation."""
    raw, W, model, env, _ = build("A", tmp_path)
    reqs = TR.random_requests(raw["vocab"], [150, 60], 3)
    cache = make_cache(model, InferenceEngineConfig(max_pages=14, max_seqs=2, page_size=16, max_pages_per_seq=16, compute_dtype="float32",
                                                    max_prefill_size=32))
    runner = ModelRunner(model, cache, env)
    a = cache.open("a")
    toks = reqs["r0"]
    rows = []
    for i in range(0, 150, 25):
        rows.append(runner.step([StepEntry(a, toks[i:i + 25], list(range(25)))]))
        cache.check_invariants()
    torch.testing.assert_close(torch.cat(rows).double(), Z.plain_logits(W, raw, torch.tensor(toks)), rtol=1e-4, atol=1e-4)
    by_window = {g.requirement.window: len(g.pages_held(a.slot)) for g in cache.groups}
    assert by_window[None] == 10 and by_window[24] <= 3 and by_window[37] <= 4 and by_window[5] <= 2
    b = cache.open("b")  # takes pages that a has given back (the pool hands out the page freed last)
    used_before = {g.index: set(range(g.pool.n_pages)) - set(g.pool._free) - set(g.pages_held(a.slot)) for g in cache.groups}
    got = runner.step([StepEntry(b, reqs["r1"], list(range(60)))])
    assert all(not used_before[g.index] for g in cache.groups)
    torch.testing.assert_close(got.double(), Z.plain_logits(W, raw, torch.tensor(reqs["r1"])), rtol=1e-4, atol=1e-4)
    cache.close(a)
    cache.close(b)
    cache.check_invariants()


def test_the_hip_library_offers_every_launcher_that_its_stand_in_has():
    from levanter_amd.kernels.library import HipKernels

    missing = [n for n in dir(EmulatedKernels) if not n.startswith("_") and callable(getattr(EmulatedKernels, n))
               and n not in ("k_view", "v_view", "gather_kv") and not hasattr(HipKernels, n)]
    assert not missing, missing
