"""Sosepel without a GPU: the configuration reader, the model the builder makes (tensor names
and shapes, the order of the layer runs, caches and state), random-weights folders, and the
plain implementation's own properties (causality, the routing rule, the pair hash)."""
import copy
import math

import pytest
import torch

import plain_sosepel
import sosepel_cases
import util


def _spec(raw):
    from ninfer_amd import build_spec
    return build_spec(raw)


@pytest.mark.parametrize("name", list(sosepel_cases.CASES))
def test_builder_names_every_tensor(name, tmp_path):
    import ninfer_amd
    make, seed = sosepel_cases.CASES[name]
    raw = make()
    cfg, spec = _spec(raw)
    specs = spec.tensor_specs()
    w = raw["width"]
    assert specs["embed"].shape == (raw["vocab"], w) and specs["final.norm"].shape == (w,)
    pairs = raw["embedding"].get("bigram")
    assert ("bigram" in specs) == bool(pairs)
    if pairs:
        assert specs["bigram"].shape == (pairs["buckets"] + 1, w)
    assert ("loop.in" in specs) == ("loop" in raw)
    for i, layer in enumerate(raw["layers"]):
        m = layer["mixer"]
        assert specs[f"l{i}.mix.q"].shape == (m["heads"] * 2 * m["dim"], w)
        assert specs[f"l{i}.mix.k"].shape == (m["kv_heads"] * 2 * m["dim"], w)
        assert specs[f"l{i}.mix.v"].shape == (m["kv_heads"] * m["vdim"], w)
        assert specs[f"l{i}.mix.o"].shape == (w, m["heads"] * m["vdim"])
        assert specs[f"l{i}.mix.lk2"].shape == (m["dim"],) and specs[f"l{i}.ls1"].shape == (w,)
        c = layer["mlp"]
        assert (f"l{i}.ls2" in specs) == bool(c)
        if c and c["kind"] == "moe":
            e = c["router"]["experts"]
            assert specs[f"l{i}.mlp.router"].shape == (e, w)
            assert specs[f"l{i}.mlp.e{e - 1}.down"].shape == (w, c["expert"]["ff"])
            assert (f"l{i}.mlp.shared.sg" in specs) == bool(c.get("shared"))
        elif c:
            assert specs[f"l{i}.mlp.up"].shape == (c["ff"], w)
    # the runs of the layers: a looped layer once per pass, each pass entered through the join
    runs = plain_sosepel.layer_order(raw)
    assert [(c.layer, c.before is not None) for c in spec.plan] == runs
    assert cfg.runs() == runs
    assert spec.embedding.state_floats() == (1 if pairs else 0)
    # a folder of random weights holds exactly these tensors, and the plain implementation runs on it
    d = str(tmp_path)
    ninfer_amd.write_random_model(d, raw, seed, dtype="float32", std=0.2)
    cfg2, w2 = util.read_folder(d)
    assert set(w2) == set(specs)
    toks = util.random_tokens(20, raw["vocab"], 1)
    logits = plain_sosepel.forward(w2, cfg2, toks)
    assert logits.shape == (20, raw["vocab"]) and torch.isfinite(logits).all()
    # causal: the logits of a prefix are those of the whole
    torch.testing.assert_close(plain_sosepel.forward(w2, cfg2, toks[:9]), logits[:9], atol=1e-12, rtol=0)


def test_config_errors_name_the_key():
    from ninfer_amd.config import ConfigError, SosepelConfig
    good = sosepel_cases.config_odd()
    SosepelConfig.from_dict(good)
    for path, value, word in (
            (("vocab",), None, "vocab"), (("norm", "eps"), 0.0, "norm.eps"),
            (("layers", 0, "type"), "lightning", "type"), (("layers", 1, "mixer", "kv_heads"), 2, "kv_heads"),
            (("layers", 1, "mlp", "router", "top"), 5, "router"), (("loop", "stop"), 9, "loop"),
            (("layers", 1, "mlp", "kind"), "mix", "kind"), (("embedding", "bigram", "buckets"), 0, "buckets"),
            (("logit_softcap",), -1.0, "logit_softcap"), (("layers", 0, "mixer", "diff"), None, "diff")):
        raw = copy.deepcopy(good)
        at = raw
        for k in path[:-1]:
            at = at[k]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError) as e:
            SosepelConfig.from_dict(raw)
        assert word in str(e.value)


def test_what_may_be_absent():
    from ninfer_amd.config import SosepelConfig
    cfg = SosepelConfig.from_dict(sosepel_cases.config_ones())
    m = cfg.layers[0].mixer
    assert m.softcap == 0.0 and m.temp_coef == 0.0 and m.kv_heads == m.heads
    assert cfg.pairs is None and cfg.logit_softcap == 0.0
    assert cfg.layers[0].mlp.groups == 1 and cfg.layers[0].mlp.shared_ff == 0
    assert SosepelConfig.from_dict(sosepel_cases.config_straight()).loop is None


def test_plain_routing_rule():
    s = torch.tensor([[0.9, 0.1, 0.5, 0.55, 0.8, 0.2]], dtype=torch.float64)
    # groups of two: sums 1.0, 1.05, 1.0 -> the middle group, then the first of the tied (the lower)
    chosen, weights, _ = plain_sosepel.route(s, {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}})
    assert chosen.tolist() == [[0, 3]]
    torch.testing.assert_close(weights, torch.tensor([[0.9, 0.55]], dtype=torch.float64) / 1.45)
    chosen, _, _ = plain_sosepel.route(s, {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}})
    assert chosen.tolist() == [[3, 2]]
    chosen, _, _ = plain_sosepel.route(s, {"experts": 6, "top": 3})
    assert chosen.tolist() == [[0, 4, 3]]


def test_plain_pair_rows_and_temperature():
    assert plain_sosepel.pair_rows([3, 4, 4], 7, 5, 2) == [7, (15 + 8) % 7, (20 + 8) % 7]
    t = plain_sosepel.query_temperature(9, {"coef": 0.5, "every": 4})
    assert t[2] == 1.0 and t[3] == 1.0 + 0.5 * math.log(2) and t[6] == t[3] and t[7] == 1.0 + 0.5 * math.log(3)


# ---- the engine's host logic on the CPU, with plain stand-ins for the kernels ------------------

@pytest.fixture(scope="module", params=["odd", "ones", "straight"])
def host_case(request, tmp_path_factory):
    import ninfer_amd
    make, seed = sosepel_cases.CASES[request.param]
    raw = make()
    d = str(tmp_path_factory.mktemp("sosepel_host_" + request.param))
    ninfer_amd.write_random_model(d, raw, seed, dtype="float32", std=0.25)
    cfg, w = util.read_folder(d)
    reqs = {f"r{i}": util.random_tokens(n, raw["vocab"], 20 + i) for i, n in enumerate([33, 1, 12, 47, 20])}
    margins = {k: [] for k in reqs}
    ref = {k: plain_sosepel.forward(w, cfg, v, margins=margins[k]) for k, v in reqs.items()}
    # rows at which a routing decision is a close call are left out of the comparisons
    clear = {k: torch.stack([m > 1e-4 for m in margins[k]]).all(0) if margins[k]
             else torch.ones(len(reqs[k]), dtype=torch.bool) for k in reqs}
    return {"dir": d, "cfg": raw, "reqs": reqs, "ref": ref, "clear": clear}


def _host_runner(case, **more):
    from ninfer_amd import EngineOptions, load_model
    from plain_ops import PlainOps
    opt = dict(dtype="float32", device="cpu", max_context=64, num_sequences=4, page_size=4, num_pages=40,
               check_pages=True)
    opt.update(more)
    return load_model(case["dir"], EngineOptions(**opt), ops=PlainOps())


def _close(case, got):
    for rid, g in got.items():
        rid = rid.split("#")[0]
        ok = case["clear"][rid]
        # a close call at one row changes what that row writes into the cache for all later rows
        upto = int((~ok).nonzero()[0]) if (~ok).any() else len(ok)
        torch.testing.assert_close(g.double()[:upto], case["ref"][rid][:upto], atol=2e-4, rtol=2e-4)


def test_host_every_way_of_cutting(host_case):
    runner = _host_runner(host_case)
    for rid, toks in host_case["reqs"].items():
        scheds = [util.schedule_whole(rid, toks), util.schedule_portions(rid, toks, seed=len(toks))]
        if len(toks) > 1:
            scheds.append(util.schedule_tail(rid, toks, 9))
        for sched in scheds:
            _close(host_case, util.run_schedule(runner, sched))
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_host_mixed_batches_reuse_pages_and_slots(host_case):
    """Portions beside single tokens, a pool that forces pages to be used again, two state
    slots for five requests and their repeats: a slot's previous token is that of its request."""
    runner = _host_runner(host_case, num_sequences=2, num_pages=26)
    reqs = dict(host_case["reqs"])
    reqs.update({k + "#2": v for k, v in host_case["reqs"].items()})
    _close(host_case, util.run_schedule(runner, util.schedule_mixed(reqs, seed=2, max_live=2)))
    assert runner.cache.pages_reused() > 0
    runner.cache.check()


def test_host_generation_through_the_scheduler(host_case):
    """Greedy generation by the scheduler (admission, portions under a token budget, batched
    decoding with fewer slots than requests), token for token the plain choice. Preemption
    gives a request's slot to another and runs it again from its first token."""
    from ninfer_amd import Request, Sampler, SamplingParams, Scheduler
    from plain_ops import PlainOps
    cfg, w = util.read_folder(host_case["dir"])
    prompts = [host_case["reqs"]["r2"], host_case["reqs"]["r1"], host_case["reqs"]["r4"][:7],
               host_case["reqs"]["r0"][:15]]
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(6):
            margins = []
            logits = plain_sosepel.forward(w, cfg, toks, margins=margins)[-1]
            top = torch.topk(logits, 2).values
            if top[0] - top[1] < 1e-3 or any(float(m.min()) < 1e-3 for m in margins):
                break
            toks.append(int(logits.argmax()))
        want.append(toks[len(p):])
    runner = _host_runner(host_case, num_sequences=2, prefill_chunk=8, num_pages=14)
    sched = Scheduler(runner, Sampler(PlainOps(), runner.device))
    reqs = [Request(f"q{i}", list(p), SamplingParams.greedy(6)) for i, p in enumerate(prompts)]
    for r in reqs:
        sched.add(r)
    sched.run()
    assert all(r.status == "finished" for r in reqs), [r.error for r in reqs]
    assert [r.output[:len(x)] for r, x in zip(reqs, want)] == want
