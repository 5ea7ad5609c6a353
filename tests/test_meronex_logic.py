"""Meronex through the engine's own step function, cache manager, scheduler and entry point, with the CPU stand-in
for the kernels: what is tested here is the logic around them (which pages and slots, which state, which kept rows of
the token shift and the convolutions, which gate meets which result), against the plain implementation."""
import copy

import pytest
import torch

from tests import meronex_cases as mc
from tests import replay_cases as rc
from tests.plain.meronex_plain import PlainMeronex

CPU = ["--device", "cpu"]
TOL = dict(atol=3e-4, rtol=3e-4)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: mc.write_model(str(tmp_path_factory.mktemp("mer_" + name)), cfg, seed, tweak, torch.float32)
            for name, cfg, seed, tweak in (("a", mc.MER_A, 3, None), ("b", mc.MER_B, 4, None), ("a_sharp", mc.MER_A, 5, mc.sharpen()),
                                        ("a_memory", mc.MER_A, 9, mc.long_memory()), ("odd", mc.MER_ODD, 2, None))}


def test_configuration_is_read_by_name_and_checked():
    from spyinfer_amd.config import ConfigError, MeronexConfig
    from spyinfer_amd.config.registry import architecture_of
    assert architecture_of(mc.MER_A).name == "Meronex"
    cfg = MeronexConfig.from_dict(copy.deepcopy(mc.MER_A))
    assert (cfg.vocab, cfg.width, cfg.norm_groups, cfg.residual_mult, len(cfg.layers)) == (97, 48, 3, 0.7, 7)
    left = cfg.layers[0]["mixer"]["left"]
    assert left["softcap"] == 4.0 and left["rot"]["scaling"]["fast"] == 4.0 and cfg.layers[3]["mixer"]["left"]["softcap"] == 0.0
    assert cfg.layers[3]["mixer"]["left"]["rot"]["scaling"] is None and cfg.layers[6]["mixer"]["left"]["rot"] is None
    assert cfg.layers[2]["mlp"] is None and cfg.layers[0]["mlp"] == dict(kind="moe", ff=24, limit=1.5, experts=8, top=3)
    for path, value in ((("layers", 0, "mixer", "left", "kv_heads"), 3), (("layers", 0, "type"), "conv"), (("layers", 0, "mixer", "left", "rot", "dims"), 3),
                        (("layers", 0, "mixer", "left", "rot", "dims"), 10), (("width",), None), (("layers", 1, "mlp", "kind"), "dense"),
                        (("layers", 0, "mlp", "router", "top"), 9), (("layers", 0, "mlp", "expert", "limit"), 0.0), (("norm", "groups"), 5),
                        (("layers", 1, "mixer", "gate_cap"), 0.0), (("layers", 2, "mixer", "conv"), 9), (("norm", "eps"), 0.0),
                        (("layers", 2, "mixer", "kv_heads"), 3), (("layers", 0, "mixer", "right", "dim"), 0)):
        bad = copy.deepcopy(mc.MER_A)
        node = bad
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError):
            MeronexConfig.from_dict(bad)


def test_cache_kinds_follow_the_layers():
    from spyinfer_amd.cache.spec import FixedState, PagedKV
    from spyinfer_amd.config import MeronexConfig
    from spyinfer_amd.models.meronex import build_meronex
    model = build_meronex(MeronexConfig.from_dict(copy.deepcopy(mc.MER_A)))
    specs = model.cache_specs()
    # a layer of two mixers has two caches: pages for the attention under the layer's own id, the time mix's slot behind
    # the layers' ids; key and value heads of different sizes share one padded head size
    assert len(specs) == 7 + 3 and model.cache_parts == {0: [0, 7], 3: [3, 8], 6: [6, 9]}
    assert specs[0] == PagedKV(2, 16, None) and specs[3] == PagedKV(1, 16, None) and specs[6] == PagedKV(3, 4, None)
    assert specs[7] == FixedState((3 * 4 * 4 + 48,), "float32") and specs[9] == FixedState((6 * 6 + 48,), "float32")
    assert specs[1] == FixedState((3 * (5 * 7 + 5 + 1),), "float32")          # (seven value channels: one slice)
    assert specs[2] == FixedState((4 * 6 * 5 + 2 * (2 * 2 * 6 + 4 * 5),), "float32")
    assert model.cache_specs() == specs


def test_an_inner_size_that_no_key_names_comes_from_the_tensors(folders, emu_ops, tmp_path):
    """The decay's two projections of the time mix: without the optional key the stored tensors decide."""
    import json
    import os
    import shutil
    folder = str(tmp_path / "m")
    shutil.copytree(folders["a"], folder)
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    for layer in cfg["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["right"].pop("decay_rank")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    requests = rc.random_requests(97, [19], 3)
    steps = rc.whole(requests)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path / "out"), steps, rc.max_live_tokens(steps), CPU)
    rc.compare(rc.collect(str(tmp_path / "out"), steps, 97), mc.plain_logits(folders["a"], requests), what="rank from tensors", **TOL)


@pytest.mark.parametrize("name", ["a", "b", "a_sharp", "a_memory", "odd"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_schedules_equal_the_plain_implementation(folders, name, mode, tmp_path, emu_ops):
    folder = folders[name]
    requests = rc.random_requests(mc.vocab_of(folder), [41, 1, 2, 67, 23, 30, 52, 38, 45], 7)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 12), "portions": rc.portions, "mixed": rc.mixed}[mode](requests)
    if mode == "mixed":
        rc.assert_mixed(steps, name)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), CPU + ["--kvcache-block-size", "8"])
    rc.compare(rc.collect(str(tmp_path), steps, mc.vocab_of(folder)), mc.plain_logits(folder, requests), what="%s/%s" % (name, mode), **TOL)


def test_recurrences_alone_run_without_any_page_group(tmp_path, emu_ops):
    folder = mc.write_model(str(tmp_path / "m"), mc.MER_REC, 1, None, torch.float32)
    requests = rc.random_requests(53, [21, 1, 2, 33, 9], 5)
    ref = mc.plain_logits(folder, requests)
    for name, steps in (("whole", rc.whole(requests)), ("portions", rc.portions(requests)), ("mixed", rc.mixed(requests))):
        out = str(tmp_path / name)
        rc.run_replay_inprocess(folder, "float32", out, steps, rc.max_live_tokens(steps), CPU)
        rc.compare(rc.collect(out, steps, 53), ref, what=name, **TOL)


def test_pages_and_slots_go_back_and_are_used_again(folders, emu_ops):
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    folder = folders["a_memory"]
    model = load_model(folder, "float32", "cpu")
    runner = ModelRunner(model, "float32", "cpu", 4, 26, 2, max_num_batched_tokens=1 << 20)
    plain = PlainMeronex.from_folder(folder)
    m = runner.manager
    for turn in range(3):                          # the same two slots and the same pages serve three pairs of requests
        reqs = rc.random_requests(97, [57, 33], 20 + turn)
        held = {rid: m.admit(rid) for rid in reqs}
        got = {rid: [] for rid in reqs}
        fed = {rid: 0 for rid in reqs}
        while any(fed[r] < len(reqs[r]) for r in reqs):
            entries = []
            for rid, toks in reqs.items():
                n = min(5 if rid == "r0" else 1, len(toks) - fed[rid])
                if n:
                    m.reserve(held[rid], n)
                    entries.append((rid, StepEntry(held[rid], toks[fed[rid]:fed[rid] + n], list(range(n)))))
                    fed[rid] += n
            logits = runner.step([e for _, e in entries])
            r = 0
            for rid, e in entries:
                got[rid].append(logits[r:r + len(e.tokens)].clone())
                r += len(e.tokens)
            m.check()
        for rid, toks in reqs.items():
            torch.testing.assert_close(torch.cat(got[rid]), plain.forward(toks).float(), **TOL)
            m.release(held[rid])
        assert m.num_free_pages() == [g.pool.num_pages for g in m.page_groups] and m.slots.num_free == 2


def test_greedy_generation_through_the_entry_point(folders, emu_ops):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    folder = folders["a"]
    plain = PlainMeronex.from_folder(folder)
    prompts = list(rc.random_requests(97, [5, 17, 2, 30, 9], 9).values())
    want = [plain.greedy(p, 10) for p in prompts]
    for opts in (dict(), dict(max_num_batched_tokens=12, prefill_chunk=7, max_num_seqs=2), dict(num_kvcache_blocks=None)):
        kw = dict(dtype="float32", max_model_len=64, num_kvcache_blocks=24, max_num_seqs=4, kvcache_block_size=8, device="cpu")
        kw.update(opts)
        eng = LLMEngine(folder, **kw)
        assert eng.generate(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True)) == want
        eng.runner.manager.check()
    # a pool too small for all requests at once: the request admitted last is preempted, gives its slot and pages back
    # and later runs again from its first token, with every state, kept row and kept input starting anew
    eng = LLMEngine(folder, dtype="float32", max_model_len=64, num_kvcache_blocks=9, max_num_seqs=4, kvcache_block_size=8, device="cpu")
    assert eng.generate(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True)) == want
    assert eng.scheduler.num_preemptions > 0
    eng.runner.manager.check()
