"""Tarunex through the engine's own step function, cache manager, scheduler and entry point, with the CPU stand-in
for the kernels: what is tested here is the logic around them (which pages, which walk's cache, what meets the stream
where a walk begins, which norm feeds which sublayer), against the plain implementation."""
import copy

import pytest
import torch

from tests import replay_cases as rc
from tests import tarunex_cases as tc
from tests.plain.tarunex_plain import PlainTarunex

CPU = ["--device", "cpu"]
TOL = dict(atol=3e-4, rtol=3e-4)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: tc.write_model(str(tmp_path_factory.mktemp("tar_" + name)), cfg, seed, tweak, torch.float32)
            for name, cfg, seed, tweak in (("a", tc.TAR_A, 3, None), ("b", tc.TAR_B, 4, None), ("a_sharp", tc.TAR_A, 5, tc.sharpen()),
                                        ("a_sink", tc.TAR_A, 6, tc.both(tc.heavy_sink(), tc.strong_penalty())),
                                        ("plain", tc.TAR_PLAIN, 2, None), ("tail", tc.TAR_TAIL, 8, None), ("bare", tc.TAR_BARE, 11, None))}


def test_configuration_is_read_by_name_and_checked():
    from spyinfer_amd.config import ConfigError, TarunexConfig
    from spyinfer_amd.config.registry import architecture_of
    assert architecture_of(tc.TAR_A).name == "Tarunex"
    cfg = TarunexConfig.from_dict(copy.deepcopy(tc.TAR_A))
    assert (cfg.vocab, cfg.width, cfg.embedding_scale, cfg.logit_scale, cfg.logit_softcap, len(cfg.layers)) == (89, 40, 3.0, 0.7, 12.0, 5)
    assert cfg.loop == dict(start=1, stop=3, times=3) and TarunexConfig.from_dict(copy.deepcopy(tc.TAR_PLAIN)).loop is None
    assert cfg.layers[1]["mixer"]["q_temp"] == dict(coef=0.4, every=5) and cfg.layers[0]["mixer"]["rot"] == dict(base=500.0, dims=6)
    assert cfg.layers[3]["mlp"] is None and cfg.layers[1]["mlp"] == dict(kind="moe", ff=20, experts=8, top=3, shared_ff=14)
    for path, value in ((("layers", 1, "mixer", "kv_heads"), 3), (("layers", 0, "type"), "conv"), (("layers", 0, "mixer", "rot", "dims"), 3),
                        (("layers", 0, "mixer", "rot", "dims"), 8), (("width",), None), (("layers", 1, "mlp", "kind"), "dense"),
                        (("layers", 0, "mlp", "router", "top"), 9), (("loop", "stop"), 6), (("loop", "start"), 3), (("loop", "times"), 0),
                        (("norm", "eps"), 0.0), (("layers", 1, "mixer", "q_temp", "every"), 0), (("layers", 0, "mixer", "q_rank"), None),
                        (("layers", 1, "mixer", "softcap"), -1.0), (("logit_softcap",), -2.0)):
        bad = copy.deepcopy(tc.TAR_A)
        node = bad
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError):
            TarunexConfig.from_dict(bad)


def test_every_walk_has_caches_of_its_own():
    from spyinfer_amd.cache.spec import PagedKV, PagedRows
    from spyinfer_amd.config import TarunexConfig
    from spyinfer_amd.models.tarunex import build_tarunex
    model = build_tarunex(TarunexConfig.from_dict(copy.deepcopy(tc.TAR_A)))
    calls = model.schedule
    assert [(c.layer, c.cache, c.enter) for c in calls] == [(0, 0, None), (1, 1, 0), (2, 2, None), (1, 3, 1), (2, 4, None), (1, 5, 2),
                                                            (2, 6, None), (3, 7, None), (4, 8, None)]
    specs = model.cache_specs()
    # key and value heads of different sizes share one padded head size; a latent layer keeps one row per token
    assert specs[1] == specs[3] == specs[5] == PagedKV(2, 16, None) and specs[2] == specs[4] == specs[6] == PagedRows(6 + 4, None)
    assert specs[0] == PagedRows(9 + 6, None) and specs[7] == PagedKV(3, 16, None) and specs[8] == PagedKV(1, 4, None)
    plain = build_tarunex(TarunexConfig.from_dict(copy.deepcopy(tc.TAR_PLAIN)))
    assert plain.pass_entry is None and [(c.layer, c.cache, c.enter) for c in plain.schedule] == [(0, 0, None), (1, 1, None), (2, 2, None)]
    assert not any(s.name == "loop.step" for s in plain.weight_specs()) and any(s.name == "loop.step" and s.shape == (3, 40) for s in model.weight_specs())
    # a layer without a feed-forward has no second norm
    names = {s.name for s in model.weight_specs()}
    assert "l3.norm1" in names and "l3.norm2" not in names and "l1.norm2" in names and "l1.mlp.shared.up" in names and "l1.mlp.router.b" in names


@pytest.mark.parametrize("name", ["a", "b", "a_sharp", "a_sink", "plain", "tail", "bare"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_schedules_equal_the_plain_implementation(folders, name, mode, tmp_path, emu_ops):
    folder = folders[name]
    requests = rc.random_requests(tc.vocab_of(folder), [41, 1, 2, 67, 23, 30, 52, 38, 45], 7)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 12), "portions": rc.portions, "mixed": rc.mixed}[mode](requests)
    if mode == "mixed":
        rc.assert_mixed(steps, name)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), CPU + ["--kvcache-block-size", "8"])
    rc.compare(rc.collect(str(tmp_path), steps, tc.vocab_of(folder)), tc.plain_logits(folder, requests), what="%s/%s" % (name, mode), **TOL)


def test_pages_go_back_and_are_used_again(folders, emu_ops):
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    folder = folders["a_sharp"]
    model = load_model(folder, "float32", "cpu")
    runner = ModelRunner(model, "float32", "cpu", 4, 26, 2, max_num_batched_tokens=1 << 20)
    plain = PlainTarunex.from_folder(folder)
    m = runner.manager
    for turn in range(3):                          # the same two slots and the same pages serve three pairs of requests
        reqs = rc.random_requests(89, [57, 33], 20 + turn)
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
    plain = PlainTarunex.from_folder(folder)
    prompts = list(rc.random_requests(89, [5, 17, 2, 30, 9], 9).values())
    want = [plain.greedy(p, 10) for p in prompts]
    for opts in (dict(), dict(max_num_batched_tokens=12, prefill_chunk=7, max_num_seqs=2), dict(num_kvcache_blocks=None)):
        kw = dict(dtype="float32", max_model_len=64, num_kvcache_blocks=24, max_num_seqs=4, kvcache_block_size=8, device="cpu")
        kw.update(opts)
        eng = LLMEngine(folder, **kw)
        assert eng.generate(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True)) == want
        eng.runner.manager.check()
    # a pool too small for all requests at once: the request admitted last is preempted, gives its pages back and later
    # runs again from its first token
    eng = LLMEngine(folder, dtype="float32", max_model_len=64, num_kvcache_blocks=9, max_num_seqs=4, kvcache_block_size=8, device="cpu")
    assert eng.generate(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True)) == want
    assert eng.scheduler.num_preemptions > 0
    eng.runner.manager.check()
