"""Sefevik through the engine's own step function, cache manager, scheduler and entry point, with the CPU stand-in
for the kernels: what is tested here is the logic around them (which pages and slots, which previous token, which
rows are kept for which window), against the plain implementation."""
import copy

import pytest
import torch

from tests import replay_cases as rc
from tests import sefevik_cases as sc
from tests.plain.sefevik_plain import PlainSefevik

CPU = ["--device", "cpu"]
TOL = dict(atol=2e-4, rtol=2e-4)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: sc.write_model(str(tmp_path_factory.mktemp("sef_" + name)), cfg, seed, tweak)
            for name, cfg, seed, tweak in (("a", sc.SEF_A, 3, None), ("b", sc.SEF_B, 4, None), ("a_sharp", sc.SEF_A, 5, sc.sharpen()),
                                        ("a_sink", sc.SEF_A, 9, sc.heavy_sinks()))}


def test_configuration_is_read_by_name_and_checked():
    from spyinfer_amd.config import ConfigError, SefevikConfig
    from spyinfer_amd.config.registry import architecture_of
    assert architecture_of(sc.SEF_A).name == "Sefevik"
    cfg = SefevikConfig.from_dict(copy.deepcopy(sc.SEF_A))
    assert (cfg.vocab, cfg.width, cfg.bigram_buckets, len(cfg.layers)) == (97, 48, 53, 5)
    assert cfg.layers[2]["mixer"]["kv_from"] == 0 and cfg.layers[3]["mixer"]["window"] is None and cfg.layers[1]["mlp"] is None
    assert SefevikConfig.from_dict(copy.deepcopy(sc.SEF_B)).bigram_buckets == 0
    for path, value in ((("layers", 2, "mixer", "kv_from"), 1), (("layers", 2, "mixer", "kv_rank"), 24), (("layers", 0, "type"), "conv"),
                        (("layers", 0, "mixer", "rot", "dims"), 3), (("width",), None), (("layers", 4, "mlp", "kind"), "gated")):
        bad = copy.deepcopy(sc.SEF_A)
        node = bad
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError):
            SefevikConfig.from_dict(bad)


def test_rows_are_kept_for_the_largest_window_that_reads_them():
    from spyinfer_amd.config import SefevikConfig
    from spyinfer_amd.models.sefevik import build_sefevik
    model = build_sefevik(SefevikConfig.from_dict(copy.deepcopy(sc.SEF_A)))
    specs = model.cache_specs()
    assert specs[0].window == 13 and specs[0].width == 24 and specs[2] is None           # layer 2 reads cache 0
    assert specs[3].window is None and specs[1].shape == (40,) and specs[5].dtype == "int32"
    assert [(c.layer, c.cache, c.store) for c in model.schedule][2] == (2, 0, False)


@pytest.mark.parametrize("name", ["a", "b", "a_sharp", "a_sink"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_schedules_equal_the_plain_implementation(folders, name, mode, tmp_path, emu_ops):
    folder = folders[name]
    requests = rc.random_requests(sc.vocab_of(folder), [41, 1, 2, 67, 23, 30, 52, 38, 45], 7)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 12), "portions": rc.portions, "mixed": rc.mixed}[mode](requests)
    if mode == "mixed":
        rc.assert_mixed(steps, name)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), CPU + ["--kvcache-block-size", "8"])
    rc.compare(rc.collect(str(tmp_path), steps, sc.vocab_of(folder)), sc.plain_logits(folder, requests), what="%s/%s" % (name, mode), **TOL)


def test_pages_of_passed_windows_and_slots_go_back_and_are_used_again(folders, emu_ops):
    from spyinfer_amd.engine.batch import StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    folder = folders["a"]
    model = load_model(folder, "float32", "cpu")
    runner = ModelRunner(model, "float32", "cpu", 4, 40, 2, max_num_batched_tokens=1 << 20)
    plain = PlainSefevik.from_folder(folder)
    m = runner.manager
    windowed = next(g for g in m.page_groups if g.spec.window == 13)
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
            # a request holds no more pages of the windowed rows than the window and the step's tokens need
            assert all(len(rcache.pages_held(windowed.index)) <= (13 + 5) // 4 + 2 for rcache in held.values())
        for rid, toks in reqs.items():
            torch.testing.assert_close(torch.cat(got[rid]), plain.forward(toks).float(), **TOL)
            m.release(held[rid])
        assert m.num_free_pages() == [g.pool.num_pages for g in m.page_groups] and m.slots.num_free == 2


def test_greedy_generation_through_the_entry_point(folders, emu_ops):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    folder = folders["a"]
    plain = PlainSefevik.from_folder(folder)
    prompts = list(rc.random_requests(97, [5, 17, 2, 30, 9], 9).values())
    want = [plain.greedy(p, 10) for p in prompts]
    # (the last: the pool sized from the device's free memory, with the slots' state and the windows' groups counted)
    for opts in (dict(), dict(max_num_batched_tokens=12, prefill_chunk=7, max_num_seqs=2), dict(num_kvcache_blocks=None)):
        kw = dict(dtype="float32", max_model_len=64, num_kvcache_blocks=24, max_num_seqs=4, kvcache_block_size=8, device="cpu")
        kw.update(opts)
        eng = LLMEngine(folder, **kw)
        assert eng.generate(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True)) == want
        eng.runner.manager.check()
    # a pool too small for all requests at once: the request admitted last is preempted, gives its slot and pages back
    # and later runs again from its first token, with the recurrences' state and the previous token starting anew
    eng = LLMEngine(folder, dtype="float32", max_model_len=64, num_kvcache_blocks=9, max_num_seqs=4, kvcache_block_size=8, device="cpu")
    assert eng.generate(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True)) == want
    assert eng.scheduler.num_preemptions > 0
    eng.runner.manager.check()
