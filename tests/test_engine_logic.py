"""The engine's logic (batch metadata, cache pages, block tables, every way of cutting) on the
CPU stand-in for the kernels, compared with the plain implementation."""
import numpy as np
import pytest
import torch

from tests import replay_cases as rc
from tests.configs import INIT, TINY_A, TINY_B, TINY_C, TINY_D
from tests.plain.qwen3_plain import PlainQwen3


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from spyinfer_amd.weights import write_random_model
    out = {}
    for name, cfg, seed in (("A", TINY_A, 11), ("B", TINY_B, 12), ("C", TINY_C, 13), ("D", TINY_D, 14)):
        out[name] = write_random_model(str(tmp_path_factory.mktemp("model_" + name)), cfg, seed, torch.bfloat16, **INIT)
    return out


CASES = {"A": (TINY_A, [5, 17, 33, 60, 44, 23, 9, 51]), "B": (TINY_B, [1, 40, 130, 75, 12, 100, 33]), "C": (TINY_C, [3, 70, 200, 45, 64, 97])}


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_cuts_match_plain(name, mode, folders, tmp_path, emu_ops):
    cfg, lengths = CASES[name]
    reqs = rc.random_requests(cfg["vocab_size"], lengths, seed=3)
    steps = getattr(rc, mode)(reqs)
    if mode == "mixed":
        rc.assert_mixed(steps, name)
    max_tokens = rc.max_live_tokens(steps)
    page = {"A": 16, "B": 8, "C": 16}[name]
    rc.run_replay_inprocess(folders[name], "float32", str(tmp_path), steps, max_tokens,
                            ["--device", "cpu", "--kvcache-block-size", str(page)])
    plain = PlainQwen3(folders[name])
    ref = {rid: plain.forward(t) for rid, t in reqs.items()}
    got = rc.collect(str(tmp_path), steps, cfg["vocab_size"])
    if mode != "mixed":
        assert len(got) == sum(lengths)
    rc.compare(got, ref, atol=2e-4, rtol=2e-4, what="%s/%s" % (name, mode))


def test_replay_lines_without_tokens_and_names_used_again(folders, tmp_path, emu_ops):
    """A line may bring no tokens at all (it only ends requests), a request may be left out of steps, and a name that
    has ended may be used again for a new request, which starts from an empty cache."""
    cfg = TINY_A
    reqs = rc.random_requests(cfg["vocab_size"], [21, 9], seed=5)
    a, b = reqs["r0"], reqs["r1"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:10], "want": [9]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": b, "want": [8]}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": a[10:], "want": [10]}, {"id": "y", "tokens": [], "want": []}], "end": []},
             {"step": 3, "entries": [], "end": ["x", "y"]},
             {"step": 4, "entries": [{"id": "x", "tokens": b, "want": [0, 8]}], "end": ["x"]}]
    rc.run_replay_inprocess(folders["A"], "float32", str(tmp_path), steps, 128, ["--device", "cpu"])
    plain = PlainQwen3(folders["A"])
    ra, rb = plain.forward(a), plain.forward(b)
    V = cfg["vocab_size"]
    read = lambda i, n: torch.from_numpy(np.fromfile(str(tmp_path / ("%d.f32" % i)), dtype="<f4").reshape(n, V).copy())
    assert not (tmp_path / "3.f32").exists()
    for got, ref in ((read(0, 1), ra[[9]]), (read(1, 1), rb[[8]]), (read(2, 1), ra[[20]]), (read(4, 2), rb[[0, 8]])):
        assert torch.allclose(got, ref, atol=2e-4, rtol=2e-4)


def test_cache_pool_is_sized_after_the_memory_of_captured_steps():
    """With graphs the pool is sized from what is left after the one logits tensor [max_num_seqs, vocab] and the
    metadata buffers of every captured step; with enforce_eager from all the free memory; never beyond what
    max_num_seqs requests of max_model_len tokens need."""
    from spyinfer_amd.config.engine_config import EngineConfig
    from spyinfer_amd.config.registry import architecture_of
    from spyinfer_amd.engine.llm_engine import pages_for_memory
    from spyinfer_amd.engine.runner import ModelRunner
    arch = architecture_of(TINY_B)
    model = arch.build(arch.config_cls.from_dict(TINY_B))
    per_page = 3 * 2 * 2 * 32 * 8 * 2                                     # layers, K and V, kv heads, head_dim, page, bfloat16
    assert ModelRunner.bytes_per_page(model, 8, "bfloat16") == per_page
    assert ModelRunner.bytes_per_page(model, 8, "float32") == 2 * per_page
    cfg = EngineConfig(max_num_seqs=64, max_model_len=512, kvcache_block_size=8, gpu_memory_utilization=0.5, enforce_eager=True)
    free = 40 << 20
    assert pages_for_memory(free, cfg, model) == int(free * 0.5 * 0.9) // per_page
    cfg.enforce_eager = False
    logits = 4 * 64 * 384
    # one page group, 512 / 8 = 64 pages per request; the attention's plan for 64 single tokens: a tile each (two arrays
    # of 64) and, the model's 2 kv heads of 32 not being a head size whose keys are cut on the host, nothing else
    planned = 2 * 64 + 2 * 4
    assert model.plan_ints(64) == planned
    meta = ModelRunner.MAX_GRAPHS * 4 * (64 * (1 * 64 + 64) + 256 + planned)
    assert ModelRunner.graph_logits_bytes(64, 384) == logits
    assert ModelRunner.MAX_GRAPHS * ModelRunner.graph_metadata_bytes(64, 1, 64, planned) == meta
    assert pages_for_memory(free, cfg, model) == int((free - logits - meta) * 0.5 * 0.9) // per_page
    assert pages_for_memory(1 << 20, cfg, model) == 1                       # less free memory than the graphs take: one page, no negative count
    cfg.gpu_memory_utilization = 1.0
    assert pages_for_memory(1 << 40, cfg, model) == 64 * 64                 # the cap


@pytest.mark.parametrize("name,act", [("B", torch.float32), ("B", torch.bfloat16), ("D", torch.bfloat16)])
def test_a_step_metadata_fits_the_bound_used_for_captured_steps(name, act, folders, emu_ops):
    """The per-entry bound of a captured step's metadata (a row of page numbers per page group, 64 further integers and
    what the parts plan) holds for real decode batches with fixed-width block tables, also where the attention's keys
    are cut on the host (bfloat16, a head size of 64)."""
    from spyinfer_amd.engine.batch import StepBatch, StepEntry
    from spyinfer_amd.engine.runner import ModelRunner, load_model
    model = load_model(folders[name], "float32", "cpu")
    runner = ModelRunner(model, "float32", "cpu", 8, 64, 6, max_model_len=128)
    caches = [runner.manager.admit(i) for i in range(6)]
    for n, c in enumerate(caches):
        runner.manager.reserve(c, 3 + 7 * n)
        runner.manager.commit(c, 3 + 7 * n)
        runner.manager.reserve(c, 1)
    for live in (1, 3, 6):
        batch = StepBatch([StepEntry(c, [5], [0]) for c in caches[:live]], runner.manager, act, "cpu", model.vocab_size, runner.fixed_max_blocks)
        model.plan(batch)
        _layout, total = batch.layout()
        assert 4 * total <= ModelRunner.graph_metadata_bytes(live, len(runner.manager.page_groups), runner.fixed_max_blocks, model.plan_ints(live))
        assert batch.has_array("decode_pieces_1_0_64") == (name == "D")


class _CacheNeeds:
    """Stands for a model where only its cache needs and vocabulary are asked."""

    def __init__(self, specs, vocab_size=100):
        self._specs, self.vocab_size = list(specs), vocab_size

    def cache_specs(self):
        return self._specs


def test_cache_pool_leaves_room_for_the_state_slots():
    """Per-request state of fixed size is allocated for max_num_seqs requests in every layer cache that has any, whatever
    the pool's size: it comes off the memory before the pages are counted, so that pages and slots together stay inside
    what was handed in.  State that does not fit by itself is an error with the way out in it; a model that keeps state
    only gets its one page after the same look at the memory."""
    from spyinfer_amd.cache import FixedState, PagedKV
    from spyinfer_amd.config.engine_config import EngineConfig
    from spyinfer_amd.engine.llm_engine import pages_for_memory
    kv, state = PagedKV(2, 64), FixedState((1 << 21,), "float32")              # 8 MB of state per request and layer
    model = _CacheNeeds([kv, state, kv, state])
    cfg = EngineConfig(max_num_seqs=16, max_model_len=1 << 20, kvcache_block_size=16, gpu_memory_utilization=1.0, enforce_eager=True)
    free = 1 << 30
    pages = pages_for_memory(free, cfg, model)
    per_page = 2 * (2 * 2 * 64 * 16 * 2)
    slots = 16 * 2 * (8 << 20)
    assert pages == (int(free * 0.9) - slots) // per_page
    assert pages * per_page + slots <= free
    cfg.max_num_seqs = 512                                                    # the default: 8 GB of state
    with pytest.raises(ValueError, match="lower max_num_seqs"):
        pages_for_memory(free, cfg, model)
    only_state = _CacheNeeds([state, None])
    cfg.max_num_seqs = 16
    assert pages_for_memory(free, cfg, only_state) == 1
    cfg.max_num_seqs = 512
    with pytest.raises(ValueError, match="lower max_num_seqs"):
        pages_for_memory(free, cfg, only_state)


def test_groups_with_a_window_take_what_their_windows_need_and_leave_the_rest():
    from spyinfer_amd.cache import CacheManager, PagedKV
    from spyinfer_amd.cache.manager import window_pages
    from spyinfer_amd.config.engine_config import EngineConfig
    from spyinfer_amd.engine.llm_engine import pages_for_memory
    full, win = PagedKV(1, 64), PagedKV(1, 64, window=100)
    cfg = EngineConfig(max_num_seqs=4, max_model_len=1 << 16, kvcache_block_size=16, gpu_memory_utilization=1.0, enforce_eager=True,
                       max_num_batched_tokens=64)
    per_page = 2 * 64 * 16 * 2
    most = 4 * window_pages(100, 16, 64)                      # (99 + 64) / 16 rounded up, one more for a start inside a page
    assert window_pages(100, 16, 64) == 12 and window_pages(100, 16) == 8
    free = 64 << 20
    budget = int(free * 0.9)
    assert pages_for_memory(free, cfg, _CacheNeeds([full, win])) == (budget - most * per_page) // per_page
    assert CacheManager.pages_of_group(win, 16, 10 ** 6, 4, 64) == most
    assert pages_for_memory(free, cfg, _CacheNeeds([win, win])) >= most          # every group is full: what is offered is not taken
    m = CacheManager([full, win], 16, 1000, 4, max_step_tokens=64)
    assert [g.pool.num_pages for g in m.page_groups] == [1000, most]
    assert [g.pool.num_pages for g in CacheManager([full, win], 16, 1000, 4).page_groups] == [1000, 1000]
