import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (gfx950) and the built HIP kernel library")


@pytest.fixture
def emu_ops(monkeypatch):
    """Replaces the engine's operations (``spyinfer_amd.kernels.ops``) by the CPU stand-in for the duration of a test, so
    that the engine's logic (batches, cache pages, block tables, scheduling) runs on a machine without a GPU.  The
    product has no such switch: the stand-in is patched in from here."""
    from spyinfer_amd.kernels import ops
    from tests.emu_ops import EmuOps
    emu = EmuOps()
    for name in ("embedding", "add_rms_norm", "rms_norm", "qk_norm_rope_store", "swiglu", "sample"):
        monkeypatch.setattr(ops, name, getattr(emu, name))

    def linear(x, w, out_dtype=None, tiled=None, out=None):
        y = emu.linear(x, w, out_dtype)
        return y if out is None else out.copy_(y)
    monkeypatch.setattr(ops, "linear", linear)
    monkeypatch.setattr(ops, "linear_swiglu", lambda x, w, tiled=None: emu.swiglu(emu.linear(x, w)))
    monkeypatch.setattr(ops, "paged_attention", lambda q, k_cache, v_cache, page_size, meta, n_q, n_kv, d, scale, window, raw=None,
                        for_product=False: emu.paged_attention(q, k_cache, v_cache, page_size, meta, n_q, n_kv, d, scale, window))
    monkeypatch.setattr(ops, "tile_weight", lambda w: None)
    monkeypatch.setattr(ops, "fused_decode_ok", lambda *a, **k: False)
    monkeypatch.setattr(ops, "fused_attention_ok", lambda *a, **k: False)
    monkeypatch.setattr(ops, "hip", lambda: None)
    # what the engine does with the device beside the operations: transfers through pinned memory, HIP graphs, the
    # device's free memory
    from spyinfer_amd.engine.llm_engine import LLMEngine, pages_for_memory
    from spyinfer_amd.engine.runner import ModelRunner
    from spyinfer_amd.sampling.sampler import Sampler
    runner_init = ModelRunner.__init__

    def init_without_graphs(self, *args, **kwargs):
        kwargs["enforce_eager"] = True
        runner_init(self, *args, **kwargs)
    monkeypatch.setattr(ModelRunner, "__init__", init_without_graphs)
    monkeypatch.setattr(ModelRunner, "_pack", lambda self, batch: None)
    monkeypatch.setattr(ModelRunner, "_upload", lambda self, batch, dev_buf, bind=True: batch.upload())
    monkeypatch.setattr(LLMEngine, "_pages_from_free_memory", lambda self: pages_for_memory(1 << 30, self.config, self.model))
    monkeypatch.setattr(Sampler, "_host_buffer", staticmethod(lambda R: torch.empty((2, R), dtype=torch.float32)))


@pytest.fixture(autouse=True)
def poisoned_cache_pool(monkeypatch):
    """Every cache pool that a test's engine makes is filled with NaN instead of zeros.  A slot is always written
    before it is read, so a correct engine never shows it; a read of a slot that was never written (a wrong page, a
    key beyond a request's length that is not masked) turns the logits into NaN instead of passing as a zero."""
    from spyinfer_amd.cache.storage import CacheStorage
    real = CacheStorage.__init__

    def init(self, *args, **kwargs):
        real(self, *args, **kwargs)
        self.fill(float("nan"))
    monkeypatch.setattr(CacheStorage, "__init__", init)
